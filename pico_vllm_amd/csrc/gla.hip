// Gated linear attention: a recurrent mixer whose state is a matrix per head.
//
//   per head, with key channels c and value channels v:
//     S_t[c][v] = alpha_t[c] * S_(t-1)[c][v] + k_t[c] * v_t[v]          (a decay per key channel)
//     o_t[v]    = sum_c S_t[c][v] * q_t[c] * qscale
//   alpha_t = sigmoid(z_t)^(1 / tau),  z_t = A2 (A1 h_t) + b           (a low-rank projection; A1 h_t comes with q, k, v)
//   out_t = rmsnorm_v(o_t) * w * silu(g_t)                             (every head by itself, one weight for all heads)
//
// The state lives in float32, one [heads, dk, dv] block per state slot; decays, their logarithms, the recurrence and
// the head norm are float32 whatever the storage type T of the projections.  Every sum runs in an order that depends
// on the sizes alone, so a token's output does not depend on how its sequence was cut into steps.
#include "common.h"

// ---------------------------------------------------------------------------
// Logarithm of the decay: out[t][c] = log(sigmoid(z)) / tau, z = sum_r a2[c][r] * x[t][r] + b[c].
// x: the low-rank activations (columns of a wider row, stride ldx); a2 [C, R]; b float32 [C].  grid (T), any C and R.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(256) void gla_decay_kernel(const T* __restrict__ x, int ldx, const T* __restrict__ a2,
                                                        const float* __restrict__ b, float inv_tau, float* __restrict__ out,
                                                        int C, int R) {
  extern __shared__ float xs[];
  const int t = blockIdx.x;
  for (int r = threadIdx.x; r < R; r += blockDim.x) xs[r] = load_f32(x + (size_t)t * ldx + r);
  __syncthreads();
  for (int c = threadIdx.x; c < C; c += blockDim.x) {
    const T* w = a2 + (size_t)c * R;
    float z = b ? b[c] : 0.f;
    for (int r = 0; r < R; r++) z = fmaf(load_f32(w + r), xs[r], z);
    // log(sigmoid(z)) = -log(1 + e^-z), without overflow on either side
    const float ls = z >= 0.f ? -log1pf(expf(-z)) : z - log1pf(expf(z));
    out[(size_t)t * C + c] = ls * inv_tau;
  }
}

extern "C" int pico_gla_decay(const void* x, int ldx, int dtype, const void* a2, const float* b, float tau, float* out,
                              int T, int C, int R, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && C > 0 && R > 0 && ldx >= R && R <= 8192, "pico_gla_decay: bad sizes");
  PICO_REQUIRE(tau > 0.f, "pico_gla_decay: tau must be positive");
  if (T == 0) return 0;
  const size_t lds = (size_t)R * sizeof(float);
  if (dtype == PICO_DTYPE_F32)
    gla_decay_kernel<float><<<T, 256, lds, stream>>>((const float*)x, ldx, (const float*)a2, b, 1.0f / tau, out, C, R);
  else if (dtype == PICO_DTYPE_BF16)
    gla_decay_kernel<bf16_t><<<T, 256, lds, stream>>>((const bf16_t*)x, ldx, (const bf16_t*)a2, b, 1.0f / tau, out, C, R);
  else
    PICO_REQUIRE(false, "pico_gla_decay: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// The recurrence, token by token.  grid (sequences, heads, ceil(dv / 64)); a workgroup owns 64 value channels of one
// head of one sequence; wave w of its ceil(dk / GLA_CPT) waves owns key channels GLA_CPT w .., lane l value channel l:
// a thread keeps GLA_CPT state elements in registers over all tokens of the step.  Tokens are taken GLA_TB at a time:
// their q, k and decays are staged in LDS (every thread reads all of its channels' from there), the waves' partial
// outputs meet in LDS and are summed in wave order.
// ---------------------------------------------------------------------------
#define GLA_CPT 32
#define GLA_TB 8

template <typename T>
__global__ __launch_bounds__(512) void gla_scan_kernel(const T* __restrict__ x, int ldx, int q_col, int k_col, int v_col,
                                                       const float* __restrict__ log_decay,
                                                       const int* __restrict__ cu_seqlens,
                                                       const int* __restrict__ state_slots, float* __restrict__ state,
                                                       float* __restrict__ out, int H, int dk, int dv, float qscale,
                                                       int num_slots) {
  extern __shared__ float lds[];
  const int nw = blockDim.x >> 6, wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int CP = nw * GLA_CPT;                          // key channels with padding
  float* qs = lds;                                      // [GLA_TB][CP]
  float* ks = qs + GLA_TB * CP;
  float* as = ks + GLA_TB * CP;
  float* po = as + GLA_TB * CP;                         // [GLA_TB][nw][64]
  const int b = blockIdx.x, h = blockIdx.y, v = blockIdx.z * 64 + lane;
  const bool v_ok = v < dv;
  const int t_begin = cu_seqlens[b], t_end = cu_seqlens[b + 1];
  const int slot = state_slots[b];
  if (slot < 0 || slot >= num_slots || t_end <= t_begin) return;
  const int c0 = wave * GLA_CPT;
  float* sp = state + (((size_t)slot * H + h) * dk + c0) * dv + v;
  float S[GLA_CPT];
#pragma unroll
  for (int c = 0; c < GLA_CPT; c++) S[c] = (v_ok && c0 + c < dk) ? sp[(size_t)c * dv] : 0.f;

  for (int t0 = t_begin; t0 < t_end; t0 += GLA_TB) {
    const int nb = min(GLA_TB, t_end - t0);
    __syncthreads();                                    // the last block's partial outputs have been read
    for (int i = threadIdx.x; i < nb * CP; i += blockDim.x) {
      const int tt = i / CP, c = i - tt * CP;
      float qv = 0.f, kv = 0.f, av = 1.f;
      if (c < dk) {
        const T* row = x + (size_t)(t0 + tt) * ldx + (size_t)h * dk + c;
        qv = load_f32(row + q_col) * qscale;
        kv = load_f32(row + k_col);
        av = expf(log_decay[(size_t)(t0 + tt) * H * dk + (size_t)h * dk + c]);
      }
      qs[i] = qv; ks[i] = kv; as[i] = av;
    }
    float vv[GLA_TB];
#pragma unroll
    for (int tt = 0; tt < GLA_TB; tt++)
      vv[tt] = (tt < nb && v_ok) ? load_f32(x + (size_t)(t0 + tt) * ldx + v_col + (size_t)h * dv + v) : 0.f;
    __syncthreads();
#pragma unroll
    for (int tt = 0; tt < GLA_TB; tt++) {
      if (tt >= nb) break;
      const float4* a4 = reinterpret_cast<const float4*>(as + tt * CP + c0);
      const float4* k4 = reinterpret_cast<const float4*>(ks + tt * CP + c0);
      const float4* q4 = reinterpret_cast<const float4*>(qs + tt * CP + c0);
      float acc = 0.f;
#pragma unroll
      for (int c = 0; c < GLA_CPT / 4; c++) {
        const float4 av = a4[c], kv = k4[c], qv = q4[c];
        S[4 * c + 0] = fmaf(av.x, S[4 * c + 0], kv.x * vv[tt]); acc = fmaf(S[4 * c + 0], qv.x, acc);
        S[4 * c + 1] = fmaf(av.y, S[4 * c + 1], kv.y * vv[tt]); acc = fmaf(S[4 * c + 1], qv.y, acc);
        S[4 * c + 2] = fmaf(av.z, S[4 * c + 2], kv.z * vv[tt]); acc = fmaf(S[4 * c + 2], qv.z, acc);
        S[4 * c + 3] = fmaf(av.w, S[4 * c + 3], kv.w * vv[tt]); acc = fmaf(S[4 * c + 3], qv.w, acc);
      }
      po[(tt * nw + wave) * 64 + lane] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < nb * 64; i += blockDim.x) {
      const int tt = i >> 6, l = i & 63, vo = blockIdx.z * 64 + l;
      if (vo >= dv) continue;
      float sum = 0.f;
      for (int w = 0; w < nw; w++) sum += po[(tt * nw + w) * 64 + l];
      out[(size_t)(t0 + tt) * H * dv + (size_t)h * dv + vo] = sum;
    }
  }
  if (v_ok) {
#pragma unroll
    for (int c = 0; c < GLA_CPT; c++)
      if (c0 + c < dk) sp[(size_t)c * dv] = S[c];
  }
}

extern "C" int pico_gla_scan(const void* x, int ldx, int dtype, int q_col, int k_col, int v_col, const float* log_decay,
                             const int* cu_seqlens, const int* state_slots, float* state, float* out, int num_seqs,
                             int T, int H, int dk, int dv, float qscale, int num_slots, hipStream_t stream) {
  PICO_REQUIRE(num_seqs >= 0 && T >= 0 && H > 0 && dk > 0 && dv > 0 && num_slots > 0, "pico_gla_scan: bad sizes");
  PICO_REQUIRE(dk <= 8 * GLA_CPT, "pico_gla_scan: at most %d key channels a head, got %d", 8 * GLA_CPT, dk);
  PICO_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && ldx >= q_col + H * dk && ldx >= k_col + H * dk && ldx >= v_col + H * dv,
               "pico_gla_scan: the row of %d columns does not hold q, k and v", ldx);
  PICO_REQUIRE(H <= 65535 && (dv + 63) / 64 <= 65535, "pico_gla_scan: sizes beyond the grid");
  if (num_seqs == 0 || T == 0) return 0;
  const int nw = (dk + GLA_CPT - 1) / GLA_CPT;
  const size_t lds = (size_t)(3 * GLA_TB * nw * GLA_CPT + GLA_TB * nw * 64) * sizeof(float);
  PICO_REQUIRE(lds <= 64 * 1024, "pico_gla_scan: key channels beyond the staging memory");
  const dim3 grid(num_seqs, H, (dv + 63) / 64);
  if (dtype == PICO_DTYPE_F32)
    gla_scan_kernel<float><<<grid, 64 * nw, lds, stream>>>((const float*)x, ldx, q_col, k_col, v_col, log_decay, cu_seqlens,
                                                          state_slots, state, out, H, dk, dv, qscale, num_slots);
  else if (dtype == PICO_DTYPE_BF16)
    gla_scan_kernel<bf16_t><<<grid, 64 * nw, lds, stream>>>((const bf16_t*)x, ldx, q_col, k_col, v_col, log_decay, cu_seqlens,
                                                           state_slots, state, out, H, dk, dv, qscale, num_slots);
  else
    PICO_REQUIRE(false, "pico_gla_scan: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Head norm and gate: out[t][h][v] = o[t][h][v] / sqrt(mean_v(o^2) + eps) * w[v] * silu(g[t][h][v]).
// o float32 [T, H dv]; g: columns of a wider row of type T (stride ldg); out type T [T, H dv].  grid (T, H), one wave.
// ---------------------------------------------------------------------------
template <typename T>
__global__ __launch_bounds__(64) void gla_out_kernel(const float* __restrict__ o, const T* __restrict__ g, int ldg,
                                                     const float* __restrict__ w, float eps, T* __restrict__ out, int H,
                                                     int dv) {
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const float* orow = o + ((size_t)t * H + h) * dv;
  float ss = 0.f;
  for (int v = lane; v < dv; v += 64) ss = fmaf(orow[v], orow[v], ss);
  ss = wave_sum(ss);
  const float r = 1.0f / sqrtf(ss / (float)dv + eps);
  const T* grow = g + (size_t)t * ldg + (size_t)h * dv;
  T* dst = out + ((size_t)t * H + h) * dv;
  for (int v = lane; v < dv; v += 64) {
    const float gv = load_f32(grow + v);
    store_f32(dst + v, orow[v] * r * w[v] * (gv / (1.0f + expf(-gv))));
  }
}

extern "C" int pico_gla_out(const float* o, const void* g, int ldg, int dtype, const float* w, float eps, void* out, int T,
                            int H, int dv, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && H > 0 && dv > 0 && ldg >= H * dv && H <= 65535, "pico_gla_out: bad sizes");
  if (T == 0) return 0;
  const dim3 grid(T, H);
  if (dtype == PICO_DTYPE_F32)
    gla_out_kernel<float><<<grid, 64, 0, stream>>>(o, (const float*)g, ldg, w, eps, (float*)out, H, dv);
  else if (dtype == PICO_DTYPE_BF16)
    gla_out_kernel<bf16_t><<<grid, 64, 0, stream>>>(o, (const bf16_t*)g, ldg, w, eps, (bf16_t*)out, H, dv);
  else
    PICO_REQUIRE(false, "pico_gla_out: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
