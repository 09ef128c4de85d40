// A routed feed-forward in bfloat16: the kernels that serve it.
//
// Few rows (a row is one (token, chosen expert) pair; single tokens and small steps): every row streams its expert's
// matrices once, 16 bytes a lane, sixteen lanes to an output element.
//
// Many rows (prompt portions): the rows are sorted by expert on the device (nothing comes back to the host), every
// expert's rows padded to whole tiles of MOE_BM rows, and two grouped products run on the matrix cores, their operands
// staged through LDS:
//   first:  y[p, f] = act(gate_e[f] . x_p, up_e[f] . x_p),  x_p = bf16(w_p * h[token of p])   (gathered while staging)
//   second: out[slot of p][token of p][n] = down_e[n] . y[p]                                   (float32, scattered)
// A row's result does not depend on which other rows share its tile: a matrix instruction keeps rows apart and the sums
// over k run in the same order for every row.
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define MOE_BM 128         // rows of a tile
#define MOE_BN 128         // matrix rows (output columns) of a tile
#define MOE_BK 64          // k of one stage
#define MOE_LD 72          // LDS row stride in bfloat16: 144 bytes, a multiple of 16 that spreads rows over the banks

// mode 0: the clipped activation, the row's weight w already in the input; mode 1: w silu(g) u (the weight on the
// expert's output, taken in front of the linear second product)
__device__ __forceinline__ float moe_act(float g, float u, float limit, float alpha, int mode, float w) {
  if (mode == 1) return w * (g / (1.0f + expf(-g))) * u;
  g = fminf(g, limit);
  u = fminf(fmaxf(u, -limit), limit);
  return g / (1.0f + expf(-alpha * g)) * (u + 1.0f);
}

__device__ __forceinline__ void unpack8(const uint4& v, float* f) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}

// 8 bfloat16 times w, each rounded to bfloat16 again
__device__ __forceinline__ uint4 scale8(const uint4& v, float w) {
  float f[8];
  unpack8(v, f);
  uint4 o;
  o.x = pack2_bf16(f[0] * w, f[1] * w);
  o.y = pack2_bf16(f[2] * w, f[3] * w);
  o.z = pack2_bf16(f[4] * w, f[5] * w);
  o.w = pack2_bf16(f[6] * w, f[7] * w);
  return o;
}

// v where keep, else zeros (component by component: the values stay in registers)
__device__ __forceinline__ uint4 keep8(const uint4& v, bool keep) {
  const uint32_t m = keep ? 0xffffffffu : 0u;
  return make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
}

__device__ __forceinline__ float dot8(const uint4& a, const float* x, float acc) {
  float f[8];
  unpack8(a, f);
#pragma unroll
  for (int i = 0; i < 8; i++) acc = fmaf(f[i], x[i], acc);
  return acc;
}

// the sum over a row of 16 lanes, in every lane of the row
__device__ __forceinline__ float row16_sum(float v) {
  v += lane_pattern<LANE_XOR_1>(v);
  v += lane_pattern<LANE_XOR_2>(v);
  v += lane_pattern<HALF_ROW_MIRROR>(v);
  v += lane_pattern<ROW_MIRROR>(v);
  return v;
}

// ---------------------------------------------------------------------------
// Few rows, first half.  grid (rows, ceil(F / 16)); 4 waves; a row of 16 lanes makes one f (its gate and its up).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_up_rows_kernel(const bf16_t* __restrict__ h, int ldh,
                                                          const bf16_t* __restrict__ gate_up,
                                                          const int* __restrict__ experts, const float* __restrict__ weights,
                                                          bf16_t* __restrict__ y, int top, int E, int F, int D, float limit,
                                                          float alpha, int mode) {
  const int r = blockIdx.x, sub = threadIdx.x & 15;
  const int f = blockIdx.y * 16 + (threadIdx.x >> 4);
  const int e = experts[r];
  if (e < 0 || e >= E || f >= F) return;
  const float wr = weights[r];
  const float w = mode == 1 ? 1.f : wr;
  const bf16_t* x = h + (size_t)(r / top) * ldh;
  const bf16_t* wg = gate_up + ((size_t)e * 2 * F + f) * D;
  const bf16_t* wu = wg + (size_t)F * D;
  float g = 0.f, u = 0.f;
#pragma unroll 2
  for (int k = sub * 8; k < D; k += 128) {
    const uint4 x8 = *reinterpret_cast<const uint4*>(x + k);
    const uint4 xv = mode == 1 ? x8 : scale8(x8, w);
    const uint4 gv = *reinterpret_cast<const uint4*>(wg + k);
    const uint4 uv = *reinterpret_cast<const uint4*>(wu + k);
    float xf[8];
    unpack8(xv, xf);
    g = dot8(gv, xf, g);
    u = dot8(uv, xf, u);
  }
  g = row16_sum(g);
  u = row16_sum(u);
  if (sub == 0) y[(size_t)r * F + f] = f32_to_bf16(moe_act(g, u, limit, alpha, mode, wr));
}

// ---------------------------------------------------------------------------
// Few rows, second half: out[t, n] = sum over the token's slots, in slot order, of down_e[n] . y[(t, slot)].
// grid (tokens, ceil(D / 16)).
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void moe_down_rows_kernel(const bf16_t* __restrict__ y, const bf16_t* __restrict__ down,
                                                            const int* __restrict__ experts, float* __restrict__ out,
                                                            int top, int E, int F, int D) {
  const int t = blockIdx.x, sub = threadIdx.x & 15;
  const int n = blockIdx.y * 16 + (threadIdx.x >> 4);
  if (n >= D) return;
  float total = 0.f;
  for (int k = 0; k < top; k++) {
    const int r = t * top + k, e = experts[r];
    if (e < 0 || e >= E) continue;
    const bf16_t* wd = down + ((size_t)e * D + n) * F;
    const bf16_t* yr = y + (size_t)r * F;
    float s = 0.f;
#pragma unroll 2
    for (int j = sub * 8; j < F; j += 128) {
      float yf[8];
      unpack8(*reinterpret_cast<const uint4*>(yr + j), yf);
      s = dot8(*reinterpret_cast<const uint4*>(wd + j), yf, s);
    }
    total += row16_sum(s);
  }
  if (sub == 0) out[(size_t)t * D + n] = total;
}

extern "C" int pico_moe_experts_rows(const void* h, int ldh, const void* gate_up, const void* down, const int* experts,
                                     const float* weights, void* y, float* out, int T, int top, int E, int F, int D,
                                     float limit, float alpha, int mode, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && top > 0 && E > 0 && F > 0 && D > 0 && ldh >= D, "pico_moe_experts_rows: bad sizes");
  PICO_REQUIRE(mode == 0 || mode == 1, "pico_moe_experts_rows: unknown mode %d", mode);
  PICO_REQUIRE(F % 8 == 0 && D % 8 == 0 && ldh % 8 == 0, "pico_moe_experts_rows: sizes must be multiples of 8");
  PICO_REQUIRE(((uintptr_t)h | (uintptr_t)gate_up | (uintptr_t)down | (uintptr_t)y) % 16 == 0,
               "pico_moe_experts_rows: operands must start on 16 bytes");
  if (T == 0) return 0;
  const dim3 g1(T * top, (F + 15) / 16), g2(T, (D + 15) / 16);
  PICO_REQUIRE(g1.y <= 65535 && g2.y <= 65535, "pico_moe_experts_rows: sizes beyond the grid");
  moe_up_rows_kernel<<<g1, 256, 0, stream>>>((const bf16_t*)h, ldh, (const bf16_t*)gate_up, experts, weights, (bf16_t*)y,
                                             top, E, F, D, limit, alpha, mode);
  moe_down_rows_kernel<<<g2, 256, 0, stream>>>((const bf16_t*)y, (const bf16_t*)down, experts, out, top, E, F, D);
  PICO_LAUNCH_CHECK();
  return 0;
}

// ---------------------------------------------------------------------------
// Sorting the rows by expert.  One workgroup an expert: it counts every expert's rows (to know where its own begin),
// then writes its own rows' numbers in ascending order; its last tile is filled up with -1.
//   sorted[tiles_cap * MOE_BM]: row numbers (token * top + slot) or -1;  tile_expert[tiles_cap]: the expert of a tile, -1: unused
// ---------------------------------------------------------------------------
#define MOE_SORT_THREADS 1024
#define MOE_SORT_MAX_E 1024

__global__ __launch_bounds__(MOE_SORT_THREADS) void moe_sort_kernel(const int* __restrict__ experts, int R, int E,
                                                                    int tiles_cap, int* __restrict__ sorted,
                                                                    int* __restrict__ tile_expert) {
  __shared__ int hist[MOE_SORT_MAX_E];
  __shared__ int wave_count[MOE_SORT_THREADS / 64];
  __shared__ int base_tiles;
  const int e = blockIdx.x, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, nw = MOE_SORT_THREADS / 64;
  for (int i = tid; i < E; i += MOE_SORT_THREADS) hist[i] = 0;
  if (tid == 0) base_tiles = 0;
  __syncthreads();
  for (int r = tid; r < R; r += MOE_SORT_THREADS) {
    const int x = experts[r];
    if (x >= 0 && x < E) atomicAdd(&hist[x], 1);
  }
  __syncthreads();
  int before = 0;
  for (int i = tid; i < e; i += MOE_SORT_THREADS) before += (hist[i] + MOE_BM - 1) / MOE_BM;
  if (before) atomicAdd(&base_tiles, before);
  __syncthreads();
  const int count = hist[e], tiles = (count + MOE_BM - 1) / MOE_BM, base = base_tiles;
  for (int i = tid; i < tiles; i += MOE_SORT_THREADS) tile_expert[base + i] = e;
  if (e == E - 1)
    for (int i = base + tiles + tid; i < tiles_cap; i += MOE_SORT_THREADS) tile_expert[i] = -1;
  // every wave takes a stretch of the rows: counts its own, then writes them behind those of the waves before it
  const int seg = ((R + nw - 1) / nw + 63) / 64 * 64, lo = wave * seg, hi = min(R, lo + seg);
  int mine = 0;
  for (int r0 = lo; r0 < hi; r0 += 64) {
    const int r = r0 + lane;
    const bool is = r < hi && experts[r] == e;
    mine += __popcll(__ballot(is));
  }
  if (lane == 0) wave_count[wave] = mine;
  __syncthreads();
  int at = 0;
  for (int i = 0; i < wave; i++) at += wave_count[i];
  int* dst = sorted + (size_t)base * MOE_BM;
  for (int r0 = lo; r0 < hi; r0 += 64) {
    const int r = r0 + lane;
    const bool is = r < hi && experts[r] == e;
    const unsigned long long m = __ballot(is);
    if (is) dst[at + __popcll(m & ((1ull << lane) - 1ull))] = r;
    at += __popcll(m);
  }
  for (int i = count + tid; i < tiles * MOE_BM; i += MOE_SORT_THREADS) dst[i] = -1;
}

// ---------------------------------------------------------------------------
// The grouped product.  grid (tiles_cap, ceil(N / columns of a tile)); a tile is MOE_BM rows x MOE_BN matrix rows, staged
// MOE_BK k at a time (the next stage travels in registers while this one is multiplied); 4 waves as 2 x 2, a wave makes
// 64 rows x 2 blocks of 32 columns with four v_mfma_f32_32x32x16_bf16 a k step.
// UP:   A = gathered, scaled rows of h (K = D); B rows = 64 gate rows f0.. and 64 up rows F + f0..; a wave holds gate and
//       up of the same 32 columns and writes act(gate, up) to y[p, f] (bfloat16).
// DOWN: A = y rows of the tile (K = F); B rows = 128 rows n0.. of down_e; float32 to out[slot][token][n].
// ---------------------------------------------------------------------------
template <bool UP>
__global__ __launch_bounds__(256) void moe_grouped_kernel(const bf16_t* __restrict__ A, int lda,
                                                          const bf16_t* __restrict__ W, const int* __restrict__ sorted,
                                                          const int* __restrict__ tile_expert,
                                                          const float* __restrict__ weights, bf16_t* __restrict__ y,
                                                          float* __restrict__ out, int T, int top, int F, int D,
                                                          float limit, float alpha, int ntile, int ncol, int mode) {
  __shared__ __attribute__((aligned(16))) bf16_t As[MOE_BM * MOE_LD];
  __shared__ __attribute__((aligned(16))) bf16_t Bs[MOE_BN * MOE_LD];
  __shared__ int rows[MOE_BM];
  // Which tile and which columns.  Workgroups go to the chip's eight dies in turn, and every die has a second-level
  // cache of its own.  Tiles are taken in pairs (neighbours in the sorted order: mostly one expert's); pair p belongs to
  // die p % 8, and a die's consecutive workgroups are the two tiles of a pair at the same columns, then at the next
  // columns: what runs together on a die shares its operands.  grid: 8 * ceil(pairs / 8) * 2 * ncol, one-dimensional.
  const int die = blockIdx.x & 7, idx = blockIdx.x >> 3;
  const int pair = (idx / (2 * ncol)) * 8 + die, rest = idx % (2 * ncol);
  const int tile = 2 * pair + (rest & 1), col = rest >> 1;
  if (tile >= ntile) return;
  const int e = tile_expert[tile];
  if (e < 0) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
  const int K = UP ? D : F;
  const int c0 = col * (UP ? MOE_BN / 2 : MOE_BN);            // first output column of this tile
  if (tid < MOE_BM) rows[tid] = sorted[(size_t)tile * MOE_BM + tid];

  // what this thread stages: 8 k of four A rows and of four B rows (rows srow, srow + 32, ...); rows that do not exist
  // point at a row that does and are cleared after the load, so that every load is unconditional
  const int srow = tid >> 3, sk = (tid & 7) * 8;
  const size_t erows = UP ? (size_t)2 * F : (size_t)D;
#define MOE_STAGE_ROW(i, A_SRC, A_W, A_OK, B_SRC, B_OK)                                   \
  const bf16_t* A_SRC;                                                                    \
  const bf16_t* B_SRC;                                                                    \
  float A_W = 1.f;                                                                        \
  bool A_OK = true, B_OK;                                                                 \
  {                                                                                       \
    const int m = srow + 32 * (i);                                                        \
    if (UP) {                                                                             \
      const int r = sorted[(size_t)tile * MOE_BM + m];                                    \
      A_OK = r >= 0;                                                                      \
      A_SRC = A + (size_t)(A_OK ? r / top : 0) * lda + sk;                                \
      A_W = A_OK ? (mode == 1 ? 1.f : weights[r]) : 0.f;                                  \
      const int f = c0 + (m & 63);                                                        \
      B_OK = f < F;                                                                       \
      B_SRC = W + ((size_t)e * erows + (B_OK ? (m >> 6) * F + f : 0)) * K + sk;           \
    } else {                                                                              \
      A_SRC = A + ((size_t)tile * MOE_BM + m) * lda + sk;                                 \
      B_OK = c0 + m < D;                                                                  \
      B_SRC = W + ((size_t)e * erows + (B_OK ? c0 + m : 0)) * K + sk;                     \
    }                                                                                     \
  }
  MOE_STAGE_ROW(0, a_src0, a_w0, a_ok0, b_src0, b_ok0)
  MOE_STAGE_ROW(1, a_src1, a_w1, a_ok1, b_src1, b_ok1)
  MOE_STAGE_ROW(2, a_src2, a_w2, a_ok2, b_src2, b_ok2)
  MOE_STAGE_ROW(3, a_src3, a_w3, a_ok3, b_src3, b_ok3)
#undef MOE_STAGE_ROW

  f32x16 acc00, acc01, acc10, acc11;
#pragma unroll
  for (int r = 0; r < 16; r++) { acc00[r] = 0.f; acc01[r] = 0.f; acc10[r] = 0.f; acc11[r] = 0.f; }

  uint4 ra0, ra1, ra2, ra3, rb0, rb1, rb2, rb3;
  // K is a multiple of 8: the 8 k of a load are in or out together; a load beyond K reads k = 0 .. instead.  What must
  // read as zero (rows that do not exist, k beyond K) is cleared where the stage is written to LDS, not here: a select
  // on a register that a load has just been asked for would wait for that load in front of the products
#define MOE_FETCH(k0)                                                      \
  {                                                                        \
    const bool k_ok = (k0) + sk < K;                                       \
    const int ko = k_ok ? (k0) : -sk;   /* the row's first 8, not 8 behind its end (the last row ends the tensor) */ \
    ra0 = *reinterpret_cast<const uint4*>(a_src0 + ko);                    \
    ra1 = *reinterpret_cast<const uint4*>(a_src1 + ko);                    \
    ra2 = *reinterpret_cast<const uint4*>(a_src2 + ko);                    \
    ra3 = *reinterpret_cast<const uint4*>(a_src3 + ko);                    \
    rb0 = *reinterpret_cast<const uint4*>(b_src0 + ko);                    \
    rb1 = *reinterpret_cast<const uint4*>(b_src1 + ko);                    \
    rb2 = *reinterpret_cast<const uint4*>(b_src2 + ko);                    \
    rb3 = *reinterpret_cast<const uint4*>(b_src3 + ko);                    \
  }
  MOE_FETCH(0)
  const int frag = (lane & 31) * MOE_LD + (lane >> 5) * 8;    // a lane's place in a block of 32 rows
  const int a_off = wm * 64 * MOE_LD + frag;
  const int b_off0 = (UP ? wn * 32 : wn * 64) * MOE_LD + frag;
  const int b_off1 = (UP ? 64 + wn * 32 : wn * 64 + 32) * MOE_LD + frag;
  for (int k0 = 0; k0 < K; k0 += MOE_BK) {
    __syncthreads();                                          // the last stage has been read
    {
      bf16_t* as = As + srow * MOE_LD + sk;
      bf16_t* bs = Bs + srow * MOE_LD + sk;
      const bool k_in = k0 + sk < K;
      const bool scaled = UP && mode != 1;        // mode 1 puts the weight on the activation instead
      *reinterpret_cast<uint4*>(as) = keep8(scaled ? scale8(ra0, a_w0) : ra0, a_ok0 && k_in);
      *reinterpret_cast<uint4*>(as + 32 * MOE_LD) = keep8(scaled ? scale8(ra1, a_w1) : ra1, a_ok1 && k_in);
      *reinterpret_cast<uint4*>(as + 64 * MOE_LD) = keep8(scaled ? scale8(ra2, a_w2) : ra2, a_ok2 && k_in);
      *reinterpret_cast<uint4*>(as + 96 * MOE_LD) = keep8(scaled ? scale8(ra3, a_w3) : ra3, a_ok3 && k_in);
      *reinterpret_cast<uint4*>(bs) = keep8(rb0, b_ok0 && k_in);
      *reinterpret_cast<uint4*>(bs + 32 * MOE_LD) = keep8(rb1, b_ok1 && k_in);
      *reinterpret_cast<uint4*>(bs + 64 * MOE_LD) = keep8(rb2, b_ok2 && k_in);
      *reinterpret_cast<uint4*>(bs + 96 * MOE_LD) = keep8(rb3, b_ok3 && k_in);
    }
    if (k0 + MOE_BK < K) MOE_FETCH(k0 + MOE_BK)               // the next stage travels while this one is multiplied
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < MOE_BK; ks += 16) {
      const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(As + a_off + ks);
      const bf16x8 a1 = *reinterpret_cast<const bf16x8*>(As + a_off + 32 * MOE_LD + ks);
      const bf16x8 b0 = *reinterpret_cast<const bf16x8*>(Bs + b_off0 + ks);
      const bf16x8 b1 = *reinterpret_cast<const bf16x8*>(Bs + b_off1 + ks);
      acc00 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b0, acc00, 0, 0, 0);
      acc01 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a0, b1, acc01, 0, 0, 0);
      acc10 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b0, acc10, 0, 0, 0);
      acc11 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a1, b1, acc11, 0, 0, 0);
    }
  }
#undef MOE_FETCH
  // a lane holds column lane % 32 of its blocks and rows 8 (r / 4) + 4 (lane / 32) + r % 4
#define MOE_WRITE(i, ACC0, ACC1)                                                                                     \
  _Pragma("unroll") for (int r = 0; r < 16; r++) {                                                                   \
    const int m = wm * 64 + 32 * (i) + 8 * (r >> 2) + 4 * (lane >> 5) + (r & 3);                                     \
    if (UP) {                                                                                                        \
      const int f = c0 + wn * 32 + (lane & 31);                                                                      \
      const float wrow = (mode == 1 && rows[m] >= 0) ? weights[rows[m]] : 0.f;                                       \
      if (f < F) y[((size_t)tile * MOE_BM + m) * F + f] = f32_to_bf16(moe_act(ACC0[r], ACC1[r], limit, alpha, mode, wrow)); \
    } else {                                                                                                         \
      const int row = rows[m];                                                                                       \
      if (row < 0) continue;                                                                                         \
      float* o = out + ((size_t)(row % top) * T + row / top) * D;                                                    \
      const int n = c0 + wn * 64 + (lane & 31);                                                                      \
      if (n < D) o[n] = ACC0[r];                                                                                     \
      if (n + 32 < D) o[n + 32] = ACC1[r];                                                                           \
    }                                                                                                                \
  }
  MOE_WRITE(0, acc00, acc01)
  MOE_WRITE(1, acc10, acc11)
#undef MOE_WRITE
}

extern "C" int pico_moe_tile_rows() { return MOE_BM; }

extern "C" int pico_moe_experts_grouped(const void* h, int ldh, const void* gate_up, const void* down, const int* experts,
                                        const float* weights, int* sorted, int* tile_expert, int tiles_cap, void* y,
                                        float* out, int T, int top, int E, int F, int D, float limit, float alpha,
                                        int mode, hipStream_t stream) {
  PICO_REQUIRE(mode == 0 || mode == 1, "pico_moe_experts_grouped: unknown mode %d", mode);
  PICO_REQUIRE(T >= 0 && top > 0 && E > 0 && F > 0 && D > 0 && ldh >= D, "pico_moe_experts_grouped: bad sizes");
  PICO_REQUIRE(E <= MOE_SORT_MAX_E, "pico_moe_experts_grouped: at most %d experts", MOE_SORT_MAX_E);
  PICO_REQUIRE(F % 8 == 0 && D % 8 == 0 && ldh % 8 == 0, "pico_moe_experts_grouped: sizes must be multiples of 8");
  PICO_REQUIRE(((uintptr_t)h | (uintptr_t)gate_up | (uintptr_t)down | (uintptr_t)y) % 16 == 0,
               "pico_moe_experts_grouped: operands must start on 16 bytes");
  if (T == 0) return 0;
  const long long R = (long long)T * top;
  PICO_REQUIRE(R < (1ll << 30), "pico_moe_experts_grouped: too many rows");
  const long long need = (R + (long long)E * (MOE_BM - 1)) / MOE_BM;
  PICO_REQUIRE(tiles_cap >= need, "pico_moe_experts_grouped: room for %d tiles, %lld may be needed", tiles_cap, need);
  const long long ncol1 = (F + MOE_BN / 2 - 1) / (MOE_BN / 2), ncol2 = (D + MOE_BN - 1) / MOE_BN;
  const long long slots = ((tiles_cap + 1) / 2 + 7) / 8 * 8 * 2;       // tiles in pairs, pairs in eights
  PICO_REQUIRE(slots * ncol1 < (1ll << 31) && slots * ncol2 < (1ll << 31), "pico_moe_experts_grouped: sizes beyond the grid");
  moe_sort_kernel<<<E, MOE_SORT_THREADS, 0, stream>>>(experts, (int)R, E, tiles_cap, sorted, tile_expert);
  moe_grouped_kernel<true><<<(unsigned)(slots * ncol1), 256, 0, stream>>>(
      (const bf16_t*)h, ldh, (const bf16_t*)gate_up, sorted, tile_expert, weights, (bf16_t*)y, nullptr, T, top, F, D, limit,
      alpha, tiles_cap, (int)ncol1, mode);
  moe_grouped_kernel<false><<<(unsigned)(slots * ncol2), 256, 0, stream>>>(
      (const bf16_t*)y, F, (const bf16_t*)down, sorted, tile_expert, nullptr, nullptr, out, T, top, F, D, limit, alpha,
      tiles_cap, (int)ncol2, mode);
  PICO_LAUNCH_CHECK();
  return 0;
}
