// Rotary position encoding over neighbouring pairs, on part of a head, fused with the store of keys and values into
// the paged cache; keys and values may differ in size.
//
//   of every q and k head the entries (2i, 2i + 1), i < rot / 2, are turned by the angle of pair i:
//     out[2i]     = x[2i] * cos_i - x[2i + 1] * sin_i
//     out[2i + 1] = x[2i + 1] * cos_i + x[2i] * sin_i
//   entries from rot on pass unchanged.  cos_sin [T][rot / 2][2] comes from pico_rope_table (float32).
// x: [T, ld]; queries at column q_col (nq heads of dk, turned in place), keys at k_col (nkv heads of dk), values at
// v_col (nkv heads of dv).  Cache of one layer: K pages [page][kv head][slot in page][dk], V pages
// [page][kv head][dv][slot in page].  slots[t] = page * P + offset; negative: nothing is stored.  With k_cache null
// only the queries are turned (a layer that reads another layer's keys and values).  One workgroup per token.
#include "common.h"

template <typename T>
__global__ __launch_bounds__(256) void rope_pairs_store_kernel(T* __restrict__ x, int ld, int q_col, int k_col, int v_col,
                                                               const float2* __restrict__ cos_sin, int rot,
                                                               const int* __restrict__ slots, T* __restrict__ k_cache,
                                                               T* __restrict__ v_cache, int nq, int nkv, int dk, int dv,
                                                               int P, int num_pages) {
  const int t = blockIdx.x;
  T* row = x + (size_t)t * ld;
  const int half = rot >> 1;
  const float2* cs = cos_sin + (size_t)t * half;
  for (int u = threadIdx.x; u < nq * half; u += blockDim.x) {
    const int head = u / half, i = u - head * half;
    T* p = row + q_col + (size_t)head * dk + 2 * i;
    const float c = cs[i].x, s = cs[i].y;
    const float a = load_f32(p), b = load_f32(p + 1);
    store_f32(p, __fmaf_rn(a, c, -__fmul_rn(b, s)));
    store_f32(p + 1, __fmaf_rn(b, c, __fmul_rn(a, s)));
  }
  if (k_cache == nullptr) return;
  const int slot = slots[t];
  if (slot < 0) return;
  const int page = slot / P, off = slot % P;
  if (page >= num_pages) return;
  for (int u = threadIdx.x; u < nkv * half; u += blockDim.x) {
    const int g = u / half, i = u - g * half;
    const T* p = row + k_col + (size_t)g * dk + 2 * i;
    T* o = k_cache + (((size_t)page * nkv + g) * P + off) * dk + 2 * i;
    const float c = cs[i].x, s = cs[i].y;
    const float a = load_f32(p), b = load_f32(p + 1);
    store_f32(o, __fmaf_rn(a, c, -__fmul_rn(b, s)));
    store_f32(o + 1, __fmaf_rn(b, c, __fmul_rn(a, s)));
  }
  const int rest = dk - rot;
  for (int u = threadIdx.x; u < nkv * rest; u += blockDim.x) {
    const int g = u / rest, j = rot + u % rest;
    k_cache[(((size_t)page * nkv + g) * P + off) * dk + j] = row[k_col + (size_t)g * dk + j];
  }
  for (int u = threadIdx.x; u < nkv * dv; u += blockDim.x) {
    const int g = u / dv, j = u - g * dv;
    v_cache[(((size_t)page * nkv + g) * dv + j) * P + off] = row[v_col + u];
  }
}

extern "C" int pico_rope_pairs_store(void* x, int dtype, int ld, int q_col, int k_col, int v_col, const float* cos_sin,
                                     int rot, const int* slots, void* k_cache, void* v_cache, int T, int nq, int nkv,
                                     int dk, int dv, int P, int num_pages, hipStream_t stream) {
  PICO_REQUIRE(T >= 0 && nq > 0 && nkv > 0 && dk > 0 && dv > 0, "pico_rope_pairs_store: bad sizes");
  PICO_REQUIRE(rot >= 0 && rot <= dk && rot % 2 == 0, "pico_rope_pairs_store: %d rotated entries do not fit a head of %d", rot, dk);
  PICO_REQUIRE(rot == 0 || (cos_sin != nullptr && (uintptr_t)cos_sin % 8 == 0), "pico_rope_pairs_store: no table of cosines and sines");
  PICO_REQUIRE(q_col >= 0 && ld >= q_col + nq * dk, "pico_rope_pairs_store: the row of %d columns does not hold the queries", ld);
  if (k_cache != nullptr) {
    PICO_REQUIRE(v_cache != nullptr && slots != nullptr && P > 0 && num_pages > 0, "pico_rope_pairs_store: a cache needs slots and sizes");
    PICO_REQUIRE(k_col >= 0 && v_col >= 0 && ld >= k_col + nkv * dk && ld >= v_col + nkv * dv,
                 "pico_rope_pairs_store: the row of %d columns does not hold the keys and values", ld);
  }
  if (T == 0) return 0;
  if (dtype == PICO_DTYPE_F32)
    rope_pairs_store_kernel<float><<<T, 256, 0, stream>>>((float*)x, ld, q_col, k_col, v_col, (const float2*)cos_sin, rot, slots,
                                                          (float*)k_cache, (float*)v_cache, nq, nkv, dk, dv, P, num_pages);
  else if (dtype == PICO_DTYPE_BF16)
    rope_pairs_store_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)x, ld, q_col, k_col, v_col, (const float2*)cos_sin, rot,
                                                           slots, (bf16_t*)k_cache, (bf16_t*)v_cache, nq, nkv, dk, dv, P,
                                                           num_pages);
  else
    PICO_REQUIRE(false, "pico_rope_pairs_store: unknown dtype %d", dtype);
  PICO_LAUNCH_CHECK();
  return 0;
}
