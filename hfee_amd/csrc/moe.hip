// A feed-forward of many small gated experts, of which every token uses `top`.
//
// Which experts a token uses is given from outside as int32 [n, top] (`chosen`), or looked up here in
// a table [vocabulary, top] under the token's id; expert e of a token counts with pair_weights[t][j]
// or, without them, with the one number `weight`.
//
//   up:    act[t][j][f] = silu(W_gate[e][f] . h_t) * (W_up[e][f] . h_t),   e = the j-th expert of t
//   down:  x[t][c] (+)= sum_j weight_tj (W_down[e_j][c] . act[t][j])
//
// A wave a dot product, lanes over the summed dimension, added up in a fixed order; the experts'
// matrices are stacked [experts][rows][columns].  Every token reads the rows of its own experts:
// this is the form for steps of few tokens, whose time is the experts' bytes.
#include "common.h"

using namespace hfee;

namespace {

__device__ __forceinline__ int expert_of(const int* chosen, const int* table, const int* token_ids, int t, int j, int top) {
  return chosen != nullptr ? chosen[(int64_t)t * top + j] : table[(int64_t)token_ids[t] * top + j];
}

constexpr int kRowsPerWave = 4;

template <typename T>
__global__ __launch_bounds__(256) void moe_up_kernel(T* __restrict__ act, const T* __restrict__ h, int64_t ldh,
                                                     const T* __restrict__ w_gate, const T* __restrict__ w_up,
                                                     const int* __restrict__ chosen, const int* __restrict__ table,
                                                     const int* __restrict__ token_ids, int top, int experts, int F,
                                                     int width) {
  const int pair = blockIdx.x, t = pair / top, j = pair - t * top;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int e = expert_of(chosen, table, token_ids, t, j, top);
  if (e < 0 || e >= experts) return;                       // (a table that names no such expert: nothing is read)
  const T* hr = h + (int64_t)t * ldh;
  const int f0 = (blockIdx.y * 4 + wave) * kRowsPerWave;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int f = f0 + r;
    if (f >= F) break;
    const T* g = w_gate + ((int64_t)e * F + f) * width;
    const T* u = w_up + ((int64_t)e * F + f) * width;
    float sg = 0.f, su = 0.f;
    for (int c = lane; c < width; c += 64) {
      const float x = to_float<T>(hr[c]);
      sg = fmaf(to_float<T>(g[c]), x, sg);
      su = fmaf(to_float<T>(u[c]), x, su);
    }
    sg = wave_sum(sg);
    su = wave_sum(su);
    if (lane == 0) act[(int64_t)pair * F + f] = from_float<T>(sg / (1.0f + expf(-sg)) * su);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_down_kernel(float* __restrict__ x, int64_t ldx, const T* __restrict__ act,
                                                       const T* __restrict__ w_down, const int* __restrict__ chosen,
                                                       const int* __restrict__ table, const int* __restrict__ token_ids,
                                                       const float* __restrict__ pair_weights, float weight, int top,
                                                       int experts, int F, int width, int accumulate) {
  const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int c0 = (blockIdx.y * 4 + wave) * kRowsPerWave;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int c = c0 + r;
    if (c >= width) break;
    float total = 0.f;
    for (int j = 0; j < top; ++j) {
      const int e = expert_of(chosen, table, token_ids, t, j, top);
      if (e < 0 || e >= experts) continue;
      const T* w = w_down + ((int64_t)e * width + c) * F;
      const T* a = act + ((int64_t)t * top + j) * F;
      float s = 0.f;
      for (int f = lane; f < F; f += 64) s = fmaf(to_float<T>(w[f]), to_float<T>(a[f]), s);
      total = fmaf(wave_sum(s), pair_weights != nullptr ? pair_weights[(int64_t)t * top + j] : weight, total);
    }
    if (lane == 0) {
      float* o = x + (int64_t)t * ldx + c;
      *o = accumulate ? *o + total : total;
    }
  }
}

}  // namespace

HFEE_API int hfee_moe_up(void* act, const void* h, int64_t ldh, const void* w_gate, const void* w_up, int dtype,
                         const int* chosen, const int* table, const int* token_ids, int top, int experts, int ff,
                         int width, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && top >= 1 && experts >= 1 && ff >= 1 && width >= 1 && ldh >= width, "moe_up: bad sizes");
  HFEE_REQUIRE(chosen != nullptr || (table != nullptr && token_ids != nullptr), "moe_up: the experts of a token, or a table and the ids");
  if (n == 0) return 0;
  const int per_block = 4 * kRowsPerWave;
  HFEE_REQUIRE((ff + per_block - 1) / per_block <= 65535, "moe_up: experts too wide");
  dim3 grid((unsigned)((int64_t)n * top), (ff + per_block - 1) / per_block);
  if (dtype == 0)
    moe_up_kernel<float><<<grid, 256, 0, stream>>>((float*)act, (const float*)h, ldh, (const float*)w_gate, (const float*)w_up,
                                                   chosen, table, token_ids, top, experts, ff, width);
  else if (dtype == 1)
    moe_up_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)act, (const bf16_t*)h, ldh, (const bf16_t*)w_gate,
                                                    (const bf16_t*)w_up, chosen, table, token_ids, top, experts, ff, width);
  else
    return fail("moe_up: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("moe_up");
  return 0;
}

HFEE_API int hfee_moe_down(float* x, int64_t ldx, const void* act, const void* w_down, int dtype, const int* chosen,
                           const int* table, const int* token_ids, const float* pair_weights, float weight, int top,
                           int experts, int ff, int width, int accumulate, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && top >= 1 && experts >= 1 && ff >= 1 && width >= 1 && ldx >= width, "moe_down: bad sizes");
  HFEE_REQUIRE(chosen != nullptr || (table != nullptr && token_ids != nullptr), "moe_down: the experts of a token, or a table and the ids");
  if (n == 0) return 0;
  const int per_block = 4 * kRowsPerWave;
  HFEE_REQUIRE((width + per_block - 1) / per_block <= 65535, "moe_down: rows too wide");
  dim3 grid(n, (width + per_block - 1) / per_block);
  if (dtype == 0)
    moe_down_kernel<float><<<grid, 256, 0, stream>>>(x, ldx, (const float*)act, (const float*)w_down, chosen, table,
                                                     token_ids, pair_weights, weight, top, experts, ff, width, accumulate);
  else if (dtype == 1)
    moe_down_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, ldx, (const bf16_t*)act, (const bf16_t*)w_down, chosen, table,
                                                      token_ids, pair_weights, weight, top, experts, ff, width, accumulate);
  else
    return fail("moe_down: unknown dtype %d", dtype);
  HFEE_CHECK_LAUNCH("moe_down");
  return 0;
}
