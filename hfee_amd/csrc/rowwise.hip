// Row-wise steps of blocks that norm a sub-layer's output before they add it to the residual
// stream, and of feed-forwards with biases:
//
//   norm_add:      x[r] += (y[r] + bias) / sqrt(mean((y[r] + bias)^2) + eps) * w,   and, if asked, in
//                  the same launch the norm of the new row for the sub-layer that follows:
//                  next[r] = x[r] / sqrt(mean(x[r]^2) + eps2) * w2
//   bias_act:      out = act(in + bias)
//   rmsnorm_cols:  a norm over a block of columns of rows in the engine's dtype (a latent's norm)
//   layernorm:     out[r] = (x[r] - mean) / sqrt(mean((x[r] - mean)^2) + eps) * w, no bias
//
// All sums in float32, one workgroup a row, a fixed order of additions.
#include "common.h"

using namespace hfee;

namespace {

enum { ACT_NONE = 0, ACT_RELU2 = 1, ACT_RELU = 2, ACT_GELU_TANH = 3, ACT_SILU = 4, ACT_XIELU = 5 };

// ACT_XIELU has two numbers: a z^2 + z / 2 above zero, b (exp(z) - 1 - z) + z / 2 at and below it.
__device__ __forceinline__ float activate(float z, int act, float a = 0.f, float b = 0.f) {
  switch (act) {
    case ACT_XIELU: return z > 0.f ? fmaf(a * z, z, 0.5f * z) : fmaf(b, expm1f(z) - z, 0.5f * z);
    case ACT_RELU2: { const float r = fmaxf(z, 0.f); return r * r; }
    case ACT_RELU: return fmaxf(z, 0.f);
    case ACT_GELU_TANH: return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
    case ACT_SILU: return z / (1.0f + expf(-z));
    default: return z;
  }
}

template <typename TW>
__device__ __forceinline__ float weight_at(const TW* w, int j, float offset) { return offset + to_float<TW>(w[j]); }

// y: float32 [n, d]; bias: engine dtype or null; w, w2: norm weights (TW), used as (offset + w).
template <typename TY, typename TB, typename TW, typename TN>
__global__ __launch_bounds__(256) void norm_add_kernel(
    float* __restrict__ x, const TY* __restrict__ y, const TB* __restrict__ bias, const TW* __restrict__ w, float offset,
    float eps, TN* __restrict__ next, const TW* __restrict__ w2, float eps2, int d) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  const TY* yr = y + r * d;
  float* xr = x + r * d;
  float ss = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float v = to_float<TY>(yr[j]) + (bias ? to_float<TB>(bias[j]) : 0.f);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  float ss2 = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float v = to_float<TY>(yr[j]) + (bias ? to_float<TB>(bias[j]) : 0.f);
    const float nx = xr[j] + v * inv * weight_at<TW>(w, j, offset);
    xr[j] = nx;
    ss2 = fmaf(nx, nx, ss2);
  }
  if (next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps2);
  TN* nr = next + r * d;
  for (int j = threadIdx.x; j < d; j += blockDim.x)      // (a thread reads back what it wrote itself)
    nr[j] = from_float<TN>(xr[j] * inv2 * weight_at<TW>(w2, j, offset));
}

// The same for float32 y, bias and weights and rows of a multiple of four that fit the workgroup's
// registers (4 NV values a thread): everything a row needs is asked for at once, so that the row
// costs one trip to memory, two sums over the workgroup and the stores.
typedef float f32x4_t __attribute__((ext_vector_type(4)));

template <typename TN> __device__ __forceinline__ void store4(TN* p, f32x4_t v);
template <> __device__ __forceinline__ void store4<float>(float* p, f32x4_t v) { *reinterpret_cast<f32x4_t*>(p) = v; }
template <> __device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4_t v) {
  typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
  const u32x2_t w = {(uint32_t)float_to_bf16(v[0]) | ((uint32_t)float_to_bf16(v[1]) << 16),
                     (uint32_t)float_to_bf16(v[2]) | ((uint32_t)float_to_bf16(v[3]) << 16)};
  *reinterpret_cast<u32x2_t*>(p) = w;
}

template <typename TN, int NV>
__global__ __launch_bounds__(1024) void norm_add_rows_kernel(
    float* __restrict__ x, const float* __restrict__ y, const float* __restrict__ bias, const float* __restrict__ w,
    float eps, TN* __restrict__ next, const float* __restrict__ w2, float eps2, int d) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  f32x4_t yv[NV], xv[NV], wv[NV], w2v[NV];
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = (k * blockDim.x + threadIdx.x) * 4;
    const bool in = j < d;
    const f32x4_t zero = {0.f, 0.f, 0.f, 0.f};
    yv[k] = in ? *reinterpret_cast<const f32x4_t*>(y + r * d + j) : zero;
    if (in && bias != nullptr) yv[k] += *reinterpret_cast<const f32x4_t*>(bias + j);
    xv[k] = in ? *reinterpret_cast<const f32x4_t*>(x + r * d + j) : zero;
    wv[k] = in ? *reinterpret_cast<const f32x4_t*>(w + j) : zero;
    w2v[k] = in && next != nullptr ? *reinterpret_cast<const f32x4_t*>(w2 + j) : zero;
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k)
#pragma unroll
    for (int i = 0; i < 4; ++i) ss = fmaf(yv[k][i], yv[k][i], ss);
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = (k * blockDim.x + threadIdx.x) * 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      xv[k][i] += yv[k][i] * inv * wv[k][i];
      ss2 = fmaf(xv[k][i], xv[k][i], ss2);
    }
    if (j < d) *reinterpret_cast<f32x4_t*>(x + r * d + j) = xv[k];
  }
  if (next == nullptr) return;
  ss2 = block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)d + eps2);
#pragma unroll
  for (int k = 0; k < NV; ++k) {
    const int j = (k * blockDim.x + threadIdx.x) * 4;
    if (j < d) store4<TN>(next + r * d + j, xv[k] * inv2 * w2v[k]);
  }
}

template <typename T>
__global__ void bias_act_kernel(T* __restrict__ out, int64_t ldo, const T* __restrict__ in, int64_t ldi,
                                const T* __restrict__ bias, int width, int act, float pa, float pb) {
  const int64_t row = blockIdx.y;
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= width) return;
  const float z = to_float<T>(in[row * ldi + j]) + (bias ? to_float<T>(bias[j]) : 0.f);
  out[row * ldo + j] = from_float<T>(activate(z, act, pa, pb));
}

// eight bfloat16 values a thread (16 bytes), for widths that are multiples of 8 and aligned rows
__global__ void bias_act_bf16x8_kernel(bf16_t* __restrict__ out, int64_t ldo, const bf16_t* __restrict__ in, int64_t ldi,
                                       const bf16_t* __restrict__ bias, int width, int act, float pa, float pb) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const int64_t row = blockIdx.y;
  const int j = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (j >= width) return;
  const u32x4_t v = *reinterpret_cast<const u32x4_t*>(in + row * ldi + j);
  u32x4_t b = {0, 0, 0, 0};
  if (bias != nullptr) b = *reinterpret_cast<const u32x4_t*>(bias + j);
  u32x4_t o;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float lo = activate(bf16_to_float((bf16_t)(v[i] & 0xffff)) + bf16_to_float((bf16_t)(b[i] & 0xffff)), act, pa, pb);
    const float hi = activate(bf16_to_float((bf16_t)(v[i] >> 16)) + bf16_to_float((bf16_t)(b[i] >> 16)), act, pa, pb);
    o[i] = (uint32_t)float_to_bf16(lo) | ((uint32_t)float_to_bf16(hi) << 16);
  }
  *reinterpret_cast<u32x4_t*>(out + row * ldo + j) = o;
}

template <typename T, typename TW>
__global__ __launch_bounds__(256) void rmsnorm_cols_kernel(T* __restrict__ out, int64_t ldo, const T* __restrict__ x,
                                                           int64_t ldx, const TW* __restrict__ w, float offset,
                                                           float eps, int width) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  const T* xr = x + r * ldx;
  float ss = 0.f;
  for (int j = threadIdx.x; j < width; j += blockDim.x) {
    const float v = to_float<T>(xr[j]);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, scratch);       // (its barriers stand between every read of the row and the writes: in place is fine)
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  T* orow = out + r * ldo;
  for (int j = threadIdx.x; j < width; j += blockDim.x)
    orow[j] = from_float<T>(to_float<T>(xr[j]) * inv * weight_at<TW>(w, j, offset));
}

// x float32 [rows, d]; row r of out is made from row rows[r] (or r) of x.  The mean first, then the
// mean of the squared deviations from it, both as sums over the workgroup in a fixed order.
// Rows of up to 16 values a thread stay in registers between the three passes; wider rows are read again.
constexpr int kLayerNormKeep = 16;

template <typename TO, typename TW>
__global__ __launch_bounds__(256) void layernorm_kernel(TO* __restrict__ out, const float* __restrict__ x,
                                                        const TW* __restrict__ w, const int* __restrict__ rows,
                                                        float eps, int d) {
  __shared__ float scratch[16];
  const int64_t r = blockIdx.x;
  const float* xr = x + (int64_t)(rows ? rows[r] : r) * d;
  TO* o = out + r * d;
  if (d <= kLayerNormKeep * 256) {
    float v[kLayerNormKeep], wv[kLayerNormKeep];
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < kLayerNormKeep; ++i) {
      const int j = threadIdx.x + i * 256;
      v[i] = j < d ? xr[j] : 0.f;
      wv[i] = j < d ? to_float<TW>(w[j]) : 0.f;
      sum += v[i];
    }
    const float mean = block_sum(sum, scratch) / (float)d;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kLayerNormKeep; ++i) {
      const int j = threadIdx.x + i * 256;
      v[i] = j < d ? v[i] - mean : 0.f;
      ss = fmaf(v[i], v[i], ss);
    }
    const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)d + eps);
#pragma unroll
    for (int i = 0; i < kLayerNormKeep; ++i) {
      const int j = threadIdx.x + i * 256;
      if (j < d) o[j] = from_float<TO>(v[i] * inv * wv[i]);
    }
    return;
  }
  float sum = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) sum += xr[j];
  const float mean = block_sum(sum, scratch) / (float)d;
  float ss = 0.f;
  for (int j = threadIdx.x; j < d; j += blockDim.x) {
    const float v = xr[j] - mean;
    ss = fmaf(v, v, ss);
  }
  const float inv = 1.0f / sqrtf(block_sum(ss, scratch) / (float)d + eps);
  for (int j = threadIdx.x; j < d; j += blockDim.x) o[j] = from_float<TO>((xr[j] - mean) * inv * to_float<TW>(w[j]));
}

}  // namespace

HFEE_API int hfee_layernorm(void* out, int out_dtype, const float* x, const void* w, int w_dtype, const int* rows,
                            float eps, int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0, "layernorm: bad sizes n=%d d=%d", n, d);
  HFEE_REQUIRE(eps >= 0.f, "layernorm: eps must not be negative");
  if (n == 0) return 0;
#define LAUNCH(TO, TW) layernorm_kernel<TO, TW><<<n, 256, 0, stream>>>((TO*)out, x, (const TW*)w, rows, eps, d)
  if (out_dtype == 0 && w_dtype == 0) LAUNCH(float, float);
  else if (out_dtype == 0 && w_dtype == 1) LAUNCH(float, bf16_t);
  else if (out_dtype == 1 && w_dtype == 0) LAUNCH(bf16_t, float);
  else if (out_dtype == 1 && w_dtype == 1) LAUNCH(bf16_t, bf16_t);
  else return fail("layernorm: unknown dtypes");
#undef LAUNCH
  HFEE_CHECK_LAUNCH("layernorm");
  return 0;
}

// y_dtype / bias_dtype / w_dtype / next_dtype: 0 float32, 1 bfloat16.
HFEE_API int hfee_norm_add(float* x, const void* y, int y_dtype, const void* bias, int bias_dtype, const void* w,
                           int w_dtype, float offset, float eps, void* next, int next_dtype, const void* w2,
                           float eps2, int n, int d, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && d > 0, "norm_add: bad sizes n=%d d=%d", n, d);
  HFEE_REQUIRE(eps >= 0.f && eps2 >= 0.f, "norm_add: eps must not be negative");
  HFEE_REQUIRE(next == nullptr || w2 != nullptr, "norm_add: the following norm needs its weight");
  if (n == 0) return 0;
  const bool aligned = ((uintptr_t)x | (uintptr_t)y | (uintptr_t)bias | (uintptr_t)w | (uintptr_t)w2) % 16 == 0 &&
                       (uintptr_t)next % 8 == 0;
  if (offset == 0.f && y_dtype == 0 && (bias == nullptr || bias_dtype == 0) && w_dtype == 0 && d % 4 == 0 && d <= 16384 &&
      aligned) {
    const int quads = d / 4;
    const int nv = quads <= 1024 ? 1 : quads <= 2048 ? 2 : 4;
    int threads = ((quads + nv - 1) / nv + 63) / 64 * 64;
    if (threads > 1024) threads = 1024;
#define ROWS(TN, NV)                                                                                                  \
  norm_add_rows_kernel<TN, NV><<<n, threads, 0, stream>>>(x, (const float*)y, (const float*)bias, (const float*)w, eps, \
      (TN*)next, (const float*)w2, eps2, d)
    if (next_dtype == 1 && next != nullptr) {
      if (nv == 1) ROWS(bf16_t, 1); else if (nv == 2) ROWS(bf16_t, 2); else ROWS(bf16_t, 4);
    } else {
      if (nv == 1) ROWS(float, 1); else if (nv == 2) ROWS(float, 2); else ROWS(float, 4);
    }
#undef ROWS
    HFEE_CHECK_LAUNCH("norm_add");
    return 0;
  }
  const int code = (y_dtype & 1) | ((bias_dtype & 1) << 1) | ((w_dtype & 1) << 2) | ((next_dtype & 1) << 3);
#define CASE(c, TY, TB, TW, TN)                                                                                      \
  case c:                                                                                                            \
    norm_add_kernel<TY, TB, TW, TN><<<n, 256, 0, stream>>>(x, (const TY*)y, (const TB*)bias, (const TW*)w, offset,   \
        eps, (TN*)next, (const TW*)w2, eps2, d);                                                                     \
    break
  switch (code) {
    CASE(0, float, float, float, float);
    CASE(1, bf16_t, float, float, float);
    CASE(2, float, bf16_t, float, float);
    CASE(3, bf16_t, bf16_t, float, float);
    CASE(4, float, float, bf16_t, float);
    CASE(5, bf16_t, float, bf16_t, float);
    CASE(6, float, bf16_t, bf16_t, float);
    CASE(7, bf16_t, bf16_t, bf16_t, float);
    CASE(8, float, float, float, bf16_t);
    CASE(9, bf16_t, float, float, bf16_t);
    CASE(10, float, bf16_t, float, bf16_t);
    CASE(11, bf16_t, bf16_t, float, bf16_t);
    CASE(12, float, float, bf16_t, bf16_t);
    CASE(13, bf16_t, float, bf16_t, bf16_t);
    CASE(14, float, bf16_t, bf16_t, bf16_t);
    CASE(15, bf16_t, bf16_t, bf16_t, bf16_t);
  }
#undef CASE
  HFEE_CHECK_LAUNCH("norm_add");
  return 0;
}

HFEE_API int hfee_bias_act(void* out, int64_t ldo, const void* in, int64_t ldi, const void* bias, int dtype, int n,
                           int width, int act, float pa, float pb, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && width > 0, "bias_act: bad sizes");
  HFEE_REQUIRE(act >= ACT_NONE && act <= ACT_XIELU, "bias_act: unknown activation %d", act);
  HFEE_REQUIRE(n <= 65535 * 32, "bias_act: too many rows");
  if (n == 0) return 0;
  const bool wide = dtype == 1 && width % 8 == 0 && ldo % 8 == 0 && ldi % 8 == 0 &&
                    ((uintptr_t)out | (uintptr_t)in | (uintptr_t)bias) % 16 == 0;
  for (int r0 = 0; r0 < n; r0 += 65535) {
    const int rows = n - r0 < 65535 ? n - r0 : 65535;
    dim3 grid((width + 255) / 256, rows);
    if (wide)
      bias_act_bf16x8_kernel<<<dim3((width / 8 + 255) / 256, rows), 256, 0, stream>>>(
          (bf16_t*)out + (int64_t)r0 * ldo, ldo, (const bf16_t*)in + (int64_t)r0 * ldi, ldi, (const bf16_t*)bias, width, act, pa, pb);
    else if (dtype == 0)
      bias_act_kernel<float><<<grid, 256, 0, stream>>>((float*)out + (int64_t)r0 * ldo, ldo, (const float*)in + (int64_t)r0 * ldi,
                                                        ldi, (const float*)bias, width, act, pa, pb);
    else if (dtype == 1)
      bias_act_kernel<bf16_t><<<grid, 256, 0, stream>>>((bf16_t*)out + (int64_t)r0 * ldo, ldo, (const bf16_t*)in + (int64_t)r0 * ldi,
                                                         ldi, (const bf16_t*)bias, width, act, pa, pb);
    else
      return fail("bias_act: unknown dtype %d", dtype);
  }
  HFEE_CHECK_LAUNCH("bias_act");
  return 0;
}

HFEE_API int hfee_rmsnorm_cols(void* out, int64_t ldo, const void* x, int64_t ldx, int dtype, const void* w, int w_dtype,
                               float offset, float eps, int n, int width, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0 && width > 0, "rmsnorm_cols: bad sizes");
  HFEE_REQUIRE(eps >= 0.f, "rmsnorm_cols: eps must not be negative");
  if (n == 0) return 0;
#define LAUNCH(T, TW)                                                                                                \
  rmsnorm_cols_kernel<T, TW><<<n, 256, 0, stream>>>((T*)out, ldo, (const T*)x, ldx, (const TW*)w, offset, eps, width)
  if (dtype == 0 && w_dtype == 0) LAUNCH(float, float);
  else if (dtype == 0 && w_dtype == 1) LAUNCH(float, bf16_t);
  else if (dtype == 1 && w_dtype == 0) LAUNCH(bf16_t, float);
  else if (dtype == 1 && w_dtype == 1) LAUNCH(bf16_t, bf16_t);
  else return fail("rmsnorm_cols: unknown dtypes");
#undef LAUNCH
  HFEE_CHECK_LAUNCH("rmsnorm_cols");
  return 0;
}
