// Attention whose heads talk to one another before the softmax, over keys that double as values.
//
//   prepare:  q and k are rotated in the first 2 * half dims of each head (pairs (i, i + half)) and
//             then, if asked, divided by their root mean square over the head (no weight); q in
//             place; the key as it is scored and the key as it was projected (the value) go into
//             the token's slot of the paged cache.
//   attend:   for a token at position p the keys j of [first(p), p], first(p) the start of p's
//             chunk (chunk = 0: position 0); raw_g(j) = q_g . k_kv(g)(j) * scale for every head g;
//             s_h(j) = sum_g mix[h][g] raw_g(j) (no mix: s = raw); a softmax over j whose
//             denominator may hold one more term exp(sink_h) without a value (a learned number a
//             head, or zero); out_h = sum_j p_h(j) v_kv(h)(j).
//
// The cache layer here is that of attention with key and value sizes of their own (`KvLayout`), both
// sizes D: [pages][kv_heads][page_size * 2 D], the scored keys of a (page, head) as [slot][D], then the
// values transposed as [D][slot].
//
// One workgroup a token takes all heads, since every head's weights need every head's scores.
// Keys are taken in tiles of 64 counted from first(p), so which thread adds which term in which
// order depends on positions only: a token's result does not change with the way its sequence
// was cut into steps, with the batch around it or with page numbers.  Everything is summed in
// float32; prompt portions and single tokens run the same kernel.
#include "attention_kv.h"

using namespace hfee;

namespace {

typedef KvLayout MixLayout;      // dk = dv = the head's size

constexpr int kPerLane = 8;     // heads of up to 512 dims: a lane holds dims lane, lane + 64, ...

// One wave a head row (query heads first, then key heads), as many rows a workgroup as it has waves.
template <typename T>
__global__ __launch_bounds__(256) void mix_prepare_kernel(
    T* __restrict__ q, int64_t ldq, const T* __restrict__ k, int64_t ldk, int num_heads, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_tables, int bt_stride,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int half, int norm, float eps,
    T* __restrict__ cache, MixLayout lay) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int wave = blockIdx.y * (blockDim.x >> 6) + (threadIdx.x >> 6), waves = gridDim.y * (blockDim.x >> 6);
  const int pos = positions[t], D = lay.dk;
  const float* c = cos_t + (int64_t)pos * half;
  const float* s = sin_t + (int64_t)pos * half;
  const int rows = num_heads + (k != nullptr ? lay.kv_heads : 0);
  for (int row = wave; row < rows; row += waves) {
    const bool is_q = row < num_heads;
    if (is_q && q == nullptr) continue;
    const T* src = is_q ? q + (int64_t)t * ldq + (int64_t)row * D : k + (int64_t)t * ldk + (int64_t)(row - num_heads) * D;
    float own[kPerLane], turned[kPerLane];
    float ss = 0.f;
#pragma unroll
    for (int r = 0; r < kPerLane; ++r) {
      const int d = lane + 64 * r;
      own[r] = turned[r] = 0.f;
      if (d < D) {
        own[r] = to_float<T>(src[d]);
        float v = own[r];
        if (d < half) v = own[r] * c[d] - to_float<T>(src[d + half]) * s[d];
        else if (d < 2 * half) v = own[r] * c[d - half] + to_float<T>(src[d - half]) * s[d - half];
        turned[r] = v;
        ss = fmaf(v, v, ss);
      }
    }
    ss = wave_sum(ss);
    const float inv = norm ? 1.0f / sqrtf(ss / (float)D + eps) : 1.0f;
    if (is_q) {
      T* dst = q + (int64_t)t * ldq + (int64_t)row * D;
#pragma unroll
      for (int r = 0; r < kPerLane; ++r) {
        const int d = lane + 64 * r;
        if (d < D) dst[d] = from_float<T>(turned[r] * inv);
      }
    } else {
      const int page = block_tables[(int64_t)token_segment[t] * bt_stride + (pos >> lay.page_shift)];
      const int kvh = row - num_heads, slot = pos & (lay.page_size - 1);
#pragma unroll
      for (int r = 0; r < kPerLane; ++r) {
        const int d = lane + 64 * r;
        if (d < D) {
          cache[lay.key_offset(page, kvh, slot, d)] = finite_for_cache<T>(from_float<T>(turned[r] * inv));
          cache[lay.value_offset(page, kvh, slot, d)] = finite_for_cache<T>(from_float<T>(own[r]));
        }
      }
    }
  }
}

constexpr int kKeyTile = 64;
constexpr int kMaxAcc = 16;     // output elements a thread: num_heads * dim <= 16 * threads

// sink_mode 0: none; 1: exp(0) joins the denominator; 2: exp(sinks[h]) does.
template <typename T>
__global__ __launch_bounds__(1024) void mix_attend_kernel(
    T* __restrict__ out, int64_t ld_out, const T* __restrict__ q, int64_t ldq, const T* __restrict__ cache, MixLayout lay,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_tables,
    int bt_stride, int num_heads, float scale, const float* __restrict__ mix, int chunk, int sink_mode,
    const float* __restrict__ sinks) {
  extern __shared__ float lds[];
  const int H = num_heads, D = lay.dk, tid = threadIdx.x, threads = blockDim.x;
  float* qs = lds;                         // [H][D]
  float* ms = qs + H * D;                  // [H][H] (unused without a mix)
  float* raw = ms + H * H;                 // [H][64]
  float* es = raw + H * kKeyTile;          // [H][64]
  float* run_m = es + H * kKeyTile;        // [H] running maximum
  float* run_l = run_m + H;                // [H] running denominator
  float* shrink = run_l + H;               // [H] what the tile before is multiplied by
  const int t = blockIdx.x;
  const int pos = positions[t];
  const int first = chunk > 0 ? pos / chunk * chunk : 0;
  const int* bt = block_tables + (int64_t)token_segment[t] * bt_stride;
  const int per_kv = H / lay.kv_heads;

  for (int e = tid; e < H * D; e += threads) qs[e] = to_float<T>(q[(int64_t)t * ldq + e]);
  if (mix != nullptr)
    for (int e = tid; e < H * H; e += threads) ms[e] = mix[e];
  for (int h = tid; h < H; h += threads) {
    run_m[h] = sink_mode == 0 ? -INFINITY : sink_mode == 1 ? 0.f : sinks[h];
    run_l[h] = sink_mode == 0 ? 0.f : 1.f;
  }
  float acc[kMaxAcc];
#pragma unroll
  for (int r = 0; r < kMaxAcc; ++r) acc[r] = 0.f;
  __syncthreads();

  for (int j0 = first; j0 <= pos; j0 += kKeyTile) {
    const int count = min(kKeyTile, pos - j0 + 1);
    // every head's raw score of every key of the tile
    for (int e = tid; e < H * kKeyTile; e += threads) {
      const int g = e / kKeyTile, jj = e - g * kKeyTile;
      float sc = 0.f;
      if (jj < count) {
        const int j = j0 + jj;
        const T* kr = cache + lay.key_offset(bt[j >> lay.page_shift], g / per_kv, j & (lay.page_size - 1), 0);
        const float* qg = qs + g * D;
        for (int d = 0; d < D; ++d) sc = fmaf(qg[d], to_float<T>(kr[d]), sc);
        sc *= scale;
      }
      raw[e] = sc;
    }
    __syncthreads();
    // the heads' scores mixed
    for (int e = tid; e < H * kKeyTile; e += threads) {
      const int h = e / kKeyTile, jj = e - h * kKeyTile;
      float sc = raw[e];
      if (mix != nullptr) {
        sc = 0.f;
        for (int g = 0; g < H; ++g) sc = fmaf(ms[h * H + g], raw[g * kKeyTile + jj], sc);
      }
      es[e] = sc;
    }
    __syncthreads();
    // a wave a head: the running maximum and denominator, the tile's weights
    for (int h = tid >> 6; h < H; h += threads >> 6) {
      const int lane = tid & 63;
      const bool valid = lane < count;
      const float sc = valid ? es[h * kKeyTile + lane] : -INFINITY;
      const float m_old = run_m[h];
      const float m_new = fmaxf(m_old, wave_max(sc));
      const float w = valid ? expf(sc - m_new) : 0.f;
      const float a = m_old == -INFINITY ? 0.f : expf(m_old - m_new);
      const float l = fmaf(run_l[h], a, wave_sum(w));
      es[h * kKeyTile + lane] = w;
      if (lane == 0) { run_m[h] = m_new; run_l[h] = l; shrink[h] = a; }
    }
    __syncthreads();
    // the weighted sum of the tile's values
#pragma unroll
    for (int r = 0; r < kMaxAcc; ++r) {
      const int e = tid + r * threads;
      if (e < H * D) {
        const int h = e / D, d = e - h * D, kvh = h / per_kv;
        float o = acc[r] * shrink[h];
        const float* w = es + h * kKeyTile;
        for (int jj = 0; jj < count; ++jj) {
          const int j = j0 + jj;
          o = fmaf(w[jj], to_float<T>(cache[lay.value_offset(bt[j >> lay.page_shift], kvh, j & (lay.page_size - 1), d)]), o);
        }
        acc[r] = o;
      }
    }
    __syncthreads();
  }
#pragma unroll
  for (int r = 0; r < kMaxAcc; ++r) {
    const int e = tid + r * threads;
    if (e < H * D) out[(int64_t)t * ld_out + e] = from_float<T>(acc[r] / run_l[e / D]);
  }
}

int make_mix_layout(MixLayout* lay, int kv_heads, int dim, int page_size) {
  return make_kv_layout(lay, kv_heads, dim, dim, page_size);
}

}  // namespace

// q: [n, num_heads * dim] or null; k: [n, kv_heads * dim] or null (then nothing is written).
HFEE_API int hfee_attention_mix_prepare(void* q, int64_t ldq, const void* k, int64_t ldk, int dtype, int num_heads,
                                        int kv_heads, int dim, const int* positions, const int* token_segment,
                                        const int* block_tables, int bt_stride, const float* cos_t, const float* sin_t,
                                        int half, int table_positions, int max_position, int norm, float eps,
                                        void* cache, int page_size, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "attention_mix_prepare: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(q != nullptr || k != nullptr, "attention_mix_prepare: nothing to do");
  HFEE_REQUIRE(num_heads > 0 && dim >= 1 && dim <= 64 * kPerLane, "attention_mix_prepare: heads of 1 to %d dims", 64 * kPerLane);
  HFEE_REQUIRE(half >= 0 && 2 * half <= dim && (half == 0 || (cos_t != nullptr && sin_t != nullptr)),
               "attention_mix_prepare: the rotated dims do not fit the head, or their tables are missing");
  HFEE_REQUIRE(half == 0 || max_position < table_positions,
               "attention_mix_prepare: position %d is beyond the rotation tables of %d positions", max_position, table_positions);
  HFEE_REQUIRE(eps >= 0.f, "attention_mix_prepare: eps must not be negative");
  MixLayout lay;
  if (make_mix_layout(&lay, kv_heads, dim, page_size)) return 1;
  if (k != nullptr)
    HFEE_REQUIRE(cache != nullptr && token_segment != nullptr && block_tables != nullptr && ldk >= (int64_t)kv_heads * dim,
                 "attention_mix_prepare: k, the cache and the block tables come together");
  HFEE_REQUIRE(q == nullptr || ldq >= (int64_t)num_heads * dim, "attention_mix_prepare: q rows too short");
  const int rows = num_heads + kv_heads;
  int parts = n >= 512 ? 1 : (rows + 3) / 4;
  if (parts > 16) parts = 16;
#define LAUNCH(T)                                                                                                     \
  mix_prepare_kernel<T><<<dim3(n, parts), 256, 0, stream>>>((T*)q, ldq, (const T*)k, ldk, num_heads, positions,       \
      token_segment, block_tables, bt_stride, cos_t, sin_t, half, norm, eps, (T*)cache, lay)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("attention_mix_prepare: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("attention_mix_prepare");
  return 0;
}

HFEE_API int hfee_attention_mix(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache, int dtype,
                                const int* positions, const int* token_segment, const int* block_tables, int bt_stride,
                                int num_heads, int kv_heads, int dim, int page_size, float scale, const float* mix,
                                int chunk, int sink_mode, const float* sinks, int n, hipStream_t stream) {
  HFEE_REQUIRE(n >= 0, "attention_mix: bad token count");
  if (n == 0) return 0;
  HFEE_REQUIRE(num_heads > 0 && kv_heads > 0 && num_heads % kv_heads == 0,
               "attention_mix: %d heads are not a multiple of %d kv heads", num_heads, kv_heads);
  HFEE_REQUIRE(chunk >= 0 && sink_mode >= 0 && sink_mode <= 2 && (sink_mode != 2 || sinks != nullptr),
               "attention_mix: bad chunk or sink");
  HFEE_REQUIRE(ldq >= (int64_t)num_heads * dim && ld_out >= (int64_t)num_heads * dim, "attention_mix: q/out row too short");
  MixLayout lay;
  if (make_mix_layout(&lay, kv_heads, dim, page_size)) return 1;
  const int64_t elements = (int64_t)num_heads * dim;
  HFEE_REQUIRE(elements <= (int64_t)kMaxAcc * 1024, "attention_mix: at most %d output elements a token", kMaxAcc * 1024);
  int threads = 256;
  while ((int64_t)threads * kMaxAcc < elements || (threads < 1024 && elements >= 4 * threads)) threads *= 2;
  if (threads > 1024) threads = 1024;
  const size_t lds = ((size_t)elements + (size_t)num_heads * num_heads + 2 * (size_t)num_heads * kKeyTile + 3 * num_heads) * sizeof(float);
  HFEE_REQUIRE(lds <= 64 * 1024, "attention_mix: %zu bytes of LDS a token are more than the 64 KB a workgroup has", lds);
#define LAUNCH(T)                                                                                                     \
  mix_attend_kernel<T><<<n, threads, lds, stream>>>((T*)out, ld_out, (const T*)q, ldq, (const T*)cache, lay, positions, \
      token_segment, block_tables, bt_stride, num_heads, scale, mix, chunk, sink_mode, sinks)
  if (dtype == 0) LAUNCH(float);
  else if (dtype == 1) LAUNCH(bf16_t);
  else return fail("attention_mix: unknown dtype %d", dtype);
#undef LAUNCH
  HFEE_CHECK_LAUNCH("attention_mix");
  return 0;
}
