// Attention whose heads' scores are mixed before the softmax, on the matrix cores; bfloat16, compiled
// for one number of heads H (HFEE_MIX_HEADS, a multiple of 4), of key heads G (HFEE_MIX_KV_HEADS) and one
// head size D (HFEE_MIX_DIM, a multiple of 32).  What is computed is what attention_mix.hip computes (keys of the query's chunk up to
// the query, scores of all heads mixed by a matrix, an optional sink, the keys as projected for values).
//
// A workgroup of four (or eight) waves takes an item: up to 16 consecutive rows of one sequence that lie in
// one chunk, and all heads, a wave a quarter (an eighth) of them.  Keys come in tiles of 16 that start at multiples of 16 of
// the sequence's positions (a tile lies in one page; keys before the chunk are masked), so what is added
// in which order depends on positions only.  A tile's steps:
//   0. everything the tile needs from memory is asked for at once: the keys of the wave's key heads (once a
//      key head, whichever of the wave's heads read it), their value columns, the rows' queries.
//   1. raw scores: v_mfma_f32_16x16x32_bf16, the tile's keys as the first operand, the rows' queries as
//      the second; lane l then holds, for row l % 16, the keys 4 (l / 16) .. + 3: sixteen bytes of
//      raw[head][row][key] in LDS.
//   2. mixing on the vector units in float32: the wave's heads h, s_h = sum_g T[h][g] raw_g for the lane's
//      row and four keys; T comes transposed ([g][h]) through scalar loads, the same for all lanes.
//   3. the softmax's running maximum and sum for each (head, row), over the lane's four keys and the
//      four lanes of a row; the weights rounded to bfloat16 are, as they lie, the second operand of
//   4. v_mfma_f32_16x16x16_bf16 with four keys of a value column (8 bytes of the page) as the first:
//      out[head][16 dims][row] a register block.
// A single token is an item of one row.  Where a step has few items, the key tiles of an item are shared
// out over several workgroups (`splits`): each leaves its running maximum, its sum and its unscaled
// output in float32, and a second kernel joins them in the order of the splits; the sink belongs to the
// first split.
#include "attention_kv.h"

using namespace hfee;

#if !defined(HFEE_MIX_HEADS) || !defined(HFEE_MIX_KV_HEADS) || !defined(HFEE_MIX_DIM)
#error "compile with -DHFEE_MIX_HEADS=<heads> -DHFEE_MIX_KV_HEADS=<key heads> -DHFEE_MIX_DIM=<head size>"
#endif

namespace {

constexpr int H = HFEE_MIX_HEADS, G = HFEE_MIX_KV_HEADS, D = HFEE_MIX_DIM, PER_KV = H / G;
static_assert(H % G == 0, "heads are a multiple of key heads");
// (what a wave keeps in registers for all tiles, its heads' queries and outputs, is 3/8 of a register a
// head and dim: four waves where that fits their 512 registers, eight waves of half as many heads and
// 256 registers beyond)
constexpr int WAVES = H / 4 * D > 512 ? 8 : 4;
constexpr int HW = H / WAVES, KS = D / 32, DB = D / 16, ROWS = 16, KEYS = 16;
static_assert(H % WAVES == 0 && D % 32 == 0 && HW * D <= 512, "heads in fours or eights, head sizes in multiples of 32");
// the most key heads that the consecutive heads of a wave read
constexpr int NKV = (HW + PER_KV - 2) / PER_KV + 1 < G ? (HW + PER_KV - 2) / PER_KV + 1 : G;
// value columns wait in registers from the tile's start where they fit beside the outputs (else they are
// asked for head by head, behind the softmax)
constexpr bool EARLY_VALUES = HW * D / 4 + NKV * D / 4 + 72 <= (WAVES == 8 ? 256 : 512);

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

union Operand8 {
  u32x4 u;
  bf16x8 v;
};
union Operand4 {
  u32x2 u;
  s16x4 v;
};

__global__ __launch_bounds__(WAVES * 64) void mix_attend_bf16_kernel(
    bf16_t* __restrict__ out, int64_t ld_out, const bf16_t* __restrict__ q, int64_t ldq, const bf16_t* __restrict__ cache,
    KvLayout lay, const int* __restrict__ items, const int* __restrict__ block_tables, int bt_stride, float scale,
    const float* __restrict__ mix_t, int chunk, int sink_mode, const float* __restrict__ sinks, int splits,
    float* __restrict__ partial_ml, float* __restrict__ partial_o) {
  __shared__ float raw[H][ROWS][KEYS];
  const int4 item = reinterpret_cast<const int4*>(items)[blockIdx.x];
  const int row0 = item.x, rows = item.y, p0 = item.z;
  const int* bt = block_tables + (int64_t)item.w * bt_stride;
  const int lane = threadIdx.x & 63, r16 = lane & 15, kq = lane >> 4;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int first = chunk > 0 ? p0 / chunk * chunk : 0, last = p0 + rows - 1;
  const int my_row = r16 < rows ? r16 : rows - 1;
  const int kv0 = wave * HW / PER_KV;                       // the first key head that this wave's heads read
  const bf16_t* q_row = q + (int64_t)(row0 + my_row) * ldq + wave * HW * D + kq * 8;

  // this workgroup's share of the item's key tiles
  const int tile0 = first / KEYS, tiles = last / KEYS - tile0 + 1, share = (tiles + splits - 1) / splits;
  const int split = blockIdx.y;
  const int j_begin = (tile0 + split * share) * KEYS, j_end = min(tile0 + tiles, tile0 + (split + 1) * share) * KEYS;
  const int sinking = split == 0 ? sink_mode : 0;

  f32x4 o[HW][DB];
  float m[HW], l[HW];
#pragma unroll
  for (int hh = 0; hh < HW; ++hh) {
    m[hh] = sinking == 0 ? -INFINITY : sinking == 1 ? 0.f : sinks[wave * HW + hh];
    l[hh] = sinking == 0 ? 0.f : 1.f;
#pragma unroll
    for (int db = 0; db < DB; ++db) o[hh][db] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  for (int j0 = j_begin; j0 < j_end; j0 += KEYS) {
    const int page = bt[j0 >> lay.page_shift], slot0 = j0 & (lay.page_size - 1);
    // 0. the tile's loads
    Operand8 kop[NKV][KS];
    Operand4 vop[EARLY_VALUES ? NKV : 1][DB];
#pragma unroll
    for (int kv = 0; kv < NKV; ++kv) {
      const int kvh = min(kv0 + kv, G - 1);
      const bf16_t* kr = cache + lay.key_offset(page, kvh, slot0 + r16, kq * 8);
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) kop[kv][ks].u = *reinterpret_cast<const u32x4*>(kr + ks * 32);
      if constexpr (EARLY_VALUES) {
        const bf16_t* vr = cache + lay.value_offset(page, kvh, slot0 + kq * 4, r16);
#pragma unroll
        for (int db = 0; db < DB; ++db) vop[kv][db].u = *reinterpret_cast<const u32x2*>(vr + (int64_t)db * 16 * lay.page_size);
      }
    }
    // 1. raw scores of the wave's heads
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      const int g = wave * HW + hh, kv = g / PER_KV - kv0;
      f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        Operand8 qop;
        qop.u = *reinterpret_cast<const u32x4*>(q_row + hh * D + ks * 32);
#pragma unroll
        for (int c = 0; c < NKV; ++c)        // (which of the wave's key heads: the same for all lanes)
          if (c == kv) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kop[c][ks].v, qop.v, s, 0, 0, 0);
      }
      *reinterpret_cast<f32x4*>(&raw[g][r16][kq * 4]) = s * scale;
    }
    __syncthreads();
    // 2. the scores that enter the softmax
    f32x4 sc[HW];
    if (mix_t != nullptr) {
#pragma unroll
      for (int hh = 0; hh < HW; ++hh) sc[hh] = f32x4{0.f, 0.f, 0.f, 0.f};
      const float* tw = mix_t + wave * HW;
#pragma unroll 8
      for (int g = 0; g < H; ++g) {
        const f32x4 r = *reinterpret_cast<const f32x4*>(&raw[g][r16][kq * 4]);
#pragma unroll
        for (int hh = 0; hh < HW; ++hh) {
          const float w = tw[g * H + hh];
#pragma unroll
          for (int i = 0; i < 4; ++i) sc[hh][i] = fmaf(w, r[i], sc[hh][i]);
        }
      }
    } else {
#pragma unroll
      for (int hh = 0; hh < HW; ++hh) sc[hh] = *reinterpret_cast<const f32x4*>(&raw[wave * HW + hh][r16][kq * 4]);
    }
    __syncthreads();
    // 3. the running softmax of all the wave's heads (their exchanges between lanes side by side)
    bool seen[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = j0 + kq * 4 + i;
      seen[i] = j >= first && j <= p0 + r16 && r16 < rows;
    }
    float tmax[HW], psum[HW], shrink[HW];
    Operand4 pop[HW];
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      tmax[hh] = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (seen[i]) tmax[hh] = fmaxf(tmax[hh], sc[hh][i]);
    }
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) tmax[hh] = fmaxf(tmax[hh], __shfl_xor(tmax[hh], 16, kWave));
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) tmax[hh] = fmaxf(tmax[hh], __shfl_xor(tmax[hh], 32, kWave));
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      const float m_new = fmaxf(m[hh], tmax[hh]);
      float p[4];
      psum[hh] = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        p[i] = seen[i] ? expf(sc[hh][i] - m_new) : 0.f;
        psum[hh] += p[i];
      }
      shrink[hh] = m[hh] == -INFINITY ? 0.f : expf(m[hh] - m_new);      // (m_new is finite wherever m is)
      m[hh] = m_new;
      pop[hh].u = u32x2{(uint32_t)float_to_bf16(p[0]) | ((uint32_t)float_to_bf16(p[1]) << 16),
                        (uint32_t)float_to_bf16(p[2]) | ((uint32_t)float_to_bf16(p[3]) << 16)};
    }
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) psum[hh] += __shfl_xor(psum[hh], 16, kWave);
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) psum[hh] += __shfl_xor(psum[hh], 32, kWave);
    // 4. the weighted values
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      l[hh] = fmaf(l[hh], shrink[hh], psum[hh]);
      const int kv = (wave * HW + hh) / PER_KV - kv0;
      if constexpr (EARLY_VALUES) {
#pragma unroll
        for (int db = 0; db < DB; ++db) {
          const f32x4 before = o[hh][db] * shrink[hh];
#pragma unroll
          for (int c = 0; c < NKV; ++c)
            if (c == kv) o[hh][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vop[c][db].v, pop[hh].v, before, 0, 0, 0);
        }
      } else {
        const bf16_t* vr = cache + lay.value_offset(page, kv0 + kv, slot0 + kq * 4, r16);
#pragma unroll
        for (int db = 0; db < DB; ++db) vop[0][db].u = *reinterpret_cast<const u32x2*>(vr + (int64_t)db * 16 * lay.page_size);
#pragma unroll
        for (int db = 0; db < DB; ++db)
          o[hh][db] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vop[0][db].v, pop[hh].v, o[hh][db] * shrink[hh], 0, 0, 0);
      }
    }
  }
  // register i of lane l: dim 16 db + 4 (l / 16) + i of row l % 16
  if (splits > 1) {
    if (r16 < rows) {
#pragma unroll
      for (int hh = 0; hh < HW; ++hh) {
        const int64_t at = (((int64_t)blockIdx.x * splits + split) * H + wave * HW + hh) * ROWS + r16;
        if (kq == 0) {
          partial_ml[2 * at] = m[hh];
          partial_ml[2 * at + 1] = l[hh];
        }
#pragma unroll
        for (int db = 0; db < DB; ++db) *reinterpret_cast<f32x4*>(partial_o + at * D + db * 16 + kq * 4) = o[hh][db];
      }
    }
    return;
  }
  if (r16 < rows) {
#pragma unroll
    for (int hh = 0; hh < HW; ++hh) {
      const float inv = 1.0f / l[hh];
      bf16_t* dst = out + (int64_t)(row0 + r16) * ld_out + (wave * HW + hh) * D + kq * 4;
#pragma unroll
      for (int db = 0; db < DB; ++db) {
        const f32x4 v = o[hh][db] * inv;
        *reinterpret_cast<u32x2*>(dst + db * 16) = u32x2{(uint32_t)float_to_bf16(v[0]) | ((uint32_t)float_to_bf16(v[1]) << 16),
                                                        (uint32_t)float_to_bf16(v[2]) | ((uint32_t)float_to_bf16(v[3]) << 16)};
      }
    }
  }
}

// grid (items, heads): out[row][head] = sum_s o_s exp(m_s - M) / sum_s l_s exp(m_s - M), the splits in their order.
__global__ __launch_bounds__(256) void mix_join_kernel(bf16_t* __restrict__ out, int64_t ld_out, const int* __restrict__ items,
                                                       int splits, const float* __restrict__ partial_ml,
                                                       const float* __restrict__ partial_o) {
  const int4 item = reinterpret_cast<const int4*>(items)[blockIdx.x];
  const int row0 = item.x, rows = item.y, h = blockIdx.y;
  for (int e = threadIdx.x; e < rows * D; e += blockDim.x) {
    const int r = e / D, d = e - r * D;
    float top = -INFINITY;
    for (int s = 0; s < splits; ++s) top = fmaxf(top, partial_ml[2 * ((((int64_t)blockIdx.x * splits + s) * H + h) * ROWS + r)]);
    float sum = 0.f, value = 0.f;
    for (int s = 0; s < splits; ++s) {
      const int64_t at = (((int64_t)blockIdx.x * splits + s) * H + h) * ROWS + r;
      const float ms = partial_ml[2 * at];
      if (ms == -INFINITY) continue;                      // (a share in which the row saw nothing)
      const float w = expf(ms - top);
      sum = fmaf(partial_ml[2 * at + 1], w, sum);
      value = fmaf(partial_o[at * D + d], w, value);
    }
    out[(int64_t)(row0 + r) * ld_out + h * D + d] = float_to_bf16(value / sum);
  }
}

}  // namespace

HFEE_DEFINE_LAST_ERROR

HFEE_API int hfee_attention_mix_bf16_heads() { return H; }
HFEE_API int hfee_attention_mix_bf16_kv_heads() { return G; }
HFEE_API int hfee_attention_mix_bf16_dim() { return D; }

// items: int32 [count][4] on the device: first row, rows (1..16), first position, block-table row; the rows
// of an item are consecutive positions of one sequence within one chunk.  mix_t: float32 [H][H], the
// mixing matrix transposed (mix_t[g][h] multiplies head g's raw score into head h's), or null.
// splits > 1: every item's key tiles over so many workgroups; partial: count * splits * H * 16 * (D + 2) float32.
HFEE_API int hfee_attention_mix_bf16(void* out, int64_t ld_out, const void* q, int64_t ldq, const void* cache,
                                     const int* items, int count, const int* block_tables, int bt_stride, int kv_heads,
                                     int page_size, float scale, const float* mix_t, int chunk, int sink_mode,
                                     const float* sinks, int splits, float* partial, int64_t partial_floats,
                                     hipStream_t stream) {
  HFEE_REQUIRE(count >= 0, "attention_mix_bf16: bad item count");
  if (count == 0) return 0;
  HFEE_REQUIRE(kv_heads == G, "attention_mix_bf16: compiled for %d key heads, called with %d", G, kv_heads);
  HFEE_REQUIRE(chunk >= 0 && sink_mode >= 0 && sink_mode <= 2 && (sink_mode != 2 || sinks != nullptr),
               "attention_mix_bf16: bad chunk or sink");
  HFEE_REQUIRE(ldq >= (int64_t)H * D && ld_out >= (int64_t)H * D && ldq % 8 == 0 && ld_out % 4 == 0 &&
               (uintptr_t)q % 16 == 0 && (uintptr_t)out % 8 == 0 && (uintptr_t)cache % 16 == 0,
               "attention_mix_bf16: q and out rows too short or not aligned");
  HFEE_REQUIRE(splits >= 1 && splits <= 65535, "attention_mix_bf16: 1 to 65535 splits");
  const int64_t places = (int64_t)count * splits * H * ROWS;
  HFEE_REQUIRE(splits == 1 || (partial != nullptr && partial_floats >= places * (D + 2) && (uintptr_t)partial % 16 == 0),
               "attention_mix_bf16: the splits need %lld float32 of scratch", (long long)(places * (D + 2)));
  KvLayout lay;
  if (make_kv_layout(&lay, kv_heads, D, D, page_size)) return 1;
  float* partial_o = partial;                               // [places][D], then [places][2]
  float* partial_ml = partial != nullptr ? partial + places * D : nullptr;
  mix_attend_bf16_kernel<<<dim3(count, splits), WAVES * 64, 0, stream>>>(
      (bf16_t*)out, ld_out, (const bf16_t*)q, ldq, (const bf16_t*)cache, lay, items, block_tables, bt_stride, scale, mix_t, chunk,
      sink_mode, sinks, splits, partial_ml, partial_o);
  HFEE_CHECK_LAUNCH("attention_mix_bf16");
  if (splits > 1) {
    mix_join_kernel<<<dim3(count, H), 256, 0, stream>>>((bf16_t*)out, ld_out, items, splits, partial_ml, partial_o);
    HFEE_CHECK_LAUNCH("attention_mix_join");
  }
  return 0;
}
