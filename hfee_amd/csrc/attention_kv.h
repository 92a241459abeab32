// The paged cache of attention whose keys and values have sizes of their own.
// One cache layer is [num_pages][kv_heads][page_size * (dk + dv)] elements: the keys of a
// (page, head) as [slot][dk], then its values transposed as [dv][slot].  A lane of the
// matrix-core kernels finds eight dims of one key in 16 contiguous bytes, and four
// neighbouring keys of one value column in 8.
#pragma once

#include "common.h"

namespace hfee {

struct KvLayout {
  int64_t page_stride;   // elements between pages: kv_heads * page_size * (dk + dv)
  int64_t head_stride;   // elements between the heads of a page: page_size * (dk + dv)
  int kv_heads;
  int dk;
  int dv;
  int page_size;
  int page_shift;        // log2(page_size)

  __host__ __device__ __forceinline__ int64_t keys_of(int page, int kvh) const {
    return (int64_t)page * page_stride + (int64_t)kvh * head_stride;
  }
  __host__ __device__ __forceinline__ int64_t values_of(int page, int kvh) const {
    return keys_of(page, kvh) + (int64_t)page_size * dk;
  }
  __host__ __device__ __forceinline__ int64_t key_offset(int page, int kvh, int slot, int d) const {
    return keys_of(page, kvh) + (int64_t)slot * dk + d;
  }
  __host__ __device__ __forceinline__ int64_t value_offset(int page, int kvh, int slot, int d) const {
    return values_of(page, kvh) + (int64_t)d * page_size + slot;
  }
};

inline int make_kv_layout(KvLayout* out, int kv_heads, int dk, int dv, int page_size) {
  if (page_size < 16 || (page_size & (page_size - 1)) != 0)
    return fail("page_size must be a power of two >= 16, got %d", page_size);
  if (kv_heads < 1 || dk < 1 || dv < 1) return fail("bad cache shape: kv_heads %d dk %d dv %d", kv_heads, dk, dv);
  out->kv_heads = kv_heads;
  out->dk = dk;
  out->dv = dv;
  out->page_size = page_size;
  out->head_stride = (int64_t)page_size * (dk + dv);
  out->page_stride = (int64_t)kv_heads * out->head_stride;
  int s = 0;
  while ((1 << s) < page_size) ++s;
  out->page_shift = s;
  return 0;
}

}  // namespace hfee
