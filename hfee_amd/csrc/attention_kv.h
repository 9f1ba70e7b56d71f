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

// What a query at position p sees: the keys first_key(p) .. p, and the pooled blocks 0 .. pooled_blocks(p) - 1
// (block b holds the positions b * pool .. b * pool + pool - 1 and is seen once all of them have left the
// window: b * pool + pool - 1 <= p - window).  The pooled blocks are a cache layer of their own, of the same
// sizes and the same arrangement a page as the tokens', with block tables of its own: block b is its entry b.
struct KeySight {
  int window;               // 0: every earlier position
  int pool;                 // 0: no pooled blocks
  float softcap;            // 0: scores as they are
  const void* pooled;       // the pooled blocks' cache layer
  const int* pool_tables;   // its block tables, a row a segment as the tokens' have
  int pool_bt_stride;

  __host__ __device__ __forceinline__ int first_key(int p) const { return window > 0 && p - window + 1 > 0 ? p - window + 1 : 0; }
  __host__ __device__ __forceinline__ int pooled_blocks(int p) const {
    return pool > 0 && window > 0 && p - window + 1 >= pool ? (p - window + 1) / pool : 0;
  }
  __device__ __forceinline__ float capped(float s) const { return softcap > 0.f ? softcap * tanhf(s / softcap) : s; }
};

inline int make_key_sight(KeySight* out, int window, int pool, float softcap, const void* pooled, const int* pool_tables,
                          int pool_bt_stride) {
  if (window < 0 || pool < 0 || !(softcap >= 0.f)) return fail("bad window %d, pool %d or softcap %f", window, pool, (double)softcap);
  if (pool > 0 && window > 0 && (pooled == nullptr || pool_tables == nullptr))
    return fail("pooled blocks need their cache layer and its block tables");
  out->window = window;
  out->pool = window > 0 ? pool : 0;
  out->softcap = softcap;
  out->pooled = pooled;
  out->pool_tables = pool_tables;
  out->pool_bt_stride = pool_bt_stride;
  return 0;
}

}  // namespace hfee
