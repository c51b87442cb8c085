// Layout of the paged key/value cache of one layer.
//
//   keys    k_pages[page][kv_head][slot][d]     one key row of head_dim values is contiguous
//   values  v_pages[page][kv_head][d][slot]     transposed inside the page: the slots of one
//                                               dimension are contiguous
// page_size slots a page, slot = position % page_size.  Everything one kv head
// holds on a page is one contiguous block (page_size * head_dim values) for keys
// and for values.  Keys are laid out for Q.K^T, whose sum runs over d; values
// are transposed so that P.V, whose sum runs over the slots, can feed the
// matrix cores straight from memory: an MFMA operand wants the summed index
// contiguous in each lane.  (The reference keeps both as [block][slot][head][d]:
// v3/crates/rvllm-mem/src/kv_layout.rs:1-46; it has no matrix-core attention of
// its own to lay values out for.)
#pragma once

#include <stddef.h>

__host__ __device__ __forceinline__ size_t rv_k_index(int page, int kvh, int slot, int d, int nkv, int page_size,
                                                       int hd) {
  return (((size_t)page * nkv + kvh) * page_size + slot) * hd + d;
}

__host__ __device__ __forceinline__ size_t rv_v_index(int page, int kvh, int slot, int d, int nkv, int page_size,
                                                       int hd) {
  return (((size_t)page * nkv + kvh) * hd + d) * page_size + slot;
}
