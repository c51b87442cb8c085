// Layout of the paged key/value cache of one layer.
//
//   keys    k_pages[page][kv_head][slot][d]               one key row of head_dim values is contiguous
//   values  v_pages[page][kv_head][slot / 16][d][slot % 16]  transposed inside groups of 16 slots: the 16
//                                                          slots of one dimension are contiguous
// page_size slots a page (a multiple of 16), slot = position % page_size.  Everything one kv head
// holds on a page is one contiguous block (page_size * head_dim values) for keys
// and for values.  Keys are laid out for Q.K^T, whose sum runs over d; values
// are transposed so that P.V, whose sum runs over the slots, can feed the
// matrix cores straight from memory: an MFMA operand wants the summed index
// contiguous in each lane.  The values are transposed by groups of 16 slots and not by the page, so that the 16
// keys a wave multiplies at a time find their values of all dimensions in one run of head_dim * 16 values,
// whatever the page size: transposed by the page, a page of 64 slots puts the 16 slots of neighbouring dimensions
// 128 bytes apart, every lane of a load touches a cache line of its own, and decode attention over pages of 64
// took a quarter longer than over pages of 16.  (The reference keeps both as [block][slot][head][d]:
// v3/crates/rvllm-mem/src/kv_layout.rs:1-46; it has no matrix-core attention of
// its own to lay values out for.)
#pragma once

#include <stddef.h>

__host__ __device__ __forceinline__ size_t rv_k_index(int page, int kvh, int slot, int d, int nkv, int page_size,
                                                       int hd) {
  return (((size_t)page * nkv + kvh) * page_size + slot) * hd + d;
}

#define RV_V_GROUP 16  // slots whose values of one dimension lie side by side

__host__ __device__ __forceinline__ size_t rv_v_index(int page, int kvh, int slot, int d, int nkv, int page_size,
                                                       int hd) {
  return (((size_t)page * nkv + kvh) * page_size + (size_t)(slot & ~(RV_V_GROUP - 1))) * hd + (size_t)d * RV_V_GROUP +
         (slot & (RV_V_GROUP - 1));
}
