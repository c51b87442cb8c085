// Attention over the paged cache for any batch of tokens: portions of prompts
// beside single decoded tokens.  One wave handles one (token, query head); it
// walks the keys that the token may see in order of position, in tiles of 64,
// with an online softmax.  The keys of the token's own portion are in the cache
// already (they are written before attention runs), so a decoded token is a
// portion of one.
//
//   visible keys   j <= p, and for a window layer j >= p - window + 1
//                  (gemma4_layer_exec.rs:801-804, paged_attention_sm89.cu:96-105)
//   score          s = scale * sum_d q[d] * k[j,d]          (paged_attention_sm89.cu:125-137)
//   grouping       kv_head = head / (nq / nkv)              (paged_attention_sm89.cu:71)
//   softmax * V    m' = max(m, s); acc = acc*e^(m-m') + e^(s-m')*v; l likewise; out = acc / l
//                  (paged_attention_sm89.cu:145-157)
// Scores, softmax and the weighted sum are 32-bit.  Tiles start at the first
// visible key, which depends on the token's position alone, so the order of
// the additions for a token is the same however the batch was cut.
//
// This is the kernel of the 32-bit path, and of the bf16 path for head sizes
// without a matrix-core kernel.
#include <math.h>

#include "common.h"
#include "kv_layout.h"

#define ATT_MAX_HD 512
#define ATT_DIMS_PER_LANE (ATT_MAX_HD / RV_WAVE)

template <typename T>
__global__ void paged_attention_generic_kernel(const T* __restrict__ q, const T* __restrict__ k_pages,
                                               const T* __restrict__ v_pages, const int* __restrict__ block_table,
                                               int table_width, const int* __restrict__ positions,
                                               const int* __restrict__ token_req, T* __restrict__ out, int nq, int nkv,
                                               int hd, int page_size, int num_pages, int window, float scale) {
  __shared__ float q_s[ATT_MAX_HD];
  __shared__ float p_s[RV_WAVE];
  __shared__ int page_s[RV_WAVE];

  const int lane = threadIdx.x;
  const int t = blockIdx.x / nq;
  const int h = blockIdx.x % nq;
  const int kvh = h / (nq / nkv);
  const int p = positions[t];
  const int req = token_req[t];
  const int* table = block_table + (size_t)req * table_width;
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;

  const T* qr = q + ((size_t)t * nq + h) * hd;
  for (int d = lane; d < hd; d += RV_WAVE) q_s[d] = rv_to_float(qr[d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[ATT_DIMS_PER_LANE];
#pragma unroll
  for (int i = 0; i < ATT_DIMS_PER_LANE; ++i) acc[i] = 0.f;

  for (int start = lo; start <= p; start += RV_WAVE) {
    const int j = start + lane;
    float s = -INFINITY;
    int my_page = -1;
    if (j <= p) {
      const int logical = j / page_size;
      const int page = logical < table_width ? table[logical] : -1;
      if (page >= 0 && page < num_pages) {
        my_page = page;
        const T* kr = k_pages + rv_k_index(page, kvh, j % page_size, 0, nkv, page_size, hd);
        float dot = 0.f;
        for (int d = 0; d < hd; ++d) dot = fmaf(q_s[d], rv_to_float(kr[d]), dot);
        s = dot * scale;
      } else {
        s = NAN;  // a visible key without a page is a fault of the caller; make it show
      }
    }
    const float tile_max = rv_wave_max(s);
    const float m_new = fmaxf(m, tile_max);
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // 0 on the first tile (m = -inf)
    l = l * corr + rv_wave_sum(pj);
    m = m_new;
    __syncthreads();  // the previous tile's p_s / page_s are no longer read
    p_s[lane] = pj;
    page_s[lane] = my_page;
    __syncthreads();
    const int count = (p - start + 1 < RV_WAVE) ? p - start + 1 : RV_WAVE;
#pragma unroll
    for (int i = 0; i < ATT_DIMS_PER_LANE; ++i) {
      const int d = lane + i * RV_WAVE;
      if (d < hd) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < count; ++jj) {
          const int pg = page_s[jj];
          const float v =
              pg >= 0 ? rv_to_float(v_pages[rv_v_index(pg, kvh, (start + jj) % page_size, d, nkv, page_size, hd)]) : 0.f;
          a = fmaf(p_s[jj], v, a);
        }
        acc[i] = a;
      }
    }
  }
  T* o = out + ((size_t)t * nq + h) * hd;
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < ATT_DIMS_PER_LANE; ++i) {
    const int d = lane + i * RV_WAVE;
    if (d < hd) o[d] = rv_from_float<T>(acc[i] * inv_l);
  }
}

extern "C" int rv_paged_attention_generic(hipStream_t stream, const void* q, const void* k_pages, const void* v_pages,
                                          const int* block_table, int table_width, const int* positions,
                                          const int* token_req, void* out, int dtype, int num_tokens, int nq, int nkv,
                                          int hd, int page_size, int num_pages, int window, float scale) {
  RV_CHECK(num_tokens >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention: bad head counts nq=%d nkv=%d", nq, nkv);
  RV_CHECK(hd > 0 && hd <= ATT_MAX_HD, "attention: head_dim %d must be in 1..%d", hd, ATT_MAX_HD);
  RV_CHECK(page_size > 0 && num_pages > 0 && table_width > 0, "attention: bad cache geometry");
  RV_CHECK(page_size % RV_V_GROUP == 0, "attention: page_size %d must be a multiple of %d", page_size, RV_V_GROUP);
  RV_CHECK(window >= 0, "attention: window %d must be >= 0 (0 = every key)", window);
  if (num_tokens == 0) return 0;
  RV_CHECK((long long)num_tokens * nq < (1ll << 31), "attention: too many (token, head) pairs");
  dim3 grid(num_tokens * nq), block(RV_WAVE);
  if (dtype == RV_F32)
    paged_attention_generic_kernel<float><<<grid, block, 0, stream>>>(
        (const float*)q, (const float*)k_pages, (const float*)v_pages, block_table, table_width, positions, token_req,
        (float*)out, nq, nkv, hd, page_size, num_pages, window, scale);
  else if (dtype == RV_BF16)
    paged_attention_generic_kernel<bf16_t><<<grid, block, 0, stream>>>(
        (const bf16_t*)q, (const bf16_t*)k_pages, (const bf16_t*)v_pages, block_table, table_width, positions,
        token_req, (bf16_t*)out, nq, nkv, hd, page_size, num_pages, window, scale);
  else
    return rv_fail("attention: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("paged_attention_generic");
  return 0;
}
