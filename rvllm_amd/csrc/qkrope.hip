// Per-head query/key RMSNorm, rotation, and the write of keys and values into
// the paged cache, in one pass over the output of the fused q|k|v projection.
//
// One wave handles one head of one token.  Row t of `qkv` is
// [q (nq*hd) | k (nkv*hd) | v (nkv*hd)]  (gemma4_layer_exec.rs:754-758).
//   norm      per head over hd, gain (offset + w[d]), w shared by all heads
//             (v3/kernels/fused_qk_rmsnorm.cu:3-6,89-95); skipped when w is null
//   rotation  pairs (i, i + hd/2) for i < rot/2:
//               x'[i]      = x[i]*cos - x[i+hd/2]*sin
//               x'[i+hd/2] = x[i]*sin + x[i+hd/2]*cos
//             angle = float(pos) * inv_freq[i]  (v3/kernels/fused_rope_partial_f16kv.cu:50-65,
//             metal_host.rs:1160-1166); dimensions past rot/2 pass through
//   write     K (normed, rotated) and V (as projected) go to slot pos % page_size of
//             page = table[req, pos / page_size], in the layout of kv_layout.h
//             (the reference writes at the same point: fused_rope_partial_f16kv.cu:69-91);
//             a negative page skips the write
// Norm, angle, sine and cosine are 32-bit.
#include "common.h"
#include "kv_layout.h"

#define QKR_MAX_HD 512

// One value of the projection's output: stored as T, or the sum of `slices`
// 32-bit partial sums (the K slices of the product), added in their order.
template <typename T>
__device__ __forceinline__ float qkr_input(const void* qkv, int slices, long long slice_stride, size_t at) {
  if (slices == 0) return rv_to_float(((const T*)qkv)[at]);
  const float* p = (const float*)qkv + at;
  float sum = 0.f;
  int s = 0;
  for (; s + 4 <= slices; s += 4) {  // four loads in flight, added in the order of the slices
    const float a = p[(size_t)s * slice_stride], b = p[(size_t)(s + 1) * slice_stride];
    const float c = p[(size_t)(s + 2) * slice_stride], d = p[(size_t)(s + 3) * slice_stride];
    sum = (((sum + a) + b) + c) + d;
  }
  for (; s < slices; ++s) sum += p[(size_t)s * slice_stride];
  return sum;
}

template <typename T>
__global__ void qk_norm_rope_kv_write_kernel(const void* __restrict__ qkv, int slices, long long slice_stride,
                                             T* __restrict__ q_out,
                                             const void* __restrict__ q_w, const void* __restrict__ k_w, int w_f32,
                                             float eps, float offset, const float* __restrict__ inv_freq, int rot,
                                             const int* __restrict__ positions, const int* __restrict__ token_req,
                                             const int* __restrict__ block_table, int table_width,
                                             T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size,
                                             int num_pages, int nq, int nkv, int hd, int write_kv) {
  __shared__ float buf[4][QKR_MAX_HD];
  const int wave = threadIdx.x / RV_WAVE;
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int t = blockIdx.x;
  const int head = blockIdx.y * 4 + wave;
  const int total_heads = nq + 2 * nkv;
  if (head >= total_heads) return;  // whole wave leaves together; no block barrier below

  const size_t src = (size_t)t * total_heads * hd + (size_t)head * hd;  // first element of this head in qkv
  const bool is_q = head < nq;
  const bool is_k = !is_q && head < nq + nkv;
  const int pos = positions[t];

  T* dst = nullptr;
  if (is_q) {
    dst = q_out + ((size_t)t * nq + head) * hd;
  } else {
    if (!write_kv) return;
    const int req = token_req[t];
    const int logical = pos / page_size;
    if (logical >= table_width) return;
    const int page = block_table[(size_t)req * table_width + logical];
    if (page < 0 || page >= num_pages) return;
    const int slot = pos % page_size;
    if (is_k) {
      dst = k_pages + rv_k_index(page, head - nq, slot, 0, nkv, page_size, hd);
    } else {
      // values are stored as projected, transposed inside the page
      T* col = v_pages + rv_v_index(page, head - nq - nkv, slot, 0, nkv, page_size, hd);
      for (int d = lane; d < hd; d += RV_WAVE)
        col[(size_t)d * page_size] = rv_from_float<T>(qkr_input<T>(qkv, slices, slice_stride, src + d));
      return;
    }
  }

  float* x = buf[wave];
  const void* w = is_q ? q_w : k_w;
  float ss = 0.f;
  for (int d = lane; d < hd; d += RV_WAVE) {
    const float v = qkr_input<T>(qkv, slices, slice_stride, src + d);
    x[d] = v;
    ss += v * v;
  }
  if (w != nullptr) {
    ss = rv_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
    for (int d = lane; d < hd; d += RV_WAVE) {
      x[d] = x[d] * inv * (offset + rv_load_w(w, w_f32, d));
    }
  }
  __builtin_amdgcn_wave_barrier();
  __threadfence_block();

  const int half = hd / 2;
  const int rot_half = rot / 2;
  for (int i = lane; i < half; i += RV_WAVE) {
    const float a = x[i];
    const float b = x[i + half];
    if (i < rot_half) {
      const float angle = (float)pos * inv_freq[i];
      float s, c;
      sincosf(angle, &s, &c);
      dst[i] = rv_from_float<T>(a * c - b * s);
      dst[i + half] = rv_from_float<T>(a * s + b * c);
    } else {
      dst[i] = rv_from_float<T>(a);
      dst[i + half] = rv_from_float<T>(b);
    }
  }
}

// `slices` 0: qkv holds T values [tokens, (nq + 2 nkv) * hd]; otherwise 32-bit
// partial sums [slices][tokens][...], slice_stride elements apart.
extern "C" int rv_qk_norm_rope_kv_write(hipStream_t stream, const void* qkv, int slices, long long slice_stride,
                                        void* q_out, const void* q_w,
                                        const void* k_w, int w_f32, float eps, float offset, const float* inv_freq,
                                        int rot, const int* positions, const int* token_req, const int* block_table,
                                        int table_width, void* k_pages, void* v_pages, int page_size, int num_pages,
                                        int dtype, int num_tokens, int nq, int nkv, int hd, int write_kv) {
  RV_CHECK(num_tokens >= 0 && nq > 0 && nkv > 0, "qk_norm_rope: bad sizes T=%d nq=%d nkv=%d", num_tokens, nq, nkv);
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= (long long)num_tokens * (nq + 2 * nkv) * hd),
           "qk_norm_rope: bad partial sums");
  RV_CHECK(hd >= 2 && hd % 2 == 0 && hd <= QKR_MAX_HD, "qk_norm_rope: head_dim %d must be even and <= %d", hd,
           QKR_MAX_HD);
  RV_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0, "qk_norm_rope: rotary_dim %d must be even and <= head_dim %d", rot, hd);
  RV_CHECK(rot == 0 || inv_freq != nullptr, "qk_norm_rope: rotation needs inverse frequencies");
  RV_CHECK((q_w == nullptr) == (k_w == nullptr), "qk_norm_rope: query and key norm weights come together");
  RV_CHECK(!write_kv || (page_size > 0 && num_pages > 0 && table_width > 0 && block_table && k_pages && v_pages),
           "qk_norm_rope: cache write needs pages and a block table");
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens, rv_div_up(nq + 2 * nkv, 4)), block(4 * RV_WAVE);
  if (dtype == RV_F32)
    qk_norm_rope_kv_write_kernel<float><<<grid, block, 0, stream>>>(
        qkv, slices, slice_stride, (float*)q_out, q_w, k_w, w_f32, eps, offset, inv_freq, rot, positions, token_req,
        block_table, table_width, (float*)k_pages, (float*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv);
  else if (dtype == RV_BF16)
    qk_norm_rope_kv_write_kernel<bf16_t><<<grid, block, 0, stream>>>(
        qkv, slices, slice_stride, (bf16_t*)q_out, q_w, k_w, w_f32, eps, offset, inv_freq, rot, positions, token_req,
        block_table, table_width, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv);
  else
    return rv_fail("qk_norm_rope: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("qk_norm_rope_kv_write");
  return 0;
}
