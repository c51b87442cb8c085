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
// Norm, angle, sine and cosine are 32-bit.  The sines and cosines of a step's
// tokens are the same in every layer that rotates alike, so they come from a
// table made once a step (rope_table_kernel) instead of being worked out
// again in every layer.
#include "common.h"
#include "kv_layout.h"

#define QKR_MAX_HD 512
#define QKR_PAIRS (QKR_MAX_HD / 2 / RV_WAVE)  // pairs (i, i + hd/2) a lane holds at most

// cos_out[t][i] = cos(float(positions[t]) * inv_freq[i]), sin alike; i < half.
__global__ void rope_table_kernel(const float* __restrict__ inv_freq, const int* __restrict__ positions,
                                  float* __restrict__ cos_out, float* __restrict__ sin_out, int num_tokens, int half) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (long long)num_tokens * half) return;
  const int t = (int)(idx / half);
  const int i = (int)(idx - (long long)t * half);
  const float angle = (float)positions[t] * inv_freq[i];
  float s, c;
  sincosf(angle, &s, &c);
  cos_out[idx] = c;
  sin_out[idx] = s;
}

extern "C" int rv_rope_table(hipStream_t stream, const float* inv_freq, const int* positions, float* cos_out,
                             float* sin_out, int num_tokens, int half) {
  RV_CHECK(num_tokens >= 0 && half > 0 && inv_freq && positions && cos_out && sin_out, "rope_table: bad arguments");
  if (num_tokens == 0) return 0;
  const long long total = (long long)num_tokens * half;
  rope_table_kernel<<<dim3((unsigned)rv_div_up(total, 256)), dim3(256), 0, stream>>>(inv_freq, positions, cos_out,
                                                                                     sin_out, num_tokens, half);
  RV_LAUNCH_CHECK("rope_table");
  return 0;
}

// Values src[d] of one head for d = i and i + half, i = lane + 64 j: stored as
// T, or the sums of `slices` 32-bit partial sums (the K slices of the
// product), added in their order, four reads of a place in flight at a time.
template <typename T>
__device__ __forceinline__ void qkr_load(const void* qkv, int slices, long long slice_stride, size_t src, int lane,
                                         int half, float (&lo)[QKR_PAIRS], float (&hi)[QKR_PAIRS]) {
#pragma unroll
  for (int j = 0; j < QKR_PAIRS; ++j) lo[j] = hi[j] = 0.f;
  if (slices == 0) {
    const T* p = (const T*)qkv + src;
#pragma unroll
    for (int j = 0; j < QKR_PAIRS; ++j) {
      const int i = lane + j * RV_WAVE;
      if (i < half) {
        lo[j] = rv_to_float(p[i]);
        hi[j] = rv_to_float(p[i + half]);
      }
    }
    return;
  }
  const float* p = (const float*)qkv + src;
  int s = 0;
  for (; s + 4 <= slices; s += 4) {
    float a[4][QKR_PAIRS], b[4][QKR_PAIRS];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float* ps = p + (size_t)(s + u) * slice_stride;
#pragma unroll
      for (int j = 0; j < QKR_PAIRS; ++j) {
        const int i = lane + j * RV_WAVE;
        const int at = i < half ? i : 0;  // a lane past the end reads a valid place and drops it
        a[u][j] = ps[at];
        b[u][j] = ps[at + half];
      }
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
#pragma unroll
      for (int j = 0; j < QKR_PAIRS; ++j) {
        lo[j] += a[u][j];
        hi[j] += b[u][j];
      }
    }
  }
  for (; s < slices; ++s) {
    const float* ps = p + (size_t)s * slice_stride;
#pragma unroll
    for (int j = 0; j < QKR_PAIRS; ++j) {
      const int i = lane + j * RV_WAVE;
      const int at = i < half ? i : 0;
      lo[j] += ps[at];
      hi[j] += ps[at + half];
    }
  }
#pragma unroll
  for (int j = 0; j < QKR_PAIRS; ++j)
    if (lane + j * RV_WAVE >= half) lo[j] = hi[j] = 0.f;
}

// The values of a step's tokens, written a page at a time.  Values lie
// transposed inside a page (kv_layout.h), so a wave per token and head
// scatters them two or four bytes at a time; for prompt portions that is most
// of such a kernel's time.  Here a block takes one page of one request and one
// key/value head: thread d gathers the page's tokens at dimension d (for a
// fixed token the threads read one contiguous row) and writes row d of the
// page, 16 bytes at a time when the portion covers the whole page.  The
// kernels below give the blocks of extra rows of their grid to this work
// (`write_kv` 2), so that a prompt step writes keys and values in one launch.
struct ValuePages {
  const int* q_start;      // [requests + 1]
  const int* chunk_start;  // [requests]: position of each portion's first token
  int num_requests;
  int pages_per_request;   // a portion of n tokens touches at most (n - 1) / page_size + 2 pages
};

template <typename T>
__device__ void v_write_page(long long unit, const ValuePages& V, const T* __restrict__ qkv, T* __restrict__ v_pages,
                             const int* __restrict__ block_table, int table_width, int page_size, int num_pages,
                             int nq, int nkv, int hd) {
  if (unit >= (long long)V.pages_per_request * nkv * V.num_requests) return;
  const int rel = (int)(unit % V.pages_per_request);
  const int kvh = (int)(unit / V.pages_per_request % nkv);
  const int b = (int)(unit / V.pages_per_request / nkv);
  const int q0 = V.q_start[b];
  const int n = V.q_start[b + 1] - q0;
  const int s = V.chunk_start[b];
  if (n <= 0) return;
  const int lp = s / page_size + rel;
  const int lo = s > lp * page_size ? s : lp * page_size;
  const int hi = s + n < (lp + 1) * page_size ? s + n : (lp + 1) * page_size;
  if (lo >= hi || lp >= table_width) return;
  const int page = block_table[(size_t)b * table_width + lp];
  if (page < 0 || page >= num_pages) return;
  const size_t width = (size_t)(nq + 2 * nkv) * hd;
  const T* src = qkv + (size_t)(q0 + lo - s) * width + (size_t)(nq + nkv + kvh) * hd;  // token at position lo
  const int slot0 = lo - lp * page_size;
  constexpr int VEC = 16 / sizeof(T);  // elements of a 16-byte store
  const bool whole = hi - lo == page_size && page_size % VEC == 0;
  static_assert(RV_V_GROUP % VEC == 0, "a 16-byte store stays inside a group of slots");
  for (int d = threadIdx.x; d < hd; d += blockDim.x) {
    if (whole) {
      for (int g = 0; g < page_size; g += VEC) {
        T v[VEC];
#pragma unroll
        for (int i = 0; i < VEC; ++i) v[i] = src[(size_t)(g + i) * width + d];
        *(uint4*)(v_pages + rv_v_index(page, kvh, g, d, nkv, page_size, hd)) = *(const uint4*)v;
      }
    } else {
      for (int i = 0; i < hi - lo; ++i)
        v_pages[rv_v_index(page, kvh, slot0 + i, d, nkv, page_size, hd)] = src[(size_t)i * width + d];
    }
  }
}

template <typename T>
__global__ void qk_norm_rope_kv_write_kernel(const void* __restrict__ qkv, int slices, long long slice_stride,
                                             T* __restrict__ q_out,
                                             const void* __restrict__ q_w, const void* __restrict__ k_w, int w_f32,
                                             float eps, float offset, const float* __restrict__ rope_cos,
                                             const float* __restrict__ rope_sin, int rot,
                                             const int* __restrict__ positions, const int* __restrict__ token_req,
                                             const int* __restrict__ block_table, int table_width,
                                             T* __restrict__ k_pages, T* __restrict__ v_pages, int page_size,
                                             int num_pages, int nq, int nkv, int hd, int write_kv, ValuePages V) {
  const int wave = threadIdx.x / RV_WAVE;
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int head_rows = ((write_kv == 1 ? nq + 2 * nkv : nq + nkv) + 3) / 4;
  if ((int)blockIdx.y >= head_rows) {  // the rows of the grid beyond the heads write values a page at a time
    v_write_page<T>((long long)(blockIdx.y - head_rows) * gridDim.x + blockIdx.x, V, (const T*)qkv, v_pages, block_table,
                    table_width, page_size, num_pages, nq, nkv, hd);
    return;
  }
  const int t = blockIdx.x;
  const int head = blockIdx.y * 4 + wave;
  const int total_heads = nq + 2 * nkv;
  if (head >= total_heads) return;  // whole wave leaves together; there is no block barrier below

  const size_t src = (size_t)t * total_heads * hd + (size_t)head * hd;  // first element of this head in qkv
  const bool is_q = head < nq;
  const bool is_k = !is_q && head < nq + nkv;
  const int half = hd / 2;
  const int rot_half = rot / 2;

  // The head's values, the angles' cosines and sines and the norm's weights are
  // asked for before anything waits (on the position, the table, the page).
  float lo[QKR_PAIRS], hi[QKR_PAIRS];
  qkr_load<T>(qkv, slices, slice_stride, src, lane, half, lo, hi);
  float c[QKR_PAIRS], s[QKR_PAIRS], w_lo[QKR_PAIRS], w_hi[QKR_PAIRS];
  const void* w = is_q ? q_w : k_w;
  const bool rotates = rot_half > 0 && (is_q || is_k);
#pragma unroll
  for (int j = 0; j < QKR_PAIRS; ++j) {
    const int i = lane + j * RV_WAVE;
    c[j] = 1.f, s[j] = 0.f, w_lo[j] = 0.f, w_hi[j] = 0.f;
    if (rotates && i < rot_half) {
      c[j] = rope_cos[(size_t)t * rot_half + i];
      s[j] = rope_sin[(size_t)t * rot_half + i];
    }
    if (w != nullptr && !(!is_q && !is_k) && i < half) {
      w_lo[j] = rv_load_w(w, w_f32, i);
      w_hi[j] = rv_load_w(w, w_f32, i + half);
    }
  }

  T* dst = nullptr;
  if (is_q) {
    dst = q_out + ((size_t)t * nq + head) * hd;
  } else {
    if (!write_kv) return;
    const int pos = positions[t];
    const int req = token_req[t];
    const int logical = pos / page_size;
    if (logical >= table_width) return;
    const int page = block_table[(size_t)req * table_width + logical];
    if (page < 0 || page >= num_pages) return;
    const int slot = pos % page_size;
    if (is_k) {
      dst = k_pages + rv_k_index(page, head - nq, slot, 0, nkv, page_size, hd);
    } else {
      if (write_kv == 2) return;  // values are written a page at a time by other blocks of this launch
      // values are stored as projected, transposed inside their group of 16 slots
      T* col = v_pages + rv_v_index(page, head - nq - nkv, slot, 0, nkv, page_size, hd);
#pragma unroll
      for (int j = 0; j < QKR_PAIRS; ++j) {
        const int i = lane + j * RV_WAVE;
        if (i < half) {
          col[(size_t)i * RV_V_GROUP] = rv_from_float<T>(lo[j]);
          col[(size_t)(i + half) * RV_V_GROUP] = rv_from_float<T>(hi[j]);
        }
      }
      return;
    }
  }

  if (w != nullptr) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < QKR_PAIRS; ++j) ss += lo[j] * lo[j] + hi[j] * hi[j];
    ss = rv_wave_sum(ss);
    const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
    for (int j = 0; j < QKR_PAIRS; ++j) {
      lo[j] = lo[j] * inv * (offset + w_lo[j]);
      hi[j] = hi[j] * inv * (offset + w_hi[j]);
    }
  }
#pragma unroll
  for (int j = 0; j < QKR_PAIRS; ++j) {
    const int i = lane + j * RV_WAVE;
    if (i >= half) continue;
    float a = lo[j], b = hi[j];
    if (i < rot_half) {
      const float ra = a * c[j] - b * s[j];
      const float rb = a * s[j] + b * c[j];
      a = ra, b = rb;
    }
    dst[i] = rv_from_float<T>(a);
    dst[i + half] = rv_from_float<T>(b);
  }
}

// The same work for head sizes that are multiples of 8 up to 256 (and rotated
// widths that are multiples of 8): a lane holds 4 neighbouring dimensions, so
// it reads and writes 8 or 16 bytes at a time instead of 2 or 4, and gets the
// other half of its pairs from the lane hd/8 away.
template <typename T>
struct QkrVec;
template <>
struct QkrVec<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 x = *(const float4*)p;
    v[0] = x.x, v[1] = x.y, v[2] = x.z, v[3] = x.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *(float4*)p = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct QkrVec<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[4]) {
    const uint2 x = *(const uint2*)p;
    v[0] = __uint_as_float(x.x << 16), v[1] = __uint_as_float(x.x & 0xffff0000u);
    v[2] = __uint_as_float(x.y << 16), v[3] = __uint_as_float(x.y & 0xffff0000u);
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[4]) {
    *(uint2*)p = make_uint2(rv_pack_bf16x2(v[0], v[1]), rv_pack_bf16x2(v[2], v[3]));
  }
};

// A wave takes HPW heads of one token, one after the other with all their reads asked for at once: the token's
// place in the cache and its cosines and sines, four times a head's bytes, are then fetched once for all of them.
// (One head a wave, a prompt portion is tens of thousands of waves that each fetch those again.)
template <typename T, int HPW>
__global__ void qk_norm_rope_kv_write_vec_kernel(const void* __restrict__ qkv, int slices, long long slice_stride,
                                                 T* __restrict__ q_out, const void* __restrict__ q_w,
                                                 const void* __restrict__ k_w, int w_f32, float eps, float offset,
                                                 const float* __restrict__ rope_cos, const float* __restrict__ rope_sin,
                                                 int rot, const int* __restrict__ positions,
                                                 const int* __restrict__ token_req, const int* __restrict__ block_table,
                                                 int table_width, T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                 int page_size, int num_pages, int nq, int nkv, int hd, int write_kv,
                                                 ValuePages V) {
  const int wave = threadIdx.x / RV_WAVE;
  const int lane = threadIdx.x & (RV_WAVE - 1);
  // the heads that waves take: queries; keys and, token by token, values if they go to the cache
  const int heads = write_kv == 0 ? nq : (write_kv == 1 ? nq + 2 * nkv : nq + nkv);
  const int head_rows = (heads + 4 * HPW - 1) / (4 * HPW);
  if ((int)blockIdx.y >= head_rows) {  // the rows of the grid beyond the heads write values a page at a time
    v_write_page<T>((long long)(blockIdx.y - head_rows) * gridDim.x + blockIdx.x, V, (const T*)qkv, v_pages, block_table,
                    table_width, page_size, num_pages, nq, nkv, hd);
    return;
  }
  const int t = blockIdx.x;
  const int head0 = (blockIdx.y * 4 + wave) * HPW;
  const int total_heads = nq + 2 * nkv;
  if (head0 >= heads) return;  // whole wave leaves together; there is no block barrier below

  const int half_lanes = hd / 8;          // lanes that hold one half of the head
  const bool active = lane < 2 * half_lanes;
  const int d0 = active ? lane * 4 : 0;   // a lane without dimensions reads a valid place and drops it
  const bool first_half = lane < half_lanes;
  const int i0 = first_half ? d0 : d0 - hd / 2;  // index of the lane's pairs
  const int rot_half = rot / 2;
  const bool lane_rotates = active && i0 < rot_half;

  // Everything is asked for up front and from places that are always there, so that no read waits behind another
  // or behind a branch: at a few tokens a step this kernel is as long as its chain of round trips to memory.
  // First the token's place in the cache, which is two reads one after the other.
  int pos = 0, req = 0;
  if (write_kv != 0) {  // the same for the whole launch
    pos = positions[t];
    req = token_req[t];
  }
  // the heads' values: stored as T, or the sums of the product's K slices in their order; a head beyond the last
  // repeats the last one and stores nothing
  float x[HPW][4];
#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int head = head0 + j < heads ? head0 + j : heads - 1;
    const size_t src = (size_t)t * total_heads * hd + (size_t)head * hd;  // first element of this head in qkv
    x[j][0] = x[j][1] = x[j][2] = x[j][3] = 0.f;
    if (slices == 0) {
      QkrVec<T>::load((const T*)qkv + src + d0, x[j]);
    } else {
      const float* p = (const float*)qkv + src + d0;
      int s = 0;
      for (; s + 4 <= slices; s += 4) {  // four reads in flight
        const float4 a = *(const float4*)(p + (size_t)s * slice_stride);
        const float4 b = *(const float4*)(p + (size_t)(s + 1) * slice_stride);
        const float4 c = *(const float4*)(p + (size_t)(s + 2) * slice_stride);
        const float4 d = *(const float4*)(p + (size_t)(s + 3) * slice_stride);
        x[j][0] = (((x[j][0] + a.x) + b.x) + c.x) + d.x;
        x[j][1] = (((x[j][1] + a.y) + b.y) + c.y) + d.y;
        x[j][2] = (((x[j][2] + a.z) + b.z) + c.z) + d.z;
        x[j][3] = (((x[j][3] + a.w) + b.w) + c.w) + d.w;
      }
      for (; s < slices; ++s) {
        const float4 a = *(const float4*)(p + (size_t)s * slice_stride);
        x[j][0] += a.x, x[j][1] += a.y, x[j][2] += a.z, x[j][3] += a.w;
      }
    }
    if (!active) x[j][0] = x[j][1] = x[j][2] = x[j][3] = 0.f;
  }
  float c[4] = {1.f, 1.f, 1.f, 1.f}, sn[4] = {0.f, 0.f, 0.f, 0.f};
  if (rot_half > 0) {  // the same for the whole launch; a lane that does not rotate reads the first pairs and drops them
    const int i_safe = lane_rotates ? i0 : 0;
    QkrVec<float>::load(rope_cos + (size_t)t * rot_half + i_safe, c);
    QkrVec<float>::load(rope_sin + (size_t)t * rot_half + i_safe, sn);
  }
  float g_q[4] = {0.f, 0.f, 0.f, 0.f}, g_k[4] = {0.f, 0.f, 0.f, 0.f};
  if (q_w != nullptr) {  // the same for the whole launch; the weights of queries and keys come together
    rv_load_w_vec<4>(q_w, w_f32, d0, g_q);
    rv_load_w_vec<4>(k_w, w_f32, d0, g_k);
  }
  const int logical = write_kv != 0 ? pos / page_size : 0;  // without a cache there is no page size either
  const bool in_table = write_kv != 0 && logical < table_width;
  int page = -1;
  if (write_kv != 0) page = block_table[(size_t)req * table_width + (in_table ? logical : 0)];
  if (!in_table || page >= num_pages) page = -1;
  const int slot = write_kv != 0 ? pos % page_size : 0;

#pragma unroll
  for (int j = 0; j < HPW; ++j) {
    const int head = head0 + j;
    if (head >= heads) break;  // the same for the whole wave, as all that follows
    const bool is_q = head < nq;
    const bool is_k = !is_q && head < nq + nkv;
    T* dst = nullptr;
    if (is_q) {
      dst = q_out + ((size_t)t * nq + head) * hd;
    } else {
      if (page < 0) continue;
      if (is_k) {
        dst = k_pages + rv_k_index(page, head - nq, slot, 0, nkv, page_size, hd);
      } else {
        // values are stored as projected, transposed inside their group of 16 slots
        T* col = v_pages + rv_v_index(page, head - nq - nkv, slot, 0, nkv, page_size, hd);
        if (active) {
#pragma unroll
          for (int i = 0; i < 4; ++i) col[(size_t)(d0 + i) * RV_V_GROUP] = rv_from_float<T>(x[j][i]);
        }
        continue;
      }
    }
    if (q_w != nullptr) {
      float ss = x[j][0] * x[j][0] + x[j][1] * x[j][1] + x[j][2] * x[j][2] + x[j][3] * x[j][3];
      ss = rv_wave_sum(ss);
      const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
      for (int i = 0; i < 4; ++i) x[j][i] = x[j][i] * inv * (offset + (is_q ? g_q[i] : g_k[i]));
    }
    if (rot_half > 0) {
      // the other half of each pair sits hd/8 lanes away; every lane takes part in the exchange
      const int partner = first_half ? lane + half_lanes : lane - half_lanes;
      const int from = active ? partner : lane;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float other = __shfl(x[j][i], from, RV_WAVE);
        if (lane_rotates) x[j][i] = first_half ? x[j][i] * c[i] - other * sn[i] : x[j][i] * c[i] + other * sn[i];
      }
    }
    if (active) QkrVec<T>::store(dst + d0, x[j]);
  }
}

// Prompt portions in bf16 (thousands of tokens, the projection whole): a lane holds 8 neighbouring dimensions
// (16 bytes), so a head of hd dimensions takes hd / 8 lanes (a power of two up to 32) and a wave works on 64 / (hd / 8)
// heads at a time, `PASSES` such sets one after the other with all their reads asked for at once; the token's
// cosines and sines, its place in the cache and the norm's weights are read once for all of them.  Sums and exchanges
// stay inside a head's lanes.  A third of the memory instructions of the kernel above for the same bytes; the values
// are written a page at a time by the extra rows of blocks, as there.
#define QKP_PASSES 3
__global__ void __launch_bounds__(256)
qk_norm_rope_prompt_kernel(const uint16_t* __restrict__ qkv, uint16_t* __restrict__ q_out, const void* __restrict__ q_w,
                           const void* __restrict__ k_w, int w_f32, float eps, float offset,
                           const float* __restrict__ rope_cos, const float* __restrict__ rope_sin, int rot,
                           const int* __restrict__ positions, const int* __restrict__ token_req,
                           const int* __restrict__ block_table, int table_width, uint16_t* __restrict__ k_pages,
                           uint16_t* __restrict__ v_pages, int page_size, int num_pages, int nq, int nkv, int hd,
                           int write_kv, int num_tokens, int waves_per_token, int head_rows, ValuePages V) {
  if ((int)blockIdx.y >= head_rows) {  // the rows of the grid beyond the heads write values a page at a time
    v_write_page<bf16_t>((long long)(blockIdx.y - head_rows) * gridDim.x + blockIdx.x, V, (const bf16_t*)qkv,
                         (bf16_t*)v_pages, block_table, table_width, page_size, num_pages, nq, nkv, hd);
    return;
  }
  const int lane = threadIdx.x & 63;
  const int wave_id = (blockIdx.y * gridDim.x + blockIdx.x) * 4 + (threadIdx.x >> 6);
  const int t = wave_id / waves_per_token;
  if (t >= num_tokens) return;  // the whole wave
  const int lph = hd >> 3;                    // lanes a head
  const int hpp = 64 / lph;                   // heads a pass
  const int hl = lane / lph;                  // this lane's head within a pass
  const int l = lane - hl * lph;              // this lane within its head
  const int d0 = l * 8;
  const int heads = write_kv != 0 ? nq + nkv : nq;  // queries, and keys if they go to the cache
  const int total_heads = nq + 2 * nkv;
  const int head_first = (wave_id - t * waves_per_token) * QKP_PASSES * hpp + hl;
  const size_t row = (size_t)t * total_heads * hd;

  uint4 raw[QKP_PASSES];
#pragma unroll
  for (int p = 0; p < QKP_PASSES; ++p) {
    const int head = head_first + p * hpp;
    raw[p] = *(const uint4*)(qkv + row + (size_t)(head < heads ? head : heads - 1) * hd + d0);  // past the end: dropped
  }
  const int rot_half = rot >> 1;
  const bool first_half = l < (lph >> 1);
  const int pd0 = first_half ? d0 : d0 - (hd >> 1);  // the pairs' index
  const bool turns = pd0 < rot_half;
  float c[8] = {1, 1, 1, 1, 1, 1, 1, 1}, sn[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  if (rot_half > 0) {
    const float* pc = rope_cos + (size_t)t * rot_half + (turns ? pd0 : 0);
    const float* pn = rope_sin + (size_t)t * rot_half + (turns ? pd0 : 0);
    const float4 c0 = *(const float4*)pc, c1 = *(const float4*)(pc + 4), n0 = *(const float4*)pn, n1 = *(const float4*)(pn + 4);
    c[0] = c0.x, c[1] = c0.y, c[2] = c0.z, c[3] = c0.w, c[4] = c1.x, c[5] = c1.y, c[6] = c1.z, c[7] = c1.w;
    sn[0] = n0.x, sn[1] = n0.y, sn[2] = n0.z, sn[3] = n0.w, sn[4] = n1.x, sn[5] = n1.y, sn[6] = n1.z, sn[7] = n1.w;
  }
  float g_q[8], g_k[8];
  if (q_w != nullptr) {
    rv_load_w_vec<8>(q_w, w_f32, d0, g_q);
    rv_load_w_vec<8>(k_w, w_f32, d0, g_k);
  }
  int page = -1, slot = 0;
  if (write_kv != 0) {
    const int pos = positions[t];
    const int logical = pos / page_size;
    slot = pos - logical * page_size;
    if (logical < table_width) page = block_table[(size_t)token_req[t] * table_width + logical];
    if (page >= num_pages) page = -1;
  }
#pragma unroll
  for (int p = 0; p < QKP_PASSES; ++p) {
    const int head = head_first + p * hpp;
    const bool there = head < heads;  // lanes of a head decide alike; the exchanges below take every lane
    const bool is_q = head < nq;
    float x[8];
    {
      const uint32_t u[4] = {raw[p].x, raw[p].y, raw[p].z, raw[p].w};
#pragma unroll
      for (int i = 0; i < 4; ++i) x[2 * i] = __uint_as_float(u[i] << 16), x[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
    }
    if (q_w != nullptr) {
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) ss += x[i] * x[i];
      for (int off = lph >> 1; off > 0; off >>= 1) ss += __shfl_xor(ss, off, RV_WAVE);  // over the head's lanes
      const float inv = 1.0f / sqrtf(ss / (float)hd + eps);
#pragma unroll
      for (int i = 0; i < 8; ++i) x[i] = x[i] * inv * (offset + (is_q ? g_q[i] : g_k[i]));
    }
    if (rot_half > 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const float other = __shfl_xor(x[i], lph >> 1, RV_WAVE);  // the other half of the pair
        if (turns) x[i] = first_half ? x[i] * c[i] - other * sn[i] : x[i] * c[i] + other * sn[i];
      }
    }
    if (!there) continue;
    uint16_t* dst;
    if (is_q) {
      dst = q_out + ((size_t)t * nq + head) * hd;
    } else {
      if (page < 0) continue;
      dst = k_pages + rv_k_index(page, head - nq, slot, 0, nkv, page_size, hd);
    }
    *(uint4*)(dst + d0) = make_uint4(rv_pack_bf16x2(x[0], x[1]), rv_pack_bf16x2(x[2], x[3]), rv_pack_bf16x2(x[4], x[5]),
                                     rv_pack_bf16x2(x[6], x[7]));
  }
}

// `slices` 0: qkv holds T values [tokens, (nq + 2 nkv) * hd]; otherwise 32-bit
// partial sums [slices][tokens][...], slice_stride elements apart.
extern "C" int rv_qk_norm_rope_kv_write(hipStream_t stream, const void* qkv, int slices, long long slice_stride,
                                        void* q_out, const void* q_w,
                                        const void* k_w, int w_f32, float eps, float offset, const float* rope_cos,
                                        const float* rope_sin, int rot, const int* positions, const int* token_req, const int* block_table,
                                        int table_width, void* k_pages, void* v_pages, int page_size, int num_pages,
                                        int dtype, int num_tokens, int nq, int nkv, int hd, int write_kv,
                                        const int* q_start, const int* chunk_start, int num_requests, int max_portion) {
  RV_CHECK(num_tokens >= 0 && nq > 0 && nkv > 0, "qk_norm_rope: bad sizes T=%d nq=%d nkv=%d", num_tokens, nq, nkv);
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= (long long)num_tokens * (nq + 2 * nkv) * hd),
           "qk_norm_rope: bad partial sums");
  RV_CHECK(hd >= 2 && hd % 2 == 0 && hd <= QKR_MAX_HD, "qk_norm_rope: head_dim %d must be even and <= %d", hd,
           QKR_MAX_HD);
  RV_CHECK(rot >= 0 && rot <= hd && rot % 2 == 0, "qk_norm_rope: rotary_dim %d must be even and <= head_dim %d", rot, hd);
  RV_CHECK(rot == 0 || (rope_cos != nullptr && rope_sin != nullptr), "qk_norm_rope: rotation needs the table of cosines and sines");
  RV_CHECK((q_w == nullptr) == (k_w == nullptr), "qk_norm_rope: query and key norm weights come together");
  RV_CHECK(!write_kv || (page_size > 0 && num_pages > 0 && table_width > 0 && block_table && k_pages && v_pages),
           "qk_norm_rope: cache write needs pages and a block table");
  RV_CHECK(!write_kv || page_size % RV_V_GROUP == 0, "qk_norm_rope: page_size %d must be a multiple of %d", page_size,
           RV_V_GROUP);
  if (num_tokens == 0) return 0;
  // write_kv 0: nothing goes to the cache; 1: keys and values, token by token; 2: keys token by token and values
  // a page at a time, by extra rows of blocks (for prompt portions; needs the step's portions and whole values,
  // not partial sums)
  RV_CHECK(write_kv >= 0 && write_kv <= 2, "qk_norm_rope: write_kv is 0, 1 or 2");
  ValuePages V = {q_start, chunk_start, num_requests, 0};
  const bool vec = hd % 8 == 0 && hd <= 4 * RV_WAVE && rot % 8 == 0;  // four dimensions a lane
  // the heads that waves take: queries; keys and, token by token, values if they go to the cache
  const int heads = write_kv == 0 ? nq : (write_kv == 1 ? nq + 2 * nkv : nq + nkv);
  // a prompt portion's waves take four heads each; a few tokens' take one, spread over the machine
  // (as many as give each of a block's four waves its share of the heads, four at most)
  const int hpw = vec && num_tokens >= 256 ? (heads >= 13 ? 4 : (heads + 3) / 4) : 1;
  int rows = rv_div_up(vec ? heads : (write_kv == 1 ? nq + 2 * nkv : nq + nkv), 4 * hpw);
  if (write_kv == 2) {
    RV_CHECK(slices == 0 && q_start && chunk_start && num_requests >= 1 && max_portion >= 1,
             "qk_norm_rope: values by pages need the step's portions and a projection that is already added up");
    V.pages_per_request = (max_portion - 1) / page_size + 2;
    const long long units = (long long)V.pages_per_request * nkv * num_requests;
    rows += (int)((units + num_tokens - 1) / num_tokens);
    RV_CHECK(rows <= 65535, "qk_norm_rope: too many pages of values for one launch");
  }
  // prompt portions in bf16 whose values go by pages: sixteen bytes a lane, several heads a wave at a time
  const int lph = hd / 8;
  if (write_kv == 2 && dtype == RV_BF16 && slices == 0 && hd % 8 == 0 && lph >= 2 && lph <= 32 && (lph & (lph - 1)) == 0 &&
      rot % 16 == 0 && num_tokens >= 256 && ((uintptr_t)qkv % 16) == 0 && ((uintptr_t)q_out % 16) == 0) {
    const int heads_kq = nq + nkv;
    const int per_wave = QKP_PASSES * (64 / lph);
    const int waves_per_token = rv_div_up(heads_kq, per_wave);
    const long long blocks = rv_div_up((long long)num_tokens * waves_per_token, 4);
    const int gx = num_tokens;  // the page writer's rows count their blocks by this width
    const int head_rows = rv_div_up(blocks, gx);
    const long long units = (long long)V.pages_per_request * nkv * num_requests;
    const int page_rows = (int)((units + gx - 1) / gx);
    RV_CHECK(head_rows + page_rows <= 65535, "qk_norm_rope: too many blocks for one launch");
    qk_norm_rope_prompt_kernel<<<dim3(gx, head_rows + page_rows), dim3(256), 0, stream>>>(
        (const uint16_t*)qkv, (uint16_t*)q_out, q_w, k_w, w_f32, eps, offset, rope_cos, rope_sin, rot, positions, token_req,
        block_table, table_width, (uint16_t*)k_pages, (uint16_t*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv,
        num_tokens, waves_per_token, head_rows, V);
    RV_LAUNCH_CHECK("qk_norm_rope_prompt");
    return 0;
  }
  dim3 grid(num_tokens, rows), block(4 * RV_WAVE);
#define QKR_VEC_LAUNCH(TT, HPW)                                                                                        \
  qk_norm_rope_kv_write_vec_kernel<TT, HPW><<<grid, block, 0, stream>>>(                                               \
      qkv, slices, slice_stride, (TT*)q_out, q_w, k_w, w_f32, eps, offset, rope_cos, rope_sin, rot, positions,         \
      token_req, block_table, table_width, (TT*)k_pages, (TT*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv, V)
  if (vec) {
    if (dtype == RV_F32) {
      if (hpw == 4) QKR_VEC_LAUNCH(float, 4); else if (hpw == 3) QKR_VEC_LAUNCH(float, 3);
      else if (hpw == 2) QKR_VEC_LAUNCH(float, 2); else QKR_VEC_LAUNCH(float, 1);
    } else if (dtype == RV_BF16) {
      if (hpw == 4) QKR_VEC_LAUNCH(bf16_t, 4); else if (hpw == 3) QKR_VEC_LAUNCH(bf16_t, 3);
      else if (hpw == 2) QKR_VEC_LAUNCH(bf16_t, 2); else QKR_VEC_LAUNCH(bf16_t, 1);
    } else {
      return rv_fail("qk_norm_rope: unsupported dtype %d", dtype);
    }
    RV_LAUNCH_CHECK("qk_norm_rope_kv_write");
    return 0;
  }
#undef QKR_VEC_LAUNCH
  if (dtype == RV_F32)
    qk_norm_rope_kv_write_kernel<float><<<grid, block, 0, stream>>>(
        qkv, slices, slice_stride, (float*)q_out, q_w, k_w, w_f32, eps, offset, rope_cos, rope_sin, rot, positions, token_req,
        block_table, table_width, (float*)k_pages, (float*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv, V);
  else if (dtype == RV_BF16)
    qk_norm_rope_kv_write_kernel<bf16_t><<<grid, block, 0, stream>>>(
        qkv, slices, slice_stride, (bf16_t*)q_out, q_w, k_w, w_f32, eps, offset, rope_cos, rope_sin, rot, positions, token_req,
        block_table, table_width, (bf16_t*)k_pages, (bf16_t*)v_pages, page_size, num_pages, nq, nkv, hd, write_kv, V);
  else
    return rv_fail("qk_norm_rope: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("qk_norm_rope_kv_write");
  return 0;
}
