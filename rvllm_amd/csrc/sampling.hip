// Choice of the next token on the device: arg-max of 32-bit logits, and the
// selection of the K largest logits for the host's seeded draw.
//
//   arg-max   NaN is skipped, equal maxima give the lowest id
//             (kernels/argmax.cu:16-25,81-130; pinned by
//             v3/crates/rvllm-invariants/tests/identity.rs:91-128)
//   top-K     the K largest by the key (ordered bits of the logit, then lower id
//             first), found by a radix select byte by byte; the output holds
//             (logit * 1/T, id) in no particular order, the host sorts it
//             (v3/kernels/sample_topk_f32.cu:1-13,68-117)
#include <math.h>

#include "common.h"

// ---------------------------------------------------------------------------
// arg-max in two stages, so that a row of 262 208 logits is read by many CUs.
// ---------------------------------------------------------------------------
struct Best {
  float v;
  int i;
};

__device__ __forceinline__ Best better(Best a, Best b) {
  // an empty slot has i < 0
  if (b.i < 0) return a;
  if (a.i < 0) return b;
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ __forceinline__ Best block_best(Best mine, Best* scratch) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int wave = threadIdx.x / RV_WAVE;
  const int nwaves = blockDim.x / RV_WAVE;
#pragma unroll
  for (int off = RV_WAVE / 2; off > 0; off >>= 1) {
    Best o;
    o.v = __shfl_xor(mine.v, off, RV_WAVE);
    o.i = __shfl_xor(mine.i, off, RV_WAVE);
    mine = better(mine, o);
  }
  if (lane == 0) scratch[wave] = mine;
  __syncthreads();
  Best r = scratch[0];
  for (int w = 1; w < nwaves; ++w) r = better(r, scratch[w]);
  return r;
}

__global__ void argmax_partial_kernel(const float* __restrict__ logits, int vocab, long long row_stride, int parts,
                                      float* __restrict__ part_val, int* __restrict__ part_idx) {
  __shared__ Best scratch[16];
  const int row = blockIdx.y;
  const int part = blockIdx.x;
  const int chunk = (vocab + parts - 1) / parts;
  const int begin = part * chunk;
  const int end = begin + chunk < vocab ? begin + chunk : vocab;
  const float* x = logits + (size_t)row * row_stride;
  Best mine;
  mine.v = 0.f;
  mine.i = -1;
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const float v = x[i];
    if (v != v) continue;  // NaN
    if (mine.i < 0 || v > mine.v) {
      mine.v = v;
      mine.i = i;
    }
  }
  const Best r = block_best(mine, scratch);
  if (threadIdx.x == 0) {
    part_val[(size_t)row * parts + part] = r.v;
    part_idx[(size_t)row * parts + part] = r.i;
  }
}

__global__ void argmax_final_kernel(const float* __restrict__ part_val, const int* __restrict__ part_idx, int parts,
                                    int* __restrict__ out) {
  __shared__ Best scratch[16];
  const int row = blockIdx.x;
  Best mine;
  mine.v = 0.f;
  mine.i = -1;
  for (int i = threadIdx.x; i < parts; i += blockDim.x) {
    Best o;
    o.v = part_val[(size_t)row * parts + i];
    o.i = part_idx[(size_t)row * parts + i];
    mine = better(mine, o);
  }
  const Best r = block_best(mine, scratch);
  if (threadIdx.x == 0) out[row] = r.i < 0 ? 0 : r.i;  // a row of NaN gives id 0
}

// Number of partial results per row that rv_argmax wants in its workspace.
extern "C" int rv_argmax_parts(int vocab) {
  int parts = rv_div_up(vocab, 4096);
  return parts < 1 ? 1 : (parts > 256 ? 256 : parts);
}

extern "C" int rv_argmax(hipStream_t stream, const float* logits, int rows, int vocab, long long row_stride,
                         float* ws_val, int* ws_idx, int* out) {
  RV_CHECK(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax: bad sizes rows=%d vocab=%d", rows, vocab);
  RV_CHECK(ws_val && ws_idx && out, "argmax: null workspace or output");
  if (rows == 0) return 0;
  RV_CHECK(rows < 65536, "argmax: too many rows %d", rows);
  const int parts = rv_argmax_parts(vocab);
  argmax_partial_kernel<<<dim3(parts, rows), dim3(256), 0, stream>>>(logits, vocab, row_stride, parts, ws_val, ws_idx);
  RV_LAUNCH_CHECK("argmax_partial");
  argmax_final_kernel<<<dim3(rows), dim3(256), 0, stream>>>(ws_val, ws_idx, parts, out);
  RV_LAUNCH_CHECK("argmax_final");
  return 0;
}

// ---------------------------------------------------------------------------
// top-K select, one block per row.
// ---------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long topk_key(float v, int i) {
  unsigned int b = __float_as_uint(v);
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // order of the floats as unsigned integers
  return ((unsigned long long)b << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned int)i);
}

__global__ void __launch_bounds__(1024)
topk_select_kernel(const float* __restrict__ logits, int vocab, long long row_stride, int k,
                   const float* __restrict__ inv_temp, float* __restrict__ out_val, int* __restrict__ out_idx) {
  __shared__ unsigned int hist[256];
  __shared__ unsigned long long prefix_s;
  __shared__ int remaining_s;
  __shared__ int out_count;
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * row_stride;

  if (threadIdx.x == 0) {
    prefix_s = 0ull;
    remaining_s = k;
    out_count = 0;
  }
  __syncthreads();

  // After the pass for byte b the top (64 - 8b) bits of the K-th largest key are known.
  for (int byte = 7; byte >= 0; --byte) {
    for (int i = threadIdx.x; i < 256; i += blockDim.x) hist[i] = 0u;
    __syncthreads();
    const unsigned long long prefix = prefix_s;
    const int shift = byte * 8;
    const unsigned long long high_mask = byte == 7 ? 0ull : (~0ull << (shift + 8));
    for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
      const unsigned long long key = topk_key(x[i], i);
      if ((key & high_mask) == prefix) atomicAdd(&hist[(unsigned int)(key >> shift) & 0xFFu], 1u);
    }
    __syncthreads();
    if (threadIdx.x == 0) {
      int remaining = remaining_s;
      int bin = 255;
      for (; bin > 0; --bin) {
        const int c = (int)hist[bin];
        if (c >= remaining) break;
        remaining -= c;
      }
      prefix_s = prefix | ((unsigned long long)bin << shift);
      remaining_s = remaining;
    }
    __syncthreads();
  }
  const unsigned long long threshold = prefix_s;  // the K-th largest key; keys are distinct
  const float scale = inv_temp[row];
  for (int i = threadIdx.x; i < vocab; i += blockDim.x) {
    const float v = x[i];
    if (topk_key(v, i) >= threshold) {
      const int slot = atomicAdd(&out_count, 1);
      if (slot < k) {
        out_val[(size_t)row * k + slot] = v * scale;
        out_idx[(size_t)row * k + slot] = i;
      }
    }
  }
}

extern "C" int rv_topk_select(hipStream_t stream, const float* logits, int rows, int vocab, long long row_stride,
                              int k, const float* inv_temp, float* out_val, int* out_idx) {
  RV_CHECK(rows >= 0 && vocab > 0 && row_stride >= vocab, "topk_select: bad sizes rows=%d vocab=%d", rows, vocab);
  RV_CHECK(k >= 1 && k <= 1024 && k <= vocab, "topk_select: k=%d must be in 1..min(1024, vocab=%d)", k, vocab);
  RV_CHECK(inv_temp && out_val && out_idx, "topk_select: null argument");
  if (rows == 0) return 0;
  topk_select_kernel<<<dim3(rows), dim3(1024), 0, stream>>>(logits, vocab, row_stride, k, inv_temp, out_val, out_idx);
  RV_LAUNCH_CHECK("topk_select");
  return 0;
}
