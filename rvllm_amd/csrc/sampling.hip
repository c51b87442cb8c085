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

#include <mutex>

#include "common.h"
#include "no_alloc.h"

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
// The same arg-max for callers that cannot allocate: the first stage's partial
// results go to an array that the library holds in device memory.  Each GPU
// has its own copy of the array at its own address; the name `scratch` is only
// a stand-in on the host, so the address is asked for once per device and kept.
// ---------------------------------------------------------------------------
#define RV_NO_ALLOC_SLOTS (RV_NO_ALLOC_MAX_ROWS * RV_NO_ALLOC_MAX_PARTS)
static __device__ __align__(256) unsigned char scratch[RV_NO_ALLOC_SLOTS * (sizeof(float) + sizeof(int))];

#define RV_MAX_DEVICES 64
static void* g_scratch_ptr[RV_MAX_DEVICES];  // the array's address on each device, once asked for
static std::mutex g_scratch_lock;

// The address of `scratch` on the current device; null (with the error set) when it cannot be had.
static void* scratch_on_current_device() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= RV_MAX_DEVICES) {
    rv_fail("argmax_no_alloc: no current device (%s, device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(g_scratch_lock);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr) {
      rv_fail("argmax_no_alloc: the address of the scratch array on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = ptr;
  }
  return g_scratch_ptr[dev];
}

extern "C" int rv_no_alloc_init(void) { return scratch_on_current_device() ? 0 : -1; }

extern "C" int rv_argmax_no_alloc(hipStream_t stream, const float* logits, int rows, int vocab, long long row_stride,
                                  int* out) {
  RV_CHECK(rows >= 0 && vocab > 0 && row_stride >= vocab, "argmax_no_alloc: bad sizes rows=%d vocab=%d", rows, vocab);
  RV_CHECK(logits && out, "argmax_no_alloc: null logits or output");
  RV_CHECK(rows <= RV_NO_ALLOC_MAX_ROWS, "argmax_no_alloc: %d rows, the scratch array holds %d", rows,
           RV_NO_ALLOC_MAX_ROWS);
  if (rows == 0) return 0;
  const int parts = rv_argmax_parts(vocab);
  RV_CHECK(parts <= RV_NO_ALLOC_MAX_PARTS, "argmax_no_alloc: %d parts a row, the scratch array holds %d", parts,
           RV_NO_ALLOC_MAX_PARTS);
  void* ptr = scratch_on_current_device();
  if (!ptr) return -1;
  // Values first, then ids.  Every slot the second stage reads is written by the first, so what an earlier
  // call left in the array is never seen.
  float* ws_val = (float*)ptr;
  int* ws_idx = (int*)((unsigned char*)ptr + RV_NO_ALLOC_SLOTS * sizeof(float));
  argmax_partial_kernel<<<dim3(parts, rows), dim3(256), 0, stream>>>(logits, vocab, row_stride, parts, ws_val, ws_idx);
  RV_LAUNCH_CHECK("argmax_partial (no alloc)");
  argmax_final_kernel<<<dim3(rows), dim3(256), 0, stream>>>(ws_val, ws_idx, parts, out);
  RV_LAUNCH_CHECK("argmax_final (no alloc)");
  return 0;
}

// ---------------------------------------------------------------------------
// top-K select.  A row of 262 208 logits is cut into parts, one block each: a
// block selects the K largest of its part (radix select over the keys
// (value, id), most significant byte first; its part stays in the caches over
// the passes), and one more block per row selects the K largest of the parts'
// candidates.  The reference selects with a single block per row
// (v3/kernels/sample_topk_f32.cu:68-117); here the first pass over a row is
// spread over many CUs, and a step's rows over the whole machine.
// ---------------------------------------------------------------------------
__device__ __forceinline__ unsigned long long topk_key(float v, int i) {
  unsigned int b = __float_as_uint(v);
  b = (b & 0x80000000u) ? ~b : (b | 0x80000000u);  // order of the floats as unsigned integers
  return ((unsigned long long)b << 32) | (unsigned long long)(0xFFFFFFFFu - (unsigned int)i);
}

#define TOPK_PART 8192   // elements of a part, about
#define TOPK_MAX_PARTS 64
#define TOPK_MAX_K 1024

// grid (parts, rows).  Block (part, row) takes the elements [part * chunk, ..) of the row's `total`; element i has
// value vals[i] and id ids[i], or i itself where ids is null.  It writes its K largest (unordered; values times
// 1/T where inv_temp is given) at slot (row * parts + part) * k.  The host sees to it that every part has at
// least k elements.
__global__ void __launch_bounds__(1024)
topk_select_kernel(const float* __restrict__ vals, const int* __restrict__ ids, long long row_stride, int total,
                   int chunk, int k, const float* __restrict__ inv_temp, float* __restrict__ out_val,
                   int* __restrict__ out_idx) {
  __shared__ unsigned int hist[256];
  __shared__ unsigned long long prefix_s;
  __shared__ int remaining_s;
  __shared__ int out_count;
  const int row = blockIdx.y;
  const int begin = blockIdx.x * chunk;
  const int count = total - begin < chunk ? total - begin : chunk;
  const float* x = vals + (size_t)row * row_stride + begin;
  const int* id_of = ids ? ids + (size_t)row * row_stride + begin : nullptr;
  auto key_of = [&](int i) { return topk_key(x[i], id_of ? id_of[i] : begin + i); };

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
    for (int i = threadIdx.x; i < count; i += blockDim.x) {
      const unsigned long long key = key_of(i);
      if ((key & high_mask) == prefix) atomicAdd(&hist[(unsigned int)(key >> shift) & 0xFFu], 1u);
    }
    __syncthreads();
    // The bin in which the count from the top reaches `remaining`: the first wave looks, four bins a lane.
    if (threadIdx.x < RV_WAVE) {
      const int lane = threadIdx.x;
      const int remaining = remaining_s;
      int c[4], mine = 0;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        c[j] = (int)hist[lane * 4 + j];
        mine += c[j];
      }
      int from_here_up = mine;  // keys in this lane's bins and all higher ones
#pragma unroll
      for (int off = 1; off < RV_WAVE; off <<= 1) {
        const int t = __shfl_down(from_here_up, off, RV_WAVE);
        if (lane + off < RV_WAVE) from_here_up += t;
      }
      const int above = from_here_up - mine;
      if (above < remaining && remaining <= from_here_up) {  // one lane: the keys that match number at least `remaining`
        int left = remaining - above, bin = lane * 4 + 3;
        for (int j = 3; j > 0; --j) {
          if (c[j] >= left) break;
          left -= c[j];
          --bin;
        }
        prefix_s = prefix | ((unsigned long long)bin << shift);
        remaining_s = left;
      }
    }
    __syncthreads();
  }
  const unsigned long long threshold = prefix_s;  // the K-th largest key; keys are distinct
  const float scale = inv_temp ? inv_temp[row] : 1.0f;
  const size_t out0 = ((size_t)row * gridDim.x + blockIdx.x) * k;
  for (int i = threadIdx.x; i < count; i += blockDim.x) {
    if (key_of(i) >= threshold) {
      const int slot = atomicAdd(&out_count, 1);
      if (slot < k) {
        out_val[out0 + slot] = x[i] * scale;
        out_idx[out0 + slot] = id_of ? id_of[i] : begin + i;
      }
    }
  }
}

// Parts a row is cut into; with more than one, rv_topk_select wants room for rows * parts * k candidates
// (values and ids).
extern "C" int rv_topk_parts(int vocab) {
  const int parts = vocab / TOPK_PART;
  return parts < 1 ? 1 : (parts > TOPK_MAX_PARTS ? TOPK_MAX_PARTS : parts);
}

extern "C" int rv_topk_select(hipStream_t stream, const float* logits, int rows, int vocab, long long row_stride,
                              int k, const float* inv_temp, float* out_val, int* out_idx, float* cand_val,
                              int* cand_idx) {
  RV_CHECK(rows >= 0 && vocab > 0 && row_stride >= vocab, "topk_select: bad sizes rows=%d vocab=%d", rows, vocab);
  RV_CHECK(k >= 1 && k <= TOPK_MAX_K && k <= vocab, "topk_select: k=%d must be in 1..min(%d, vocab=%d)", k, TOPK_MAX_K,
           vocab);
  RV_CHECK(inv_temp && out_val && out_idx, "topk_select: null argument");
  if (rows == 0) return 0;
  RV_CHECK(rows < 65536, "topk_select: too many rows %d", rows);
  const int parts = rv_topk_parts(vocab);
  if (parts == 1) {
    topk_select_kernel<<<dim3(1, rows), dim3(1024), 0, stream>>>(logits, nullptr, row_stride, vocab, vocab, k, inv_temp,
                                                               out_val, out_idx);
    RV_LAUNCH_CHECK("topk_select");
    return 0;
  }
  RV_CHECK(cand_val && cand_idx, "topk_select: a row in %d parts needs room for the parts' candidates", parts);
  // parts of at least TOPK_PART - TOPK_MAX_PARTS elements each: more than k
  const int chunk = rv_div_up(vocab, parts);
  topk_select_kernel<<<dim3(parts, rows), dim3(1024), 0, stream>>>(logits, nullptr, row_stride, vocab, chunk, k, nullptr,
                                                                 cand_val, cand_idx);
  RV_LAUNCH_CHECK("topk_select (parts)");
  topk_select_kernel<<<dim3(1, rows), dim3(1024), 0, stream>>>(cand_val, cand_idx, (long long)parts * k, parts * k,
                                                             parts * k, k, inv_temp, out_val, out_idx);
  RV_LAUNCH_CHECK("topk_select (candidates)");
  return 0;
}

// ---------------------------------------------------------------------------
// The draw on the device, from the candidates that topk_select left: what the host does with them
// (v3/crates/rvllm-sampling/src/sampler.rs:71-135), step for step and in its order of additions, so that a
// request gets the same tokens either way: sort by (value descending, id ascending), keep top_k, weigh by
// exp(v - max) in 64-bit, add up from the left, cut the nucleus at the first prefix that reaches top_p of the
// total, draw one number from the request's SplitMix64 stream and walk along the weights.  One block a row: all
// threads sort and weigh, one thread adds and walks (the sums are one after the other by definition).  A row
// one of whose own top_k candidates is no finite number gets -1 and keeps its stream, as the host refuses it.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float topk_value_of(unsigned long long key) {
  unsigned int b = (unsigned int)(key >> 32);
  b = (b & 0x80000000u) ? (b & 0x7FFFFFFFu) : ~b;  // topk_key's order of the floats, undone
  return __uint_as_float(b);
}

__global__ void __launch_bounds__(256)
draw_kernel(const float* __restrict__ vals, const int* __restrict__ ids, int k, const int* __restrict__ top_k,
            const double* __restrict__ top_p, unsigned long long* __restrict__ rng_state, int* __restrict__ chosen) {
  __shared__ unsigned long long keys[TOPK_MAX_K];
  __shared__ double weight[TOPK_MAX_K];
  __shared__ int bad;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  int padded = 1;
  while (padded < k) padded <<= 1;
  if (tid == 0) bad = 0;
  __syncthreads();
  for (int j = tid; j < padded; j += blockDim.x) {
    unsigned long long key = 0ull;  // below every candidate's
    if (j < k) {
      const float v = vals[(size_t)row * k + j] + 0.0f;  // -0 as +0: the two compare equal on the host
      key = topk_key(v, ids[(size_t)row * k + j]);
    }
    keys[j] = key;
  }
  __syncthreads();
  // bitonic sort, largest key first
  for (int size = 2; size <= padded; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int t = tid; t < (padded >> 1); t += blockDim.x) {
        const int i = 2 * t - (t & (stride - 1));
        const int j = i + stride;
        const unsigned long long a = keys[i], b = keys[j];
        const bool falling = (i & size) == 0;
        if ((a < b) == falling) {
          keys[i] = b;
          keys[j] = a;
        }
      }
      __syncthreads();
    }
  }
  // What the row keeps: its own top_k of the sorted candidates (0: all of them); -1 marks a row that decodes
  // greedily among rows that draw, which keeps one and takes it as the arg-max does.
  const int own = top_k[row];
  const bool arg_max = own < 0;
  const int n = arg_max ? 1 : (own > 0 ? (own < k ? own : k) : k);
  const double top = (double)topk_value_of(keys[0]);
  for (int j = tid; j < n; j += blockDim.x) {
    const float v = topk_value_of(keys[j]);
    // the host refuses a row one of whose own candidates is no finite number; what lies beyond the row's top_k
    // was selected for another row's sake and is not looked at
    if (!arg_max && !(fabsf(v) <= 3.402823466e38f)) bad = 1;
    weight[j] = exp((double)v - top);
  }
  __syncthreads();
  if (tid != 0) return;
  if (arg_max) {
    // the largest logit that is a number (the arg-max skips NaN; equal values go by the lower id, which is the
    // order of the sort); -1 if all k candidates are NaN
    int pick = -1;
    for (int i = 0; i < k && pick < 0; ++i) {
      const float v = topk_value_of(keys[i]);
      if (v == v) pick = i;
    }
    chosen[row] = pick < 0 ? -1 : (int)(0xFFFFFFFFu - (unsigned int)(keys[pick] & 0xFFFFFFFFull));
    return;
  }
  if (bad) {
    chosen[row] = -1;
    return;
  }
  double total = 0.0;
  for (int i = 0; i < n; ++i) total += weight[i];
  int cut = n;
  const double p = top_p[row];
  if (p < 1.0) {
    const double target = (p > 0.0 ? p : 0.0) * total;
    double cum = 0.0;
    for (int i = 0; i < n; ++i) {
      cum += weight[i];
      if (cum >= target) {
        cut = i + 1;
        break;
      }
    }
  }
  double z = 0.0;
  for (int i = 0; i < cut; ++i) z += weight[i];
  unsigned long long state = rng_state[row] + 0x9E3779B97F4A7C15ull;  // SplitMix64, sampler.rs:17-36
  rng_state[row] = state;
  unsigned long long r = state;
  r = (r ^ (r >> 30)) * 0xBF58476D1CE4E5B9ull;
  r = (r ^ (r >> 27)) * 0x94D049BB133111EBull;
  r ^= r >> 31;
  double u = ((double)(r >> 11) * (1.0 / 9007199254740992.0)) * z;
  int pick = cut - 1;
  for (int i = 0; i < cut; ++i) {
    u -= weight[i];
    if (u <= 0.0) {
      pick = i;
      break;
    }
  }
  chosen[row] = (int)(0xFFFFFFFFu - (unsigned int)(keys[pick] & 0xFFFFFFFFull));
}

// vals, ids [rows, k]: the candidates of topk_select (values times 1/T, any order); top_k [rows] (0: all k; -1: no
// draw, the arg-max of the candidates, for a greedy request among requests that sample),
// top_p [rows] (64-bit), rng_state [rows] (each request's stream, moved one draw on), chosen [rows].
extern "C" int rv_draw(hipStream_t stream, const float* vals, const int* ids, int rows, int k, const int* top_k,
                       const double* top_p, unsigned long long* rng_state, int* chosen) {
  RV_CHECK(rows >= 0 && k >= 1 && k <= TOPK_MAX_K, "draw: k=%d must be in 1..%d (rows=%d)", k, TOPK_MAX_K, rows);
  RV_CHECK(vals && ids && top_k && top_p && rng_state && chosen, "draw: null argument");
  if (rows == 0) return 0;
  draw_kernel<<<dim3(rows), dim3(256), 0, stream>>>(vals, ids, k, top_k, top_p, rng_state, chosen);
  RV_LAUNCH_CHECK("draw");
  return 0;
}

// ---------------------------------------------------------------------------
// From one decode step to the next without the host: every request's chosen
// token becomes its next token, one position on.  A step of decoded tokens is
// described by these arrays alone (token t belongs to request t), so the same
// launches, or the same captured graph, run the next step from them.
// ---------------------------------------------------------------------------
__global__ void advance_decode_kernel(const int* __restrict__ chosen, int* __restrict__ token_ids,
                                      int* __restrict__ positions, int* __restrict__ chunk_start,
                                      int* __restrict__ context_len, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= n) return;
  token_ids[i] = chosen[i];
  positions[i] += 1;
  chunk_start[i] += 1;
  context_len[i] += 1;
}

extern "C" int rv_advance_decode(hipStream_t stream, const int* chosen, int* token_ids, int* positions,
                                 int* chunk_start, int* context_len, int n) {
  RV_CHECK(n >= 0 && chosen && token_ids && positions && chunk_start && context_len, "advance_decode: bad arguments");
  if (n == 0) return 0;
  advance_decode_kernel<<<dim3(rv_div_up(n, 256)), dim3(256), 0, stream>>>(chosen, token_ids, positions, chunk_start,
                                                                         context_len, n);
  RV_LAUNCH_CHECK("advance_decode");
  return 0;
}
