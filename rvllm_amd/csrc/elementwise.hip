// Row-wise kernels: embedding lookup with scale, RMSNorm, RMSNorm of a branch
// added into the residual stream (optionally followed by the next RMSNorm),
// gated activation, logit soft-cap.  All arithmetic is in 32-bit floats; the
// storage type T is float or bf16.
//
// What they compute follows the reference's kernels:
//   embedding     kernels/embedding_gather_f16.cu:12-39 (scale: gemma4_load.rs:219-253)
//   RMSNorm       v3/kernels/rmsnorm_inplace_f16.cu:29-62 (eps inside the root)
//   norm + add    v3/kernels/fused_norm_add_residual.cu:8-57
//   gelu * up     v3/kernels/fused_gelu_mul_f16.cu:7-29
//   soft-cap      v3/kernels/logit_softcap.cu:12-31
// with one difference that the Gemma-3 decoder needs: the norm's gain is
// (offset + weight), offset being 1 for the zero-centred weights.
#include <stdarg.h>
#include <stdio.h>

#include "common.h"

// ---------------------------------------------------------------------------
// error channel (defined once, here)
// ---------------------------------------------------------------------------
static thread_local char g_err[512] = "";
extern "C" const char* rv_last_error() { return g_err; }
int rv_fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return -1;
}

// ---------------------------------------------------------------------------
// embedding: out[t,:] = table[ids[t],:] * scale
// ---------------------------------------------------------------------------
template <typename TT, typename TO>
__global__ void embed_gather_kernel(const TT* __restrict__ table, const int* __restrict__ ids, TO* __restrict__ out,
                                    int hidden, int vocab, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  TO* o = out + (size_t)t * hidden;
  if (id < 0 || id >= vocab) {  // the host rejects such ids; never read outside the table
    for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = rv_from_float<TO>(0.f);
    return;
  }
  const TT* row = table + (size_t)id * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) o[i] = rv_from_float<TO>(rv_to_float(row[i]) * scale);
}

extern "C" int rv_embed_gather(hipStream_t stream, const void* table, int table_dtype, const int* ids, void* out,
                               int out_dtype, int num_tokens, int hidden, int vocab, float scale) {
  RV_CHECK(num_tokens >= 0 && hidden > 0 && vocab > 0, "embed_gather: bad sizes T=%d H=%d V=%d", num_tokens, hidden, vocab);
  if (num_tokens == 0) return 0;
  dim3 grid(num_tokens), block(256);
  if (table_dtype == RV_F32 && out_dtype == RV_F32)
    embed_gather_kernel<float, float><<<grid, block, 0, stream>>>((const float*)table, ids, (float*)out, hidden, vocab, scale);
  else if (table_dtype == RV_BF16 && out_dtype == RV_BF16)
    embed_gather_kernel<bf16_t, bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)table, ids, (bf16_t*)out, hidden, vocab, scale);
  else if (table_dtype == RV_BF16 && out_dtype == RV_F32)
    embed_gather_kernel<bf16_t, float><<<grid, block, 0, stream>>>((const bf16_t*)table, ids, (float*)out, hidden, vocab, scale);
  else if (table_dtype == RV_F32 && out_dtype == RV_BF16)
    embed_gather_kernel<float, bf16_t><<<grid, block, 0, stream>>>((const float*)table, ids, (bf16_t*)out, hidden, vocab, scale);
  else
    return rv_fail("embed_gather: unsupported dtypes %d -> %d", table_dtype, out_dtype);
  RV_LAUNCH_CHECK("embed_gather");
  return 0;
}

// ---------------------------------------------------------------------------
// Row kernels keep a row in registers: one block per row, a thread owns E
// groups of V consecutive elements (V = 16 bytes' worth when the width allows,
// else 1), so a row is read once and written once whatever the number of
// passes over it.
// ---------------------------------------------------------------------------
#define ROW_MAX_E 16

template <typename T>
struct RowVec {
  static constexpr int V = 16 / sizeof(T);
};

template <typename T, int V>
__device__ __forceinline__ void row_load(const T* p, float* out) {
  if constexpr (V == 1) {
    out[0] = rv_to_float(p[0]);
  } else if constexpr (sizeof(T) == 4) {
    const float4 v = *(const float4*)p;
    out[0] = v.x, out[1] = v.y, out[2] = v.z, out[3] = v.w;
  } else {
    const uint4 v = *(const uint4*)p;
    const uint32_t u[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      out[2 * i] = __uint_as_float(u[i] << 16);
      out[2 * i + 1] = __uint_as_float(u[i] & 0xffff0000u);
    }
  }
}

template <typename T, int V>
__device__ __forceinline__ void row_store(T* p, const float* in) {
  if constexpr (V == 1) {
    p[0] = rv_from_float<T>(in[0]);
  } else if constexpr (sizeof(T) == 4) {
    *(float4*)p = make_float4(in[0], in[1], in[2], in[3]);
  } else {
    uint32_t u[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      u[i] = (uint32_t)rv_f32_to_bf16_bits(in[2 * i]) | ((uint32_t)rv_f32_to_bf16_bits(in[2 * i + 1]) << 16);
    *(uint4*)p = make_uint4(u[0], u[1], u[2], u[3]);
  }
}

// V weights starting at element i; the weight vector may be float or bf16.
template <int V>
__device__ __forceinline__ void row_load_w(const void* w, int w_f32, int i, float* out) {
  rv_load_w_vec<V>(w, w_f32, i, out);
}

// V values of a branch starting at element i of row `row`: either stored as T,
// or as the sum of `slices` 32-bit partial sums (the K slices of a product),
// added in the order of the slices.
template <int V>
__device__ __forceinline__ void row_load_f32(const float* p, float* out) {
  if constexpr (V >= 4) {
#pragma unroll
    for (int v = 0; v < V; v += 4) {
      const float4 q = *(const float4*)(p + v);
      out[v] = q.x, out[v + 1] = q.y, out[v + 2] = q.z, out[v + 3] = q.w;
    }
  } else {
    out[0] = p[0];
  }
}

template <typename T, int V>
__device__ __forceinline__ void row_load_branch(const void* branch, int slices, long long slice_stride, size_t at,
                                                float* out) {
  if (slices == 0) {
    row_load<T, V>((const T*)branch + at, out);
    return;
  }
#pragma unroll
  for (int v = 0; v < V; ++v) out[v] = 0.f;
  const float* p = (const float*)branch + at;
  int s = 0;
  // four slices are read at a time, so that their loads are in flight together;
  // they are added in the order of the slices all the same
  for (; s + 4 <= slices; s += 4) {
    float q[4][V];
#pragma unroll
    for (int j = 0; j < 4; ++j) row_load_f32<V>(p + (size_t)(s + j) * slice_stride, q[j]);
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < V; ++v) out[v] += q[j][v];
  }
  for (; s < slices; ++s) {
    float q[V];
    row_load_f32<V>(p + (size_t)s * slice_stride, q);
#pragma unroll
    for (int v = 0; v < V; ++v) out[v] += q[v];
  }
}

static void row_geometry(int width, int v, int* block, int* e) {
  const int groups = rv_div_up(width, v);
  int b = rv_div_up(groups, 64) * 64;
  if (b > 1024) b = 1024;
  *block = b;
  *e = rv_div_up(groups, b);
}

// ---------------------------------------------------------------------------
// RMSNorm: y = x * rsqrt(mean(x^2) + eps) * (offset + w)
// ---------------------------------------------------------------------------
template <typename T, int V, int E>
__global__ void rmsnorm_kernel(const T* __restrict__ x, const int* __restrict__ row_index, const void* __restrict__ w,
                               int w_f32, T* __restrict__ y, int width, float eps, float offset) {
  __shared__ float scratch[16];
  const int in_row = row_index ? row_index[blockIdx.x] : (int)blockIdx.x;
  const T* xr = x + (size_t)in_row * width;
  T* yr = y + (size_t)blockIdx.x * width;
  float val[E][V], g[E][V];  // the weights are asked for with the row, not after the sum's barrier
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * blockDim.x + threadIdx.x) * V;
    if (i < width) {
      row_load<T, V>(xr + i, val[e]);
      row_load_w<V>(w, w_f32, i, g[e]);
#pragma unroll
      for (int v = 0; v < V; ++v) ss += val[e][v] * val[e][v];
    }
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * blockDim.x + threadIdx.x) * V;
    if (i < width) {
#pragma unroll
      for (int v = 0; v < V; ++v) val[e][v] = val[e][v] * inv * (offset + g[e][v]);
      row_store<T, V>(yr + i, val[e]);
    }
  }
}

// Picks the instantiation for a width: vectors when the width is a multiple of
// 16 bytes' worth of elements, and as many groups a thread as the width needs.
#define ROW_DISPATCH(KERNEL, T, width, grid, stream, ...)                                               \
  do {                                                                                                  \
    constexpr int VV = RowVec<T>::V;                                                                    \
    int block_, e_;                                                                                     \
    if ((width) % VV == 0) {                                                                            \
      row_geometry(width, VV, &block_, &e_);                                                            \
      if (e_ <= 1) KERNEL<T, VV, 1><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__);                    \
      else if (e_ <= 2) KERNEL<T, VV, 2><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__);               \
      else if (e_ <= 4) KERNEL<T, VV, 4><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__);               \
      else return rv_fail("row kernel: width %d is too large", width);                                  \
    } else {                                                                                            \
      row_geometry(width, 1, &block_, &e_);                                                             \
      if (e_ <= 1) KERNEL<T, 1, 1><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__);                     \
      else if (e_ <= 4) KERNEL<T, 1, 4><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__);                \
      else if (e_ <= ROW_MAX_E) KERNEL<T, 1, ROW_MAX_E><<<grid, dim3(block_), 0, stream>>>(__VA_ARGS__); \
      else return rv_fail("row kernel: width %d is too large", width);                                  \
    }                                                                                                   \
  } while (0)

// Output row r is the norm of input row row_index[r] (of row r when row_index
// is null); the caller guarantees the indices are inside x.
extern "C" int rv_rmsnorm(hipStream_t stream, const void* x, const int* row_index, const void* w, int w_f32, void* y,
                          int dtype, int rows, int width, float eps, float offset) {
  RV_CHECK(rows >= 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", rows, width);
  if (rows == 0) return 0;
  dim3 grid(rows);
  if (dtype == RV_F32)
    ROW_DISPATCH(rmsnorm_kernel, float, width, grid, stream, (const float*)x, row_index, w, w_f32, (float*)y, width,
                 eps, offset);
  else if (dtype == RV_BF16)
    ROW_DISPATCH(rmsnorm_kernel, bf16_t, width, grid, stream, (const bf16_t*)x, row_index, w, w_f32, (bf16_t*)y,
                 width, eps, offset);
  else
    return rv_fail("rmsnorm: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// residual += RMSNorm(branch; w_post); optionally next = RMSNorm(residual; w_next)
// The normed branch is added in 32-bit and the sum rounded once; the second
// norm sees the residual as it is stored (rounded to T).  The branch is either
// stored as T or given as `slices` 32-bit partial sums of a product.
// ---------------------------------------------------------------------------
template <typename T, int V, int E>
__global__ void add_rmsnorm_kernel(const void* __restrict__ branch, int slices, long long slice_stride,
                                   const void* __restrict__ w_post, int w_post_f32, T* __restrict__ residual,
                                   const void* __restrict__ w_next, int w_next_f32, T* __restrict__ next, int width,
                                   float eps, float offset, float eps_next, float offset_next) {
  __shared__ float scratch[16];
  const size_t row0 = (size_t)blockIdx.x * width;
  T* rr = residual + row0;
  // Everything the row needs is asked for at once, before the first sum: a load behind a barrier would only
  // start after it, and at a few rows a step the kernel is as long as its chain of round trips to memory.
  float val[E][V], res[E][V], g_post[E][V], g_next[E][V];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * blockDim.x + threadIdx.x) * V;
    if (i < width) {
      row_load_branch<T, V>(branch, slices, slice_stride, row0 + i, val[e]);
      row_load<T, V>(rr + i, res[e]);
      row_load_w<V>(w_post, w_post_f32, i, g_post[e]);
      if (next != nullptr) row_load_w<V>(w_next, w_next_f32, i, g_next[e]);
#pragma unroll
      for (int v = 0; v < V; ++v) ss += val[e][v] * val[e][v];
    }
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * blockDim.x + threadIdx.x) * V;
    if (i < width) {
#pragma unroll
      for (int v = 0; v < V; ++v) {
        // the residual as it reads back after the store
        val[e][v] = rv_round_to<T>(res[e][v] + val[e][v] * inv * (offset + g_post[e][v]));
        ss2 += val[e][v] * val[e][v];
      }
      row_store<T, V>(rr + i, val[e]);
    }
  }
  if (next == nullptr) return;
  ss2 = rv_block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  T* nr = next + row0;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * blockDim.x + threadIdx.x) * V;
    if (i < width) {
#pragma unroll
      for (int v = 0; v < V; ++v) val[e][v] = val[e][v] * inv2 * (offset_next + g_next[e][v]);
      row_store<T, V>(nr + i, val[e]);
    }
  }
}

// The same for many rows in bf16 (a prompt portion): a wave takes a whole row, eight values a lane and turn, so
// both sums are exchanges inside the wave and no barrier stands between a row's reads and its writes.  The
// arithmetic is the block kernel's, value by value; only the order in which a row's squares are added differs.
template <int E>
__global__ void __launch_bounds__(256)
add_rmsnorm_rows_kernel(const uint16_t* __restrict__ branch, const void* __restrict__ w_post, int w_post_f32,
                        uint16_t* __restrict__ residual, const void* __restrict__ w_next, int w_next_f32,
                        uint16_t* __restrict__ next, int rows, int width, float eps, float offset, float eps_next,
                        float offset_next) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;  // the whole wave
  const size_t row0 = (size_t)row * width;
  float val[E][8], res[E][8], g_post[E][8], g_next[E][8];
  float ss = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * RV_WAVE + lane) * 8;
    if (i < width) {
      row_load<bf16_t, 8>((const bf16_t*)branch + row0 + i, val[e]);
      row_load<bf16_t, 8>((const bf16_t*)residual + row0 + i, res[e]);
      row_load_w<8>(w_post, w_post_f32, i, g_post[e]);
      if (next != nullptr) row_load_w<8>(w_next, w_next_f32, i, g_next[e]);
#pragma unroll
      for (int v = 0; v < 8; ++v) ss += val[e][v] * val[e][v];
    }
  }
  ss = rv_wave_sum(ss);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * RV_WAVE + lane) * 8;
    if (i < width) {
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        val[e][v] = rv_round_to<bf16_t>(res[e][v] + val[e][v] * inv * (offset + g_post[e][v]));
        ss2 += val[e][v] * val[e][v];
      }
      row_store<bf16_t, 8>((bf16_t*)residual + row0 + i, val[e]);
    }
  }
  if (next == nullptr) return;
  ss2 = rv_wave_sum(ss2);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
#pragma unroll
  for (int e = 0; e < E; ++e) {
    const int i = (e * RV_WAVE + lane) * 8;
    if (i < width) {
#pragma unroll
      for (int v = 0; v < 8; ++v) val[e][v] = val[e][v] * inv2 * (offset_next + g_next[e][v]);
      row_store<bf16_t, 8>((bf16_t*)next + row0 + i, val[e]);
    }
  }
}
#define ADD_RMSNORM_ROWS_MIN 256   // from this many rows on a wave takes a row
#define ADD_RMSNORM_ROWS_MAX_E 6   // turns of 512 values a wave takes at most (its registers)

// `slices` 0: branch holds T values [rows, width].  Otherwise branch holds
// 32-bit partial sums [slices][rows][width] (slice_stride elements apart).
extern "C" int rv_add_rmsnorm(hipStream_t stream, const void* branch, int slices, long long slice_stride,
                              const void* w_post, int w_post_f32, void* residual, const void* w_next, int w_next_f32,
                              void* next, int dtype, int rows, int width, float eps, float offset, float eps_next,
                              float offset_next) {
  RV_CHECK(rows >= 0 && width > 0, "add_rmsnorm: bad sizes rows=%d width=%d", rows, width);
  RV_CHECK((w_next == nullptr) == (next == nullptr), "add_rmsnorm: next norm needs both weight and output");
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= (long long)rows * width), "add_rmsnorm: bad partial sums");
  if (rows == 0) return 0;
  const int turns = rv_div_up(width, 8 * RV_WAVE);
  if (dtype == RV_BF16 && slices == 0 && rows >= ADD_RMSNORM_ROWS_MIN && width % 8 == 0 &&
      turns <= ADD_RMSNORM_ROWS_MAX_E) {
#define RV_ARR(E)                                                                                                  \
  add_rmsnorm_rows_kernel<E><<<dim3(rv_div_up(rows, 4)), dim3(256), 0, stream>>>(                                 \
      (const uint16_t*)branch, w_post, w_post_f32, (uint16_t*)residual, w_next, w_next_f32, (uint16_t*)next, rows, \
      width, eps, offset, eps_next, offset_next)
    switch (turns) {
      case 1: RV_ARR(1); break;
      case 2: RV_ARR(2); break;
      case 3: RV_ARR(3); break;
      case 4: RV_ARR(4); break;
      case 5: RV_ARR(5); break;
      default: RV_ARR(6); break;
    }
#undef RV_ARR
    RV_LAUNCH_CHECK("add_rmsnorm_rows");
    return 0;
  }
  dim3 grid(rows);
  if (dtype == RV_F32)
    ROW_DISPATCH(add_rmsnorm_kernel, float, width, grid, stream, branch, slices, slice_stride, w_post, w_post_f32,
                 (float*)residual, w_next, w_next_f32, (float*)next, width, eps, offset, eps_next, offset_next);
  else if (dtype == RV_BF16)
    ROW_DISPATCH(add_rmsnorm_kernel, bf16_t, width, grid, stream, branch, slices, slice_stride, w_post, w_post_f32,
                 (bf16_t*)residual, w_next, w_next_f32, (bf16_t*)next, width, eps, offset, eps_next, offset_next);
  else
    return rv_fail("add_rmsnorm: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// gated activation: out[t,i] = act(gate[t,i]) * up[t,i]
// act 0: gelu, tanh form; act 1: silu
// The two lie in one row of gu: halves (gates, then ups: gate i at i, up i at
// I + i) or, FOURS, as a product against weight rows in fours leaves them (two
// gates, then their two ups: gate i at 4 (i / 2) + i % 2, up i two further).
// ---------------------------------------------------------------------------

// A thread takes GA_ITEMS groups of V outputs, a block's width apart, and asks for all their inputs before it
// uses the first: at thousands of rows the kernel is a stream of 126 MB, and two 16-byte reads in flight per
// thread do not draw the memory's full rate.
#define GA_ITEMS 4
template <typename T, int V, int ACT, bool FOURS>
__global__ void gated_act_kernel(const void* __restrict__ gu, int slices, long long slice_stride, T* __restrict__ out,
                                 int inter, long long groups_total) {
  const long long g0 = (long long)blockIdx.x * (blockDim.x * GA_ITEMS) + threadIdx.x;
  const int groups_per_row = inter / V;
  float a[GA_ITEMS][V], b[GA_ITEMS][V];
  long long t[GA_ITEMS];
  int i[GA_ITEMS];
#pragma unroll
  for (int n = 0; n < GA_ITEMS; ++n) {
    long long gidx = g0 + (long long)n * blockDim.x;
    gidx = gidx < groups_total ? gidx : groups_total - 1;  // a thread past the end repeats the last group's reads
    t[n] = gidx / groups_per_row;
    i[n] = (int)(gidx - t[n] * groups_per_row) * V;
    if constexpr (FOURS) {  // V is a multiple of 4 here: the thread's outputs are its 2 V neighbouring values
      const size_t at = (size_t)t[n] * 2 * inter + 2 * (size_t)i[n];
      row_load_branch<T, V>(gu, slices, slice_stride, at, a[n]);
      row_load_branch<T, V>(gu, slices, slice_stride, at + V, b[n]);
    } else {
      const size_t at = (size_t)t[n] * 2 * inter + i[n];
      row_load_branch<T, V>(gu, slices, slice_stride, at, a[n]);
      row_load_branch<T, V>(gu, slices, slice_stride, at + inter, b[n]);
    }
  }
#pragma unroll
  for (int n = 0; n < GA_ITEMS; ++n) {
    if (g0 + (long long)n * blockDim.x >= groups_total) break;
    float g[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      if constexpr (FOURS) {
        const int at4 = 4 * (v / 2) + v % 2;  // among the 2 V values
        const float gate = at4 < V ? a[n][at4] : b[n][at4 - V];
        const float up = at4 + 2 < V ? a[n][at4 + 2] : b[n][at4 + 2 - V];
        g[v] = rv_gated<T, ACT>(gate, up);
      } else {
        g[v] = rv_gated<T, ACT>(a[n][v], b[n][v]);
      }
    }
    row_store<T, V>(out + (size_t)t[n] * inter + i[n], g);
  }
}

// `slices` 0: gu holds T values [rows, 2*inter]; otherwise 32-bit partial sums
// [slices][rows][2*inter], slice_stride elements apart.
extern "C" int rv_gated_act(hipStream_t stream, const void* gu, int slices, long long slice_stride, void* out,
                            int dtype, int rows, int inter, int act, int fours) {
  RV_CHECK(rows >= 0 && inter > 0, "gated_act: bad sizes rows=%d inter=%d", rows, inter);
  RV_CHECK(act == 0 || act == 1, "gated_act: unknown activation %d", act);
  RV_CHECK(!fours || inter % 4 == 0, "gated_act: rows in fours need a width that is a multiple of 4, got %d", inter);
  RV_CHECK(slices >= 0 && (slices == 0 || slice_stride >= 2ll * rows * inter), "gated_act: bad partial sums");
  if (rows == 0) return 0;
#define RV_GA(T, V, A, F)                                                                                          \
  do {                                                                                                             \
    const long long groups = (long long)rows * (inter / V);                                                        \
    gated_act_kernel<T, V, A, F><<<dim3(rv_div_up(groups, 256 * GA_ITEMS)), dim3(256), 0, stream>>>(gu, slices, slice_stride, \
                                                                                        (T*)out, inter, groups);   \
  } while (0)
#define RV_GA_A(T, V, F)                              \
  do {                                                \
    if (act == 0) RV_GA(T, V, 0, F); else RV_GA(T, V, 1, F); \
  } while (0)
#define RV_GA_T(T)                                                       \
  do {                                                                   \
    constexpr int VV = RowVec<T>::V; /* a multiple of 4 */               \
    if (fours) {                                                         \
      if (inter % VV != 0)                                               \
        return rv_fail("gated_act: rows in fours need a width that is a multiple of %d, got %d", VV, inter); \
      RV_GA_A(T, VV, true);                                              \
    } else {                                                             \
      if (inter % VV == 0) RV_GA_A(T, VV, false); else RV_GA_A(T, 1, false); \
    }                                                                    \
  } while (0)
  if (dtype == RV_F32) RV_GA_T(float);
  else if (dtype == RV_BF16) RV_GA_T(bf16_t);
  else return rv_fail("gated_act: unsupported dtype %d", dtype);
#undef RV_GA_T
#undef RV_GA_A
#undef RV_GA
  RV_LAUNCH_CHECK("gated_act");
  return 0;
}

// ---------------------------------------------------------------------------
// soft-cap on f32 logits, in place: cap * tanh(x / cap)
// ---------------------------------------------------------------------------
__global__ void softcap_kernel(float* __restrict__ x, long long total, float cap) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < total) x[idx] = cap * tanhf(x[idx] / cap);
}

extern "C" int rv_softcap(hipStream_t stream, float* logits, long long total, float cap) {
  RV_CHECK(total >= 0 && cap > 0.f, "softcap: bad arguments total=%lld cap=%f", total, (double)cap);
  if (total == 0) return 0;
  softcap_kernel<<<dim3(rv_div_up(total, 256)), dim3(256), 0, stream>>>(logits, total, cap);
  RV_LAUNCH_CHECK("softcap");
  return 0;
}

// ---------------------------------------------------------------------------
// bias of a projection, in place: x[r][c] += bias[c], the sum in 32-bit.  With `slices` > 0, x is the result of
// adding up that many 32-bit partial sums [slices][rows][width] (the K slices of a product) and the bias.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ x, const float* __restrict__ part, int slices, const void* __restrict__ bias,
                                int bias_f32, long long total, int width) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  float v;
  if (slices > 0) {
    v = 0.f;
    for (int s = 0; s < slices; ++s) v += part[(long long)s * total + idx];
  } else {
    v = rv_to_float(x[idx]);
  }
  x[idx] = rv_from_float<T>(v + rv_load_w(bias, bias_f32, (int)(idx % width)));
}

extern "C" int rv_add_bias(hipStream_t stream, void* x, int dtype, const float* part, int slices, const void* bias,
                           int bias_f32, int rows, int width) {
  RV_CHECK(rows >= 0 && width > 0 && x && bias && slices >= 0 && (slices == 0 || part), "add_bias: bad arguments");
  if (rows == 0) return 0;
  const long long total = (long long)rows * width;
  dim3 grid(rv_div_up(total, 256)), block(256);
  if (dtype == RV_F32)
    add_bias_kernel<float><<<grid, block, 0, stream>>>((float*)x, part, slices, bias, bias_f32, total, width);
  else if (dtype == RV_BF16)
    add_bias_kernel<bf16_t><<<grid, block, 0, stream>>>((bf16_t*)x, part, slices, bias, bias_f32, total, width);
  else
    return rv_fail("add_bias: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("add_bias");
  return 0;
}
