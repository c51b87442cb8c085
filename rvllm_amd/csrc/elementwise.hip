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
// RMSNorm: y = x * rsqrt(mean(x^2) + eps) * (offset + w)
// One block per row.
// ---------------------------------------------------------------------------
template <typename T>
__global__ void rmsnorm_kernel(const T* __restrict__ x, const int* __restrict__ row_index, const void* __restrict__ w,
                               int w_f32, T* __restrict__ y, int width, float eps, float offset) {
  __shared__ float scratch[16];
  const int in_row = row_index ? row_index[blockIdx.x] : (int)blockIdx.x;
  const T* xr = x + (size_t)in_row * width;
  T* yr = y + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = rv_to_float(xr[i]);
    ss += v * v;
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = rv_to_float(xr[i]);
    yr[i] = rv_from_float<T>(v * inv * (offset + rv_load_w(w, w_f32, i)));
  }
}

static int norm_block(int width) {
  int b = 64;
  while (b < width / 4 && b < 1024) b *= 2;  // about four elements a thread
  return b;
}

// Output row r is the norm of input row row_index[r] (of row r when row_index
// is null); the caller guarantees the indices are inside x.
extern "C" int rv_rmsnorm(hipStream_t stream, const void* x, const int* row_index, const void* w, int w_f32, void* y,
                          int dtype, int rows, int width, float eps, float offset) {
  RV_CHECK(rows >= 0 && width > 0, "rmsnorm: bad sizes rows=%d width=%d", rows, width);
  if (rows == 0) return 0;
  dim3 grid(rows), block(norm_block(width));
  if (dtype == RV_F32)
    rmsnorm_kernel<float><<<grid, block, 0, stream>>>((const float*)x, row_index, w, w_f32, (float*)y, width, eps,
                                                      offset);
  else if (dtype == RV_BF16)
    rmsnorm_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)x, row_index, w, w_f32, (bf16_t*)y, width, eps,
                                                       offset);
  else
    return rv_fail("rmsnorm: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// residual += RMSNorm(branch; w_post); optionally next = RMSNorm(residual; w_next)
// The normed branch is added in 32-bit and the sum rounded once; the second
// norm sees the residual as it is stored (rounded to T).
// ---------------------------------------------------------------------------
template <typename T>
__global__ void add_rmsnorm_kernel(const T* __restrict__ branch, const void* __restrict__ w_post, int w_post_f32,
                                   T* __restrict__ residual, const void* __restrict__ w_next, int w_next_f32,
                                   T* __restrict__ next, int width, float eps, float offset, float eps_next,
                                   float offset_next) {
  __shared__ float scratch[16];
  const T* br = branch + (size_t)blockIdx.x * width;
  T* rr = residual + (size_t)blockIdx.x * width;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float v = rv_to_float(br[i]);
    ss += v * v;
  }
  ss = rv_block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)width + eps);
  float ss2 = 0.f;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    const float n = rv_to_float(br[i]) * inv * (offset + rv_load_w(w_post, w_post_f32, i));
    const T stored = rv_from_float<T>(rv_to_float(rr[i]) + n);
    rr[i] = stored;
    const float r = rv_to_float(stored);
    ss2 += r * r;
  }
  if (next == nullptr) return;
  ss2 = rv_block_sum(ss2, scratch);
  const float inv2 = 1.0f / sqrtf(ss2 / (float)width + eps_next);
  T* nr = next + (size_t)blockIdx.x * width;
  for (int i = threadIdx.x; i < width; i += blockDim.x) {
    // each thread re-reads only what it wrote itself
    const float r = rv_to_float(rr[i]);
    nr[i] = rv_from_float<T>(r * inv2 * (offset_next + rv_load_w(w_next, w_next_f32, i)));
  }
}

extern "C" int rv_add_rmsnorm(hipStream_t stream, const void* branch, const void* w_post, int w_post_f32,
                              void* residual, const void* w_next, int w_next_f32, void* next, int dtype, int rows,
                              int width, float eps, float offset, float eps_next, float offset_next) {
  RV_CHECK(rows >= 0 && width > 0, "add_rmsnorm: bad sizes rows=%d width=%d", rows, width);
  RV_CHECK((w_next == nullptr) == (next == nullptr), "add_rmsnorm: next norm needs both weight and output");
  if (rows == 0) return 0;
  dim3 grid(rows), block(norm_block(width));
  if (dtype == RV_F32)
    add_rmsnorm_kernel<float><<<grid, block, 0, stream>>>((const float*)branch, w_post, w_post_f32, (float*)residual,
                                                          w_next, w_next_f32, (float*)next, width, eps, offset,
                                                          eps_next, offset_next);
  else if (dtype == RV_BF16)
    add_rmsnorm_kernel<bf16_t><<<grid, block, 0, stream>>>((const bf16_t*)branch, w_post, w_post_f32,
                                                           (bf16_t*)residual, w_next, w_next_f32, (bf16_t*)next, width,
                                                           eps, offset, eps_next, offset_next);
  else
    return rv_fail("add_rmsnorm: unsupported dtype %d", dtype);
  RV_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// ---------------------------------------------------------------------------
// gated activation: out[t,i] = act(gu[t,i]) * gu[t,I+i]
// act 0: gelu, tanh form; act 1: silu
// ---------------------------------------------------------------------------
__device__ __forceinline__ float rv_gelu_tanh(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float rv_silu(float z) { return z / (1.0f + expf(-z)); }

template <typename T, int ACT>
__global__ void gated_act_kernel(const T* __restrict__ gu, T* __restrict__ out, int inter, long long total) {
  const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const long long t = idx / inter;
  const int i = (int)(idx - t * inter);
  const T* row = gu + t * 2 * (long long)inter;
  const float g = rv_to_float(row[i]);
  const float u = rv_to_float(row[inter + i]);
  const float a = ACT == 0 ? rv_gelu_tanh(g) : rv_silu(g);
  out[idx] = rv_from_float<T>(a * u);
}

extern "C" int rv_gated_act(hipStream_t stream, const void* gu, void* out, int dtype, int rows, int inter, int act) {
  RV_CHECK(rows >= 0 && inter > 0, "gated_act: bad sizes rows=%d inter=%d", rows, inter);
  RV_CHECK(act == 0 || act == 1, "gated_act: unknown activation %d", act);
  if (rows == 0) return 0;
  const long long total = (long long)rows * inter;
  dim3 grid(rv_div_up(total, 256)), block(256);
#define RV_GA(T, A) gated_act_kernel<T, A><<<grid, block, 0, stream>>>((const T*)gu, (T*)out, inter, total)
  if (dtype == RV_F32 && act == 0) RV_GA(float, 0);
  else if (dtype == RV_F32 && act == 1) RV_GA(float, 1);
  else if (dtype == RV_BF16 && act == 0) RV_GA(bf16_t, 0);
  else if (dtype == RV_BF16 && act == 1) RV_GA(bf16_t, 1);
  else return rv_fail("gated_act: unsupported dtype %d", dtype);
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
