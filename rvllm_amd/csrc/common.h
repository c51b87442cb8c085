// Shared device helpers for the gfx950 kernels: storage types, wave64
// reductions, and the error channel of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#define RV_WAVE 64

// ---------------------------------------------------------------------------
// Error channel.  Every entry point returns 0 or a negative code and leaves a
// message that rv_last_error() returns; it validates shapes on the host before
// it launches anything.
// ---------------------------------------------------------------------------
extern "C" const char* rv_last_error();
int rv_fail(const char* fmt, ...);

#define RV_CHECK(cond, ...)                 \
  do {                                      \
    if (!(cond)) return rv_fail(__VA_ARGS__); \
  } while (0)

#define RV_LAUNCH_CHECK(name)                                              \
  do {                                                                     \
    hipError_t e_ = hipGetLastError();                                     \
    if (e_ != hipSuccess) return rv_fail("%s: launch failed: %s", name,    \
                                         hipGetErrorString(e_));           \
  } while (0)

// dtype codes shared with Python
enum RvDType { RV_F32 = 0, RV_BF16 = 1 };

// ---------------------------------------------------------------------------
// bfloat16 storage: 16 bits, round to nearest even on store.
// ---------------------------------------------------------------------------
struct bf16_t {
  uint16_t bits;
};

__device__ __forceinline__ float rv_to_float(float x) { return x; }
__device__ __forceinline__ float rv_to_float(bf16_t x) {
  return __uint_as_float(((uint32_t)x.bits) << 16);
}

// Round to nearest even, NaN stays NaN: gfx950 has an instruction for it
// (v_cvt_pk_bf16_f32), which the cast compiles to.
__device__ __forceinline__ uint16_t rv_f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(uint16_t, (__bf16)f);
}

// Two values in one register, `lo` in the low half: one instruction.
__device__ __forceinline__ uint32_t rv_pack_bf16x2(float lo, float hi) {
  typedef float rv_float2_t __attribute__((ext_vector_type(2)));
  typedef __bf16 rv_bf16x2_t __attribute__((ext_vector_type(2)));
  const rv_float2_t f = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, rv_bf16x2_t));
}

template <typename T>
__device__ __forceinline__ T rv_from_float(float x);
template <>
__device__ __forceinline__ float rv_from_float<float>(float x) {
  return x;
}
template <>
__device__ __forceinline__ bf16_t rv_from_float<bf16_t>(float x) {
  bf16_t r;
  r.bits = rv_f32_to_bf16_bits(x);
  return r;
}

// Value as it reads back after a store in T.
template <typename T>
__device__ __forceinline__ float rv_round_to(float x) {
  return rv_to_float(rv_from_float<T>(x));
}

// Gated activations, act(gate) * up; ACT 0: gelu in its tanh form
// (v3/kernels/fused_gelu_mul_f16.cu:20-27), ACT 1: silu.  The 32-bit path uses
// the accurate library functions.  Where the result is rounded to bf16 anyway,
// the hardware's exponential and reciprocal (an error of some 1e-6) cost a
// fifth of that; every bf16 kernel that applies an activation goes through
// here, so they all round alike.
template <typename T, int ACT>
__device__ __forceinline__ float rv_gated(float gate, float up);
template <>
__device__ __forceinline__ float rv_gated<float, 0>(float z, float up) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z))) * up;
}
template <>
__device__ __forceinline__ float rv_gated<float, 1>(float z, float up) {
  return z / (1.0f + expf(-z)) * up;
}
template <>
__device__ __forceinline__ float rv_gated<bf16_t, 0>(float z, float up) {
  // 0.5 (1 + tanh y) = 1 / (1 + e^-2y) with y = c (z + 0.044715 z^3): one exponential of base two, one
  // reciprocal and six multiply-adds; where thousands of rows pass through, the arithmetic is a third of the time.
  // e^-2y = inf gives 0, 0 gives z * up.
  const float k = -2.0f * 0.7978845608028654f * 1.4426950408889634f;  // -2 c log2(e)
  const float e = __builtin_amdgcn_exp2f(k * z * __builtin_fmaf(z * z, 0.044715f, 1.0f));
  return z * up * __builtin_amdgcn_rcpf(1.0f + e);
}
template <>
__device__ __forceinline__ float rv_gated<bf16_t, 1>(float z, float up) {
  return z * up * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * z));
}

// A weight vector that may be stored in either type (norm weights keep the
// type they were stored in).
__device__ __forceinline__ float rv_load_w(const void* w, int is_f32, int i) {
  return is_f32 ? ((const float*)w)[i] : rv_to_float(((const bf16_t*)w)[i]);
}
// V of them from element i on (i a multiple of V): in 16-byte reads where V is a multiple of 4 and the vector
// lies on a 16-byte boundary, as tensors do; one read for what element by element would be eight.
template <int V>
__device__ __forceinline__ void rv_load_w_vec(const void* w, int is_f32, int i, float* out) {
  if constexpr (V % 4 == 0) {
    if (((uintptr_t)w & 15) == 0) {  // the same for the whole launch
      if (is_f32) {
#pragma unroll
        for (int v = 0; v < V; v += 4) {
          const float4 q = *(const float4*)((const float*)w + i + v);
          out[v] = q.x, out[v + 1] = q.y, out[v + 2] = q.z, out[v + 3] = q.w;
        }
      } else if constexpr (V % 8 == 0) {
#pragma unroll
        for (int v = 0; v < V; v += 8) {
          const uint4 q = *(const uint4*)((const uint16_t*)w + i + v);
          const uint32_t u[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            out[v + 2 * j] = __uint_as_float(u[j] << 16);
            out[v + 2 * j + 1] = __uint_as_float(u[j] & 0xffff0000u);
          }
        }
      } else {
#pragma unroll
        for (int v = 0; v < V; v += 4) {
          const uint2 q = *(const uint2*)((const uint16_t*)w + i + v);
          out[v] = __uint_as_float(q.x << 16), out[v + 1] = __uint_as_float(q.x & 0xffff0000u);
          out[v + 2] = __uint_as_float(q.y << 16), out[v + 3] = __uint_as_float(q.y & 0xffff0000u);
        }
      }
      return;
    }
  }
#pragma unroll
  for (int v = 0; v < V; ++v) out[v] = rv_load_w(w, is_f32, i + v);
}

// ---------------------------------------------------------------------------
// wave64 and block reductions
// ---------------------------------------------------------------------------
__device__ __forceinline__ float rv_wave_sum(float v) {
#pragma unroll
  for (int off = RV_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, RV_WAVE);
  return v;
}
__device__ __forceinline__ float rv_wave_max(float v) {
#pragma unroll
  for (int off = RV_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, RV_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads (16 waves).  Every thread gets the
// result.  `scratch` holds 16 floats of LDS.  The order of the additions is
// fixed by the block size alone.
__device__ __forceinline__ float rv_block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (RV_WAVE - 1);
  const int wave = threadIdx.x / RV_WAVE;
  const int nwaves = (blockDim.x + RV_WAVE - 1) / RV_WAVE;
  v = rv_wave_sum(v);
  __syncthreads();  // scratch may still be read from an earlier call
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < nwaves; ++w) total += scratch[w];
  return total;
}

static inline int rv_div_up(long long a, long long b) { return (int)((a + b - 1) / b); }
