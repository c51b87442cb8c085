// A probe of what the memory delivers to a kernel that only reads: every
// block streams its share of a buffer in 16-byte loads, several in flight per
// lane, and folds what it read into one word so that no load can be dropped.
// Measurements price a decode step (which reads every weight and the cache
// once) against the rate this reaches as well as against the vendor's figure.
// The reference has a stand-alone bandwidth micro-benchmark of this kind for
// its GEMV (v3/crates/rvllm-bench/src/main.rs:488-551).
#include "common.h"

typedef unsigned int rv_u32x4 __attribute__((ext_vector_type(4)));

__global__ void __launch_bounds__(256) probe_read_kernel(const rv_u32x4* __restrict__ data, long long n16,
                                                         unsigned int* __restrict__ out) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  rv_u32x4 acc = {0u, 0u, 0u, 0u};
  for (; i + 3 * stride < n16; i += 4 * stride) {  // four loads asked for before any is used
    const rv_u32x4 a = __builtin_nontemporal_load(data + i);
    const rv_u32x4 b = __builtin_nontemporal_load(data + i + stride);
    const rv_u32x4 c = __builtin_nontemporal_load(data + i + 2 * stride);
    const rv_u32x4 d = __builtin_nontemporal_load(data + i + 3 * stride);
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n16; i += stride) acc ^= __builtin_nontemporal_load(data + i);
  unsigned int v = acc.x ^ acc.y ^ acc.z ^ acc.w;
#pragma unroll
  for (int off = RV_WAVE / 2; off > 0; off >>= 1) v ^= __shfl_xor(v, off, RV_WAVE);
  if ((threadIdx.x & (RV_WAVE - 1)) == 0) atomicXor(out + (blockIdx.x & 63), v);
}

// Reads `bytes` (a multiple of 16, from a 16-byte aligned address) once; `out` holds 64 words that the
// caller has cleared.
extern "C" int rv_probe_read(hipStream_t stream, const void* data, long long bytes, unsigned int* out, int blocks) {
  RV_CHECK(data && out && bytes > 0 && bytes % 16 == 0 && ((uintptr_t)data % 16) == 0,
           "probe_read: a 16-byte aligned buffer of a multiple of 16 bytes expected");
  RV_CHECK(blocks >= 1 && blocks <= 65536, "probe_read: bad number of blocks %d", blocks);
  probe_read_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const rv_u32x4*)data, bytes / 16, out);
  RV_LAUNCH_CHECK("probe_read");
  return 0;
}
