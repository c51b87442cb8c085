// C[M,N] = A[M,K] * W[N,K]^T with 32-bit multiply-adds (no matrix cores, no
// reduced-precision mode): the matrix product of the true 32-bit path, and the
// fallback that turns bf16 inputs into 32-bit logits.  The reference's products
// have the same form, D = A * B^T with 32-bit accumulation
// (v3/crates/rvllm-cutlass/src/cublaslt.rs:184,224,277).
//
// Tiles of 64x64 outputs, K in steps of 16 through LDS, 256 threads with 4x4
// outputs each.  Every output element is one chain of fused multiply-adds over
// k = 0..K-1 in order, so its value does not depend on M or on where its row
// lies in the batch.
#include "common.h"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TA* __restrict__ a, const TW* __restrict__ w, TC* __restrict__ c, int M, int N, int K,
                  long long lda, long long ldw, long long ldc) {
  __shared__ float a_s[GP_BK][GP_BM + 4];
  __shared__ float w_s[GP_BK][GP_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16;  // output columns tx*4 .. tx*4+3
  const int ty = tid / 16;  // output rows    ty*4 .. ty*4+3
  const int m0 = blockIdx.y * GP_BM;
  const int n0 = blockIdx.x * GP_BN;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  // each thread loads 4 elements of A and 4 of W per step: row = tid / 4, k = (tid % 4) * 4 ..
  const int lr = tid / 4;
  const int lk = (tid % 4) * 4;

  for (int k0 = 0; k0 < K; k0 += GP_BK) {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int k = k0 + lk + e;
      const int am = m0 + lr;
      const int wn = n0 + lr;
      a_s[lk + e][lr] = (am < M && k < K) ? rv_to_float(a[(size_t)am * lda + k]) : 0.f;
      w_s[lk + e][lr] = (wn < N && k < K) ? rv_to_float(w[(size_t)wn * ldw + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = a_s[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = w_s[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) c[(size_t)m * ldc + n] = rv_from_float<TC>(acc[i][j]);
    }
  }
}

extern "C" int rv_gemm_plain(hipStream_t stream, const void* a, int a_dtype, const void* w, int w_dtype, void* c,
                             int c_dtype, int M, int N, int K, long long lda, long long ldw, long long ldc) {
  RV_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  RV_CHECK(lda >= K && ldw >= K && ldc >= N, "gemm: leading dimensions too small");
  if (M == 0) return 0;
  dim3 grid(rv_div_up(N, GP_BN), rv_div_up(M, GP_BM)), block(256);
  RV_CHECK(grid.y < 65536, "gemm: M=%d too large for one launch", M);
#define RV_GP(TA, TW, TC)                                                                                     \
  gemm_plain_kernel<TA, TW, TC><<<grid, block, 0, stream>>>((const TA*)a, (const TW*)w, (TC*)c, M, N, K, lda, \
                                                            ldw, ldc)
  if (a_dtype == RV_F32 && w_dtype == RV_F32 && c_dtype == RV_F32) RV_GP(float, float, float);
  else if (a_dtype == RV_BF16 && w_dtype == RV_BF16 && c_dtype == RV_F32) RV_GP(bf16_t, bf16_t, float);
  else if (a_dtype == RV_BF16 && w_dtype == RV_BF16 && c_dtype == RV_BF16) RV_GP(bf16_t, bf16_t, bf16_t);
  else if (a_dtype == RV_F32 && w_dtype == RV_BF16 && c_dtype == RV_F32) RV_GP(float, bf16_t, float);
  else return rv_fail("gemm: unsupported dtypes a=%d w=%d c=%d", a_dtype, w_dtype, c_dtype);
#undef RV_GP
  RV_LAUNCH_CHECK("gemm_plain");
  return 0;
}
