// out[M, N] = x[M, K] * W[N, K]^T for few rows (decode steps, the logits of a
// few positions): bf16 inputs, 32-bit accumulation on the matrix cores, bf16 or
// 32-bit output.  The time of such a product is the time to read W once, so the
// kernel is laid out around that read:
//
//   * a wave owns 16 rows of W and a slice of K; the waves of a block are the
//     K-slices of the same 16 rows, so that even a matrix with few rows keeps
//     every CU busy;
//   * W is the A operand of MFMA 16x16x32 (16 rows x 32 k): a lane reads 64
//     contiguous bytes of its row per step (four 16-byte loads, four MFMAs), the
//     four lanes of a row together 256 contiguous bytes; nothing passes
//     through LDS;
//   * x is the B operand, read from L2 (it is a few tens of kilobytes); up to
//     four column sets of 16 rows of x share each read of W;
//   * the partial sums of the K-slices are added through LDS in a fixed order,
//     so a row of x gives the same bits whatever else is in the batch.
//
// The reference hands these products to cuBLASLt, with its own kernels for the
// one-row case (v3/crates/rvllm-cutlass/src/cublaslt.rs:184-277, kernels/fp8_gemv.cu);
// this is the bf16 counterpart of the latter for up to 64 rows.
#include "common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 sk_bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float sk_f32x4;

union SkFrag {
  sk_bf16x8 v;
  uint4 u4;
};

#define SK_MAX_WAVES 16

template <typename TC>
__device__ __forceinline__ void sk_store4(TC* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void sk_store4<float>(float* p, float a, float b, float c, float d) {
  p[0] = a;
  p[1] = b;
  p[2] = c;
  p[3] = d;
}
template <>
__device__ __forceinline__ void sk_store4<uint16_t>(uint16_t* p, float a, float b, float c, float d) {
  p[0] = rv_f32_to_bf16_bits(a);
  p[1] = rv_f32_to_bf16_bits(b);
  p[2] = rv_f32_to_bf16_bits(c);
  p[3] = rv_f32_to_bf16_bits(d);
}

template <typename TC>
__device__ __forceinline__ void sk_store1(TC* p, float a);
template <>
__device__ __forceinline__ void sk_store1<float>(float* p, float a) {
  p[0] = a;
}
template <>
__device__ __forceinline__ void sk_store1<uint16_t>(uint16_t* p, float a) {
  p[0] = rv_f32_to_bf16_bits(a);
}

template <int MT, typename TC>
__global__ void __launch_bounds__(SK_MAX_WAVES * 64)
gemm_skinny_kernel(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w, TC* __restrict__ out, int M, int N,
                   int K, long long ldx, long long ldw, long long ldc, int slice_len) {
  extern __shared__ float red[];  // [waves][MT][64][4]
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int waves = blockDim.x >> 6;
  const int r16 = lane & 15;
  const int kb = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int row = n0 + r16 < N ? n0 + r16 : N - 1;
  const int kbeg = wave * slice_len;
  const int kend = kbeg + slice_len < K ? kbeg + slice_len : K;

  sk_f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (sk_f32x4){0.f, 0.f, 0.f, 0.f};

  const uint16_t* wrow = w + (size_t)row * ldw;
  const uint16_t* xrow[MT];
  bool xok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    xok[mt] = m < M;
    xrow[mt] = x + (size_t)(xok[mt] ? m : 0) * ldx;
  }

  for (int k0 = kbeg; k0 < kend; k0 += 128) {
    SkFrag a[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int off = k0 + kb * 32 + j * 8;
      if (off < kend)
        a[j].u4 = *(const uint4*)(wrow + off);
      else
        a[j].u4 = make_uint4(0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int off = k0 + kb * 32 + j * 8;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        SkFrag bfrag;
        if (off < kend && xok[mt])
          bfrag.u4 = *(const uint4*)(xrow[mt] + off);
        else
          bfrag.u4 = make_uint4(0, 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j].v, bfrag.v, acc[mt], 0, 0, 0);
      }
    }
  }

  if (waves > 1) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float* dst = red + (((size_t)wave * MT + mt) * 64 + lane) * 4;
      dst[0] = acc[mt][0];
      dst[1] = acc[mt][1];
      dst[2] = acc[mt][2];
      dst[3] = acc[mt][3];
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
      for (int wv = 0; wv < waves; ++wv) {  // fixed order: the sum does not depend on timing
        const float* src = red + (((size_t)wv * MT + mt) * 64 + lane) * 4;
        s0 += src[0];
        s1 += src[1];
        s2 += src[2];
        s3 += src[3];
      }
      acc[mt] = (sk_f32x4){s0, s1, s2, s3};
    }
  }
  // a lane holds out[m = mt*16 + r16][n0 + kb*4 .. + 3]
  const int nb = n0 + kb * 4;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r16;
    if (m >= M) continue;
    TC* o = out + (size_t)m * ldc + nb;
    if (nb + 3 < N) {
      sk_store4<TC>(o, acc[mt][0], acc[mt][1], acc[mt][2], acc[mt][3]);
    } else {
      if (nb + 0 < N) sk_store1<TC>(o + 0, acc[mt][0]);
      if (nb + 1 < N) sk_store1<TC>(o + 1, acc[mt][1]);
      if (nb + 2 < N) sk_store1<TC>(o + 2, acc[mt][2]);
    }
  }
}

// How many K-slices (waves a block) a product of this shape gets: enough that
// about 2048 waves run, each slice a multiple of 128 long.
extern "C" int rv_gemm_skinny_waves(int N, int K) {
  const int tiles = rv_div_up(N, 16);
  int waves = rv_div_up(2048, tiles);
  const int max_by_k = K / 128 > 0 ? K / 128 : 1;
  if (waves > max_by_k) waves = max_by_k;
  if (waves > SK_MAX_WAVES) waves = SK_MAX_WAVES;
  if (waves < 1) waves = 1;
  return waves;
}

template <int MT, typename TC>
static int sk_launch(hipStream_t stream, const uint16_t* x, const uint16_t* w, TC* out, int M, int N, int K,
                     long long ldx, long long ldw, long long ldc) {
  const int waves = rv_gemm_skinny_waves(N, K);
  const int slice_len = rv_div_up(rv_div_up(K, waves), 128) * 128;
  const size_t lds = waves > 1 ? (size_t)waves * MT * 64 * 4 * sizeof(float) : 0;
  gemm_skinny_kernel<MT, TC><<<dim3(rv_div_up(N, 16)), dim3(waves * 64), lds, stream>>>(x, w, out, M, N, K, ldx, ldw,
                                                                                       ldc, slice_len);
  RV_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

extern "C" int rv_gemm_skinny(hipStream_t stream, const void* x, const void* w, void* out, int out_dtype, int M, int N,
                              int K, long long ldx, long long ldw, long long ldc) {
  RV_CHECK(M >= 0 && M <= 64 && N > 0 && K > 0, "gemm_skinny: M=%d must be at most 64 (N=%d K=%d)", M, N, K);
  RV_CHECK(K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0, "gemm_skinny: K and the row strides must be multiples of 8");
  RV_CHECK(ldx >= K && ldw >= K && ldc >= N, "gemm_skinny: leading dimensions too small");
  RV_CHECK(((uintptr_t)x % 16) == 0 && ((uintptr_t)w % 16) == 0, "gemm_skinny: operands must be 16-byte aligned");
  if (M == 0) return 0;
  const int mt = rv_div_up(M, 16);
  const uint16_t* xp = (const uint16_t*)x;
  const uint16_t* wp = (const uint16_t*)w;
#define SK_CASE(MTV)                                                                                      \
  case MTV:                                                                                               \
    if (out_dtype == RV_F32) return sk_launch<MTV, float>(stream, xp, wp, (float*)out, M, N, K, ldx, ldw, ldc); \
    if (out_dtype == RV_BF16)                                                                             \
      return sk_launch<MTV, uint16_t>(stream, xp, wp, (uint16_t*)out, M, N, K, ldx, ldw, ldc);           \
    break;
  switch (mt) {
    SK_CASE(1)
    SK_CASE(2)
    SK_CASE(3)
    SK_CASE(4)
  }
#undef SK_CASE
  return rv_fail("gemm_skinny: unsupported output dtype %d", out_dtype);
}
