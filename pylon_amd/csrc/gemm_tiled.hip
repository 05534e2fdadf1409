// out[M, N] = a[M, K] * w[N, K]^T with float accumulation on the vector ALUs (no matrix
// cores, no reduced-precision mode): the matrix product of the true 32-bit path, and
// the fallback for element type pairings the fast kernels do not take.  Each output
// element is one chain of fused multiply-adds over k = 0..K-1 in ascending order, so its
// value does not depend on M, on the tile it falls in, or on what else is in the batch.
#include "common.h"

#define GT_BM 64
#define GT_BN 64
#define GT_BK 16

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(TC* __restrict__ out, const TA* __restrict__ a,
                                                         const TW* __restrict__ w, int M, int N, int K,
                                                         long long lda, long long ldw, long long ldc) {
  __shared__ float As[GT_BK][GT_BM + 4];
  __shared__ float Ws[GT_BK][GT_BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT_BM, n0 = blockIdx.x * GT_BN;
  const int lrow = tid >> 2, lk = (tid & 3) * 4;

  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GT_BK) {
    {
      const int m = m0 + lrow;
      const TA* ap = a + static_cast<size_t>(m) * lda + k0 + lk;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        As[lk + i][lrow] = (m < M && k0 + lk + i < K) ? to_float(ap[i]) : 0.f;
      const int n = n0 + lrow;
      const TW* wp = w + static_cast<size_t>(n) * ldw + k0 + lk;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        Ws[lk + i][lrow] = (n < N && k0 + lk + i < K) ? to_float(wp[i]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GT_BK; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[kk][tx * 4 + j];
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
      if (n < N) out[static_cast<size_t>(m) * ldc + n] = from_float<TC>(acc[i][j]);
    }
  }
}

template <typename TA, typename TW, typename TC>
static void launch_tiled(void* out, const void* a, const void* w, int M, int N, int K, long long lda,
                         long long ldw, long long ldc, hipStream_t stream) {
  dim3 grid((N + GT_BN - 1) / GT_BN, (M + GT_BM - 1) / GT_BM), block(256);
  hipLaunchKernelGGL((gemm_tiled_kernel<TA, TW, TC>), grid, block, 0, stream, (TC*)out, (const TA*)a,
                     (const TW*)w, M, N, K, lda, ldw, ldc);
}

extern "C" int pylon_gemm_tiled(void* out, int out_dtype, const void* a, int a_dtype, const void* w,
                                int w_dtype, int M, int N, int K, long long lda, long long ldw,
                                long long ldc, hipStream_t stream) {
  PYLON_REQUIRE(pylon_valid_dtype(out_dtype) && pylon_valid_dtype(a_dtype) && pylon_valid_dtype(w_dtype),
                "gemm_tiled: unknown dtype");
  PYLON_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_tiled: bad sizes M=%d N=%d K=%d", M, N, K);
  PYLON_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_tiled: a leading dimension is too short");
  if (M == 0) return 0;
  PYLON_REQUIRE((M + GT_BM - 1) / GT_BM <= 65535, "gemm_tiled: M=%d is too large for one launch", M);
  const int key = a_dtype * 100 + w_dtype * 10 + out_dtype;
  switch (key) {
    case 0:  // f32 f32 f32
      launch_tiled<float, float, float>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    case 111:
      launch_tiled<bf16_t, bf16_t, bf16_t>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    case 110:
      launch_tiled<bf16_t, bf16_t, float>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    case 101:
      launch_tiled<bf16_t, float, bf16_t>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    case 100:
      launch_tiled<bf16_t, float, float>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    case 10:  // f32 activations, bf16 weights, f32 out
      launch_tiled<float, bf16_t, float>(out, a, w, M, N, K, lda, ldw, ldc, stream);
      break;
    default:
      PYLON_REFUSE("gemm_tiled: no kernel for activations dtype %d, weights dtype %d, output dtype %d",
                   a_dtype, w_dtype, out_dtype);
  }
  PYLON_LAUNCHED("gemm_tiled");
}
