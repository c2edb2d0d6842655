// C[M,N] (+)= A[M,K] * W[N,K]^T with float accumulation in plain FMA: the
// product of the true 32-bit path, and the fallback for operand types that
// the MFMA kernels do not take.  Weights are row-major [out, in] as the
// checkpoint stores them (out[r] = sum_c W[r,c] x[c],
// src/loader/parameters.rs:551-594 of the reference).  Each output element is
// summed over k in ascending order whatever M is, so a row's result does not
// depend on what else is in the batch.
#include "common.hpp"

namespace tl {

constexpr int BM = 64, BN = 64, BK = 16;

template <typename TA, typename TW, bool ACCUMULATE>
__global__ void __launch_bounds__(256)
gemm_plain_kernel(const TA* __restrict__ A, const TW* __restrict__ W, float* __restrict__ C, int M,
                  int N, int K, int lda, int ldw, int ldc) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  const int lr = tid / 4, lk = (tid % 4) * 4;     // this thread loads row lr, 4 k's from lk
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  const bool a_row = m0 + lr < M, w_row = n0 + lr < N;
  const TA* ap = A + (size_t)(m0 + lr) * lda;
  const TW* wp = W + (size_t)(n0 + lr) * ldw;
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int kk = k0 + lk + i;
      As[lk + i][lr] = (a_row && kk < K) ? to_f32(ap[kk]) : 0.f;
      Ws[lk + i][lr] = (w_row && kk < K) ? to_f32(wp[kk]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
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
      if (n >= N) continue;
      float* c = C + (size_t)m * ldc + n;
      *c = ACCUMULATE ? *c + acc[i][j] : acc[i][j];
    }
  }
}

template <typename TA, typename TW>
static int launch_plain(const void* A, const void* W, float* C, int M, int N, int K, int lda, int ldw,
                        int ldc, int accumulate, hipStream_t st) {
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  if (accumulate)
    gemm_plain_kernel<TA, TW, true><<<grid, 256, 0, st>>>((const TA*)A, (const TW*)W, C, M, N, K, lda,
                                                          ldw, ldc);
  else
    gemm_plain_kernel<TA, TW, false><<<grid, 256, 0, st>>>((const TA*)A, (const TW*)W, C, M, N, K,
                                                           lda, ldw, ldc);
  TL_LAUNCH_CHECK("gemm_plain");
  return 0;
}

}  // namespace tl

using namespace tl;

extern "C" int tl_gemm_plain(const void* A, int a_dt, const void* W, int w_dt, float* C, int M, int N,
                             int K, int lda, int ldw, int ldc, int accumulate, hipStream_t st) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm: leading dimensions lda=%d ldw=%d ldc=%d too small "
             "for K=%d N=%d", lda, ldw, ldc, K, N);
  TL_REQUIRE((M + BM - 1) / BM <= 65535, "gemm: M=%d has more row tiles than a grid holds", M);
  if (M == 0) return 0;
  if (a_dt == DT_F32 && w_dt == DT_F32)
    return launch_plain<float, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, st);
  if (a_dt == DT_BF16 && w_dt == DT_BF16)
    return launch_plain<bf16, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, st);
  if (a_dt == DT_BF16 && w_dt == DT_F32)
    return launch_plain<bf16, float>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, st);
  if (a_dt == DT_F32 && w_dt == DT_BF16)
    return launch_plain<float, bf16>(A, W, C, M, N, K, lda, ldw, ldc, accumulate, st);
  TL_REQUIRE(false, "gemm: unknown dtype codes a=%d w=%d", a_dt, w_dt);
}
