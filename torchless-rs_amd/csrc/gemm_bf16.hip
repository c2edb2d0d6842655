// bfloat16 products on the matrix cores, C[M,N] (+)= A[M,K] * W[N,K]^T, float
// accumulation, weights row-major [out, in] as the checkpoint stores them.
//
//  * gemm_skinny: M <= 64 rows (decode).  The step is bound by reading W once
//    from HBM, so W streams from global memory straight into MFMA operands:
//    a workgroup owns 16*NT output channels, its 8 waves split K between them
//    and every lane keeps several 16-byte loads in flight; the partial sums
//    meet in LDS.  The activations are the other operand, read through the
//    caches.  A row's result does not depend on M.
//  * gemm_tiled: any M (prefill).  128x128x64 tiles staged through LDS,
//    4 waves of 64x64, 32x32x16 MFMA, next tile prefetched into registers.
//
// Both need K % 8 == 0 and 16-byte aligned rows; callers fall back to the
// plain kernel otherwise.
#include "common.hpp"

namespace tl {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// ---------------------------------------------------------------- skinny ----
constexpr int SK_WAVES = 8;

template <int NT, int MT>
__global__ void __launch_bounds__(SK_WAVES * 64)
gemm_skinny_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M,
                   int N, int K, int accumulate) {
  __shared__ float red[SK_WAVES][NT * MT * 256];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int li = lane % 16, kg = lane / 16;
  const int n0 = blockIdx.x * (16 * NT);
  const int steps = (K + 63) / 64;
  const int per = (steps + SK_WAVES - 1) / SK_WAVES;
  const int s0 = wave * per;
  const int s1 = min(steps, s0 + per);

  const bf16* wrow[NT];
  const bf16* arow[MT];
#pragma unroll
  for (int t = 0; t < NT; ++t) wrow[t] = W + (size_t)min(n0 + t * 16 + li, N - 1) * K;
#pragma unroll
  for (int u = 0; u < MT; ++u) arow[u] = A + (size_t)min(u * 16 + li, M - 1) * K;

  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = f32x4{0.f, 0.f, 0.f, 0.f};

  // this lane's 16 consecutive k of a step: two chunks of 8
  auto load_step = [&](int s, bf16x8 (&wv)[NT][2], bf16x8 (&av)[MT][2]) {
    const int k = s * 64 + kg * 16;
    const bool ok0 = k + 8 <= K, ok1 = k + 16 <= K;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      wv[t][0] = ok0 ? load8(wrow[t] + k) : zero8();
      wv[t][1] = ok1 ? load8(wrow[t] + k + 8) : zero8();
    }
#pragma unroll
    for (int u = 0; u < MT; ++u) {
      av[u][0] = ok0 ? load8(arow[u] + k) : zero8();
      av[u][1] = ok1 ? load8(arow[u] + k + 8) : zero8();
    }
  };
  auto mma_step = [&](bf16x8 (&wv)[NT][2], bf16x8 (&av)[MT][2]) {
#pragma unroll
    for (int t = 0; t < NT; ++t)
#pragma unroll
      for (int u = 0; u < MT; ++u) {
        acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[t][0], av[u][0], acc[t][u], 0, 0, 0);
        acc[t][u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[t][1], av[u][1], acc[t][u], 0, 0, 0);
      }
  };

  bf16x8 w0[NT][2], a0[MT][2], w1[NT][2], a1[MT][2];
  int s = s0;
  if (s < s1) load_step(s, w0, a0);
  for (; s + 1 < s1; s += 2) {
    load_step(s + 1, w1, a1);
    mma_step(w0, a0);
    if (s + 2 < s1) load_step(s + 2, w0, a0);
    mma_step(w1, a1);
  }
  if (s < s1) mma_step(w0, a0);

  // acc[t][u][r] is D[n = 4*kg + r][m = li] of tile (t, u)
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][((t * MT + u) * 4 + r) * 64 + lane] = acc[t][u][r];
  __syncthreads();
  constexpr int NB = 16 * NT;
  for (int e = threadIdx.x; e < NB * 16 * MT; e += SK_WAVES * 64) {
    const int nl = e % NB, m = e / NB;
    const int t = nl / 16, u = m / 16;
    const int idx = ((t * MT + u) * 4 + (nl % 4)) * 64 + ((nl % 16) / 4) * 16 + (m % 16);
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) v += red[w][idx];
    const int n = n0 + nl;
    if (n < N && m < M) {
      float* c = C + (size_t)m * N + n;
      *c = accumulate ? *c + v : v;
    }
  }
}

template <int NT, int MT>
static int launch_skinny(const bf16* A, const bf16* W, float* C, int M, int N, int K, int accumulate,
                         hipStream_t st) {
  const int grid = (N + 16 * NT - 1) / (16 * NT);
  gemm_skinny_kernel<NT, MT><<<grid, SK_WAVES * 64, 0, st>>>(A, W, C, M, N, K, accumulate);
  TL_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

// ----------------------------------------------------------------- tiled ----
constexpr int TM = 128, TN = 128, TK = 64, TPAD = 8, TLD = TK + TPAD;

__global__ void __launch_bounds__(256)
gemm_tiled_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M,
                  int N, int K, int accumulate) {
  __shared__ __attribute__((aligned(16))) bf16 As[TM * TLD];
  __shared__ __attribute__((aligned(16))) bf16 Ws[TN * TLD];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int wm = (wave / 2) * 64, wn = (wave % 2) * 64;     // this wave's 64x64 corner in the tile
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;
  const int l32 = lane % 32, kh = lane / 32;

  // global -> register staging: 128 rows x 8 chunks of 8; thread takes chunk (tid%8) of rows tid/8 + 32*i
  const int lc = (tid % 8) * 8, lr = tid / 8;
  const bf16* ap[4];
  const bf16* wp[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    ap[i] = A + (size_t)min(m0 + lr + 32 * i, M - 1) * K + lc;
    wp[i] = W + (size_t)min(n0 + lr + 32 * i, N - 1) * K + lc;
  }
  bf16x8 ra[4], rw[4];
  auto fetch = [&](int k0) {
    const bool ok = k0 + lc + 8 <= K;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      ra[i] = ok ? load8(ap[i] + k0) : zero8();
      rw[i] = ok ? load8(wp[i] + k0) : zero8();
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      *reinterpret_cast<bf16x8*>(&As[(lr + 32 * i) * TLD + lc]) = ra[i];
      *reinterpret_cast<bf16x8*>(&Ws[(lr + 32 * i) * TLD + lc]) = rw[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  fetch(0);
  for (int k0 = 0; k0 < K; k0 += TK) {
    __syncthreads();                 // everyone is done reading the previous tile
    stash();
    __syncthreads();
    if (k0 + TK < K) fetch(k0 + TK);
#pragma unroll
    for (int kk = 0; kk < TK; kk += 16) {
      bf16x8 a[2], b[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        a[i] = *reinterpret_cast<const bf16x8*>(&As[(wm + 32 * i + l32) * TLD + kk + 8 * kh]);
        b[i] = *reinterpret_cast<const bf16x8*>(&Ws[(wn + 32 * i + l32) * TLD + kk + 8 * kh]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
    }
  }
  // acc[i][j][r]: row = 8*(r/4) + 4*kh + r%4, column = l32 of the 32x32 block
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn + 32 * j + l32;
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm + 32 * i + 8 * (r / 4) + 4 * kh + (r % 4);
        if (m < M) {
          float* c = C + (size_t)m * N + n;
          *c = accumulate ? *c + acc[i][j][r] : acc[i][j][r];
        }
      }
    }
}

}  // namespace tl

using namespace tl;

extern "C" int tl_gemm_bf16(const void* A, const void* W, float* C, int M, int N, int K, int accumulate,
                            hipStream_t st) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(K % 8 == 0, "gemm_bf16: K=%d must be a multiple of 8", K);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  if (M == 0) return 0;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if (M <= 16) return launch_skinny<1, 1>(a, w, C, M, N, K, accumulate, st);
  if (M <= 32) return launch_skinny<2, 2>(a, w, C, M, N, K, accumulate, st);
  if (M <= 64) return launch_skinny<2, 4>(a, w, C, M, N, K, accumulate, st);
  TL_REQUIRE((M + TM - 1) / TM <= 65535, "gemm_bf16: M=%d has more row tiles than a grid holds", M);
  dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
  gemm_tiled_kernel<<<grid, 256, 0, st>>>(a, w, C, M, N, K, accumulate);
  TL_LAUNCH_CHECK("gemm_tiled");
  return 0;
}

// For tests: force one of the two kernels whatever M is (M <= 64 for skinny).
extern "C" int tl_gemm_bf16_variant(const void* A, const void* W, float* C, int M, int N, int K,
                                    int accumulate, int variant, hipStream_t st) {
  TL_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  if (variant == 0) {
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
    gemm_tiled_kernel<<<grid, 256, 0, st>>>(a, w, C, M, N, K, accumulate);
    TL_LAUNCH_CHECK("gemm_tiled");
    return 0;
  }
  TL_REQUIRE(M <= 64, "gemm_skinny: M=%d is more than 64", M);
  if (variant == 1 && M <= 16) return launch_skinny<1, 1>(a, w, C, M, N, K, accumulate, st);
  if (variant == 2 && M <= 32) return launch_skinny<2, 2>(a, w, C, M, N, K, accumulate, st);
  if (variant == 3) return launch_skinny<2, 4>(a, w, C, M, N, K, accumulate, st);
  if (variant == 4 && M <= 16) return launch_skinny<4, 1>(a, w, C, M, N, K, accumulate, st);
  TL_REQUIRE(false, "gemm_bf16: variant %d does not take M=%d", variant, M);
}
