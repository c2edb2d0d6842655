// bfloat16 products on the matrix cores, C[M,N] (+)= A[M,K] * W[N,K]^T, float
// accumulation, weights row-major [out, in] as the checkpoint stores them.
//
//  * gemm_skinny: at most 16 rows a tile (decode).  The step is bound by reading
//    W once from HBM, so W streams from global memory straight into MFMA
//    operands: a workgroup owns 16*NT output channels, its waves split K
//    between them and every lane keeps several 16-byte loads in flight; the
//    partial sums meet in LDS.  The activations are the other operand, read
//    through the caches.  A row's result does not depend on M.  The epilogue
//    may carry the halves of an RMSNorm (NormSplit).  It can also read W from a
//    copy laid out in tiles (see tile_weights_kernel): a wave's loads are then one
//    run of consecutive bytes, which the memory serves faster than 16 rows apart.
//  * gemm_rows: at most 16 rows against many channels (gate|up, the head) when K is a multiple
//    of 512: W is read 1 KB of a row at a time, which the memory serves fastest, and turned
//    into MFMA operands in LDS.
//  * gemm_qkv_rope_commit: the skinny product for the fused q|k|v projection of
//    single-token steps, with rotation and the write into the cache's pages.
//  * gemm_mid: 17..128 rows.  The activations of a k-step are shared by the four
//    waves through LDS; K may be cut over workgroups into partial sums.
// Products with more rows (prefill, large decode batches) are the BLAS library's, as the
// reference hands its products to the vendor's library.
//
// All need K % 8 == 0 and 16-byte aligned rows; callers fall back to the
// plain kernel otherwise.
#include "common.hpp"

namespace tl {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
// A load of weights that a step of at most 16 rows reads once: marked non-temporal.  A plain read of a
// large buffer reaches 6.7 to 6.95 TB/s with such loads against 6.0 without (csrc/measure/ceilings.hip); gate|up
// at 8 rows went from 41.6 to 38.0 us, down from 21.9 to 20.4, o from 9.0 to 8.3.  Not for the kernels
// whose cache lines are shared between load instructions or waves (gemm_mid: a decode step at batch 64
// 11.9 against 10.85 ms; the keys and values of decode attention: 11.56 against 10.85 ms), and the fused
// q|k|v kernel gains nothing from it.
__device__ __forceinline__ bf16x8 load8_once(const bf16* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
}
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// what happens to the product
constexpr int EPI_STORE = 0;        // C = product (float)
constexpr int EPI_ACCUMULATE = 1;   // C += product (float; the residual stream)
constexpr int EPI_SILU_PAIR = 2;    // W's rows come in groups of 64 (32 gate rows, their 32 up rows):
                                    // C is bfloat16 [M, N/2] = silu(gate) * up

// An RMSNorm cut in two around a product of at most 16 rows, so that the norm needs no
// kernel of its own.  The product that completes the residual stream (accumulate epilogue)
// also writes xt = bfloat16(x * norm_w) and, per workgroup and row, the sum of x^2 over its
// channels (`ssq_out`, [16][workgroups]).  The product that reads xt adds those sums up in
// a fixed order and multiplies its results by rsqrt(sum * inv_h + eps) (`ssq_in`, `n_part`):
// y = x / sqrt(mean(x^2) + eps) * w  (src/kernels/mod.rs:558-568 of the reference), with the
// division moved behind the product, where it is a factor per row.
struct NormSplit {
  const float* ssq_in;      // reader: partial sums [16][n_part]; null: no factor
  int n_part;
  float inv_h, eps;
  const float* norm_w;      // writer: the next norm's weight [N]; null: plain epilogue
  bf16* xt;                 // [M][N]
  float* ssq_out;           // [16][gridDim.x]
};

// rsqrt(mean + eps) of rows 0..15 into rs[16], by the first 256 threads (16 per row), in two
// steps so that the loads are under way while the product runs: `fetch` early, `finish` before
// the barrier that precedes the epilogue.  ssq_in is [16][n_part].
struct RowFactors {
  f32x4 part[4];
  __device__ __forceinline__ void fetch(const NormSplit& ns) {
    const int tid = threadIdx.x, m = tid / 16, jl = tid % 16;
    if (tid >= 256) return;
    const float* row = ns.ssq_in + (size_t)m * ns.n_part;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int j = jl * 4 + 64 * i;
      f32x4 v = f32x4{0.f, 0.f, 0.f, 0.f};
      if (j + 3 < ns.n_part && ns.n_part % 4 == 0) {
        v = *reinterpret_cast<const f32x4*>(row + j);
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (j + e < ns.n_part) v[e] = row[j + e];
      }
      part[i] = v;
    }
  }
  __device__ __forceinline__ void finish(const NormSplit& ns, float* rs) {
    const int tid = threadIdx.x, m = tid / 16, jl = tid % 16;
    if (tid >= 256) return;
    float v = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) v += (part[i][0] + part[i][1]) + (part[i][2] + part[i][3]);
    const float* row = ns.ssq_in + (size_t)m * ns.n_part;
    for (int j = 256 + jl; j < ns.n_part; j += 16) v += row[j];      // more than 256 workgroups wrote
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
    if (jl == 0) rs[m] = rsqrtf(v * ns.inv_h + ns.eps);
  }
};

// ----------------------------------------------------------- tiled copy ----
// The copy of W [N, K] that the kernels for at most 16 rows stream from, when N % 16 == 0 and
// K % 64 == 0: [tiles of R rows][K/64 steps][2 halves][4 groups][R rows][8], where element
// (tile T, step s, half c, group g, row r, e) is W[rows[R T + r]][64 s + 16 g + 8 c + e]
// (`rows`: a permutation of the rows, or null for none; the last tile may have fewer rows than
// places).  R is 16, or the share of channels of a workgroup of the kernel that reads the copy where
// that is more (20 for 5,120 channels on 256 compute units): a workgroup's weights are then one run of
// memory, and no line of it is another workgroup's as well.  With R = 16 one MFMA operand of a wave
// (row r = lane % 16, group g = lane / 16, 8 values) is 1 KB of consecutive memory in the order of the
// lanes, a step 2 KB, and a tile's steps follow each other.
constexpr int TILE_STEP = 1024;        // elements of one step of a tile of 16 rows

__global__ void __launch_bounds__(256)
tile_weights_kernel(const bf16* __restrict__ W, const int* __restrict__ rows, int N, int K, int R,
                    bf16* __restrict__ Wt) {
  const size_t chunks = (size_t)N * K / 8;
  const size_t per_row = K / 8, steps = K / 64;
  for (size_t c = (size_t)blockIdx.x * 256 + threadIdx.x; c < chunks; c += (size_t)gridDim.x * 256) {
    const size_t n = c / per_row, kc = c % per_row;              // row of the copy, chunk of 8 along k
    const size_t step = kc / 8, g = (kc % 8) / 2, half = kc % 2, tile = n / R, r = n % R;
    const size_t src = rows ? (size_t)rows[n] : n;
    *reinterpret_cast<bf16x8*>(Wt + (((((tile * steps + step) * 2 + half) * 4 + g) * R + r) * 8)) =
        load8(W + src * K + kc * 8);
  }
}

// ---------------------------------------------------------------- skinny ----
// TILED: W is the tiled copy (N % 16 == 0, K % 64 == 0, hence FULLK)
template <int NT, int MT, int SK_WAVES, bool FULLK, bool TILED = false>      // FULLK: K % 64 == 0, no load needs a guard (and a branch)
__global__ void __launch_bounds__(SK_WAVES * 64)
gemm_skinny_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M,
                   int N, int K, int epilogue, NormSplit ns, int rows_per_wg) {
  // rows_per_wg: the channels a workgroup owns, at most 16 NT (0: all 16 NT).  A compute unit streams
  // at a rate of its own, so a product is fastest when every unit has the same share of W: the
  // launcher picks N / units where that is no multiple of 16, and the lanes of an MFMA tile that
  // have no channel read another's again and their sums are dropped.
  __shared__ float red[SK_WAVES][NT * MT * 256];
  __shared__ float rs[16];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  const int li = lane % 16, kg = lane / 16;
  const int R = rows_per_wg > 0 ? rows_per_wg : 16 * NT;
  const int TH = R > 16 ? R : 16;                     // rows of a tile of the tiled copy: the workgroup's share
  const int n0 = blockIdx.x * R;
  const int steps = (K + 63) / 64;
  const int per = (steps + SK_WAVES - 1) / SK_WAVES;
  const int s0 = wave * per;
  const int s1 = min(steps, s0 + per);

  const bf16* wrow[NT];
  const bf16* arow[MT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int gr = min(n0 + min(t * 16 + li, R - 1), N - 1);          // this lane's channel (clamped: never a branch)
    wrow[t] = TILED ? W + (size_t)(gr / TH) * TH * K + kg * (TH * 8) + (gr % TH) * 8 : W + (size_t)gr * K;
  }
#pragma unroll
  for (int u = 0; u < MT; ++u) arow[u] = A + (size_t)min(u * 16 + li, M - 1) * K;

  f32x4 acc[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u) acc[t][u] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int tile_step = TH * 64;                      // elements of one step of such a tile
  // this lane's 16 consecutive k of a step: two chunks of 8
  auto load_step = [&](int s, bf16x8 (&wv)[NT][2], bf16x8 (&av)[MT][2]) {
    const int k = s * 64 + kg * 16;
    const bool ok0 = FULLK || k + 8 <= K, ok1 = FULLK || k + 16 <= K;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (TILED && NT == 1) {
        wv[t][0] = load8_once(wrow[t] + (size_t)s * tile_step);
        wv[t][1] = load8_once(wrow[t] + (size_t)s * tile_step + tile_step / 2);
      } else if constexpr (TILED) {
        // two tiles a workgroup (widths whose share of channels is above 16): the mark loses here, a decode
        // step of 40 layers 5,120 wide takes 6.0 instead of 6.3 ms at 16 rows without it
        wv[t][0] = load8(wrow[t] + (size_t)s * tile_step);
        wv[t][1] = load8(wrow[t] + (size_t)s * tile_step + tile_step / 2);
      } else {
        wv[t][0] = ok0 ? load8_once(wrow[t] + k) : zero8();
        wv[t][1] = ok1 ? load8_once(wrow[t] + k + 8) : zero8();
      }
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

  // What the accumulating epilogue adds to and scales by is asked for now, where a thread has
  // one element of it at most: the answers are there when the sums are.
  constexpr int NB = 16 * NT;
  constexpr bool one_each = NB * 16 * MT <= SK_WAVES * 64;
  const bool writer = MT == 1 && ns.norm_w != nullptr;          // with EPI_ACCUMULATE only (checked on the host)
  float c_old = 0.f, w_norm = 0.f;
  if (one_each && epilogue == EPI_ACCUMULATE) {
    const int nl = threadIdx.x % NB, m = threadIdx.x / NB;
    if ((int)threadIdx.x < NB * 16 * MT && nl < R && n0 + nl < N && m < M) {
      c_old = C[(size_t)m * N + n0 + nl];
      if (writer) w_norm = ns.norm_w[n0 + nl];
    }
  }
  bf16x8 w0[NT][2], a0[MT][2], w1[NT][2], a1[MT][2];
  int s = s0;
  if (s < s1) load_step(s, w0, a0);
  const bool scaled = MT == 1 && ns.ssq_in != nullptr;
  RowFactors rf;
  if (scaled) rf.fetch(ns);
  for (; s + 1 < s1; s += 2) {
    load_step(s + 1, w1, a1);
    mma_step(w0, a0);
    if (s + 2 < s1) load_step(s + 2, w0, a0);
    mma_step(w1, a1);
  }
  if (s < s1) mma_step(w0, a0);

  if (scaled) rf.finish(ns, rs);
  // acc[t][u][r] is D[n = 4*kg + r][m = li] of tile (t, u)
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[wave][((t * MT + u) * 4 + r) * 64 + lane] = acc[t][u][r];
  __syncthreads();
  auto total = [&](int nl, int m) {
    const int t = nl / 16, u = m / 16;
    const int idx = ((t * MT + u) * 4 + (nl % 4)) * 64 + ((nl % 16) / 4) * 16 + (m % 16);
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < SK_WAVES; ++w) v += red[w][idx];
    return scaled ? v * rs[m % 16] : v;
  };
  if (epilogue == EPI_SILU_PAIR) {
    // rows come in groups of 64: 32 gate rows, then the 32 up rows that belong to them
    if constexpr (NB % 64 == 0) {
      bf16* H = reinterpret_cast<bf16*>(C);
      const int NH = N / 2;
      for (int e = threadIdx.x; e < (NB / 2) * 16 * MT; e += SK_WAVES * 64) {
        const int jl = e % (NB / 2), m = e / (NB / 2);
        const int grp = jl / 32, j = jl % 32;
        const int n = (n0 / 2) + jl;
        if (n < NH && m < M) {
          const float g = total(grp * 64 + j, m), u = total(grp * 64 + 32 + j, m);
          H[(size_t)m * NH + n] = (bf16)((g / (1.0f + expf(-g))) * u);
        }
      }
    }
    return;
  }
  for (int e = threadIdx.x; e < NB * 16 * MT; e += SK_WAVES * 64) {
    const int nl = e % NB, m = e / NB;
    const float v = total(nl, m);
    const int n = n0 + nl;
    float xn = 0.f;
    if (nl < R && n < N && m < M) {
      float* c = C + (size_t)m * N + n;
      xn = (epilogue == EPI_ACCUMULATE) ? (one_each ? c_old : *c) + v : v;
      *c = xn;
      if (writer) ns.xt[(size_t)m * N + n] = (bf16)(xn * (one_each ? w_norm : ns.norm_w[n]));
    }
    if (writer) {                  // whole waves get here: NB lanes in a row share m
      float q = xn * xn;
#pragma unroll
      for (int o = NB / 2; o > 0; o >>= 1) q += __shfl_xor(q, o, WAVE);
      if (nl == 0) ns.ssq_out[(size_t)m * gridDim.x + blockIdx.x] = q;
    }
  }
}

static bool tiles_fit(int N, int K) { return N % 16 == 0 && K % 64 == 0; }
// rows of a tile of the copy that a workgroup with R channels reads
static int tile_height(int R) { return R > 16 ? R : 16; }

template <int NT, int MT, int SK_WAVES = 8>
static int launch_skinny(const bf16* A, const bf16* W, float* C, int M, int N, int K, int epilogue,
                         hipStream_t st, NormSplit ns = NormSplit{}, const bf16* Wt = nullptr, int rows_per_wg = 0,
                         int wt_height = 16) {
  const int R = rows_per_wg > 0 ? rows_per_wg : 16 * NT;
  const int grid = (N + R - 1) / R;
  if constexpr (MT == 1 && SK_WAVES == 8 && NT <= 2) {
    if (Wt != nullptr && tiles_fit(N, K)) {
      TL_REQUIRE(wt_height == tile_height(R), "gemm: the tiled copy has tiles of %d rows, the kernel reads tiles of %d",
                 wt_height, tile_height(R));
      gemm_skinny_kernel<NT, MT, SK_WAVES, true, true><<<grid, SK_WAVES * 64, 0, st>>>(A, Wt, C, M, N, K, epilogue, ns, R);
      TL_LAUNCH_CHECK("gemm_skinny");
      return 0;
    }
  }
  if (K % 64 == 0)
    gemm_skinny_kernel<NT, MT, SK_WAVES, true><<<grid, SK_WAVES * 64, 0, st>>>(A, W, C, M, N, K, epilogue, ns, R);
  else
    gemm_skinny_kernel<NT, MT, SK_WAVES, false><<<grid, SK_WAVES * 64, 0, st>>>(A, W, C, M, N, K, epilogue, ns, R);
  TL_LAUNCH_CHECK("gemm_skinny");
  return 0;
}

static int compute_units() {
  static int cus = 0;
  if (cus == 0) {
    int dev = 0, n = 0;
    if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cus = n;
  }
  return cus;
}

// The channels a workgroup of the kernel for at most 16 rows owns (16 to 32).  One tile of 16 each
// while the device has a unit for every tile; beyond that the tiles would go round the units
// unevenly (320 tiles on 256 units take as long as 512), so the channels are dealt in equal shares
// to a whole number of rounds of workgroups.
static int balanced_share(int N) {
  const int cus = compute_units();
  if ((N + 15) / 16 <= cus) return 16;
  const long long rounds = ((long long)N + 32LL * cus - 1) / (32LL * cus);
  const long long wgs = rounds * cus;
  const int share = (int)((N + wgs - 1) / wgs);
  return share < 16 ? 16 : share;
}

// the product for at most 16 rows and not many channels, in balanced shares
static int launch_shares(const bf16* A, const bf16* W, const bf16* Wt, int wt_height, float* C, int M, int N, int K,
                         int epilogue, hipStream_t st, NormSplit ns, int share) {
  if (share <= 16) return launch_skinny<1, 1, 8>(A, W, C, M, N, K, epilogue, st, ns, Wt, share, wt_height);
  return launch_skinny<2, 1, 8>(A, W, C, M, N, K, epilogue, st, ns, Wt, share, wt_height);
}

// ------------------------------------------------------- rows, 1 KB at a time ----
// At most 16 rows of activations against many channels (gate|up, the head), from the weights as
// stored.  The memory serves a load fastest when a wave's 64 lanes take 1 KB of one row, not
// sixteen pieces of sixteen rows, so that is how W is read here: a workgroup owns 64 channels,
// its 4 waves split K in chunks of 512; a wave reads 16 rows x 512 k with 16 loads, turns them in
// its own 16 KB of LDS into MFMA operands (channel = lane % 16), and multiplies them with the
// activations of that chunk, which it keeps in registers for the workgroup's 4 groups of 16
// channels.  No barrier until the waves' sums meet; the epilogues are those of gemm_skinny
// (store, accumulate, silu(gate) * up in groups of 64 rows, a factor per row).
constexpr int ROWS_CHUNK = 512;                          // k a load instruction takes of one row
constexpr int ROWS_LDS = 4 * 16 * ROWS_CHUNK * 2;        // bytes: a tile of 16 rows x 512 k for each wave
constexpr int NRB = 4;                                   // groups of 16 channels a workgroup

__global__ void __launch_bounds__(256, 2)
gemm_rows_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M, int N,
                 int K, int epilogue, NormSplit ns) {
  extern __shared__ __attribute__((aligned(16))) unsigned char rows_smem[];
  __shared__ float rs[16];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, li = lane % 16, kg = lane / 16;
  const int n0 = blockIdx.x * (16 * NRB);
  bf16* T = reinterpret_cast<bf16*>(rows_smem) + wave * (16 * ROWS_CHUNK);
  const int chunks = K / ROWS_CHUNK;
  const int c0 = wave * chunks / 4, c1 = (wave + 1) * chunks / 4;       // this wave's chunks of K
  const bf16* alane = A + (size_t)min(li, M - 1) * K + kg * 8;          // + chunk * 512 + j * 32

  f32x4 acc[NRB];
#pragma unroll
  for (int t = 0; t < NRB; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 wcur[16], areg[16];
  auto load_w = [&](int c, int rb, bf16x8 (&w)[16]) {
    // a uniform base and 32-bit offsets in bytes, worked out anew each time (kept across the loop,
    // sixteen 64-bit addresses would take the registers that the loads in flight need)
    const bf16* base = W + (size_t)(n0 + rb * 16) * K + (size_t)c * ROWS_CHUNK;
    unsigned off = lane * 16, row_bytes = 2u * K;
    asm volatile("" : "+v"(off), "+v"(row_bytes));
#pragma unroll
    for (int i = 0; i < 16; ++i)
      w[i] = load8_once(reinterpret_cast<const bf16*>(reinterpret_cast<const char*>(base) + (off + i * row_bytes)));
  };
  const bool scaled = ns.ssq_in != nullptr;
  RowFactors rf;
  if (c0 < c1) load_w(c0, 0, wcur);
  if (scaled) rf.fetch(ns);
  for (int c = c0; c < c1; ++c) {
#pragma unroll
    for (int j = 0; j < 16; ++j) areg[j] = load8(alane + (size_t)c * ROWS_CHUNK + j * 32);
#pragma unroll
    for (int rb = 0; rb < NRB; ++rb) {
      // row i's chunk of 8 values q goes to place q ^ i of the row: the reads below, 16 rows at the
      // same q, then fall on 16 different groups of banks
#pragma unroll
      for (int i = 0; i < 16; ++i) *reinterpret_cast<bf16x8*>(&T[i * ROWS_CHUNK + ((lane ^ i) * 8)]) = wcur[i];
      __builtin_amdgcn_wave_barrier();
      // the next 16 rows are asked for as soon as these have left their registers; a wave spends
      // most of its time waiting for them, with other waves' loads under way meanwhile
      if (rb < NRB - 1) load_w(c, rb + 1, wcur);
      else if (c + 1 < c1) load_w(c + 1, 0, wcur);
#pragma unroll
      for (int j = 0; j < 16; ++j) {
        const bf16x8 wf = *reinterpret_cast<const bf16x8*>(&T[li * ROWS_CHUNK + (((4 * j + kg) ^ li) * 8)]);
        acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, areg[j], acc[rb], 0, 0, 0);
      }
      __builtin_amdgcn_wave_barrier();
    }
  }
  if (scaled) rf.finish(ns, rs);
  __syncthreads();                                     // every wave is done with its tile: the sums take its place
  float* red = reinterpret_cast<float*>(rows_smem);   // [4 waves][NRB tiles][4][64]
#pragma unroll
  for (int t = 0; t < NRB; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave * (NRB * 256) + (t * 4 + r) * 64 + lane] = acc[t][r];   // D[n = 4 kg + r][m = li] of tile t
  __syncthreads();
  auto total = [&](int nl, int m) {
    const int idx = ((nl / 16) * 4 + (nl % 4)) * 64 + ((nl % 16) / 4) * 16 + m;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) v += red[w * (NRB * 256) + idx];
    return scaled ? v * rs[m] : v;
  };
  if (epilogue == EPI_SILU_PAIR) {                     // the 64 rows are 32 gate rows and their 32 up rows
    bf16* H = reinterpret_cast<bf16*>(C);
    const int NH = N / 2;
    for (int e = threadIdx.x; e < 32 * 16; e += 256) {
      const int j = e % 32, m = e / 32;
      if (m < M) {
        const float g = total(j, m), u = total(32 + j, m);
        H[(size_t)m * NH + n0 / 2 + j] = (bf16)((g / (1.0f + expf(-g))) * u);
      }
    }
    return;
  }
  for (int e = threadIdx.x; e < 16 * NRB * 16; e += 256) {
    const int nl = e % (16 * NRB), m = e / (16 * NRB);
    if (m < M) {
      float* c = C + (size_t)m * N + n0 + nl;
      *c = (epilogue == EPI_ACCUMULATE) ? *c + total(nl, m) : total(nl, m);
    }
  }
}

static bool rows_fit(int M, int N, int K) { return M <= 16 && N % 64 == 0 && K % ROWS_CHUNK == 0; }

static int launch_rows(const bf16* A, const bf16* W, float* C, int M, int N, int K, int epilogue, hipStream_t st,
                       NormSplit ns = NormSplit{}) {
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_rows_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, ROWS_LDS);
    if (e != hipSuccess) {
      set_error("gemm_rows: cannot have %d bytes of LDS: %s", ROWS_LDS, hipGetErrorString(e));
      return 2;
    }
    raised = true;
  }
  gemm_rows_kernel<<<N / (16 * NRB), 256, ROWS_LDS, st>>>(A, W, C, M, N, K, epilogue, ns);
  TL_LAUNCH_CHECK("gemm_rows");
  return 0;
}

// ------------------------------------------------- q|k|v of single tokens ----
// The skinny product (8 waves over K, up to 16 rows) for the fused projection of a step with
// one token a sequence, with what follows it done on the sums while they are in LDS: rotation
// of q and k by the position, q to its buffer, k and v into the sequence's page (v transposed).
// The projection's channels are dealt in units of 8 weight rows, d / 8 a head: unit h of a q or
// k head holds the first channels of its pairs 4h..4h+3 and then their second channels
// (`pair_channels`: with all of a head rotated in halves these are 4h..4h+3 and d/2+4h..d/2+4h+3),
// so that both channels of a rotated pair meet in one workgroup; a unit of a v head holds 8
// channels in a row.  A workgroup owns `units` consecutive units (at most 2 NT, two to an MFMA
// tile of 16 rows; rows of a tile without a unit load nothing).  The launcher deals the
// units in equal shares to the compute units, because each of them streams at a rate of its own
// (7B: 768 units are 3 for each of 256).
// The sums and the rotation are those of the unfused kernels, bit for bit
// (a' = a c - b s; b' = a s + b c; src/kernels/mod.rs:603-605 of the reference).
// TILED: W is the tiled copy whose tile (head, t) holds units 2t and 2t+1 of the head, first
// channels in its rows 0..7, second channels in 8..15 (`tl_qkv_tile_rows`).
constexpr int QKV_WAVES = 8;

template <bool TILED, int NT>
__global__ void __launch_bounds__(QKV_WAVES * 64)
gemm_qkv_rope_commit_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, int M, int K,
                            const int* __restrict__ row_pos, Rotation rot,
                            const int* __restrict__ table, int table_stride, int ring_pages, int nq,
                            int nkv, int d, bf16* __restrict__ q, bf16* __restrict__ pages, NormSplit ns,
                            int units) {
  __shared__ float red[QKV_WAVES][NT * 256];
  __shared__ float cs[2 * NT][16][4], sn[2 * NT][16][4];
  __shared__ float rs[16];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64;
  const int li = lane % 16, kg = lane / 16;
  const int per_head = d / 8, n_units = (nq + 2 * nkv) * per_head;
  const int g0 = blockIdx.x * units;
  const int mine = min(units, n_units - g0);           // units of this workgroup
  const bf16* wrow[NT];
  bool loads[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) {
    const int u = 2 * t + li / 8, j = li % 8;          // this lane's row of tile t: row j of unit u
    loads[t] = u < mine;
    const int g = g0 + (loads[t] ? u : 0);
    const int head = g / per_head, h = g % per_head;
    const bool rotated = head < nq + nkv;
    if constexpr (TILED) {
      const int sub = h % 2;
      const int r = rotated ? (j < 4 ? 4 * sub + j : 8 + 4 * sub + j - 4) : 8 * sub + j;
      wrow[t] = W + (size_t)(head * (d / 16) + h / 2) * 16 * K + kg * 128 + r * 8;
    } else {
      int ch = 8 * h + j;
      if (rotated) {
        int ca, cb;
        pair_channels(4 * h + (j < 4 ? j : j - 4), rot.rotary_dim, rot.interleaved, ca, cb);
        ch = j < 4 ? ca : cb;
      }
      wrow[t] = W + ((size_t)head * d + ch) * K;
    }
  }
  const bf16* arow = A + (size_t)min(li, M - 1) * K;
  const int steps = (K + 63) / 64;
  const int per = (steps + QKV_WAVES - 1) / QKV_WAVES;
  const int s0 = wave * per, s1 = min(steps, s0 + per);

  f32x4 acc[NT];
#pragma unroll
  for (int t = 0; t < NT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  auto load_step = [&](int s, bf16x8 (&wv)[NT][2], bf16x8 (&av)[2]) {
    const int k = s * 64 + kg * 16;
    const bool ok0 = k + 8 <= K, ok1 = k + 16 <= K;
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      if constexpr (TILED) {
        wv[t][0] = loads[t] ? load8(wrow[t] + (size_t)s * TILE_STEP) : zero8();
        wv[t][1] = loads[t] ? load8(wrow[t] + (size_t)s * TILE_STEP + TILE_STEP / 2) : zero8();
      } else {
        wv[t][0] = (ok0 && loads[t]) ? load8(wrow[t] + k) : zero8();
        wv[t][1] = (ok1 && loads[t]) ? load8(wrow[t] + k + 8) : zero8();
      }
    }
    av[0] = ok0 ? load8(arow + k) : zero8();
    av[1] = ok1 ? load8(arow + k + 8) : zero8();
  };
  auto mma_step = [&](bf16x8 (&wv)[NT][2], bf16x8 (&av)[2]) {
#pragma unroll
    for (int t = 0; t < NT; ++t) {
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[t][0], av[0], acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[t][1], av[1], acc[t], 0, 0, 0);
    }
  };
  bf16x8 w0[NT][2], a0[2], w1[NT][2], a1[2];
  int s = s0;
  if (s < s1) load_step(s, w0, a0);
  // the threads of the epilogue: 128 a unit; of a rotated unit 64 work, one a row and pair
  const int eu = tid / 128, et = tid % 128;
  const int eg = g0 + min(eu, mine - 1);
  const int ehead = eg / per_head, eh = eg % per_head;
  const bool e_on = eu < mine, e_rot = ehead < nq + nkv;
  if (e_on && e_rot && et < 64) {              // while the first loads are under way
    const int m = et / 4, j = et % 4, i = 4 * eh + j;
    if (m < M && 2 * i < rot.rotary_dim) sincosf(rot.inv_freq[i] * (float)row_pos[m], &sn[eu][m][j], &cs[eu][m][j]);
  }
  const bool scaled = ns.ssq_in != nullptr;
  RowFactors rf;
  if (scaled) rf.fetch(ns);
  for (; s + 1 < s1; s += 2) {
    load_step(s + 1, w1, a1);
    mma_step(w0, a0);
    if (s + 2 < s1) load_step(s + 2, w0, a0);
    mma_step(w1, a1);
  }
  if (s < s1) mma_step(w0, a0);
  if (scaled) rf.finish(ns, rs);
#pragma unroll
  for (int t = 0; t < NT; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) red[wave][(t * 4 + r) * 64 + lane] = acc[t][r];     // D[n = 4 kg + r][m = li] of tile t
  __syncthreads();
  auto total = [&](int row, int m) {               // row: 8 u + j, row j of the workgroup's unit u
    const int nl = row % 16;
    const int idx = ((row / 16) * 4 + nl % 4) * 64 + (nl / 4) * 16 + m;
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < QKV_WAVES; ++w) v += red[w][idx];
    return scaled ? v * rs[m] : v;
  };
  if (!e_on) return;
  const size_t page_elems = 2 * (size_t)nkv * PAGE * d;
  if (e_rot) {
    const int m = et / 4, j = et % 4;
    if (et < 64 && m < M) {
      const int i = 4 * eh + j;
      float ra = total(8 * eu + j, m), rb = total(8 * eu + 4 + j, m);
      if (2 * i < rot.rotary_dim) rotate_pair(ra, rb, cs[eu][m][j], sn[eu][m][j], ra, rb);
      int ia, ib;
      pair_channels(i, rot.rotary_dim, rot.interleaved, ia, ib);
      bf16* dst;
      if (ehead < nq) {
        dst = q + ((size_t)m * nq + ehead) * d;
      } else {
        const int p = row_pos[m];
        const int page = table[(size_t)m * table_stride + (p / PAGE) % ring_pages];
        dst = pages + (size_t)page * page_elems + ((size_t)(ehead - nq) * PAGE + p % PAGE) * d;
      }
      dst[ia] = (bf16)ra;
      dst[ib] = (bf16)rb;
    }
  } else {
    const int m = et / 8, nl = et % 8;
    if (m < M) {
      const int p = row_pos[m];
      const int page = table[(size_t)m * table_stride + (p / PAGE) % ring_pages];
      bf16* vd = pages + (size_t)page * page_elems + (size_t)nkv * PAGE * d;
      vd[((size_t)(ehead - nq - nkv) * d + 8 * eh + nl) * PAGE + p % PAGE] = (bf16)total(8 * eu + nl, m);
    }
  }
}

// ------------------------------------------------------------------- mid ----
// 17..128 rows (decode at larger batches, short prompts).  Per byte of W there are now enough
// MFMAs that the activations must be shared: a workgroup owns 64 output
// channels (one 16-channel tile per wave) and a slice of K; the activations of
// a k-step go through LDS once for the four waves, W streams from global
// memory into registers.  With n_split > 1 the slices of K go to different
// workgroups, which write partial sums P[split][M][N]; the kernel that reads
// them next adds them up (always in the order of the splits).
template <int MT, int KS, bool FULLK>   // KS: k per step (a multiple of 64), everything of a step is in flight at once;
__global__ void __launch_bounds__(256)  // FULLK: K % KS == 0, no load needs a guard (and a branch)
gemm_mid_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M,
                int N, int K, int steps_per_split, int epilogue) {
  constexpr int ROWS = MT * 16, LD = KS + 8, SUB = KS / 64;
  __shared__ __attribute__((aligned(16))) bf16 As[ROWS * LD];
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, li = lane % 16, kg = lane / 16;
  const int n0 = blockIdx.x * 64 + wave * 16;
  const bf16* wrow = W + (size_t)min(n0 + li, N - 1) * K;
  const int steps = (K + KS - 1) / KS;
  const int s_begin = blockIdx.y * steps_per_split, s_end = min(steps, s_begin + steps_per_split);

  // activations: ROWS x KS/8 chunks of 8 per step, shared out over the 256 threads
  constexpr int CPR = KS / 8, CHUNKS = ROWS * CPR, PER = (CHUNKS + 255) / 256;
  bf16x8 areg[PER];
  auto fetch_a = [&](int s) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c = tid + 256 * i;
      const int row = c / CPR, k = s * KS + (c % CPR) * 8;
      areg[i] = (c < CHUNKS && (FULLK || k + 8 <= K)) ? load8(A + (size_t)min(row, M - 1) * K + k) : zero8();
    }
  };
  auto stash_a = [&]() {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int c = tid + 256 * i;
      if (c < CHUNKS) *reinterpret_cast<bf16x8*>(&As[(c / CPR) * LD + (c % CPR) * 8]) = areg[i];
    }
  };
  bf16x8 wreg[SUB][2], wnext[SUB][2];
  auto fetch_w = [&](int s, bf16x8 (&w)[SUB][2]) {
#pragma unroll
    for (int j = 0; j < SUB; ++j) {
      const int k = s * KS + j * 64 + kg * 16;
      w[j][0] = (FULLK || k + 8 <= K) ? load8(wrow + k) : zero8();
      w[j][1] = (FULLK || k + 16 <= K) ? load8(wrow + k + 8) : zero8();
    }
  };

  f32x4 acc[MT];
#pragma unroll
  for (int u = 0; u < MT; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};

  if (s_begin < s_end) {
    fetch_a(s_begin);
    fetch_w(s_begin, wreg);
  }
  for (int s = s_begin; s < s_end; ++s) {
    __syncthreads();                 // the previous step's activations have been read
    stash_a();
    __syncthreads();
    if (s + 1 < s_end) {
      fetch_a(s + 1);
      fetch_w(s + 1, wnext);
    }
#pragma unroll
    for (int j = 0; j < SUB; ++j)
#pragma unroll
      for (int u = 0; u < MT; ++u) {
        const bf16* ar = &As[(u * 16 + li) * LD + j * 64 + kg * 16];
        const bf16x8 a0 = *reinterpret_cast<const bf16x8*>(ar), a1 = *reinterpret_cast<const bf16x8*>(ar + 8);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, wreg[j][0], acc[u], 0, 0, 0);
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, wreg[j][1], acc[u], 0, 0, 0);
      }
#pragma unroll
    for (int j = 0; j < SUB; ++j) {
      wreg[j][0] = wnext[j][0];
      wreg[j][1] = wnext[j][1];
    }
  }
  // acc[u][r] = D[m = 16 u + 4 kg + r][n = n0 + li]
  if (epilogue == EPI_SILU_PAIR) {
    // the workgroup's 64 rows are one group: waves 0,1 hold gate rows, waves 2,3 their up rows
    __syncthreads();
    float* ex = reinterpret_cast<float*>(&As[0]);           // [2 waves][MT][4][64] floats: 2 KB a row tile
    if (wave >= 2) {
#pragma unroll
      for (int u = 0; u < MT; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) ex[(((wave - 2) * MT + u) * 4 + r) * 64 + lane] = acc[u][r];
    }
    __syncthreads();
    if (wave < 2) {
      bf16* H = reinterpret_cast<bf16*>(C);
      const int NH = N / 2;
      const int n = blockIdx.x * 32 + wave * 16 + li;
#pragma unroll
      for (int u = 0; u < MT; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = 16 * u + 4 * kg + r;
          if (m < M && n < NH) {
            const float g = acc[u][r], up = ex[((wave * MT + u) * 4 + r) * 64 + lane];
            H[(size_t)m * NH + n] = (bf16)((g / (1.0f + expf(-g))) * up);
          }
        }
    }
    return;
  }
  float* dst = C + (size_t)blockIdx.y * M * N;              // the split's own partial (split 0: C itself)
  const int n = n0 + li;
  if (n < N) {
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = 16 * u + 4 * kg + r;
        if (m < M) {
          float* c = dst + (size_t)m * N + n;
          *c = (epilogue == EPI_ACCUMULATE) ? *c + acc[u][r] : acc[u][r];
        }
      }
  }
}

constexpr int MID_KS = 256;       // k per step up to 64 rows; half of it above, where the rows in LDS are twice as many
constexpr int MID_ROWS = 128;

template <int MT>
static int launch_mid(const bf16* A, const bf16* W, float* C, int M, int N, int K, int n_split, int epilogue,
                      hipStream_t st) {
  constexpr int KS = MT > 4 ? MID_KS / 2 : MID_KS;
  const int steps = (K + KS - 1) / KS, per = (steps + n_split - 1) / n_split;
  dim3 grid((N + 63) / 64, n_split);
  if (K % KS == 0)
    gemm_mid_kernel<MT, KS, true><<<grid, 256, 0, st>>>(A, W, C, M, N, K, per, epilogue);
  else
    gemm_mid_kernel<MT, KS, false><<<grid, 256, 0, st>>>(A, W, C, M, N, K, per, epilogue);
  TL_LAUNCH_CHECK("gemm_mid");
  return 0;
}

// ------------------------------------------------------------------ ring ----
// 17..128 rows when K is a multiple of 128: the same product as gemm_mid, with both operands going
// from memory straight into a ring of stages in LDS (global_load_lds, 16 bytes a lane, no register in
// between), several stages ahead of the matrix cores.  A stage is KC k (64 or 128): KC * 2 bytes of each
// of the workgroup's channels (16 a wave) and of each row of activations.  A load instruction takes
// whole runs of that length from four or eight rows (1 KB, which lands in LDS lane after lane); within a
// row the 16-byte chunk c lies at a swizzled place, so that the operand reads of 16 lanes fall on 16
// different groups of banks.  The compiler places no waits for such loads: the waves count them (vmcnt)
// and meet at one barrier a stage.  The weights' loads are marked non-temporal (whole lines, read once).
constexpr int RING_LDS = 156 * 1024;         // most LDS a workgroup takes
constexpr int RING_W_AUX = 2;                // cache policy of the weights' loads: non-temporal

template <int N> __device__ __forceinline__ void wait_loads_but() {       // until at most N loads are under way
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

#define TL_AS1 __attribute__((address_space(1)))
#define TL_AS3 __attribute__((address_space(3)))

template <int MT, int WAVES, int KC, int NS>
__global__ void __launch_bounds__(WAVES * 64)
gemm_ring_kernel(const bf16* __restrict__ A, const bf16* __restrict__ W, float* __restrict__ C, int M, int N,
                 int K, int stages_per_split, int epilogue) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char ring_smem[];
  constexpr int ROWB = KC * 2;                              // bytes of a row in a stage
  constexpr int RPI = 1024 / ROWB;                          // rows a load instruction takes
  constexpr int CPR = ROWB / 16;                            // 16-byte chunks of a row
  constexpr int W_INSTR = 16 / RPI;                         // loads of a wave's 16 channels
  constexpr int A_BYTES = MT * 16 * ROWB, W_BYTES = WAVES * 16 * ROWB, STAGE = A_BYTES + W_BYTES;
  constexpr int A_INSTR = MT * 16 / RPI;                    // loads of a stage's activations
  constexpr int A_PER = (A_INSTR + WAVES - 1) / WAVES;      // a wave's share of them
  constexpr int LPS = W_INSTR + A_PER;                      // loads a wave issues for a stage
  constexpr int SPARE = NS * STAGE;                         // 1 KB that takes the loads of shares that do not exist
  constexpr int STEPS = KC / 32;                            // matrix-core steps of a stage
  static_assert(KC == 64 || KC == 128, "a stage is 64 or 128 k");
  static_assert((NS - 2) * LPS <= 63 && NS >= 2, "the count of loads under way has six bits");
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, li = lane % 16, kg = lane / 16;
  const int n0 = blockIdx.x * (WAVES * 16) + wave * 16;
  const int stages = K / KC;
  const int t_begin = blockIdx.y * stages_per_split;
  const int n_t = min(stages, t_begin + stages_per_split) - t_begin;
  // chunk c of row r lies at place c ^ key(r) of the row: 16 lanes that read the same chunk of 16 rows
  // then fall on 16 groups of banks (rows of 128 bytes lie two to a line of banks)
  auto key = [](int r) { return CPR == 16 ? r % 16 : (r / 2) % 8; };

  // this lane's sources: of load i of the weights (row RPI i + lane / CPR of the wave's 16) and of its
  // shares of the activations
  const int sub = lane / CPR, place = lane % CPR;
  const char* wsrc[W_INSTR];
#pragma unroll
  for (int i = 0; i < W_INSTR; ++i) {
    const int r = RPI * i + sub;
    wsrc[i] = reinterpret_cast<const char*>(W + (size_t)min(n0 + r, N - 1) * K) + (size_t)t_begin * ROWB +
              ((place ^ key(r)) * 16);
  }
  const char* asrc[A_PER];
  int adst[A_PER];
#pragma unroll
  for (int x = 0; x < A_PER; ++x) {
    const int q = wave + WAVES * x, r = RPI * q + sub;
    asrc[x] = reinterpret_cast<const char*>(A + (size_t)min(r, M - 1) * K) + (size_t)t_begin * ROWB +
              ((place ^ key(r)) * 16);
    adst[x] = q < A_INSTR ? q * 1024 : -1;
  }
  auto issue = [&](int i) {                                 // stage i of this split into its place in the ring
    unsigned char* slot = ring_smem + (i % NS) * STAGE;
    const size_t off = (size_t)i * ROWB;
#pragma unroll
    for (int x = 0; x < A_PER; ++x) {
      unsigned char* dst = adst[x] >= 0 ? slot + adst[x] : ring_smem + SPARE;
      __builtin_amdgcn_global_load_lds((const TL_AS1 void*)(asrc[x] + off), (TL_AS3 void*)dst, 16, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < W_INSTR; ++j)
      __builtin_amdgcn_global_load_lds((const TL_AS1 void*)(wsrc[j] + off),
                                       (TL_AS3 void*)(slot + A_BYTES + wave * (16 * ROWB) + j * 1024), 16, 0,
                                       RING_W_AUX);
  };

  f32x4 acc[MT];
#pragma unroll
  for (int u = 0; u < MT; ++u) acc[u] = f32x4{0.f, 0.f, 0.f, 0.f};

#pragma unroll
  for (int i = 0; i < NS - 1; ++i)
    if (i < n_t) issue(i);
  const int kl = key(li);
  for (int i = 0; i < n_t; ++i) {
    // stage i has arrived for this wave when only the stages behind it are under way
    if (n_t - 1 - i >= NS - 2) wait_loads_but<(NS - 2) * LPS>();
    else wait_loads_but<0>();
    __builtin_amdgcn_s_barrier();                           // ... and for all; everyone has left stage i - 1
    if (i + NS - 1 < n_t) issue(i + NS - 1);                // into the place of stage i - 1
    const unsigned char* slot = ring_smem + (i % NS) * STAGE;
    const unsigned char* wrow = slot + A_BYTES + wave * (16 * ROWB) + li * ROWB;
    // all operands of the stage are asked for before the first product: a wave is alone on its SIMD, and
    // nothing else hides the way from LDS
    bf16x8 wreg[STEPS], areg[MT][STEPS];
#pragma unroll
    for (int j = 0; j < STEPS; ++j) wreg[j] = *reinterpret_cast<const bf16x8*>(wrow + (((4 * j + kg) ^ kl) * 16));
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int j = 0; j < STEPS; ++j)
        areg[u][j] = *reinterpret_cast<const bf16x8*>(slot + (u * 16 + li) * ROWB + (((4 * j + kg) ^ kl) * 16));
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int j = 0; j < STEPS; ++j)
        acc[u] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(areg[u][j], wreg[j], acc[u], 0, 0, 0);
  }
  // acc[u][r] = D[m = 16 u + 4 kg + r][n = n0 + li]
  if (epilogue == EPI_SILU_PAIR) {
    // the workgroup's channels are groups of 64: of a group's four waves, the first two hold gate
    // rows, the other two their up rows
    __builtin_amdgcn_s_barrier();                           // the ring is free
    float* ex = reinterpret_cast<float*>(ring_smem);        // [up wave][MT][4][64] floats
    const int grp = wave / 4, wq = wave % 4;
    if (wq >= 2) {
#pragma unroll
      for (int u = 0; u < MT; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) ex[(((grp * 2 + wq - 2) * MT + u) * 4 + r) * 64 + lane] = acc[u][r];
    }
    __syncthreads();
    if (wq < 2) {
      bf16* H = reinterpret_cast<bf16*>(C);
      const int NH = N / 2;
      const int n = (blockIdx.x * (WAVES / 4) + grp) * 32 + wq * 16 + li;
#pragma unroll
      for (int u = 0; u < MT; ++u)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int m = 16 * u + 4 * kg + r;
          if (m < M && n < NH) {
            const float g = acc[u][r], up = ex[(((grp * 2 + wq) * MT + u) * 4 + r) * 64 + lane];
            H[(size_t)m * NH + n] = (bf16)((g / (1.0f + expf(-g))) * up);
          }
        }
    }
    return;
  }
  float* dst = C + (size_t)blockIdx.y * M * N;              // the split's own partial (split 0: C itself)
  const int n = n0 + li;
  if (n < N) {
#pragma unroll
    for (int u = 0; u < MT; ++u)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = 16 * u + 4 * kg + r;
        if (m < M) {
          float* c = dst + (size_t)m * N + n;
          *c = (epilogue == EPI_ACCUMULATE) ? *c + acc[u][r] : acc[u][r];
        }
      }
  }
}

template <int MT, int WAVES, int KC>
static int launch_ring(const bf16* A, const bf16* W, float* C, int M, int N, int K, int n_split, int epilogue,
                       hipStream_t st) {
  constexpr int STAGE = (MT + WAVES) * 16 * KC * 2;
  constexpr int FIT = (RING_LDS - 1024) / STAGE;
  constexpr int NS = FIT > 8 ? 8 : FIT;
  static_assert(NS >= 2, "two stages at least");
  constexpr int LDS = NS * STAGE + 1024;
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&gemm_ring_kernel<MT, WAVES, KC, NS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
    if (e != hipSuccess) {
      set_error("gemm_ring: cannot have %d bytes of LDS: %s", LDS, hipGetErrorString(e));
      return 2;
    }
    raised = true;
  }
  const int stages = K / KC, per = (stages + n_split - 1) / n_split;
  dim3 grid((N + WAVES * 16 - 1) / (WAVES * 16), n_split);
  gemm_ring_kernel<MT, WAVES, KC, NS><<<grid, WAVES * 64, LDS, st>>>(A, W, C, M, N, K, per, epilogue);
  TL_LAUNCH_CHECK("gemm_ring");
  return 0;
}

template <int WAVES, int KC>
static int launch_ring_rows(const bf16* A, const bf16* W, float* C, int M, int N, int K, int n_split, int epilogue,
                            hipStream_t st) {
  if (M <= 32) return launch_ring<2, WAVES, KC>(A, W, C, M, N, K, n_split, epilogue, st);
  if (M <= 64) return launch_ring<4, WAVES, KC>(A, W, C, M, N, K, n_split, epilogue, st);
  if (M <= 96) return launch_ring<6, WAVES, KC>(A, W, C, M, N, K, n_split, epilogue, st);
  return launch_ring<8, WAVES, KC>(A, W, C, M, N, K, n_split, epilogue, st);
}

}  // namespace tl

using namespace tl;

// epilogue: 0 store float, 1 accumulate into float, 2 silu(gate) * up into bfloat16 [M, N/2]
// (W's rows in groups of 64: 32 gate rows and their 32 up rows; N a multiple of 64).
// Wt (or null): the tiled copy of W with tiles of wt_height rows, see tl_gemm_bf16_norm.
extern "C" int tl_gemm_bf16(const void* A, const void* W, const void* Wt, int wt_height, void* C, int M, int N, int K,
                            int epilogue, hipStream_t st) {
  TL_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(K % 8 == 0, "gemm_bf16: K=%d must be a multiple of 8", K);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0) && ((uintptr_t)Wt % 16 == 0),
             "gemm_bf16: operands must be 16-byte aligned");
  TL_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm_bf16: unknown epilogue %d", epilogue);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || N % 64 == 0, "gemm_bf16: the paired epilogue needs N=%d to be "
             "a multiple of 64", N);
  if (M == 0) return 0;
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  float* c = (float*)C;
  const bool wide = N >= 16384 || epilogue == EPI_SILU_PAIR;     // many rows: 64 a workgroup
  if (M <= 16) {
    if (wide && rows_fit(M, N, K)) return launch_rows(a, w, c, M, N, K, epilogue, st);
    if (wide && (M > 4 || epilogue == EPI_SILU_PAIR)) return launch_skinny<4, 1, 4>(a, w, c, M, N, K, epilogue, st);
    return launch_shares(a, w, (const bf16*)Wt, wt_height, c, M, N, K, epilogue, st, NormSplit{}, balanced_share(N));
  }
  if (M <= 32) {
    if (wide) return launch_skinny<4, 2, 4>(a, w, c, M, N, K, epilogue, st);
    return launch_skinny<2, 2, 8>(a, w, c, M, N, K, epilogue, st);
  }
  if (M <= 64) {
    if (wide) return launch_skinny<4, 4, 4>(a, w, c, M, N, K, epilogue, st);
    return launch_skinny<1, 4, 8>(a, w, c, M, N, K, epilogue, st);
  }
  TL_REQUIRE(false, "gemm_bf16: %d rows; this entry point serves at most 64 (tl_gemm_mid_bf16 takes up to 128, "
             "the BLAS library more)", M);
}

// For tests and tuning: force one kernel whatever M is.  variant 2: rows; 1000 + R: the kernel for at
// most 16 rows with R channels a workgroup (1 to 32); else NT*100 + MT*10 + waves/4.
extern "C" int tl_gemm_bf16_variant(const void* A, const void* W, void* C, int M, int N, int K,
                                    int epilogue, int variant, hipStream_t st) {
  TL_REQUIRE(M > 0 && N > 0 && K > 0 && K % 8 == 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || N % 64 == 0, "gemm_bf16: the paired epilogue needs N=%d to be "
             "a multiple of 64", N);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  float* c = (float*)C;
  if (variant == 2) {
    TL_REQUIRE(rows_fit(M, N, K), "gemm_rows: M=%d N=%d K=%d (at most 16 rows, N a multiple of 64, K of %d)", M, N,
               K, ROWS_CHUNK);
    return launch_rows(a, w, c, M, N, K, epilogue, st);
  }
  if (variant > 1000 && variant <= 1032) {
    TL_REQUIRE(M <= 16 && epilogue != EPI_SILU_PAIR, "gemm_skinny: variant %d takes at most 16 rows and no pairs", variant);
    const int R = variant - 1000;
    if (R <= 16) return launch_skinny<1, 1, 8>(a, w, c, M, N, K, epilogue, st, NormSplit{}, nullptr, R);
    return launch_skinny<2, 1, 8>(a, w, c, M, N, K, epilogue, st, NormSplit{}, nullptr, R);
  }
  const int mt = (variant / 10) % 10;
  TL_REQUIRE(M <= 16 * mt, "gemm_skinny: variant %d takes at most %d rows, not %d", variant, 16 * mt, M);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || variant / 100 == 4, "gemm_skinny: the paired epilogue needs 64 rows "
             "a workgroup (variant 4xx)");
  switch (variant) {
    case 112: return launch_skinny<1, 1, 8>(a, w, c, M, N, K, epilogue, st);
    case 111: return launch_skinny<1, 1, 4>(a, w, c, M, N, K, epilogue, st);
    case 212: return launch_skinny<2, 1, 8>(a, w, c, M, N, K, epilogue, st);
    case 411: return launch_skinny<4, 1, 4>(a, w, c, M, N, K, epilogue, st);
    case 222: return launch_skinny<2, 2, 8>(a, w, c, M, N, K, epilogue, st);
    case 421: return launch_skinny<4, 2, 4>(a, w, c, M, N, K, epilogue, st);
    case 242: return launch_skinny<2, 4, 8>(a, w, c, M, N, K, epilogue, st);
    case 441: return launch_skinny<4, 4, 4>(a, w, c, M, N, K, epilogue, st);
    case 142: return launch_skinny<1, 4, 8>(a, w, c, M, N, K, epilogue, st);
  }
  TL_REQUIRE(false, "gemm_bf16: unknown variant %d", variant);
}

extern "C" int tl_gemm_ring_bf16(const void* A, const void* W, void* C, int M, int N, int K, int n_split,
                                 int epilogue, int waves, int kc, hipStream_t st);

// 17..128 rows.  n_split == 1: C as in tl_gemm_bf16 (all three epilogues).  n_split > 1: C is
// float [n_split][M][N] and receives partial sums (epilogue must be 0).  K a multiple of 128: the
// ring kernel, 8 waves (128 channels) a workgroup, stages of 128 k, every split with one stage at
// least; other K: gemm_mid, every split with one k-step of 256 at least.
extern "C" int tl_gemm_mid_bf16(const void* A, const void* W, void* C, int M, int N, int K, int n_split,
                                int epilogue, hipStream_t st) {
  if (K > 0 && K % 128 == 0) return tl_gemm_ring_bf16(A, W, C, M, N, K, n_split, epilogue, 8, 128, st);
  TL_REQUIRE(M > 0 && M <= MID_ROWS && N > 0 && K > 0 && K % 8 == 0, "gemm_mid: bad sizes M=%d N=%d K=%d (M at most "
             "%d, K a multiple of 8)", M, N, K, MID_ROWS);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_mid: operands must be 16-byte aligned");
  TL_REQUIRE(n_split >= 1 && n_split <= (K + MID_KS - 1) / MID_KS && n_split <= 65535,
             "gemm_mid: %d splits do not fit K=%d (one step of %d at least each)", n_split, K, MID_KS);
  TL_REQUIRE(epilogue >= 0 && epilogue <= 2 && (n_split == 1 || epilogue == EPI_STORE),
             "gemm_mid: epilogue %d cannot go with %d splits", epilogue, n_split);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || N % 64 == 0, "gemm_mid: the paired epilogue needs N=%d to be a "
             "multiple of 64", N);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  float* c = (float*)C;
  if (M <= 16) return launch_mid<1>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 32) return launch_mid<2>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 48) return launch_mid<3>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 64) return launch_mid<4>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 80) return launch_mid<5>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 96) return launch_mid<6>(a, w, c, M, N, K, n_split, epilogue, st);
  if (M <= 112) return launch_mid<7>(a, w, c, M, N, K, n_split, epilogue, st);
  return launch_mid<8>(a, w, c, M, N, K, n_split, epilogue, st);
}

// The same product through the ring kernel (see gemm_ring_kernel): K a multiple of 128.  waves: the waves of a
// workgroup, each with 16 channels: 4, 7 or 8 (the paired epilogue needs whole groups of 64 channels: 4 or 8);
// kc: the k of a stage, 64 or 128.
extern "C" int tl_gemm_ring_bf16(const void* A, const void* W, void* C, int M, int N, int K, int n_split,
                                 int epilogue, int waves, int kc, hipStream_t st) {
  TL_REQUIRE(M > 0 && M <= MID_ROWS && N > 0 && K > 0 && K % 128 == 0, "gemm_ring: bad sizes M=%d N=%d K=%d (M at "
             "most %d, K a multiple of 128)", M, N, K, MID_ROWS);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_ring: operands must be 16-byte aligned");
  TL_REQUIRE(kc == 64 || kc == 128, "gemm_ring: a stage of %d k (64 or 128)", kc);
  TL_REQUIRE(n_split >= 1 && n_split <= K / kc && n_split <= 65535,
             "gemm_ring: %d splits do not fit K=%d (one stage of %d at least each)", n_split, K, kc);
  TL_REQUIRE(epilogue >= 0 && epilogue <= 2 && (n_split == 1 || epilogue == EPI_STORE),
             "gemm_ring: epilogue %d cannot go with %d splits", epilogue, n_split);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || (N % 64 == 0 && waves % 4 == 0), "gemm_ring: the paired epilogue needs N=%d "
             "to be a multiple of 64 and whole groups of four waves (%d)", N, waves);
  const bf16* a = (const bf16*)A;
  const bf16* w = (const bf16*)W;
  float* c = (float*)C;
#define TL_RING(WV)                                                                                     \
  if (waves == WV)                                                                                      \
    return kc == 64 ? launch_ring_rows<WV, 64>(a, w, c, M, N, K, n_split, epilogue, st)                 \
                    : launch_ring_rows<WV, 128>(a, w, c, M, N, K, n_split, epilogue, st)
  TL_RING(4);
  TL_RING(7);
  TL_RING(8);
#undef TL_RING
  TL_REQUIRE(false, "gemm_ring: %d waves a workgroup (4, 7 or 8)", waves);
}

// q|k|v of a step with one token a sequence (row m is sequence m, at position row_pos[m]):
// W is [(nq + 2 nkv) d, K]; q receives [M, nq, d], the pages k and v of the new position.
// With ssq_in, row m's sums are multiplied by rsqrt(sum_j ssq_in[m][j] * inv_h + eps) first.
// units: the units of 8 weight rows (see the kernel) a workgroup owns, 1 to 4; 0 lets the
// launcher deal them in equal shares to the device's compute units.
// Wt (or null): the tiled copy of W with the rows of `tl_qkv_tile_rows`, read instead of W
// when K % 64 == 0.
extern "C" int tl_gemm_qkv_rope_commit(const void* A, const void* W, const void* Wt, int M, int K, const int* row_pos,
                                       const float* inv_freq, int rotary_dim, int interleaved,
                                       const int* table, int table_stride,
                                       int ring_pages, int nq, int nkv, int d, void* q, void* pages,
                                       const float* ssq_in, int n_part, float inv_h, float eps,
                                       int units, hipStream_t st) {
  TL_REQUIRE(M >= 0 && M <= 16 && K > 0 && K % 8 == 0, "qkv_rope_commit: bad sizes M=%d K=%d (at most 16 rows, "
             "K a multiple of 8)", M, K);
  TL_REQUIRE(nq > 0 && nkv > 0 && d >= 16 && d % 16 == 0, "qkv_rope_commit: bad heads nq=%d nkv=%d d=%d (head "
             "sizes in steps of 16)", nq, nkv, d);
  TL_REQUIRE(ring_pages > 0 && table_stride > 0, "qkv_rope_commit: bad cache geometry ring_pages=%d "
             "table_stride=%d", ring_pages, table_stride);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "qkv_rope_commit: operands must be 16-byte aligned");
  TL_REQUIRE(ssq_in == nullptr || n_part > 0, "qkv_rope_commit: %d partial sums of squares", n_part);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0 && (rotary_dim == 0 || inv_freq != nullptr),
             "qkv_rope_commit: %d rotated channels of a head of %d (even, at most the head, with their "
             "frequencies)", rotary_dim, d);
  TL_REQUIRE(units >= 0 && units <= 4, "qkv_rope_commit: %d units a workgroup (1 to 4, or 0 for the launcher's choice)", units);
  const Rotation rot{inv_freq, rotary_dim, interleaved != 0};
  if (M == 0) return 0;
  const long long n_units = (long long)(nq + 2 * nkv) * (d / 8);
  if (units == 0) {
    // a whole number of rounds of workgroups over the compute units, of at most 4 units each
    const int cus = compute_units();
    const long long wgs = ((n_units + 4LL * cus - 1) / (4LL * cus)) * cus;
    units = (int)((n_units + wgs - 1) / wgs);
  }
  const int grid = (int)((n_units + units - 1) / units);
  NormSplit ns{};
  ns.ssq_in = ssq_in; ns.n_part = n_part; ns.inv_h = inv_h; ns.eps = eps;
  const bool tiled = Wt != nullptr && K % 64 == 0;
  TL_REQUIRE(!tiled || (uintptr_t)Wt % 16 == 0, "qkv_rope_commit: operands must be 16-byte aligned");
  const bf16* w = tiled ? (const bf16*)Wt : (const bf16*)W;
#define TL_QKV(TILED, NT)                                                                               \
  gemm_qkv_rope_commit_kernel<TILED, NT><<<grid, QKV_WAVES * 64, 0, st>>>(                              \
      (const bf16*)A, w, M, K, row_pos, rot, table, table_stride, ring_pages, nq, nkv, d, (bf16*)q, \
      (bf16*)pages, ns, units)
  if (units <= 2) {
    if (tiled) TL_QKV(true, 1); else TL_QKV(false, 1);
  } else {
    if (tiled) TL_QKV(true, 2); else TL_QKV(false, 2);
  }
#undef TL_QKV
  TL_LAUNCH_CHECK("gemm_qkv_rope_commit");
  return 0;
}

// The product for at most 16 rows with an RMSNorm cut in two around it (see NormSplit).
// ssq_in [16][n_part] (or null): a factor per row on the results.  norm_w [N], xt [M][N],
// ssq_out [16][workgroups] (or all null): with the accumulate epilogue, also write
// xt = bfloat16(C * norm_w) and the workgroups' sums of C^2; *n_groups receives the number
// of workgroups, which is the n_part of the product that reads xt.  Wt (or null): the tiled
// copy of W (rows in their own order, tiles of wt_height = tl_tile_height(N) rows), read instead of W
// by the kernel with 16 to 32 channels a workgroup when N % 16 == 0 and K % 64 == 0; a copy with tiles
// of another height is refused.
extern "C" int tl_gemm_bf16_norm(const void* A, const void* W, const void* Wt, int wt_height, void* C, int M, int N, int K,
                                 int epilogue,
                                 const float* ssq_in, int n_part, float inv_h, float eps,
                                 const float* norm_w, void* xt, float* ssq_out, int ssq_capacity,
                                 int* n_groups, hipStream_t st) {
  TL_REQUIRE(M >= 0 && M <= 16 && N > 0 && K > 0 && K % 8 == 0, "gemm_bf16_norm: bad sizes M=%d N=%d K=%d (at most "
             "16 rows, K a multiple of 8)", M, N, K);
  TL_REQUIRE(((uintptr_t)A % 16 == 0) && ((uintptr_t)W % 16 == 0), "gemm_bf16_norm: operands must be 16-byte aligned");
  TL_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm_bf16_norm: unknown epilogue %d", epilogue);
  TL_REQUIRE(epilogue != EPI_SILU_PAIR || N % 64 == 0, "gemm_bf16_norm: the paired epilogue needs N=%d to be "
             "a multiple of 64", N);
  TL_REQUIRE(ssq_in == nullptr || n_part > 0, "gemm_bf16_norm: %d partial sums of squares", n_part);
  const bool writer = norm_w != nullptr;
  TL_REQUIRE(!writer || (epilogue == EPI_ACCUMULATE && xt != nullptr && ssq_out != nullptr),
             "gemm_bf16_norm: the next norm's half goes with the accumulate epilogue, xt and ssq_out");
  const bool wide = N >= 16384 || epilogue == EPI_SILU_PAIR;
  const bool rows = wide && !writer && rows_fit(M, N, K);        // many channels, K in chunks of 512: whole rows, 1 KB a load
  const bool four = wide && (M > 4 || epilogue == EPI_SILU_PAIR);
  const int share = four ? 64 : balanced_share(N);
  const int groups = (N + share - 1) / share;
  if (n_groups) *n_groups = groups;
  TL_REQUIRE(!writer || ssq_capacity >= groups * 16, "gemm_bf16_norm: ssq_out holds %d floats, %d are needed",
             ssq_capacity, groups * 16);
  if (M == 0) return 0;
  NormSplit ns{};
  ns.ssq_in = ssq_in; ns.n_part = n_part; ns.inv_h = inv_h; ns.eps = eps;
  ns.norm_w = norm_w; ns.xt = (bf16*)xt; ns.ssq_out = ssq_out;
  if (rows) return launch_rows((const bf16*)A, (const bf16*)W, (float*)C, M, N, K, epilogue, st, ns);
  if (four) return launch_skinny<4, 1, 4>((const bf16*)A, (const bf16*)W, (float*)C, M, N, K, epilogue, st, ns);
  TL_REQUIRE((uintptr_t)Wt % 16 == 0, "gemm_bf16_norm: operands must be 16-byte aligned");
  return launch_shares((const bf16*)A, (const bf16*)W, (const bf16*)Wt, wt_height, (float*)C, M, N, K, epilogue, st, ns,
                       share);
}

// The rows of a tile of the copy that the products for at most 16 rows read of a weight with N rows: the
// share of channels of a workgroup, 16 at least.
extern "C" int tl_tile_height(int N) { return tile_height(balanced_share(N)); }

// Wt [ceil(N / height)][K/64][2][4][height][8] = the tiled copy of W [N, K] (N % 16 == 0, K % 64 == 0)
// with its rows taken in the order `rows` [N] (null: as they are).  height: 16 for the kernel that
// has its own order of rows (tl_gemm_qkv_rope_commit), tl_tile_height(N) for the others.
extern "C" int tl_tile_weights(const void* W, const int* rows, int N, int K, int height, void* Wt, hipStream_t st) {
  TL_REQUIRE(N > 0 && K > 0 && tiles_fit(N, K), "tile_weights: N=%d must be a multiple of 16 and K=%d of 64", N, K);
  TL_REQUIRE(height >= 16 && height <= 32, "tile_weights: tiles of %d rows (16 to 32)", height);
  TL_REQUIRE(((uintptr_t)W % 16 == 0) && ((uintptr_t)Wt % 16 == 0), "tile_weights: operands must be 16-byte aligned");
  const size_t chunks = (size_t)N * K / 8;
  const int grid = (chunks + 255) / 256 < 8192 ? (int)((chunks + 255) / 256) : 8192;
  tile_weights_kernel<<<grid, 256, 0, st>>>((const bf16*)W, rows, N, K, height, (bf16*)Wt);
  TL_LAUNCH_CHECK("tile_weights");
  return 0;
}

// The order of W's rows in the tiled copy that tl_gemm_qkv_rope_commit reads: tile t of a q or
// k head holds the first channels of pairs 8t..8t+7 and then their second channels (with all of a
// head rotated in halves: 8t..8t+7 and d/2+8t..d/2+8t+7), v heads keep theirs.
// rows: [(nq + 2 nkv) d], host.
extern "C" int tl_qkv_tile_rows(int nq, int nkv, int d, int rotary_dim, int interleaved, int* rows) {
  TL_REQUIRE(nq > 0 && nkv > 0 && d >= 16 && d % 16 == 0, "qkv_tile_rows: bad heads nq=%d nkv=%d d=%d", nq, nkv, d);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0,
             "qkv_tile_rows: %d rotated channels of a head of %d (even, at most the head)", rotary_dim, d);
  for (int head = 0; head < nq + 2 * nkv; ++head)
    for (int t = 0; t < d / 16; ++t)
      for (int r = 0; r < 16; ++r) {
        int ch = 16 * t + r;
        if (head < nq + nkv) {
          int ca, cb;
          pair_channels(8 * t + r % 8, rotary_dim, interleaved != 0, ca, cb);
          ch = r < 8 ? ca : cb;
        }
        rows[(head * (d / 16) + t) * 16 + r] = head * d + ch;
      }
  return 0;
}
