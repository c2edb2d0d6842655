// What the machine gives to the simplest possible kernels: a read of a large buffer
// (the ceiling of every step that is bound by reading weights and cache) and a chain of
// independent bfloat16 MFMAs on registers (the ceiling of the products).  bench.py quotes
// both next to the published peaks.  A library of its own (libtorchless_measure.so): nothing
// that a model's step needs is here, and a step's first call does not compile it.
#include "../common.hpp"
#include <stdarg.h>

namespace tl {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// Every thread reads 16-byte vectors, 8 in flight, a grid-stride apart; the sums go to one
// float a workgroup so that nothing is optimised away.
__global__ void __launch_bounds__(256)
stream_read_kernel(const f32x4* __restrict__ src, size_t n_vec, float* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (; i + 7 * stride < n_vec; i += 8 * stride) {
    f32x4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < 8; ++u) acc += v[u];
  }
  for (; i < n_vec; i += stride) acc += src[i];
  __shared__ float sh[4];
  const float s = block_sum<256>(acc[0] + acc[1] + acc[2] + acc[3], sh);
  if (threadIdx.x == 0) sink[blockIdx.x] = s;
}

// The same read in other shapes, to see whether the machine gives more to any of them: U loads
// in flight a lane; SPAN: a workgroup reads one contiguous share of the buffer (U * 4 KB an
// iteration) instead of pieces a grid stride apart; NT: loads marked non-temporal.
template <int U, bool SPAN, bool NT>
__global__ void __launch_bounds__(256)
stream_read_shape_kernel(const f32x4* __restrict__ src, size_t n_vec, float* __restrict__ sink) {
  size_t i, end, step, apart;
  if (SPAN) {
    const size_t share = (n_vec / gridDim.x) / (256 * U) * (256 * U);     // whole iterations; the rest is left unread
    i = (size_t)blockIdx.x * share + threadIdx.x;
    end = (size_t)(blockIdx.x + 1) * share;
    step = (size_t)256 * U;
    apart = 256;
  } else {
    apart = (size_t)gridDim.x * 256;
    i = (size_t)blockIdx.x * 256 + threadIdx.x;
    end = n_vec;
    step = apart * U;
  }
  f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
  for (; i + (U - 1) * apart < end; i += step) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = NT ? __builtin_nontemporal_load(src + i + u * apart) : src[i + u * apart];
#pragma unroll
    for (int u = 0; u < U; ++u) acc += v[u];
  }
  __shared__ float sh[4];
  const float s = block_sum<256>(acc[0] + acc[1] + acc[2] + acc[3], sh);
  if (threadIdx.x == 0) sink[blockIdx.x] = s;
}

// The read with the data going from memory straight into LDS (16 bytes a lane, no register in
// between), U loads a wave under way; nothing reads the LDS but one value at the end.
template <int U>
__global__ void __launch_bounds__(256)
stream_read_lds_kernel(const f32x4* __restrict__ src, size_t n_vec, float* __restrict__ sink) {
  __shared__ __attribute__((aligned(16))) f32x4 buf[4][U][WAVE];
  const int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  const size_t apart = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + (U - 1) * apart < n_vec; i += apart * U) {
#pragma unroll
    for (int u = 0; u < U; ++u)
      __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void*)(src + i + u * apart),
                                       (__attribute__((address_space(3))) void*)&buf[w][u][0], 16, 0, 0);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  const f32x4 v = buf[w][l % U][l];
  if (v[0] == 12345.678f) sink[blockIdx.x] = v[1];      // never true in practice
}

// A copy: as many bytes written as read, a cross-check of the total traffic the memory takes.
template <int U>
__global__ void __launch_bounds__(256)
stream_copy_kernel(const f32x4* __restrict__ src, f32x4* __restrict__ dst, size_t n_vec) {
  const size_t apart = (size_t)gridDim.x * 256;
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + (U - 1) * apart < n_vec; i += apart * U) {
    f32x4 v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = src[i + u * apart];
#pragma unroll
    for (int u = 0; u < U; ++u) dst[i + u * apart] = v[u];
  }
  for (; i < n_vec; i += apart) dst[i] = src[i];
}

// Eight independent accumulators a wave, 32x32x16 bfloat16 MFMAs back to back.
__global__ void __launch_bounds__(256)
mfma_chain_kernel(int iters, float* __restrict__ sink) {
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16)(0.001f * (threadIdx.x % 7 + i));
    b[i] = (bf16)(0.002f * (threadIdx.x % 5 + i));
  }
  f32x16 acc[8];
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 8; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[j][r];
  if (s == 12345.678f) sink[0] = s;          // never true in practice: keeps the chain alive
}

// Do the matrix pipe and the vector pipe of a SIMD work at the same time?  Per iteration a wave issues four
// 32x32x16 MFMAs (independent accumulators), or 32 FMAs and 8 exponentials (the vector work of a softmax), or
// both one after the other.  ROLE 0: every wave the MFMAs only; 1: every wave the vector work only; 2: every
// wave both; 3: the first half of a workgroup's waves the MFMAs, the second half the vector work (waves go
// round the four SIMDs, so with 8 waves every SIMD holds one wave of each kind).
template <int ROLE>
__global__ void __launch_bounds__(512)
pipes_kernel(int iters, float* __restrict__ sink) {
  const int wave = threadIdx.x / 64, n_waves = blockDim.x / 64;
  const bool mfmas = ROLE == 0 || ROLE == 2 || (ROLE == 3 && wave < n_waves / 2);
  const bool vectors = ROLE == 1 || ROLE == 2 || (ROLE == 3 && wave >= n_waves / 2);
  bf16x8 a, b;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    a[i] = (bf16)(0.001f * (threadIdx.x % 7 + i));
    b[i] = (bf16)(0.002f * (threadIdx.x % 5 + i));
  }
  f32x16 acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;
  float v[32];
#pragma unroll
  for (int i = 0; i < 32; ++i) v[i] = 0.001f * (float)(threadIdx.x + i);
  const float c0 = 0.999f, c1 = 1e-4f;
  for (int it = 0; it < iters; ++it) {
    if (mfmas) {
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, acc[j], 0, 0, 0);
    }
    if (vectors) {
#pragma unroll
      for (int i = 0; i < 32; ++i) v[i] = fmaf(v[i], c0, c1);
#pragma unroll
      for (int i = 0; i < 8; ++i) v[i] = __builtin_amdgcn_exp2f(-v[i] * v[i]);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) s += acc[j][r];
#pragma unroll
  for (int i = 0; i < 32; ++i) s += v[i];
  if (s == 12345.678f) sink[0] = s;          // never true in practice: keeps the work alive
}

}  // namespace tl

using namespace tl;

extern "C" {

const char* tl_measure_last_error() { return g_err; }

// reads n_bytes (a multiple of 16) once; sink holds at least `blocks` floats
int tl_stream_read(const void* src, size_t n_bytes, float* sink, int blocks, hipStream_t st) {
  TL_REQUIRE(n_bytes % 16 == 0 && blocks > 0 && ((uintptr_t)src % 16 == 0), "stream_read: %zu bytes in %d blocks",
             n_bytes, blocks);
  stream_read_kernel<<<blocks, 256, 0, st>>>((const f32x4*)src, n_bytes / 16, sink);
  TL_LAUNCH_CHECK("stream_read");
  return 0;
}

// The read in another shape (see the kernels): 1: 16 loads in flight a lane; 2: 32; 3: 8, a contiguous share a
// workgroup; 4: 16, contiguous; 5: 8, non-temporal; 6: 16, non-temporal, contiguous; 7: 8 a wave straight into
// LDS; 8: 16 a wave straight into LDS.  (0 is tl_stream_read's.)  The shapes read whole iterations only: up to
// blocks * 256 * 32 * 16 bytes at the end are left out, which the caller's sizes make negligible.
int tl_stream_read_shape(const void* src, size_t n_bytes, float* sink, int blocks, int shape, hipStream_t st) {
  TL_REQUIRE(n_bytes % 16 == 0 && blocks > 0 && ((uintptr_t)src % 16 == 0), "stream_read: %zu bytes in %d blocks",
             n_bytes, blocks);
  const f32x4* s = (const f32x4*)src;
  const size_t n = n_bytes / 16;
  switch (shape) {
    case 0: stream_read_kernel<<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 1: stream_read_shape_kernel<16, false, false><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 2: stream_read_shape_kernel<32, false, false><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 3: stream_read_shape_kernel<8, true, false><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 4: stream_read_shape_kernel<16, true, false><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 5: stream_read_shape_kernel<8, false, true><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 6: stream_read_shape_kernel<16, true, true><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 7: stream_read_lds_kernel<8><<<blocks, 256, 0, st>>>(s, n, sink); break;
    case 8: stream_read_lds_kernel<16><<<blocks, 256, 0, st>>>(s, n, sink); break;
    default: TL_REQUIRE(false, "stream_read: unknown shape %d", shape);
  }
  TL_LAUNCH_CHECK("stream_read_shape");
  return 0;
}

// copies n_bytes (a multiple of 16) from src to dst, which must not overlap
int tl_stream_copy(const void* src, void* dst, size_t n_bytes, int blocks, hipStream_t st) {
  TL_REQUIRE(n_bytes % 16 == 0 && blocks > 0 && ((uintptr_t)src % 16 == 0) && ((uintptr_t)dst % 16 == 0),
             "stream_copy: %zu bytes in %d blocks", n_bytes, blocks);
  stream_copy_kernel<8><<<blocks, 256, 0, st>>>((const f32x4*)src, (f32x4*)dst, n_bytes / 16);
  TL_LAUNCH_CHECK("stream_copy");
  return 0;
}

// `blocks` workgroups of `waves` waves (4 or 8), `iters` iterations each, in one of the roles of pipes_kernel
int tl_pipes(int role, int waves, int iters, int blocks, float* sink, hipStream_t st) {
  TL_REQUIRE(iters > 0 && blocks > 0 && (waves == 4 || waves == 8) && role >= 0 && role <= 3,
             "pipes: role=%d waves=%d iters=%d blocks=%d", role, waves, iters, blocks);
  switch (role) {
    case 0: pipes_kernel<0><<<blocks, waves * 64, 0, st>>>(iters, sink); break;
    case 1: pipes_kernel<1><<<blocks, waves * 64, 0, st>>>(iters, sink); break;
    case 2: pipes_kernel<2><<<blocks, waves * 64, 0, st>>>(iters, sink); break;
    default: pipes_kernel<3><<<blocks, waves * 64, 0, st>>>(iters, sink); break;
  }
  TL_LAUNCH_CHECK("pipes");
  return 0;
}

// blocks * 4 waves, each iters * 8 MFMAs of 2 * 32 * 32 * 16 flop
int tl_mfma_chain(int iters, int blocks, float* sink, hipStream_t st) {
  TL_REQUIRE(iters > 0 && blocks > 0, "mfma_chain: iters=%d blocks=%d", iters, blocks);
  mfma_chain_kernel<<<blocks, 256, 0, st>>>(iters, sink);
  TL_LAUNCH_CHECK("mfma_chain");
  return 0;
}

}  // extern "C"
