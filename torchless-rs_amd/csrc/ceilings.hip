// What the machine gives to the simplest possible kernels: a read of a large buffer
// (the ceiling of every step that is bound by reading weights and cache) and a chain of
// independent bfloat16 MFMAs on registers (the ceiling of the products).  bench.py quotes
// both next to the published peaks.
#include "common.hpp"

namespace tl {

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

}  // namespace tl

using namespace tl;

extern "C" {

// reads n_bytes (a multiple of 16) once; sink holds at least `blocks` floats
int tl_stream_read(const void* src, size_t n_bytes, float* sink, int blocks, hipStream_t st) {
  TL_REQUIRE(n_bytes % 16 == 0 && blocks > 0 && ((uintptr_t)src % 16 == 0), "stream_read: %zu bytes in %d blocks",
             n_bytes, blocks);
  stream_read_kernel<<<blocks, 256, 0, st>>>((const f32x4*)src, n_bytes / 16, sink);
  TL_LAUNCH_CHECK("stream_read");
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
