// Shared helpers of the gfx950 kernels: element types, loads that widen to
// float, wave and block reductions, and the error channel of the C interface.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "page.h"

namespace tl {

typedef __bf16 bf16;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;

constexpr int WAVE = 64;
constexpr int PAGE = TL_PAGE;     // positions per cache page
static_assert(PAGE == 64, "the attention kernels tile a page by 64 positions");

// dtype codes of the C interface
constexpr int DT_F32 = 0;
constexpr int DT_BF16 = 1;

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }  // nearest even

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, WAVE));
  return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every
// thread gets the result.  `sh` holds at least NT/64 floats.
template <int NT> __device__ __forceinline__ float block_sum(float v, float* sh) {
  v = wave_sum(v);
  const int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) sh[w] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int i = 0; i < NT / WAVE; ++i) r += sh[i];
  return r;
}
template <int NT> __device__ __forceinline__ float block_max(float v, float* sh) {
  v = wave_max(v);
  const int w = threadIdx.x / WAVE, l = threadIdx.x % WAVE;
  __syncthreads();
  if (l == 0) sh[w] = v;
  __syncthreads();
  float r = sh[0];
#pragma unroll
  for (int i = 1; i < NT / WAVE; ++i) r = fmaxf(r, sh[i]);
  return r;
}

// Rotation of a pair by (c, s), each product and the sum rounded on its own (no fused
// multiply-add), so that every kernel that rotates gives the same bits:
// a' = a c - b s ; b' = a s + b c   (src/kernels/mod.rs:603-605 of the reference)
__device__ __forceinline__ void rotate_pair(float a, float b, float c, float s, float& ra, float& rb) {
#pragma clang fp contract(off)
  const float ac = a * c, bs = b * s, as = a * s, bc = b * c;
  ra = ac - bs;
  rb = as + bc;
}

// How q and k are rotated by position: the first `rotary_dim` channels of a head (even, at most
// the head size; 0: no rotation at all) in pairs, pair i by the angle pos * inv_freq[i]; the
// channels behind them are passed through.
struct Rotation {
  const float* inv_freq;   // [rotary_dim / 2]
  int rotary_dim;
  int interleaved;         // pairs (2i, 2i+1); else (i, i + rotary_dim/2)
};
// The two channels of pair i of a head, i < d/2.  Pairs from rotary_dim/2 on are not rotated;
// they are numbered so that the d/2 pairs cover every channel once.
__host__ __device__ __forceinline__ void pair_channels(int i, int rotary_dim, int interleaved, int& a, int& b) {
  if (interleaved || 2 * i >= rotary_dim) {
    a = 2 * i;
    b = 2 * i + 1;
  } else {
    a = i;
    b = i + rotary_dim / 2;
  }
}

// ---- error channel -------------------------------------------------------
void set_error(const char* fmt, ...);

#define TL_REQUIRE(cond, ...)            \
  do {                                   \
    if (!(cond)) {                       \
      tl::set_error(__VA_ARGS__);        \
      return 1;                          \
    }                                    \
  } while (0)

#define TL_LAUNCH_CHECK(name)                                              \
  do {                                                                     \
    hipError_t e_ = hipGetLastError();                                     \
    if (e_ != hipSuccess) {                                                \
      tl::set_error("%s: launch failed: %s", name, hipGetErrorString(e_)); \
      return 2;                                                            \
    }                                                                      \
  } while (0)

}  // namespace tl
