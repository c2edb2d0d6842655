// Attention over the cache and the keys of this step, one wave per (row, head):
// the kernel of the true 32-bit path and the reference that the faster
// kernels are checked against.  It serves any mix of rows: whole prompts, a
// prompt that goes on from cached context, single decoded tokens.
//
// For the query at position p of sequence b, key j is visible iff j <= p and
// (no window or j > p - W)  (src/model/modules/attention.rs:90 and
// src/model/models/gpt_oss.rs:168-175 of the reference).  Keys j < n_cached[b]
// are read from the sequence's pages, later ones from this step's k/v rows.
// score = (k.q) * scale, scale applied after the dot; softmax with running
// maximum over tiles of 64 keys, all in float
// (src/model/modules/attention.rs:82-121, src/kernels/mod.rs:494-543).
#include "common.hpp"

namespace tl {

constexpr int MAX_D = 256;

template <typename T>
__global__ void __launch_bounds__(64)
attn_plain_kernel(const T* __restrict__ q, const T* __restrict__ k_new, const T* __restrict__ v_new,
                  const T* __restrict__ pages, const int* __restrict__ table, int table_stride,
                  int ring_pages, const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                  const int* __restrict__ cu_seqlens, const int* __restrict__ n_cached, int nq,
                  int nkv, int d, int window, float scale, T* __restrict__ out) {
  __shared__ float q_s[MAX_D];
  __shared__ float p_s[WAVE];
  __shared__ const T* v_s[WAVE];
  __shared__ int vstride_s[WAVE];
  const int n = blockIdx.x / nq, h = blockIdx.x % nq;
  const int lane = threadIdx.x;
  const int b = row_seq[n], p = row_pos[n];
  const int kvh = h / (nq / nkv);
  const int cached = n_cached[b];
  const int row0 = cu_seqlens[b];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const size_t head_elems = (size_t)PAGE * d;
  const size_t page_elems = 2 * (size_t)nkv * head_elems;
  const size_t v_off = (size_t)nkv * head_elems;

  const T* qr = q + ((size_t)n * nq + h) * d;
  for (int i = lane; i < d; i += WAVE) q_s[i] = to_f32(qr[i]);
  __syncthreads();

  float m = -INFINITY, l = 0.f;
  float acc[MAX_D / WAVE];
#pragma unroll
  for (int i = 0; i < MAX_D / WAVE; ++i) acc[i] = 0.f;

  for (int j0 = lo; j0 <= p; j0 += WAVE) {
    const int j = j0 + lane;
    float s = -INFINITY;
    const T* vp = nullptr;
    int vstride = 1;                 // values: [d][PAGE] in a page, [d] in the step's rows
    if (j <= p) {
      const T* kp;
      if (j < cached) {
        const int page = table[(size_t)b * table_stride + (j / PAGE) % ring_pages];
        kp = pages + (size_t)page * page_elems + (size_t)kvh * head_elems + (size_t)(j % PAGE) * d;
        vp = pages + (size_t)page * page_elems + v_off + (size_t)kvh * head_elems + (j % PAGE);
        vstride = PAGE;
      } else {
        const size_t r = ((size_t)(row0 + j - cached) * nkv + kvh) * d;
        kp = k_new + r;
        vp = v_new + r;
      }
      float dot = 0.f;
      for (int t = 0; t < d; ++t) dot = fmaf(to_f32(kp[t]), q_s[t], dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));       // finite: key j0 is visible
    const float pj = (j <= p) ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);              // 0 in the first tile (m = -inf)
    l = l * alpha + wave_sum(pj);
    m = m_new;
    __syncthreads();
    p_s[lane] = pj;
    v_s[lane] = vp;
    vstride_s[lane] = vstride;
    __syncthreads();
    const int cnt = (p - j0 + 1 < WAVE) ? p - j0 + 1 : WAVE;
#pragma unroll
    for (int i = 0; i < MAX_D / WAVE; ++i) {
      const int dim = lane + WAVE * i;
      if (dim < d) {
        float a = acc[i] * alpha;
        for (int jj = 0; jj < cnt; ++jj) a = fmaf(p_s[jj], to_f32(v_s[jj][(size_t)dim * vstride_s[jj]]), a);
        acc[i] = a;
      }
    }
  }
  T* o = out + ((size_t)n * nq + h) * d;
#pragma unroll
  for (int i = 0; i < MAX_D / WAVE; ++i) {
    const int dim = lane + WAVE * i;
    if (dim < d) o[dim] = from_f32<T>(acc[i] / l);
  }
}

}  // namespace tl

using namespace tl;

extern "C" int tl_attn_plain(const void* q, const void* k_new, const void* v_new, const void* pages,
                             int dt, const int* table, int table_stride, int ring_pages,
                             const int* row_seq, const int* row_pos, const int* cu_seqlens,
                             const int* n_cached, int n, int nq, int nkv, int d, int window,
                             float scale, void* out, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attention: bad head counts nq=%d nkv=%d",
             nq, nkv);
  TL_REQUIRE(d > 0 && d <= MAX_D, "attention: head size %d is not served (1..%d)", d, MAX_D);
  TL_REQUIRE(ring_pages > 0 && table_stride > 0 && window >= 0,
             "attention: bad cache geometry ring_pages=%d table_stride=%d window=%d", ring_pages,
             table_stride, window);
  TL_REQUIRE((long long)n * nq < 2147483647LL, "attention: too many (row, head) pairs");
  if (n == 0) return 0;
  if (dt == DT_F32)
    attn_plain_kernel<float><<<n * nq, 64, 0, st>>>(
        (const float*)q, (const float*)k_new, (const float*)v_new, (const float*)pages, table,
        table_stride, ring_pages, row_seq, row_pos, cu_seqlens, n_cached, nq, nkv, d, window, scale,
        (float*)out);
  else if (dt == DT_BF16)
    attn_plain_kernel<bf16><<<n * nq, 64, 0, st>>>(
        (const bf16*)q, (const bf16*)k_new, (const bf16*)v_new, (const bf16*)pages, table,
        table_stride, ring_pages, row_seq, row_pos, cu_seqlens, n_cached, nq, nkv, d, window, scale,
        (bf16*)out);
  else
    TL_REQUIRE(false, "attention: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("attn_plain");
  return 0;
}
