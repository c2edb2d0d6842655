// Row-wise kernels: embedding gather, RMSNorm, rotation + split of the fused
// q|k|v projection, commit of keys and values to cache pages, SiLU-gate,
// row gather.  Reductions, angles and the norm are computed in float.
#include "common.hpp"
#include <stdarg.h>

namespace tl {

static thread_local char g_err[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
}

// ---- embedding: out[n, :] = table[ids[n], :] (no scaling) -------------------
// src/model/modules/embedding.rs:15-21 of the reference.
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids, int H,
                             float* __restrict__ out) {
  const int n = blockIdx.x;
  const T* row = table + (size_t)ids[n] * H;
  float* o = out + (size_t)n * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_f32(row[i]);
}

// ---- RMSNorm: y = x / sqrt(mean(x^2) + eps) * w ------------------------------
// src/kernels/mod.rs:558-568 of the reference: eps inside the root, divide,
// then multiply by the weight.
template <typename TO>
__global__ void __launch_bounds__(256) rmsnorm_kernel(const float* __restrict__ x,
                                                      const float* __restrict__ w, float eps,
                                                      TO* __restrict__ out, int H) {
  __shared__ float sh[4];
  const int n = blockIdx.x;
  const float* xr = x + (size_t)n * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float v = xr[i];
    ss += v * v;
  }
  ss = block_sum<256>(ss, sh);
  const float rms = sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)n * H;
  for (int i = threadIdx.x; i < H; i += 256) o[i] = from_f32<TO>((xr[i] / rms) * w[i]);
}

// ---- rotation and split ------------------------------------------------------
// qkv[n, :] = [q (nq*d) | k (nkv*d) | v (nkv*d)] in float.  q and k are rotated
// in pairs (i, i + d/2) by the angle pos * inv_freq[i]; v is copied.
// src/kernels/mod.rs:582-608, src/model/modules/attention.rs:68-78.
template <typename TO>
__global__ void rope_split_kernel(const float* __restrict__ qkv, const int* __restrict__ row_pos,
                                  const float* __restrict__ inv_freq, int nq, int nkv, int d,
                                  TO* __restrict__ q, TO* __restrict__ k, TO* __restrict__ v) {
  const int n = blockIdx.x;
  const int half = d / 2;
  const float pos = (float)row_pos[n];
  const float* src = qkv + (size_t)n * (nq + 2 * nkv) * d;
  const int n_rot = (nq + nkv) * half;
  for (int t = threadIdx.x; t < n_rot; t += blockDim.x) {
    const int h = t / half, i = t % half;
    const float ang = inv_freq[i] * pos;
    const float c = cosf(ang), s = sinf(ang);
    const float a = src[h * d + i], b = src[h * d + i + half];
    const float ra = a * c - b * s, rb = a * s + b * c;
    TO* dst = (h < nq) ? q + ((size_t)n * nq + h) * d : k + ((size_t)n * nkv + (h - nq)) * d;
    dst[i] = from_f32<TO>(ra);
    dst[i + half] = from_f32<TO>(rb);
  }
  const float* vs = src + (size_t)(nq + nkv) * d;
  TO* vd = v + (size_t)n * nkv * d;
  for (int t = threadIdx.x; t < nkv * d; t += blockDim.x) vd[t] = from_f32<TO>(vs[t]);
}

// ---- commit keys and values of this step to the pages -----------------------
// Position p of sequence b goes to page table[b][(p / PAGE) % ring_pages], row
// p % PAGE.  Rows that would be overwritten within this same step (older than
// the last ring_pages * PAGE positions) are skipped.  A page holds, per KV
// head, keys as [PAGE][d] and values transposed as [d][PAGE], so that both
// are read along their contraction index by the matrix cores.
template <typename T>
__global__ void kv_commit_kernel(const T* __restrict__ k, const T* __restrict__ v,
                                 const int* __restrict__ row_seq, const int* __restrict__ row_pos,
                                 const int* __restrict__ len_after, const int* __restrict__ table,
                                 int table_stride, int ring_pages, int nkv, int d,
                                 T* __restrict__ pages) {
  const int n = blockIdx.x;
  const int b = row_seq[n], p = row_pos[n];
  if (p < len_after[b] - ring_pages * PAGE) return;
  const int page = table[(size_t)b * table_stride + (p / PAGE) % ring_pages];
  const int r = p % PAGE;
  const size_t page_elems = (size_t)2 * nkv * PAGE * d;
  T* kd = pages + (size_t)page * page_elems;
  T* vd = kd + (size_t)nkv * PAGE * d;
  const T* ks = k + (size_t)n * nkv * d;
  const T* vs = v + (size_t)n * nkv * d;
  for (int t = threadIdx.x; t < nkv * d; t += blockDim.x) {
    const int h = t / d, i = t % d;
    kd[((size_t)h * PAGE + r) * d + i] = ks[t];
    vd[((size_t)h * d + i) * PAGE + r] = vs[t];
  }
}

// ---- h = silu(gate) * up, silu(g) = g / (1 + exp(-g)) ------------------------
// src/kernels/mod.rs:546-548, src/model/modules/mlp.rs:33-39.
template <typename TO>
__global__ void silu_mul_kernel(const float* __restrict__ gu, int I, TO* __restrict__ out) {
  const int n = blockIdx.x;
  const float* row = gu + (size_t)n * 2 * I;
  for (int i = threadIdx.x; i < I; i += blockDim.x) {
    const float g = row[i], u = row[I + i];
    out[(size_t)n * I + i] = from_f32<TO>((g / (1.0f + expf(-g))) * u);
  }
}

__global__ void gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ idx, int H,
                                   float* __restrict__ out) {
  const int m = blockIdx.x;
  const float* s = x + (size_t)idx[m] * H;
  float* o = out + (size_t)m * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = s[i];
}

}  // namespace tl

using namespace tl;

extern "C" {

const char* tl_last_error() { return g_err; }

int tl_embed(const void* table, int table_dt, const int* ids, int n, int H, float* out,
             hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0, "embed: bad sizes n=%d H=%d", n, H);
  if (n == 0) return 0;
  const int nt = H >= 256 ? 256 : 64;
  if (table_dt == DT_F32)
    embed_kernel<float><<<n, nt, 0, st>>>((const float*)table, ids, H, out);
  else if (table_dt == DT_BF16)
    embed_kernel<bf16><<<n, nt, 0, st>>>((const bf16*)table, ids, H, out);
  else
    TL_REQUIRE(false, "embed: unknown dtype code %d", table_dt);
  TL_LAUNCH_CHECK("embed");
  return 0;
}

int tl_rmsnorm(const float* x, const float* w, float eps, void* out, int out_dt, int n, int H,
               hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0, "rmsnorm: bad sizes n=%d H=%d", n, H);
  if (n == 0) return 0;
  if (out_dt == DT_F32)
    rmsnorm_kernel<float><<<n, 256, 0, st>>>(x, w, eps, (float*)out, H);
  else if (out_dt == DT_BF16)
    rmsnorm_kernel<bf16><<<n, 256, 0, st>>>(x, w, eps, (bf16*)out, H);
  else
    TL_REQUIRE(false, "rmsnorm: unknown dtype code %d", out_dt);
  TL_LAUNCH_CHECK("rmsnorm");
  return 0;
}

int tl_rope_split(const float* qkv, const int* row_pos, const float* inv_freq, int n, int nq,
                  int nkv, int d, void* q, void* k, void* v, int out_dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv >= 0 && d > 0 && d % 2 == 0,
             "rope_split: bad sizes n=%d nq=%d nkv=%d d=%d (d must be even)", n, nq, nkv, d);
  if (n == 0) return 0;
  if (out_dt == DT_F32)
    rope_split_kernel<float><<<n, 256, 0, st>>>(qkv, row_pos, inv_freq, nq, nkv, d, (float*)q,
                                                 (float*)k, (float*)v);
  else if (out_dt == DT_BF16)
    rope_split_kernel<bf16><<<n, 256, 0, st>>>(qkv, row_pos, inv_freq, nq, nkv, d, (bf16*)q,
                                                (bf16*)k, (bf16*)v);
  else
    TL_REQUIRE(false, "rope_split: unknown dtype code %d", out_dt);
  TL_LAUNCH_CHECK("rope_split");
  return 0;
}

int tl_kv_commit(const void* k, const void* v, int dt, const int* row_seq, const int* row_pos,
                 const int* len_after, const int* table, int table_stride, int ring_pages, int n,
                 int nkv, int d, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nkv > 0 && d > 0 && ring_pages > 0 && table_stride > 0,
             "kv_commit: bad sizes n=%d nkv=%d d=%d ring_pages=%d table_stride=%d", n, nkv, d,
             ring_pages, table_stride);
  if (n == 0) return 0;
  const int nt = nkv * d >= 256 ? 256 : 64;
  if (dt == DT_F32)
    kv_commit_kernel<float><<<n, nt, 0, st>>>((const float*)k, (const float*)v, row_seq, row_pos,
                                               len_after, table, table_stride, ring_pages, nkv, d,
                                               (float*)pages);
  else if (dt == DT_BF16)
    kv_commit_kernel<bf16><<<n, nt, 0, st>>>((const bf16*)k, (const bf16*)v, row_seq, row_pos,
                                              len_after, table, table_stride, ring_pages, nkv, d,
                                              (bf16*)pages);
  else
    TL_REQUIRE(false, "kv_commit: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("kv_commit");
  return 0;
}

int tl_silu_mul(const float* gu, int n, int I, void* out, int out_dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && I > 0, "silu_mul: bad sizes n=%d I=%d", n, I);
  if (n == 0) return 0;
  const int grid = n;
  if (out_dt == DT_F32)
    silu_mul_kernel<float><<<grid, 256, 0, st>>>(gu, I, (float*)out);
  else if (out_dt == DT_BF16)
    silu_mul_kernel<bf16><<<grid, 256, 0, st>>>(gu, I, (bf16*)out);
  else
    TL_REQUIRE(false, "silu_mul: unknown dtype code %d", out_dt);
  TL_LAUNCH_CHECK("silu_mul");
  return 0;
}

int tl_gather_rows(const float* x, const int* idx, int m, int H, float* out, hipStream_t st) {
  TL_REQUIRE(m >= 0 && H > 0, "gather_rows: bad sizes m=%d H=%d", m, H);
  if (m == 0) return 0;
  gather_rows_kernel<<<m, 256, 0, st>>>(x, idx, H, out);
  TL_LAUNCH_CHECK("gather_rows");
  return 0;
}

}  // extern "C"
