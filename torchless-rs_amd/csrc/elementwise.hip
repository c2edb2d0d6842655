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

// The same with the row held in registers: one read of x.  H % 4 == 0, H <= 1024 * IT.
template <typename TO, int IT>
__global__ void __launch_bounds__(256) rmsnorm_reg_kernel(const float* __restrict__ x,
                                                          const float* __restrict__ w, float eps,
                                                          TO* __restrict__ out, int H) {
  __shared__ float sh[4];
  const int n = blockIdx.x;
  const float4* xr = reinterpret_cast<const float4*>(x + (size_t)n * H);
  const float4* wr = reinterpret_cast<const float4*>(w);
  const int nv = H / 4;
  float4 v[IT], g[IT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      v[i] = xr[c];
      g[i] = wr[c];
      ss += v[i].x * v[i].x + v[i].y * v[i].y + v[i].z * v[i].z + v[i].w * v[i].w;
    }
  }
  ss = block_sum<256>(ss, sh);
  const float rms = sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)n * H;
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      o[4 * c + 0] = from_f32<TO>((v[i].x / rms) * g[i].x);
      o[4 * c + 1] = from_f32<TO>((v[i].y / rms) * g[i].y);
      o[4 * c + 2] = from_f32<TO>((v[i].z / rms) * g[i].z);
      o[4 * c + 3] = from_f32<TO>((v[i].w / rms) * g[i].w);
    }
  }
}

// x += sum of the partial products P[s][n][H] (in the order of s), then the norm of the new x.
template <typename TO, int IT>
__global__ void __launch_bounds__(256)
add_rmsnorm_reg_kernel(float* __restrict__ x, const float* __restrict__ parts, int n_parts, size_t part_stride,
                       const float* __restrict__ w, float eps, TO* __restrict__ out, int H) {
  __shared__ float sh[4];
  const int n = blockIdx.x;
  float4* xr = reinterpret_cast<float4*>(x + (size_t)n * H);
  const float4* wr = reinterpret_cast<const float4*>(w);
  const int nv = H / 4;
  float4 v[IT], g[IT];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      float4 a = xr[c];
#pragma unroll 4
      for (int s = 0; s < n_parts; ++s) {
        const float4 p = reinterpret_cast<const float4*>(parts + s * part_stride + (size_t)n * H)[c];
        a.x += p.x; a.y += p.y; a.z += p.z; a.w += p.w;
      }
      xr[c] = a;
      v[i] = a;
      g[i] = wr[c];
      ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
    }
  }
  ss = block_sum<256>(ss, sh);
  const float rms = sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)n * H;
#pragma unroll
  for (int i = 0; i < IT; ++i) {
    const int c = threadIdx.x + 256 * i;
    if (c < nv) {
      o[4 * c + 0] = from_f32<TO>((v[i].x / rms) * g[i].x);
      o[4 * c + 1] = from_f32<TO>((v[i].y / rms) * g[i].y);
      o[4 * c + 2] = from_f32<TO>((v[i].z / rms) * g[i].z);
      o[4 * c + 3] = from_f32<TO>((v[i].w / rms) * g[i].w);
    }
  }
}

__global__ void add_partials_kernel(float* __restrict__ x, const float* __restrict__ parts, int n_parts,
                                    size_t part_stride, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  float a = x[i];
  for (int s = 0; s < n_parts; ++s) a += parts[s * part_stride + i];
  x[i] = a;
}

// ---- rotation and split ------------------------------------------------------
// qkv[n, :] = [q (nq*d) | k (nkv*d) | v (nkv*d)] in float.  q and k are rotated
// in pairs by the angle pos * inv_freq[i] (which channels make pair i, and how many
// of a head's channels are rotated: `Rotation`, `pair_channels`); v is copied.
// The reference rotates all channels in pairs (i, i + d/2):
// src/kernels/mod.rs:582-608, src/model/modules/attention.rs:68-78.
constexpr int ROPE_MAX_HALF = 128;      // head sizes up to 256

template <typename TO>
__device__ __forceinline__ void rope_split_row(int n, float* cs, float* sn, const float* __restrict__ qkv,
                                               const int* __restrict__ row_pos, Rotation rot, int nq, int nkv, int d,
                                               TO* __restrict__ q, TO* __restrict__ k, TO* __restrict__ v,
                                               TO* __restrict__ vt, int vt_cols, const int* __restrict__ row_seq,
                                               const int* __restrict__ tile_off, const int* __restrict__ n_cached) {
  const int half = d / 2, rot_pairs = rot.rotary_dim / 2;
  const float pos = (float)row_pos[n];
  for (int i = threadIdx.x; i < rot_pairs; i += blockDim.x) {     // the row's angles, once
    const float ang = rot.inv_freq[i] * pos;
    sincosf(ang, &sn[i], &cs[i]);          // one routine for both, the same in every kernel that rotates
  }
  __syncthreads();
  const float* src = qkv + (size_t)n * (nq + 2 * nkv) * d;
  const int n_rot = (nq + nkv) * half;
  for (int t = threadIdx.x; t < n_rot; t += blockDim.x) {
    const int h = t / half, i = t % half;
    int ia, ib;
    pair_channels(i, rot.rotary_dim, rot.interleaved, ia, ib);
    const float a = src[h * d + ia], b = src[h * d + ib];
    float ra = a, rb = b;
    if (i < rot_pairs) rotate_pair(a, b, cs[i], sn[i], ra, rb);
    TO* dst = (h < nq) ? q + ((size_t)n * nq + h) * d : k + ((size_t)n * nkv + (h - nq)) * d;
    dst[ia] = from_f32<TO>(ra);
    dst[ib] = from_f32<TO>(rb);
  }
  const float* vs = src + (size_t)(nq + nkv) * d;
  if (v != nullptr) {
    TO* vd = v + (size_t)n * nkv * d;
    for (int t = threadIdx.x; t < nkv * d; t += blockDim.x) vd[t] = from_f32<TO>(vs[t]);
  }
  if (vt != nullptr) {      // the same values transposed: [kv head][d][column of this row]
    const int b = row_seq[n];
    const int col = tile_off[b] + row_pos[n] - (n_cached[b] / PAGE) * PAGE;
    for (int t = threadIdx.x; t < nkv * d; t += blockDim.x) vt[(size_t)t * vt_cols + col] = from_f32<TO>(vs[t]);
  }
}

template <typename TO>
__global__ void rope_split_kernel(const float* __restrict__ qkv, const int* __restrict__ row_pos,
                                  Rotation rot, int nq, int nkv, int d,
                                  TO* __restrict__ q, TO* __restrict__ k, TO* __restrict__ v,
                                  TO* __restrict__ vt, int vt_cols, const int* __restrict__ row_seq,
                                  const int* __restrict__ tile_off, const int* __restrict__ n_cached) {
  __shared__ float cs[ROPE_MAX_HALF], sn[ROPE_MAX_HALF];
  rope_split_row<TO>(blockIdx.x, cs, sn, qkv, row_pos, rot, nq, nkv, d, q, k, v, vt, vt_cols, row_seq, tile_off,
                     n_cached);
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

// ---- values by tiles of 64 positions ------------------------------------------
// Buffers laid out by aligned columns hold sequence b from column tile_off[b] on, position
// 64 * (n_cached[b] / 64) first, so that a tile of 64 columns is one cache page.  Which
// sequence and which positions a tile of columns holds:
struct ColumnTile {
  int b, p0, lo, hi;        // sequence, position of column 0, positions [lo, hi) of this step in it
};
__device__ __forceinline__ ColumnTile column_tile(int col0, int B, const int* tile_off, const int* n_cached,
                                                  const int* len_after) {
  int b = 0;
  while (b + 1 < B && tile_off[b + 1] <= col0) ++b;
  const int cached = n_cached[b], after = len_after[b];
  ColumnTile t;
  t.b = b;
  t.p0 = (cached / PAGE) * PAGE + (col0 - tile_off[b]);
  t.lo = max(t.p0, cached);
  t.hi = min(t.p0 + PAGE, after);            // lo >= hi: padding, nothing of this step
  return t;
}

// vt[kv head][dv][column] = v of the row at that column, from the fused projection (float):
// the transposed values of a step, written in whole lines (a row-by-row kernel writes them
// two bytes at a time, a line apart).  grid: (columns / 64, kv heads, d / 64 rounded up).
template <typename TO>
__device__ __forceinline__ void v_tile(int col_block, int kvh, int d_block, TO (*tile)[PAGE + 2],
                                       const float* __restrict__ qkv, int width, int v_off, int d,
                                       TO* __restrict__ vt, int vt_cols, int B, const int* __restrict__ cu_seqlens,
                                       const int* __restrict__ tile_off, const int* __restrict__ n_cached,
                                       const int* __restrict__ len_after) {
  const int col0 = col_block * PAGE;
  const ColumnTile t = column_tile(col0, B, tile_off, n_cached, len_after);
  if (t.lo >= t.hi) return;
  const int row0 = cu_seqlens[t.b] - n_cached[t.b];       // row of position p is row0 + p
  const int c0 = d_block * 64, dc = min(64, d - c0);       // this block's 64 of the d values
  // all loads first (16 a thread), then the stores: one trip to memory
  float tmp[16];
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int idx = threadIdx.x + 256 * u;
    const int r = idx / dc, i = idx % dc, p = t.p0 + r;
    tmp[u] = (idx < PAGE * dc && p >= t.lo && p < t.hi)
                 ? qkv[(size_t)(row0 + p) * width + v_off + kvh * d + c0 + i] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int idx = threadIdx.x + 256 * u;
    if (idx < PAGE * dc) tile[idx % dc][idx / dc] = from_f32<TO>(tmp[u]);
  }
  __syncthreads();
#pragma unroll
  for (int u = 0; u < 16; ++u) {
    const int idx = threadIdx.x + 256 * u;
    const int i = idx / PAGE, r = idx % PAGE, p = t.p0 + r;
    if (i < dc && p >= t.lo && p < t.hi) vt[((size_t)kvh * d + c0 + i) * vt_cols + col0 + r] = tile[i][r];
  }
}

template <typename TO>
__global__ void __launch_bounds__(256)
v_tiles_kernel(const float* __restrict__ qkv, int width, int v_off, int d, TO* __restrict__ vt,
               int vt_cols, int B, const int* __restrict__ cu_seqlens, const int* __restrict__ tile_off,
               const int* __restrict__ n_cached, const int* __restrict__ len_after) {
  __shared__ TO tile[64][PAGE + 2];
  v_tile<TO>(blockIdx.x, blockIdx.y, blockIdx.z, tile, qkv, width, v_off, d, vt, vt_cols, B, cu_seqlens, tile_off,
             n_cached, len_after);
}

// Both of the above in one launch, for a step with several rows a sequence: the first n workgroups
// rotate a row each (q and k; the values are the tiles' business), the others transpose a tile of
// values each.  The two read the same buffer and write different ones.
template <typename TO>
__global__ void __launch_bounds__(256)
rope_v_tiles_kernel(const float* __restrict__ qkv, const int* __restrict__ row_pos, Rotation rot, int n, int nq,
                    int nkv, int d, TO* __restrict__ q, TO* __restrict__ k, TO* __restrict__ vt, int vt_cols, int B,
                    const int* __restrict__ cu_seqlens, const int* __restrict__ tile_off,
                    const int* __restrict__ n_cached, const int* __restrict__ len_after) {
  __shared__ __attribute__((aligned(16))) unsigned char sh[sizeof(TO) * 64 * (PAGE + 2) > 2 * sizeof(float) * ROPE_MAX_HALF
                                                            ? sizeof(TO) * 64 * (PAGE + 2)
                                                            : 2 * sizeof(float) * ROPE_MAX_HALF];
  if ((int)blockIdx.x < n) {
    float* cs = reinterpret_cast<float*>(sh);
    rope_split_row<TO>(blockIdx.x, cs, cs + ROPE_MAX_HALF, qkv, row_pos, rot, nq, nkv, d, q, k, (TO*)nullptr,
                       (TO*)nullptr, 0, nullptr, nullptr, nullptr);
    return;
  }
  const int item = blockIdx.x - n, d_blocks = (d + 63) / 64;
  const int d_block = item % d_blocks, kvh = (item / d_blocks) % nkv, col_block = item / (d_blocks * nkv);
  v_tile<TO>(col_block, kvh, d_block, reinterpret_cast<TO(*)[PAGE + 2]>(sh), qkv, (nq + 2 * nkv) * d, (nq + nkv) * d, d,
             vt, vt_cols, B, cu_seqlens, tile_off, n_cached, len_after);
}

// Commit of a step whose values lie transposed by tiles: the first blocks put the keys of 8 rows
// each into their pages, the others copy a tile of values [d][64] of one KV head in whole lines.
// Positions that the same step overwrites in a ring are skipped, as in kv_commit.
template <typename T>
__global__ void __launch_bounds__(256)
kv_commit_tiles_kernel(const T* __restrict__ k, const T* __restrict__ vt, int vt_cols, int n,
                       const int* __restrict__ row_seq, const int* __restrict__ row_pos, int B,
                       const int* __restrict__ tile_off, const int* __restrict__ n_cached,
                       const int* __restrict__ len_after, const int* __restrict__ table, int table_stride,
                       int ring_pages, int nkv, int d, T* __restrict__ pages) {
  const size_t page_elems = (size_t)2 * nkv * PAGE * d;
  const int k_blocks = (n + 7) / 8;
  if ((int)blockIdx.x < k_blocks) {
    // 8 rows a block, 32 threads a row, 16 bytes at a time where the head size allows
    constexpr int VEC = 16 / sizeof(T);
    const int r_n = blockIdx.x * 8 + threadIdx.x / 32, lane = threadIdx.x % 32;
    if (r_n >= n) return;
    const int b = row_seq[r_n], p = row_pos[r_n];
    if (p < len_after[b] - ring_pages * PAGE) return;
    const int page = table[(size_t)b * table_stride + (p / PAGE) % ring_pages];
    T* kd = pages + (size_t)page * page_elems;
    const T* ks = k + (size_t)r_n * nkv * d;
    if (d % VEC == 0 && ((uintptr_t)k % 16 == 0) && ((uintptr_t)pages % 16 == 0)) {
      for (int c = lane; c < nkv * d / VEC; c += 32) {
        const int e = c * VEC, h = e / d, i = e % d;
        *reinterpret_cast<f32x4*>(&kd[((size_t)h * PAGE + p % PAGE) * d + i]) =
            *reinterpret_cast<const f32x4*>(&ks[e]);
      }
    } else {
      for (int t = lane; t < nkv * d; t += 32) {
        const int h = t / d, i = t % d;
        kd[((size_t)h * PAGE + p % PAGE) * d + i] = ks[t];
      }
    }
    return;
  }
  const int v_block = blockIdx.x - k_blocks;
  const int col0 = (v_block / nkv) * PAGE, kvh = v_block % nkv;
  const ColumnTile t = column_tile(col0, B, tile_off, n_cached, len_after);
  const int lo = max(t.lo, len_after[t.b] - ring_pages * PAGE);
  if (lo >= t.hi) return;
  const int page = table[(size_t)t.b * table_stride + (t.p0 / PAGE) % ring_pages];
  T* vd = pages + (size_t)page * page_elems + (size_t)nkv * PAGE * d + (size_t)kvh * d * PAGE;
  const T* vs = vt + (size_t)kvh * d * vt_cols + col0;
  for (int base = 0; base < d * PAGE; base += 256 * 16) {      // 16 loads a thread, then their stores
    T tmp[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int idx = base + threadIdx.x + 256 * u;
      const int i = idx / PAGE, r = idx % PAGE, p = t.p0 + r;
      if (i < d && p >= lo && p < t.hi) tmp[u] = vs[(size_t)i * vt_cols + r];
    }
#pragma unroll
    for (int u = 0; u < 16; ++u) {
      const int idx = base + threadIdx.x + 256 * u;
      const int i = idx / PAGE, r = idx % PAGE, p = t.p0 + r;
      if (i < d && p >= lo && p < t.hi) vd[(size_t)i * PAGE + r] = tmp[u];
    }
  }
}

// ---- single-token steps: rotate, and put k and v straight into the pages ------
// Row n is the one new token of sequence n (position row_pos[n]).
// qkv may come as n_parts partial products (part_stride elements apart) that are added up here.
template <typename T>
__global__ void rope_commit_kernel(const float* __restrict__ qkv, int n_parts, size_t part_stride,
                                   const int* __restrict__ row_pos,
                                   Rotation rot, const int* __restrict__ table,
                                   int table_stride, int ring_pages, int nq, int nkv, int d,
                                   T* __restrict__ q, T* __restrict__ pages) {
  // blockIdx.y of gridDim.y takes its share of the (q and k) heads and of the values
  __shared__ float cs[ROPE_MAX_HALF], sn[ROPE_MAX_HALF];
  const int n = blockIdx.x;
  const int half = d / 2, rot_pairs = rot.rotary_dim / 2;
  const int p = row_pos[n];
  const float pos = (float)p;
  const float* src = qkv + (size_t)n * (nq + 2 * nkv) * d;
  const int page = table[(size_t)n * table_stride + (p / PAGE) % ring_pages];
  const int r = p % PAGE;
  T* kd = pages + (size_t)page * 2 * nkv * PAGE * d;
  T* vd = kd + (size_t)nkv * PAGE * d;
  for (int i = threadIdx.x; i < rot_pairs; i += blockDim.x) {
    const float ang = rot.inv_freq[i] * pos;
    sincosf(ang, &sn[i], &cs[i]);          // one routine for both, the same in every kernel that rotates
  }
  __syncthreads();
  const int heads = nq + nkv;
  const int h_lo = (int)((long long)heads * blockIdx.y / gridDim.y), h_hi = (int)((long long)heads * (blockIdx.y + 1) / gridDim.y);
  for (int t = h_lo * half + threadIdx.x; t < h_hi * half; t += blockDim.x) {
    const int h = t / half, i = t % half;
    int ia, ib;
    pair_channels(i, rot.rotary_dim, rot.interleaved, ia, ib);
    float a = src[h * d + ia], b = src[h * d + ib];
#pragma unroll 4
    for (int sp = 1; sp < n_parts; ++sp) {
      a += src[sp * part_stride + h * d + ia];
      b += src[sp * part_stride + h * d + ib];
    }
    float ra = a, rb = b;
    if (i < rot_pairs) rotate_pair(a, b, cs[i], sn[i], ra, rb);
    T* dst = (h < nq) ? q + ((size_t)n * nq + h) * d : kd + ((size_t)(h - nq) * PAGE + r) * d;
    dst[ia] = from_f32<T>(ra);
    dst[ib] = from_f32<T>(rb);
  }
  const float* vs = src + (size_t)(nq + nkv) * d;
  const int v_lo = (int)((long long)nkv * d * blockIdx.y / gridDim.y), v_hi = (int)((long long)nkv * d * (blockIdx.y + 1) / gridDim.y);
  for (int t = v_lo + threadIdx.x; t < v_hi; t += blockDim.x) {
    float a = vs[t];
#pragma unroll 4
    for (int sp = 1; sp < n_parts; ++sp) a += vs[sp * part_stride + t];
    vd[(size_t)t * PAGE + r] = from_f32<T>(a);
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

// gu[n, 2I] in bfloat16 with columns in groups of 64 (32 of gate, then the 32 of up
// that belong to them); out[n, I] = silu(gate) * up.  A thread takes 8 pairs.
__global__ void silu_mul_pairs_kernel(const bf16* __restrict__ gu, long long chunks, int I,
                                      bf16* __restrict__ out) {
  const long long c = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= chunks) return;
  const int per_row = I / 8;
  const long long n = c / per_row;
  const int i = (int)(c % per_row), group = i / 4, part = i % 4;
  const bf16* src = gu + n * 2 * I + group * 64 + part * 8;
  const bf16x8 g = *reinterpret_cast<const bf16x8*>(src);
  const bf16x8 u = *reinterpret_cast<const bf16x8*>(src + 32);
  bf16x8 o;
#pragma unroll
  for (int t = 0; t < 8; ++t) {
    const float gv = (float)g[t];
    o[t] = (bf16)((gv / (1.0f + expf(-gv))) * (float)u[t]);
  }
  *reinterpret_cast<bf16x8*>(out + n * I + group * 32 + part * 8) = o;
}

// tokens[j] = src[idx[j]]: the ids that the sampler left on the device become the next step's
// input without a trip to the host.  An id outside the vocabulary becomes 0 (no row of the
// embedding lies there).
__global__ void take_tokens_kernel(const int* __restrict__ src, const int* __restrict__ idx, int n,
                                   int n_src, int vocab, int* __restrict__ tokens) {
  const int j = blockIdx.x * blockDim.x + threadIdx.x;
  if (j >= n) return;
  const int r = idx[j];
  const int t = (r >= 0 && r < n_src) ? src[r] : 0;
  tokens[j] = (t >= 0 && t < vocab) ? t : 0;
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
int tl_page_size() { return PAGE; }      // what this library was compiled with (csrc/page.h)

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
  TL_REQUIRE(out_dt == DT_F32 || out_dt == DT_BF16, "rmsnorm: unknown dtype code %d", out_dt);
  const bool vec = H % 4 == 0 && H <= 8192 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0);
#define TL_RMS(IT)                                                                        \
  do {                                                                                    \
    if (out_dt == DT_F32) rmsnorm_reg_kernel<float, IT><<<n, 256, 0, st>>>(x, w, eps, (float*)out, H); \
    else rmsnorm_reg_kernel<bf16, IT><<<n, 256, 0, st>>>(x, w, eps, (bf16*)out, H);        \
  } while (0)
  if (vec && H <= 1024) TL_RMS(1);
  else if (vec && H <= 2048) TL_RMS(2);
  else if (vec && H <= 4096) TL_RMS(4);
  else if (vec) TL_RMS(8);
  else if (out_dt == DT_F32)
    rmsnorm_kernel<float><<<n, 256, 0, st>>>(x, w, eps, (float*)out, H);
  else
    rmsnorm_kernel<bf16><<<n, 256, 0, st>>>(x, w, eps, (bf16*)out, H);
#undef TL_RMS
  TL_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// vt (may be null): values also transposed, [nkv][d][vt_cols], row n in column
// tile_off[row_seq[n]] + row_pos[n] - 64 * (n_cached[row_seq[n]] / 64)
// x[n, H] += parts[0..n_parts)[n, H]; out = rmsnorm(x)
int tl_add_rmsnorm(float* x, const float* parts, int n_parts, const float* w, float eps, void* out, int out_dt,
                   int n, int H, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && n_parts >= 0, "add_rmsnorm: bad sizes n=%d H=%d parts=%d", n, H, n_parts);
  TL_REQUIRE(out_dt == DT_F32 || out_dt == DT_BF16, "add_rmsnorm: unknown dtype code %d", out_dt);
  TL_REQUIRE(H % 4 == 0 && H <= 8192 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
             ((uintptr_t)parts % 16 == 0), "add_rmsnorm: H=%d must be a multiple of 4, at most 8192, rows 16-byte aligned", H);
  if (n == 0) return 0;
  const size_t stride = (size_t)n * H;
#define TL_ARMS(IT)                                                                                        \
  do {                                                                                                     \
    if (out_dt == DT_F32) add_rmsnorm_reg_kernel<float, IT><<<n, 256, 0, st>>>(x, parts, n_parts, stride, w, eps, (float*)out, H); \
    else add_rmsnorm_reg_kernel<bf16, IT><<<n, 256, 0, st>>>(x, parts, n_parts, stride, w, eps, (bf16*)out, H);                   \
  } while (0)
  if (H <= 1024) TL_ARMS(1);
  else if (H <= 2048) TL_ARMS(2);
  else if (H <= 4096) TL_ARMS(4);
  else TL_ARMS(8);
#undef TL_ARMS
  TL_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

// x[n, H] += parts[0..n_parts)[n, H]
int tl_add_partials(float* x, const float* parts, int n_parts, int n, int H, hipStream_t st) {
  TL_REQUIRE(n >= 0 && H > 0 && n_parts >= 0, "add_partials: bad sizes n=%d H=%d parts=%d", n, H, n_parts);
  if (n == 0 || n_parts == 0) return 0;
  const size_t total = (size_t)n * H;
  add_partials_kernel<<<(unsigned)((total + 255) / 256), 256, 0, st>>>(x, parts, n_parts, total, total);
  TL_LAUNCH_CHECK("add_partials");
  return 0;
}

// inv_freq [rotary_dim / 2], rotary_dim (even, 0..d; 0: no rotation), interleaved: see `Rotation`
int tl_rope_split(const float* qkv, const int* row_pos, const float* inv_freq, int rotary_dim, int interleaved,
                  int n, int nq, int nkv, int d, void* q, void* k, void* v, void* vt, int vt_cols,
                  const int* row_seq, const int* tile_off, const int* n_cached, int out_dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv >= 0 && d > 0 && d % 2 == 0,
             "rope_split: bad sizes n=%d nq=%d nkv=%d d=%d (d must be even)", n, nq, nkv, d);
  TL_REQUIRE(d <= 2 * ROPE_MAX_HALF, "rope_split: head size %d is not served (at most %d)", d, 2 * ROPE_MAX_HALF);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0 && (rotary_dim == 0 || inv_freq != nullptr),
             "rope_split: %d rotated channels of a head of %d (even, at most the head, with their frequencies)",
             rotary_dim, d);
  const Rotation rot{inv_freq, rotary_dim, interleaved != 0};
  if (n == 0) return 0;
  if (out_dt == DT_F32)
    rope_split_kernel<float><<<n, 256, 0, st>>>(qkv, row_pos, rot, nq, nkv, d, (float*)q,
                                                 (float*)k, (float*)v, (float*)vt, vt_cols, row_seq,
                                                 tile_off, n_cached);
  else if (out_dt == DT_BF16)
    rope_split_kernel<bf16><<<n, 256, 0, st>>>(qkv, row_pos, rot, nq, nkv, d, (bf16*)q,
                                                (bf16*)k, (bf16*)v, (bf16*)vt, vt_cols, row_seq, tile_off,
                                                n_cached);
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

int tl_v_tiles(const float* qkv, int n, int nq, int nkv, int d, void* vt, int vt_cols, int dt, int B,
               const int* cu_seqlens, const int* tile_off, const int* n_cached, const int* len_after,
               hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq >= 0 && nkv > 0 && d > 0 && B > 0, "v_tiles: bad sizes n=%d nq=%d nkv=%d d=%d B=%d", n, nq,
             nkv, d, B);
  TL_REQUIRE(vt_cols > 0 && vt_cols % PAGE == 0 && nkv <= 65535, "v_tiles: %d columns (a multiple of 64), %d KV heads",
             vt_cols, nkv);
  if (n == 0) return 0;
  const int width = (nq + 2 * nkv) * d, v_off = (nq + nkv) * d;
  const dim3 grid(vt_cols / PAGE, nkv, (d + 63) / 64);
  if (dt == DT_F32)
    v_tiles_kernel<float><<<grid, 256, 0, st>>>(qkv, width, v_off, d, (float*)vt, vt_cols, B, cu_seqlens,
                                                 tile_off, n_cached, len_after);
  else if (dt == DT_BF16)
    v_tiles_kernel<bf16><<<grid, 256, 0, st>>>(qkv, width, v_off, d, (bf16*)vt, vt_cols, B, cu_seqlens,
                                                tile_off, n_cached, len_after);
  else
    TL_REQUIRE(false, "v_tiles: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("v_tiles");
  return 0;
}

int tl_kv_commit_tiles(const void* k, const void* vt, int vt_cols, int dt, const int* row_seq, const int* row_pos,
                       int B, const int* tile_off, const int* n_cached, const int* len_after, const int* table,
                       int table_stride, int ring_pages, int n, int nkv, int d, void* pages, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nkv > 0 && d > 0 && ring_pages > 0 && table_stride > 0 && B > 0,
             "kv_commit_tiles: bad sizes n=%d nkv=%d d=%d ring_pages=%d table_stride=%d B=%d", n, nkv, d,
             ring_pages, table_stride, B);
  TL_REQUIRE(vt_cols > 0 && vt_cols % PAGE == 0, "kv_commit_tiles: %d columns (a multiple of 64)", vt_cols);
  if (n == 0) return 0;
  const long long blocks = (long long)((n + 7) / 8) + (long long)(vt_cols / PAGE) * nkv;
  TL_REQUIRE(blocks < 2147483647LL, "kv_commit_tiles: too many blocks");
  if (dt == DT_F32)
    kv_commit_tiles_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(
        (const float*)k, (const float*)vt, vt_cols, n, row_seq, row_pos, B, tile_off, n_cached, len_after, table,
        table_stride, ring_pages, nkv, d, (float*)pages);
  else if (dt == DT_BF16)
    kv_commit_tiles_kernel<bf16><<<(unsigned)blocks, 256, 0, st>>>(
        (const bf16*)k, (const bf16*)vt, vt_cols, n, row_seq, row_pos, B, tile_off, n_cached, len_after, table,
        table_stride, ring_pages, nkv, d, (bf16*)pages);
  else
    TL_REQUIRE(false, "kv_commit_tiles: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("kv_commit_tiles");
  return 0;
}

// tl_rope_split (q and k only) and tl_v_tiles in one launch: see rope_v_tiles_kernel
int tl_rope_v_tiles(const float* qkv, const int* row_pos, const float* inv_freq, int rotary_dim, int interleaved,
                    int n, int nq, int nkv, int d, void* q, void* k, void* vt, int vt_cols, int B,
                    const int* cu_seqlens, const int* tile_off, const int* n_cached, const int* len_after, int dt,
                    hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv > 0 && d > 0 && d % 2 == 0 && d <= 2 * ROPE_MAX_HALF && B > 0,
             "rope_v_tiles: bad sizes n=%d nq=%d nkv=%d d=%d B=%d (d even, at most %d)", n, nq, nkv, d, B,
             2 * ROPE_MAX_HALF);
  TL_REQUIRE(vt_cols > 0 && vt_cols % PAGE == 0, "rope_v_tiles: %d columns are no multiple of %d", vt_cols, PAGE);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0 && (rotary_dim == 0 || inv_freq != nullptr),
             "rope_v_tiles: %d rotated channels of a head of %d (even, at most the head, with their frequencies)",
             rotary_dim, d);
  if (n == 0) return 0;
  const Rotation rot{inv_freq, rotary_dim, interleaved != 0};
  const long long blocks = (long long)n + (long long)(vt_cols / PAGE) * nkv * ((d + 63) / 64);
  TL_REQUIRE(blocks < 2147483647LL, "rope_v_tiles: %lld workgroups are too many", blocks);
  if (dt == DT_F32)
    rope_v_tiles_kernel<float><<<(unsigned)blocks, 256, 0, st>>>(qkv, row_pos, rot, n, nq, nkv, d, (float*)q, (float*)k,
                                                                  (float*)vt, vt_cols, B, cu_seqlens, tile_off, n_cached,
                                                                  len_after);
  else if (dt == DT_BF16)
    rope_v_tiles_kernel<bf16><<<(unsigned)blocks, 256, 0, st>>>(qkv, row_pos, rot, n, nq, nkv, d, (bf16*)q, (bf16*)k,
                                                                 (bf16*)vt, vt_cols, B, cu_seqlens, tile_off, n_cached,
                                                                 len_after);
  else
    TL_REQUIRE(false, "rope_v_tiles: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("rope_v_tiles");
  return 0;
}

// n_parts >= 1: qkv is [n_parts][n][(nq + 2 nkv) d], summed on the way in
int tl_rope_commit(const float* qkv, int n_parts, const int* row_pos, const float* inv_freq, int rotary_dim,
                   int interleaved, const int* table, int table_stride, int ring_pages, int n, int nq, int nkv,
                   int d, void* q, void* pages, int dt, hipStream_t st) {
  TL_REQUIRE(n >= 0 && nq > 0 && nkv > 0 && d > 0 && d % 2 == 0 && ring_pages > 0 && table_stride > 0,
             "rope_commit: bad sizes n=%d nq=%d nkv=%d d=%d ring_pages=%d table_stride=%d", n, nq, nkv, d,
             ring_pages, table_stride);
  TL_REQUIRE(d <= 2 * ROPE_MAX_HALF, "rope_commit: head size %d is not served (at most %d)", d, 2 * ROPE_MAX_HALF);
  TL_REQUIRE(n_parts >= 1, "rope_commit: n_parts=%d", n_parts);
  TL_REQUIRE(rotary_dim >= 0 && rotary_dim <= d && rotary_dim % 2 == 0 && (rotary_dim == 0 || inv_freq != nullptr),
             "rope_commit: %d rotated channels of a head of %d (even, at most the head, with their frequencies)",
             rotary_dim, d);
  const Rotation rot{inv_freq, rotary_dim, interleaved != 0};
  if (n == 0) return 0;
  const size_t stride = (size_t)n * (nq + 2 * nkv) * d;
  const dim3 grid(n, n >= 128 ? 1 : (n >= 32 ? 4 : 8));       // few rows: cut the heads over more workgroups
  if (dt == DT_F32)
    rope_commit_kernel<float><<<grid, 256, 0, st>>>(qkv, n_parts, stride, row_pos, rot, table, table_stride,
                                                  ring_pages, nq, nkv, d, (float*)q, (float*)pages);
  else if (dt == DT_BF16)
    rope_commit_kernel<bf16><<<grid, 256, 0, st>>>(qkv, n_parts, stride, row_pos, rot, table, table_stride,
                                                 ring_pages, nq, nkv, d, (bf16*)q, (bf16*)pages);
  else
    TL_REQUIRE(false, "rope_commit: unknown dtype code %d", dt);
  TL_LAUNCH_CHECK("rope_commit");
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

int tl_silu_mul_pairs(const void* gu, int n, int I, void* out, hipStream_t st) {
  TL_REQUIRE(n >= 0 && I > 0 && I % 32 == 0, "silu_mul_pairs: bad sizes n=%d I=%d (I in steps of 32)", n, I);
  TL_REQUIRE((uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0, "silu_mul_pairs: buffers must be 16-byte aligned");
  if (n == 0) return 0;
  const long long chunks = (long long)n * (I / 8);
  TL_REQUIRE((chunks + 255) / 256 < 2147483647LL, "silu_mul_pairs: too many elements");
  silu_mul_pairs_kernel<<<(unsigned)((chunks + 255) / 256), 256, 0, st>>>((const bf16*)gu, chunks, I, (bf16*)out);
  TL_LAUNCH_CHECK("silu_mul_pairs");
  return 0;
}

int tl_take_tokens(const int* src, const int* idx, int n, int n_src, int vocab, int* tokens, hipStream_t st) {
  TL_REQUIRE(n >= 0 && n_src > 0 && vocab > 0, "take_tokens: bad sizes n=%d n_src=%d vocab=%d", n, n_src, vocab);
  if (n == 0) return 0;
  take_tokens_kernel<<<(n + 255) / 256, 256, 0, st>>>(src, idx, n, n_src, vocab, tokens);
  TL_LAUNCH_CHECK("take_tokens");
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
