// bfloat16 attention on the matrix cores: one kernel for steps that bring many
// rows per sequence (prefill), one for single-token steps (decode).
//
// Visibility, scaling and softmax are those of the plain kernel (key j is seen
// by the query at p iff j <= p and, with a window W, j > p - W; score =
// (k.q) * scale; softmax with a running maximum), with the statistics in
// float.  Both kernels compute the transposed products S^T = K Q^T and
// O^T = V^T P^T: a lane then owns one query (or head) column, the softmax
// over keys runs inside the lane, and the probabilities leave the first
// product in exactly the register layout the second one takes.  The value
// operand must be read along keys; pages store values transposed ([d][PAGE])
// for that, and the prefill kernel transposes the step's own value rows on
// their way into LDS.
#include "common.hpp"
#include "no_alloc.h"
#include <mutex>

namespace tl {

#define TL_AS1 __attribute__((address_space(1)))      // global memory and LDS, as global_load_lds takes them
#define TL_AS3 __attribute__((address_space(3)))

__device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 ld4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }
// 16 bytes at a uniform base plus a lane's offset in bytes (32 bits: one address register)
__device__ __forceinline__ bf16x8 ld8_at(const bf16* base, unsigned bytes) {
  return *reinterpret_cast<const bf16x8*>(reinterpret_cast<const char*>(base) + bytes);
}
__device__ __forceinline__ bf16x8 z8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// ------------------------------------------------------------------ prefill --
// One workgroup: 128 consecutive new rows of one sequence (4 waves x 32) and
// one query head.  Keys go by tiles of 64 positions (aligned to 64, so a tile
// below n_cached is one cache page).  The step's own values come transposed,
// vt_new[kv head][d][column], column = tile_off[b] + (position - 64 *
// (n_cached[b] / 64)): positions that are multiples of 64 lie on columns that
// are, so tiles are read with aligned 16-byte loads.  The next tile is
// fetched into registers while the current one is worked on.
constexpr int PF_BM = 128, PF_BN = 64, PF_VLD = PF_BN + 4;
constexpr int PF_PART_HEAD = 4;       // floats before O in a half block's partial result: maximum, sum, two of padding

template <int DPAD, bool LEAN>       // LEAN (d == DPAD, 256 % (DPAD / 8) == 0): whole tiles are fetched the short way
__global__ void __launch_bounds__(256, DPAD <= 128 ? 2 : 1)
attn_prefill_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_new,
                    const bf16* __restrict__ vt_new, int vt_cols, const int* __restrict__ tile_off,
                    const bf16* __restrict__ pages, const int* __restrict__ table, int table_stride,
                    int ring_pages, const int* __restrict__ row_pos, const int* __restrict__ cu_seqlens,
                    const int* __restrict__ n_cached, int B, int n_tiles, int nq, int nkv, int d,
                    int window, float scale, bf16* __restrict__ out, const int4* __restrict__ items,
                    float* __restrict__ part, int part_ways) {
  constexpr int KB = DPAD / 16, VB = DPAD / 32, KLD = DPAD + 8, CH = DPAD / 8;
  constexpr int PT = DPAD / 32;        // 16-byte chunks of keys, and of values, per thread and tile
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  bf16* Ks = reinterpret_cast<bf16*>(smem);          // [PF_BN][KLD]
  bf16* Vt = Ks + PF_BN * KLD;                       // [DPAD][PF_VLD]

  // Which head and which block of rows.  Workgroups are dealt round to the 8 XCDs and start in the order
  // of their numbers.  An XCD takes nq / 8 neighbouring heads, whose one or two KV heads stay in its L2,
  // and goes through the step's blocks of rows from the last to the first, those heads side by side: they
  // read the same tiles of keys at the same time, and under a causal mask the blocks with the most tiles
  // start first and the short ones fill the compute units as they come free.  The nq % 8 heads that are
  // left over are dealt to all XCDs in the same order, ahead of the others.
  // A wave raises its priority while it issues the MFMAs of a tile's two products, so that of the two
  // waves of a SIMD the one that feeds the matrix cores goes first and the other's exponentials fill in:
  // up to a tenth faster where tiles are many (4 x 512 rows over 65,536 cached keys 1.85 against 2.03 ms),
  // 3 us slower for one prompt of 2,048 tokens, whose longest chain of tiles decides.
  const int hpx = nq / 8, rest = nq % 8;
  int h, t, b = 0;
  if ((int)blockIdx.x < rest * n_tiles) {
    h = 8 * hpx + (int)blockIdx.x % rest;
    t = n_tiles - 1 - (int)blockIdx.x / rest;
  } else {
    const int i = (int)blockIdx.x - rest * n_tiles, idx = i / 8;
    h = (i % 8) * hpx + idx % hpx;
    t = n_tiles - 1 - idx / hpx;
  }
  // With `items` the host has laid the work out (n_tiles counts its entries, the dearest last).  An entry
  // is (sequence, block, 0, 0) for a whole block, or (sequence, block, first tile of keys, one past the
  // last | slot << 24 | (ways - 1) << 27 | 1 << 30) for one of the `ways` runs of tiles into which the
  // block's keys are cut: a workgroup a run, which writes its sums to place `slot` of the block's rows in
  // `part` for attn_prefill_merge_kernel.  A launch with fewer workgroups than the device has compute units
  // waits for its longest chain of tiles while units stand idle, and this is what shortens it.
  int cut_lo = 0, cut_hi = 0, slot = 0, ways = 0;
  if (items != nullptr) {
    const int4 it = items[t];
    b = it.x;
    t = it.y;
    cut_lo = it.z;
    cut_hi = it.w & 0xffffff;
    slot = (it.w >> 24) & 7;
    ways = (it.w >> 30) & 1 ? ((it.w >> 27) & 7) + 1 : 0;
  } else {
    for (; b < B; ++b) {
      const int tiles = (cu_seqlens[b + 1] - cu_seqlens[b] + PF_BM - 1) / PF_BM;
      if (t < tiles) break;
      t -= tiles;
    }
    if (b == B) return;
  }
  const int tid = threadIdx.x, wave = tid / 64, lane = tid % 64, l32 = lane % 32, half = lane / 32;
  const int kvh = h / (nq / nkv);
  const int row0 = cu_seqlens[b], n_new = cu_seqlens[b + 1] - row0;
  const int cached = n_cached[b];
  const int p_first = row_pos[row0];
  const size_t head_elems = (size_t)PAGE * d, page_elems = 2 * (size_t)nkv * head_elems;
  const int j_base = (cached / PAGE) * PAGE;
  const bf16* vt_head = vt_new + (size_t)kvh * d * vt_cols + tile_off[b];
  const int seq_end = p_first + n_new;               // one past the sequence's last position
  static_assert(PF_BN == PAGE, "a tile of keys below n_cached is one page");
  static_assert(!LEAN || 256 % CH == 0, "the short way needs every thread's chunks in one column of chunks");
  const unsigned k_row = tid / CH, k_col = (tid % CH) * 16;                        // offsets in bytes
  const unsigned v_row = tid / (PF_BN / 8), v_col = (tid % (PF_BN / 8)) * 16;

  const int qt0 = t * PF_BM;
  const int qr = qt0 + wave * 32 + l32;               // this lane's query row among the new rows
  const bool q_ok = qr < n_new;
  const int p_me = p_first + qr;

  bf16x8 qreg[KB];
  {
    const bf16* qp = q + ((size_t)(row0 + min(qr, n_new - 1)) * nq + h) * d;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int k = kb * 16 + 8 * half;
      qreg[kb] = (k + 8 <= d) ? ld8(qp + k) : z8();
    }
  }
  f32x16 o[VB];
#pragma unroll
  for (int vb = 0; vb < VB; ++vb)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[vb][r] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int p_lo = p_first + qt0, p_hi = p_first + min(qt0 + PF_BM, n_new) - 1;
  const int pw_lo = p_lo + wave * 32, pw_hi = min(p_hi, pw_lo + 31);    // this wave's positions
  const int j_lo = (window > 0 && p_lo - window + 1 > 0) ? p_lo - window + 1 : 0;

  bf16x8 kfetch[PT], vfetch[PT];
  // tile j0 -> registers: keys as rows [key][d], values as rows [dv][key]
  // Whole tiles of a head that fills its padded size take the short way: the workgroup's base
  // address is uniform and a thread's chunks lie at fixed offsets from it, one stride apart.
  auto fetch_lean = [&](const bf16* kbase, unsigned k_stride, const bf16* vbase, unsigned v_stride) {
    // the offsets are worked out anew for every tile (a multiply-add each): kept across the loop
    // they would take sixteen registers that the loop does not have
    unsigned kr = k_row, vr = v_row;
    asm volatile("" : "+v"(kr), "+v"(vr));
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      kfetch[i] = ld8_at(kbase, (kr + i * (256 / CH)) * k_stride + k_col);
      vfetch[i] = ld8_at(vbase, (vr + i * (256 / (PF_BN / 8))) * v_stride + v_col);
    }
  };
  // tiles are fetched in their order: the place in the ring of pages is counted along, and the
  // page of the tile after the next is looked up a tile early, so that no fetch waits for it
  int jt_first = j_lo / PF_BN, jt_last = p_hi / PF_BN;          // this workgroup's tiles of keys
  if (ways != 0) {
    jt_first = max(jt_first, cut_lo);
    jt_last = min(jt_last, cut_hi - 1);
  }
  int f_ring = jt_first % ring_pages;
  int page_nxt = ((jt_first + 1) * PF_BN <= cached) ? table[(size_t)b * table_stride + f_ring] : 0;
  auto fetch = [&](int j0) {
    const int page = page_nxt;
    f_ring = (f_ring + 1 == ring_pages) ? 0 : f_ring + 1;
    if (j0 + 2 * PF_BN <= cached) page_nxt = table[(size_t)b * table_stride + f_ring];
    if (j0 + PF_BN <= cached) {
      // a cached page: keys [64][d], values [d][64]
      const bf16* kpage = pages + (size_t)page * page_elems + (size_t)kvh * head_elems;
      const bf16* vpage = kpage + (size_t)nkv * head_elems;
      if constexpr (LEAN) {
        fetch_lean(kpage, 2u * d, vpage, 2u * PAGE);        // rows [64][d] and [d][64]
        return;
      }
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const int c = tid + 256 * i;
        const int row = c / CH, col = (c % CH) * 8;
        kfetch[i] = (col < d) ? ld8(kpage + (size_t)row * d + col) : z8();
        const int dv = c / (PF_BN / 8), kc = (c % (PF_BN / 8)) * 8;
        vfetch[i] = (dv < d) ? ld8(vpage + (size_t)dv * PAGE + kc) : z8();
      }
      return;
    }
    if (j0 >= cached && j0 + PF_BN <= seq_end) {
      // rows of this step, all of them written
      const bf16* krows = k_new + ((size_t)(row0 + j0 - cached) * nkv + kvh) * d;
      const bf16* vcols = vt_head + (j0 - j_base);
      if constexpr (LEAN) {
        fetch_lean(krows, 2u * nkv * d, vcols, 2u * vt_cols);
        return;
      }
#pragma unroll
      for (int i = 0; i < PT; ++i) {
        const int c = tid + 256 * i;
        const int row = c / CH, col = (c % CH) * 8;
        kfetch[i] = (col < d) ? ld8(krows + (size_t)row * nkv * d + col) : z8();
        const int dv = c / (PF_BN / 8), kc = (c % (PF_BN / 8)) * 8;
        vfetch[i] = (dv < d) ? ld8(vcols + (size_t)dv * vt_cols + kc) : z8();
      }
      return;
    }
    // the tile that holds the boundary between cached and new rows, or the sequence's end
    const bool has_cached = j0 < cached, has_new = j0 + PF_BN > cached;
    const bf16* kpage = nullptr;
    if (has_cached) {
      const int page = table[(size_t)b * table_stride + (j0 / PAGE) % ring_pages];
      kpage = pages + (size_t)page * page_elems + (size_t)kvh * head_elems;
    }
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int c = tid + 256 * i;
      {   // keys: chunk c = (row, 8 columns)
        const int row = c / CH, col = (c % CH) * 8, j = j0 + row;
        bf16x8 kv = z8();
        if (col < d && j < seq_end) {
          if (j < cached) kv = ld8(kpage + (size_t)row * d + col);
          else kv = ld8(k_new + ((size_t)(row0 + j - cached) * nkv + kvh) * d + col);
        }
        kfetch[i] = kv;
      }
      {   // values: chunk c = (dv, 8 keys); columns past the sequence's end were never written
        const int dv = c / (PF_BN / 8), kc = (c % (PF_BN / 8)) * 8;
        bf16x8 vv = z8();
        if (dv < d) {
          bf16x8 cv = z8(), nv = z8();
          if (has_cached) cv = ld8(kpage + (size_t)nkv * head_elems + (size_t)dv * PAGE + kc);
          if (has_new) nv = ld8(vt_head + (size_t)dv * vt_cols + (j0 - j_base) + kc);
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const int j = j0 + kc + e;
            vv[e] = (j < cached) ? cv[e] : ((j < seq_end) ? nv[e] : (bf16)0.f);
          }
        }
        vfetch[i] = vv;
      }
    }
  };
  auto stash = [&]() {
#pragma unroll
    for (int i = 0; i < PT; ++i) {
      const int c = tid + 256 * i;
      const int row = c / CH, col = (c % CH) * 8;
      *reinterpret_cast<bf16x8*>(&Ks[row * KLD + col]) = kfetch[i];
      const int dv = c / (PF_BN / 8), kc = (c % (PF_BN / 8)) * 8;
      bf16x4 lo4, hi4;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        lo4[e] = vfetch[i][e];
        hi4[e] = vfetch[i][4 + e];
      }
      *reinterpret_cast<bf16x4*>(&Vt[dv * PF_VLD + kc]) = lo4;
      *reinterpret_cast<bf16x4*>(&Vt[dv * PF_VLD + kc + 4]) = hi4;
    }
  };

  if (jt_first <= jt_last) fetch(jt_first * PF_BN);
  for (int jt = jt_first; jt <= jt_last; ++jt) {
    const int j0 = jt * PF_BN;
    __syncthreads();                  // the previous tile has been worked on
    stash();
    __syncthreads();
    if (jt < jt_last) fetch((jt + 1) * PF_BN);
    // does any query of this wave see any key of this tile?
    if (pw_lo > p_hi || j0 > pw_hi || (window > 0 && j0 + PF_BN - 1 <= pw_lo - window)) continue;

    f32x16 s[2];
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) s[nb][r] = 0.f;
    __builtin_amdgcn_s_setprio(1);       // see above: first among the SIMD's waves while it feeds the matrix cores
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int nb = 0; nb < 2; ++nb) {
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(&Ks[(nb * 32 + l32) * KLD + kb * 16 + 8 * half]);
        s[nb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qreg[kb], s[nb], 0, 0, 0);
      }
    __builtin_amdgcn_s_setprio(0);
    // s[nb][r] = k.q of key j0 + 32 nb + 8 (r/4) + 4 half + r%4 with this lane's query.
    // Only tiles that cross the wave's causal edge, the window's edge or the rows' end need masks.
    const bool edge = j0 + PF_BN - 1 > pw_lo || (window > 0 && j0 <= pw_hi - window) ||
                      pw_lo + 31 > pw_hi;
    if (edge) {
#pragma unroll
      for (int nb = 0; nb < 2; ++nb)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int j = j0 + nb * 32 + 8 * (r / 4) + 4 * half + (r % 4);
          const bool ok = q_ok && j <= p_me && (window == 0 || j > p_me - window);
          s[nb][r] = ok ? s[nb][r] : -INFINITY;
        }
    }
    float tmax = -INFINITY;
#pragma unroll
    for (int nb = 0; nb < 2; ++nb)
#pragma unroll
      for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, s[nb][r]);
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m, tmax * scale);          // scale > 0: the maximum of the scaled scores
    const float m_use = (m_new == -INFINITY) ? 0.f : m_new;
    if (__ballot(m_new != m) != 0ull) {                  // the running maximum moved in some lane
      const float alpha = __expf(m - m_use);
      l *= alpha;
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[vb][r] *= alpha;
      m = m_new;
    }
    // p = exp(s * scale - m) = 2^(s * c1 + c0)
    const float c1 = scale * 1.44269504088896f, c0 = -m_use * 1.44269504088896f;
    float psum = 0.f;
    bf16x8 pb[2][2];
    // probability e of the tile's 32 (e = 16 nb + r), in the order of the sum
    auto soft = [&](int e) {
      const int nb = e / 16, r = e % 16;
      const float pv = __builtin_amdgcn_exp2f(fmaf(s[nb][r], c1, c0));
      psum += pv;
      pb[nb][r / 8][r % 8] = (bf16)pv;
    };
    // values of block vb against probabilities 8 qd .. 8 qd + 7 (qd = 2 nb + mm): these are keys
    // kk + {0..3} and kk + 8 + {0..3}, kk = 32 nb + 16 mm + 4 half
    auto vfrag = [&](int qd, int vb) {
      const bf16* vrow = &Vt[(vb * 32 + l32) * PF_VLD + (qd / 2) * 32 + 16 * (qd % 2) + 4 * half];
      const bf16x4 lo4 = ld4(vrow), hi4 = ld4(vrow + 8);
      bf16x8 a;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        a[e] = lo4[e];
        a[4 + e] = hi4[e];
      }
      return a;
    };
    // The second product goes quarter by quarter of the tile's keys, and while the matrix cores
    // work on one quarter the vector unit makes the probabilities of the next: the order below is
    // pinned, one MFMA and its share of the next quarter's eight probabilities at a time.
#pragma unroll
    for (int e = 0; e < 8; ++e) soft(e);
    __builtin_amdgcn_s_setprio(1);
#pragma unroll
    for (int qd = 0; qd < 4; ++qd) {
#pragma unroll
      for (int vb = 0; vb < VB; ++vb) {
        o[vb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vfrag(qd, vb), pb[qd / 2][qd % 2], o[vb], 0, 0, 0);
        if (qd < 3) {
#pragma unroll
          for (int e = (8 * vb) / VB; e < (8 * (vb + 1)) / VB; ++e) soft(8 * (qd + 1) + e);
        }
      }
    }
    __builtin_amdgcn_s_setprio(0);
    psum += __shfl_xor(psum, 32, WAVE);
    l += psum;
  }
  if (ways != 0) {
    // a run of a block's keys: running maximum, sum and unscaled O of every row, for the merge
    if (q_ok) {
      float* pp = part + (((size_t)(row0 + qr) * nq + h) * part_ways + slot) * (size_t)(d + PF_PART_HEAD);
      if (half == 0) {
        pp[0] = m;
        pp[1] = l;
      }
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {                 // four values in a row: 16 bytes a store
          const int dv = vb * 32 + 8 * g4 + 4 * half;
          if (dv < d)
            *reinterpret_cast<f32x4*>(pp + PF_PART_HEAD + dv) =
                f32x4{o[vb][4 * g4], o[vb][4 * g4 + 1], o[vb][4 * g4 + 2], o[vb][4 * g4 + 3]};
        }
    }
    return;
  }
  if (q_ok) {
    bf16* op = out + ((size_t)(row0 + qr) * nq + h) * d;
    const float inv = 1.0f / l;
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int dv = vb * 32 + 8 * (r / 4) + 4 * half + (r % 4);
        if (dv < d) op[dv] = (bf16)(o[vb][r] * inv);
      }
  }
}

// The runs of a block whose keys were cut between workgroups (see `items` above) become its rows of the
// output: common maximum, weighted sums, in the order of the runs.  A workgroup takes PF_MERGE values of
// one (block, head): blockIdx.x = block * pieces + piece.  blocks: (sequence, block, ways, -) each.
constexpr int PF_MERGE = 1024, PF_MAX_WAYS = 8;

__global__ void __launch_bounds__(256)
attn_prefill_merge_kernel(const float* __restrict__ part, int part_ways, const int4* __restrict__ blocks,
                          const int* __restrict__ cu_seqlens, int pieces, int nq, int d, bf16* __restrict__ out) {
  const int4 bt = blocks[blockIdx.x / pieces];
  const int piece = blockIdx.x % pieces, h = blockIdx.y, ways = bt.z;
  const int row0 = cu_seqlens[bt.x] + bt.y * PF_BM;
  const int rows = min(PF_BM, cu_seqlens[bt.x + 1] - row0);
  const size_t stride = (size_t)(d + PF_PART_HEAD);
#pragma unroll
  for (int i = 0; i < PF_MERGE / 256; ++i) {
    const int e = piece * PF_MERGE + i * 256 + threadIdx.x;
    const int r = e / d, dv = e % d;
    if (r >= rows) continue;
    const float* p = part + (((size_t)(row0 + r) * nq + h) * part_ways) * stride;
    float ms[PF_MAX_WAYS], mm = -INFINITY;
#pragma unroll
    for (int w = 0; w < PF_MAX_WAYS; ++w) {
      ms[w] = (w < ways) ? p[w * stride] : -INFINITY;
      mm = fmaxf(mm, ms[w]);
    }
    float l = 0.f, acc = 0.f;
#pragma unroll
    for (int w = 0; w < PF_MAX_WAYS; ++w) {
      if (w < ways && ms[w] != -INFINITY) {
        const float f = __expf(ms[w] - mm);
        l += p[w * stride + 1] * f;
        acc += p[w * stride + PF_PART_HEAD + dv] * f;
      }
    }
    out[((size_t)(row0 + r) * nq + h) * d + dv] = (bf16)(acc / l);
  }
}

// ------------------------------------------------------------------- decode --
// One query token per sequence, everything in the pages.  A workgroup owns one
// (sequence, KV head, group of up to 16 query heads, split); its 4 waves take
// the split's pages in turn, each page as two groups of 32 keys read straight
// from global memory into MFMA operands.  Per wave: running (max, sum, O^T);
// the waves meet in LDS and the workgroup writes one partial per head:
// part[(b, h, split)] = (max, sum, O[d]), merged by attn_decode_combine; with one split the
// result is written at once.
constexpr int DC_WAVES = 4;

template <int DPAD, bool LEAN>   // DPAD: multiple of 32; LEAN: d == DPAD, loads without guards at fixed offsets
__global__ void __launch_bounds__(DC_WAVES * 64)
attn_decode_kernel(const bf16* __restrict__ q, const bf16* __restrict__ pages,
                   const int* __restrict__ table, int table_stride, int ring_pages,
                   const int* __restrict__ row_pos, int nq, int nkv, int d, int window, float scale,
                   int n_splits, int head_groups, float* __restrict__ part, bf16* __restrict__ out) {
  constexpr int KB = DPAD / 32, VB = DPAD / 16;
  constexpr bool APART = DPAD <= 128;        // room in LDS for every wave's scaled O^T: one barrier instead of four
  __shared__ float red_o[(APART ? DC_WAVES : 1) * VB * 4 * 64];
  __shared__ float red_ml[DC_WAVES][2][16];
  const int g = nq / nkv;
  const int hg = blockIdx.x % head_groups;
  const int kvh = (blockIdx.x / head_groups) % nkv;
  const int b = blockIdx.x / (head_groups * nkv);
  const int split = blockIdx.y;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, li = lane % 16, kg = lane / 16;
  const int hl = hg * 16 + li;                        // head within the KV group (column of S^T)
  const int h = kvh * g + min(hl, g - 1);
  const int p = row_pos[b];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int pg_lo = lo / PAGE, pg_hi = p / PAGE, n_pg = pg_hi - pg_lo + 1;
  // [my_lo, my_hi): the pages in shares that differ by one at most (65 pages in 8 splits are 8 or 9 each,
  // not seven times 9 and once 2: the compute units then end together)
  const int my_lo = pg_lo + (int)((long long)split * n_pg / n_splits);
  const int my_hi = pg_lo + (int)((long long)(split + 1) * n_pg / n_splits);
  const size_t head_elems = (size_t)PAGE * d, page_elems = 2 * (size_t)nkv * head_elems;

  bf16x8 qreg[KB];
  {
    const bf16* qp = q + ((size_t)b * nq + h) * d;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) {
      const int k = kb * 32 + 8 * kg;
      qreg[kb] = (k + 8 <= d) ? ld8(qp + k) : z8();
    }
  }
  f32x4 o[VB];
#pragma unroll
  for (int vb = 0; vb < VB; ++vb) o[vb] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

  // the split's groups of 32 keys go round the waves; a wave's pages are two apart, and the id of
  // its next page is looked up while it works on this one
  static_assert(DC_WAVES == 4, "a wave's groups are two pages apart");
  const int* trow = table + (size_t)b * table_stride;
  const int gi0 = 2 * my_lo + wave;
  int ring = (gi0 / 2) % ring_pages;
  int page_nxt = gi0 < 2 * my_hi ? trow[ring] : 0;
  for (int gi = gi0; gi < 2 * my_hi; gi += DC_WAVES) {
    const int pg = gi / 2, grp = gi % 2;
    const int page = page_nxt;
    ring += 2;
    if (ring >= ring_pages) ring -= ring_pages;
    if (ring >= ring_pages) ring -= ring_pages;          // (a ring of one page)
    if (gi + DC_WAVES < 2 * my_hi) page_nxt = trow[ring];
    const bf16* kbase = pages + (size_t)page * page_elems + (size_t)kvh * head_elems;
    const bf16* vbase = kbase + (size_t)nkv * head_elems;
    {
      const int j0 = pg * PAGE + grp * 32;
      if (j0 > p || j0 + 31 < lo) continue;
      // block bs holds keys j0 + 8 (i/4) + 4 bs + i%4 in its rows i: then a lane's 8 scores of
      // the two blocks are 8 consecutive keys, j0 + 8 kg .. + 7
      // all loads of the group first: keys (two blocks) and values
      bf16x8 kreg[2][KB], vreg[VB];
      if constexpr (LEAN) {
        // a uniform base for the group plus this lane's offset in bytes; the rest are constants
        const bf16* kgrp = kbase + grp * 32 * DPAD;
        const bf16* vgrp = vbase + grp * 32;
        unsigned k_lane = ((8 * (li / 4) + (li % 4)) * DPAD + 8 * kg) * 2, v_lane = (li * PAGE + 8 * kg) * 2;
        asm volatile("" : "+v"(k_lane), "+v"(v_lane));     // (worked out here, not kept in 24 registers)
#pragma unroll
        for (int bs = 0; bs < 2; ++bs)
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) kreg[bs][kb] = ld8_at(kgrp, k_lane + (bs * 4 * DPAD + kb * 32) * 2);
#pragma unroll
        for (int vb = 0; vb < VB; ++vb) vreg[vb] = ld8_at(vgrp, v_lane + vb * 16 * PAGE * 2);
      } else {
#pragma unroll
        for (int bs = 0; bs < 2; ++bs) {
          const bf16* krow = kbase + (size_t)(grp * 32 + 8 * (li / 4) + 4 * bs + (li % 4)) * d;
#pragma unroll
          for (int kb = 0; kb < KB; ++kb) {
            const int k = kb * 32 + 8 * kg;
            kreg[bs][kb] = (k + 8 <= d) ? ld8(krow + k) : z8();
          }
        }
#pragma unroll
        for (int vb = 0; vb < VB; ++vb) {
          const int dv = vb * 16 + li;
          vreg[vb] = (dv < d) ? ld8(vbase + (size_t)dv * PAGE + grp * 32 + 8 * kg) : z8();
        }
      }
      f32x4 s[2];
#pragma unroll
      for (int bs = 0; bs < 2; ++bs) {
        s[bs] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          s[bs] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[bs][kb], qreg[kb], s[bs], 0, 0, 0);
      }
      float sv[8];
      float tmax = -INFINITY;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = j0 + 8 * kg + e;
        const bool ok = j <= p && j >= lo;
        sv[e] = ok ? s[e / 4][e % 4] * scale : -INFINITY;
        tmax = fmaxf(tmax, sv[e]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
      const float m_new = fmaxf(m, tmax);              // finite: the group holds a visible key
      const float alpha = __expf(m - m_new);
      float psum = 0.f;
      bf16x8 pb;
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float pv = __expf(sv[e] - m_new);
        psum += pv;
        pb[e] = (bf16)pv;
      }
      psum += __shfl_xor(psum, 16, WAVE);
      psum += __shfl_xor(psum, 32, WAVE);
      l = l * alpha + psum;
      m = m_new;
      // O^T[dv][head] += V^T[dv][keys] P^T[keys][head]; values lie as [d][PAGE] in the page
      if (j0 + 31 > p) {           // rows past the sequence's end were never written: 0 * garbage
        typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
        u32x4 keep;                // this lane's 8 keys are 4 pairs of 16 bits
#pragma unroll
        for (int w2 = 0; w2 < 4; ++w2)
          keep[w2] = (j0 + 8 * kg + 2 * w2 <= p ? 0x0000ffffu : 0u) | (j0 + 8 * kg + 2 * w2 + 1 <= p ? 0xffff0000u : 0u);
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
          vreg[vb] = __builtin_bit_cast(bf16x8, __builtin_bit_cast(u32x4, vreg[vb]) & keep);
      }
      if (__ballot(alpha != 1.0f) != 0ull) {      // the running maximum moved in some lane
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
#pragma unroll
          for (int r = 0; r < 4; ++r) o[vb][r] *= alpha;
      }
#pragma unroll
      for (int vb = 0; vb < VB; ++vb) o[vb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vreg[vb], pb, o[vb], 0, 0, 0);
    }
  }
  // o[vb][r] = O[dv = 16 vb + 4 kg + r][head li]; m, l are per head li (equal in the 4 kg lanes).
  // Merge the waves: common maximum, then wave after wave adds its scaled share in LDS.
  if (kg == 0) {
    red_ml[wave][0][li] = m;
    red_ml[wave][1][li] = l;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < DC_WAVES; ++w) mm = fmaxf(mm, red_ml[w][0][li]);
  const float f = (m == -INFINITY) ? 0.f : __expf(m - mm);
  if constexpr (APART) {
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
#pragma unroll
      for (int r = 0; r < 4; ++r) red_o[wave * (VB * 4 * 64) + (vb * 4 + r) * 64 + lane] = o[vb][r] * f;
    __syncthreads();
  } else {
    for (int w = 0; w < DC_WAVES; ++w) {
      if (wave == w) {
#pragma unroll
        for (int vb = 0; vb < VB; ++vb)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            float* dst = &red_o[(vb * 4 + r) * 64 + lane];
            *dst = (w == 0) ? o[vb][r] * f : *dst + o[vb][r] * f;
          }
      }
      __syncthreads();
    }
  }
  // the waves' shares in their order (the sum that the one-after-the-other way makes)
  auto o_sum = [&](int idx) {
    float v = red_o[idx];
    if constexpr (APART) {
#pragma unroll
      for (int w = 1; w < DC_WAVES; ++w) v += red_o[w * (VB * 4 * 64) + idx];
    }
    return v;
  };
  for (int e = threadIdx.x; e < 16 * DPAD; e += DC_WAVES * 64) {
    const int hd = e / DPAD, dv = e % DPAD;
    if (hg * 16 + hd >= g || dv >= d) continue;
    float mh = -INFINITY;
#pragma unroll
    for (int w = 0; w < DC_WAVES; ++w) mh = fmaxf(mh, red_ml[w][0][hd]);
    float ll = 0.f;
#pragma unroll
    for (int w = 0; w < DC_WAVES; ++w) {
      const float mw = red_ml[w][0][hd];
      ll += (mw == -INFINITY) ? 0.f : red_ml[w][1][hd] * __expf(mw - mh);
    }
    const int idx = ((dv / 16) * 4 + (dv % 4)) * 64 + ((dv % 16) / 4) * 16 + hd;
    const size_t bh = (size_t)b * nq + kvh * g + hg * 16 + hd;
    if (n_splits == 1) {                                // nothing to merge with
      out[bh * d + dv] = (bf16)(o_sum(idx) / ll);
      continue;
    }
    float* dst = part + (bh * n_splits + split) * (d + 2);
    dst[2 + dv] = o_sum(idx);
    if (dv == 0) {
      dst[0] = mh;
      dst[1] = ll;
    }
  }
}

// ------------------------------------------------------ decode, through LDS --
// The same step for head sizes 64, 128 and 256, with the pages going from memory straight into a
// ring of stages in LDS (global_load_lds, 16 bytes a lane), several pages ahead of the matrix cores.
// A stage is one page of one KV head: its keys [64][d] and its values [d][64], each one run of
// memory, so that every load instruction takes 1 KB of whole lines, which may then be marked
// non-temporal (a plain read gains a seventh from that, csrc/measure/ceilings.hip; with the loads of
// attn_decode_kernel, which take a line in halves, it loses).  The workgroup's four waves take 16
// keys of the page each: S^T = K Q^T (16x16x32), softmax with the wave's own running maximum,
// O^T += V^T P (16x16x16: the scores leave the first product in the second's operand layout).
// In LDS the 16-byte chunk c of a row lies at a swizzled place, so that the operand reads of 16
// lanes fall on 16 groups of banks.  The compiler places no waits for such loads: the waves count
// them (vmcnt) and meet at one barrier a page.  Partial results as attn_decode_kernel writes them.
typedef short s16x4 __attribute__((ext_vector_type(4)));

template <int N> __device__ __forceinline__ void wait_page_loads_but() {     // until at most N loads are under way
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

template <int D, int NS>
__global__ void __launch_bounds__(DC_WAVES * 64)
attn_decode_ring_kernel(const bf16* __restrict__ q, const bf16* __restrict__ pages,
                        const int* __restrict__ table, int table_stride, int ring_pages,
                        const int* __restrict__ row_pos, int nq, int nkv, int window, float scale,
                        int n_splits, int head_groups, float* __restrict__ part, bf16* __restrict__ out) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char dr_smem[];
  constexpr int KB = D / 32, VB = D / 16;
  constexpr int K_BYTES = PAGE * D * 2, STAGE = 2 * K_BYTES;   // keys, then values, as many bytes each
  constexpr int K_CPR = D / 8;                        // 16-byte chunks of a key's row
  constexpr int K_RPI = 64 / K_CPR;                   // keys a load instruction takes
  constexpr int K_INSTR = PAGE / K_RPI, V_INSTR = D / 8;       // (a load of values takes 8 rows of 128 bytes)
  constexpr int LPS = (K_INSTR + V_INSTR) / DC_WAVES; // loads a wave issues for a page
  static_assert(D == 64 || D == 128 || D == 256, "head sizes whose rows have a power of two of chunks");
  static_assert((K_INSTR + V_INSTR) % DC_WAVES == 0 && (NS - 2) * LPS <= 63 && NS >= 2, "loads a wave counts");
  const int g = nq / nkv;
  const int hg = blockIdx.x % head_groups;
  const int kvh = (blockIdx.x / head_groups) % nkv;
  const int b = blockIdx.x / (head_groups * nkv);
  const int split = blockIdx.y;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, li = lane % 16, kg = lane / 16;
  const int hl = hg * 16 + li;
  const int h = kvh * g + min(hl, g - 1);
  const int p = row_pos[b];
  const int lo = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int pg_lo = lo / PAGE, pg_hi = p / PAGE, n_pg = pg_hi - pg_lo + 1;
  const int my_lo = pg_lo + (int)((long long)split * n_pg / n_splits);
  const int my_hi = pg_lo + (int)((long long)(split + 1) * n_pg / n_splits);
  const int n_st = my_hi - my_lo;                     // this split's pages: the stages
  const size_t head_elems = (size_t)PAGE * D, page_elems = 2 * (size_t)nkv * head_elems;
  auto kkey = [](int r) { return K_CPR >= 16 ? r % 16 : (r / 2) % 8; };   // swizzle of a key's row
  auto vkey = [](int r) { return (r / 2) % 8; };                          // ... of a row of values (128 bytes)

  bf16x8 qreg[KB];
  {
    const bf16* qp = q + ((size_t)b * nq + h) * D;
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) qreg[kb] = ld8(qp + kb * 32 + 8 * kg);
  }
  // this lane's share of a page's loads: where in the page's keys or values (bytes from the KV head's keys)
  unsigned src_off[LPS];
#pragma unroll
  for (int x = 0; x < LPS; ++x) {
    const int i = wave + DC_WAVES * x;
    if (i < K_INSTR) {
      const int r = i * K_RPI + lane / K_CPR, place = lane % K_CPR;
      src_off[x] = (unsigned)(r * (2 * D) + ((place ^ kkey(r)) * 16));
    } else {
      const int r = (i - K_INSTR) * 8 + lane / 8, place = lane % 8;
      src_off[x] = (unsigned)((size_t)nkv * head_elems * 2 + r * 128 + ((place ^ vkey(r)) * 16));
    }
  }
  // the page ids of this split's stages lie in LDS behind the ring (a load from memory inside the loop
  // would make the compiler wait for every load under way, the pages' among them)
  int* ids = reinterpret_cast<int*>(dr_smem + NS * STAGE);
  {
    const int* trow = table + (size_t)b * table_stride;
    for (int st = threadIdx.x; st < n_st; st += DC_WAVES * 64) ids[st] = trow[(my_lo + st) % ring_pages];
  }
  __syncthreads();
  auto issue = [&](int st) {
    const int page = __builtin_amdgcn_readfirstlane(ids[st]);
    const char* base = reinterpret_cast<const char*>(pages + (size_t)page * page_elems + (size_t)kvh * head_elems);
    unsigned char* slot = dr_smem + (st % NS) * STAGE;
#pragma unroll
    for (int x = 0; x < LPS; ++x)
      __builtin_amdgcn_global_load_lds((const TL_AS1 void*)(base + src_off[x]),
                                       (TL_AS3 void*)(slot + (wave + DC_WAVES * x) * 1024), 16, 0, 2);
  };

  f32x4 o[VB];
#pragma unroll
  for (int vb = 0; vb < VB; ++vb) o[vb] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;

#pragma unroll
  for (int st = 0; st < NS - 1; ++st)
    if (st < n_st) issue(st);
  const int krow = 16 * wave + li;                    // this lane's key of a page (row of the first product)
  const int kk = kkey(krow), vk = vkey(li);           // (16 vb + li has li's swizzle: 16 rows are a whole period)
  for (int st = 0; st < n_st; ++st) {
    if (n_st - 1 - st >= NS - 2) wait_page_loads_but<(NS - 2) * LPS>();
    else wait_page_loads_but<0>();
    __builtin_amdgcn_s_barrier();                     // the page is there for all; everyone has left the one before
    if (st + NS - 1 < n_st) issue(st + NS - 1);
    const int j0 = (my_lo + st) * PAGE + 16 * wave;   // this wave's 16 keys
    if (j0 > p || j0 + 15 < lo) continue;             // none of them visible
    const unsigned char* slot = dr_smem + (st % NS) * STAGE;
    bf16x8 kreg[KB];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
      kreg[kb] = *reinterpret_cast<const bf16x8*>(slot + krow * (2 * D) + (((4 * kb + kg) ^ kk) * 16));
    s16x4 vreg[VB];
#pragma unroll
    for (int vb = 0; vb < VB; ++vb)
      vreg[vb] = *reinterpret_cast<const s16x4*>(slot + K_BYTES + (16 * vb + li) * 128 +
                                                 (((2 * wave + kg / 2) ^ vk) * 16) + 8 * (kg % 2));
    f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kb = 0; kb < KB; ++kb) s = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kreg[kb], qreg[kb], s, 0, 0, 0);
    // s[r]: key j0 + 4 kg + r against head li
    float sv[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int j = j0 + 4 * kg + r;
      sv[r] = (j <= p && j >= lo) ? s[r] * scale : -INFINITY;
      tmax = fmaxf(tmax, sv[r]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, WAVE));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
    const float m_new = fmaxf(m, tmax);               // finite: one of the 16 keys is visible
    const float alpha = __expf(m - m_new);
    float psum = 0.f;
    bf16x4 pb;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const float pv = __expf(sv[r] - m_new);
      psum += pv;
      pb[r] = (bf16)pv;
    }
    psum += __shfl_xor(psum, 16, WAVE);
    psum += __shfl_xor(psum, 32, WAVE);
    l = l * alpha + psum;
    m = m_new;
    if (j0 + 15 > p) {                                // rows past the sequence's end were never written: 0 * garbage
      typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
      u32x2 keep;
#pragma unroll
      for (int w2 = 0; w2 < 2; ++w2)
        keep[w2] = (j0 + 4 * kg + 2 * w2 <= p ? 0x0000ffffu : 0u) | (j0 + 4 * kg + 2 * w2 + 1 <= p ? 0xffff0000u : 0u);
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
        vreg[vb] = __builtin_bit_cast(s16x4, __builtin_bit_cast(u32x2, vreg[vb]) & keep);
    }
    if (__ballot(alpha != 1.0f) != 0ull) {
#pragma unroll
      for (int vb = 0; vb < VB; ++vb)
#pragma unroll
        for (int r = 0; r < 4; ++r) o[vb][r] *= alpha;
    }
    const s16x4 pbits = __builtin_bit_cast(s16x4, pb);
#pragma unroll
    for (int vb = 0; vb < VB; ++vb) o[vb] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(vreg[vb], pbits, o[vb], 0, 0, 0);
  }
  // o[vb][r] = O[dv = 16 vb + 4 kg + r][head li]; m, l are per head li (equal in the 4 kg lanes).
  // Merge the waves in the ring's memory: common maximum, then every wave's scaled share.
  __builtin_amdgcn_s_barrier();                       // everyone has left the last page
  float* red_o = reinterpret_cast<float*>(dr_smem);                              // [waves][VB * 4 * 64]
  float* red_ml = red_o + DC_WAVES * VB * 4 * 64;                               // [waves][2][16]
  if (kg == 0) {
    red_ml[(wave * 2 + 0) * 16 + li] = m;
    red_ml[(wave * 2 + 1) * 16 + li] = l;
  }
  __syncthreads();
  float mm = -INFINITY;
#pragma unroll
  for (int w = 0; w < DC_WAVES; ++w) mm = fmaxf(mm, red_ml[(w * 2) * 16 + li]);
  const float f = (m == -INFINITY) ? 0.f : __expf(m - mm);
#pragma unroll
  for (int vb = 0; vb < VB; ++vb)
#pragma unroll
    for (int r = 0; r < 4; ++r) red_o[wave * (VB * 4 * 64) + (vb * 4 + r) * 64 + lane] = o[vb][r] * f;
  __syncthreads();
  for (int e = threadIdx.x; e < 16 * D; e += DC_WAVES * 64) {
    const int hd = e / D, dv = e % D;
    if (hg * 16 + hd >= g) continue;
    float mh = -INFINITY;
#pragma unroll
    for (int w = 0; w < DC_WAVES; ++w) mh = fmaxf(mh, red_ml[(w * 2) * 16 + hd]);
    float ll = 0.f;
#pragma unroll
    for (int w = 0; w < DC_WAVES; ++w) {
      const float mw = red_ml[(w * 2) * 16 + hd];
      ll += (mw == -INFINITY) ? 0.f : red_ml[(w * 2 + 1) * 16 + hd] * __expf(mw - mh);
    }
    const int idx = ((dv / 16) * 4 + (dv % 4)) * 64 + ((dv % 16) / 4) * 16 + hd;
    float osum = red_o[idx];
#pragma unroll
    for (int w = 1; w < DC_WAVES; ++w) osum += red_o[w * (VB * 4 * 64) + idx];
    const size_t bh = (size_t)b * nq + kvh * g + hg * 16 + hd;
    if (n_splits == 1) {
      out[bh * D + dv] = (bf16)(osum / ll);
      continue;
    }
    float* dst = part + (bh * n_splits + split) * (D + 2);
    dst[2 + dv] = osum;
    if (dv == 0) {
      dst[0] = mh;
      dst[1] = ll;
    }
  }
}

// Merge the splits of one (sequence, head): common maximum, weighted sums, in the order of the
// splits.  (A second kernel and not the last workgroup of the first: what other XCDs wrote is
// only sure to be seen across a kernel boundary or after a device-wide fence, and that fence
// writes back and invalidates the XCD's L2.  Measured with the last workgroup merging behind a
// counter: one fence a workgroup makes a step of 32 layers at batch 8 4.7 ms instead of 4.0, one
// a thread 6.3.)
// One wave per (row, head).  Splits are taken 8 at a time with all their loads (maxima, sums and
// this lane's elements) issued together, so that a usual split count costs one trip to memory;
// chunks merge by the running-maximum rule.
__global__ void __launch_bounds__(64)
attn_decode_combine_kernel(const float* __restrict__ part, int n_splits, int d, bf16* __restrict__ out) {
  constexpr int CH = 8, MAXV = 4;                      // d <= 256: at most 4 elements a lane
  const size_t bh = blockIdx.x;
  const float* src = part + bh * n_splits * (d + 2);
  const int lane = threadIdx.x;
  const size_t stride = d + 2;
  float mm = -INFINITY, ll = 0.f, acc[MAXV];
#pragma unroll
  for (int v = 0; v < MAXV; ++v) acc[v] = 0.f;
  for (int s0 = 0; s0 < n_splits; s0 += CH) {
    float ms[CH], ls[CH], vs[CH][MAXV];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const bool ok = s0 + c < n_splits;
      const float* p = src + (size_t)(ok ? s0 + c : s0) * stride;
      ms[c] = ok ? p[0] : -INFINITY;
      ls[c] = p[1];
#pragma unroll
      for (int v = 0; v < MAXV; ++v) vs[c][v] = (lane + 64 * v < d) ? p[2 + lane + 64 * v] : 0.f;
    }
    float mc = mm;
#pragma unroll
    for (int c = 0; c < CH; ++c) mc = fmaxf(mc, ms[c]);
    if (mc == -INFINITY) continue;                     // nothing visible so far
    const float keep = (mm == -INFINITY) ? 0.f : __expf(mm - mc);
    ll *= keep;
#pragma unroll
    for (int v = 0; v < MAXV; ++v) acc[v] *= keep;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const float f = (ms[c] == -INFINITY) ? 0.f : __expf(ms[c] - mc);
      ll += ls[c] * f;
#pragma unroll
      for (int v = 0; v < MAXV; ++v) acc[v] += vs[c][v] * f;
    }
    mm = mc;
  }
#pragma unroll
  for (int v = 0; v < MAXV; ++v)
    if (lane + 64 * v < d) out[bh * d + lane + 64 * v] = (bf16)(acc[v] / ll);
}

template <int DPAD>
static int launch_prefill(const bf16* q, const bf16* k_new, const bf16* vt_new, int vt_cols,
                          const int* tile_off, const bf16* pages, const int* table, int table_stride, int ring_pages, const int* row_pos,
                          const int* cu_seqlens, const int* n_cached, int B, int n_tiles, int nq, int nkv,
                          int d, int window, float scale, bf16* out, const int4* items, const int4* cut_blocks,
                          int n_cut, float* part, int part_ways, hipStream_t st) {
  const size_t smem = ((size_t)PF_BN * (DPAD + 8) + (size_t)DPAD * PF_VLD) * sizeof(bf16);
  constexpr bool can_lean = 256 % (DPAD / 8) == 0;
  if (smem > 48 * 1024) {
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_kernel<DPAD, false>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if constexpr (can_lean)
        if (e == hipSuccess)
          e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_prefill_kernel<DPAD, true>),
                                  hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem);
      if (e != hipSuccess) {
        set_error("attn_prefill: cannot have %zu bytes of LDS: %s", smem, hipGetErrorString(e));
        return 2;
      }
      raised = true;
    }
  }
  const long long total = (long long)n_tiles * nq;
  if (total > 2147483000LL) {
    set_error("attn_prefill: %lld (head, block of rows) pairs are too many", total);
    return 1;
  }
  const unsigned grid = (unsigned)total;
  if (can_lean && d == DPAD)
    attn_prefill_kernel<DPAD, can_lean><<<grid, 256, smem, st>>>(q, k_new, vt_new, vt_cols, tile_off, pages, table,
                                                             table_stride, ring_pages, row_pos, cu_seqlens,
                                                             n_cached, B, n_tiles, nq, nkv, d, window, scale, out,
                                                             items, part, part_ways);
  else
    attn_prefill_kernel<DPAD, false><<<grid, 256, smem, st>>>(q, k_new, vt_new, vt_cols, tile_off, pages, table,
                                                              table_stride, ring_pages, row_pos, cu_seqlens,
                                                              n_cached, B, n_tiles, nq, nkv, d, window, scale, out,
                                                              items, part, part_ways);
  TL_LAUNCH_CHECK("attn_prefill");
  if (n_cut > 0) {
    const int pieces = (PF_BM * d + PF_MERGE - 1) / PF_MERGE;
    attn_prefill_merge_kernel<<<dim3(n_cut * pieces, nq), 256, 0, st>>>(part, part_ways, cut_blocks, cu_seqlens, pieces,
                                                                        nq, d, out);
    TL_LAUNCH_CHECK("attn_prefill_merge");
  }
  return 0;
}

// which decode kernel serves head sizes 64, 128 and 256 (tests and measurements may switch)
static bool decode_through_lds = true;
constexpr int DR_MAX_PAGES = 2048;      // most pages of a sequence that the kernel through LDS keeps the ids of (8 KB)

template <int DPAD>
static int launch_decode(const bf16* q, const bf16* pages, const int* table, int table_stride,
                         int ring_pages, const int* row_pos, int B, int nq, int nkv, int d, int window,
                         float scale, int n_splits, float* part, bf16* out, hipStream_t st) {
  const int g = nq / nkv, head_groups = (g + 15) / 16;
  dim3 grid(B * nkv * head_groups, n_splits);
  if constexpr (DPAD == 64 || DPAD == 128 || DPAD == 256) {
    if (d == DPAD && decode_through_lds && table_stride <= DR_MAX_PAGES) {
      constexpr int NS = DPAD == 64 ? 4 : 2;         // 64 KB of LDS, two workgroups a compute unit; heads of 256: 128 KB, one
      constexpr int LDS = NS * PAGE * DPAD * 4 + DR_MAX_PAGES * 4;              // the ring, and the page ids of a split
      static bool raised = false;
      if (!raised) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&attn_decode_ring_kernel<DPAD, NS>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, LDS);
        if (e != hipSuccess) {
          set_error("attn_decode: cannot have %d bytes of LDS: %s", LDS, hipGetErrorString(e));
          return 2;
        }
        raised = true;
      }
      attn_decode_ring_kernel<DPAD, NS><<<grid, DC_WAVES * 64, LDS, st>>>(q, pages, table, table_stride, ring_pages,
                                                                          row_pos, nq, nkv, window, scale, n_splits,
                                                                          head_groups, part, out);
      TL_LAUNCH_CHECK("attn_decode_ring");
      if (n_splits > 1) {
        attn_decode_combine_kernel<<<B * nq, 64, 0, st>>>(part, n_splits, d, out);
        TL_LAUNCH_CHECK("attn_decode_combine");
      }
      return 0;
    }
  }
  if (d == DPAD)
    attn_decode_kernel<DPAD, true><<<grid, DC_WAVES * 64, 0, st>>>(q, pages, table, table_stride, ring_pages,
                                                                    row_pos, nq, nkv, d, window, scale, n_splits,
                                                                    head_groups, part, out);
  else
    attn_decode_kernel<DPAD, false><<<grid, DC_WAVES * 64, 0, st>>>(q, pages, table, table_stride, ring_pages,
                                                                     row_pos, nq, nkv, d, window, scale, n_splits,
                                                                     head_groups, part, out);
  TL_LAUNCH_CHECK("attn_decode");
  if (n_splits > 1) {
    attn_decode_combine_kernel<<<B * nq, 64, 0, st>>>(part, n_splits, d, out);
    TL_LAUNCH_CHECK("attn_decode_combine");
  }
  return 0;
}

}  // namespace tl

using namespace tl;

#define TL_BY_DPAD(fn, ...)                                          \
  switch ((d + 31) / 32) {                                           \
    case 1: return fn<32>(__VA_ARGS__);                              \
    case 2: return fn<64>(__VA_ARGS__);                              \
    case 3: return fn<96>(__VA_ARGS__);                              \
    case 4: return fn<128>(__VA_ARGS__);                             \
    case 5: return fn<160>(__VA_ARGS__);                             \
    case 6: return fn<192>(__VA_ARGS__);                             \
    case 7: return fn<224>(__VA_ARGS__);                             \
    case 8: return fn<256>(__VA_ARGS__);                             \
  }

// vt_new: this step's values transposed, [nkv][d][vt_cols]; the value of sequence b at position p
// lies in column tile_off[b] + p - 64 * (n_cached[b] / 64); tile_off and vt_cols multiples of 64
extern "C" int tl_attn_prefill_bf16(const void* q, const void* k_new, const void* vt_new, int vt_cols,
                                    const int* tile_off, const void* pages, const int* table, int table_stride,
                                    int ring_pages, const int* row_pos, const int* cu_seqlens,
                                    const int* n_cached, int B, int n_tiles, int nq, int nkv, int d,
                                    int window, float scale, void* out, const int* items, const int* cut_blocks,
                                    int n_cut, float* part, int part_ways, long long part_floats, int n_rows,
                                    hipStream_t st) {
  TL_REQUIRE(B > 0 && n_tiles > 0 && nq > 0 && nkv > 0 && nq % nkv == 0 && nq <= 65535,
             "attn_prefill: bad sizes B=%d tiles=%d nq=%d nkv=%d", B, n_tiles, nq, nkv);
  // items (or null): n_tiles entries laid out by the host, see the kernel; cut_blocks: the n_cut blocks
  // (sequence, block, ways, -) whose keys several entries share; part: room for their sums, part_ways places a row
  TL_REQUIRE(n_cut >= 0 && (n_cut == 0 || (items != nullptr && cut_blocks != nullptr && part != nullptr && n_rows > 0 &&
                                          part_ways >= 2 && part_ways <= PF_MAX_WAYS &&
                                          part_floats >= (long long)n_rows * nq * part_ways * (d + PF_PART_HEAD))),
             "attn_prefill: %d blocks cut %d ways at most (2 to 8) need the entries, the blocks and %lld floats for "
             "their sums (%lld given)", n_cut, part_ways, (long long)n_rows * nq * part_ways * (d + PF_PART_HEAD),
             part_floats);
  TL_REQUIRE(((uintptr_t)items % 16 == 0) && ((uintptr_t)cut_blocks % 16 == 0) && ((uintptr_t)part % 16 == 0),
             "attn_prefill: the entries and the room for the sums must be 16-byte aligned");
  TL_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attn_prefill: head size %d is not served "
             "(multiples of 16 up to 256)", d);
  TL_REQUIRE(ring_pages > 0 && table_stride > 0 && window >= 0,
             "attn_prefill: bad cache geometry ring_pages=%d table_stride=%d window=%d", ring_pages,
             table_stride, window);
  TL_REQUIRE(vt_cols > 0 && vt_cols % 64 == 0 && ((uintptr_t)vt_new % 16 == 0),
             "attn_prefill: the transposed values need a multiple of 64 columns (%d) and 16-byte alignment",
             vt_cols);
  // (a thread's offsets into the step's keys and transposed values are 32 bits)
  TL_REQUIRE((long long)vt_cols * 2 * 256 < (1LL << 32) && (long long)nkv * d * 2 * 64 < (1LL << 32),
             "attn_prefill: %d columns of transposed values (or %d KV heads of %d) are too many for one step",
             vt_cols, nkv, d);
  TL_BY_DPAD(launch_prefill, (const bf16*)q, (const bf16*)k_new, (const bf16*)vt_new, vt_cols, tile_off,
             (const bf16*)pages, table, table_stride, ring_pages, row_pos, cu_seqlens, n_cached, B,
             n_tiles, nq, nkv, d, window, scale, (bf16*)out, reinterpret_cast<const int4*>(items),
             reinterpret_cast<const int4*>(cut_blocks), n_cut, part, part_ways, st);
  return 1;
}

// For tests and measurements: 1 (the default) lets head sizes 64, 128 and 256 go through the kernel that stages the
// pages in LDS, 0 sends every head size through the kernel that reads them into registers.  Returns the old setting.
extern "C" int tl_attn_decode_through_lds(int on) {
  const int was = decode_through_lds ? 1 : 0;
  decode_through_lds = on != 0;
  return was;
}

// part: float scratch of B * nq * n_splits * (d + 2) elements (not touched when n_splits is 1)
extern "C" int tl_attn_decode_bf16(const void* q, const void* pages, const int* table, int table_stride,
                                   int ring_pages, const int* row_pos, int B, int nq, int nkv, int d,
                                   int window, float scale, int n_splits, float* part, void* out,
                                   hipStream_t st) {
  TL_REQUIRE(B > 0 && nq > 0 && nkv > 0 && nq % nkv == 0, "attn_decode: bad sizes B=%d nq=%d nkv=%d", B,
             nq, nkv);
  TL_REQUIRE(d >= 16 && d <= 256 && d % 16 == 0, "attn_decode: head size %d is not served "
             "(multiples of 16 up to 256)", d);
  TL_REQUIRE(ring_pages > 0 && table_stride > 0 && window >= 0 && n_splits > 0 && n_splits <= 4096,
             "attn_decode: bad geometry ring_pages=%d table_stride=%d window=%d splits=%d", ring_pages,
             table_stride, window, n_splits);
  TL_BY_DPAD(launch_decode, (const bf16*)q, (const bf16*)pages, table, table_stride, ring_pages, row_pos,
             B, nq, nkv, d, window, scale, n_splits, part, (bf16*)out, st);
  return 1;
}

// ---- the entry point that allocates nothing (declared in no_alloc.h) --------
// The partial results of the splits lie in this array instead of a buffer of the
// caller's.  In host code its name is only a stand-in: the address that kernels
// and copies take is looked up per device, once, and kept.
static __device__ __align__(256) unsigned char scratch[TL_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
std::mutex scratch_lock;
float* scratch_of_device[MAX_DEVICES] = {};

// The device address of `scratch` on the current device (0 and an error message if it cannot be had).
float* static_scratch() {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= MAX_DEVICES) {
    set_error("attn_decode_static: no current device (%s, device %d)", hipGetErrorString(e), dev);
    return nullptr;
  }
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (scratch_of_device[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      set_error("attn_decode_static: the scratch array has no address on device %d: %s", dev,
                hipGetErrorString(e));
      return nullptr;
    }
    scratch_of_device[dev] = static_cast<float*>(ptr);
  }
  return scratch_of_device[dev];
}
}  // namespace

extern "C" size_t tl_static_scratch_bytes(void) { return TL_STATIC_SCRATCH_BYTES; }

extern "C" int tl_static_scratch_ready(void) { return static_scratch() == nullptr ? 2 : 0; }

extern "C" int tl_attn_decode_bf16_static(const void* q, const void* pages, const int* table, int table_stride,
                                          int ring_pages, const int* row_pos, int B, int nq, int nkv, int d,
                                          int window, float scale, int n_splits, void* out, hipStream_t st) {
  TL_REQUIRE(B > 0 && nq > 0 && nkv > 0 && d > 0 && n_splits > 0,
             "attn_decode_static: bad sizes B=%d nq=%d nkv=%d d=%d splits=%d", B, nq, nkv, d, n_splits);
  const unsigned long long need = 4ull * (unsigned long long)B * (unsigned long long)nq *
                                  (unsigned long long)n_splits * (unsigned long long)(d + 2);
  TL_REQUIRE(n_splits == 1 || need <= TL_STATIC_SCRATCH_BYTES,
             "attn_decode_static: the partial results of B=%d, %d heads, %d splits, head size %d take %llu "
             "bytes, the static scratch holds %u", B, nq, n_splits, d, need, (unsigned)TL_STATIC_SCRATCH_BYTES);
  float* part = static_scratch();
  if (part == nullptr) return 2;
  return tl_attn_decode_bf16(q, pages, table, table_stride, ring_pages, row_pos, B, nq, nkv, d, window, scale,
                             n_splits, part, out, st);
}
