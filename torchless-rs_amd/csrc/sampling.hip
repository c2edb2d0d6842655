// Sampling of one token per row of logits, one block per row, all in float.
//
// Order as in the reference (src/sampler/mod.rs:194-238): temperature <= 0 is
// the argmax (of equal maxima the last index, as `max_by` keeps it, :60-68);
// else z = logit / T, top-k on z (:93-119, ties at the threshold kept in index
// order), softmax, top-p on the probabilities (:144-170), then the first index
// whose running sum reaches r, else the last index (:225-238).  The reference
// draws r from an unseeded generator; here r comes from Philox4x32-10 keyed by
// the seed with the counter (step, sequence), so a sequence's draws do not
// depend on its batch-mates.
#include "common.hpp"

namespace tl {

constexpr int SNT = 1024;

__device__ __forceinline__ uint32_t order_key(float v) {
  const uint32_t b = __float_as_uint(v);
  return (b & 0x80000000u) ? ~b : (b | 0x80000000u);   // ascending with the value
}

__device__ inline float philox_uniform(uint32_t seed_lo, uint32_t seed_hi, uint32_t step,
                                       uint32_t seq) {
  uint32_t c0 = step, c1 = seq, c2 = 0u, c3 = 0u, k0 = seed_lo, k1 = seed_hi;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    if (r > 0) {
      k0 += 0x9E3779B9u;
      k1 += 0xBB67AE85u;
    }
    const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
    const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
    const uint32_t n0 = hi1 ^ c1 ^ k0, n1 = lo1, n2 = hi0 ^ c3 ^ k1, n3 = lo0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
  }
  return (float)(c0 >> 8) * (1.0f / 16777216.0f);      // [0, 1)
}

__device__ __forceinline__ int block_sum_i(int v, int* sh) {
#pragma unroll
  for (int o = WAVE / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, WAVE);
  __syncthreads();
  if (threadIdx.x % WAVE == 0) sh[threadIdx.x / WAVE] = v;
  __syncthreads();
  int r = 0;
#pragma unroll
  for (int i = 0; i < SNT / WAVE; ++i) r += sh[i];
  return r;
}

// exclusive prefix over the threads of the block, in thread order
template <typename V> __device__ __forceinline__ V block_excl_scan(V v, V* sh, V* total) {
  __syncthreads();
  sh[threadIdx.x] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    V run = 0;
    for (int i = 0; i < SNT; ++i) {
      const V t = sh[i];
      sh[i] = run;
      run += t;
    }
    sh[SNT] = run;
  }
  __syncthreads();
  *total = sh[SNT];
  return sh[threadIdx.x];
}

__global__ void __launch_bounds__(SNT)
sample_kernel(const float* __restrict__ logits, int V, float temperature, int top_k, float top_p,
              uint32_t seed_lo, uint32_t seed_hi, const int* __restrict__ counters,
              float* __restrict__ probs, int* __restrict__ out) {
  __shared__ float shf[SNT + 1];
  __shared__ int shi[SNT + 1];
  __shared__ int sh_pick;
  const int b = blockIdx.x, tid = threadIdx.x;
  const float* z_in = logits + (size_t)b * V;
  float* p = probs + (size_t)b * V;

  if (!(temperature > 0.f)) {                           // greedy
    float best = -INFINITY;
    int bi = -1;
    for (int i = tid; i < V; i += SNT) {
      const float v = z_in[i];
      if (bi < 0 || v >= best) { best = v; bi = i; }
    }
    shf[tid] = best;
    shi[tid] = bi;
    __syncthreads();
    for (int o = SNT / 2; o > 0; o >>= 1) {
      if (tid < o) {
        const float v2 = shf[tid + o];
        const int i2 = shi[tid + o];
        if (i2 >= 0 && (shi[tid] < 0 || v2 > shf[tid] || (v2 == shf[tid] && i2 > shi[tid]))) {
          shf[tid] = v2;
          shi[tid] = i2;
        }
      }
      __syncthreads();
    }
    if (tid == 0) out[b] = shi[0];
    return;
  }

  // contiguous chunk of this thread, for the steps that go by index order
  const int chunk = (V + SNT - 1) / SNT;
  const int c0 = min(V, tid * chunk), c1 = min(V, c0 + chunk);

  for (int i = tid; i < V; i += SNT) p[i] = z_in[i] / temperature;
  __syncthreads();

  if (top_k > 0 && top_k < V) {
    // k-th largest by bisection on the ordered bit pattern
    uint32_t thr = 0u;
    for (int bit = 31; bit >= 0; --bit) {
      const uint32_t cand = thr | (1u << bit);
      int c = 0;
      for (int i = tid; i < V; i += SNT) c += order_key(p[i]) >= cand;
      if (block_sum_i(c, shi) >= top_k) thr = cand;
    }
    int cge = 0, cgt = 0;
    for (int i = c0; i < c1; ++i) {
      const uint32_t k = order_key(p[i]);
      cge += k >= thr;
      cgt += k > thr;
    }
    const int n_ge = block_sum_i(cge, shi), n_gt = block_sum_i(cgt, shi);
    if (n_ge <= top_k) {
      for (int i = c0; i < c1; ++i)
        if (order_key(p[i]) < thr) p[i] = -INFINITY;
    } else {
      int total;
      int rank = block_excl_scan<int>(cge - cgt, shi, &total);   // ties before this chunk
      const int keep_ties = top_k - n_gt;
      for (int i = c0; i < c1; ++i) {
        const uint32_t k = order_key(p[i]);
        if (k < thr) p[i] = -INFINITY;
        else if (k == thr) {
          if (rank >= keep_ties) p[i] = -INFINITY;
          ++rank;
        }
      }
    }
    __syncthreads();
  }

  // softmax
  float mx = -INFINITY;
  for (int i = tid; i < V; i += SNT) mx = fmaxf(mx, p[i]);
  mx = block_max<SNT>(mx, shf);
  float sum = 0.f;
  for (int i = tid; i < V; i += SNT) {
    const float e = expf(p[i] - mx);
    p[i] = e;
    sum += e;
  }
  sum = block_sum<SNT>(sum, shf);
  for (int i = tid; i < V; i += SNT) p[i] = p[i] / sum;
  __syncthreads();

  if (top_p > 0.f && top_p < 1.f) {
    // the largest t with sum(p_i >= t) >= top_p is the smallest kept probability
    uint32_t thr = 0u;
    for (int bit = 30; bit >= 0; --bit) {
      const uint32_t cand = thr | (1u << bit);
      float s = 0.f;
      for (int i = tid; i < V; i += SNT) s += (__float_as_uint(p[i]) >= cand) ? p[i] : 0.f;
      if (block_sum<SNT>(s, shf) >= top_p) thr = cand;
    }
    const float thr_f = __uint_as_float(thr);
    float sgt = 0.f;
    int ties = 0;
    for (int i = c0; i < c1; ++i) {
      const uint32_t k = __float_as_uint(p[i]);
      if (k > thr) sgt += p[i];
      ties += k == thr;
    }
    const float sum_gt = block_sum<SNT>(sgt, shf);
    int n_ties;
    int rank = block_excl_scan<int>(ties, shi, &n_ties);
    int keep_ties = (thr_f > 0.f) ? (int)ceilf((top_p - sum_gt) / thr_f) : n_ties;
    keep_ties = max(1, min(keep_ties, n_ties));
    const float new_sum = sum_gt + (float)keep_ties * thr_f;
    for (int i = c0; i < c1; ++i) {
      const uint32_t k = __float_as_uint(p[i]);
      float v = p[i];
      if (k < thr) v = 0.f;
      else if (k == thr) {
        if (rank >= keep_ties) v = 0.f;
        ++rank;
      }
      p[i] = (new_sum > 0.f) ? v / new_sum : v;
    }
    __syncthreads();
  }

  // draw: first index whose running sum reaches r
  const float r = philox_uniform(seed_lo, seed_hi, (uint32_t)counters[2 * b + 1],
                                 (uint32_t)counters[2 * b]);
  float local = 0.f;
  for (int i = c0; i < c1; ++i) local += p[i];
  float total;
  const float before = block_excl_scan<float>(local, shf, &total);
  if (tid == 0) sh_pick = V - 1;
  __syncthreads();
  if (c0 < c1 && before + local >= r) {
    float run = before;
    for (int i = c0; i < c1; ++i) {
      run += p[i];
      if (run >= r) {
        atomicMin(&sh_pick, i);
        break;
      }
    }
  }
  __syncthreads();
  if (tid == 0) out[b] = sh_pick;
}

}  // namespace tl

using namespace tl;

extern "C" int tl_sample(const float* logits, int B, int V, float temperature, int top_k, float top_p,
                         unsigned long long seed, const int* counters, float* probs, int* out,
                         hipStream_t st) {
  TL_REQUIRE(B >= 0 && V > 0, "sample: bad sizes B=%d V=%d", B, V);
  if (B == 0) return 0;
  sample_kernel<<<B, SNT, 0, st>>>(logits, V, temperature, top_k, top_p, (uint32_t)(seed & 0xffffffffu),
                                   (uint32_t)(seed >> 32), counters, probs, out);
  TL_LAUNCH_CHECK("sample");
  return 0;
}
