// Next-token choice on the device, one block per row of 32-bit logits.
//
// What is computed follows the reference's sampler (ullm/layers/sampler.py:39-56): logits / T, top-k
// (keep values >= the k-th largest, ties kept, sampler.py:67-76), top-p on the softmax of what top-k
// left (drop the low tail whose cumulative probability is <= 1 - p, sampler.py:78-92), min-p
// (drop probabilities below min_p * max, sampler.py:95-107), softmax, draw.  How it is computed
// differs: no sort of the vocabulary.  Every filter is a threshold on the value, found by bisection
// over the order-preserving integer image of the floats with fixed-order block reductions, and the
// draw is an inverse-CDF walk in index order with a counter-based uniform from (seed, position), so
// a row's token depends on nothing else in the batch.  T == 0 picks the first index of the maximum
// (the reference has no greedy path that its runner reaches, sampler.py:28-36).
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

__device__ __forceinline__ int block_sum_int(int v, int* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  int r = 0;
  for (int w = 0; w < nwaves; ++w) r += scratch[w];
  return r;
}

// splitmix64 of (seed, position) -> uniform in [0, 1) with 24 bits
__device__ __forceinline__ float uniform_from_seed(uint64_t seed, uint32_t position) {
  uint64_t z = seed * 0x9E3779B97F4A7C15ull + ((uint64_t)position + 1ull) * 0xD1B54A32D192ED03ull;
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return (float)(uint32_t)(z >> 40) * (1.0f / 16777216.0f);
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int V, int ld, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const float* __restrict__ min_p, const unsigned* __restrict__ seed_lo,
              const unsigned* __restrict__ seed_hi, const int* __restrict__ position,
              int* __restrict__ out) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ float wave_incl[16];
  __shared__ int chosen;
  __shared__ float part[SAMPLE_THREADS];
  const int row = blockIdx.x, tid = threadIdx.x, nthreads = blockDim.x;
  const float* x = logits + (size_t)row * ld;
  const float t = temperature[row];
  const int chunk = (V + nthreads - 1) / nthreads;
  const int begin = tid * chunk < V ? tid * chunk : V;
  const int end = begin + chunk < V ? begin + chunk : V;

  if (t == 0.f) {  // greedy: first index of the maximum
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for (int i = begin; i < end; ++i) {
      const float v = x[i];
      if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }
    }
    const float m = block_max(best, fscratch);
    int cand = (best == m && best_i != 0x7fffffff) ? best_i : 0x7fffffff;
    // smallest index among the holders of the maximum
#pragma unroll
    for (int s = WAVE / 2; s > 0; s >>= 1) { const int o = __shfl_xor(cand, s, WAVE); cand = o < cand ? o : cand; }
    __syncthreads();
    if ((tid & (WAVE - 1)) == 0) iscratch[tid / WAVE] = cand;
    __syncthreads();
    if (tid == 0) {
      int r = 0x7fffffff;
      for (int w = 0; w < (nthreads + WAVE - 1) / WAVE; ++w) r = iscratch[w] < r ? iscratch[w] : r;
      out[row] = r == 0x7fffffff ? 0 : r;
    }
    return;
  }

  const float temp = t < 0.f ? 1.f : t;  // the reference maps T <= 0 to 1 (sampler.py:41)
  float mloc = -INFINITY;
  for (int i = begin; i < end; ++i) mloc = fmaxf(mloc, x[i] / temp);
  const float m = block_max(mloc, fscratch);
  const uint32_t key_max = order_key(m);
  uint32_t kmin = 0;

  const int k = top_k[row];
  if (k > 0 && k < V) {  // largest key v with #{key >= v} >= k
    uint32_t lo = 0, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      int c = 0;
      for (int i = begin; i < end; ++i) c += order_key(x[i] / temp) >= mid;
      if (block_sum_int(c, iscratch) >= k) lo = mid; else hi = mid - 1;
    }
    kmin = lo;
  }

  const float p = top_p[row];
  if (p > 0.f && p < 1.f) {  // smallest key v with (mass of keys > v) < p * (mass kept so far)
    float s = 0.f;
    for (int i = begin; i < end; ++i) {
      const float z = x[i] / temp;
      if (order_key(z) >= kmin) s += expf(z - m);
    }
    const float bound = p * block_sum(s, fscratch);
    uint32_t lo = kmin, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float a = 0.f;
      for (int i = begin; i < end; ++i) {
        const float z = x[i] / temp;
        if (order_key(z) > mid) a += expf(z - m);
      }
      if (block_sum(a, fscratch) < bound) hi = mid; else lo = mid + 1;
    }
    kmin = lo;
  }

  const float mp = min_p[row];
  // partial sums over contiguous index ranges, then a scan in thread (= index) order
  float s = 0.f;
  for (int i = begin; i < end; ++i) {
    const float z = x[i] / temp;
    const float e = expf(z - m);
    if (order_key(z) >= kmin && e >= mp) s += e;
  }
  // inclusive scan in thread order, built from sequential sums only, so that it never decreases
  const int lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int nwaves = (nthreads + WAVE - 1) / WAVE;
  if (tid == 0) chosen = -1;
  part[tid] = s;
  __syncthreads();
  if (lane == 0) {
    float run = 0.f;
    const int stop = (wave + 1) * WAVE < nthreads ? (wave + 1) * WAVE : nthreads;
    for (int j = wave * WAVE; j < stop; ++j) { run += part[j]; part[j] = run; }
    wave_incl[wave] = run;
  }
  __syncthreads();
  float wave_base = 0.f, total = 0.f;
  for (int w = 0; w < nwaves; ++w) {
    if (w == wave) wave_base = total;
    total += wave_incl[w];
  }
  const float incl = wave_base + part[tid];
  const float prev_incl = lane == 0 ? wave_base : wave_base + part[tid - 1];
  const uint64_t seed = ((uint64_t)seed_hi[row] << 32) | (uint64_t)seed_lo[row];
  const float target = uniform_from_seed(seed, (uint32_t)position[row]) * total;
  const bool mine = s > 0.f && incl > target && !(prev_incl > target);
  if (mine) {
    // walk this thread's range from the exact running value of the scan
    float run = prev_incl;
    int pick = -1, last_kept = -1;
    for (int i = begin; i < end; ++i) {
      const float z = x[i] / temp;
      const float e = expf(z - m);
      if (order_key(z) >= kmin && e >= mp) {
        run += e;
        last_kept = i;
        if (run > target) { pick = i; break; }
      }
    }
    chosen = pick >= 0 ? pick : last_kept;
  }
  __syncthreads();
  if (chosen < 0) {  // rounding pushed the target past the total: take the last kept index
    int last = -1;
    for (int i = begin; i < end; ++i) {
      const float z = x[i] / temp;
      if (order_key(z) >= kmin && expf(z - m) >= mp) last = i;
    }
#pragma unroll
    for (int sft = WAVE / 2; sft > 0; sft >>= 1) { const int o = __shfl_xor(last, sft, WAVE); last = o > last ? o : last; }
    __syncthreads();
    if (lane == 0) iscratch[wave] = last;
    __syncthreads();
    if (tid == 0) {
      int r = 0;
      for (int w = 0; w < nwaves; ++w) r = iscratch[w] > r ? iscratch[w] : r;
      out[row] = r;
    }
  } else if (tid == 0) {
    out[row] = chosen;
  }
}

extern "C" int ullm_sample(const float* logits, int n_rows, int V, int ld, const float* temperature,
                           const int* top_k, const float* top_p, const float* min_p,
                           const unsigned* seed_lo, const unsigned* seed_hi, const int* position,
                           int* out, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ld < V) return ULLM_ERR_SHAPE;
  hipLaunchKernelGGL(sample_kernel, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, V, ld,
                     temperature, top_k, top_p, min_p, seed_lo, seed_hi, position, out);
  ULLM_LAUNCH_CHECK();
}
