// Next-token choice on the device from rows of 32-bit logits: one block per row, after a first kernel that
// cuts the rows into parts over many blocks for the settings it serves (temperature alone, a small top-k).
//
// What is computed follows the reference's sampler (ullm/layers/sampler.py:39-56): logits / T, top-k
// (keep values >= the k-th largest, ties kept, sampler.py:67-76), top-p on the softmax of what top-k
// left (drop the low tail whose cumulative probability is <= 1 - p, sampler.py:78-92), min-p
// (drop probabilities below min_p * max, sampler.py:95-107), softmax, draw.  How it is computed
// differs: no sort of the vocabulary.  Every filter is a threshold on the value: among a few gathered
// candidates where the setting and the row allow it, else by bins of the distance from the maximum (counts and
// fixed-point weights, so that no sum depends on the order of its additions) and a search inside one bin, else by
// bisection over the order-preserving integer image of the floats with fixed-order block reductions; and the
// draw is an inverse-CDF walk in index order with a counter-based uniform from (seed, position), so
// a row's token depends on nothing else in the batch.  T == 0 picks the first index of the maximum
// (the reference has no greedy path that its runner reaches, sampler.py:28-36).
#include "common.h"

#define SAMPLE_THREADS 1024

// An unsigned integer that orders as the float does; -0.0 and +0.0, which compare equal, get one key
// (-0.0 + 0.0 is +0.0, and the sum of anything else with 0.0 is itself).
__device__ __forceinline__ uint32_t order_key(float f) {
  const uint32_t u = __float_as_uint(f + 0.f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

// A logit over the temperature, as a product of its own: never fused into the subtraction of the maximum that
// follows, so that the largest value's distance from the maximum is exactly zero and its weight exactly one
// in every pass (a min-p of one keeps the ties for the maximum, and the same ones in each pass).
__device__ __forceinline__ float scaled(float v, float inv_t) {
#pragma clang fp contract(off)
  return v * inv_t;
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

// Visits the elements [wbeg, wend) of a wave's range, lane-strided, with several independent loads
// in flight per lane.  VEC: 16-byte loads (the row must be 16-byte aligned and wbeg, wend multiples
// of 4): a lane gets 4 consecutive values, the wave 256 consecutive values per access.
// U: loads a lane has in flight.  The passes that every sampled row takes (maximum, sum) run with 8: a wave's
// share of 150 K values is then five round trips to memory instead of ten.
template <bool VEC, int U = 4, typename F>
__device__ __forceinline__ void for_range(const float* __restrict__ x, int wbeg, int wend, int lane, F f) {
  if (VEC) {
    for (int i0 = wbeg + 4 * lane; i0 < wend; i0 += U * 4 * WAVE) {
      float4 v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int ii = i0 + u * 4 * WAVE;
        v[u] = ii < wend ? *reinterpret_cast<const float4*>(x + ii) : make_float4(0.f, 0.f, 0.f, 0.f);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int ii = i0 + u * 4 * WAVE;
        if (ii < wend) { f(ii, v[u].x); f(ii + 1, v[u].y); f(ii + 2, v[u].z); f(ii + 3, v[u].w); }
      }
    }
  } else {
    for (int i0 = wbeg + lane; i0 < wend; i0 += U * WAVE) {
      float v[U];
#pragma unroll
      for (int u = 0; u < U; ++u) v[u] = i0 + u * WAVE < wend ? x[i0 + u * WAVE] : 0.f;
#pragma unroll
      for (int u = 0; u < U; ++u)
        if (i0 + u * WAVE < wend) f(i0 + u * WAVE, v[u]);
    }
  }
}

// ------------------------------------------------------------------------------ few candidates
// With top-k at work and k small, or with top-p alone on a peaked row, the values that can matter
// are few.  Two passes find a distance d = 2^(5-j), j = 0..15, such that {z >= max - d} has at least
// k members (top-k) or a little more than the share p of all weight (top-p alone) but not much
// more; one more pass gathers these candidates, in index order, into shared memory (each wave its
// own range and its own segment); every filter and the draw then run over the candidates only, by
// the same rules as over the whole vocabulary.  Where this does not work out (fewer than k values
// within 32 of the maximum, or more candidates than a segment holds: many equal values, a flat row
// under top-p alone) the caller takes the long way (thresholds by bins, see below).
#define SMALL_K_MAX 1024
#define SEG 256                       // candidates a wave can hold
#define DELTA_STEPS 16

struct Candidates {
  float z[16 * SEG];                  // as gathered: a segment per wave
  int idx[16 * SEG];
  int n[16];
  float lz[16 * SEG];                 // side by side
  float le[16 * SEG];                 // their weights exp(z - max)
  int lidx[16 * SEG];
  int result;
};

// draw_from_list for up to 4 * 64 candidates: a lane keeps its four in registers, counts are ballots, and
// top-p needs no search: a candidate stays if the weight of the larger ones (of those top-k left) is below
// the bound, which every lane adds up for its own candidates in index order.
__device__ int draw_from_short_list(const Candidates& cand, int n_all, bool by_count, int k, float p, float mp,
                                    float all_weight, uint32_t key_thr, uint32_t key_max, float uniform, int lane) {
  constexpr int H = 4;
  float zr[H], er[H];
  uint32_t kr[H];
  bool have[H];
#pragma unroll
  for (int i = 0; i < H; ++i) {
    const int j = lane + i * WAVE;
    have[i] = j < n_all;
    zr[i] = cand.lz[have[i] ? j : 0];
    er[i] = have[i] ? cand.le[j] : 0.f;
    kr[i] = order_key(zr[i]);
  }
  uint32_t kmin = key_thr;
  if (by_count) {                           // the largest key v with #{key >= v} >= k
    uint32_t lo = key_thr, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      int c = 0;
#pragma unroll
      for (int i = 0; i < H; ++i) c += __popcll(__ballot(have[i] && kr[i] >= mid));
      if (c >= k) lo = mid; else hi = mid - 1;
    }
    kmin = lo;
  }
  if (p > 0.f && p < 1.f) {
    float a = 0.f;
#pragma unroll
    for (int i = 0; i < H; ++i) a += (have[i] && kr[i] >= kmin) ? er[i] : 0.f;
    const float listed = wave_sum(a);
    const float bound = p * (by_count ? listed : all_weight);
    if (!by_count && listed < bound) return -1;
    float above[H] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int src = 0; src < H; ++src) {
      const int n_here = n_all - src * WAVE < WAVE ? n_all - src * WAVE : WAVE;
      const float e_src = kr[src] >= kmin ? er[src] : 0.f;
      for (int j = 0; j < n_here; ++j) {
        const float zj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(zr[src]), j));
        const float ej = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(e_src), j));
#pragma unroll
        for (int i = 0; i < H; ++i) above[i] += zj > zr[i] ? ej : 0.f;
      }
    }
    uint32_t least = 0xffffffffu;           // the smallest key that stays
#pragma unroll
    for (int i = 0; i < H; ++i)
      if (have[i] && kr[i] >= kmin && above[i] < bound) least = kr[i] < least ? kr[i] : least;
#pragma unroll
    for (int d = WAVE / 2; d > 0; d >>= 1) { const uint32_t o = __shfl_xor(least, d, WAVE); least = o < least ? o : least; }
    if (least != 0xffffffffu) kmin = least;
  }
  // min-p and the draw
  float w[H], total = 0.f;
#pragma unroll
  for (int i = 0; i < H; ++i) {
    w[i] = (have[i] && kr[i] >= kmin && er[i] >= mp) ? er[i] : 0.f;
    total += w[i];
  }
  total = wave_sum(total);
  const float target = uniform * total;
  float run = 0.f;
  int token = -1, last_kept = -1;
#pragma unroll
  for (int i = 0; i < H; ++i) {
    if (i * WAVE >= n_all || token >= 0) continue;
    float incl = w[i];
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
      const float o = __shfl_up(incl, d, WAVE);
      if (lane >= d) incl += o;
    }
    const unsigned long long kept = __ballot(w[i] > 0.f);
    const unsigned long long crossed = __ballot(w[i] > 0.f && run + incl > target);
    if (crossed) token = cand.lidx[i * WAVE + __ffsll((long long)crossed) - 1];
    if (kept) last_kept = cand.lidx[i * WAVE + 63 - __clzll((long long)kept)];
    run += __shfl(incl, WAVE - 1, WAVE);
  }
  if (token < 0) token = last_kept < 0 ? 0 : last_kept;
  return token;
}

// Top-k, top-p, min-p and the draw over a list of candidates in index order (lz: values / T, le: weights
// exp(z - max), lidx: vocabulary indices), the work of one wave.  by_count: top-k is at work and every value
// >= the k-th largest is in the list; else the list holds the nucleus of all weight `all_weight`.  key_thr: a key
// with at least k candidates at or above it (by_count) / the key all candidates reach.  -1: the list does not
// hold the nucleus (take the long way); else the token.
__device__ int draw_from_list(const Candidates& cand, int n_all, bool by_count, int k, float p, float mp,
                              float all_weight, uint32_t key_thr, uint32_t key_max, float uniform, int lane) {
  if (n_all <= 4 * WAVE)
    return draw_from_short_list(cand, n_all, by_count, k, p, mp, all_weight, key_thr, key_max, uniform, lane);
  auto count_if = [&](auto pred) {
    int c = 0;
    for (int j0 = 0; j0 < n_all; j0 += WAVE)
      c += __popcll(__ballot(j0 + lane < n_all && pred(cand.lz[j0 + lane < n_all ? j0 + lane : 0])));
    return c;
  };
  auto mass_if = [&](auto pred) {
    float a = 0.f;
    for (int j = lane; j < n_all; j += WAVE) {
      if (pred(cand.lz[j])) a += cand.le[j];
    }
    return wave_sum(a);
  };
  // 3. top-k: the largest key v with #{key >= v} >= k; all such keys are candidates
  uint32_t kmin = key_thr;
  if (by_count) {
    uint32_t lo = key_thr, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      if (count_if([&](float zz) { return order_key(zz) >= mid; }) >= k) lo = mid; else hi = mid - 1;
    }
    kmin = lo;
  }
  // 4. top-p on what top-k left (without top-k: on everything, and the candidates must hold the nucleus)
  if (p > 0.f && p < 1.f) {
    const float listed = mass_if([&](float zz) { return order_key(zz) >= kmin; });
    const float bound = p * (by_count ? listed : all_weight);
    if (!by_count && listed < bound) return -1;
    uint32_t lo = kmin, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      if (mass_if([&](float zz) { return order_key(zz) > mid; }) < bound) hi = mid; else lo = mid + 1;
    }
    kmin = lo;
  }
  // 5. min-p and the draw: a walk along the list, 64 candidates at a time
  auto weight = [&](int j) {
    if (j >= n_all) return 0.f;
    const float e = cand.le[j];
    return (order_key(cand.lz[j]) >= kmin && e >= mp) ? e : 0.f;
  };
  float total = 0.f;
  for (int j = lane; j < n_all; j += WAVE) total += weight(j);
  total = wave_sum(total);
  const float target = uniform * total;
  float run = 0.f;
  int token = -1, last_kept = -1;
  for (int j0 = 0; j0 < n_all && token < 0; j0 += WAVE) {
    const float e = weight(j0 + lane);
    float incl = e;
#pragma unroll
    for (int d = 1; d < WAVE; d <<= 1) {
      const float o = __shfl_up(incl, d, WAVE);
      if (lane >= d) incl += o;
    }
    const unsigned long long kept = __ballot(e > 0.f);
    const unsigned long long crossed = __ballot(e > 0.f && run + incl > target);
    if (crossed) token = cand.lidx[j0 + __ffsll((long long)crossed) - 1];
    if (kept) last_kept = cand.lidx[j0 + 63 - __clzll((long long)kept)];
    run += __shfl(incl, WAVE - 1, WAVE);
  }
  if (token < 0) token = last_kept < 0 ? 0 : last_kept;   // rounding pushed the target past the total: the last index kept
  return token;
}

// -1: take the long way.  Otherwise the token.  Every thread of the block returns the same value.
template <bool VEC>
__device__ int sample_small_k(const float* __restrict__ x, int wbeg, int wend, float inv_t, float m, int k, float p,
                              float mp, float uniform, Candidates& cand, float* fscratch, int* iscratch) {
  constexpr int PER = VEC ? 4 : 1;
  constexpr int STEP = PER * WAVE;
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE, nwaves = blockDim.x / WAVE;
  const float L2E = 1.4426950408889634f;
  const uint32_t key_max = order_key(m);
  // 1. the distance: the largest j whose set still holds what is needed: k members with top-k; without
  // it (top-p alone) a little more than the share p of all weight, so that the nucleus ends inside
  const bool by_count = k > 0;
  float all_weight = 0.f;
  int j_lo = 0;
#pragma unroll 1
  for (int round = 0; round < 2; ++round) {
    const int stride = round == 0 ? 4 : 1;
    const uint32_t k1 = order_key(m - exp2f((float)(5 - (j_lo + stride)))), k2 = order_key(m - exp2f((float)(5 - (j_lo + 2 * stride)))),
                   k3 = order_key(m - exp2f((float)(5 - (j_lo + 3 * stride))));
    if (by_count) {
      int c1 = 0, c2 = 0, c3 = 0;
      for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
        const uint32_t key = order_key(scaled(v, inv_t));
        c1 += key >= k1; c2 += key >= k2; c3 += key >= k3;
      });
      c1 = block_sum_int(c1, iscratch); c2 = block_sum_int(c2, iscratch); c3 = block_sum_int(c3, iscratch);
      j_lo += stride * ((c1 >= k) + (c2 >= k) + (c3 >= k));
    } else {
      float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
      for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
        const float zz = scaled(v, inv_t);
        const uint32_t key = order_key(zz);
        const float e = __builtin_amdgcn_exp2f((zz - m) * L2E);
        a0 += e;
        a1 += key >= k1 ? e : 0.f; a2 += key >= k2 ? e : 0.f; a3 += key >= k3 ? e : 0.f;
      });
      // the sum over all values is taken exactly as the pass over the whole vocabulary takes it
      if (round == 0) all_weight = block_sum(a0, fscratch);
      a1 = block_sum(a1, fscratch); a2 = block_sum(a2, fscratch); a3 = block_sum(a3, fscratch);
      const float need = p * all_weight * 1.001f;
      j_lo += stride * ((a1 >= need) + (a2 >= need) + (a3 >= need));
    }
  }
  const uint32_t key_thr = order_key(m - exp2f((float)(5 - j_lo)));
  // 2. gather, in index order: a wave walks its range and appends what it keeps to its segment
  int pos = 0;
  bool overflow = false;
  constexpr int AHEAD = 4;                                 // steps whose loads are under way together
  for (int base = wbeg; base < wend && !overflow; base += AHEAD * STEP) {
    float raw[AHEAD][PER];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int ii = base + u * STEP + PER * lane;
      if (VEC) {
        const float4 v = ii < wend ? *reinterpret_cast<const float4*>(x + ii) : make_float4(0.f, 0.f, 0.f, 0.f);
        raw[u][0] = v.x;
        if (PER > 1) { raw[u][1] = v.y; raw[u][2] = v.z; raw[u][3] = v.w; }
      } else {
        raw[u][0] = ii < wend ? x[ii] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int ii = base + u * STEP + PER * lane;
      float z[PER];
      bool keep[PER];
      int cnt = 0;
#pragma unroll
      for (int c = 0; c < PER; ++c) {
        z[c] = scaled(raw[u][c], inv_t);
        keep[c] = ii + c < wend && order_key(z[c]) >= key_thr;
        cnt += keep[c];
      }
      if (overflow || !__any(cnt)) continue;
      int incl = cnt;
#pragma unroll
      for (int d = 1; d < WAVE; d <<= 1) {
        const int o = __shfl_up(incl, d, WAVE);
        if (lane >= d) incl += o;
      }
      const int total = __shfl(incl, WAVE - 1, WAVE);
      if (pos + total > SEG) { overflow = true; continue; }
      int o = wave * SEG + pos + incl - cnt;
#pragma unroll
      for (int c = 0; c < PER; ++c)
        if (keep[c]) { cand.z[o] = z[c]; cand.idx[o] = ii + c; ++o; }
      pos += total;
    }
  }
  if (lane == 0) cand.n[wave] = overflow ? -1 : pos;
  __syncthreads();
  int n_all = 0;
  bool bad = false;
  for (int w = 0; w < nwaves; ++w) { bad = bad || cand.n[w] < 0; n_all += cand.n[w] < 0 ? 0 : cand.n[w]; }
  if (bad || n_all < (by_count ? k : 1)) return -1;
  // the candidates side by side (still in index order) with their weights; the rest is the work of
  // one wave, with reductions inside the wave
#define E_OF(zz) __builtin_amdgcn_exp2f(((zz) - m) * L2E)
  {
    int off = 0;
    for (int w = 0; w < wave; ++w) off += cand.n[w];
    for (int j = lane; j < cand.n[wave]; j += WAVE) {
      const float zz = cand.z[wave * SEG + j];
      cand.lz[off + j] = zz;
      cand.le[off + j] = E_OF(zz);
      cand.lidx[off + j] = cand.idx[wave * SEG + j];
    }
  }
  __syncthreads();
  if (wave == 0) {
    const int token = draw_from_list(cand, n_all, by_count, k, p, mp, all_weight, key_thr, key_max, uniform, lane);
    if (lane == 0) cand.result = token;
  }
  __syncthreads();
#undef E_OF
  return cand.result;
}

// The draw inside [rbeg, rend) (not empty; with VEC a multiple of 4 long, from a multiple of 4), by the whole
// block: `run` is the weight before the range, the token is the first index at which the running sum passes
// `target`.  The walk over the range in index order, STEP values at a time, is a chain of sums; the sums of the
// steps are not: the block's waves take the steps of the range in turn, then every thread adds the steps' sums
// in order until one crosses the target, and takes running sums inside that step (a lane's values in order,
// the lanes by a scan).  Returns the token, or the last index of the range that counts if
// rounding kept the running sum from passing the target (-1: none counts).  Every thread gets the same value.
template <bool VEC>
__device__ int walk_range(const float* __restrict__ x, int rbeg, int rend, float run, float target, float inv_t,
                          float m, uint32_t kmin, float mp, float* step_sum, int* step_kept) {
  constexpr int PER = VEC ? 4 : 1;
  constexpr int STEP = PER * WAVE;
  constexpr int HELD = 4;                 // steps a wave takes per round
  const float L2E = 1.4426950408889634f;
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE, nwaves = blockDim.x / WAVE;
  int pick = -1, last_kept = -1;
  // the values of the step at i0 that count, as a lane holds them; the highest index among them that counts
  auto weights_of = [&](const float (&cur)[PER], int i0, float (&e)[PER], int& kept_hi) {
    kept_hi = -1;
#pragma unroll
    for (int c = 0; c < PER; ++c) {
      const int i = i0 + PER * lane + c;
      const float z = scaled(cur[c], inv_t);
      const float ev = __builtin_amdgcn_exp2f((z - m) * L2E);
      e[c] = (i < rend && order_key(z) >= kmin && ev >= mp) ? ev : 0.f;
      if (e[c] > 0.f) kept_hi = i;
    }
#pragma unroll
    for (int sft = WAVE / 2; sft > 0; sft >>= 1) { const int o = __shfl_xor(kept_hi, sft, WAVE); kept_hi = o > kept_hi ? o : kept_hi; }
  };
  auto fetch = [&](int i0, float (&dst)[PER]) {
    const int last = rend - PER;
    if (VEC) {
      const int ii = i0 + 4 * lane;
      const float4 v = *reinterpret_cast<const float4*>(x + (ii < last ? ii : last));
      dst[0] = v.x; if (PER > 1) { dst[1] = v.y; dst[2] = v.z; dst[3] = v.w; }
    } else {
      const int ii = i0 + lane;
      dst[0] = x[ii < last ? ii : last];
    }
  };
  const int round_span = HELD * nwaves * STEP;
  for (int r0 = rbeg; r0 < rend && pick < 0; r0 += round_span) {
    float cur[HELD][PER];
#pragma unroll
    for (int j = 0; j < HELD; ++j) fetch(r0 + (wave + nwaves * j) * STEP, cur[j]);
#pragma unroll
    for (int j = 0; j < HELD; ++j) {
      const int i0 = r0 + (wave + nwaves * j) * STEP;
      float e[PER], esum = 0.f;
      int kept_hi;
      weights_of(cur[j], i0, e, kept_hi);
#pragma unroll
      for (int c = 0; c < PER; ++c) esum += e[c];
      const float step = wave_sum(esum);
      if (lane == 0) { step_sum[wave + nwaves * j] = step; step_kept[wave + nwaves * j] = kept_hi; }
    }
    __syncthreads();
    const float my_step = step_sum[lane];
    const int my_kept = step_kept[lane];
    const int steps_here = (rend - r0 + STEP - 1) / STEP < HELD * nwaves ? (rend - r0 + STEP - 1) / STEP : HELD * nwaves;
    for (int c = 0; c < steps_here && pick < 0; ++c) {
      const float step = __shfl(my_step, c, WAVE);
      const int kept_hi = __shfl(my_kept, c, WAVE);
      if (kept_hi >= 0) last_kept = kept_hi;
      if (run + step > target) {            // the crossing is among these: running sums inside the step
        const int i0 = r0 + c * STEP;
        float one[PER], e[PER];
        int unused;
        fetch(i0, one);
        weights_of(one, i0, e, unused);
        float upto[PER];                      // a lane's values, added in order
        upto[0] = e[0];
#pragma unroll
        for (int cc = 1; cc < PER; ++cc) upto[cc] = upto[cc - 1] + e[cc];
        float incl = upto[PER - 1];           // then the lanes, by a scan
#pragma unroll
        for (int d = 1; d < WAVE; d <<= 1) {
          const float o = __shfl_up(incl, d, WAVE);
          if (lane >= d) incl += o;
        }
        float before = __shfl_up(incl, 1, WAVE);
        if (lane == 0) before = 0.f;
        int first = PER;                      // the lane's first value at which the sum has passed the target
#pragma unroll
        for (int cc = PER - 1; cc >= 0; --cc)
          if (e[cc] > 0.f && run + (before + upto[cc]) > target) first = cc;
        const unsigned long long crossed = __ballot(first < PER);
        if (crossed) {
          const int at = __ffsll((long long)crossed) - 1;
          pick = i0 + PER * at + __shfl(first, at, WAVE);
        }
        run += __shfl(incl, WAVE - 1, WAVE);
      } else {
        run += step;
      }
    }
    __syncthreads();                        // the next round writes the steps' sums again
  }
  return pick >= 0 ? pick : last_kept;
}

// ------------------------------------------------------------------------------ thresholds by bins
// The long way's thresholds (the k-th largest key; the key at which the weight of the larger values falls below
// the share p) without a pass per halving.  One pass puts every value that still counts into one of BIN_COUNT
// bins by its distance from the maximum (1/64 wide; the last bin takes everything from BIN_RANGE on) and adds the
// bins' counts and weights in shared memory.  Weights are 32.32 fixed-point integers (a weight is at most one),
// so their sums do not depend on the order in which the atomic additions land, and neither does the token.  A scan
// over the bins from the maximum down finds the bin in which the count reaches k or the weight reaches the
// share; if that bin holds too many values for a list, a second pass cuts it into BIN_COUNT finer bins (the
// difference of two distances inside one bin is exact) and notes every fine bin's smallest and largest key: a
// fine bin of equal values is its own answer.  Otherwise a pass gathers the bin's values and the halvings run
// over that list.  false: not decided here (the k-th largest or the nucleus's end lies 32 or more below the
// maximum, or thousands of different values share one fine bin); the caller halves over the whole vocabulary as
// before.  Every thread of the block returns the same.
#define BIN_COUNT 2048
#define BIN_PER_UNIT 64.f
#define BIN_FINE (BIN_PER_UNIT * BIN_COUNT)
#define BIN_LIST 2048                 // a bin with more values than this is cut again (a wave's segment holds SEG of them)

__device__ __forceinline__ unsigned long long block_sum_u64(unsigned long long v, unsigned long long* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE, nwaves = blockDim.x / WAVE;
#pragma unroll
  for (int d = WAVE / 2; d > 0; d >>= 1) v += __shfl_xor(v, d, WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  unsigned long long r = 0;
  for (int w = 0; w < nwaves; ++w) r += scratch[w];
  return r;
}

// the sum of the threads before this one
__device__ __forceinline__ unsigned long long block_sum_before_u64(unsigned long long v, unsigned long long* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  unsigned long long incl = v;
#pragma unroll
  for (int d = 1; d < WAVE; d <<= 1) {
    const unsigned long long o = __shfl_up(incl, d, WAVE);
    if (lane >= d) incl += o;
  }
  __syncthreads();
  if (lane == WAVE - 1) scratch[wave] = incl;
  __syncthreads();
  unsigned long long base = 0;
  for (int w = 0; w < wave; ++w) base += scratch[w];
  return base + incl - v;
}

struct BinPick {
  int bin, count;
  unsigned long long above;           // count or weight of everything in the bins before it
  uint32_t key;                       // the threshold, from the wave that found it to the block
};

template <bool VEC, bool BY_COUNT>
__device__ __noinline__ bool threshold_by_bins(const float* __restrict__ x, int wbeg, int wend, float inv_t, float m,
                                  uint32_t kmin_in, int k, float p, Candidates& cand, unsigned long long* wide,
                                  BinPick* pick, uint32_t* found) {
  constexpr int PER = VEC ? 4 : 1;
  constexpr int STEP = PER * WAVE;
  const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE, nwaves = blockDim.x / WAVE;
  const float L2E = 1.4426950408889634f;
  unsigned long long* const bin_w = reinterpret_cast<unsigned long long*>(cand.lz);   // BIN_COUNT of them
  unsigned* const bin_n = reinterpret_cast<unsigned*>(cand.le);
  uint32_t* const bin_lo = reinterpret_cast<uint32_t*>(cand.lidx);                    // of the fine bins: smallest key,
  uint32_t* const bin_hi = bin_lo + BIN_COUNT;                                        // largest key
  static_assert(sizeof(cand.lidx) >= 2 * BIN_COUNT * sizeof(uint32_t), "the fine bins' keys lie in the list's indices");
  static_assert(sizeof(cand.lz) >= BIN_COUNT * sizeof(unsigned long long) && sizeof(cand.le) >= BIN_COUNT * sizeof(unsigned),
                "the bins lie where the list of candidates lies otherwise");
  // a value's bin: by its distance from the maximum; inside bin `coarse`, by the rest of that distance
  auto bin_of = [&](float z, int coarse) {
    const float dist = m - z;                                       // >= 0; +inf for a masked value
    const int b1 = (int)fminf(dist * BIN_PER_UNIT, (float)(BIN_COUNT - 1));
    if (coarse < 0) return b1;
    if (b1 != coarse) return -1;
    const float rest = dist - (float)b1 * (1.f / BIN_PER_UNIT);     // exact: both are multiples of the distance's last bit
    const int b2 = (int)fminf(rest * BIN_FINE, (float)(BIN_COUNT - 1));
    return b2 < 0 ? 0 : b2;
  };
  auto weight_of = [&](float z) {
    return (unsigned long long)(__builtin_amdgcn_exp2f((z - m) * L2E) * 4294967296.f);
  };
  unsigned long long above = 0, bound = BY_COUNT ? (unsigned long long)k : 0;
  int coarse = -1, fine = -1, count = 0;
#pragma unroll 1
  for (int level = 0; level < 2; ++level) {
    for (int b = tid; b < BIN_COUNT; b += blockDim.x) { bin_w[b] = 0; bin_n[b] = 0; bin_lo[b] = 0xffffffffu; bin_hi[b] = 0u; }
    if (tid == 0) pick->bin = -1;
    __syncthreads();
    for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
      const float z = scaled(v, inv_t);
      const uint32_t key = order_key(z);
      const int b = key < kmin_in ? -1 : bin_of(z, coarse);
      // the last coarse bin (32 or more below the maximum: masked values, the far tail) is not filled: its weights
      // are below the fixed point's last bit, and a k-th largest value in it is not found here anyway
      if (b < 0 || (level == 0 && b == BIN_COUNT - 1)) return;
      atomicAdd(&bin_n[b], 1u);
      if (!BY_COUNT) atomicAdd(&bin_w[b], weight_of(z));
      if (level == 1) { atomicMin(&bin_lo[b], key); atomicMax(&bin_hi[b], key); }
    });
    __syncthreads();
    // this thread's bins, in order from the maximum down
    const int per_thread = BIN_COUNT / SAMPLE_THREADS;
    unsigned long long mine[per_thread], sum = 0;
#pragma unroll
    for (int i = 0; i < per_thread; ++i) {
      mine[i] = BY_COUNT ? (unsigned long long)bin_n[per_thread * tid + i] : bin_w[per_thread * tid + i];
      sum += mine[i];
    }
    if (!BY_COUNT && level == 0) {
      const unsigned long long total = block_sum_u64(sum, wide);
      bound = (unsigned long long)((double)p * (double)total);
      if (bound == 0) bound = 1;
    }
    unsigned long long before = above + block_sum_before_u64(sum, wide);
#pragma unroll
    for (int i = 0; i < per_thread; ++i) {
      if (before < bound && before + mine[i] >= bound) {             // one thread at most
        pick->bin = per_thread * tid + i;
        pick->count = (int)bin_n[per_thread * tid + i];
        pick->above = before;
      }
      before += mine[i];
    }
    __syncthreads();
    const int at = pick->bin;
    count = pick->count;
    above = pick->above;
    __syncthreads();
    if (at < 0) return false;                 // the k-th largest lies further from the maximum than the bins reach
    if (level == 0) {
      coarse = at;
      if (count <= BIN_LIST) break;
    } else {
      fine = at;
      if (bin_lo[at] == bin_hi[at]) {                                // equal values: the k-th largest, the nucleus's end
        *found = bin_lo[at];
        return true;
      }
    }
  }
  if (count > 16 * SEG) return false;
  // the bin's values, a wave's in its segment
  int pos = 0;
  bool overflow = false;
  constexpr int AHEAD = 4;
  for (int base = wbeg; base < wend && !overflow; base += AHEAD * STEP) {
    float raw[AHEAD][PER];
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int ii = base + u * STEP + PER * lane;
      if (VEC) {
        const float4 v = ii < wend ? *reinterpret_cast<const float4*>(x + ii) : make_float4(0.f, 0.f, 0.f, 0.f);
        raw[u][0] = v.x;
        if (PER > 1) { raw[u][1] = v.y; raw[u][2] = v.z; raw[u][3] = v.w; }
      } else {
        raw[u][0] = ii < wend ? x[ii] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < AHEAD; ++u) {
      const int ii = base + u * STEP + PER * lane;
      float z[PER];
      bool keep[PER];
      int cnt = 0;
#pragma unroll
      for (int c = 0; c < PER; ++c) {
        z[c] = scaled(raw[u][c], inv_t);
        keep[c] = ii + c < wend && order_key(z[c]) >= kmin_in &&
                  (fine >= 0 ? bin_of(z[c], coarse) == fine : bin_of(z[c], -1) == coarse);
        cnt += keep[c];
      }
      if (overflow || !__any(cnt)) continue;
      int incl = cnt;
#pragma unroll
      for (int d = 1; d < WAVE; d <<= 1) {
        const int o = __shfl_up(incl, d, WAVE);
        if (lane >= d) incl += o;
      }
      const int total = __shfl(incl, WAVE - 1, WAVE);
      if (pos + total > SEG) { overflow = true; continue; }
      int o = wave * SEG + pos + incl - cnt;
#pragma unroll
      for (int c = 0; c < PER; ++c)
        if (keep[c]) cand.z[o++] = z[c];
      pos += total;
    }
  }
  if (lane == 0) cand.n[wave] = overflow ? -1 : pos;
  __syncthreads();
  bool bad = false;
  for (int w = 0; w < nwaves; ++w) bad = bad || cand.n[w] < 0;
  if (bad) return false;
  // The list's keys and weights side by side where the bins lay (the 64-bit weights of the first 8 SEG fill
  // cand.lz, those of the others cand.lidx), the smallest and the largest key; then one wave halves between
  // them with no barrier.
  uint32_t* const slot_key = reinterpret_cast<uint32_t*>(cand.le);
  unsigned long long* const slot_w = reinterpret_cast<unsigned long long*>(cand.lz);
  unsigned long long* const slot_w_hi = reinterpret_cast<unsigned long long*>(cand.lidx);
  static_assert(sizeof(cand.lz) == 8 * SEG * sizeof(unsigned long long) && sizeof(cand.lidx) == sizeof(cand.lz) &&
                sizeof(cand.le) == 16 * SEG * sizeof(uint32_t), "the slots' keys and weights fill these arrays");
  uint32_t lo = 0xffffffffu, hi = 0;
  int n_all = 0;
  for (int w = 0; w < nwaves; ++w) n_all += cand.n[w];
  for (int e = tid; e < 16 * SEG; e += blockDim.x) {
    const int seg = e / SEG, j = e & (SEG - 1);
    if (j >= cand.n[seg]) continue;
    int to = j;
    for (int w = 0; w < seg; ++w) to += cand.n[w];
    const float z = cand.z[e];
    const uint32_t key = order_key(z);
    slot_key[to] = key;
    (to < 8 * SEG ? slot_w[to] : slot_w_hi[to - 8 * SEG]) = BY_COUNT ? 1ull : weight_of(z);
    lo = key < lo ? key : lo;
    hi = key > hi ? key : hi;
  }
#pragma unroll
  for (int d = WAVE / 2; d > 0; d >>= 1) {
    const uint32_t ol = __shfl_xor(lo, d, WAVE), oh = __shfl_xor(hi, d, WAVE);
    lo = ol < lo ? ol : lo;
    hi = oh > hi ? oh : hi;
  }
  __syncthreads();
  if (lane == 0) { wide[wave] = lo; wide[16 + wave] = hi; }
  __syncthreads();
  for (int w = 0; w < nwaves; ++w) {
    lo = (uint32_t)wide[w] < lo ? (uint32_t)wide[w] : lo;
    hi = (uint32_t)wide[16 + w] > hi ? (uint32_t)wide[16 + w] : hi;
  }
  if (lo > hi) return false;                                         // an empty list: cannot be
  if (wave == 0) {
    auto weight_where = [&](auto pred) {
      unsigned long long a = 0;
#pragma unroll 4
      for (int e = lane; e < n_all; e += WAVE)
        a += pred(slot_key[e]) ? (e < 8 * SEG ? slot_w[e] : slot_w_hi[e - 8 * SEG]) : 0ull;
#pragma unroll
      for (int d = WAVE / 2; d > 0; d >>= 1) a += __shfl_xor(a, d, WAVE);
      return a;
    };
    if (BY_COUNT) {                          // the largest key v with (values above the bin) + #{key >= v} >= k
      while (lo < hi) {
        const uint32_t mid = lo + (hi - lo + 1) / 2;
        if (above + weight_where([&](uint32_t key) { return key >= mid; }) >= bound) lo = mid; else hi = mid - 1;
      }
    } else {                                 // the smallest key v with (weight above the bin) + (weight of keys > v) < bound
      while (lo < hi) {
        const uint32_t mid = lo + (hi - lo) / 2;
        if (above + weight_where([&](uint32_t key) { return key > mid; }) < bound) hi = mid; else lo = mid + 1;
      }
    }
    if (lane == 0) pick->key = lo;
  }
  __syncthreads();
  lo = pick->key;
  *found = lo;
  return true;
}

// ------------------------------------------------------------------------------ parts of a row
// One block per row reads 150 K values with one compute unit, pass after pass.  For the common settings
// (temperature alone; top-k with a small k, with or without top-p and min-p; top-p or min-p without top-k) a first
// kernel cuts every row into parts of PART_VALUES values, one block each, which hold their values in
// registers and leave per part: the maximum, the sum of exp(z - that maximum) and, unless temperature stands
// alone, the candidates: every value of the part at or above a threshold that at least k of its values reach
// (k = PART_K_MAX without top-k), in index order, and that threshold.  With top-k the k largest values of
// the row, ties included, are then among the parts' candidates, and the row's k-th largest value is at or
// above every part's threshold; without top-k every value of the row at or above the highest threshold is
// a candidate.  The row's block then only scales and adds the parts' sums and walks the one part the draw
// falls into, or runs the list phase over the candidates at or above a bound it raises from the highest
// threshold.  A part with more candidates than it can pass on (many equal values) says so, and what top-p or
// min-p keep may reach below the highest threshold: the row's block then takes the way over the whole vocabulary.
#define PART_THREADS 256
#define PART_HOLD 10                                         // 16-byte pieces a thread holds
#define PART_WAVE_VALUES (4 * WAVE * PART_HOLD)              // a wave's consecutive values
#define PART_VALUES (PART_THREADS / WAVE * PART_WAVE_VALUES)
#define PART_CAND 128                                        // candidates a part can pass on
#define PART_K_MAX 64
#define PART_WORDS (4 + 2 * PART_CAND)                       // maximum, sum, candidates (-1: unbounded), their threshold; values; indices
#define MAX_PARTS 32
#define TOP_K_PARTS 16                                       // with top-k: one wave holds all candidates, two per lane and part

// What the parts leave for a row: nothing (greedy, a large top-k: the row's block does it all), maxima and
// sums (temperature alone), or also candidates: the largest k values of every part with top-k, the largest
// PART_K_MAX of every part with top-p or min-p and no top-k (what these keep is served from them if it lies
// within them).
enum { PARTS_NONE = 0, PARTS_SUMS = 1, PARTS_TOP_K = 2, PARTS_TOP_P = 3 };
__device__ __forceinline__ int parts_mode(float t, int k, int V, float p, float mp) {
  if (t == 0.f) return PARTS_NONE;
  const bool lists_fit = V <= TOP_K_PARTS * PART_VALUES;
  if (k > 0 && k < V) return (k <= PART_K_MAX && lists_fit) ? PARTS_TOP_K : PARTS_NONE;
  if ((p > 0.f && p < 1.f) || mp > 0.f) return lists_fit ? PARTS_TOP_P : PARTS_NONE;
  return PARTS_SUMS;
}

// grid (parts, rows); V a multiple of 4 and rows 16-byte aligned
__global__ void __launch_bounds__(PART_THREADS)
sample_parts_kernel(const float* __restrict__ logits, int V, int ld, const float* __restrict__ temperature,
                    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ min_p,
                    float* __restrict__ parts, int n_parts) {
  constexpr int NW = PART_THREADS / WAVE;
  __shared__ float fscratch[16];
  __shared__ float lane_max[PART_THREADS];
  __shared__ float seg_z[NW][PART_CAND];
  __shared__ int seg_i[NW][PART_CAND];
  __shared__ int seg_n[NW];
  const int part = blockIdx.x, row = blockIdx.y, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const float t = temperature[row];
  const int k = top_k[row];
  const int mode = parts_mode(t, k, V, top_p[row], min_p[row]);
  if (mode == PARTS_NONE) return;
  const float* x = logits + (size_t)row * ld;
  float* const mine = parts + ((size_t)row * n_parts + part) * PART_WORDS;
  const int pbeg = part * PART_VALUES;
  const int pend = pbeg + PART_VALUES < V ? pbeg + PART_VALUES : V;
  const int wbeg = pbeg + wave * PART_WAVE_VALUES;
  const float inv_t = 1.f / (t < 0.f ? 1.f : t);
  const float L2E = 1.4426950408889634f;
  // piece j of a lane: values wbeg + (64 j + lane) * 4 ..; past the part the part's last piece, which then does not count
  float z[PART_HOLD][4];
  bool in[PART_HOLD];
#pragma unroll
  for (int j = 0; j < PART_HOLD; ++j) {
    const int ii = wbeg + (j * WAVE + lane) * 4;
    in[j] = ii < pend;
    const float4 v = *reinterpret_cast<const float4*>(x + (in[j] ? ii : pend - 4));
    z[j][0] = scaled(v.x, inv_t); z[j][1] = scaled(v.y, inv_t); z[j][2] = scaled(v.z, inv_t); z[j][3] = scaled(v.w, inv_t);
  }
  float mloc = -INFINITY;
#pragma unroll
  for (int j = 0; j < PART_HOLD; ++j)
#pragma unroll
    for (int c = 0; c < 4; ++c) mloc = in[j] ? fmaxf(mloc, z[j][c]) : mloc;
  const float m = block_max(mloc, fscratch);
  float s = 0.f;
  if (m > -INFINITY) {
#pragma unroll
    for (int j = 0; j < PART_HOLD; ++j)
#pragma unroll
      for (int c = 0; c < 4; ++c) s += in[j] ? __builtin_amdgcn_exp2f((z[j][c] - m) * L2E) : 0.f;
  }
  s = wave_sum(s);
  __syncthreads();
  if (lane == 0) fscratch[wave] = s;
  __syncthreads();
  if (tid == 0) {
    float total = 0.f;
    for (int w = 0; w < NW; ++w) total += fscratch[w];
    mine[0] = m;
    mine[1] = total;
    reinterpret_cast<int*>(mine)[2] = 0;
  }
  if (mode == PARTS_SUMS) return;
  // A threshold that at least kk of the part's values reach, and not many more: one that kk of the threads'
  // own maxima reach (the largest values of a part mostly lie with different threads).  Every wave looks
  // for it by itself, halving the span of the maxima twelve times, with counts by ballot.
  const int asked = mode == PARTS_TOP_K ? k : PART_K_MAX;
  const int kk = asked < pend - pbeg ? asked : pend - pbeg;
  lane_max[tid] = mloc;
  __syncthreads();
  float lm[NW];
  float lowest = INFINITY;
  int with_values = 0;
#pragma unroll
  for (int i = 0; i < NW; ++i) {
    lm[i] = lane_max[lane + i * WAVE];
    lowest = lm[i] > -INFINITY ? fminf(lowest, lm[i]) : lowest;
    with_values += __popcll(__ballot(lm[i] > -INFINITY));
  }
#pragma unroll
  for (int d = WAVE / 2; d > 0; d >>= 1) lowest = fminf(lowest, __shfl_xor(lowest, d, WAVE));
  float wide = -INFINITY;                   // fewer threads with values than kk: everything is a candidate
  if (with_values >= kk) {
    float lo = lowest, hi = m;
    for (int it = 0; it < 12; ++it) {
      const float mid = 0.5f * (lo + hi);
      if (!(mid > lo && mid < hi)) break;
      int c = 0;
#pragma unroll
      for (int i = 0; i < NW; ++i) c += __popcll(__ballot(lm[i] >= mid));
      if (c >= kk) lo = mid; else hi = mid;
    }
    wide = lo;
  }
  // the candidates, in index order: a wave appends what it keeps to its segment
  int pos = 0;
  bool overflow = false;
#pragma unroll
  for (int j = 0; j < PART_HOLD; ++j) {
    unsigned long long kept[4];
    int total = 0;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      kept[c] = __ballot(in[j] && z[j][c] >= wide);
      total += __popcll(kept[c]);
    }
    if (overflow || total == 0) continue;
    if (pos + total > PART_CAND) { overflow = true; continue; }
    const unsigned long long below = (1ull << lane) - 1ull;
    int o = pos;                            // values of lower lanes first, then this lane's own in order
#pragma unroll
    for (int c = 0; c < 4; ++c) o += __popcll(kept[c] & below);
    const int ii = wbeg + (j * WAVE + lane) * 4;
#pragma unroll
    for (int c = 0; c < 4; ++c)
      if ((kept[c] >> lane) & 1ull) { seg_z[wave][o] = z[j][c]; seg_i[wave][o] = ii + c; ++o; }
    pos += total;
  }
  if (lane == 0) seg_n[wave] = overflow ? -1 : pos;
  __syncthreads();
  int n_all = 0, off = 0;
  bool bad = false;
  for (int w = 0; w < NW; ++w) {
    bad = bad || seg_n[w] < 0;
    if (w < wave) off += seg_n[w];
    n_all += seg_n[w];
  }
  if (bad || n_all > PART_CAND || n_all < kk) {
    if (tid == 0) reinterpret_cast<int*>(mine)[2] = -1;
    return;
  }
  for (int j = lane; j < seg_n[wave]; j += WAVE) {
    mine[4 + off + j] = seg_z[wave][j];
    reinterpret_cast<int*>(mine)[4 + PART_CAND + off + j] = seg_i[wave][j];
  }
  if (tid == 0) {
    reinterpret_cast<int*>(mine)[2] = n_all;
    // With top-k: k values of the row are at or above it, so the row's k-th largest is.  With top-p: every
    // value of the part at or above it is listed.  A part that lists all it has sets no bound (-inf).
    mine[3] = kk == asked ? wide : -INFINITY;
  }
}

// Each wave owns a contiguous range of the vocabulary, so sums over a wave's range are sums over
// consecutive indices and the draw can walk the index order wave by wave.
// With `parts` (what sample_parts_kernel left for each row, n_parts parts a row) the two settings it serves take
// their sums or candidates from there.
template <bool VEC>
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(const float* __restrict__ logits, int V, int ld, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const float* __restrict__ min_p, const unsigned* __restrict__ seed_lo,
              const unsigned* __restrict__ seed_hi, const int* __restrict__ position,
              int* __restrict__ out, const float* __restrict__ parts, int n_parts) {
  __shared__ float fscratch[16];
  __shared__ int iscratch[16];
  __shared__ float wave_tot[16];
  __shared__ int chosen, range_of;
  __shared__ float part_m[MAX_PARTS], part_s[MAX_PARTS];
  __shared__ int part_n[MAX_PARTS];
  __shared__ float part_w[MAX_PARTS];
  __shared__ float step_sum[WAVE];
  __shared__ int step_kept[WAVE];
  __shared__ unsigned long long wide[32];
  __shared__ BinPick bin_pick;
  __shared__ Candidates cand;
  constexpr int STEP = VEC ? 4 * WAVE : WAVE;        // values a wave reads per access
  const int row = blockIdx.x, tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
  const int nwaves = blockDim.x / WAVE;
  const float* x = logits + (size_t)row * ld;
  // every per-row number, and this thread's part of what the first kernel left, asked for at once
  const float t = temperature[row];
  const int k_row = top_k[row];
  const float p_row = top_p[row], mp_row = min_p[row];
  const uint64_t seed = ((uint64_t)seed_hi[row] << 32) | (uint64_t)seed_lo[row];
  const uint32_t position_row = (uint32_t)position[row];
  float4 header = make_float4(0.f, 0.f, 0.f, 0.f);
  if (parts && tid < n_parts) header = *reinterpret_cast<const float4*>(parts + ((size_t)row * n_parts + tid) * PART_WORDS);
  const int per = ((V + nwaves - 1) / nwaves + STEP - 1) / STEP * STEP;
  const int wbeg = wave * per < V ? wave * per : V;
  const int wend = wbeg + per < V ? wbeg + per : V;

  const int mode = parts ? parts_mode(t, k_row, V, p_row, mp_row) : PARTS_NONE;
  if (mode != PARTS_NONE) {
    const float* const mine = parts + (size_t)row * n_parts * PART_WORDS;
    const int* const mine_i = reinterpret_cast<const int*>(mine);
    const float inv_t = 1.f / (t < 0.f ? 1.f : t);
    const float L2E = 1.4426950408889634f;
    // the parts' maxima, sums and numbers of candidates: one load each, side by side, then shared
    if (tid < n_parts) {
      part_m[tid] = header.x;
      part_s[tid] = header.y;
      part_n[tid] = __float_as_int(header.z);
      part_w[tid] = header.w;
    }
    __syncthreads();
    float m = -INFINITY;
    for (int p = 0; p < n_parts; ++p) m = fmaxf(m, part_m[p]);
    const float uniform = uniform_from_seed(seed, position_row);
    if (mode == PARTS_TOP_K || mode == PARTS_TOP_P) {
      bool bad = false;
      float bound = -INFINITY;              // the highest of the parts' thresholds
      float all_weight = 0.f;               // every part's sum, brought to the row's maximum, in order
      for (int p = 0; p < n_parts; ++p) {
        bad = bad || part_n[p] < 0;
        bound = fmaxf(bound, part_w[p]);
        all_weight += part_s[p] * __builtin_amdgcn_exp2f((part_m[p] - m) * L2E);
      }
      // min-p alone keeps the values within -log(min_p) of the maximum (logf: the hardware's log2)
      const bool top_p_row = p_row > 0.f && p_row < 1.f;
      const float min_p_reach = m + (__builtin_amdgcn_logf(mp_row) - 0.01f) / L2E;
      if (!bad) {
        // One wave does the rest.  It holds all candidates (two per lane and part).  With top-k the row's k-th
        // largest value is at or above every part's threshold; with top-p alone every value of the row at or
        // above the highest threshold is a candidate, so a nucleus that ends above it is among them.  The wave
        // raises that bound by halving the span to the maximum twelve times, as long as k candidates (counts by
        // ballot), or a little more than the share p of all weight, stay at or above it, puts what does side
        // by side, still in index order, and runs the list phase on that short list.
        if (wave == 0) {
          constexpr int HELD = 2 * TOP_K_PARTS;
          float held[HELD];
#pragma unroll
          for (int i = 0; i < HELD; ++i) {
            const int pp = i >> 1, j = lane + (i & 1) * WAVE;
            held[i] = (pp < n_parts && j < part_n[pp]) ? mine[pp * PART_WORDS + 4 + j] : -INFINITY;
          }
          float lo = bound, hi = m;
          bool served = true;
          const bool min_p_alone = mode == PARTS_TOP_P && !top_p_row;
          if (min_p_alone && lo > -INFINITY) {
            served = min_p_reach >= lo;     // all that min-p keeps are candidates, or the row is not served
            lo = min_p_reach;
          }
          if (mode == PARTS_TOP_K) {
            if (lo > -INFINITY) {
              for (int it = 0; it < 12; ++it) {
                const float mid = 0.5f * (lo + hi);
                if (!(mid > lo && mid < hi)) break;
                int c = 0;
#pragma unroll
                for (int i = 0; i < HELD; ++i) c += __popcll(__ballot(held[i] >= mid));
                if (c >= k_row) lo = mid; else hi = mid;
              }
            }
          } else if (!min_p_alone && lo > -INFINITY) {
            // first the weight at the bound itself (the nucleus must lie within the candidates), then the halvings
            const float need = p_row * all_weight * 1.001f;
            for (int it = 0; it <= 12 && served; ++it) {
              const float mid = it == 0 ? lo : 0.5f * (lo + hi);
              if (it > 0 && !(mid > lo && mid < hi)) break;
              float a = 0.f;
#pragma unroll
              for (int i = 0; i < HELD; ++i) a += held[i] >= mid ? __builtin_amdgcn_exp2f((held[i] - m) * L2E) : 0.f;
              const bool enough = wave_sum(a) >= need;
              if (it == 0) served = enough;
              else if (enough) lo = mid;
              else hi = mid;
            }
          }
          int n_all = 0;
#pragma unroll
          for (int i = 0; i < HELD; ++i) {
            const int pp = i >> 1, j = lane + (i & 1) * WAVE;
            const bool keep = pp < n_parts && j < part_n[pp] && held[i] >= lo;
            const unsigned long long kept = __ballot(keep);
            const int o = n_all + __popcll(kept & ((1ull << lane) - 1ull));
            if (keep && o < 4 * WAVE) {
              cand.lz[o] = held[i];
              cand.le[o] = __builtin_amdgcn_exp2f((held[i] - m) * L2E);
              cand.lidx[o] = mine_i[pp * PART_WORDS + 4 + PART_CAND + j];
            }
            n_all += __popcll(kept);
          }
          __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
          __builtin_amdgcn_wave_barrier();
          __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
          int token = -1;                   // stays so where the short list cannot serve the row: the long way
          if (served && n_all <= 4 * WAVE)
            token = draw_from_short_list(cand, n_all, mode == PARTS_TOP_K, k_row, p_row, mp_row, all_weight, order_key(lo),
                                         order_key(m), uniform, lane);
          if (lane == 0) {
            if (token >= 0) out[row] = token;
            chosen = token >= 0 ? 0 : -1;
          }
        }
        __syncthreads();
        if (chosen >= 0) return;
      }
    } else {
      // every part's sum, brought to the row's maximum, in order; the part in which the running sum passes the target
      float total = 0.f;
      for (int p = 0; p < n_parts; ++p) total += part_s[p] * __builtin_amdgcn_exp2f((part_m[p] - m) * L2E);
      const float target = uniform * total;
      float run = 0.f;
      int in_part = -1;
      for (int p = 0; p < n_parts && in_part < 0; ++p) {
        const float w = part_s[p] * __builtin_amdgcn_exp2f((part_m[p] - m) * L2E);
        if (w > 0.f && run + w > target) in_part = p;
        else run += w;
      }
      if (in_part >= 0) {
        const int rbeg = in_part * PART_VALUES;
        const int picked = walk_range<VEC>(x, rbeg, rbeg + PART_VALUES < V ? rbeg + PART_VALUES : V, run, target, inv_t, m,
                                           0u, 0.f, step_sum, step_kept);
        if (picked >= 0) {
          if (tid == 0) out[row] = picked;
          return;
        }
      }
    }
    __syncthreads();                        // the way over the whole vocabulary
  }

  if (t == 0.f) {  // greedy: first index of the maximum
    float best = -INFINITY;
    int best_i = 0x7fffffff;
    for_range<VEC>(x, wbeg, wend, lane, [&](int i, float v) {
      if (v > best || best_i == 0x7fffffff) { best = v; best_i = i; }
    });
    const float m = block_max(best, fscratch);
    int cand = (best == m && best_i != 0x7fffffff) ? best_i : 0x7fffffff;
#pragma unroll
    for (int s = WAVE / 2; s > 0; s >>= 1) { const int o = __shfl_xor(cand, s, WAVE); cand = o < cand ? o : cand; }
    __syncthreads();
    if (lane == 0) iscratch[wave] = cand;
    __syncthreads();
    if (tid == 0) {
      int r = 0x7fffffff;
      for (int w = 0; w < nwaves; ++w) r = iscratch[w] < r ? iscratch[w] : r;
      out[row] = r == 0x7fffffff ? 0 : r;
    }
    return;
  }

  // z = x / T is taken as x * (1 / T); the exponential is the hardware's 2^x
  const float inv_t = 1.f / (t < 0.f ? 1.f : t);  // the reference maps T <= 0 to 1 (sampler.py:41)
  const float L2E = 1.4426950408889634f;
  float mloc = -INFINITY;
  for_range<VEC, 8>(x, wbeg, wend, lane, [&](int, float v) { mloc = fmaxf(mloc, v); });   // 1 / T is positive
  const float m = scaled(block_max(mloc, fscratch), inv_t);
  const uint32_t key_max = order_key(m);
  uint32_t kmin = 0;
#define E_OF(z) __builtin_amdgcn_exp2f(((z) - m) * L2E)

  const int k = k_row;
  const bool top_k_on = k > 0 && k < V, top_p_on = p_row > 0.f && p_row < 1.f;
  // (top-p alone on a row that the parts' candidates could not serve: its nucleus is long, the bins find its end)
  if (((top_k_on && k <= SMALL_K_MAX) || (!top_k_on && top_p_on && mode != PARTS_TOP_P)) && blockDim.x == SAMPLE_THREADS) {
    const int token = sample_small_k<VEC>(x, wbeg, wend, inv_t, m, top_k_on ? k : 0, p_row, mp_row,
                                          uniform_from_seed(seed, position_row), cand, fscratch, iscratch);
    if (token >= 0) {
      if (tid == 0) out[row] = token;
      return;
    }
    __syncthreads();
  }
  bool by_bins = false;
  if (k > 0 && k < V && blockDim.x == SAMPLE_THREADS)
    by_bins = threshold_by_bins<VEC, true>(x, wbeg, wend, inv_t, m, 0u, k, 0.f, cand, wide, &bin_pick, &kmin);
  if (k > 0 && k < V && !by_bins) {  // largest key v with #{key >= v} >= k
    uint32_t lo = 0, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1) / 2;
      int c = 0;
      for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) { c += order_key(scaled(v, inv_t)) >= mid; });
      if (block_sum_int(c, iscratch) >= k) lo = mid; else hi = mid - 1;
    }
    kmin = lo;
  }

  const float p = p_row;
  by_bins = false;
  if (p > 0.f && p < 1.f && blockDim.x == SAMPLE_THREADS) {
    uint32_t at = 0;
    by_bins = threshold_by_bins<VEC, false>(x, wbeg, wend, inv_t, m, kmin, 0, p, cand, wide, &bin_pick, &at);
    if (by_bins) kmin = at;
  }
  if (p > 0.f && p < 1.f && !by_bins) {  // smallest key v with (mass of keys > v) < p * (mass kept so far)
    float s = 0.f;
    for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
      const float z = scaled(v, inv_t);
      if (order_key(z) >= kmin) s += E_OF(z);
    });
    const float bound = p * block_sum(s, fscratch);
    uint32_t lo = kmin, hi = key_max;
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo) / 2;
      float a = 0.f;
      for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
        const float z = scaled(v, inv_t);
        if (order_key(z) > mid) a += E_OF(z);
      });
      if (block_sum(a, fscratch) < bound) hi = mid; else lo = mid + 1;
    }
    kmin = lo;
  }

  const float mp = mp_row;
  float s = 0.f;
  if (kmin == 0 && !(mp > 0.f)) {          // nothing filtered: every value counts (3 instructions a value)
    for_range<VEC, 8>(x, wbeg, wend, lane, [&](int, float v) { s += E_OF(scaled(v, inv_t)); });
  } else {
    for_range<VEC>(x, wbeg, wend, lane, [&](int, float v) {
      const float z = scaled(v, inv_t);
      const float e = E_OF(z);
      if (order_key(z) >= kmin && e >= mp) s += e;
    });
  }
  s = wave_sum(s);
  if (tid == 0) { chosen = -1; range_of = -1; }
  if (lane == 0) wave_tot[wave] = s;
  __syncthreads();
  float base = 0.f, total = 0.f;
  for (int w = 0; w < nwaves; ++w) {       // sequential sums: the running total never decreases
    if (w == wave) base = total;
    total += wave_tot[w];
  }
  const float target = uniform_from_seed(seed, position_row) * total;
  const bool mine = s > 0.f && base + s > target && !(base > target);   // exactly one wave
  if (mine && lane == 0) range_of = wave;
  __syncthreads();
  const int rw = range_of;
  if (rw >= 0) {
    float run = 0.f;
    for (int w = 0; w < rw; ++w) run += wave_tot[w];
    const int rbeg = rw * per < V ? rw * per : V;
    const int picked = walk_range<VEC>(x, rbeg, rbeg + per < V ? rbeg + per : V, run, target, inv_t, m, kmin, mp,
                                       step_sum, step_kept);
    if (tid == 0) chosen = picked;
  }
  __syncthreads();
  if (chosen < 0) {  // rounding pushed the target past the total: take the last kept index
    int last = -1;
    for_range<VEC>(x, wbeg, wend, lane, [&](int i, float v) {
      const float z = scaled(v, inv_t);
      if (order_key(z) >= kmin && E_OF(z) >= mp) last = i > last ? i : last;
    });
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
#undef E_OF
}

// Floats of workspace with which ullm_sample cuts the rows into parts (0: it would not: rows that are not
// 16-byte aligned, or a vocabulary of more than MAX_PARTS parts).
extern "C" long long ullm_sample_workspace(int n_rows, int V, int ld) {
  if (n_rows <= 0 || V <= 0 || V % 4 || ld % 4 || n_rows > 65535) return 0;
  const int n_parts = (V + PART_VALUES - 1) / PART_VALUES;
  return n_parts > MAX_PARTS ? 0 : (long long)n_rows * n_parts * PART_WORDS;
}

// `workspace`: null, or ullm_sample_workspace(n_rows, V, ld) floats (then, if that is not 0, the rows are cut into
// parts by a first kernel).
extern "C" int ullm_sample(const float* logits, int n_rows, int V, int ld, const float* temperature,
                           const int* top_k, const float* top_p, const float* min_p,
                           const unsigned* seed_lo, const unsigned* seed_hi, const int* position,
                           int* out, float* workspace, hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (V <= 0 || ld < V) return ULLM_ERR_SHAPE;
  const bool vec = V % 4 == 0 && ld % 4 == 0 && !((uintptr_t)logits & 15);
  const int n_parts = (V + PART_VALUES - 1) / PART_VALUES;
  float* const parts = vec && workspace && ullm_sample_workspace(n_rows, V, ld) > 0 ? workspace : nullptr;
  if (parts) {
    hipLaunchKernelGGL(sample_parts_kernel, dim3(n_parts, n_rows), dim3(PART_THREADS), 0, stream, logits, V, ld,
                       temperature, top_k, top_p, min_p, parts, n_parts);
    const int rc = (int)hipGetLastError();
    if (rc != 0) return rc;
  }
  if (vec)
    hipLaunchKernelGGL(sample_kernel<true>, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, V, ld,
                       temperature, top_k, top_p, min_p, seed_lo, seed_hi, position, out, parts, n_parts);
  else
    hipLaunchKernelGGL(sample_kernel<false>, dim3(n_rows), dim3(SAMPLE_THREADS), 0, stream, logits, V, ld,
                       temperature, top_k, top_p, min_p, seed_lo, seed_hi, position, out, nullptr, 0);
  ULLM_LAUNCH_CHECK();
}
