// Paged grouped-query attention on the matrix cores (bfloat16 operands, 32-bit accumulation),
// for decoded tokens (split over the keys, then reduced) and for prompt portions.
//
// One wave owns 16 "columns": in decode mode the query heads of one token that share a kv head,
// in prompt mode 16 consecutive tokens of one request for one query head.  Per 32 keys it computes
//   S^T[key, col]   = K[key, :] . Q[col, :]        (v_mfma_f32_16x16x32_bf16: A = K rows, B = Q columns)
//   O^T[dim, col]  += V^T[dim, key] * P^T[key, col] (A = values, transposed inside the page, B = P)
// In the 16x16 result layout a lane holds 4 keys of one column, so the probabilities a lane has are
// exactly the ones it must feed as the B operand of the second product: nothing moves between lanes.
// Both operands of both products are plain 8- or 16-byte loads from the paged cache:
//   keys   [page, kv_head, row, head_dim],  values [page, kv_head, head_dim, row].
// Softmax state (maximum, sum) is 32-bit and per column; the scale and log2(e) are folded into one
// multiply so that the exponential is a single v_exp_f32.
//
// Semantics as in the general kernel: causal with the queries at the end of the keys, optional
// window, query head h reads kv head h / (nq / nkv) (ullm/layers/attention.py:76-104,271,298-309).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define NEG_BIG (-1.0e30f)

union Pack8 {
  bf16x8_t v;
  uint4 u4;
  uint2 u2[2];
  uint32_t w[4];
  bf16_t h[8];
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// One 32-key tile of a request's cache in registers: the operands of both products.
template <int NQK>
struct KVTile {
  Pack8 k[2][NQK];        // k[sb][ch]: keys key0 + 16 sb + (lane & 15), dims 32 ch + 8 g .. +8
  uint2 v[2 * NQK][2];    // v[n][sb]: dim 16 n + (lane & 15), keys key0 + 16 sb + 4 g .. +4
  int ok[2];              // the 16-key half holds a page
};

// Page ids of up to 64 consecutive 16-key sub-blocks, one per lane, fetched with a single load so
// that the key and value loads of later tiles do not wait for a table lookup each.
struct PageWindow {
  int base;               // first sub-block (key / 16) held
  int page;               // lane i: page id of sub-block base + i (or -1)
};

__device__ __forceinline__ PageWindow load_pages(int key_from, int key_end, const int* __restrict__ bt, int page_size) {
  PageWindow w;
  w.base = key_from >> 4;
  const int kb = (w.base + (int)(threadIdx.x & 63)) << 4;
  w.page = kb < key_end ? bt[kb / page_size] : -1;
  return w;
}

template <int NQK>
__device__ __forceinline__ void load_tile(KVTile<NQK>& t, int key0, const PageWindow& pw,
                                          const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                                          int page_size, int nkv, int kvh) {
  constexpr int HD = 32 * NQK;
  const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    const int kb = key0 + 16 * sb;
    const int page = __builtin_amdgcn_readlane(pw.page, (kb >> 4) - pw.base);
    const int off = kb % page_size;
    t.ok[sb] = page >= 0;
    if (page >= 0) {
      const bf16_t* kp = k_pool + (((size_t)page * nkv + kvh) * page_size + off + c) * HD + 8 * g;
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) t.k[sb][ch].u4 = *reinterpret_cast<const uint4*>(kp + 32 * ch);
      const bf16_t* vp = v_pool + (((size_t)page * nkv + kvh) * HD + c) * page_size + off + 4 * g;
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) t.v[n][sb] = *reinterpret_cast<const uint2*>(vp + (size_t)16 * n * page_size);
    } else {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) t.k[sb][ch].u4 = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) t.v[n][sb] = make_uint2(0, 0);
    }
  }
}

// Scores, softmax update and value product for one tile held in registers.
template <int NQK>
__device__ __forceinline__ void process_tile(const KVTile<NQK>& cur, int key0, const Pack8 (&qreg)[NQK], int col_lo,
                                             int col_hi, int max_hi, float scale_log2e, f32x4_t (&acc)[2 * NQK],
                                             float& m, float& l) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
  f32x4_t s[2];
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    s[sb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch)
      s[sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(cur.k[sb][ch].v, qreg[ch].v, s[sb], 0, 0, 0);
  }
  // scores of keys key0 + 16 sb + 4 g + r for this lane's column; mask, running maximum
  float tile_max = NEG_BIG;
#pragma unroll
  for (int sb = 0; sb < 2; ++sb)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int kk = key0 + 16 * sb + 4 * g + r;
      const bool ok = cur.ok[sb] && kk >= col_lo && kk <= col_hi;
      const float v = ok ? s[sb][r] * scale_log2e : NEG_BIG;
      s[sb][r] = v;
      tile_max = fmaxf(tile_max, v);
    }
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 16, 64));
  tile_max = fmaxf(tile_max, __shfl_xor(tile_max, 32, 64));
  const float m_new = fmaxf(m, tile_max);
  const float alpha = fast_exp2(m - m_new);
  Pack8 p;
  float psum = 0.f;
#pragma unroll
  for (int sb = 0; sb < 2; ++sb) {
    float e[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      // a masked score stays at NEG_BIG: its weight is zero even while m_new is still NEG_BIG
      e[r] = s[sb][r] > 0.5f * NEG_BIG ? fast_exp2(s[sb][r] - m_new) : 0.f;
      psum += e[r];
    }
    p.w[2 * sb] = pack2_bf16(e[0], e[1]);
    p.w[2 * sb + 1] = pack2_bf16(e[2], e[3]);
  }
  l = l * alpha + psum;
  m = m_new;
  const bool edge = key0 + 32 > max_hi + 1;     // some keys of the tile hold no written data
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) {
    Pack8 a;
    a.u2[0] = cur.v[n][0];
    a.u2[1] = cur.v[n][1];
    if (edge) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (key0 + 16 * (j >> 2) + 4 * g + (j & 3) > max_hi) a.h[j] = 0;
    }
    f32x4_t o = acc[n];
    o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
    acc[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, p.v, o, 0, 0, 0);
  }
}

// The work of one wave.  NQK = head_dim / 32.
//   col_q      : pointer to this lane's column's query row (null if the column is padding)
//   col_lo/hi  : first and last key the column may see (hi < lo for padding)
//   key_begin/key_end : the wave's key range [begin, end), begin a multiple of 32
//   max_hi     : largest key position that holds written data for this request
// Results: acc[n][r] = O^T[16n + 4g + r][col] (unnormalised), m (log2 domain), l (this lane's share
// of the sum; the four lanes of a column add up to the column's sum).
// Page ids are fetched 1024 keys at a time; the loads of the next DEPTH (1 or 2) tiles are in flight
// while the current one is worked on (2 needs about 230 registers, 1 about 130).
template <int NQK, int DEPTH = 2>
__device__ __forceinline__ void attend_range(
    const bf16_t* __restrict__ col_q, int col_lo, int col_hi, int key_begin, int key_end, int max_hi,
    const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool, const int* __restrict__ bt,
    int page_size, int nkv, int kvh, float scale_log2e, f32x4_t (&acc)[2 * NQK], float& m, float& l) {
  const int lane = threadIdx.x & 63, g = lane >> 4;
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) acc[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  m = NEG_BIG;
  l = 0.f;
  if (key_begin >= key_end) return;
  PageWindow pw = load_pages(key_begin, key_end, bt, page_size);
  Pack8 qreg[NQK];
#pragma unroll
  for (int ch = 0; ch < NQK; ++ch) {
    if (col_q) qreg[ch].u4 = *reinterpret_cast<const uint4*>(col_q + 32 * ch + 8 * g);
    else qreg[ch].u4 = make_uint4(0, 0, 0, 0);
  }
  for (int base = key_begin; base < key_end; base += 1024) {
    if (base != key_begin) pw = load_pages(base, key_end, bt, page_size);
    const int stop = base + 1024 < key_end ? base + 1024 : key_end;
    if (DEPTH == 1) {
      KVTile<NQK> a, b;
      load_tile<NQK>(a, base, pw, k_pool, v_pool, page_size, nkv, kvh);
      for (int key0 = base; key0 < stop; key0 += 64) {
        if (key0 + 32 < stop) load_tile<NQK>(b, key0 + 32, pw, k_pool, v_pool, page_size, nkv, kvh);
        process_tile<NQK>(a, key0, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l);
        if (key0 + 32 >= stop) break;
        if (key0 + 64 < stop) load_tile<NQK>(a, key0 + 64, pw, k_pool, v_pool, page_size, nkv, kvh);
        process_tile<NQK>(b, key0 + 32, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l);
      }
      continue;
    }
    KVTile<NQK> t0, t1, t2;
    load_tile<NQK>(t0, base, pw, k_pool, v_pool, page_size, nkv, kvh);
    if (base + 32 < stop) load_tile<NQK>(t1, base + 32, pw, k_pool, v_pool, page_size, nkv, kvh);
    // three buffers in rotation: while tile i is worked on, tiles i+1 and i+2 are loading
    for (int key0 = base; key0 < stop; key0 += 96) {
      if (key0 + 64 < stop) load_tile<NQK>(t2, key0 + 64, pw, k_pool, v_pool, page_size, nkv, kvh);
      process_tile<NQK>(t0, key0, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l);
      if (key0 + 32 >= stop) break;
      if (key0 + 96 < stop) load_tile<NQK>(t0, key0 + 96, pw, k_pool, v_pool, page_size, nkv, kvh);
      process_tile<NQK>(t1, key0 + 32, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l);
      if (key0 + 64 >= stop) break;
      if (key0 + 128 < stop) load_tile<NQK>(t1, key0 + 128, pw, k_pool, v_pool, page_size, nkv, kvh);
      process_tile<NQK>(t2, key0 + 64, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l);
    }
  }
}

// ------------------------------------------------------------------------------- decode
// grid (num_splits, nkv * col_groups, n_tokens), block 64 * WAVES.  The keys [lo, pos] of a token are
// cut into num_splits * WAVES equal shares of whole 32-key tiles (so the cut depends on the token's
// own length, not on the batch); block x takes shares x * WAVES ..., one per wave.  The waves then merge
// their (maximum, sum, output) pairwise through shared memory, lane by lane (a lane's values have the
// same meaning in every wave), halving the number of waves each round in a fixed order.  Wave 0 ends
// with the block's result: with one split that is the output; otherwise it goes to the workspace and
// a second, small kernel adds the splits in split order.  (A single kernel in which the last block to
// finish does that sum needs a device-wide memory fence per block, which on a part with one L2 per
// XCD costs far more than the second launch.)
template <int NQK, int WAVES>
__global__ void __launch_bounds__(64 * WAVES)
attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                        const int* __restrict__ token_list, const int* __restrict__ positions,
                        const int* __restrict__ token_entry, const int* __restrict__ block_table,
                        int bt_stride, int page_size, int nq, int nkv, float scale_log2e, int window,
                        int num_splits, float* __restrict__ part) {
  constexpr int HD = 32 * NQK;
  constexpr int ROW = HD + 4;                       // output dims, then maximum and sum (rows stay 16-byte aligned)
  constexpr int PER_LANE = 8 * NQK + 2;             // a lane's accumulators, maximum and sum share
  __shared__ float merge[WAVES / 2][PER_LANE][64];  // [writer][value][lane]: conflict-free
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, c = lane & 15;
  const int split = blockIdx.x;
  const int G = nq / nkv;
  const int groups = (G + 15) / 16;
  const int kvh = blockIdx.y / groups, cg = blockIdx.y % groups;
  const int item = blockIdx.z;
  const int t = token_list ? token_list[item] : item;
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first = lo & ~31;
  const int tiles = (pos + 1 - first + 31) / 32;
  const int share = 32 * ((tiles + num_splits * WAVES - 1) / (num_splits * WAVES));
  int begin = first + (split * WAVES + wave) * share, end = begin + share;
  if (end > pos + 1) end = pos + 1;
  const int head_in_group = cg * 16 + c;
  const bool col_ok = head_in_group < G;
  const int head = kvh * G + head_in_group;
  f32x4_t acc[2 * NQK];
  float m, l;
  attend_range<NQK, (WAVES > 4 ? 1 : 2)>(
      col_ok ? q + (size_t)t * q_stride + (size_t)head * HD : nullptr, lo, col_ok ? pos : -1, begin, end, pos,
      k_pool, v_pool, block_table + (size_t)token_entry[t] * bt_stride, page_size, nkv, kvh, scale_log2e, acc, m, l);
#pragma unroll
  for (int half = WAVES / 2; half >= 1; half >>= 1) {
    if (wave >= half && wave < 2 * half) {          // the upper half of the live waves hands over
      float (*w)[64] = merge[wave - half];
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) w[4 * n + r][lane] = acc[n][r];
      w[8 * NQK][lane] = m;
      w[8 * NQK + 1][lane] = l;
    }
    __syncthreads();
    if (wave < half) {
      const float (*w)[64] = merge[wave];
      const float m_b = w[8 * NQK][lane], l_b = w[8 * NQK + 1][lane];
      const float M = fmaxf(m, m_b);
      const float fa = fast_exp2(m - M), fb = fast_exp2(m_b - M);
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[n][r] = acc[n][r] * fa + w[4 * n + r][lane] * fb;
      l = l * fa + l_b * fb;
      m = M;
    }
    __syncthreads();
  }
  if (wave != 0) return;
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!col_ok) return;
  if (num_splits == 1) {
    const float inv = l > 0.f ? 1.f / l : 0.f;
    bf16_t* op = out + (size_t)t * out_stride + (size_t)head * HD;
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n)
      *reinterpret_cast<uint2*>(op + 16 * n + 4 * g) =
          make_uint2(pack2_bf16(acc[n][0] * inv, acc[n][1] * inv), pack2_bf16(acc[n][2] * inv, acc[n][3] * inv));
    return;
  }
  // partial of this block: [item][head][split][ROW]
  float* pp = part + (((size_t)item * nq + head) * num_splits + split) * ROW;
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n)
    *reinterpret_cast<float4*>(pp + 16 * n + 4 * g) = make_float4(acc[n][0], acc[n][1], acc[n][2], acc[n][3]);
  if (g == 0) {
    pp[HD] = m;
    pp[HD + 1] = l;
  }
}

// Adds the splits' partials [item][head][split][head_dim + 4] in split order.  grid (n_items, nq),
// one wave: lane s first reads split s's maximum and sum (64 splits at a time), then every lane sums
// its output dims over the splits with the splits' weights passed round by shuffles.
__global__ void __launch_bounds__(64)
attention_reduce_kernel(const float* __restrict__ part, bf16_t* __restrict__ out, int out_stride,
                        const int* __restrict__ token_list, int nq, int hd, int num_splits) {
  const int item = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int t = token_list ? token_list[item] : item;
  const int row = hd + 4;
  const float* pp = part + ((size_t)item * nq + head) * num_splits * row;
  float M = NEG_BIG;
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const int sp = s0 + lane;
    M = fmaxf(M, wave_max(sp < num_splits ? pp[sp * row + hd] : NEG_BIG));
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};       // head_dim <= 256: dims lane, lane + 64, ...
  float L = 0.f;
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const int sp = s0 + lane;
    const bool ok = sp < num_splits;
    const float f = ok ? fast_exp2(pp[sp * row + hd] - M) : 0.f;
    L += wave_sum(ok ? pp[sp * row + hd + 1] * f : 0.f);
    const int n = num_splits - s0 < 64 ? num_splits - s0 : 64;
    for (int j = 0; j < n; ++j) {
      const float fj = __shfl(f, j, 64);
      const float* pj = pp + (size_t)(s0 + j) * row;
#pragma unroll
      for (int r = 0; r < 4; ++r)
        if (lane + 64 * r < hd) acc[r] += pj[lane + 64 * r] * fj;
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  bf16_t* op = out + (size_t)t * out_stride + (size_t)head * hd;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (lane + 64 * r < hd) op[lane + 64 * r] = f32_to_bf16_bits(acc[r] * inv);
}

// ------------------------------------------------------------------------------- prompt portions
// grid (n_tiles, nkv * ceil(G / waves)), block 64 * waves with waves = min(G, 4): one wave per query
// head, the waves of a block share a kv head (and so the cache lines they read); tile = (first
// token, number of tokens <= 16) of one request; every wave walks all keys its tokens see.
template <int NQK>
__global__ void __launch_bounds__(256)
attention_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                         const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                         const int* __restrict__ tiles, const int* __restrict__ positions,
                         const int* __restrict__ token_entry, const int* __restrict__ block_table,
                         int bt_stride, int page_size, int nq, int nkv, float scale_log2e, int window) {
  constexpr int HD = 32 * NQK;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, g = lane >> 4, c = lane & 15;
  const int G = nq / nkv;
  const int waves = blockDim.x >> 6, hgroups = (G + waves - 1) / waves;
  const int kvh = blockIdx.y / hgroups;
  const int head_in_group = (blockIdx.y % hgroups) * waves + wave;
  if (head_in_group >= G) return;
  const int head = kvh * G + head_in_group;
  const int first = tiles[2 * blockIdx.x], count = tiles[2 * blockIdx.x + 1];
  const bool col_ok = c < count;
  const int t = first + (col_ok ? c : 0);
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int last_pos = positions[first + count - 1];
  const int first_pos = positions[first];
  const int tile_lo = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  f32x4_t acc[2 * NQK];
  float m, l;
  attend_range<NQK>(col_ok ? q + (size_t)t * q_stride + (size_t)head * HD : nullptr, lo, col_ok ? pos : -1,
                    tile_lo & ~31, last_pos + 1, last_pos, k_pool, v_pool,
                    block_table + (size_t)token_entry[first] * bt_stride, page_size, nkv, kvh, scale_log2e,
                    acc, m, l);
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!col_ok) return;
  const float inv = l > 0.f ? 1.f / l : 0.f;
  bf16_t* op = out + (size_t)t * out_stride + (size_t)head * HD;
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) {
    uint2 w;
    w.x = (uint32_t)f32_to_bf16_bits(acc[n][0] * inv) | ((uint32_t)f32_to_bf16_bits(acc[n][1] * inv) << 16);
    w.y = (uint32_t)f32_to_bf16_bits(acc[n][2] * inv) | ((uint32_t)f32_to_bf16_bits(acc[n][3] * inv) << 16);
    *reinterpret_cast<uint2*>(op + 16 * n + 4 * g) = w;
  }
}

static bool supported_hd(int hd) { return hd == 32 || hd == 64 || hd == 96 || hd == 128 || hd == 256; }

#define DISPATCH_NQK(hd, CALL)            \
  switch ((hd) / 32) {                    \
    case 1: { CALL(1); break; }           \
    case 2: { CALL(2); break; }           \
    case 3: { CALL(3); break; }           \
    case 4: { CALL(4); break; }           \
    case 8: { CALL(8); break; }           \
    default: return ULLM_ERR_UNSUPPORTED; \
  }

// 1 if this family takes the shape (bfloat16 only), else 0.
extern "C" int ullm_attention_mfma_supports(int hd, int page_size, int nq, int nkv) {
  return supported_hd(hd) && page_size > 0 && page_size % 16 == 0 && nkv > 0 && nq % nkv == 0;
}

// Workspace floats needed for `n_items` tokens split `num_splits` ways.
extern "C" long long ullm_attention_decode_workspace(int n_items, int nq, int hd, int num_splits) {
  return num_splits <= 1 ? 0 : (long long)n_items * nq * num_splits * (hd + 4);
}
extern "C" int ullm_attention_decode(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, float* workspace, hipStream_t stream) {
  if (n_items <= 0) return 0;
  if (!ullm_attention_mfma_supports(hd, page_size, nq, nkv)) return ULLM_ERR_UNSUPPORTED;
  if (waves != 4 && waves != 8) return ULLM_ERR_UNSUPPORTED;
  if (hd == 256) waves = 4;                              // shared memory of the merge
  if (num_splits < 1 || num_splits > 65535 || window < 0) return ULLM_ERR_SHAPE;
  if (num_splits > 1 && !workspace) return ULLM_ERR_SHAPE;
  const int G = nq / nkv, groups = (G + 15) / 16;
  if (n_items > 65535 || nkv * groups > 65535) return ULLM_ERR_SHAPE;
  const float sl = scale * 1.4426950408889634f;
  dim3 grid(num_splits, nkv * groups, n_items), block(64 * waves);
#define CALL(N) do { if (waves == 8) hipLaunchKernelGGL((attention_decode_kernel<N, 8>), grid, block, 0, stream, \
    (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, token_list, \
    positions, token_entry, block_table, bt_stride, page_size, nq, nkv, sl, window, num_splits, workspace); \
  else hipLaunchKernelGGL((attention_decode_kernel<N, 4>), grid, block, 0, stream, \
    (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, token_list, \
    positions, token_entry, block_table, bt_stride, page_size, nq, nkv, sl, window, num_splits, workspace); \
  } while (0)
  DISPATCH_NQK(hd, CALL)
#undef CALL
  int rc = (int)hipGetLastError();
  if (rc != 0 || num_splits == 1) return rc;
  hipLaunchKernelGGL(attention_reduce_kernel, dim3(n_items, nq), dim3(64), 0, stream, workspace, (bf16_t*)out,
                     out_stride, token_list, nq, hd, num_splits);
  ULLM_LAUNCH_CHECK();
}

extern "C" int ullm_attention_prefill(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* tiles, int n_tiles, const int* positions, const int* token_entry, const int* block_table,
    int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (!ullm_attention_mfma_supports(hd, page_size, nq, nkv)) return ULLM_ERR_UNSUPPORTED;
  if (window < 0) return ULLM_ERR_SHAPE;
  const int G = nq / nkv, waves = G < 4 ? G : 4, hgroups = (G + waves - 1) / waves;
  const float sl = scale * 1.4426950408889634f;
  dim3 grid(n_tiles, nkv * hgroups), block(64 * waves);
#define CALL(N) hipLaunchKernelGGL(attention_prefill_kernel<N>, grid, block, 0, stream, (const bf16_t*)q, q_stride, \
    (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, tiles, positions, token_entry, \
    block_table, bt_stride, page_size, nq, nkv, sl, window)
  DISPATCH_NQK(hd, CALL)
#undef CALL
  ULLM_LAUNCH_CHECK();
}
