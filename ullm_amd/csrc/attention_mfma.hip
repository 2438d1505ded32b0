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
// Softmax state (reference value, sum) is 32-bit and per column; the scale and log2(e) are folded into
// one multiply so that the exponential is a single v_exp_f32.  The reference value a column's
// exponentials are taken against follows the column's running maximum lazily: it moves only when a
// tile's maximum exceeds it by more than RESCALE_STEP (so weights stay below 2^RESCALE_STEP), and the
// output is rescaled only then: the result is the same sum, and most tiles skip the rescaling.
//
// Semantics as in the general kernel: causal with the queries at the end of the keys, optional
// window, query head h reads kv head h / (nq / nkv) (ullm/layers/attention.py:76-104,271,298-309).
#include "common.h"
#include <type_traits>
#include "no_alloc.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

#define NEG_BIG (-1.0e30f)
#define RESCALE_STEP 8.0f

union Pack8 {
  bf16x8_t v;
  uint4 u4;
  uint2 u2[2];
  uint32_t w[4];
  bf16_t h[8];
};

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// acc + both bfloat16 halves of w (v_dot2c_f32_bf16 with a pair of ones)
__device__ __forceinline__ float add_pair_bf16(uint32_t w, float acc) {
  typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
  return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(pair_t, w), __builtin_bit_cast(pair_t, 0x3f803f80u), acc, false);
}

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
  int off;                // lane i: row of that sub-block's first key inside its page
};

__device__ __forceinline__ PageWindow load_pages(int key_from, int key_end, const int* __restrict__ bt, int page_size) {
  PageWindow w;
  w.base = key_from >> 4;
  const int kb = (w.base + (int)(threadIdx.x & 63)) << 4;
  w.page = kb < key_end ? bt[kb / page_size] : -1;
  w.off = kb % page_size;
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
    const int off = __builtin_amdgcn_readlane(pw.off, (kb >> 4) - pw.base);
    t.ok[sb] = page >= 0;
    if (page >= 0) {
      const bf16_t* kp = k_pool + (((size_t)page * nkv + kvh) * page_size + off + c) * HD + 8 * g;
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) t.k[sb][ch].u4 = ld_stream16(kp + 32 * ch);   // a decode step reads a key once
      const bf16_t* vp = v_pool + (((size_t)page * nkv + kvh) * HD + c) * page_size + off + 4 * g;
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) t.v[n][sb] = ld_stream8(vp + (size_t)16 * n * page_size);
    } else {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) t.k[sb][ch].u4 = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) t.v[n][sb] = make_uint2(0, 0);
    }
  }
}

// Scores, softmax update and value product for one tile held in registers, for NG groups of 16
// columns that share the tile (each group has its own queries, limits, maximum, sum and output).
// `own` (or null): the key (head_dim values) and value (head_dim values) of the token itself, at
// position max_hi, in shared memory.  The tile that holds that position takes them from there instead
// of from the cache, where the same kernel is only just writing them.
// INNER: every key of the tile is written data that every column may see (no key before a window's start, none
// past the newest): no test per score, no zeroing of values, and the token's own key is not in it.
template <int NQK, int NG, bool OWN, bool INNER>
__device__ __forceinline__ void process_tile(const KVTile<NQK>& cur, int key0, const Pack8 (&qreg)[NG][NQK],
                                             const int (&col_lo)[NG], const int (&col_hi)[NG], int max_hi,
                                             float scale_log2e, f32x4_t (&acc)[NG][2 * NQK], float (&m)[NG],
                                             float (&l)[NG], const bf16_t* own) {
  // no product fused with a following sum here: the variant with tests keeps the scaled score in a select, the
  // variant without would fuse it into the subtraction of the maximum, and the two would round differently
#pragma clang fp contract(off)
  constexpr int HD = 32 * NQK;
  const int lane = threadIdx.x & 63, g = lane >> 4;
  const bool edge = !INNER && key0 + 32 > max_hi + 1;     // some keys of the tile hold no written data
  Pack8 vals[2 * NQK], keys[2][NQK];
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) {
    vals[n].u2[0] = cur.v[n][0];
    vals[n].u2[1] = cur.v[n][1];
    if (edge) {
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (key0 + 16 * (j >> 2) + 4 * g + (j & 3) > max_hi) vals[n].h[j] = 0;
    }
  }
  const Pack8 (*kp)[NQK] = cur.k;
  if constexpr (OWN && !INNER) {
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) keys[sb][ch] = cur.k[sb][ch];
    kp = keys;
  }
  if (OWN && !INNER && own && key0 + 32 > max_hi) {
    const int c = lane & 15;
    const int at = max_hi - key0;               // 0 .. 31: sub-block at >> 4, row at & 15, which lane group at >> 2 & 3 holds
    if (c == (at & 15)) {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) {
        const uint4 k = ld16(own + 32 * ch + 8 * g);
        if (at < 16) keys[0][ch].u4 = k;
        else keys[1][ch].u4 = k;
      }
    }
    if (g == ((at >> 2) & 3)) {
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) {
        const bf16_t v = own[HD + 16 * n + c];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (j == 4 * (at >> 4) + (at & 3)) vals[n].h[j] = v;
      }
    }
  }
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    f32x4_t s[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      s[sb] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch)
        s[sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kp[sb][ch].v, qreg[q][ch].v, s[sb], 0, 0, 0);
    }
    // scores of keys key0 + 16 sb + 4 g + r for this lane's column; mask, running maximum
    float tile_max = NEG_BIG;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int kk = key0 + 16 * sb + 4 * g + r;
        const bool ok = INNER || (cur.ok[sb] && kk >= col_lo[q] && kk <= col_hi[q]);
        const float v = ok ? s[sb][r] * scale_log2e : NEG_BIG;
        s[sb][r] = v;
        tile_max = fmaxf(tile_max, v);
      }
    tile_max = max_with_lane_xor32(max_with_lane_xor16(tile_max));     // over the four lanes of the column
    const float m_new = fmaxf(m[q], tile_max);
    const float alpha = fast_exp2(m[q] - m_new);
    Pack8 p;
    float psum = 0.f;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float e[4];
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        // a masked score stays at NEG_BIG: its weight is zero even while m_new is still NEG_BIG
        e[r] = INNER || s[sb][r] > 0.5f * NEG_BIG ? fast_exp2(s[sb][r] - m_new) : 0.f;
        psum += e[r];
      }
      p.w[2 * sb] = pack2_bf16(e[0], e[1]);
      p.w[2 * sb + 1] = pack2_bf16(e[2], e[3]);
    }
    l[q] = l[q] * alpha + psum;
    m[q] = m_new;
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n) {
      f32x4_t o = acc[q][n];
      o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
      acc[q][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vals[n].v, p.v, o, 0, 0, 0);
    }
  }
}

// The work of one wave.  NQK = head_dim / 32; NG groups of 16 columns share every tile.
//   queries       : fetch() queues the loads of what the queries are made from, before the loads of the
//                   first tiles; finish(qreg), behind them, fills qreg[q][ch] = this lane's column's
//                   query in group q, dims 32 ch + 8 g .. +8 (zeros if padding), while the tiles are on
//                   their way, and returns where the token's own key and value lie (or null)
//   col_lo/hi[q]  : first and last key the column may see (hi < lo for padding)
//   key_begin/key_end : the wave's key range [begin, end), begin a multiple of 32
//   max_hi     : largest key position that holds written data for this request
// Results per group: acc[q][n][r] = O^T[16n + 4g + r][col] (unnormalised), m (log2 domain), l (this
// lane's share of the sum; the four lanes of a column add up to the column's sum).
// Page ids are fetched 1024 keys at a time; the loads of the next tile are in flight while the current one
// is worked on (two tiles ahead, in three sets of registers, was slower at every batch size and context: the
// third set costs moves between the two halves of the register file, and a wave's products are the longer
// part of a tile's time).
template <int NQK, int NG, bool OWN, class Queries>
__device__ __forceinline__ void attend_range(
    Queries& queries, const int (&col_lo)[NG], const int (&col_hi)[NG], int key_begin, int key_end,
    int max_hi, int all_lo, const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
    const int* __restrict__ bt, int page_size, int nkv, int kvh, float scale_log2e, f32x4_t (&acc)[NG][2 * NQK],
    float (&m)[NG], float (&l)[NG]) {
#pragma unroll
  for (int q = 0; q < NG; ++q) {
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n) acc[q][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    m[q] = NEG_BIG;
    l[q] = 0.f;
  }
  if (key_begin >= key_end) return;
  queries.fetch();
  PageWindow pw = load_pages(key_begin, key_end, bt, page_size);
  Pack8 qreg[NG][NQK];
  const bf16_t* own = nullptr;
#define TILE_LOAD(T, K0) load_tile<NQK>(T, K0, pw, k_pool, v_pool, page_size, nkv, kvh)
  // a tile all of whose keys every column of the wave sees (all_lo: the columns' common first key, or a value no
  // tile reaches where they have none in common) takes the variant without tests; with OWN not the tile of the
  // newest key, which comes from shared memory
#define TILE_WORK(T, K0)                                                                                          \
  do {                                                                                                            \
    if ((K0) >= all_lo && (K0) + 31 < max_hi + (OWN ? 0 : 1) && T.ok[0] && T.ok[1])                               \
      process_tile<NQK, NG, OWN, true>(T, K0, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l, own);         \
    else                                                                                                          \
      process_tile<NQK, NG, OWN, false>(T, K0, qreg, col_lo, col_hi, max_hi, scale_log2e, acc, m, l, own);        \
  } while (0)
  KVTile<NQK> t0, t1;                                     // in turns: one is worked on while the other loads
  int base = key_begin, stop = base + 1024 < key_end ? base + 1024 : key_end;
  TILE_LOAD(t0, base);
  own = queries.finish(qreg);
  for (;;) {
    for (int key0 = base; key0 < stop; key0 += 64) {
      if (key0 + 32 < stop) TILE_LOAD(t1, key0 + 32);
      TILE_WORK(t0, key0);
      if (key0 + 32 >= stop) break;
      if (key0 + 64 < stop) TILE_LOAD(t0, key0 + 64);
      TILE_WORK(t1, key0 + 32);
    }
    base += 1024;
    if (base >= key_end) break;
    pw = load_pages(base, key_end, bt, page_size);        // the next 1024 keys' page ids
    stop = base + 1024 < key_end ? base + 1024 : key_end;
    TILE_LOAD(t0, base);
  }
#undef TILE_LOAD
#undef TILE_WORK
}

// Merge the waves of a block pairwise, lane by lane (a lane's values mean the same in every wave),
// halving the number of live waves each round in a fixed order; wave 0 ends with the block's result.
// `buf` holds (WAVES / 2) x (NG * (8 NQK + 2)) x 64 floats.  Every wave of the block must call this.
template <int NQK, int NG, int WAVES>
__device__ __forceinline__ void merge_waves(f32x4_t (&acc)[NG][2 * NQK], float (&m)[NG], float (&l)[NG], float* buf) {
  constexpr int PER_LANE = NG * (8 * NQK + 2);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int half = WAVES / 2; half >= 1; half >>= 1) {
    if (wave >= half && wave < 2 * half) {          // the upper half of the live waves hands over
      float* w = buf + (size_t)(wave - half) * PER_LANE * 64 + lane;
#pragma unroll
      for (int q = 0; q < NG; ++q) {
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int r = 0; r < 4; ++r) w[(q * (8 * NQK + 2) + 4 * n + r) * 64] = acc[q][n][r];
        w[(q * (8 * NQK + 2) + 8 * NQK) * 64] = m[q];
        w[(q * (8 * NQK + 2) + 8 * NQK + 1) * 64] = l[q];
      }
    }
    __syncthreads();
    if (wave < half) {
      const float* w = buf + (size_t)wave * PER_LANE * 64 + lane;
#pragma unroll
      for (int q = 0; q < NG; ++q) {
        const float m_b = w[(q * (8 * NQK + 2) + 8 * NQK) * 64], l_b = w[(q * (8 * NQK + 2) + 8 * NQK + 1) * 64];
        const float M = fmaxf(m[q], m_b);
        const float fa = fast_exp2(m[q] - M), fb = fast_exp2(m_b - M);
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int r = 0; r < 4; ++r)
            acc[q][n][r] = acc[q][n][r] * fa + w[(q * (8 * NQK + 2) + 4 * n + r) * 64] * fb;
        l[q] = l[q] * fa + l_b * fb;
        m[q] = M;
      }
    }
    __syncthreads();
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
//
// FUSE: `q` is the row of the fused projection q | k | v, not yet normed or rotated.  Every wave norms
// and rotates its queries itself (a few hundred operations on values it loads anyway), and the one wave
// whose keys end at the token's own position does the same for the token's key, writes key and value
// to the cache for the steps to come, and hands them to its last tile through shared memory: a decode
// step then needs no kernel of its own for norm, rotation and cache write.
struct DecodeFuse {
  const float* q_gain;    // per-head norm gains [head_dim], or null: no norm
  const float* k_gain;
  float eps;
  const float* cos_sin;   // [table_rows, head_dim]: cos of the head_dim / 2 angles, then sin; or null: no rotation
  int table_rows;
  bf16_t* k_pool;         // the pools again, writable; null: this layer reads a cache that another layer writes
  bf16_t* v_pool;
};

// Queries as the projection left them (bfloat16, normed and rotated by an earlier kernel).
template <int NQK>
struct ReadyQueries {
  const bf16_t* row;                    // the column's head, or null for a padding column
  int g;
  Pack8 raw[NQK];
  __device__ __forceinline__ void fetch_early() {       // needs the token alone, not its position
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      if (row) raw[ch].u4 = *reinterpret_cast<const uint4*>(row + 32 * ch + 8 * g);
      else raw[ch].u4 = make_uint4(0, 0, 0, 0);
    }
  }
  __device__ __forceinline__ void fetch() {}
  __device__ __forceinline__ const bf16_t* finish(Pack8 (&qreg)[1][NQK]) {
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) qreg[0][ch] = raw[ch];
    return nullptr;
  }
};

// Queries, and for one wave the token's own key and value, from the raw projection row.
template <int NQK>
struct RawQueries {
  static constexpr int HD = 32 * NQK;
  const DecodeFuse& fuse;
  const bf16_t* q_head;                 // the column's query head in the projection row
  const bf16_t* k_head;                 // the token's key and value heads there, if this wave's keys end with the
  const bf16_t* v_head;                 //   token itself and the layer writes its cache; else null
  const float* cs;                      // the position's row of the table, or null
  bf16_t* k_dst;                        // where key and value go in the cache (null: nowhere)
  bf16_t* v_dst;
  int page_size, g, c;
  bf16_t* own_kv;                       // shared memory: head_dim values of the key, then of the value
  Pack8 q_raw[NQK], k_raw[NQK];
  bf16_t v_raw[2 * NQK];
  float q_gain[NQK][8], k_gain[NQK][8], cos_[NQK / 2][8], sin_[NQK / 2][8];

  __device__ __forceinline__ static void load8(float (&to)[8], const float* from) {
    const float4 a = *reinterpret_cast<const float4*>(from), b = *reinterpret_cast<const float4*>(from + 4);
    to[0] = a.x; to[1] = a.y; to[2] = a.z; to[3] = a.w; to[4] = b.x; to[5] = b.y; to[6] = b.z; to[7] = b.w;
  }
  // What needs neither the token's position nor its pages goes out first, while those are still on their way:
  // the query head's row of the projection and the norms' gains.
  __device__ __forceinline__ void fetch_early() {
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) q_raw[ch].u4 = ld16(q_head + 32 * ch + 8 * g);
    if (fuse.q_gain) {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) load8(q_gain[ch], fuse.q_gain + 32 * ch + 8 * g);
    }
    if (fuse.k_gain) {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) load8(k_gain[ch], fuse.k_gain + 32 * ch + 8 * g);
    }
  }
  // The rest, once the position is known: the table's row, and the token's key and value where this wave has them.
  __device__ __forceinline__ void fetch() {
    if (k_head) {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) k_raw[ch].u4 = ld16(k_head + 32 * ch + 8 * g);
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) v_raw[n] = v_head[16 * n + c];
    }
    if (cs) {
#pragma unroll
      for (int ch = 0; ch < NQK / 2; ++ch) {
        load8(cos_[ch], cs + 32 * ch + 8 * g);
        load8(sin_[ch], cs + HD / 2 + 32 * ch + 8 * g);
      }
    }
  }
  // Per-head norm and half-split rotation of a head held by the four lanes of a column: chunk ch,
  // element j = dim 32 ch + 8 g + j.  The same operations in the same order as ullm_qk_norm_rope_write's
  // kernel for these head sizes (which serves prompt portions), multiply-adds spelled out in both, so
  // that a key has the same bits whichever of the two wrote it; the partner of a dim in the first half
  // is the dim head_dim / 2 further on, which for head sizes of 64, 128 and 256 lies in the same lane.
  __device__ __forceinline__ void norm_rotate(const Pack8 (&raw)[NQK], const float (*gain)[8], Pack8 (&to)[NQK]) const {
    static_assert(NQK % 2 == 0, "the partner dim must lie in the same lane");
    float x[NQK][8];
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        x[ch][2 * w] = __uint_as_float(raw[ch].w[w] << 16);
        x[ch][2 * w + 1] = __uint_as_float(raw[ch].w[w] & 0xffff0000u);
      }
    if (gain) {
      // the sum of squares in the order of ullm_qk_norm_rope_write's kernel for these head sizes: runs of
      // 8 consecutive dims summed in turn, then the runs pairwise, the most distant pairs first (run p of
      // the head is chunk p / 4 of lane group p % 4 here)
      float part[NQK];
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) {
        float a = 0.f;
#pragma unroll
        for (int j = 0; j < 8; ++j) a = fmaf(x[ch][j], x[ch][j], a);
        part[ch] = a;
      }
#pragma unroll
      for (int m = NQK / 2; m >= 1; m >>= 1)
#pragma unroll
        for (int ch = 0; ch < m; ++ch) part[ch] += part[ch + m];
      float ss = part[0];
      ss += __shfl_xor(ss, 32, 64);
      ss += __shfl_xor(ss, 16, 64);
      const float rs = rsqrtf(ss / (float)HD + fuse.eps);
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch)
#pragma unroll
        for (int j = 0; j < 8; ++j) x[ch][j] = (x[ch][j] * rs) * gain[ch][j];
    }
    if (cs) {
#pragma unroll
      for (int ch = 0; ch < NQK / 2; ++ch)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const float a = x[ch][j], b = x[ch + NQK / 2][j];
          x[ch][j] = fmaf(a, cos_[ch][j], -(b * sin_[ch][j]));
          x[ch + NQK / 2][j] = fmaf(b, cos_[ch][j], a * sin_[ch][j]);
        }
    }
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch)
#pragma unroll
      for (int w = 0; w < 4; ++w) to[ch].w[w] = pack2_bf16(x[ch][2 * w], x[ch][2 * w + 1]);
  }
  __device__ __forceinline__ const bf16_t* finish(Pack8 (&qreg)[1][NQK]) {
    norm_rotate(q_raw, fuse.q_gain ? q_gain : nullptr, qreg[0]);
    if (!k_head) return nullptr;
    // only one wave of the block gets here, so the one place in shared memory is its own
    Pack8 key[NQK];
    norm_rotate(k_raw, fuse.k_gain ? k_gain : nullptr, key);
    if (c == 0) {
#pragma unroll
      for (int ch = 0; ch < NQK; ++ch) {
        st16(own_kv + 32 * ch + 8 * g, key[ch].u4);
        if (k_dst) st16(k_dst + 32 * ch + 8 * g, key[ch].u4);
      }
    }
    if (g == 0) {
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n) {
        own_kv[HD + 16 * n + c] = v_raw[n];
        if (v_dst) v_dst[(size_t)(16 * n + c) * page_size] = v_raw[n];
      }
    }
    // the lanes of this wave read each other's values from there at the last tile
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    return own_kv;
  }
};

template <int NQK, int WAVES, bool FUSE>
__global__ void __launch_bounds__(64 * WAVES)
attention_decode_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                        const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                        const int* __restrict__ token_list, const int* __restrict__ positions,
                        const int* __restrict__ token_entry, const int* __restrict__ block_table,
                        int bt_stride, int page_size, int nq, int nkv, float scale_log2e, int window,
                        int num_splits, float* __restrict__ part, DecodeFuse fuse) {
  constexpr int HD = 32 * NQK;
  constexpr int ROW = HD + 4;                       // output dims, then maximum and sum (rows stay 16-byte aligned)
  __shared__ float merge[(WAVES > 1 ? WAVES / 2 : 1) * (WAVES > 1 ? (8 * NQK + 2) * 64 : 1)];   // [writer][value][lane]: conflict-free
  __shared__ __attribute__((aligned(16))) bf16_t own_kv[FUSE ? 2 * HD : 8];   // the token's own key, then its value
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, g = lane >> 4, c = lane & 15;
  const int split = blockIdx.x;
  const int G = nq / nkv;
  const int groups = (G + 15) / 16;
  const int kvh = blockIdx.y / groups, cg = blockIdx.y % groups;
  const int item = blockIdx.z;
  const int t = token_list ? token_list[item] : item;
  const int head_in_group = cg * 16 + c;
  const bool col_ok = head_in_group < G;
  const int head = kvh * G + head_in_group;
  const bf16_t* const row = q + (size_t)t * q_stride;
  // the queries' loads that need the token alone go out before its position is asked for
  using Queries = typename std::conditional<FUSE, RawQueries<NQK>, ReadyQueries<NQK>>::type;
  Queries queries = [&]() {
    if constexpr (FUSE)       // a padding column takes the group's first head: never stored
      return RawQueries<NQK>{fuse, row + (size_t)(col_ok ? head : kvh * G) * HD, nullptr, nullptr, nullptr, nullptr, nullptr,
                             page_size, g, c, own_kv};
    else
      return ReadyQueries<NQK>{col_ok ? row + (size_t)head * HD : nullptr, g};
  }();
  queries.fetch_early();
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int first = lo & ~31;
  const int tiles = (pos + 1 - first + 31) / 32;
  const int share = 32 * ((tiles + num_splits * WAVES - 1) / (num_splits * WAVES));
  int begin = first + (split * WAVES + wave) * share, end = begin + share;
  if (end > pos + 1) end = pos + 1;
  f32x4_t accs[1][2 * NQK];
  float ms[1], ls[1];
  {
    const int* const bt = block_table + (size_t)token_entry[t] * bt_stride;
    const int clo[1] = {lo}, chi[1] = {col_ok ? pos : -1};
    if constexpr (FUSE) {
      const bool has_own = fuse.k_pool && begin < end && end == pos + 1;
      // no page (a padding entry), no write, as in the kernel for prompt portions; one block per kv head writes
      const int page = has_own && cg == 0 ? bt[pos / page_size] : -1;
      const int off = pos % page_size;
      if (has_own) {
        queries.k_head = row + (size_t)(nq + kvh) * HD;
        queries.v_head = row + (size_t)(nq + nkv + kvh) * HD;
      }
      if (fuse.cos_sin) queries.cs = fuse.cos_sin + (size_t)(pos < fuse.table_rows ? pos : fuse.table_rows - 1) * HD;
      if (page >= 0) {
        queries.k_dst = fuse.k_pool + (((size_t)page * nkv + kvh) * page_size + off) * HD;
        queries.v_dst = fuse.v_pool + ((size_t)page * nkv + kvh) * HD * page_size + off;
      }
    }
    attend_range<NQK, 1, FUSE>(queries, clo, chi, begin, end, pos, lo, k_pool, v_pool, bt, page_size, nkv, kvh,
                               scale_log2e, accs, ms, ls);
  }
  merge_waves<NQK, 1, WAVES>(accs, ms, ls, merge);
  f32x4_t (&acc)[2 * NQK] = accs[0];
  float& m = ms[0];
  float& l = ls[0];
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
  // Eight splits at a time: their loads are all queued before the first is used, and those of the first eight go
  // out before anything else (no load under a condition: an index past the end reads the last element), so that
  // the splits' maxima and their values come back in one round trip instead of two.
  float v[8][4];
  int dim[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) dim[r] = lane + 64 * r < hd ? lane + 64 * r : hd - 1;
  auto fetch = [&](int s0, int j0, int n) __attribute__((always_inline)) {
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const float* pj = pp + (size_t)(s0 + (j0 + u < n ? j0 + u : n - 1)) * row;
#pragma unroll
      for (int r = 0; r < 4; ++r) v[u][r] = pj[dim[r]];
    }
  };
  fetch(0, 0, num_splits < 64 ? num_splits : 64);
  float M = NEG_BIG;
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const int sp = s0 + lane;
    M = fmaxf(M, wave_max(pp[(sp < num_splits ? sp : num_splits - 1) * row + hd]));
  }
  float acc[4] = {0.f, 0.f, 0.f, 0.f};       // head_dim <= 256: dims lane, lane + 64, ...
  float L = 0.f;
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const int sp = s0 + lane;
    const bool ok = sp < num_splits;
    const float* mine = pp + (ok ? sp : num_splits - 1) * row + hd;
    const float f = ok ? fast_exp2(mine[0] - M) : 0.f;
    L += wave_sum(ok ? mine[1] * f : 0.f);
    const int n = num_splits - s0 < 64 ? num_splits - s0 : 64;
    for (int j0 = 0; j0 < n; j0 += 8) {
      if (s0 + j0 > 0) fetch(s0, j0, n);
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const float fj = j0 + u < n ? __shfl(f, j0 + u, 64) : 0.f;
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[r] += v[u][r] * fj;
      }
    }
  }
  const float inv = L > 0.f ? 1.f / L : 0.f;
  bf16_t* op = out + (size_t)t * out_stride + (size_t)head * hd;
#pragma unroll
  for (int r = 0; r < 4; ++r)
    if (lane + 64 * r < hd) op[lane + 64 * r] = f32_to_bf16_bits(acc[r] * inv);
}

// ------------------------------------------------------------------------------- prompt portions
// Tile = (first token, number of tokens <= 32) of one request.  A block of PREFILL_WAVES waves works
// on one tile for up to PREFILL_WAVES query heads that share a kv head, one head per wave (two groups
// of 16 tokens each), so every 32-key tile of keys and values is fetched from memory once per block
// and shared through LDS:
//   keys   LDS row = one key, head_dim values + 16 bytes of padding
//   values LDS row = one dim, its 32 keys in the order [g][half][4] (the 8 keys lane group g feeds to
//          one product are 16 adjacent bytes) + 16 bytes of padding
// With these paddings the 16 lanes that the hardware serves together read 16 different bank groups.
// Loads run two tiles ahead of the products (two register sets in rotation); two LDS tiles take turns,
// so a wave writes the next tile right after its own products and one barrier a tile is enough.
// grid (n_tiles * nkv * head_chunks).  Workgroups go to the 8 XCDs round-robin by their linear id and
// each XCD has an L2 of its own, so the id is decoded such that all work on one kv head lands on one
// XCD (kv head = id mod 8 when the kv heads are a multiple of 8): that head's keys and values then
// stay in that L2 instead of every XCD streaming every head from memory.
// The caller lists the tiles by rising number of keys; blocks take them from the end, the longest
// first (measured against orders that alternate long and short tiles, this one was the fastest).
#define PREFILL_GROUPS 2
#define PREFILL_WAVES 4

template <int NQK>
struct PrefillStage {                     // one 32-key tile on its way from the cache to LDS
  static constexpr int HD = 32 * NQK;
  static constexpr int THREADS = 64 * PREFILL_WAVES;
  static constexpr int CHUNKS = 4 * HD;   // 16-byte pieces of the key tile, and as many of the value tile
  static constexpr int PER_THREAD = (CHUNKS + THREADS - 1) / THREADS;
  static constexpr int KROW = 2 * HD + 32, VROW = 64 + 32;     // bytes
  static constexpr int KBYTES = 32 * KROW, VBYTES = HD * VROW;
  uint4 k[PER_THREAD], v[PER_THREAD];
  int ok;                                 // bit j: piece j comes from a page that exists (the same in the whole wave)
};

// What a thread's pieces need that does not change from tile to tile: byte offsets in the cache
// relative to the sub-block's first row and positions in the LDS tile (bytes).
template <int NQK>
struct PrefillLanes {
  unsigned kofs[PrefillStage<NQK>::PER_THREAD], vofs[PrefillStage<NQK>::PER_THREAD];
  int klds[PrefillStage<NQK>::PER_THREAD], vlds[PrefillStage<NQK>::PER_THREAD];
};

template <int NQK>
__device__ __forceinline__ PrefillLanes<NQK> prefill_lanes(int page_size) {
  using S = PrefillStage<NQK>;
  constexpr int HD = S::HD;
  PrefillLanes<NQK> pl;
  const int tid = threadIdx.x & (S::THREADS - 1);
#pragma unroll
  for (int j = 0; j < S::PER_THREAD; ++j) {
    const int piece = tid + j * S::THREADS;
    const int sb = piece / (2 * HD), rem = piece % (2 * HD);      // 2 HD pieces per sub-block
    // keys: row rem / (HD / 8) of the sub-block, 8 values at column 8 (rem % (HD / 8))
    pl.kofs[j] = 2u * (unsigned)((rem / (HD / 8)) * HD + 8 * (rem % (HD / 8)));
    pl.klds[j] = (16 * sb + rem / (HD / 8)) * S::KROW + 16 * (rem % (HD / 8));
    // values: dim rem / 2, keys 8 (rem % 2) .. +8 of the sub-block; in LDS the first four go to lane
    // group 2 (rem % 2), the other four to the group after it
    pl.vofs[j] = 2u * (unsigned)((rem / 2) * page_size + 8 * (rem % 2));
    pl.vlds[j] = (rem / 2) * S::VROW + 8 * sb + 32 * (rem % 2);
  }
  return pl;
}

// Page ids for the prompt kernel's loads: as load_pages, but the table is read by every lane (a lane
// past the end of the data reads the entry of the last key) and the result is made -1 by arithmetic,
// so the load stands outside any condition and the compiler can count it among the loads in flight.
__device__ __forceinline__ PageWindow prefill_pages(int key_from, int key_end, const int* __restrict__ bt, int page_size) {
  PageWindow w;
  w.base = key_from >> 4;
  const int kb = (w.base + (int)(threadIdx.x & 63)) << 4;
  const int at = kb < key_end ? kb : key_end - 1;
  w.page = bt[at / page_size] | ((key_end - 1 - kb) >> 31);
  w.off = kb % page_size;
  return w;
}

// Queue the loads of the tile at key0.  A wave's 64 pieces of one round lie in one 16-key sub-block,
// so its page id is a single lane of the page window and the cache address is a base common to the
// wave (scalar registers) plus the thread's own 32-bit offset.  `k_head` / `v_head` point at this kv
// head inside page 0; `page_elems` is the distance between pages.  Every load is issued whatever the
// page table says, so that the waits in the loop are for the loads of two steps ago and not for all
// of them: a sub-block without a page (given back behind a window, or past the end of the data) reads
// page 0 instead.  Its keys are never seen (it lies in a tile with tests, and they fail for such a
// key), and its values are replaced by zeros on the way to LDS.
template <int NQK>
__device__ __forceinline__ void stage_load(PrefillStage<NQK>& st, int key0, const PageWindow& pw,
                                           const PrefillLanes<NQK>& pl, const bf16_t* __restrict__ k_head,
                                           const bf16_t* __restrict__ v_head, unsigned page_elems) {
  using S = PrefillStage<NQK>;
  constexpr int HD = S::HD;
  const int tid = threadIdx.x & (S::THREADS - 1);
  st.ok = 0;
#pragma unroll
  for (int j = 0; j < S::PER_THREAD; ++j) {
    const int piece = tid + j * S::THREADS;
    const int sub = (__builtin_amdgcn_readfirstlane(piece / (2 * HD)) + (key0 >> 4) - pw.base) & 63;
    const int page = __builtin_amdgcn_readlane(pw.page, sub);
    const unsigned off = (unsigned)__builtin_amdgcn_readlane(pw.off, sub);
    const size_t base = (size_t)(unsigned)(page < 0 ? 0 : page) * page_elems;
    st.ok |= (page < 0 ? 0 : 1) << j;
    st.k[j] = ld16(reinterpret_cast<const char*>(k_head + base + off * HD) + pl.kofs[j]);
    st.v[j] = ld16(reinterpret_cast<const char*>(v_head + base + off) + pl.vofs[j]);
  }
}

// Write a loaded tile to LDS; values of keys past max_hi (never written, may hold anything) and of
// sub-blocks without a page become 0.
template <int NQK>
__device__ __forceinline__ void stage_store(const PrefillStage<NQK>& st, int key0, int max_hi,
                                            const PrefillLanes<NQK>& pl, unsigned char* __restrict__ kl,
                                            unsigned char* __restrict__ vl) {
  using S = PrefillStage<NQK>;
  constexpr int HD = S::HD;
  const int tid = threadIdx.x & (S::THREADS - 1);
  const bool plain = key0 + 32 <= max_hi + 1 && st.ok == (1 << S::PER_THREAD) - 1;
#pragma unroll
  for (int j = 0; j < S::PER_THREAD; ++j) {
    const int piece = tid + j * S::THREADS;
    if (piece >= S::CHUNKS) continue;
    st16(kl + pl.klds[j], st.k[j]);
    if (plain) {
      *reinterpret_cast<uint2*>(vl + pl.vlds[j]) = make_uint2(st.v[j].x, st.v[j].y);       // keys 8 half .. +4
      *reinterpret_cast<uint2*>(vl + pl.vlds[j] + 16) = make_uint2(st.v[j].z, st.v[j].w);  // keys 8 half + 4 .. +4
      continue;
    }
    Pack8 v;
    v.u4 = st.v[j];
    const int sb = piece / (2 * HD), half = piece % 2;
    const bool ok = (st.ok >> j) & 1;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      if (!ok || key0 + 16 * sb + 8 * half + e > max_hi) v.h[e] = 0;
    *reinterpret_cast<uint2*>(vl + pl.vlds[j]) = v.u2[0];
    *reinterpret_cast<uint2*>(vl + pl.vlds[j] + 16) = v.u2[1];
  }
}

// scale * log2(e) = pow2 * frac with pow2 a power of two and 1 <= frac < 2.  The prompt kernels multiply the
// bfloat16 queries by pow2 (exact) and the 32-bit scores by frac, so a score is the exponent of its weight with
// no rounding but that of the 32-bit product, as in the decode kernel, which scales the 32-bit score whole.
struct ScoreScale {
  float pow2, frac, inv_frac;
};
__device__ __forceinline__ ScoreScale split_scale(float scale_log2e) {
  int e;
  const float f = frexpf(scale_log2e, &e);              // scale_log2e = f * 2^e, 0.5 <= f < 1
  ScoreScale sc;
  sc.frac = 2.f * f;
  sc.pow2 = ldexpf(1.f, e - 1);
  sc.inv_frac = 1.f / sc.frac;
  return sc;
}

// The softmax step both prompt kernels share, between the score products and the value products of a tile.
// `s[q][sb][r]` holds the exponents of this lane's eight keys for column q (the products started from minus
// the column's reference value); `key_of(sb, r)` is the key's offset in the tile.  Does any exponent exceed
// RESCALE_STEP, or does a column meet its first key?  Each lane looks at its own scores only and the wave votes;
// most tiles pass, and then no value crosses lanes and nothing is rescaled.  Otherwise the columns' maxima are
// formed (a column's keys lie in four lanes); where one is more than RESCALE_STEP above the reference value, or
// there was none (m == NEG_BIG counts from zero), it becomes the new one, and the exponents and the output so
// far are brought to it.  Leaves the weights in `p`, rounded to bfloat16 as they multiply the values, and adds
// those rounded weights to the sums `l`, two per instruction.
template <int NQK, int NG, bool masked, typename KeyOf>
__device__ __forceinline__ void prompt_tile_softmax(f32x4_t (&s)[NG][2], int key0, KeyOf key_of,
                                                    const int (&col_lo)[NG], const int (&col_hi)[NG],
                                                    f32x4_t (&acc)[NG][2 * NQK], float (&m)[NG], f32x4_t (&negm)[NG],
                                                    float (&l)[NG], Pack8 (&p)[NG], const ScoreScale& scale) {
  float lane_max[NG], alpha[NG];
  bool exceeds = false;
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    lane_max[q] = NEG_BIG;
    alpha[q] = 1.f;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        s[q][sb][r] *= scale.frac;                      // the part of scale * log2(e) that is no power of two, in 32-bit
        if (masked) {
          const int kk = key0 + key_of(sb, r);
          if (!(kk >= col_lo[q] && kk <= col_hi[q])) s[q][sb][r] = NEG_BIG;
        }
        lane_max[q] = fmaxf(lane_max[q], s[q][sb][r]);
      }
    const bool sees = !masked || lane_max[q] > 0.5f * NEG_BIG;
    exceeds = exceeds || (sees && (lane_max[q] > RESCALE_STEP || m[q] < 0.5f * NEG_BIG));
  }
  if (__any(exceeds)) {
#pragma unroll
    for (int q = 0; q < NG; ++q) {
      float col_max = lane_max[q];
      col_max = fmaxf(col_max, __shfl_xor(col_max, 16, 64));
      col_max = fmaxf(col_max, __shfl_xor(col_max, 32, 64));
      const bool had = m[q] > 0.5f * NEG_BIG;
      const bool moves = col_max > 0.5f * NEG_BIG && (!had || col_max > RESCALE_STEP);
      if (moves) {
        m[q] = (had ? m[q] : 0.f) + col_max;
        const float start = -m[q] * scale.inv_frac;     // the products start from here and are multiplied by frac
        negm[q] = f32x4_t{start, start, start, start};
        if (had) alpha[q] = fast_exp2(-col_max);
#pragma unroll
        for (int sb = 0; sb < 2; ++sb)
#pragma unroll
          for (int r = 0; r < 4; ++r) s[q][sb][r] -= col_max;     // a hidden score stays far below
      }
#pragma unroll
      for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          float o = acc[q][n][r] * alpha[q];
#ifdef __HIP_DEVICE_COMPILE__
          asm volatile("" : "+v"(o));       // pins the multiply inside the branch: most tiles skip it
#endif
          acc[q][n][r] = o;
        }
    }
  }
#pragma unroll
  for (int q = 0; q < NG; ++q) {
    float psum = l[q] * alpha[q];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      float e[4];
#pragma unroll
      for (int r = 0; r < 4; ++r)
        e[r] = (!masked || s[q][sb][r] > 0.5f * NEG_BIG) ? fast_exp2(s[q][sb][r]) : 0.f;
      p[q].w[2 * sb] = pack2_bf16(e[0], e[1]);
      p[q].w[2 * sb + 1] = pack2_bf16(e[2], e[3]);
      psum = add_pair_bf16(p[q].w[2 * sb], psum);
      psum = add_pair_bf16(p[q].w[2 * sb + 1], psum);
    }
    l[q] = psum;
  }
}

// Scores, softmax update and value product of one wave for the tile in LDS.  `masked` = some key of
// the tile is hidden from some column (diagonal, window or end of data); otherwise no per-score test.
// The queries come multiplied by the power of two in scale * log2(e), and the first product of a score
// starts from minus the column's reference value over the remaining factor (`negm`, the same in all four
// elements) instead of zero, so the products times that factor are the exponent itself: exp2 of it is the weight.  A column without a reference
// value yet (m == NEG_BIG) counts from zero, and the first tile that shows it a key gives it one.
template <int NQK, int NG, bool masked>
__device__ __forceinline__ void process_tile_lds(const unsigned char* __restrict__ kl, const unsigned char* __restrict__ vl,
                                                 int key0, const Pack8 (&qreg)[NG][NQK],
                                                 const int (&col_lo)[NG], const int (&col_hi)[NG],
                                                 f32x4_t (&acc)[NG][2 * NQK], float (&m)[NG], f32x4_t (&negm)[NG],
                                                 float (&l)[NG], const ScoreScale& scale) {
  using S = PrefillStage<NQK>;
  const int lane = threadIdx.x & 63, g = lane >> 4, c = lane & 15;
  f32x4_t s[NG][2];
#pragma unroll
  for (int sb = 0; sb < 2; ++sb)
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      Pack8 kf;
      kf.u4 = *reinterpret_cast<const uint4*>(kl + (16 * sb + c) * S::KROW + 64 * ch + 16 * g);
#pragma unroll
      for (int q = 0; q < NG; ++q)
        s[q][sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qreg[q][ch].v, ch == 0 ? negm[q] : s[q][sb], 0, 0, 0);
    }
  Pack8 p[NG];
  prompt_tile_softmax<NQK, NG, masked>(s, key0, [g](int sb, int r) { return 16 * sb + 4 * g + r; }, col_lo, col_hi,
                                       acc, m, negm, l, p, scale);
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) {
    Pack8 vf;
    vf.u4 = *reinterpret_cast<const uint4*>(vl + (16 * n + c) * S::VROW + 16 * g);
#pragma unroll
    for (int q = 0; q < NG; ++q)
      acc[q][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, p[q].v, acc[q][n], 0, 0, 0);
  }
}

// KS = 2: eight waves; the upper four take the second half of the tile's keys through an LDS tile of
// their own and hand their (reference value, sum, output) to the lower four at the end.  A block then
// lasts half as long and a compute unit holds one block at a time, so that blocks that finish early
// (tiles with few keys) make room for the next ones instead of idling beside a long one.
template <int NQK, int KS>
__global__ void __launch_bounds__(64 * PREFILL_WAVES * KS, NQK <= 4 ? 2 / KS : 1)
attention_prefill_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                         const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                         const int* __restrict__ tiles, const int* __restrict__ positions,
                         const int* __restrict__ token_entry, const int* __restrict__ block_table,
                         int bt_stride, int page_size, int nq, int nkv, float scale_log2e, int window,
                         int n_tiles) {
  using S = PrefillStage<NQK>;
  constexpr int HD = 32 * NQK;
  constexpr int NG = PREFILL_GROUPS;
  constexpr int TILE_BYTES = S::KBYTES + S::VBYTES;
  constexpr int PER_LANE = NG * (8 * NQK + 2);            // floats a lane hands over in the merge
  static_assert(KS == 1 || PREFILL_WAVES * PER_LANE * 64 * 4 <= KS * 2 * TILE_BYTES, "the merge reuses the tiles' memory");
  __shared__ __attribute__((aligned(16))) unsigned char lds[KS * 2 * TILE_BYTES];   // [half][even | odd tile]
  const int wave_id = (int)(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, wave = wave_id % PREFILL_WAVES, half = wave_id / PREFILL_WAVES;
  const int g = lane >> 4, c = lane & 15;
  unsigned char* const tile_lds = lds + half * 2 * TILE_BYTES;
  const int G = nq / nkv, chunks = (G + PREFILL_WAVES - 1) / PREFILL_WAVES, per_kv = n_tiles * chunks;
  int kvh, rest;
  if (nkv % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    kvh = (slot / per_kv) * 8 + xcd;
    rest = slot % per_kv;
  } else {
    kvh = blockIdx.x / per_kv;
    rest = blockIdx.x % per_kv;
  }
  const int tile_idx = n_tiles - 1 - rest / chunks;
  const int head_in_group = (rest % chunks) * PREFILL_WAVES + wave;
  const bool head_ok = head_in_group < G;                 // a wave without a head still helps to load
  const int head = kvh * G + (head_ok ? head_in_group : G - 1);
  const int first = tiles[2 * tile_idx], count = tiles[2 * tile_idx + 1];
  int clo[NG], chi[NG], tok[NG];
  Pack8 qreg[NG][NQK];
  const ScoreScale score_scale = split_scale(scale_log2e);
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
    const bool ok = head_ok && 16 * qg + c < count;
    tok[qg] = first + (16 * qg + c < count ? 16 * qg + c : 0);
    const int pos = positions[tok[qg]];
    clo[qg] = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    chi[qg] = ok ? pos : -1;
    const bf16_t* qp = q + (size_t)tok[qg] * q_stride + (size_t)head * HD + 8 * g;
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      if (ok) qreg[qg][ch].u4 = *reinterpret_cast<const uint4*>(qp + 32 * ch);
      else qreg[qg][ch].u4 = make_uint4(0, 0, 0, 0);
      // the power of two in scale * log2(e) goes into the queries once (exact); the scores take the rest
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t two = qreg[qg][ch].w[w];
        qreg[qg][ch].w[w] = pack2_bf16(__uint_as_float(two << 16) * score_scale.pow2,
                                       __uint_as_float(two & 0xffff0000u) * score_scale.pow2);
      }
    }
  }
  const int last_pos = positions[first + count - 1];
  const int first_pos = positions[first];
  // keys every column of the tile sees without a test: from the last column's window start up to the first column
  const int open_lo = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int key_begin = ((window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0) & ~31;
  const int key_end = last_pos + 1;
  // this half's share of the 32-key tiles
  const int steps = ((key_end - key_begin + 31) / 32 + KS - 1) / KS;
  const int my_begin = key_begin + half * steps * 32;
  const int my_end = my_begin + steps * 32 < key_end ? my_begin + steps * 32 : key_end;
  const int* bt = block_table + (size_t)token_entry[first] * bt_stride;
  f32x4_t acc[NG][2 * NQK];
  float m[NG], l[NG];
  f32x4_t negm[NG];                                       // minus the reference value, 0 while there is none
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n) acc[qg][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    m[qg] = NEG_BIG;
    negm[qg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    l[qg] = 0.f;
  }
  // The page window serves the loads, which run ahead of the products.  It holds 32 tiles; every 16
  // steps the next one takes over, fetched 16 steps earlier.
  PageWindow pw = prefill_pages(my_begin, key_end, bt, page_size);
  PrefillStage<NQK> st0, st1;
  const PrefillLanes<NQK> lanes = prefill_lanes<NQK>(page_size);
  const unsigned page_elems = (unsigned)(nkv * page_size * HD);
  const bf16_t* const k_head = k_pool + (size_t)kvh * page_size * HD;
  const bf16_t* const v_head = v_pool + (size_t)kvh * page_size * HD;
#define STAGE_LOAD(ST, K0) stage_load<NQK>(ST, (K0), pw, lanes, k_head, v_head, page_elems)
#define STAGE_STORE(ST, K0, BUF)                                                   \
  stage_store<NQK>(ST, (K0), last_pos, lanes, tile_lds + (BUF) * TILE_BYTES,       \
                   tile_lds + (BUF) * TILE_BYTES + S::KBYTES)
  // The tile at K0 is in LDS tile BUF; NEXT holds the tile after it, which goes to the other LDS tile
  // (last read one step ago, before the barrier) and is then refilled with the tile three further on.
  // Every wave runs every step: a wave without a head has no visible key (its limits are empty), and
  // a step past the end of this half's keys finds keys that no column sees and values of zero, so
  // neither changes a sum and the loop needs no test around the products.
#define STAGE_WORK(K0, BUF, NEXT)                                                  \
  do {                                                                             \
    const unsigned char* kl = tile_lds + (BUF) * TILE_BYTES;                       \
    if ((K0) + 31 > first_pos || (K0) < open_lo)                                   \
      process_tile_lds<NQK, NG, true>(kl, kl + S::KBYTES, (K0), qreg, clo, chi, acc, m, negm, l, score_scale);  \
    else                                                                           \
      process_tile_lds<NQK, NG, false>(kl, kl + S::KBYTES, (K0), qreg, clo, chi, acc, m, negm, l, score_scale); \
    STAGE_STORE(NEXT, (K0) + 32, 1 - (BUF));                                       \
    STAGE_LOAD(NEXT, (K0) + 96);                                                   \
    __syncthreads();                                                               \
  } while (0)
  STAGE_LOAD(st0, my_begin);
  STAGE_LOAD(st1, my_begin + 32);
  STAGE_STORE(st0, my_begin, 0);
  STAGE_LOAD(st0, my_begin + 64);
  __syncthreads();
#define STAGE_PRODUCTS(K0, BUF)                                                    \
  do {                                                                             \
    const unsigned char* kl = tile_lds + (BUF) * TILE_BYTES;                       \
    if ((K0) + 31 > first_pos || (K0) < open_lo)                                   \
      process_tile_lds<NQK, NG, true>(kl, kl + S::KBYTES, (K0), qreg, clo, chi, acc, m, negm, l, score_scale);  \
    else                                                                           \
      process_tile_lds<NQK, NG, false>(kl, kl + S::KBYTES, (K0), qreg, clo, chi, acc, m, negm, l, score_scale); \
  } while (0)
  // Steps go in pairs, so that the two register stages and the two LDS tiles take turns in a way the
  // compiler can see (it then waits for the loads of two steps ago only); an odd last step follows the
  // loops and has nothing left to fetch.  Both halves pass the same number of barriers.
  const int paired = steps & ~1;
  for (int o = 0; o < paired; o += 16) {
    const PageWindow pw_next = prefill_pages(my_begin + 32 * (o + 16), key_end, bt, page_size);
    const int n = paired - o < 16 ? paired - o : 16;
    for (int j = 0; j < n; j += 2) {
      STAGE_WORK(my_begin + 32 * (o + j), 0, st1);
      STAGE_WORK(my_begin + 32 * (o + j) + 32, 1, st0);
    }
    pw = pw_next;
  }
  if (steps & 1) {
    STAGE_PRODUCTS(my_begin + 32 * paired, 0);
    if (KS == 2) __syncthreads();                         // the merge below reuses the tiles' memory
  }
#undef STAGE_PRODUCTS
#undef STAGE_STORE
#undef STAGE_LOAD
#undef STAGE_WORK
  if (KS == 2) {
    // waves 4..7 hand over to waves 0..3 through the tiles' memory (free since the loop's last barrier),
    // lane by lane
    float* w = reinterpret_cast<float*>(lds) + (size_t)wave * PER_LANE * 64 + lane;
    if (half == 1) {
#pragma unroll
      for (int qg = 0; qg < NG; ++qg) {
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int e = 0; e < 4; ++e) w[(qg * (8 * NQK + 2) + 4 * n + e) * 64] = acc[qg][n][e];
        w[(qg * (8 * NQK + 2) + 8 * NQK) * 64] = m[qg];
        w[(qg * (8 * NQK + 2) + 8 * NQK + 1) * 64] = l[qg];
      }
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int qg = 0; qg < NG; ++qg) {
        const float m_b = w[(qg * (8 * NQK + 2) + 8 * NQK) * 64], l_b = w[(qg * (8 * NQK + 2) + 8 * NQK + 1) * 64];
        const float M = fmaxf(m[qg], m_b);
        const float fa = fast_exp2(m[qg] - M), fb = fast_exp2(m_b - M);
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[qg][n][e] = acc[qg][n][e] * fa + w[(qg * (8 * NQK + 2) + 4 * n + e) * 64] * fb;
        l[qg] = l[qg] * fa + l_b * fb;
        m[qg] = M;
      }
    }
    if (half == 1) return;
  }
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
    float lt = l[qg];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (chi[qg] < 0) continue;
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
    bf16_t* op = out + (size_t)tok[qg] * out_stride + (size_t)head * HD;
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n)
      *reinterpret_cast<uint2*>(op + 16 * n + 4 * g) =
          make_uint2(pack2_bf16(acc[qg][n][0] * inv, acc[qg][n][1] * inv),
                     pack2_bf16(acc[qg][n][2] * inv, acc[qg][n][3] * inv));
  }
}

// ------------------------------------------------------------------------------- prompt portions, tiles straight to LDS
// The same work split as attention_prefill_kernel, for head size 128, with the 32-key tiles of
// keys and values fetched by loads that write shared memory themselves (global_load_lds_dwordx4: a
// wave's 64 lanes fill 1024 consecutive bytes, every lane from an address of its own).  No register
// holds a tile on its way, no instruction copies it, and four tiles of shared memory take turns, so the
// loads run three tiles ahead of the products.
//   keys   32 rows of head_dim values, unpadded; the 16-byte piece p of key k lies at piece p ^ f(k),
//          f such that the 16 keys a product's lanes read together fall into 16 different bank groups
//   values one row of 32 keys per dim (64 bytes); piece p of dim d lies at piece p ^ (d / 4 % 4)
// A score product's 16 rows are the keys 8 (r / 4) + 4 sb + r % 4 of the tile (sb = which of the two
// products), so that in its result a lane group holds eight consecutive keys (4 from each product): the
// order in which a 16-byte piece of the values holds them, and the value product needs no shuffle.
// The loads are issued in inline assembly: the compiler, which cannot tell which of such loads a read of
// shared memory depends on, would otherwise wait for all of them before every read.  The waits for them
// stand in the code, by count (a wave's loads complete in order), and the loop holds no load of the
// compiler's own whose wait could be off by the ones it does not see: the page ids lie in shared memory.
#define DMA_TILES 4                       // tiles of shared memory that take turns
#define DMA_TABLE_TILES 128               // tiles whose page ids shared memory holds at a time (and 4 more, for the loads ahead)

// 16 bytes per lane from `src` to shared memory at lds_base + 16 * lane (lds_base the same in the whole wave).
// The instruction takes the place in shared memory from M0, which the compiler keeps for itself and warns
// about; nothing else in these kernels uses it.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load16_to_lds(const void* src, unsigned char* lds_base) {
#ifdef __HIP_DEVICE_COMPILE__
  typedef __attribute__((address_space(3))) unsigned char lds_byte_t;
  const unsigned at = (unsigned)__builtin_amdgcn_readfirstlane((int)(uintptr_t)(lds_byte_t*)lds_base);
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(src), "s"(at) : "memory", "m0");
#else
  __builtin_amdgcn_global_load_lds(src, lds_base, 16, 0, 0);
#endif
}
#pragma clang diagnostic pop
// at most N of this wave's loads are still on their way
template <int N>
__device__ __forceinline__ void loads_left() {
  static_assert(N >= 0 && N < 64, "the counter has six bits");
#ifdef __HIP_DEVICE_COMPILE__
  asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
#endif
}

template <int NQK>
struct DmaTile {
  static constexpr int HD = 32 * NQK;
  static constexpr int PR = HD / 8;       // 16-byte pieces of a key row
  static constexpr int ROUNDS = NQK / 2;  // load instructions per wave for a tile's keys, and as many for its values
  static constexpr int KBYTES = 32 * 2 * HD, VBYTES = HD * 64;
  static constexpr int BYTES = KBYTES + VBYTES;
  static_assert(NQK == 4, "head size 128 (with 64 the staged kernel is the faster one)");
  // the row that key k (0 .. 31) has in its score product, and what its pieces' places are xor-ed with
  __host__ __device__ static constexpr int row_of_key(int k) { return (k & 3) | (((k >> 3) & 3) << 2); }
  __host__ __device__ static constexpr int key_swizzle(int k) { return PR == 16 ? row_of_key(k) : row_of_key(k) >> 1; }
};

// What a lane's loads need that does not change from tile to tile.
template <int NQK>
struct DmaLanes {
  unsigned k_off[DmaTile<NQK>::ROUNDS];   // bytes from the first key row of the instruction's 16-key sub-block
  int k_sub[DmaTile<NQK>::ROUNDS];        // which of the tile's two sub-blocks (the same in the whole wave)
  unsigned v_off[DmaTile<NQK>::ROUNDS];   // bytes from the sub-block's first key in dim 0
  int v_sub[DmaTile<NQK>::ROUNDS];        // which sub-block this lane's piece lies in
  int dest[DmaTile<NQK>::ROUNDS];         // where the instruction's 1024 bytes go inside the tile's keys (and values)
};

template <int NQK>
__device__ __forceinline__ DmaLanes<NQK> dma_lanes(int page_size) {
  using T = DmaTile<NQK>;
  DmaLanes<NQK> d;
  const int lane = threadIdx.x & 63, wave = (threadIdx.x >> 6) % PREFILL_WAVES;
#pragma unroll
  for (int rd = 0; rd < T::ROUNDS; ++rd) {
    const int ins = wave + PREFILL_WAVES * rd;
    const int at = 64 * ins + lane;                       // the lane's place among the tile's pieces, as they lie in LDS
    const int key = at / T::PR, kpiece = (at % T::PR) ^ T::key_swizzle(key);
    d.k_sub[rd] = __builtin_amdgcn_readfirstlane(key >> 4);
    d.k_off[rd] = 2u * (unsigned)((key & 15) * T::HD + 8 * kpiece);
    const int dim = 16 * ins + (lane >> 2), vpiece = (lane & 3) ^ ((dim >> 2) & 3);
    d.v_sub[rd] = vpiece >> 1;
    d.v_off[rd] = 2u * (unsigned)(dim * page_size + 8 * (vpiece & 1));
    d.dest[rd] = 1024 * ins;
  }
  return d;
}

// Start the loads of the tile at key0 into the tile of shared memory at `tile` (keys, then values); page0 / page1
// are the page ids of its two 16-key sub-blocks.  A sub-block without a page reads page 0: its keys are
// never seen, and its values count as zero in the products.
template <int NQK>
__device__ __forceinline__ void dma_tile_load(unsigned char* tile, int key0, int page0, int page1, int page_size,
                                              const DmaLanes<NQK>& dl, const bf16_t* __restrict__ k_head,
                                              const bf16_t* __restrict__ v_head, unsigned page_elems) {
  using T = DmaTile<NQK>;
  const unsigned off0 = (unsigned)(key0 % page_size), off1 = (unsigned)((key0 + 16) % page_size);
  const size_t base0 = (size_t)(unsigned)(page0 < 0 ? 0 : page0) * page_elems;
  const size_t base1 = (size_t)(unsigned)(page1 < 0 ? 0 : page1) * page_elems;
  const char* const k0 = reinterpret_cast<const char*>(k_head + base0 + off0 * T::HD);
  const char* const k1 = reinterpret_cast<const char*>(k_head + base1 + off1 * T::HD);
  const char* const v0 = reinterpret_cast<const char*>(v_head + base0 + off0);
  const char* const v1 = reinterpret_cast<const char*>(v_head + base1 + off1);
#pragma unroll
  for (int rd = 0; rd < T::ROUNDS; ++rd) load16_to_lds((dl.k_sub[rd] ? k1 : k0) + dl.k_off[rd], tile + dl.dest[rd]);
#pragma unroll
  for (int rd = 0; rd < T::ROUNDS; ++rd)
    load16_to_lds((dl.v_sub[rd] ? v1 : v0) + dl.v_off[rd], tile + T::KBYTES + dl.dest[rd]);
}

// Scores, softmax update and value product of one wave for the tile in shared memory; as process_tile_lds,
// with the keys' order and the tile's layout as described above.
template <int NQK, int NG, bool masked>
__device__ __forceinline__ void dma_tile_products(const unsigned char* __restrict__ tile, int key0, const Pack8 (&qreg)[NG][NQK],
                                                  const int (&col_lo)[NG], const int (&col_hi)[NG],
                                                  f32x4_t (&acc)[NG][2 * NQK], float (&m)[NG], f32x4_t (&negm)[NG],
                                                  float (&l)[NG], const int (&k_at)[2][NQK], int v_at, int max_hi,
                                                  bool ok0, bool ok1, const ScoreScale& scale) {
  using T = DmaTile<NQK>;
  const int lane = threadIdx.x & 63, g = lane >> 4;
  f32x4_t s[NG][2];
#pragma unroll
  for (int sb = 0; sb < 2; ++sb)
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      Pack8 kf;
      kf.u4 = ld16(tile + k_at[sb][ch]);
#pragma unroll
      for (int q = 0; q < NG; ++q)
        s[q][sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qreg[q][ch].v, ch == 0 ? negm[q] : s[q][sb], 0, 0, 0);
    }
  // s[q][sb][r] is the exponent of key key0 + 8 g + 4 sb + r for this lane's column
  Pack8 p[NG];
  prompt_tile_softmax<NQK, NG, masked>(s, key0, [g](int sb, int r) { return 8 * g + 4 * sb + r; }, col_lo, col_hi,
                                       acc, m, negm, l, p, scale);
  // masked tiles only: which of this lane's eight keys (8 g ..) hold written values.  The others (past the end
  // of the data, or in a sub-block without a page, which reads page 0) may hold anything and must count as 0.
  uint32_t live[4] = {0xffffffffu, 0xffffffffu, 0xffffffffu, 0xffffffffu};
  if (masked) {
    const bool ok = g >> 1 ? ok1 : ok0;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const int kk = key0 + 8 * g + 2 * w;
      live[w] = (ok && kk <= max_hi ? 0x0000ffffu : 0u) | (ok && kk + 1 <= max_hi ? 0xffff0000u : 0u);
    }
  }
#pragma unroll
  for (int n = 0; n < 2 * NQK; ++n) {
    Pack8 vf;
    vf.u4 = ld16(tile + T::KBYTES + v_at + 1024 * n);
    if (masked) {
#pragma unroll
      for (int w = 0; w < 4; ++w) vf.w[w] &= live[w];
    }
#pragma unroll
    for (int q = 0; q < NG; ++q) acc[q][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, p[q].v, acc[q][n], 0, 0, 0);
  }
}

template <int NQK, int KS>
__global__ void __launch_bounds__(64 * PREFILL_WAVES * KS, 2 / KS)
attention_prefill_dma_kernel(const bf16_t* __restrict__ q, int q_stride, bf16_t* __restrict__ out, int out_stride,
                             const bf16_t* __restrict__ k_pool, const bf16_t* __restrict__ v_pool,
                             const int* __restrict__ tiles, const int* __restrict__ positions,
                             const int* __restrict__ token_entry, const int* __restrict__ block_table,
                             int bt_stride, int page_size, int nq, int nkv, float scale_log2e, int window,
                             int n_tiles) {
  using T = DmaTile<NQK>;
  constexpr int HD = 32 * NQK;
  constexpr int NG = PREFILL_GROUPS;
  constexpr int PER_LANE = NG * (8 * NQK + 2);            // floats a lane hands over in the merge
  constexpr int PER = 2 * T::ROUNDS;                      // load instructions of a wave per tile
  constexpr int TABLE = 2 * (DMA_TABLE_TILES + 4);        // page ids in shared memory, one per 16-key sub-block
  static_assert(KS == 1 || PREFILL_WAVES * PER_LANE * 64 * 4 <= KS * DMA_TILES * T::BYTES, "the merge reuses the tiles' memory");
  __shared__ __attribute__((aligned(1024))) unsigned char lds[KS * DMA_TILES * T::BYTES];   // [half][tile][keys | values]
  __shared__ int page_ids[KS][TABLE];
  const int wave_id = (int)(threadIdx.x >> 6);
  const int lane = threadIdx.x & 63, wave = wave_id % PREFILL_WAVES, half = wave_id / PREFILL_WAVES;
  const int g = lane >> 4, c = lane & 15;
  unsigned char* const tile_lds = lds + half * DMA_TILES * T::BYTES;
  int* const pages = page_ids[half];
  const int G = nq / nkv, chunks = (G + PREFILL_WAVES - 1) / PREFILL_WAVES, per_kv = n_tiles * chunks;
  int kvh, rest;
  if (nkv % 8 == 0) {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    kvh = (slot / per_kv) * 8 + xcd;
    rest = slot % per_kv;
  } else {
    kvh = blockIdx.x / per_kv;
    rest = blockIdx.x % per_kv;
  }
  const int tile_idx = n_tiles - 1 - rest / chunks;
  const int head_in_group = (rest % chunks) * PREFILL_WAVES + wave;
  const bool head_ok = head_in_group < G;                 // a wave without a head still helps to load
  const int head = kvh * G + (head_ok ? head_in_group : G - 1);
  const int first = tiles[2 * tile_idx], count = tiles[2 * tile_idx + 1];
  int clo[NG], chi[NG], tok[NG];
  Pack8 qreg[NG][NQK];
  const ScoreScale score_scale = split_scale(scale_log2e);
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
    const bool ok = head_ok && 16 * qg + c < count;
    tok[qg] = first + (16 * qg + c < count ? 16 * qg + c : 0);
    const int pos = positions[tok[qg]];
    clo[qg] = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
    chi[qg] = ok ? pos : -1;
    const bf16_t* qp = q + (size_t)tok[qg] * q_stride + (size_t)head * HD + 8 * g;
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      if (ok) qreg[qg][ch].u4 = *reinterpret_cast<const uint4*>(qp + 32 * ch);
      else qreg[qg][ch].u4 = make_uint4(0, 0, 0, 0);
      // the power of two in scale * log2(e) goes into the queries once (exact); the scores take the rest
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t two = qreg[qg][ch].w[w];
        qreg[qg][ch].w[w] = pack2_bf16(__uint_as_float(two << 16) * score_scale.pow2,
                                       __uint_as_float(two & 0xffff0000u) * score_scale.pow2);
      }
    }
  }
  const int last_pos = positions[first + count - 1];
  const int first_pos = positions[first];
  const int open_lo = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int key_begin = ((window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0) & ~31;
  const int key_end = last_pos + 1;
  const int steps = ((key_end - key_begin + 31) / 32 + KS - 1) / KS;    // this half's share of the 32-key tiles
  const int my_begin = key_begin + half * steps * 32;
  const int* bt = block_table + (size_t)token_entry[first] * bt_stride;
  f32x4_t acc[NG][2 * NQK];
  float m[NG], l[NG];
  f32x4_t negm[NG];
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n) acc[qg][n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    m[qg] = NEG_BIG;
    negm[qg] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    l[qg] = 0.f;
  }
  // where this lane reads its operands inside a tile: key row 8 (c / 4) + 4 sb + c % 4, piece 4 ch + g; dim 16 n + c, piece g
  int k_at[2][NQK];
#pragma unroll
  for (int sb = 0; sb < 2; ++sb)
#pragma unroll
    for (int ch = 0; ch < NQK; ++ch) {
      const int key = 8 * (c >> 2) + 4 * sb + (c & 3);
      k_at[sb][ch] = key * 2 * HD + 16 * ((4 * ch + g) ^ T::key_swizzle(key));
    }
  const int v_at = c * 64 + 16 * (g ^ (c >> 2));
  const DmaLanes<NQK> dl = dma_lanes<NQK>(page_size);
  const unsigned page_elems = (unsigned)(nkv * page_size * HD);
  const bf16_t* const k_head = k_pool + (size_t)kvh * page_size * HD;
  const bf16_t* const v_head = v_pool + (size_t)kvh * page_size * HD;
  // Tile i of this half is loaded with the page ids pages[2 (i - t0)], pages[2 (i - t0) + 1].
#define TILE_LOAD(I, T0) dma_tile_load<NQK>(tile_lds + ((I) % DMA_TILES) * T::BYTES, my_begin + 32 * (I), pages[2 * ((I) - (T0))], \
                                            pages[2 * ((I) - (T0)) + 1], page_size, dl, k_head, v_head, page_elems)
  // Tiles 0, 1 and 2 go on their way; in step i tile i + 3 follows, into the place of tile i - 1, which every wave
  // has left behind when it passes the step's barrier.  Loads are started for the tiles of this half's steps only,
  // so the last steps wait for fewer loads to be left.
  for (int t0 = 0; t0 < steps; t0 += DMA_TABLE_TILES) {
    // page ids of the tiles t0 .. t0 + DMA_TABLE_TILES + 3 (the loads run up to three tiles ahead of the steps)
    __syncthreads();
    for (int e = threadIdx.x & (64 * PREFILL_WAVES - 1); e < TABLE; e += 64 * PREFILL_WAVES) {
      const int kb = my_begin + 32 * t0 + 16 * e;
      pages[e] = kb < key_end ? bt[kb / page_size] : -1;
    }
    __syncthreads();
    if (t0 == 0) {
      if (steps > 0) TILE_LOAD(0, 0);
      if (steps > 1) TILE_LOAD(1, 0);
      if (steps > 2) TILE_LOAD(2, 0);
    }
    const int t1 = t0 + DMA_TABLE_TILES < steps ? t0 + DMA_TABLE_TILES : steps;
    for (int i = t0; i < t1; ++i) {
      const int K0 = my_begin + 32 * i;
      unsigned char* const tile = tile_lds + (i % DMA_TILES) * T::BYTES;
      // this wave's part of tile i has landed once only the loads of the tiles after it are left
      if (i + 2 < steps) loads_left<2 * PER>();
      else if (i + 1 < steps) loads_left<PER>();
      else loads_left<0>();
      // The bare barrier: with the fence of __syncthreads the compiler would wait here for every load it
      // knows of.  No access to memory may move across it: the next loads overwrite what other waves read
      // until here.
      asm volatile("" ::: "memory");
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");
      if (i + 3 < steps) TILE_LOAD(i + 3, t0);
      if (K0 + 31 > first_pos || K0 < open_lo) {
        const bool ok0 = pages[2 * (i - t0)] >= 0, ok1 = pages[2 * (i - t0) + 1] >= 0;
        dma_tile_products<NQK, NG, true>(tile, K0, qreg, clo, chi, acc, m, negm, l, k_at, v_at, last_pos, ok0, ok1, score_scale);
      } else {
        dma_tile_products<NQK, NG, false>(tile, K0, qreg, clo, chi, acc, m, negm, l, k_at, v_at, last_pos, true, true, score_scale);
      }
    }
  }
#undef TILE_LOAD
  // nothing is on its way any more, and every wave is done with the tiles: their memory serves the merge
  loads_left<0>();
  __syncthreads();
  if (KS == 2) {
    float* w = reinterpret_cast<float*>(lds) + (size_t)wave * PER_LANE * 64 + lane;
    if (half == 1) {
#pragma unroll
      for (int qg = 0; qg < NG; ++qg) {
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int e = 0; e < 4; ++e) w[(qg * (8 * NQK + 2) + 4 * n + e) * 64] = acc[qg][n][e];
        w[(qg * (8 * NQK + 2) + 8 * NQK) * 64] = m[qg];
        w[(qg * (8 * NQK + 2) + 8 * NQK + 1) * 64] = l[qg];
      }
    }
    __syncthreads();
    if (half == 0) {
#pragma unroll
      for (int qg = 0; qg < NG; ++qg) {
        const float m_b = w[(qg * (8 * NQK + 2) + 8 * NQK) * 64], l_b = w[(qg * (8 * NQK + 2) + 8 * NQK + 1) * 64];
        const float M = fmaxf(m[qg], m_b);
        const float fa = fast_exp2(m[qg] - M), fb = fast_exp2(m_b - M);
#pragma unroll
        for (int n = 0; n < 2 * NQK; ++n)
#pragma unroll
          for (int e = 0; e < 4; ++e)
            acc[qg][n][e] = acc[qg][n][e] * fa + w[(qg * (8 * NQK + 2) + 4 * n + e) * 64] * fb;
        l[qg] = l[qg] * fa + l_b * fb;
        m[qg] = M;
      }
    }
    if (half == 1) return;
  }
#pragma unroll
  for (int qg = 0; qg < NG; ++qg) {
    float lt = l[qg];
    lt += __shfl_xor(lt, 16, 64);
    lt += __shfl_xor(lt, 32, 64);
    if (chi[qg] < 0) continue;
    const float inv = lt > 0.f ? 1.f / lt : 0.f;
    bf16_t* op = out + (size_t)tok[qg] * out_stride + (size_t)head * HD;
#pragma unroll
    for (int n = 0; n < 2 * NQK; ++n)
      *reinterpret_cast<uint2*>(op + 16 * n + 4 * g) =
          make_uint2(pack2_bf16(acc[qg][n][0] * inv, acc[qg][n][1] * inv),
                     pack2_bf16(acc[qg][n][2] * inv, acc[qg][n][3] * inv));
  }
}

// tokens of one request a prompt tile may hold
extern "C" int ullm_attention_prefill_tile(void) { return 16 * PREFILL_GROUPS; }

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
static int decode_launch(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, float* workspace, hipStream_t stream, const DecodeFuse* fuse = nullptr) {
  if (n_items <= 0) return 0;
  if (!ullm_attention_mfma_supports(hd, page_size, nq, nkv)) return ULLM_ERR_UNSUPPORTED;
  if (waves != 1 && waves != 4 && waves != 8) return ULLM_ERR_UNSUPPORTED;
  if (hd == 256 && waves == 8) waves = 4;                // shared memory of the merge
  if (num_splits < 1 || num_splits > 65535 || window < 0) return ULLM_ERR_SHAPE;
  if (num_splits > 1 && !workspace) return ULLM_ERR_SHAPE;
  const int G = nq / nkv, groups = (G + 15) / 16;
  if (n_items > 65535 || nkv * groups > 65535) return ULLM_ERR_SHAPE;
  const float sl = scale * 1.4426950408889634f;
  dim3 grid(num_splits, nkv * groups, n_items), block(64 * waves);
  const DecodeFuse f = fuse ? *fuse : DecodeFuse{nullptr, nullptr, 0.f, nullptr, 0, nullptr, nullptr};
#define ARGS (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, (const bf16_t*)k_pool, (const bf16_t*)v_pool, token_list, \
    positions, token_entry, block_table, bt_stride, page_size, nq, nkv, sl, window, num_splits, workspace, f
#define CALL_AS(N, F) do {                                                                                     \
    if (waves == 8) hipLaunchKernelGGL((attention_decode_kernel<N, 8, F>), grid, block, 0, stream, ARGS);      \
    else if (waves == 4) hipLaunchKernelGGL((attention_decode_kernel<N, 4, F>), grid, block, 0, stream, ARGS); \
    else hipLaunchKernelGGL((attention_decode_kernel<N, 1, F>), grid, block, 0, stream, ARGS);                 \
  } while (0)
  if (fuse) {
    switch (hd) {
      case 64: CALL_AS(2, true); break;
      case 128: CALL_AS(4, true); break;
      case 256: CALL_AS(8, true); break;
      default: return ULLM_ERR_UNSUPPORTED;
    }
  } else {
#define CALL(N) CALL_AS(N, false)
    DISPATCH_NQK(hd, CALL)
#undef CALL
  }
#undef CALL_AS
#undef ARGS
  int rc = (int)hipGetLastError();
  if (rc != 0 || num_splits == 1) return rc;
  hipLaunchKernelGGL(attention_reduce_kernel, dim3(n_items, nq), dim3(64), 0, stream, workspace, (bf16_t*)out,
                     out_stride, token_list, nq, hd, num_splits);
  ULLM_LAUNCH_CHECK();
}

extern "C" int ullm_attention_decode(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, float* workspace, hipStream_t stream) {
  return decode_launch(q, q_stride, out, out_stride, k_pool, v_pool, token_list, n_items, positions, token_entry,
                       block_table, bt_stride, page_size, nq, nkv, hd, scale, window, num_splits, waves, workspace,
                       stream);
}

// Head sizes and position encodings the fused decode step takes: rotation of the whole head in
// half-split pairs (style 1, rot == hd) or none (style 0 or rot 0), head sizes whose halves are whole
// 32-dim chunks.
extern "C" int ullm_attention_decode_fused_supports(int hd, int page_size, int nq, int nkv, int rot, int style) {
  if (!ullm_attention_mfma_supports(hd, page_size, nq, nkv)) return 0;
  if (hd != 64 && hd != 128 && hd != 256) return 0;
  const bool rotates = style != 0 && rot > 0;
  return !rotates || (style == 1 && rot == hd);
}

// ullm_attention_decode with the per-head norm, the rotation and the cache write of the step folded in:
// `qkv` [tokens, (nq + 2 nkv) * hd] is the fused projection as it leaves the matrix product.  q_gain /
// k_gain float32 [hd] or null (no norm); cos_sin float32 [table_rows, rot] or null; write_kv = 0 for a
// layer that reads a cache another layer writes (then k and v of the projection are not used).
// Every item must be the last token of its request so far (its position is the newest key).
extern "C" int ullm_attention_decode_fused(
    const void* qkv, int qkv_stride, void* out, int out_stride, void* k_pool, void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, float* workspace, const float* q_gain, const float* k_gain, float eps,
    const float* cos_sin, int table_rows, int rot, int style, int write_kv, hipStream_t stream) {
  if (!ullm_attention_decode_fused_supports(hd, page_size, nq, nkv, rot, style)) return ULLM_ERR_UNSUPPORTED;
  const bool rotates = style != 0 && rot > 0;
  if (rotates && (!cos_sin || table_rows <= 0)) return ULLM_ERR_SHAPE;
  if ((qkv_stride & 7) || ((uintptr_t)qkv & 15) || ((uintptr_t)k_pool & 15) || ((uintptr_t)q_gain & 15) ||
      ((uintptr_t)k_gain & 15) || ((uintptr_t)cos_sin & 15))
    return ULLM_ERR_SHAPE;
  const DecodeFuse f = {q_gain, k_gain, eps, rotates ? cos_sin : nullptr, table_rows,
                        write_kv ? (bf16_t*)k_pool : nullptr, write_kv ? (bf16_t*)v_pool : nullptr};
  return decode_launch(qkv, qkv_stride, out, out_stride, k_pool, v_pool, token_list, n_items, positions, token_entry,
                       block_table, bt_stride, page_size, nq, nkv, hd, scale, window, num_splits, waves, workspace,
                       stream, &f);
}

// ------------------------------------------------------------------------------- no allocation
// The splits' partial results of ullm_attention_decode_static (see no_alloc.h).  In host code this
// name is only a stand-in for the symbol: the address kernels can use is looked up per device.
static __device__ __align__(256) float scratch[ULLM_DECODE_SCRATCH_FLOATS];

#define ULLM_MAX_DEVICES 64
static float* scratch_ptr[ULLM_MAX_DEVICES];      // per device: that GPU's copy of the array

// The current device's copy of the array: looked up at the first call on the device (which is current),
// kept per device.  0 and *err set if the lookup fails.
static float* scratch_of_current_device(int* err) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) { *err = (int)e; return nullptr; }
  if (dev < 0 || dev >= ULLM_MAX_DEVICES) { *err = ULLM_ERR_UNSUPPORTED; return nullptr; }
  float* ws = __atomic_load_n(&scratch_ptr[dev], __ATOMIC_ACQUIRE);
  if (!ws) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) { *err = (int)e; return nullptr; }
    if (!p) { *err = (int)hipErrorInvalidSymbol; return nullptr; }
    ws = static_cast<float*>(p);
    __atomic_store_n(&scratch_ptr[dev], ws, __ATOMIC_RELEASE);   // two first callers store the same address
  }
  return ws;
}

extern "C" long long ullm_attention_decode_static_capacity(void) {
  int err = 0;
  scratch_of_current_device(&err);                // also the warm-up: the lookup is not stream-ordered
  return ULLM_DECODE_SCRATCH_FLOATS;
}

extern "C" int ullm_attention_decode_static(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* token_list, int n_items, const int* positions, const int* token_entry,
    const int* block_table, int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window,
    int num_splits, int waves, hipStream_t stream) {
  if (n_items <= 0) return 0;
  if (num_splits < 1 || nq < 1 || hd < 1) return ULLM_ERR_SHAPE;
  if (ullm_attention_decode_workspace(n_items, nq, hd, num_splits) > (long long)ULLM_DECODE_SCRATCH_FLOATS)
    return ULLM_ERR_SCRATCH;
  int err = 0;
  float* ws = scratch_of_current_device(&err);
  if (!ws) return err;
  return decode_launch(q, q_stride, out, out_stride, k_pool, v_pool, token_list, n_items, positions, token_entry,
                       block_table, bt_stride, page_size, nq, nkv, hd, scale, window, num_splits, waves, ws, stream);
}

template <int N, typename... Args>
static void prefill_launch(int halves, bool staged, unsigned blocks, hipStream_t stream, Args... args) {
  if constexpr (N == 4) {
    if (!staged) {                                        // tiles straight to shared memory
      if (halves == 2)
        hipLaunchKernelGGL((attention_prefill_dma_kernel<N, 2>), dim3(blocks), dim3(64 * PREFILL_WAVES * 2), 0, stream, args...);
      else
        hipLaunchKernelGGL((attention_prefill_dma_kernel<N, 1>), dim3(blocks), dim3(64 * PREFILL_WAVES), 0, stream, args...);
      return;
    }
  }
  if constexpr (N <= 4) {
    if (halves == 2) {
      hipLaunchKernelGGL((attention_prefill_kernel<N, 2>), dim3(blocks), dim3(64 * PREFILL_WAVES * 2), 0, stream, args...);
      return;
    }
  }
  hipLaunchKernelGGL((attention_prefill_kernel<N, 1>), dim3(blocks), dim3(64 * PREFILL_WAVES), 0, stream, args...);
}

// Compute units of the current device (asked once per device).
static int compute_units() {
  static int units[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
  if (units[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
    units[dev] = n;
  }
  return units[dev];
}

// `halves`: 2 = a block's eight waves share the keys of a tile between two halves (blocks last half as
// long, one block per compute unit: best when a few long tiles would otherwise set the time);
// 1 = four waves per block take all keys (two independent blocks per compute unit, which drift apart
// so that one block's products overlap the other's exponentials: best when there is enough work to
// keep every unit busy to the end); 0 = choose.  The choice compares the work per unit,
// `keys_total` (sum over the tiles of the keys each sees) spread over two blocks per unit, with the
// longest tile `keys_max`; without these figures (0) it goes by the number of blocks.
extern "C" int ullm_attention_prefill(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* tiles, int n_tiles, const int* positions, const int* token_entry, const int* block_table,
    int bt_stride, int page_size, int nq, int nkv, int hd, float scale, int window, int halves,
    long long keys_total, int keys_max, hipStream_t stream) {
  if (n_tiles <= 0) return 0;
  if (!ullm_attention_mfma_supports(hd, page_size, nq, nkv)) return ULLM_ERR_UNSUPPORTED;
  const bool staged = halves >= 10;                       // 10, 11, 12: as 0, 1, 2 with the kernel that stages tiles in registers
  if (staged) halves -= 10;
  if (window < 0 || halves < 0 || halves > 2) return ULLM_ERR_SHAPE;
  const int chunks = (nq / nkv + PREFILL_WAVES - 1) / PREFILL_WAVES;
  const long long blocks = (long long)n_tiles * nkv * chunks;
  if (blocks > 0x7fffffffLL) return ULLM_ERR_SHAPE;
  if ((long long)nkv * page_size * hd > 0x7fffffffLL) return ULLM_ERR_SHAPE;   // 32-bit distance between pages
  if (hd > 128) halves = 1;                              // shared memory holds one half's tiles only
  if (halves == 0) {
    const long long units = compute_units();
    bool enough;
    if (keys_total > 0 && keys_max > 0) {
      if (window > 0) {
        if (keys_max > window + 32) keys_max = window + 32;
        if (keys_total > (long long)n_tiles * (window + 32)) keys_total = (long long)n_tiles * (window + 32);
      }
      enough = (double)keys_total * nkv * chunks / (2.0 * units) >= 0.6 * keys_max;
    } else {
      enough = blocks >= 3 * units;
    }
    halves = (enough && blocks >= 2 * units) ? 1 : 2;
  }
  const float sl = scale * 1.4426950408889634f;
#define CALL(N) prefill_launch<N>(halves, staged, (unsigned)blocks, stream, (const bf16_t*)q, q_stride, (bf16_t*)out, out_stride, \
    (const bf16_t*)k_pool, (const bf16_t*)v_pool, tiles, positions, token_entry, block_table, bt_stride, page_size,    \
    nq, nkv, sl, window, n_tiles)
  DISPATCH_NQK(hd, CALL)
#undef CALL
  ULLM_LAUNCH_CHECK();
}
