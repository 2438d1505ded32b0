// Paged grouped-query attention, general form: any head size up to 512, any number of heads and
// groups, any page size, any mix of prompt portions and single decoded tokens, optional window.
// One block per (token, query head); keys are visited in tiles of the block size in a fixed order
// that depends only on the token's own position, so the result for a token is the same however
// the batch was cut.  Scores, running maximum, sum and output are 32-bit.
// Pools: keys [page, kv_head, row, head_dim]; values [page, kv_head, head_dim, row].
//
// Semantics as the reference asks of its attention library (ullm/layers/attention.py:76-104,
// 298-309): scale = given (head_dim^-0.5, ullm/models/qwen3.py:81), causal with the queries at the
// end of the keys, query head h reads kv head h / (nq / nkv).
#include "common.h"

#define ATT_THREADS 128
#define ATT_MAX_HD 512

template <typename T>
__global__ void __launch_bounds__(ATT_THREADS)
paged_attention_generic_kernel(const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride,
                               const T* __restrict__ k_pool, const T* __restrict__ v_pool,
                               const int* __restrict__ positions, const int* __restrict__ token_entry,
                               const int* __restrict__ block_table, int bt_stride, int page_size,
                               int nq, int nkv, int hd, float scale, int window) {
  __shared__ float q_s[ATT_MAX_HD];
  __shared__ float p_s[ATT_THREADS];
  __shared__ long long row_s[ATT_THREADS];
  __shared__ float scratch[16];
  const int t = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (nq / nkv);
  const int pos = positions[t];
  const int* bt = block_table + (size_t)token_entry[t] * bt_stride;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int hi = pos;
  const T* qp = q + (size_t)t * q_stride + (size_t)h * hd;
  for (int i = tid; i < hd; i += ATT_THREADS) q_s[i] = ld_f32(qp + i) * scale;
  __syncthreads();

  constexpr int DPT = ATT_MAX_HD / ATT_THREADS;  // output dims per thread
  float acc[DPT];
#pragma unroll
  for (int r = 0; r < DPT; ++r) acc[r] = 0.f;
  float m = -INFINITY, l = 0.f;

  for (int base = lo; base <= hi; base += ATT_THREADS) {
    const int j = base + tid;
    float s = -INFINITY;
    long long row = -1;
    if (j <= hi) {
      const int page = bt[j / page_size];
      if (page >= 0) {
        row = ((long long)page * nkv + kvh) * page_size + (j % page_size);
        const T* kp = k_pool + row * hd;
        float d = 0.f;
        for (int i = 0; i < hd; ++i) d += q_s[i] * ld_f32(kp + i);
        s = d;
      }
    }
    const float tile_max = block_max(s, scratch);
    const float m_new = fmaxf(m, tile_max);
    // the token's own key is always present, so m_new is finite from the first tile that holds it;
    // a tile without any valid key leaves everything unchanged
    const float p = (row >= 0) ? expf(s - m_new) : 0.f;
    const float tile_sum = block_sum(p, scratch);
    __syncthreads();
    p_s[tid] = p;
    row_s[tid] = row;
    __syncthreads();
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * alpha + tile_sum;
    const int n_tile = (hi - base + 1 < ATT_THREADS) ? hi - base + 1 : ATT_THREADS;
#pragma unroll
    for (int r = 0; r < DPT; ++r) {
      const int d = tid + r * ATT_THREADS;
      if (d < hd) {
        float a = acc[r] * alpha;
        for (int jj = 0; jj < n_tile; ++jj) {
          const long long vr = row_s[jj];
          if (vr >= 0) a += p_s[jj] * ld_f32(v_pool + (vr / page_size) * page_size * hd + (size_t)d * page_size + vr % page_size);
        }
        acc[r] = a;
      }
    }
    if (m_new > -INFINITY) m = m_new;
  }
  T* op = out + (size_t)t * out_stride + (size_t)h * hd;
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int r = 0; r < DPT; ++r) {
    const int d = tid + r * ATT_THREADS;
    if (d < hd) st_f32(op + d, acc[r] * inv);
  }
}

extern "C" int ullm_paged_attention_generic(
    const void* q, int q_stride, void* out, int out_stride, const void* k_pool, const void* v_pool,
    const int* positions, const int* token_entry, const int* block_table, int bt_stride, int page_size,
    int T_, int nq, int nkv, int hd, float scale, int window, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (hd <= 0 || hd > ATT_MAX_HD || nq <= 0 || nkv <= 0 || nq % nkv != 0 || page_size <= 0 || window < 0)
    return ULLM_ERR_SHAPE;
  dim3 grid(T_, nq), block(ATT_THREADS);
#define GO(TT) hipLaunchKernelGGL(paged_attention_generic_kernel<TT>, grid, block, 0, stream, \
    (const TT*)q, q_stride, (TT*)out, out_stride, (const TT*)k_pool, (const TT*)v_pool, positions, \
    token_entry, block_table, bt_stride, page_size, nq, nkv, hd, scale, window)
  if (dtype == ULLM_F32) GO(float);
  else if (dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}
