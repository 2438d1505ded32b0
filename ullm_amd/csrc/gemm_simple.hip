// C[M, N] = A[M, K] * W[N, K]^T (+ bias[N]) with 32-bit multiply-add in a fixed K order.
// The product of row m never depends on M or on the other rows, so a token's result is the same
// in every batch.  This is the true 32-bit matrix product of the float32 mode (no matrix-core
// input rounding) and the general fallback for bfloat16 operands with 32-bit output.
// Weights are [out, in] as the reference stores them for F.linear (ullm/layers/linear.py:165,268).
#include "common.h"

#define GS_BM 64
#define GS_BN 64
#define GS_BK 16

template <typename TA, typename TW, typename TC>
__global__ void __launch_bounds__(256)
gemm_simple_kernel(const TA* __restrict__ A, int lda, const TW* __restrict__ W, int ldw,
                   const float* __restrict__ bias, TC* __restrict__ C, int ldc, int M, int N, int K) {
  __shared__ float As[GS_BK][GS_BM + 4];
  __shared__ float Ws[GS_BK][GS_BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * GS_BM, n0 = blockIdx.x * GS_BN;
  const int tm = (tid / 16) * 4, tn = (tid % 16) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GS_BK) {
    // 64 rows x 16 k = 1024 elements per operand, 4 per thread; consecutive threads read along k
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int e = tid + r * 256;
      const int row = e / GS_BK, kk = e % GS_BK;
      const int gm = m0 + row, gn = n0 + row, gk = k0 + kk;
      As[kk][row] = (gm < M && gk < K) ? ld_f32(A + (size_t)gm * lda + gk) : 0.f;
      Ws[kk][row] = (gn < N && gk < K) ? ld_f32(W + (size_t)gn * ldw + gk) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GS_BK; ++kk) {
      float a[4], w[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][tm + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) w[j] = Ws[kk][tn + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], w[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int gm = m0 + tm + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int gn = n0 + tn + j;
      if (gn >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[gn];
      st_f32(C + (size_t)gm * ldc + gn, v);
    }
  }
}

extern "C" int ullm_gemm_simple(const void* A, int lda, const void* W, int ldw, const float* bias,
                                void* C, int ldc, int M, int N, int K, int a_dtype, int w_dtype,
                                int c_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (K <= 0 || lda < K || ldw < K || ldc < N) return ULLM_ERR_SHAPE;
  if ((a_dtype | w_dtype | c_dtype) & ~1) return ULLM_ERR_DTYPE;
  dim3 grid((N + GS_BN - 1) / GS_BN, (M + GS_BM - 1) / GS_BM), block(256);
#define GO(TA, TW, TC) hipLaunchKernelGGL((gemm_simple_kernel<TA, TW, TC>), grid, block, 0, stream, \
    (const TA*)A, lda, (const TW*)W, ldw, bias, (TC*)C, ldc, M, N, K)
  const int key = a_dtype * 4 + w_dtype * 2 + c_dtype;
  switch (key) {
    case 0: GO(float, float, float); break;
    case 7: GO(bf16_t, bf16_t, bf16_t); break;
    case 6: GO(bf16_t, bf16_t, float); break;
    case 2: GO(float, bf16_t, float); break;
    default: return ULLM_ERR_DTYPE;
  }
#undef GO
  ULLM_LAUNCH_CHECK();
}
