// C[M, N] = A[M, K] * W[N, K]^T (+ bias) for few rows (M <= 64), bfloat16 operands, 32-bit
// accumulation, output bfloat16 or float32.  This is the decode-time matrix product: its time is the
// time to stream W once from HBM, so the kernel is built around the weight loads.
//
// A block owns 16 consecutive rows of W (16 output columns); its waves split K between them.  Per 32
// values of K a wave issues one 16-byte load per lane straight from global memory for the W tile
// (A operand of v_mfma_f32_16x16x32_bf16: lane (r, g) holds W[n0 + r][k + 8g .. +8]) and one per
// 16 rows of the activations (B operand: lane (m, g) holds A[m][k + 8g .. +8]; the activations are
// small and stay in cache).  The loop is unrolled so that many loads are in flight.  The waves'
// partial 16x16 results are added in wave order through shared memory, so the result does not depend
// on timing.  Weights are [out, in] (ullm/layers/linear.py:165).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack8 {
  bf16x8_t v;
  uint4 u4;
};

#define SK_MAX_WAVES 16
#define SK_UNROLL 4

// MT = number of 16-row tiles of A (M <= 16 * MT).
template <int MT, typename TC>
__global__ void __launch_bounds__(64 * SK_MAX_WAVES)
gemm_skinny_kernel(const bf16_t* __restrict__ A, int lda, const bf16_t* __restrict__ W, int ldw,
                   const float* __restrict__ bias, TC* __restrict__ C, int ldc, int M, int N, int K,
                   int k_per_wave) {
  __shared__ float red[SK_MAX_WAVES - 1][MT][64 * 4];   // wave 0 adds the others' partials to its own
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int g = lane >> 4, r = lane & 15;
  const int n0 = blockIdx.x * 16;
  const int n = n0 + r < N ? n0 + r : N - 1;          // rows past N repeat the last row; never stored
  const bf16_t* wp = W + (size_t)n * ldw + 8 * g;
  const bf16_t* ap[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r < M ? 16 * t + r : M - 1;
    ap[t] = A + (size_t)m * lda + 8 * g;
  }
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  const int k_begin = wave * k_per_wave;
  int k_end = k_begin + k_per_wave;
  if (k_end > K) k_end = K;
  int k = k_begin;
  // full steps of SK_UNROLL * 32 values
  for (; k + 32 * SK_UNROLL <= k_end; k += 32 * SK_UNROLL) {
    Pack8 w[SK_UNROLL], a[SK_UNROLL][MT];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) w[u].u4 = *reinterpret_cast<const uint4*>(wp + k + 32 * u);
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t) a[u][t].u4 = *reinterpret_cast<const uint4*>(ap[t] + k + 32 * u);
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w[u].v, a[u][t].v, acc[t], 0, 0, 0);
  }
  // remaining steps of 32, the last one possibly short (K is a multiple of 8)
  for (; k < k_end; k += 32) {
    Pack8 w;
    const bool in = k + 8 * g < k_end;
    w.u4 = in ? *reinterpret_cast<const uint4*>(wp + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      Pack8 a;
      a.u4 = in ? *reinterpret_cast<const uint4*>(ap[t] + k) : make_uint4(0, 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w.v, a.v, acc[t], 0, 0, 0);
    }
  }
  // acc[t][j] = partial C[m = 16 t + r][n0 + 4 g + j]; add the waves' partials in wave order
  if (nwaves > 1) {
    if (wave != 0) {
#pragma unroll
      for (int t = 0; t < MT; ++t)
        *reinterpret_cast<float4*>(&red[wave - 1][t][lane * 4]) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int t = 0; t < MT; ++t)
      for (int w = 1; w < nwaves; ++w) {
        const float4 o = *reinterpret_cast<const float4*>(&red[w - 1][t][lane * 4]);
        acc[t][0] += o.x; acc[t][1] += o.y; acc[t][2] += o.z; acc[t][3] += o.w;
      }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int nn = n0 + 4 * g + j;
      if (nn < N) st_f32(C + (size_t)m * ldc + nn, acc[t][j] + (bias ? bias[nn] : 0.f));
    }
  }
}

extern "C" int ullm_gemm_skinny_supports(int M, int N, int K, int lda, int ldw) {
  return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && lda % 8 == 0 && ldw % 8 == 0;
}

extern "C" int ullm_gemm_skinny(const void* A, int lda, const void* W, int ldw, const float* bias, void* C,
                                int ldc, int M, int N, int K, int c_dtype, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ullm_gemm_skinny_supports(M, N, K, lda, ldw) || ldc < N) return ULLM_ERR_SHAPE;
  if (((uintptr_t)A & 15) || ((uintptr_t)W & 15)) return ULLM_ERR_SHAPE;
  const int tiles = (N + 15) / 16;
  // waves per block: enough blocks x waves to fill the chip, each wave with at least 128 values of K
  int waves = 1;
  while (waves < SK_MAX_WAVES && tiles * waves < 4096 && K / (waves * 2) >= 128) waves *= 2;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 31) / 32 * 32;
  const int mt = (M + 15) / 16;
  dim3 grid(tiles), block(64 * waves);
#define GO(MT, TC) hipLaunchKernelGGL((gemm_skinny_kernel<MT, TC>), grid, block, 0, stream, (const bf16_t*)A, lda, \
    (const bf16_t*)W, ldw, bias, (TC*)C, ldc, M, N, K, k_per_wave)
#define GO_MT(TC)                 \
  switch (mt) {                   \
    case 1: GO(1, TC); break;     \
    case 2: GO(2, TC); break;     \
    case 3: GO(3, TC); break;     \
    default: GO(4, TC); break;    \
  }
  if (c_dtype == ULLM_BF16) { GO_MT(bf16_t) }
  else if (c_dtype == ULLM_F32) { GO_MT(float) }
  else return ULLM_ERR_DTYPE;
#undef GO_MT
#undef GO
  ULLM_LAUNCH_CHECK();
}
