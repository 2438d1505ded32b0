// P[s][M, N] = X[M, K(s)] * W[N, K(s)]^T for 17 to 256 rows: partial sums over S slices of K, 32-bit.
//
// With this many rows a block that reads all of X for 16 rows of W (the few-rows kernel's shape)
// fetches more of X than of W.  Here the 8 waves of a block take 16 rows of W each and share the
// rows of X: a stage of 64 values of K of all rows of X goes through shared memory once per block
// (every thread fetches one 16-byte piece of it), the waves' own tiles of W through wave-private
// shared memory, both in whole 128-byte lines, two stages ahead in registers, one barrier a stage.
// No load stands under a condition, so the compiler waits for the stage it works on and not for the one
// on its way: a row of W past N reads the last row and a row of X past M row M - 1 (never stored), a piece
// past the end of K reads the row's last piece and the piece of X is replaced by zeros.
// So a block reads X once per 128 rows of W.  The matrices this is for (the output and down
// projections, 4096 to 8192 rows) then give 32 to 64 blocks, too few for the chip; K is therefore
// cut into S slices, one per blockIdx.y, and every slice stores its own partial sum.  Who adds the
// partial sums is the caller's business (the add + norm kernel takes a stack of them, in order, so
// the result does not depend on timing).  From 128 rows on the time is set by the shared-memory reads of X
// (one matrix instruction per 16-byte read), still well ahead of what the library picks for these shapes.
//
// A operand of v_mfma_f32_16x16x32_bf16 = a W tile (lane (r, g) holds W[n0 + r][k + 8g .. +8]), B
// operand = 16 rows of X.  Shared-memory rows are 128 bytes; piece c of row r lies at piece
// c ^ ((r >> 1) & 7), which keeps the 16-byte writes and reads of the hardware's lane groups on
// different banks.  Weights are [out, in] (ullm/layers/linear.py:165).
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack8 {
  bf16x8_t v;
  uint4 u4;
};

#define MID_WAVES 8
#define MID_MAX_SLICES 16

// MT = 16-row tiles of X (M <= 16 MT)
template <int MT>
__global__ void __launch_bounds__(64 * MID_WAVES)
gemm_partial_sums_kernel(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw,
                         float* __restrict__ P, int M, int N, int K, int k_per_slice) {
  constexpr int TILE = 16 * 128;                        // 16 rows x 64 values
  constexpr int XB = MT * TILE;                         // a stage of X
  __shared__ __attribute__((aligned(16))) unsigned char xs[2 * XB + 64 * 16];   // two stages, then a spare place per lane
  __shared__ __attribute__((aligned(16))) unsigned char ws[MID_WAVES * TILE];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int g = lane >> 4, r = lane & 15, lrow = lane >> 3, lcol = lane & 7;
  const int n0 = (blockIdx.x * MID_WAVES + wave) * 16;
  const int k_begin = blockIdx.y * k_per_slice;
  int k_end = k_begin + k_per_slice;
  if (k_end > K) k_end = K;
  // W: a lane fetches rows lrow and 8 + lrow of the wave's tile, piece lcol
  const bf16_t* wsrc[2];
  int put[2], get[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = 8 * h + lrow, n = n0 + row;
    put[h] = row * 128 + ((lcol ^ ((row >> 1) & 7)) << 4);
    get[h] = r * 128 + (((4 * h + g) ^ ((r >> 1) & 7)) << 4);       // h here: the step of 32 inside the stage
    wsrc[h] = W + (size_t)(n < N ? n : N - 1) * ldw;                // rows past N repeat the last row; never stored
  }
  // X: piece p = tid + 512 q of the stage is row p / 8, piece p % 8
  constexpr int XPIECES = MT * 16 * 8;
  constexpr int XQ = (XPIECES + 64 * MID_WAVES - 1) / (64 * MID_WAVES);
  // a thread whose piece lies past the stage reads piece 0 and stores to the spare place instead of skipping either
  // (a store of a loaded value under a condition would again wait for every load in flight)
  const bf16_t* xsrc[XQ];
  int xput[XQ], xstep[XQ];
  const int last_piece = K / 8 - 1, xcol = tid & 7;               // 64 MID_WAVES is a multiple of 8: the same for every q
#pragma unroll
  for (int q = 0; q < XQ; ++q) {
    const int p = tid + 64 * MID_WAVES * q;
    const bool ok = p < XPIECES;
    const int row = ok ? p >> 3 : 0;
    xsrc[q] = X + (size_t)(row < M ? row : M - 1) * ldx;
    xput[q] = ok ? (row >> 4) * TILE + (row & 15) * 128 + ((xcol ^ (((row & 15) >> 1) & 7)) << 4) : 2 * XB + 16 * lane;
    xstep[q] = ok ? XB : 0;
  }
  unsigned char* const mine = ws + wave * TILE;
  f32x4_t acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  struct Stage { uint4 w[2]; uint4 x[XQ]; };
  Stage st[2];
  auto fetch = [&](Stage& s, int k0) __attribute__((always_inline)) {
    const int wp = k0 / 8 + lcol, xp = k0 / 8 + xcol;
    const int wat = 8 * (wp < last_piece ? wp : last_piece), xat = 8 * (xp < last_piece ? xp : last_piece);
#pragma unroll
    for (int h = 0; h < 2; ++h) s.w[h] = ld_stream16(wsrc[h] + wat);
#pragma unroll
    for (int q = 0; q < XQ; ++q) s.x[q] = ld16(xsrc[q] + xat);
  };
  // One stage: the registers that hold stage s go to shared memory (stage s to the X buffer that was last read two
  // stages ago, before the previous barrier) and are refilled with stage s + 2 if the slice holds one; a barrier;
  // the products.
  auto stage = [&](Stage& sr, int s, bool more) __attribute__((always_inline)) {
    const int k0 = k_begin + 64 * s;
    unsigned char* xb = xs + (s & 1) * XB;
    const bool xin = k0 + 8 * xcol < k_end;                         // K is a multiple of 8
#pragma unroll
    for (int q = 0; q < XQ; ++q) st16(xs + xput[q] + (s & 1) * xstep[q], xin ? sr.x[q] : make_uint4(0, 0, 0, 0));
#pragma unroll
    for (int h = 0; h < 2; ++h) st16(mine + put[h], sr.w[h]);
    if (more) fetch(sr, k0 + 128);
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Pack8 wf, xf[MT];
      wf.u4 = *reinterpret_cast<const uint4*>(mine + get[j]);
#pragma unroll
      for (int t = 0; t < MT; ++t) xf[t].u4 = *reinterpret_cast<const uint4*>(xb + t * TILE + get[j]);
#pragma unroll
      for (int t = 0; t < MT; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf.v, xf[t].v, acc[t], 0, 0, 0);
    }
  };
  const int stages = k_begin < k_end ? (k_end - k_begin + 63) / 64 : 0;   // the same for every wave of the block
  fetch(st[0], k_begin);
  fetch(st[1], k_begin + 64);
  int s0 = 0;
  for (; s0 + 4 <= stages; s0 += 2) {                              // whole rounds whose fetches lie in the slice
    stage(st[0], s0, true);
    stage(st[1], s0 + 1, true);
  }
  for (; s0 < stages; s0 += 2) {
    stage(st[0], s0, s0 + 2 < stages);
    if (s0 + 1 < stages) stage(st[1], s0 + 1, s0 + 3 < stages);
  }
  // acc[t][j] = P[slice][m = 16 t + r][n0 + 4 g + j]
  float* out = P + (size_t)blockIdx.y * M * N;
  const int nn = n0 + 4 * g;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r;
    if (m < M && nn + 3 < N)
      *reinterpret_cast<float4*>(out + (size_t)m * N + nn) = make_float4(acc[t][0], acc[t][1], acc[t][2], acc[t][3]);
  }
}

// Slices of K for a matrix [N, K]: as many as give at most one block per compute unit (256 on this
// part), so that all blocks run side by side: one more slice, and the blocks left over for a second
// round cost half as much again.  Every slice is a multiple of 64 and at least 256 values long.  A
// function of the matrix alone, so that the order of the sums does not depend on the batch.
extern "C" int ullm_gemm_partial_sums_slices(int N, int K) {
  if (N <= 0 || K <= 0) return 0;
  const int blocks = (N + 16 * MID_WAVES - 1) / (16 * MID_WAVES);
  int s = 256 / blocks;
  if (s > MID_MAX_SLICES) s = MID_MAX_SLICES;
  while (s > 1 && K / s < 256) --s;
  return s < 1 ? 1 : s;
}

extern "C" int ullm_gemm_partial_sums_supports(int M, int N, int K, int ldx, int ldw) {
  return M >= 1 && M <= 256 && N >= 4 && N % 4 == 0 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

// X bfloat16 [M, K]; W bfloat16 [N, K]; P float32 [slices, M, N] with slices = ullm_gemm_partial_sums_slices(N, K).
extern "C" int ullm_gemm_partial_sums(const void* X, int ldx, const void* W, int ldw, float* P, int M, int N, int K,
                                      hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ullm_gemm_partial_sums_supports(M, N, K, ldx, ldw)) return ULLM_ERR_SHAPE;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15) || ((uintptr_t)P & 15)) return ULLM_ERR_SHAPE;
  const int slices = ullm_gemm_partial_sums_slices(N, K);
  int per = (K + slices - 1) / slices;
  per = (per + 63) / 64 * 64;
  dim3 grid((N + 16 * MID_WAVES - 1) / (16 * MID_WAVES), slices), block(64 * MID_WAVES);
#define GO(MT) hipLaunchKernelGGL((gemm_partial_sums_kernel<MT>), grid, block, 0, stream, (const bf16_t*)X, ldx, \
    (const bf16_t*)W, ldw, P, M, N, K, per)
  if (M <= 16) GO(1);
  else if (M <= 32) GO(2);
  else if (M <= 48) GO(3);
  else if (M <= 64) GO(4);
  else if (M <= 96) GO(6);
  else if (M <= 128) GO(8);
  else if (M <= 192) GO(12);
  else GO(16);
#undef GO
  ULLM_LAUNCH_CHECK();
}
