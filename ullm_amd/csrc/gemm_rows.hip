// C[M, N] = X[M, K] * W[N, K]^T for 17 to 128 rows, bfloat16 in and out, 32-bit accumulation, with what
// follows the product folded in:
//   STORE : C = result (+ bias)
//   SILU  : W is the stacked gate|up matrix [2 N, K]; C[M, N] = silu(gate) * up on the 32-bit sums
//           (ullm/layers/activation.py:16-18 after gate_up_proj, ullm/models/qwen3.py:43-45)
//
// At these row counts the product is still a read of W from HBM, once, and its time is set by how many
// bytes of W the chip keeps on their way.  So the matrix is cut into as many blocks as there are compute
// units (a block's columns need not be a multiple of 16: the last tile of a wave is used in part), and a
// wave keeps four to six stages of 64 values of K of its tiles of W in flight in registers.  The rows of X
// are shared: a stage of X goes through shared memory once per block and every wave reads its operand
// from there.  A result column is summed by one wave in the order of K, so it does not depend on timing
// or on the batch.
//
// A norm handed ahead by the product before (RowSquares): X is then the stream times the norm's gain in
// bfloat16, and the 32-bit results of row m are scaled by rsqrt(sum of the parts' squares of row m / K + eps)
// before the epilogue (ullm/layers/layernorm.py:28-33 with the scale taken out of the product).  The parts are
// added in a fixed order: a lane's parts in turn, the four lanes of a row, the waves.
//
// A operand of v_mfma_f32_16x16x32_bf16 = a W tile (lane (r, g) holds W[n0 + r][k + 8g .. +8]), B
// operand = 16 rows of X; W tiles reach that layout through the wave's own part of shared memory (a
// wave fetches whole 128-byte lines, 8 rows per instruction).  Shared-memory rows are 128 bytes; piece
// c of row r lies at piece c ^ ((r >> 1) & 7), which keeps the 16-byte writes and reads of the
// hardware's lane groups on different banks.  Weights are [out, in] (ullm/layers/linear.py:165).
#include "common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack8 {
  bf16x8_t v;
  uint4 u4;
};

enum { ROWS_STORE = 0, ROWS_SILU = 1 };

// Sums of squares left by the product before (sq == nullptr: none): sq[m][0 .. 4 quads), row stride 4 quads,
// 16-byte aligned
struct RowSquares {
  const float* sq;
  int quads;
  float eps;
};

#define ROWS_SQ_HELD 8   // groups of four partial sums of squares a lane fetches before the product starts

// f(0), f(1), .. f(N - 1) with the index a constant of the language, not of the optimiser: registers that
// hold stages in flight are then never indexed by a variable, and so never end up in scratch memory
template <int I, int N, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}

#define ROWS_MAX_WAVES 8   // waves of a block (512 threads: two waves a SIMD, 256 registers each)
#define ROWS_MAX_TILES 8   // 16-row tiles of X: 128 rows

// Stages of W and of X a wave has in flight (of X as many as of W: loads complete in order, so waiting for a stage
// of X waits for every load issued before it, and a stage of X fetched later than a stage of W would cut short
// what W has in flight).  As many as about 150 registers hold: ntw tiles of W (two 16-byte pieces each) and xq
// pieces of X per stage; from five tiles of rows on, as many as the sums (4 ntw mt registers), the operands of a
// step (4 (ntw + mt)) and 64 more leave of the 256, and two stages at least.
__host__ __device__ constexpr int rows_depth(int ntw, int xq, int mt) {
  const int stage = (2 * ntw + xq) * 4;
  if (mt > 4) {
    const int d = (256 - 4 * ntw * mt - 4 * (ntw + mt) - 64) / stage;
    return d < 2 ? 2 : (d > 8 ? 8 : d);
  }
  const int d = 150 / stage;
  return d < 3 ? 3 : (d > 8 ? 8 : d);
}

// MT = 16-row tiles of X (M <= 16 MT); XQ = 16-byte pieces of a stage of X per thread (MT * 128 pieces over the
// block's threads).  Wave wn of a block's WN owns columns n0 .. n0 + cols_per_wave of the block's cols_per_block.
template <int MT, int XQ, int EPI>
__global__ void __launch_bounds__(64 * ROWS_MAX_WAVES)
gemm_rows_kernel(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw,
                 const float* __restrict__ bias, bf16_t* __restrict__ C, int ldc, int M, int N, int K,
                 int WN, int cols_per_wave, int cols_per_block, RowSquares before) {
  constexpr int NTW = EPI == ROWS_SILU ? 2 : 1;         // tiles of W per wave: gate and up rows of the same columns
  constexpr int D = rows_depth(NTW, XQ, MT);
  constexpr int TILE = 16 * 128;                        // 16 rows x 64 values
  constexpr int XB = MT * TILE;                         // a stage of X
  __shared__ __attribute__((aligned(16))) unsigned char xs[2 * XB + 64 * 16];   // two stages, then a spare place per lane
  __shared__ __attribute__((aligned(16))) unsigned char ws[ROWS_MAX_WAVES * NTW * TILE];
  __shared__ float sqs[ROWS_MAX_WAVES][16];
  const int tid = threadIdx.x, lane = tid & 63, wn = tid >> 6;
  const int g = lane >> 4, r = lane & 15, lrow = lane >> 3, lcol = lane & 7;
  // The sums of squares the product before left (one tile of rows): lane (r, g) of wave wn adds groups 4 wn + g,
  // + 4 WN, ... of row r, the four lanes of a row add theirs, the waves' sums meet in `sqs`.  The loads go out
  // before the first stages' (unconditional, with the index held in range) and are added while those are on
  // their way, so nothing waits for them.
  const bool scaled = MT == 1 && before.sq != nullptr;
  const int sq_step = 4 * WN, sq_first = 4 * wn + g;
  float4 held[ROWS_SQ_HELD];
  const float* const sq_row = before.sq + (size_t)(r < M ? r : M - 1) * 4 * before.quads;
  if (scaled) {
#pragma unroll
    for (int i = 0; i < ROWS_SQ_HELD; ++i) {
      const int j = sq_first + i * sq_step;
      held[i] = *reinterpret_cast<const float4*>(sq_row + 4 * (j < before.quads ? j : before.quads - 1));
    }
  }
  const int block_n0 = blockIdx.x * cols_per_block;
  const int block_end = block_n0 + cols_per_block < N ? block_n0 + cols_per_block : N;
  const int n0 = block_n0 + wn * cols_per_wave;
  const int n_end = n0 + cols_per_wave < block_end ? n0 + cols_per_wave : block_end;   // may lie below n0: a wave without columns
  // W: a lane fetches rows lrow and 8 + lrow of each of the wave's tiles, piece lcol.  No load stands
  // under a condition and no loaded value under a select (either makes the compiler wait for every load
  // in flight at the next use, which would undo the stages in flight).  Nothing needs one: a row of W
  // past the wave's columns reads the wave's last row again (a line the same instruction fetches anyway)
  // and only feeds result columns that are never stored; a row of X past M reads row 0 and only feeds
  // result rows that are never stored; K is a whole number of stages, so no stage has a tail; and the
  // stages fetched past the end of the loop read the matrix's last stage again and are not used.
  const bf16_t* wsrc[NTW][2];
  int put[2], get[2];
  const int last_col = n_end > n0 ? n_end - 1 : 0;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = 8 * h + lrow, col = n0 + row;
    put[h] = row * 128 + ((lcol ^ ((row >> 1) & 7)) << 4);
    get[h] = r * 128 + (((4 * h + g) ^ ((r >> 1) & 7)) << 4);       // h here: the step of 32 inside the stage
#pragma unroll
    for (int i = 0; i < NTW; ++i)
      wsrc[i][h] = W + ((size_t)(col < n_end ? col : last_col) + (size_t)i * N) * ldw + 8 * lcol;
  }
  // X: piece p = tid + 64 WN q of the stage is row p / 8, piece p % 8.  Where the piece goes in shared
  // memory: xput + (stage & 1) * xstep.  A thread whose piece lies past the stage reads piece 0 and stores
  // to a spare place instead of skipping either (a store of a loaded value under a condition would again
  // wait for every load in flight).
  const bf16_t* xsrc[XQ];
  int xput[XQ], xstep[XQ];
#pragma unroll
  for (int q = 0; q < XQ; ++q) {
    const int p = tid + 64 * WN * q;
    const bool ok = p < MT * 128;
    const int row = ok ? p >> 3 : 0, col = ok ? p & 7 : 0;
    xsrc[q] = X + (size_t)(row < M ? row : 0) * ldx + 8 * col;
    xput[q] = ok ? (row >> 4) * TILE + (row & 15) * 128 + ((col ^ (((row & 15) >> 1) & 7)) << 4) : 2 * XB + 16 * lane;
    xstep[q] = ok ? XB : 0;
  }
  unsigned char* const mine = ws + wn * NTW * TILE;
  f32x4_t acc[NTW][MT];
#pragma unroll
  for (int i = 0; i < NTW; ++i)
#pragma unroll
    for (int t = 0; t < MT; ++t) acc[i][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  struct Stage { uint4 w[NTW][2], x[XQ]; };
  const int k_last = K - 64;                                        // first value of the matrix's last stage
  auto fetch = [&](Stage& s, int k0) __attribute__((always_inline)) {
    const int k = k0 < k_last ? k0 : k_last;
    static_for<0, NTW>([&](auto i) {
      static_for<0, 2>([&](auto h) { s.w[i][h] = ld_stream16(wsrc[i][h] + k); });
    });
    static_for<0, XQ>([&](auto q) { s.x[q] = ld16(xsrc[q] + k); });
  };
  // One stage: the registers that hold stage s go to shared memory and are refilled with the stage that
  // will need them next; a barrier; the products.  Stage s goes to the X buffer that was last read two
  // stages ago, before the previous barrier.
  auto stage = [&](Stage& st, int s) __attribute__((always_inline)) {
    unsigned char* xb = xs + (s & 1) * XB;
    static_for<0, XQ>([&](auto q) { st16(xs + xput[q] + (s & 1) * xstep[q], st.x[q]); });
    static_for<0, NTW>([&](auto i) {
      static_for<0, 2>([&](auto h) { st16(mine + i * TILE + put[h], st.w[i][h]); });
    });
    fetch(st, 64 * (s + D));
    __syncthreads();
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Pack8 wf[NTW], xf[MT];
#pragma unroll
      for (int i = 0; i < NTW; ++i) wf[i].u4 = *reinterpret_cast<const uint4*>(mine + i * TILE + get[j]);
#pragma unroll
      for (int t = 0; t < MT; ++t) xf[t].u4 = *reinterpret_cast<const uint4*>(xb + t * TILE + get[j]);
#pragma unroll
      for (int i = 0; i < NTW; ++i)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, xf[t].v, acc[i][t], 0, 0, 0);
    }
  };
  // D stages in flight: registers st[d] hold the stages s = d (mod D)
  Stage st[D];
  const int stages = K / 64;
  static_for<0, D>([&](auto d) { fetch(st[d], 64 * d); });
  if (scaled) {
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < ROWS_SQ_HELD; ++i) {
      const float4 v = held[i];
      q += sq_first + i * sq_step < before.quads ? (v.x + v.y) + (v.z + v.w) : 0.f;
    }
    for (int j = sq_first + ROWS_SQ_HELD * sq_step; j < before.quads; j += sq_step) {
      const float4 v = *reinterpret_cast<const float4*>(sq_row + 4 * j);
      q += (v.x + v.y) + (v.z + v.w);
    }
    q += __shfl_xor(q, 16);
    q += __shfl_xor(q, 32);
    if (g == 0) sqs[wn][r] = q;             // read after the barriers of the stages
  }
  int s = 0;
  for (; s + D <= stages; s += D) static_for<0, D>([&](auto d) { stage(st[d], s + d); });
  static_for<0, D - 1>([&](auto d) {
    if (s + d < stages) stage(st[d], s + d);
  });
  if (scaled) {
    float total = 0.f;
    for (int w = 0; w < WN; ++w) total += sqs[w][r];
    const float rs = rsqrtf(total / (float)K + before.eps);
#pragma unroll
    for (int i = 0; i < NTW; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][0][j] *= rs;
  }
  // acc[i][t][j] = sum for row m = 16 t + r, column n0 + 4 g + j (of half i of the stacked matrix)
  const int nn = n0 + 4 * g;
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r;
    if (m >= M || nn >= n_end) continue;
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (EPI == ROWS_SILU) v[j] = fast_silu(acc[0][t][j]) * acc[NTW - 1][t][j];
      else v[j] = acc[0][t][j] + (bias && nn + j < n_end ? bias[nn + j] : 0.f);
    }
    bf16_t* cp = C + (size_t)m * ldc + nn;
    if (nn + 3 < n_end) {
      *reinterpret_cast<uint2*>(cp) = make_uint2(pack2_bf16(v[0], v[1]), pack2_bf16(v[2], v[3]));
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (nn + j < n_end) cp[j] = f32_to_bf16_bits(v[j]);
    }
  }
}

static int rows_compute_units() {
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

// 16-row tiles of X that the kernel is compiled for: 1 to 6, then 8
static int rows_tiles(int M) {
  const int mt = (M + 15) / 16;
  return mt <= 6 ? mt : ROWS_MAX_TILES;
}

struct RowsShape {
  int cols_per_block, cols_per_wave, wn, xq, blocks;
};

// How a matrix of N result columns is cut: a whole number of rounds of one block per compute unit, and
// the block's columns over its waves in steps of 4 (at most 16 per wave).  A function of the matrix, the
// epilogue and the number of 16-row tiles of X alone.
static bool rows_shape(int N, int mt, int epi, int units, RowsShape* s) {
  const int rounds = (N + units * 16 * ROWS_MAX_WAVES - 1) / (units * 16 * ROWS_MAX_WAVES);
  int cpb = (N + rounds * units - 1) / (rounds * units);
  cpb = (cpb + 3) / 4 * 4;
  if (cpb < 8) cpb = 8;
  int wn = (cpb + 15) / 16;
  if (wn < 2) wn = 2;                                   // at least two waves: a wave alone hides no latency of the other's products
  if (wn > ROWS_MAX_WAVES) return false;
  int cpw = (cpb + wn - 1) / wn;
  cpw = (cpw + 3) / 4 * 4;
  s->cols_per_block = cpb;
  s->cols_per_wave = cpw;
  s->wn = wn;
  s->xq = (mt * 128 + 64 * wn - 1) / (64 * wn);
  s->blocks = (N + cpb - 1) / cpb;
  // 128 rows of X over the 128 threads of two waves, with two tiles of W per wave: more registers than a lane has
  if (epi == ROWS_SILU && mt == ROWS_MAX_TILES && s->xq > 6) return false;
  return true;
}

// What a launch takes, and the kernel picked step by step: only the combinations that rows_shape can give are
// compiled (a thread never has more pieces of a stage of X than there are tiles of rows).
struct RowsLaunch {
  const bf16_t* X; int ldx;
  const bf16_t* W; int ldw;
  const float* bias;
  bf16_t* C; int ldc;
  int M, N, K;
  RowsShape s;
  RowSquares before;
  hipStream_t stream;
};

template <int MT, int XQ, int EPI>
static void rows_pick_pieces(const RowsLaunch& a) {
  if constexpr (XQ >= MT) {
    hipLaunchKernelGGL((gemm_rows_kernel<MT, XQ, EPI>), dim3(a.s.blocks), dim3(64 * a.s.wn), 0, a.stream, a.X, a.ldx, a.W,
                       a.ldw, a.bias, a.C, a.ldc, a.M, a.N, a.K, a.s.wn, a.s.cols_per_wave, a.s.cols_per_block, a.before);
  } else {
    if (a.s.xq <= XQ)
      hipLaunchKernelGGL((gemm_rows_kernel<MT, XQ, EPI>), dim3(a.s.blocks), dim3(64 * a.s.wn), 0, a.stream, a.X, a.ldx,
                         a.W, a.ldw, a.bias, a.C, a.ldc, a.M, a.N, a.K, a.s.wn, a.s.cols_per_wave, a.s.cols_per_block,
                         a.before);
    else rows_pick_pieces<MT, XQ + 1, EPI>(a);
  }
}

// tiles of rows: 1 to 6, then 8 (the row counts that steps are padded to: 16 .. 96, 128)
template <int EPI>
static void rows_pick_tiles(const RowsLaunch& a, int mt) {
  if (mt == 1) rows_pick_pieces<1, 1, EPI>(a);
  else if (mt == 2) rows_pick_pieces<2, 1, EPI>(a);
  else if (mt == 3) rows_pick_pieces<3, 1, EPI>(a);
  else if (mt == 4) rows_pick_pieces<4, 1, EPI>(a);
  else if (mt == 5) rows_pick_pieces<5, 1, EPI>(a);
  else if (mt == 6) rows_pick_pieces<6, 1, EPI>(a);
  else rows_pick_pieces<8, 1, EPI>(a);
}

// N: columns of the result (with epi 1 the weights have 2 N rows)
extern "C" int ullm_gemm_rows_supports(int M, int N, int K, int ldx, int ldw, int ldc, int epi) {
  RowsShape s;
  return M >= 1 && M <= 16 * ROWS_MAX_TILES && N >= 4 && K >= 64 && K % 64 == 0 && ldx % 8 == 0 && ldw % 8 == 0 && ldc % 4 == 0 &&
         ldc >= N && (epi == ROWS_STORE || epi == ROWS_SILU) && rows_shape(N, rows_tiles(M), epi, rows_compute_units(), &s);
}

// X bfloat16 [M <= 128, K], K a multiple of 64; W bfloat16 [N, K] (epi 1: [2 N, K], gate rows then up rows);
// C bfloat16 [M, N] with row stride ldc; bias float32 [N] or null (epi 0 only).
// With row_sq (float32 [M <= 16, sq_parts], sq_parts a multiple of 4): the results of row m are scaled by
// rsqrt(sum of row_sq[m][.] / K + eps) before the epilogue.
extern "C" int ullm_gemm_rows(const void* X, int ldx, const void* W, int ldw, const float* bias, void* C, int ldc,
                              int M, int N, int K, int epi, const float* row_sq, int sq_parts, float eps,
                              hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ullm_gemm_rows_supports(M, N, K, ldx, ldw, ldc, epi)) return ULLM_ERR_SHAPE;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15) || ((uintptr_t)C & 7)) return ULLM_ERR_SHAPE;
  if (epi == ROWS_SILU && bias) return ULLM_ERR_UNSUPPORTED;
  if (row_sq && (M > 16 || sq_parts < 4 || sq_parts % 4 || ((uintptr_t)row_sq & 15))) return ULLM_ERR_UNSUPPORTED;
  const RowSquares before{row_sq, sq_parts / 4, eps};
  const int mt = rows_tiles(M);
  RowsShape s;
  rows_shape(N, mt, epi, rows_compute_units(), &s);
  const RowsLaunch go{(const bf16_t*)X, ldx, (const bf16_t*)W, ldw, bias, (bf16_t*)C, ldc, M, N, K, s, before, stream};
  if (epi == ROWS_SILU) rows_pick_tiles<ROWS_SILU>(go, mt);
  else rows_pick_tiles<ROWS_STORE>(go, mt);
  ULLM_LAUNCH_CHECK();
}
