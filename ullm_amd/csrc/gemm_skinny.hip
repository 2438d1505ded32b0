// C[M, N] = X[M, K] * W[N, K]^T for few rows (M <= 64), bfloat16 weights streamed once from HBM through
// the matrix cores, 32-bit accumulation.  This is the decode-time matrix product: its time is the time
// to read W, so the kernel is built around the weight loads, and the small row-wise operations that
// surround a projection in a decoder layer are folded into it so that they cost no launch and no
// pass over memory of their own:
//
//   what happens to the result (EPI)
//     STORE : C = result (+ bias), bfloat16 or float32
//     RESADD: R[M, N] += result, the 32-bit residual stream (the add the reference leaves to the next
//             norm, ullm/layers/layernorm.py:24-26)
//     SILU  : W is the stacked gate|up matrix [2 I, K]; a block takes rows n of the gate half and the same
//             rows of the up half and stores C[M, I] = silu(gate) * up, computed on the 32-bit sums
//             (ullm/layers/activation.py:16-18 after gate_up_proj, ullm/models/qwen3.py:43-45)
//
// A block owns NT x 16 consecutive rows of W; its waves split K between them.  The A operand of
// v_mfma_f32_16x16x32_bf16 is a W tile (lane (r, g) holds W[n0 + r][k + 8g .. +8]), the B operand 16
// rows of X (lane (m, g) holds X[m][k + 8g .. +8]); both reach the registers through the wave's own
// part of shared memory.  The waves' partial results are added in wave order through shared memory,
// so the result does not depend on timing.
// Weights are [out, in] (ullm/layers/linear.py:165).
//
//   what comes before it (NORMX)
//     the RMS norm of the 32-bit residual stream (ullm/layers/layernorm.py:28-33): X is then the stream
//     itself, float32 [M, K].  The kernel reads every row of X in full anyway, so it multiplies by the
//     gain and rounds to bfloat16 on the way into shared memory, adds up the squares beside that, and
//     multiplies the finished sums by rsqrt(mean of squares + eps): y = rs * ((x * gain) W^T).  Against
//     a norm kernel of its own this saves a launch and a pass, which at these sizes is all latency.
//
//   a norm handed from one product to the next (NormAhead, RowSquares)
//     A product that ends in the stream (RESADD) owns the final values of its columns.  Given the gain of
//     the norm that comes next it also stores x * gain rounded to bfloat16 and, per block, the sum of the
//     squares of its columns of every row.  The next product then takes those bfloat16 rows as its X, adds
//     up the blocks' sums and scales its 32-bit results by rsqrt(mean of squares + eps): the same
//     arithmetic as NORMX, without a norm kernel between the two and without 32-bit rows of X in the
//     second.  The sums are added in a fixed order (a lane's blocks in turn, lanes, waves).
#include "common.h"
#include <type_traits>

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack8 {
  bf16x8_t v;
  uint4 u4;
  uint32_t w[4];
  bf16_t h[8];
};

enum { EPI_STORE = 0, EPI_RESADD = 1, EPI_SILU = 2 };

// What a RESADD product leaves for the norm that follows it (gain == nullptr: nothing): x[m][n] = stream * gain
// in bfloat16 (row stride ldx), sq[m][block] = the block's sum of squares of row m of the stream (row stride
// ld_sq, a multiple of 4; the last block clears the entries from the number of blocks to ld_sq).
struct NormAhead {
  const float* gain;
  bf16_t* x;
  float* sq;
  int ldx, ld_sq;
};

// Sums of squares left by the product before (sq == nullptr: none): sq[m][0 .. 4 quads), row stride 4 quads,
// 16-byte aligned; the results of row m are scaled by rsqrt(sum of the row / K + eps).
struct RowSquares {
  const float* sq;
  int quads;
};


// Most waves per block for a tile shape,
// bounded by the shared memory that holds a stage per wave (and later the waves' partials): at most 8
// waves, so that several blocks fit a compute unit
__host__ __device__ constexpr int sk_max_waves(int mt, int nt) { return mt * nt >= 8 ? 4 : 8; }

// The waves' partial results of a block are added in wave order through `red` and the sum goes where
// EPI says.  acc[i][t][j] = partial C[m = 16 t + r][n0 + 16 i + 4 g + j].
// With `scaled`, sq[w][m] holds wave w's sum of squares of row m of X (or its share of the sums the product
// before left) and the sums are scaled by rsqrt(their total / K + eps) first.
template <int MT, int NT, int EPI, typename TC, typename RedT>
__device__ __forceinline__ void skinny_finish(f32x4_t (&acc)[NT][MT], RedT& red, const float* __restrict__ bias,
                                              TC* __restrict__ C, float* __restrict__ R, int ldc, int M, int N, int n0,
                                              bool scaled, const float (*sq)[16 * MT], int K, float eps,
                                              const NormAhead& ahead) {
  constexpr int OT = EPI == EPI_SILU ? NT / 2 : NT;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
  const int g = lane >> 4, r = lane & 15;
  if (nwaves > 1) {
    if (wave != 0) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          *reinterpret_cast<float4*>(&red[wave - 1][i * MT + t][lane * 4]) =
              make_float4(acc[i][t][0], acc[i][t][1], acc[i][t][2], acc[i][t][3]);
    }
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int i = 0; i < NT; ++i)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        for (int w = 1; w < nwaves; ++w) {
          const float4 o = *reinterpret_cast<const float4*>(&red[w - 1][i * MT + t][lane * 4]);
          acc[i][t][0] += o.x; acc[i][t][1] += o.y; acc[i][t][2] += o.z; acc[i][t][3] += o.w;
        }
  }
  if (scaled) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float total = 0.f;
      for (int w = 0; w < nwaves; ++w) total += sq[w][16 * t + r];
      const float rs = rsqrtf(total / (float)K + eps);
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][t][j] *= rs;
    }
  }
  if (EPI == EPI_RESADD && ahead.gain) {
    // the stream's new values, the same times the next norm's gain in bfloat16, and the block's share of
    // the rows' sums of squares: a lane's columns in turn, then the four lanes of a row
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = 16 * t + r;
      float q = 0.f;
      if (m < M) {
#pragma unroll
        for (int i = 0; i < OT; ++i) {
          const int nn = n0 + 16 * i + 4 * g;
          float* rp = R + (size_t)m * ldc + nn;
          bf16_t* xp = ahead.x + (size_t)m * ahead.ldx + nn;
          if (nn + 3 < N) {
            float4 o = *reinterpret_cast<float4*>(rp);
            const float4 gn = *reinterpret_cast<const float4*>(ahead.gain + nn);
            o.x += acc[i][t][0]; o.y += acc[i][t][1]; o.z += acc[i][t][2]; o.w += acc[i][t][3];
            *reinterpret_cast<float4*>(rp) = o;
            *reinterpret_cast<uint2*>(xp) = make_uint2(pack2_bf16(o.x * gn.x, o.y * gn.y), pack2_bf16(o.z * gn.z, o.w * gn.w));
            q = fmaf(o.x, o.x, q); q = fmaf(o.y, o.y, q); q = fmaf(o.z, o.z, q); q = fmaf(o.w, o.w, q);
          } else {
#pragma unroll
            for (int j = 0; j < 4; ++j)
              if (nn + j < N) {
                const float o = rp[j] + acc[i][t][j];
                rp[j] = o;
                xp[j] = f32_to_bf16_bits(o * ahead.gain[nn + j]);
                q = fmaf(o, o, q);
              }
          }
        }
      }
      q += __shfl_xor(q, 16);
      q += __shfl_xor(q, 32);
      if (g == 0 && m < M) {
        ahead.sq[(size_t)m * ahead.ld_sq + blockIdx.x] = q;
        if (blockIdx.x == gridDim.x - 1)
          for (int b = gridDim.x; b < ahead.ld_sq; ++b) ahead.sq[(size_t)m * ahead.ld_sq + b] = 0.f;
      }
    }
    return;
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = 16 * t + r;
    if (m >= M) continue;
#pragma unroll
    for (int i = 0; i < OT; ++i) {
      const int nn = n0 + 16 * i + 4 * g;
      if (EPI == EPI_SILU) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (nn + j < N) st_f32(C + (size_t)m * ldc + nn + j, fast_silu(acc[i][t][j]) * acc[i + OT][t][j]);
      } else if (EPI == EPI_RESADD) {
        float* rp = R + (size_t)m * ldc + nn;
        if (nn + 3 < N) {
          float4 o = *reinterpret_cast<float4*>(rp);
          o.x += acc[i][t][0]; o.y += acc[i][t][1]; o.z += acc[i][t][2]; o.w += acc[i][t][3];
          *reinterpret_cast<float4*>(rp) = o;
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (nn + j < N) rp[j] += acc[i][t][j];
        }
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j)
          if (nn + j < N) st_f32(C + (size_t)m * ldc + nn + j, acc[i][t][j] + (bias ? bias[nn + j] : 0.f));
      }
    }
  }
}

// MT = 16-row tiles of X (M <= 16 MT); NT = 16-row tiles of W per block.
// With EPI_SILU the NT tiles of W are NT / 2 of the gate half followed by the same rows of the up half.
// A wave fetches whole 128-byte lines, 8 rows per instruction (lane = row l / 8, 16-byte piece l % 8),
// two stages of 64 values of K ahead in registers, writes a stage to its own part of shared memory and
// reads the operands from there in the layout the matrix instruction wants (lane (r, g) holds row r,
// values 8 g .. +8 of a step of 32).  A row takes 128 bytes; piece c of row r lies at piece
// c ^ ((r >> 1) & 7), which keeps both the 16-byte writes and the 16-byte reads of the hardware's lane
// groups on different banks.  No barrier in the loop: a wave only reads what it wrote.
// (Loading the operands straight from memory in the matrix layout, 64 bytes of each of 16 rows per
// instruction and of X as many rows as the batch has, was slower the more rows X had.)
// The stages in flight are real: every load is issued without a condition, so the compiler waits for exactly the
// stage it works on while the next is on its way (with loads under conditions it waited for all of them; the
// output and down projections of few columns, one block a compute unit, then ran 0.8 to 2 us slower, gate|up
// at 9 to 16 rows 6 us).  Three stages in flight cost a wave per SIMD and bring nothing.
// NORMX: X is float32 and gain [K] float32, see above; else X is bfloat16.
// XH: 8-row halves of a tile of X that are fetched: 1 for M <= 8 (then MT = 1), where the other half
// stays zero in shared memory and costs neither loads nor the registers that hold them in flight
// (with NORMX 75 against 116 registers, that is 6 against 4 waves per SIMD).
#ifndef SK_DEPTH
#define SK_DEPTH 2
#endif

template <int MT, int NT, int EPI, typename TC, bool NORMX, int XH>
__global__ void __launch_bounds__(64 * sk_max_waves(MT, NT))
gemm_skinny_kernel(const void* __restrict__ Xv, int ldx, const bf16_t* __restrict__ W, int ldw,
                   const float* __restrict__ bias, const float* __restrict__ gain, float eps, TC* __restrict__ C,
                   float* __restrict__ R, int ldc, int M, int N, int K, int k_per_wave, int rows_per_block,
                   NormAhead ahead, RowSquares before) {
  constexpr int MAXW = sk_max_waves(MT, NT);
  constexpr int TILE_BYTES = 16 * 128, STAGE_BYTES = (NT + MT) * TILE_BYTES;
  constexpr int RED_BYTES = (MAXW - 1) * NT * MT * 256 * 4;
  constexpr int LDS_BYTES = MAXW * STAGE_BYTES > RED_BYTES ? MAXW * STAGE_BYTES : RED_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];
  __shared__ float sq[MAXW][16 * MT];
  using XT = typename std::conditional<NORMX, float, bf16_t>::type;
  constexpr int XV = NORMX ? 2 : 1;                       // 16-byte loads per 8 values of X
  const XT* const X = reinterpret_cast<const XT*>(Xv);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, r = lane & 15, lrow = lane >> 3, lcol = lane & 7;
  constexpr int OT = EPI == EPI_SILU ? NT / 2 : NT;
  // a block's columns of the result: rows_per_block <= 16 OT of them (the host picks the number that spreads
  // the matrix evenly over the compute units); rows of W past them are not stored
  const int n0 = blockIdx.x * rows_per_block;
  const int n_end = n0 + rows_per_block < N ? n0 + rows_per_block : N;
  // No load stands under a condition (a load under one makes the compiler wait for every load in flight at
  // the next use of any, which would undo the stages in flight).  Nothing needs one: a row of W past the block's
  // columns reads the block's last row again and only feeds result columns that are never stored; a row of X past M
  // reads row M - 1 and only feeds result rows that are never stored; a piece past the end of K reads the row's last
  // piece again, and the piece of X is then replaced by zeros on its way into shared memory.
  const bf16_t* wsrc[NT][2];
  static_assert(XH == 2 || MT == 1, "half a tile of X only where it is the only tile");
  const XT* xsrc[MT][XH];
  int put[2], get[2];
  const int last_piece = K / 8 - 1;
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = 8 * h + lrow;
    put[h] = row * 128 + ((lcol ^ ((row >> 1) & 7)) << 4);
    get[h] = r * 128 + (((4 * h + g) ^ ((r >> 1) & 7)) << 4);      // h here: the step of 32 inside the stage
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int col = n0 + 16 * (i % OT) + row;
      const int n = (col < n_end ? col : n_end - 1) + (i / OT) * N;
      wsrc[i][h] = W + (size_t)n * ldw;
    }
    if (h < XH) {
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        xsrc[t][h] = X + (size_t)(16 * t + row < M ? 16 * t + row : M - 1) * ldx;
      }
    }
  }
  // The sums of squares the product before left: the lanes of a wave that share a row (8 of them where the
  // batch has up to 8 rows, else 4) take groups of four sums in turn, add theirs, and the waves' sums meet in `sq`.
  // The loads go out before the first stage's (unconditional, with the index held in range) and are added while
  // that stage is on its way, so nothing waits for them.
  constexpr bool SQUARES = !NORMX && EPI != EPI_RESADD && MT == 1;      // one tile of rows: what a norm handed ahead covers
  constexpr int SQ_LANES = XH == 1 ? 8 : 4, SQ_HELD = XH == 1 ? 1 : 2;
  const bool scaled = NORMX || (SQUARES && before.sq != nullptr);
  const int sq_row = lane & (64 / SQ_LANES - 1), sq_step = SQ_LANES * (blockDim.x >> 6),
            sq_first = SQ_LANES * wave + lane / (64 / SQ_LANES);
  const float* const sq_src = before.sq + (size_t)(sq_row < M ? sq_row : M - 1) * 4 * before.quads;
  float4 held[SQ_HELD];
  if (SQUARES && before.sq) {
#pragma unroll
    for (int i = 0; i < SQ_HELD; ++i) {
      const int j = sq_first + i * sq_step;
      held[i] = *reinterpret_cast<const float4*>(sq_src + 4 * (j < before.quads ? j : before.quads - 1));
    }
  }
  unsigned char* const mine = lds + wave * STAGE_BYTES;
  if (XH == 1) *reinterpret_cast<uint4*>(mine + NT * TILE_BYTES + put[1]) = make_uint4(0, 0, 0, 0);
  f32x4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[i][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int k_begin = wave * k_per_wave;
  int k_end = k_begin + k_per_wave;
  if (k_end > K) k_end = K;
  struct Stage { uint4 w[NT][2], x[MT][XH][XV], gm[XV]; };
  float ss[MT][XH];                                        // squares of rows 16 t + 8 h + lrow, this lane's pieces
#pragma unroll
  for (int t = 0; t < MT; ++t) ss[t][0] = ss[t][XH - 1] = 0.f;
  constexpr int DEPTH = SK_DEPTH;                         // stages of 64 values of K on their way
  Stage st[DEPTH];
  auto fetch = [&](Stage& st, int k0) __attribute__((always_inline)) {
    const int piece = k0 / 8 + lcol, at = 8 * (piece < last_piece ? piece : last_piece);
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < NT; ++i) st.w[i][h] = ld_stream16(wsrc[i][h] + at);
      if (h < XH) {
#pragma unroll
        for (int t = 0; t < MT; ++t)
#pragma unroll
          for (int v = 0; v < XV; ++v) st.x[t][h][v] = ld16(xsrc[t][h] + at + 4 * v);
      }
    }
    if (NORMX) {
#pragma unroll
      for (int v = 0; v < XV; ++v) st.gm[v] = ld16(gain + at + 4 * v);
    }
  };
  auto work = [&](const Stage& st, int k0) __attribute__((always_inline)) {
    const bool in = k0 + 8 * lcol < k_end;                        // K is a multiple of 8
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < NT; ++i) *reinterpret_cast<uint4*>(mine + i * TILE_BYTES + put[h]) = st.w[i][h];
      if (h >= XH) continue;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        uint4 piece;
        if constexpr (NORMX) {
          const float4 a = __builtin_bit_cast(float4, st.x[t][h][0]), b = __builtin_bit_cast(float4, st.x[t][h][XV - 1]);
          const float4 ga = __builtin_bit_cast(float4, st.gm[0]), gb = __builtin_bit_cast(float4, st.gm[XV - 1]);
          float q = ss[t][h];
          q = fmaf(a.x, a.x, q); q = fmaf(a.y, a.y, q); q = fmaf(a.z, a.z, q); q = fmaf(a.w, a.w, q);
          q = fmaf(b.x, b.x, q); q = fmaf(b.y, b.y, q); q = fmaf(b.z, b.z, q); q = fmaf(b.w, b.w, q);
          ss[t][h] = in ? q : ss[t][h];
          piece = make_uint4(pack2_bf16(a.x * ga.x, a.y * ga.y), pack2_bf16(a.z * ga.z, a.w * ga.w),
                             pack2_bf16(b.x * gb.x, b.y * gb.y), pack2_bf16(b.z * gb.z, b.w * gb.w));
        } else {
          piece = st.x[t][h][0];
        }
        if (!in) piece = make_uint4(0, 0, 0, 0);                     // past the end of K: zeros, whatever was read
        *reinterpret_cast<uint4*>(mine + (NT + t) * TILE_BYTES + put[h]) = piece;
      }
    }
    __builtin_amdgcn_wave_barrier();       // the wave's lanes read each other's pieces: writes stay before reads
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      Pack8 wf[NT], xf[MT];
#pragma unroll
      for (int i = 0; i < NT; ++i) wf[i].u4 = *reinterpret_cast<const uint4*>(mine + i * TILE_BYTES + get[j]);
#pragma unroll
      for (int t = 0; t < MT; ++t) xf[t].u4 = *reinterpret_cast<const uint4*>(mine + (NT + t) * TILE_BYTES + get[j]);
#pragma unroll
      for (int i = 0; i < NT; ++i)
#pragma unroll
        for (int t = 0; t < MT; ++t)
          acc[i][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[i].v, xf[t].v, acc[i][t], 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();       // and the reads before the next stage's writes
  };
#pragma unroll
  for (int d = 0; d < DEPTH; ++d) fetch(st[d], k_begin + 64 * d);
  if (SQUARES && before.sq) {
    float q = 0.f;
#pragma unroll
    for (int i = 0; i < SQ_HELD; ++i) {
      const float4 v = held[i];
      q += sq_first + i * sq_step < before.quads ? (v.x + v.y) + (v.z + v.w) : 0.f;
    }
    for (int j = sq_first + SQ_HELD * sq_step; j < before.quads; j += sq_step) {
      const float4 v = *reinterpret_cast<const float4*>(sq_src + 4 * j);
      q += (v.x + v.y) + (v.z + v.w);
    }
    if (SQ_LANES == 8) q += __shfl_xor(q, 8);
    q += __shfl_xor(q, 16);
    q += __shfl_xor(q, 32);
    if (lane < 16) sq[wave][lane] = lane < 64 / SQ_LANES ? q : 0.f;
  }
  // DEPTH stages in flight: registers st[d] hold the stages s = d (mod DEPTH).  Whole rounds whose fetches all lie
  // in the wave's share run without a condition; the last rounds fetch only what the share still holds.
  const int stages = k_begin < k_end ? (k_end - k_begin + 63) / 64 : 0;
  int sn = 0;
  for (; sn + 2 * DEPTH <= stages; sn += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      work(st[d], k_begin + 64 * (sn + d));
      fetch(st[d], k_begin + 64 * (sn + d + DEPTH));
    }
  }
  for (; sn < stages; sn += DEPTH) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
      if (sn + d < stages) work(st[d], k_begin + 64 * (sn + d));
      if (sn + d + DEPTH < stages) fetch(st[d], k_begin + 64 * (sn + d + DEPTH));
    }
  }
  if (NORMX) {
    // the 8 lanes of a row hold its pieces: add them, one lane of each row stores the wave's sum
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int h = 0; h < XH; ++h) {
        float q = ss[t][h];
        q += __shfl_xor(q, 1);
        q += __shfl_xor(q, 2);
        q += __shfl_xor(q, 4);
        if (lcol == 0) sq[wave][16 * t + 8 * h + lrow] = q;
      }
    if (XH == 1 && lcol == 0) sq[wave][8 + lrow] = 0.f;
  }
  __syncthreads();                                        // the partial sums take the place of the stages
  auto& red = *reinterpret_cast<float (*)[MAXW - 1][NT * MT][64 * 4]>(lds);
  skinny_finish<MT, NT, EPI, TC>(acc, red, bias, C, R, ldc, M, n_end, n0, scaled, sq, K, eps, ahead);
}

template <int MT, int NT, int EPI, typename TC, bool NORMX, typename... Args>
static void skinny_launch(dim3 grid, dim3 block, hipStream_t stream, const void* X, int ldx, const bf16_t* W, int ldw,
                          const float* bias, const float* gain, float eps, TC* C, float* R, int ldc, int M,
                          Args... rest) {
  if constexpr (MT == 1) {
    if (M <= 8) {
      hipLaunchKernelGGL((gemm_skinny_kernel<1, NT, EPI, TC, NORMX, 1>), grid, block, 0, stream, X, ldx, W, ldw, bias,
                         gain, eps, C, R, ldc, M, rest...);
      return;
    }
  }
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, EPI, TC, NORMX, 2>), grid, block, 0, stream, X, ldx, W, ldw, bias,
                     gain, eps, C, R, ldc, M, rest...);
}

static int skinny_compute_units() {
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

// Columns of the result per block for a block shape that holds up to `cap` of them: the matrix is cut into a
// whole multiple of the compute units' number of blocks (a matrix whose 16-column tiles are 1.25 or 1.5 times
// that number otherwise leaves most units idle for the last part of the run), in steps of 4 columns.
// Returns the share of block slots that do work, in 1/1024.
static int skinny_rows(int N, int cap, int units, int* rows) {
  const int bmin = (N + cap - 1) / cap;
  const int rounds = (bmin + units - 1) / units;
  int r = (N + rounds * units - 1) / (rounds * units);
  r = (r + 3) / 4 * 4;
  if (r > cap) r = cap;
  *rows = r;
  const int blocks = (N + r - 1) / r;
  return (int)(1024LL * blocks / ((long long)((blocks + units - 1) / units) * units));
}

extern "C" int ullm_gemm_skinny_supports(int M, int N, int K, int ldx, int ldw) {
  return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

struct SkinnyPlan {
  int mt, nt, rows, tiles, waves, k_per_wave;
};

// The launch shape of a product: a function of the sizes, the epilogue and whether the norm is folded in.
static int skinny_plan(int M, int N, int K, int ldx, int ldw, int epi, int force_nt, int force_waves, bool normed,
                       int force_rows, SkinnyPlan* p) {
  if (!ullm_gemm_skinny_supports(M, N, K, ldx, ldw)) return ULLM_ERR_SHAPE;
  if (epi < 0 || epi > 2) return ULLM_ERR_UNSUPPORTED;
  int mt = (M + 15) / 16;
  if (mt == 3) mt = 4;                                  // instantiated for 1, 2 and 4 tiles of rows
  const int tiles16 = (N + 15) / 16;
  int nt = 1;
  if (force_nt > 0) nt = force_nt;
  else if (tiles16 >= 4096) nt = mt >= 2 ? 4 : 2;
  else if (tiles16 >= 1024 && mt >= 2) nt = 2;
  // with the norm folded in, a tile of X costs a wave as much as a tile of W: two tiles of W per tile of X
  if (normed && force_nt <= 0) nt = 2;
  if (epi == EPI_SILU) nt = (force_nt == 4 || mt >= 4) ? 4 : 2;   // gate and up tiles come in pairs
  if (nt != 1 && nt != 2 && nt != 4) return ULLM_ERR_UNSUPPORTED;
  if (nt == 4 && mt == 1) nt = 2;                       // not instantiated
  // Columns of the result per block.  Up to 16 rows of X, a matrix that fills the chip is spread evenly over
  // the compute units; for store and add that may take two tiles of W a block of which only a part is used
  // (5120 columns: 256 blocks of 20 instead of 320 of 16, which would leave most units idle in a second round).
  int rows = 16 * (epi == EPI_SILU ? nt / 2 : nt);
  const int units = skinny_compute_units();
  if (force_rows <= 0 && mt == 1 && N >= 16 * units) {
    if (epi == EPI_SILU || force_nt > 0 || nt == 2) {
      skinny_rows(N, rows, units, &rows);
    } else {
      int r1 = 16, r2 = 32;
      const int e1 = skinny_rows(N, 16, units, &r1), e2 = skinny_rows(N, 32, units, &r2);
      if (e2 > e1) { nt = 2; rows = r2; } else { nt = 1; rows = r1; }
    }
  }
  const int out_tiles = epi == EPI_SILU ? nt / 2 : nt;  // 16-column tiles of the result per block
  if (force_rows > 0) {
    if (force_rows > 16 * out_tiles || force_rows % 4) return ULLM_ERR_UNSUPPORTED;
    rows = force_rows;
  }
  // waves per block: 8 tiles of W in flight per block (8 waves with one tile each, 4 with two),
  // each wave with at least 128 values of K
  const int max_waves = sk_max_waves(mt, nt);
  int waves = 1;
  const int in_flight = (normed && epi == EPI_STORE) || epi == EPI_SILU || nt == 4 ? 16 : 8;   // in 16-row tiles of W
  const int w_rows = rows * (nt / out_tiles);           // rows of W a block fetches
  while (waves < max_waves && waves * w_rows < 16 * in_flight && K / (waves * 2) >= 128) waves *= 2;
  if (force_waves > 0) waves = force_waves < max_waves ? force_waves : max_waves;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
  *p = SkinnyPlan{mt, nt, rows, (N + rows - 1) / rows, waves, k_per_wave};
  return 0;
}

// Blocks of the product that adds into the stream (epi 1) for these sizes: the number of partial sums of squares it
// leaves per row when it hands the next norm ahead.  Negative: an error code.
extern "C" int ullm_gemm_skinny_blocks(int M, int N, int K, int ldx, int ldw, int epi, int force_nt, int force_waves,
                                       int force_rows) {
  SkinnyPlan p;
  const int err = skinny_plan(M, N, K, ldx, ldw, epi, force_nt, force_waves, false, force_rows, &p);
  return err ? err : p.tiles;
}

// X bfloat16 [M, K]; W bfloat16 [N, K] (with epi 2: [2 N, K]).  epi: 0 store to C (c_dtype, bias optional),
// 1 add into R (float32 [M, N], row stride ldc), 2 silu(gate) * up to C (bfloat16 [M, N]).
// With gain (float32 [K]): X is float32 [M <= 16, K] and its RMS norm with this gain and eps is what
// is multiplied (epi 0 and 2).  force_nt / force_waves: 0 = chosen here.
// With next_gain (float32 [N], epi 1): the norm that follows is handed ahead: next_x (bfloat16 [M, N], row stride
// ld_next) = the stream's new values * next_gain, next_sq (float32 [M, P], P = ullm_gemm_skinny_blocks(..) rounded
// up to a multiple of 4) = every block's sum of squares of its columns of a row, zeros behind the last block's.
// With row_sq (float32 [M, sq_parts], sq_parts a multiple of 4; epi 0 and 2, no gain): X is such a next_x and the
// results of row m are scaled by rsqrt(sum of row_sq[m][.] / K + eps).
extern "C" int ullm_gemm_skinny(const void* X, int ldx, const void* W, int ldw, const float* bias, void* C,
                                int ldc, int M, int N, int K, int epi, int c_dtype, int force_nt,
                                int force_waves, const float* gain, float eps, int force_rows,
                                const float* next_gain, void* next_x, int ld_next, float* next_sq,
                                const float* row_sq, int sq_parts, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ullm_gemm_skinny_supports(M, N, K, ldx, ldw) || ldc < N) return ULLM_ERR_SHAPE;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return ULLM_ERR_SHAPE;
  if (epi < 0 || epi > 2) return ULLM_ERR_UNSUPPORTED;
  if (gain && (M > 16 || epi == EPI_RESADD || ((uintptr_t)gain & 15))) return ULLM_ERR_UNSUPPORTED;
  if (epi == EPI_RESADD && (((uintptr_t)C & 15) || ldc % 4 != 0 || bias)) return ULLM_ERR_SHAPE;
  if (epi == EPI_SILU && (bias || c_dtype != ULLM_BF16)) return ULLM_ERR_UNSUPPORTED;
  if (next_gain && (epi != EPI_RESADD || !next_x || !next_sq || ld_next < N || ld_next % 4 != 0 ||
                    ((uintptr_t)next_x & 7) || ((uintptr_t)next_gain & 15)))
    return ULLM_ERR_UNSUPPORTED;
  if (row_sq && (gain || M > 16 || epi == EPI_RESADD || sq_parts < 4 || sq_parts % 4 || ((uintptr_t)row_sq & 15))) return ULLM_ERR_UNSUPPORTED;
  SkinnyPlan plan;
  const int err = skinny_plan(M, N, K, ldx, ldw, epi, force_nt, force_waves, gain != nullptr, force_rows, &plan);
  if (err) return err;
  const int mt = plan.mt, nt = plan.nt, rows = plan.rows, tiles = plan.tiles, waves = plan.waves,
            k_per_wave = plan.k_per_wave;
  const NormAhead ahead{next_gain, (bf16_t*)next_x, next_sq, ld_next, (tiles + 3) / 4 * 4};
  const RowSquares before{row_sq, sq_parts / 4};
  dim3 grid(tiles), block(64 * waves);
  float* R = (float*)C;
#define GO_(MT, NT, EPI, TC, NORMX) skinny_launch<MT, NT, EPI, TC, NORMX>(grid, block, stream, X, ldx, \
    (const bf16_t*)W, ldw, bias, gain, eps, (TC*)C, R, ldc, M, N, K, k_per_wave, rows, ahead, before)
#define GO(MT, NT, EPI, TC) GO_(MT, NT, EPI, TC, false)
#define GO_SHAPE(EPI, TC)                                              \
  switch (mt * 8 + nt) {                                               \
    case 1 * 8 + 1: GO(1, 1, EPI, TC); break;                          \
    case 1 * 8 + 2: GO(1, 2, EPI, TC); break;                          \
    case 2 * 8 + 1: GO(2, 1, EPI, TC); break;                          \
    case 2 * 8 + 2: GO(2, 2, EPI, TC); break;                          \
    case 2 * 8 + 4: GO(2, 4, EPI, TC); break;                          \
    case 4 * 8 + 1: GO(4, 1, EPI, TC); break;                          \
    case 4 * 8 + 2: GO(4, 2, EPI, TC); break;                          \
    case 4 * 8 + 4: GO(4, 4, EPI, TC); break;                          \
    default: return ULLM_ERR_UNSUPPORTED;                              \
  }
#define GO_PAIRS(EPI, TC)                                              \
  switch (mt * 8 + nt) {                                               \
    case 1 * 8 + 2: GO(1, 2, EPI, TC); break;                          \
    case 2 * 8 + 2: GO(2, 2, EPI, TC); break;                          \
    case 2 * 8 + 4: GO(2, 4, EPI, TC); break;                          \
    case 4 * 8 + 4: GO(4, 4, EPI, TC); break;                          \
    default: return ULLM_ERR_UNSUPPORTED;                              \
  }
  if (gain) {                                            // one tile of rows
    if (epi == EPI_SILU) {
      if (nt != 2) return ULLM_ERR_UNSUPPORTED;
      GO_(1, 2, EPI_SILU, bf16_t, true);
    } else if (c_dtype == ULLM_BF16) {
      if (nt == 1) GO_(1, 1, EPI_STORE, bf16_t, true); else GO_(1, 2, EPI_STORE, bf16_t, true);
    } else if (c_dtype == ULLM_F32) {
      if (nt == 1) GO_(1, 1, EPI_STORE, float, true); else GO_(1, 2, EPI_STORE, float, true);
    } else return ULLM_ERR_DTYPE;
  } else if (epi == EPI_STORE) {
    if (c_dtype == ULLM_BF16) { GO_SHAPE(EPI_STORE, bf16_t) }
    else if (c_dtype == ULLM_F32) { GO_SHAPE(EPI_STORE, float) }
    else return ULLM_ERR_DTYPE;
  } else if (epi == EPI_RESADD) {
    GO_SHAPE(EPI_RESADD, float)
  } else {
    GO_PAIRS(EPI_SILU, bf16_t)
  }
#undef GO_PAIRS
#undef GO_SHAPE
#undef GO
#undef GO_
  ULLM_LAUNCH_CHECK();
}
