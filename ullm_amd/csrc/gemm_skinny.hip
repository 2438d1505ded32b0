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
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;

union Pack8 {
  bf16x8_t v;
  uint4 u4;
  uint32_t w[4];
  bf16_t h[8];
};

enum { EPI_STORE = 0, EPI_RESADD = 1, EPI_SILU = 2 };

// Most waves per block for a tile shape,
// bounded by the shared memory that holds a stage per wave (and later the waves' partials): at most 8
// waves, so that several blocks fit a compute unit
__host__ __device__ constexpr int sk_max_waves(int mt, int nt) { return mt * nt >= 8 ? 4 : 8; }

// The waves' partial results of a block are added in wave order through `red` and the sum goes where
// EPI says.  acc[i][t][j] = partial C[m = 16 t + r][n0 + 16 i + 4 g + j].
template <int MT, int NT, int EPI, typename TC, typename RedT>
__device__ __forceinline__ void skinny_finish(f32x4_t (&acc)[NT][MT], RedT& red, const float* __restrict__ bias,
                                              TC* __restrict__ C, float* __restrict__ R, int ldc, int M, int N, int n0) {
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
// instruction and of X as many rows as the batch has, was slower the more rows X had: 92 against 80 us
// for the four projections of a Qwen3-8B layer at 8 rows, 105 against 83 us at 16.)
template <int MT, int NT, int EPI, typename TC>
__global__ void __launch_bounds__(64 * sk_max_waves(MT, NT))
gemm_skinny_kernel(const bf16_t* __restrict__ X, int ldx, const bf16_t* __restrict__ W, int ldw,
                          const float* __restrict__ bias, TC* __restrict__ C, float* __restrict__ R, int ldc, int M,
                          int N, int K, int k_per_wave) {
  constexpr int MAXW = sk_max_waves(MT, NT);
  constexpr int TILE_BYTES = 16 * 128, STAGE_BYTES = (NT + MT) * TILE_BYTES;
  constexpr int RED_BYTES = (MAXW - 1) * NT * MT * 256 * 4;
  constexpr int LDS_BYTES = MAXW * STAGE_BYTES > RED_BYTES ? MAXW * STAGE_BYTES : RED_BYTES;
  __shared__ __attribute__((aligned(16))) unsigned char lds[LDS_BYTES];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int g = lane >> 4, r = lane & 15, lrow = lane >> 3, lcol = lane & 7;
  constexpr int OT = EPI == EPI_SILU ? NT / 2 : NT;
  const int n0 = blockIdx.x * (16 * OT);
  const bf16_t* wsrc[NT][2];
  const bf16_t* xsrc[MT][2];
  int put[2], get[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int row = 8 * h + lrow;
    put[h] = row * 128 + ((lcol ^ ((row >> 1) & 7)) << 4);
    get[h] = r * 128 + (((4 * h + g) ^ ((r >> 1) & 7)) << 4);      // h here: the step of 32 inside the stage
#pragma unroll
    for (int i = 0; i < NT; ++i) {
      const int col = n0 + 16 * (i % OT) + row;
      const int n = (col < N ? col : N - 1) + (i / OT) * N;       // rows past N repeat the last row; never stored
      wsrc[i][h] = W + (size_t)n * ldw + 8 * lcol;
    }
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = 16 * t + row < M ? 16 * t + row : M - 1;
      xsrc[t][h] = X + (size_t)m * ldx + 8 * lcol;
    }
  }
  unsigned char* const mine = lds + wave * STAGE_BYTES;
  f32x4_t acc[NT][MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int i = 0; i < NT; ++i) acc[i][t] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int k_begin = wave * k_per_wave;
  int k_end = k_begin + k_per_wave;
  if (k_end > K) k_end = K;
  struct Stage { uint4 w[NT][2], x[MT][2]; };
  constexpr int DEPTH = 2;                                // stages of 64 values of K on their way (3 and 4 were slower)
  Stage st[DEPTH];
  auto fetch = [&](Stage& st, int k0) {
    const bool in = k0 + 8 * lcol < k_end;                        // K is a multiple of 8
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < NT; ++i)
        st.w[i][h] = in ? *reinterpret_cast<const uint4*>(wsrc[i][h] + k0) : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int t = 0; t < MT; ++t)
        st.x[t][h] = in ? *reinterpret_cast<const uint4*>(xsrc[t][h] + k0) : make_uint4(0, 0, 0, 0);
    }
  };
  auto work = [&](const Stage& st) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
#pragma unroll
      for (int i = 0; i < NT; ++i) *reinterpret_cast<uint4*>(mine + i * TILE_BYTES + put[h]) = st.w[i][h];
#pragma unroll
      for (int t = 0; t < MT; ++t) *reinterpret_cast<uint4*>(mine + (NT + t) * TILE_BYTES + put[h]) = st.x[t][h];
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
  if (k_begin < k_end) {
#pragma unroll
    for (int d = 0; d < DEPTH; ++d) fetch(st[d], k_begin + 64 * d);
    for (int k = k_begin; k < k_end; k += 64 * DEPTH) {
#pragma unroll
      for (int d = 0; d < DEPTH; ++d) {
        if (k + 64 * d < k_end) {
          work(st[d]);
          fetch(st[d], k + 64 * (d + DEPTH));
        }
      }
    }
  }
  __syncthreads();                                        // the partial sums take the place of the stages
  auto& red = *reinterpret_cast<float (*)[MAXW - 1][NT * MT][64 * 4]>(lds);
  skinny_finish<MT, NT, EPI, TC>(acc, red, bias, C, R, ldc, M, N, n0);
}

extern "C" int ullm_gemm_skinny_supports(int M, int N, int K, int ldx, int ldw) {
  return M >= 1 && M <= 64 && N >= 1 && K >= 8 && K % 8 == 0 && ldx % 8 == 0 && ldw % 8 == 0;
}

// X bfloat16 [M, K]; W bfloat16 [N, K] (with epi 2: [2 N, K]).  epi: 0 store to C (c_dtype, bias optional),
// 1 add into R (float32 [M, N], row stride ldc), 2 silu(gate) * up to C (bfloat16 [M, N]).
// force_nt / force_waves: 0 = chosen here.
extern "C" int ullm_gemm_skinny(const void* X, int ldx, const void* W, int ldw, const float* bias, void* C,
                                int ldc, int M, int N, int K, int epi, int c_dtype, int force_nt,
                                int force_waves, hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (!ullm_gemm_skinny_supports(M, N, K, ldx, ldw) || ldc < N) return ULLM_ERR_SHAPE;
  if (((uintptr_t)X & 15) || ((uintptr_t)W & 15)) return ULLM_ERR_SHAPE;
  if (epi < 0 || epi > 2) return ULLM_ERR_UNSUPPORTED;
  if (epi == EPI_RESADD && (((uintptr_t)C & 15) || ldc % 4 != 0 || bias)) return ULLM_ERR_SHAPE;
  if (epi == EPI_SILU && (bias || c_dtype != ULLM_BF16)) return ULLM_ERR_UNSUPPORTED;
  int mt = (M + 15) / 16;
  if (mt == 3) mt = 4;                                  // instantiated for 1, 2 and 4 tiles of rows
  const int tiles16 = (N + 15) / 16;
  int nt = 1;
  if (force_nt > 0) nt = force_nt;
  else if (tiles16 >= 4096) nt = mt >= 2 ? 4 : 2;
  else if (tiles16 >= 1024 && mt >= 2) nt = 2;
  if (epi == EPI_SILU) nt = (force_nt == 4 || mt >= 4) ? 4 : 2;   // gate and up tiles come in pairs
  if (nt != 1 && nt != 2 && nt != 4) return ULLM_ERR_UNSUPPORTED;
  if (nt == 4 && mt == 1) nt = 2;                       // not instantiated
  const int out_tiles = epi == EPI_SILU ? nt / 2 : nt;  // 16-column tiles of the result per block
  const int tiles = (tiles16 + out_tiles - 1) / out_tiles;
  // waves per block: 8 tiles of W in flight per block (measured: 8 waves with one tile each, 4 with two),
  // each wave with at least 128 values of K
  const int max_waves = sk_max_waves(mt, nt);
  int waves = 1;
  while (waves < max_waves && waves * nt < 8 && K / (waves * 2) >= 128) waves *= 2;
  if (force_waves > 0) waves = force_waves < max_waves ? force_waves : max_waves;
  int k_per_wave = (K + waves - 1) / waves;
  k_per_wave = (k_per_wave + 63) / 64 * 64;
  dim3 grid(tiles), block(64 * waves);
  float* R = (float*)C;
#define GO(MT, NT, EPI, TC) hipLaunchKernelGGL((gemm_skinny_kernel<MT, NT, EPI, TC>), grid, block, 0, stream, \
    (const bf16_t*)X, ldx, (const bf16_t*)W, ldw, bias, (TC*)C, R, ldc, M, N, K, k_per_wave)
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
  if (epi == EPI_STORE) {
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
  ULLM_LAUNCH_CHECK();
}
