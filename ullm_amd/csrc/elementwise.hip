// Row-wise kernels of the layer: embedding gather into the 32-bit residual stream, fused
// residual add + RMS norm, per-head q/k norm + rotary position encoding + paged cache write,
// and SiLU(gate)*up.  All arithmetic is 32-bit; T selects the storage type only.
//
// Formulas follow the reference's layers: RMS norm (ullm/layers/layernorm.py:20-34),
// half-split rotary pairs (ullm/layers/rotary_embedding.py:5-24), SiLU-and-mul
// (ullm/layers/activation.py:16-18), cache write of k after norm+rotation and raw v
// (ullm/layers/attention.py:288-296).
#include "common.h"

__device__ __forceinline__ float4 ld4_f32(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 ld4_f32(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                     __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
// the same for values that are read once (a branch result, the gate|up product): non-temporal loads
__device__ __forceinline__ float4 ld4_f32_stream(const float* p) {
  const uint4 u = ld_stream16(p);
  return make_float4(__uint_as_float(u.x), __uint_as_float(u.y), __uint_as_float(u.z), __uint_as_float(u.w));
}
__device__ __forceinline__ float4 ld4_f32_stream(const bf16_t* p) {
  const uint2 u = ld_stream8(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u),
                     __uint_as_float(u.y << 16), __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ void st4_f32(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void st4_f32(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack2_bf16(v.x, v.y), pack2_bf16(v.z, v.w));
}


// ------------------------------------------------------------------ embedding
// residual[t, :] = scale * float(table[ids[t], :]); ids outside [0, V) give a zero row.
template <typename T>
__global__ void embedding_kernel(const int* __restrict__ ids, const T* __restrict__ table,
                                 float* __restrict__ residual, int H, int V, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  float* out = residual + (size_t)t * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = 0.f;
    return;
  }
  const T* row = table + (size_t)id * H;
  if (H % 4 == 0 && !(((uintptr_t)table | (uintptr_t)residual) & 15)) {
    for (int i = 4 * threadIdx.x; i < H; i += 4 * blockDim.x) {
      const float4 v = ld4_f32(row + i);
      *reinterpret_cast<float4*>(out + i) = make_float4(v.x * scale, v.y * scale, v.z * scale, v.w * scale);
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[i] = ld_f32(row + i) * scale;
}

extern "C" int ullm_embedding(const int* ids, const void* table, float* residual, int T_, int H,
                              int V, int dtype, float scale, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (H <= 0 || V <= 0) return ULLM_ERR_SHAPE;
  dim3 grid(T_), block(256);
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(embedding_kernel<float>, grid, block, 0, stream, ids, (const float*)table, residual, H, V, scale);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(embedding_kernel<bf16_t>, grid, block, 0, stream, ids, (const bf16_t*)table, residual, H, V, scale);
  else
    return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ a soft cap on the logits
// x = cap * tanh(x / cap), in place, float32 [rows, cols] with row stride ld
__global__ void softcap_kernel(float* __restrict__ x, int cols, int ld, float cap) {
  float* row = x + (size_t)blockIdx.y * ld;
  const float inv = 1.f / cap;
  for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < cols; i += gridDim.x * blockDim.x) row[i] = cap * tanhf(row[i] * inv);
}

extern "C" int ullm_softcap(float* x, int rows, int cols, int ld, float cap, hipStream_t stream) {
  if (rows <= 0 || cols <= 0) return 0;
  if (!(cap > 0.f) || ld < cols || rows > 65535) return ULLM_ERR_SHAPE;
  int bx = (cols + 1023) / 1024;
  if (bx > 256) bx = 256;
  hipLaunchKernelGGL(softcap_kernel, dim3(bx, rows), dim3(256), 0, stream, x, cols, ld, cap);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ token ids that are still on the device
// ids[t] = source[feed[t]] where feed[t] >= 0: the token a request sampled in the step before is taken
// from that step's output, so the next step can be queued before the host has seen the token
// (reference: the device-resident last sampled token, ullm/core/input_batch.py:184-186,
// ullm/core/model_runner.py:277-280).
__global__ void feed_tokens_kernel(int* __restrict__ ids, const int* __restrict__ feed, const int* __restrict__ source,
                                   int n, int n_source) {
  const int t = blockIdx.x * blockDim.x + threadIdx.x;
  if (t >= n) return;
  const int f = feed[t];
  if (f >= 0 && f < n_source) ids[t] = source[f];
}

extern "C" int ullm_feed_tokens(int* ids, const int* feed, const int* source, int n, int n_source, hipStream_t stream) {
  if (n <= 0) return 0;
  if (n_source <= 0) return ULLM_ERR_SHAPE;
  hipLaunchKernelGGL(feed_tokens_kernel, dim3((n + 255) / 256), dim3(256), 0, stream, ids, feed, source, n, n_source);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ rows of per-request state, rows of results
// The state rows (row_bytes bytes each) of the requests that step from their first token are zeroed:
// entry b's row is slot[b], and it starts afresh if start[b] == 0.  grid (entries, pieces of a row).
// The words of a row are 16, 4 or 1 bytes wide, whichever the row size and the base address allow.
template <typename W>
__global__ void zero_fresh_rows_kernel(unsigned char* __restrict__ state, long long row_bytes, int n_rows,
                                       const int* __restrict__ slot, const int* __restrict__ start) {
  const int b = blockIdx.x;
  if (start[b] != 0) return;
  const int row = slot[b];
  if (row < 0 || row >= n_rows) return;
  W* words = reinterpret_cast<W*>(state + (size_t)row * row_bytes);
  const long long n = row_bytes / (long long)sizeof(W);
  W zero;
  memset(&zero, 0, sizeof(W));
  for (long long i = (long long)blockIdx.y * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.y * blockDim.x)
    words[i] = zero;
}

extern "C" int ullm_zero_fresh_rows(void* state, long long row_bytes, int n_rows, const int* slot, const int* start,
                                    int n_entries, hipStream_t stream) {
  if (n_entries <= 0 || row_bytes <= 0) return 0;
  if (n_rows <= 0) return ULLM_ERR_SHAPE;
  const int width = (row_bytes % 16 == 0 && ((uintptr_t)state & 15) == 0) ? 16
                    : (row_bytes % 4 == 0 && ((uintptr_t)state & 3) == 0) ? 4 : 1;
  long long pieces = (row_bytes / width + 255) / 256;
  if (pieces > 64) pieces = 64;
  dim3 grid(n_entries, (unsigned)pieces), block(256);
  if (width == 16)
    hipLaunchKernelGGL(zero_fresh_rows_kernel<uint4>, grid, block, 0, stream, (unsigned char*)state, row_bytes, n_rows, slot, start);
  else if (width == 4)
    hipLaunchKernelGGL(zero_fresh_rows_kernel<uint32_t>, grid, block, 0, stream, (unsigned char*)state, row_bytes, n_rows, slot, start);
  else
    hipLaunchKernelGGL(zero_fresh_rows_kernel<unsigned char>, grid, block, 0, stream, (unsigned char*)state, row_bytes, n_rows, slot, start);
  ULLM_LAUNCH_CHECK();
}

// out[i, :] = src[index[i], :] for float32 rows (an index outside [0, n_src) gives a row of zeros).
// grid (rows, pieces of a row).
__global__ void gather_rows_kernel(const float* __restrict__ src, long long src_stride, int n_src,
                                   const int* __restrict__ index, float* __restrict__ out, int cols, int vec) {
  const int i = blockIdx.x;
  const int from = index[i];
  const bool ok = from >= 0 && from < n_src;
  const float* row = src + (size_t)(ok ? from : 0) * src_stride;
  float* dst = out + (size_t)i * cols;
  if (vec) {
    for (int c = 4 * (blockIdx.y * blockDim.x + threadIdx.x); c < cols; c += 4 * gridDim.y * blockDim.x)
      *reinterpret_cast<float4*>(dst + c) = ok ? ld4_f32_stream(row + c) : make_float4(0.f, 0.f, 0.f, 0.f);
    return;
  }
  for (int c = blockIdx.y * blockDim.x + threadIdx.x; c < cols; c += gridDim.y * blockDim.x) dst[c] = ok ? row[c] : 0.f;
}

extern "C" int ullm_gather_rows(const float* src, long long src_stride, int n_src, const int* index, float* out,
                                int n, int cols, hipStream_t stream) {
  if (n <= 0 || cols <= 0) return 0;
  if (n_src <= 0 || src_stride < cols) return ULLM_ERR_SHAPE;
  const int vec = cols % 4 == 0 && src_stride % 4 == 0 && !(((uintptr_t)src | (uintptr_t)out) & 15);
  int pieces = (cols / (vec ? 4 : 1) + 255) / 256;
  if (pieces > 256) pieces = 256;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(n, pieces), dim3(256), 0, stream, src, src_stride, n_src, index, out, cols, vec);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ a plain streaming read, for measurement
// Every block reads its share of `bytes` once with non-temporal 16-byte loads, eight in flight per thread,
// and stores one word per block (the xor of what it read, so that no load can be dropped).  What this
// reaches is the practical ceiling of a kernel that only reads, as a decode step's weight streaming does.
__global__ void __launch_bounds__(256)
stream_read_kernel(const uint4* __restrict__ src, long long n16, unsigned* __restrict__ sink) {
  const long long stride = (long long)gridDim.x * blockDim.x;
  long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x;
  unsigned acc = 0;
  for (; i + 7 * stride < n16; i += 8 * stride) {
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = ld_stream16(src + i + u * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
  }
  for (; i < n16; i += stride) {
    const uint4 v = ld_stream16(src + i);
    acc ^= v.x ^ v.y ^ v.z ^ v.w;
  }
  for (int m = WAVE / 2; m > 0; m >>= 1) acc ^= __shfl_xor(acc, m, WAVE);
  if ((threadIdx.x & (WAVE - 1)) == 0) sink[blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE] = acc;
}

// sink: at least blocks * 4 words.  blocks <= 0: eight per compute unit.
extern "C" int ullm_stream_read(const void* src, long long bytes, unsigned* sink, int blocks, hipStream_t stream) {
  if (bytes <= 0) return 0;
  if (((uintptr_t)src & 15) || bytes % 16) return ULLM_ERR_SHAPE;
  if (blocks <= 0) {
    int dev = 0, units = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || units <= 0)
      units = 256;
    blocks = 8 * units;
  }
  hipLaunchKernelGGL(stream_read_kernel, dim3(blocks), dim3(256), 0, stream, (const uint4*)src, bytes / 16, sink);
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ add + RMS norm
// For output row r (input row i = rows ? rows[r] : r):
//   s = residual[i] + float(branch[i])      (branch may be null: s = residual[i]; it may also be a stack
//                                            of n_branch arrays branch_stride apart, added in order)
//   if write_res: residual[i] = s           (the stream stays 32-bit, never rounded)
//   y[r] = s * rsqrt(mean(s^2) + eps) * gain
// One block per row.  The general kernel walks the row twice with scalar loads; the fast one
// (H a multiple of 4 and at most 4 * 4 * blockDim) keeps the row's sums in registers between the
// reduction and the scaling and moves 16 bytes per lane and access.
template <typename TB, typename TY>
__global__ void add_rmsnorm_kernel(const TB* __restrict__ branch, float* __restrict__ residual,
                                   const float* __restrict__ gain, float eps, TY* __restrict__ y,
                                   const int* __restrict__ rows, int H, int write_res, int n_branch,
                                   long long branch_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int i = rows ? rows[r] : r;
  float* res = residual + (size_t)i * H;
  const TB* br = branch ? branch + (size_t)i * H : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    float s = res[c];
    if (br)
      for (int p = 0; p < n_branch; ++p) s += ld_f32(br + (size_t)p * branch_stride + c);
    if (write_res && br) res[c] = s;
    ss += s * s;
  }
  const float total = block_sum(ss, scratch);
  const float rs = rsqrtf(total / (float)H + eps);
  TY* out = y + (size_t)r * H;
  for (int c = threadIdx.x; c < H; c += blockDim.x) {
    float s = res[c];
    if (br && !write_res)
      for (int p = 0; p < n_branch; ++p) s += ld_f32(br + (size_t)p * branch_stride + c);
    st_f32(out + c, (s * rs) * gain[c]);
  }
}

#define NORM_VEC_MAX 4     // float4 groups per thread
template <typename TB, typename TY>
__global__ void add_rmsnorm_vec_kernel(const TB* __restrict__ branch, float* __restrict__ residual,
                                       const float* __restrict__ gain, float eps, TY* __restrict__ y,
                                       const int* __restrict__ rows, int H, int write_res, int n_branch,
                                       long long branch_stride) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const int i = rows ? rows[r] : r;
  float* res = residual + (size_t)i * H;
  const TB* br = branch ? branch + (size_t)i * H : nullptr;
  float4 v[NORM_VEC_MAX], gn[NORM_VEC_MAX];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < NORM_VEC_MAX; ++j) {
    const int c = 4 * (threadIdx.x + j * blockDim.x);
    if (c < H) {
      float4 s = ld4_f32(res + c);
      gn[j] = ld4_f32(gain + c);                     // on its way during the reduction
      if (br) {
        // a stack is added in order, eight of its arrays fetched at a time (a load per turn of the loop would
        // wait for each before the next goes out)
        // a stack is added in order, eight (then four) of its arrays fetched at a time: a load per turn of
        // the loop would wait for each before the next goes out
        int p = 0;
        for (; p + 8 <= n_branch; p += 8) {
          float4 b[8];
#pragma unroll
          for (int u = 0; u < 8; ++u) b[u] = ld4_f32_stream(br + (size_t)(p + u) * branch_stride + c);
#pragma unroll
          for (int u = 0; u < 8; ++u) { s.x += b[u].x; s.y += b[u].y; s.z += b[u].z; s.w += b[u].w; }
        }
        if (p + 4 <= n_branch) {
          float4 b[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) b[u] = ld4_f32_stream(br + (size_t)(p + u) * branch_stride + c);
#pragma unroll
          for (int u = 0; u < 4; ++u) { s.x += b[u].x; s.y += b[u].y; s.z += b[u].z; s.w += b[u].w; }
          p += 4;
        }
        for (; p < n_branch; ++p) {
          const float4 b = ld4_f32_stream(br + (size_t)p * branch_stride + c);
          s.x += b.x; s.y += b.y; s.z += b.z; s.w += b.w;
        }
        if (write_res) st4_f32(res + c, s);
      }
      v[j] = s;
      ss += s.x * s.x + s.y * s.y + s.z * s.z + s.w * s.w;
    }
  }
  const float rs = rsqrtf(block_sum(ss, scratch) / (float)H + eps);
  TY* out = y + (size_t)r * H;
#pragma unroll
  for (int j = 0; j < NORM_VEC_MAX; ++j) {
    const int c = 4 * (threadIdx.x + j * blockDim.x);
    if (c < H) {
      const float4 g = gn[j];
      st4_f32(out + c, make_float4((v[j].x * rs) * g.x, (v[j].y * rs) * g.y, (v[j].z * rs) * g.z, (v[j].w * rs) * g.w));
    }
  }
}

extern "C" int ullm_add_rmsnorm(const void* branch, float* residual, const float* gain, float eps,
                                void* y, const int* rows, int n_rows, int H, int branch_dtype,
                                int y_dtype, int write_res, int n_branch, long long branch_stride,
                                hipStream_t stream) {
  if (n_rows <= 0) return 0;
  if (H <= 0 || n_branch < 1 || (n_branch > 1 && branch_stride % 4 != 0)) return ULLM_ERR_SHAPE;
  if (rows && write_res) return ULLM_ERR_UNSUPPORTED;  // a gathered row could be updated twice
  // a block a row; with few rows the chip is far from full, so wide rows get as many threads as they have
  // groups of four values (up to 1024), which puts all of a row's loads on their way at once
  const int threads = H >= 4096 ? (n_rows <= 1024 ? 1024 : 512) : (H >= 2048 && n_rows <= 1024 ? 512 : 256);
  const bool vec = H % 4 == 0 && H <= 4 * NORM_VEC_MAX * threads && !(((uintptr_t)residual | (uintptr_t)gain |
                   (uintptr_t)y | (uintptr_t)branch) & 15);
  dim3 grid(n_rows), block(threads);
#define GO(TB, TY) do { if (vec) hipLaunchKernelGGL((add_rmsnorm_vec_kernel<TB, TY>), grid, block, 0, stream, \
    (const TB*)branch, residual, gain, eps, (TY*)y, rows, H, write_res, n_branch, branch_stride); \
  else hipLaunchKernelGGL((add_rmsnorm_kernel<TB, TY>), grid, block, 0, stream, \
    (const TB*)branch, residual, gain, eps, (TY*)y, rows, H, write_res, n_branch, branch_stride); } while (0)
  if (branch_dtype == ULLM_F32 && y_dtype == ULLM_F32) GO(float, float);
  else if (branch_dtype == ULLM_BF16 && y_dtype == ULLM_BF16) GO(bf16_t, bf16_t);
  else if (branch_dtype == ULLM_BF16 && y_dtype == ULLM_F32) GO(bf16_t, float);
  else if (branch_dtype == ULLM_F32 && y_dtype == ULLM_BF16) GO(float, bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ residual += branch
template <typename T>
__global__ void residual_add_kernel(const T* __restrict__ branch, float* __restrict__ residual, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx < total) residual[idx] += ld_f32(branch + idx);
}

extern "C" int ullm_residual_add(const void* branch, float* residual, long long total, int dtype, hipStream_t stream) {
  if (total <= 0) return 0;
  dim3 block(256), grid((unsigned)((total + 255) / 256));
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(residual_add_kernel<float>, grid, block, 0, stream, (const float*)branch, residual, (size_t)total);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(residual_add_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)branch, residual, (size_t)total);
  else
    return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ y[t, :] += bias (float32 [N]), in place
template <typename T>
__global__ void add_bias_kernel(T* __restrict__ y, const float* __restrict__ bias, int N, long long row_stride, size_t total) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / N;
  const int n = (int)(idx - t * N);
  T* p = y + t * row_stride + n;
  st_f32(p, ld_f32(p) + bias[n]);
}

extern "C" int ullm_add_bias(void* y, const float* bias, int T_, int N, long long row_stride, int dtype, hipStream_t stream) {
  if (T_ <= 0 || N <= 0) return 0;
  const size_t total = (size_t)T_ * N;
  dim3 block(256), grid((unsigned)((total + 255) / 256));
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(add_bias_kernel<float>, grid, block, 0, stream, (float*)y, bias, N, row_stride, total);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(add_bias_kernel<bf16_t>, grid, block, 0, stream, (bf16_t*)y, bias, N, row_stride, total);
  else
    return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ SiLU(gate) * up
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= total) return;
  const size_t t = idx / I;
  const int i = (int)(idx - t * I);
  const T* row = gu + t * (size_t)(2 * I);
  const float g = ld_f32(row + i), u = ld_f32(row + I + i);
  // 32-bit mode: exact exponential and division; bfloat16: the hardware's, then rounded
  const float s = sizeof(T) == 4 ? g / (1.f + expf(-g)) : fast_silu(g);
  st_f32(out + idx, s * u);
}

template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total4) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;    // group of 4 consecutive outputs
  if (idx >= total4) return;
  const size_t per_row = (size_t)(I / 4);
  const size_t t = idx / per_row;
  const int i = 4 * (int)(idx - t * per_row);
  const T* row = gu + t * (size_t)(2 * I);
  const float4 g = ld4_f32_stream(row + i), u = ld4_f32_stream(row + I + i);
  float4 o;
  if (sizeof(T) == 4) {
    o = make_float4(g.x / (1.f + expf(-g.x)) * u.x, g.y / (1.f + expf(-g.y)) * u.y,
                    g.z / (1.f + expf(-g.z)) * u.z, g.w / (1.f + expf(-g.w)) * u.w);
  } else {
    o = make_float4(fast_silu(g.x) * u.x, fast_silu(g.y) * u.y, fast_silu(g.z) * u.z, fast_silu(g.w) * u.w);
  }
  st4_f32(out + t * (size_t)I + i, o);
}

extern "C" int ullm_silu_mul(const void* gu, void* out, int T_, int I, int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (I <= 0) return ULLM_ERR_SHAPE;
  const size_t total = (size_t)T_ * I;
  if (I % 4 == 0 && !(((uintptr_t)gu | (uintptr_t)out) & 15)) {
    const size_t total4 = total / 4;
    dim3 vblock(256), vgrid((unsigned)((total4 + 255) / 256));
    if (dtype == ULLM_F32)
      hipLaunchKernelGGL(silu_mul_vec_kernel<float>, vgrid, vblock, 0, stream, (const float*)gu, (float*)out, I, total4);
    else if (dtype == ULLM_BF16)
      hipLaunchKernelGGL(silu_mul_vec_kernel<bf16_t>, vgrid, vblock, 0, stream, (const bf16_t*)gu, (bf16_t*)out, I, total4);
    else
      return ULLM_ERR_DTYPE;
    ULLM_LAUNCH_CHECK();
  }
  dim3 block(256), grid((unsigned)((total + 255) / 256));
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, block, 0, stream, (const float*)gu, (float*)out, I, total);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, grid, block, 0, stream, (const bf16_t*)gu, (bf16_t*)out, I, total);
  else
    return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ stacks of partial sums to one result
// out[m][n] = sum over s of stacks[s][m][n] (+ bias[n]), the stacks added in order, four columns a thread.
// What a first projection needs from the partial-sums product (the last projections' stacks are added by
// the norm that follows them).
template <typename T>
__global__ void __launch_bounds__(256)
sum_stacks_kernel(const float* __restrict__ stacks, size_t stack_stride, int n_stacks, const float* __restrict__ bias,
                  T* __restrict__ out, int N, size_t total4) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total4) return;
  const size_t at = 4 * i;
  float4 a = ld4_f32(stacks + at);
  for (int s = 1; s < n_stacks; ++s) {
    const float4 b = ld4_f32(stacks + (size_t)s * stack_stride + at);
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
  }
  if (bias) {
    const float4 b = ld4_f32(bias + at % N);
    a.x += b.x; a.y += b.y; a.z += b.z; a.w += b.w;
  }
  st4_f32(out + at, a);
}

// stacks float32 [n_stacks, M, N] contiguous, N a multiple of 4; out [M, N] contiguous, float32 or bfloat16
extern "C" int ullm_sum_stacks(const float* stacks, int n_stacks, const float* bias, void* out, int M, int N, int dtype,
                               hipStream_t stream) {
  if (M <= 0 || N <= 0) return 0;
  if (n_stacks < 1 || N % 4 || (((uintptr_t)stacks | (uintptr_t)out | (uintptr_t)bias) & 15)) return ULLM_ERR_SHAPE;
  const size_t total4 = (size_t)M * N / 4;
  dim3 block(256), grid((unsigned)((total4 + 255) / 256));
  if (dtype == ULLM_F32)
    hipLaunchKernelGGL(sum_stacks_kernel<float>, grid, block, 0, stream, stacks, (size_t)M * N, n_stacks, bias, (float*)out, N, total4);
  else if (dtype == ULLM_BF16)
    hipLaunchKernelGGL(sum_stacks_kernel<bf16_t>, grid, block, 0, stream, stacks, (size_t)M * N, n_stacks, bias, (bf16_t*)out, N, total4);
  else
    return ULLM_ERR_DTYPE;
  ULLM_LAUNCH_CHECK();
}

// ------------------------------------------------------------------ q/k norm + rotary + cache write
// One wave per (token, head) of the fused projection row  [q heads | k heads | v heads].
//   q heads: per-head RMS norm (gain shared by all heads, may be null), rotation, written to q_out
//   k heads: the same with the k gain, written into the token's cache page
//   v heads: copied into the cache page
// Rotation: pair (i, i + rot/2) for style 1 (half split), (2i, 2i+1) for style 2, i < rot/2;
//   o_a = a cos - b sin, o_b = b cos + a sin with cos/sin = table[pos, i], table[pos, rot/2 + i];
//   dims >= rot pass through.  style 0: no rotation.
// Cache page of token t: block_table[entry[t], pos / page_size], row pos % page_size.
// Key pool layout [page, kv_head, row, head_dim]; value pool layout [page, kv_head, head_dim, row]
// (values are kept transposed inside a page so that the attention kernels can load eight keys of
// one dimension as one vector).  Tokens whose page id is negative are not written.
#define MAX_HEAD_DIM 512
template <typename T>
__global__ void qk_norm_rope_write_kernel(
    const T* __restrict__ qkv, int qkv_stride, T* __restrict__ q_out, int q_out_stride,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_sin, int table_rows, int rot, int style,
    const int* __restrict__ positions, const int* __restrict__ token_entry,
    const int* __restrict__ block_table, int bt_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
    int page_size, int nq, int nkv, int hd, int write_kv) {
  __shared__ float vals[MAX_HEAD_DIM];
  const int t = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  const T* src = qkv + (size_t)t * qkv_stride + (size_t)head * hd;
  const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
  T* dst;
  if (is_q) {
    dst = q_out + (size_t)t * q_out_stride + (size_t)head * hd;
  } else {
    if (!write_kv) return;
    const int kvh = is_k ? head - nq : head - nq - nkv;
    const int page = block_table[(size_t)token_entry[t] * bt_stride + pos / page_size];
    if (page < 0) return;
    if (!is_k) {  // v: transposed copy
      T* vdst = v_pool + ((size_t)page * nkv + kvh) * hd * page_size + (pos % page_size);
      for (int i = lane; i < hd; i += WAVE) vdst[(size_t)i * page_size] = src[i];
      return;
    }
    dst = k_pool + (((size_t)page * nkv + kvh) * page_size + (pos % page_size)) * hd;
  }
  const float* gain = is_q ? q_gain : k_gain;
  float ss = 0.f;
  for (int i = lane; i < hd; i += WAVE) {
    const float x = ld_f32(src + i);
    vals[i] = x;
    ss += x * x;
  }
  if (gain) {
    ss = wave_sum(ss);
    const float rs = rsqrtf(ss / (float)hd + eps);
    for (int i = lane; i < hd; i += WAVE) vals[i] = (vals[i] * rs) * gain[i];
  }
  __syncthreads();
  if (style == 0 || rot <= 0) {
    for (int i = lane; i < hd; i += WAVE) st_f32(dst + i, vals[i]);
    return;
  }
  const int half = rot / 2;
  const int p = pos < table_rows ? pos : table_rows - 1;  // host rejects positions past the table
  const float* cs = cos_sin + (size_t)p * rot;
  for (int i = lane; i < half; i += WAVE) {
    const int ia = style == 1 ? i : 2 * i, ib = style == 1 ? i + half : 2 * i + 1;
    const float c = cs[i], s = cs[half + i];
    const float a = vals[ia], b = vals[ib];
    st_f32(dst + ia, a * c - b * s);
    st_f32(dst + ib, b * c + a * s);
  }
  for (int i = rot + lane; i < hd; i += WAVE) st_f32(dst + i, vals[i]);
}

// Values of many tokens at once: a block takes VALUE_RUN_TOKENS consecutive tokens of the batch and one
// kv head, gathers their value rows in LDS and writes them transposed.  Eight tokens of one request at
// positions 8k .. 8k+7 lie side by side in one row of a page (page sizes that are multiples of 8), so a
// thread writes them as one 16-byte (bfloat16) or two 16-byte (float) stores per dim instead of eight
// single elements; tokens that do not fill such a group are written one by one.
#define VALUE_RUN_TOKENS 16
#define VALUE_RUN_MAX_HD 256
template <typename T>
__device__ __forceinline__ void value_runs_block(
    const T* __restrict__ qkv, int qkv_stride, const int* __restrict__ positions, const int* __restrict__ token_entry,
    const int* __restrict__ block_table, int bt_stride, T* __restrict__ v_pool, int page_size, int nq, int nkv,
    int hd, int n_tokens, int block) {
  __shared__ __attribute__((aligned(16))) T tile[VALUE_RUN_TOKENS * VALUE_RUN_MAX_HD];
  __shared__ int s_page[VALUE_RUN_TOKENS], s_off[VALUE_RUN_TOKENS], s_run[VALUE_RUN_TOKENS];
  const int kvh = block % nkv, tok0 = (block / nkv) * VALUE_RUN_TOKENS;
  const int n = n_tokens - tok0 < VALUE_RUN_TOKENS ? n_tokens - tok0 : VALUE_RUN_TOKENS;
  constexpr int PER16 = 16 / (int)sizeof(T);                // elements per 16-byte piece
  const int pieces = hd / PER16;
  for (int c = threadIdx.x; c < n * pieces; c += blockDim.x) {
    const int tok = c / pieces, part = c % pieces;
    *reinterpret_cast<uint4*>(tile + tok * hd + part * PER16) = *reinterpret_cast<const uint4*>(
        qkv + (size_t)(tok0 + tok) * qkv_stride + (size_t)(nq + nkv + kvh) * hd + part * PER16);
  }
  if ((int)threadIdx.x < n) {
    // a token leads a run if it is the block's first or does not continue its predecessor's group of 8
    const int i = threadIdx.x, t = tok0 + i;
    const int pos = positions[t], ent = token_entry[t];
    s_page[i] = block_table[(size_t)ent * bt_stride + pos / page_size];
    s_off[i] = pos % page_size;
    const bool leads = i == 0 || token_entry[t - 1] != ent || positions[t - 1] != pos - 1 || (pos & 7) == 0;
    int run = 0;
    if (leads) {
      run = 1;
      while (i + run < n && token_entry[t + run] == ent && positions[t + run] == pos + run && ((pos + run) & 7) != 0) ++run;
    }
    s_run[i] = run;
  }
  __syncthreads();
  // item = (dim, half of the block's tokens)
  for (int item = threadIdx.x; item < 2 * hd; item += blockDim.x) {
    const int d = item % hd, first = (item / hd) * (VALUE_RUN_TOKENS / 2);
    for (int i = first; i < first + VALUE_RUN_TOKENS / 2 && i < n; ++i) {
      const int run = s_run[i];
      if (run == 0 || s_page[i] < 0) continue;
      T* dst = v_pool + (((size_t)s_page[i] * nkv + kvh) * hd + d) * page_size + s_off[i];
      if (run == 8 && (s_off[i] & 7) == 0) {                // one row of one page, aligned
        __attribute__((aligned(16))) T eight[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) eight[j] = tile[(i + j) * hd + d];
#pragma unroll
        for (int j = 0; j < 8 / PER16; ++j)
          reinterpret_cast<uint4*>(dst)[j] = reinterpret_cast<const uint4*>(eight)[j];
      } else {
        // the run's tokens follow each other in the page as long as the page does not end
        for (int j = 0; j < run; ++j) {
          if (s_page[i + j] < 0) continue;
          v_pool[(((size_t)s_page[i + j] * nkv + kvh) * hd + d) * page_size + s_off[i + j]] = tile[(i + j) * hd + d];
        }
      }
    }
  }
}

// The same for head sizes of 8 * (a power of two): a head is held by head_dim / 8 neighbouring lanes
// with 8 consecutive dims each (16-byte loads and stores for bfloat16), a block of 256 threads takes
// 2048 / head_dim heads of one token at a time, heads_per_thread times in turn.  For half-split pairs the partner dims come from the lane
// rot / 16 further on (or back) by shuffles, which needs rot to be a multiple of 16.
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_rope_write_vec_kernel(
    const T* __restrict__ qkv, int qkv_stride, T* __restrict__ q_out, int q_out_stride,
    const float* __restrict__ q_gain, const float* __restrict__ k_gain, float eps,
    const float* __restrict__ cos_sin, int table_rows, int rot, int style,
    const int* __restrict__ positions, const int* __restrict__ token_entry,
    const int* __restrict__ block_table, int bt_stride, T* __restrict__ k_pool, T* __restrict__ v_pool,
    int page_size, int nq, int nkv, int hd, int write_kv, int n_tokens, int blocks_per_token, int heads_per_thread) {
  if (blockIdx.x >= (unsigned)(n_tokens * blocks_per_token)) {
    value_runs_block<T>(qkv, qkv_stride, positions, token_entry, block_table, bt_stride, v_pool, page_size, nq, nkv,
                        hd, n_tokens, (int)blockIdx.x - n_tokens * blocks_per_token);
    return;
  }
  const int lph = hd >> 3;                                  // lanes per head
  const int t = blockIdx.x / blocks_per_token;
  const int part = threadIdx.x % lph, d0 = 8 * part;
  const int pos = positions[t];
  const int off = pos % page_size;
  // what depends on the token and the lane's dims alone is fetched once for all the heads the thread takes
  const bool rotates = style != 0 && rot > 0;
  const int half = rot / 2;
  const bool first = d0 < half, in = d0 < rot;              // rot and half are multiples of 8: a lane is on one side
  float c[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f}, sn[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const float* cs = nullptr;
  if (rotates) {
    const int p = pos < table_rows ? pos : table_rows - 1;  // host rejects positions past the table
    cs = cos_sin + (size_t)p * rot;
    if (style == 1 && in) {
      const int i0 = first ? d0 : d0 - half;
      const float4 c0 = *reinterpret_cast<const float4*>(cs + i0), c1 = *reinterpret_cast<const float4*>(cs + i0 + 4);
      const float4 s0 = *reinterpret_cast<const float4*>(cs + half + i0), s1 = *reinterpret_cast<const float4*>(cs + half + i0 + 4);
      c[0] = c0.x; c[1] = c0.y; c[2] = c0.z; c[3] = c0.w; c[4] = c1.x; c[5] = c1.y; c[6] = c1.z; c[7] = c1.w;
      sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
    }
  }
  for (int pass = 0; pass < heads_per_thread; ++pass) {
    const int head = ((blockIdx.x % blocks_per_token) * heads_per_thread + pass) * (256 / lph) + threadIdx.x / lph;
    const bool live = head < nq + 2 * nkv;
    const bool is_q = head < nq, is_k = !is_q && head < nq + nkv;
    float x[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    if (live) {
      const T* src = qkv + (size_t)t * qkv_stride + (size_t)head * hd + d0;
      const float4 lo = ld4_f32_stream(src), hi = ld4_f32_stream(src + 4);     // the projection row is read once
      x[0] = lo.x; x[1] = lo.y; x[2] = lo.z; x[3] = lo.w; x[4] = hi.x; x[5] = hi.y; x[6] = hi.z; x[7] = hi.w;
    }
    int page = -1;
    if (live && !is_q && (write_kv & (is_k ? 1 : 2)))
      page = block_table[(size_t)token_entry[t] * bt_stride + pos / page_size];
    if (live && !is_q && !is_k) {                             // v: transposed copy, no arithmetic
      if (page >= 0) {
        const int kvh = head - nq - nkv;
        T* vdst = v_pool + ((size_t)page * nkv + kvh) * hd * page_size + (size_t)d0 * page_size + off;
#pragma unroll
        for (int j = 0; j < 8; ++j) st_f32(vdst + (size_t)j * page_size, x[j]);
      }
    }
    // every lane takes part in the shuffles below; lanes of value heads and dead lanes carry zeros
    const float* gain = is_q ? q_gain : k_gain;
    const bool arith = live && (is_q || is_k);
    if (gain) {
      float ss = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(x[j], x[j], ss);
      // pairwise, the most distant lanes of a head first: the decode attention kernel, which does this
      // norm itself for single new tokens, adds in the same order (multiply-adds spelled out in both)
      for (int m = lph >> 1; m > 0; m >>= 1) ss += __shfl_xor(ss, m, WAVE);
      const float rs = rsqrtf(ss / (float)hd + eps);
      if (arith) {
        const float4 g0 = *reinterpret_cast<const float4*>(gain + d0), g1 = *reinterpret_cast<const float4*>(gain + d0 + 4);
        const float gg[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) x[j] = (x[j] * rs) * gg[j];
      }
    }
    if (rotates) {
      if (style == 1) {
        const int src_lane = (int)(threadIdx.x & (WAVE - 1)) + (first ? half / 8 : -(half / 8));
        float y[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) y[j] = __shfl(x[j], in ? src_lane : (int)(threadIdx.x & (WAVE - 1)), WAVE);
        if (in && arith) {
#pragma unroll
          for (int j = 0; j < 8; ++j) x[j] = first ? fmaf(x[j], c[j], -(y[j] * sn[j])) : fmaf(x[j], c[j], y[j] * sn[j]);
        }
      } else if (arith) {
#pragma unroll
        for (int j = 0; j < 8; j += 2) {
          if (d0 + j < rot) {
            const int i = (d0 + j) >> 1;
            const float cc = cs[i], ss2 = cs[half + i], a = x[j], b2 = x[j + 1];
            x[j] = a * cc - b2 * ss2;
            x[j + 1] = b2 * cc + a * ss2;
          }
        }
      }
    }
    if (!arith) continue;
    T* dst;
    if (is_q) {
      dst = q_out + (size_t)t * q_out_stride + (size_t)head * hd + d0;
    } else {
      if (page < 0) continue;
      dst = k_pool + (((size_t)page * nkv + (head - nq)) * page_size + off) * hd + d0;
    }
    st4_f32(dst, make_float4(x[0], x[1], x[2], x[3]));
    st4_f32(dst + 4, make_float4(x[4], x[5], x[6], x[7]));
  }
}

extern "C" int ullm_qk_norm_rope_write(
    const void* qkv, int qkv_stride, void* q_out, int q_out_stride, const float* q_gain,
    const float* k_gain, float eps, const float* cos_sin, int table_rows, int rot, int style,
    const int* positions, const int* token_entry, const int* block_table, int bt_stride,
    void* k_pool, void* v_pool, int page_size, int T_, int nq, int nkv, int hd, int write_kv,
    int dtype, hipStream_t stream) {
  if (T_ <= 0) return 0;
  if (hd <= 0 || hd > MAX_HEAD_DIM || nq <= 0 || nkv <= 0 || page_size <= 0) return ULLM_ERR_SHAPE;
  if (rot < 0 || rot > hd || (rot & 1) || (style != 0 && style != 1 && style != 2)) return ULLM_ERR_SHAPE;
  if (style != 0 && rot > 0 && (!cos_sin || table_rows <= 0)) return ULLM_ERR_SHAPE;
  const int lph = hd / 8;
  const bool vec = hd % 8 == 0 && lph >= 4 && lph <= 64 && (lph & (lph - 1)) == 0 && qkv_stride % 8 == 0 &&
                   q_out_stride % 8 == 0 && (style != 1 || rot % 16 == 0) && ((uintptr_t)qkv & 15) == 0 &&
                   ((uintptr_t)q_out & 15) == 0 && (!k_pool || ((uintptr_t)k_pool & 15) == 0) &&
                   (!cos_sin || ((uintptr_t)cos_sin & 15) == 0) && (!q_gain || ((uintptr_t)q_gain & 15) == 0) &&
                   (!k_gain || ((uintptr_t)k_gain & 15) == 0) && rot % 8 == 0;
  if (vec) {
    // with few tokens a thread takes one head, so that many blocks are under way; with many it takes up to four
    // in turn, for which it fetches its cosines and sines once
    const int heads_per_block = 256 / lph;
    int blocks_per_token = (nq + 2 * nkv + heads_per_block - 1) / heads_per_block;
    int heads_per_thread = 1;
    if (T_ >= 1024) {
      heads_per_thread = blocks_per_token < 4 ? blocks_per_token : 4;
      blocks_per_token = (blocks_per_token + heads_per_thread - 1) / heads_per_thread;
    }
    // with many tokens the values go through blocks of their own that write runs of eight at once
    const bool runs = write_kv && T_ >= 128 && page_size % 8 == 0 && hd <= VALUE_RUN_MAX_HD &&
                      ((uintptr_t)v_pool & 15) == 0;
    const long long value_blocks = runs ? (long long)((T_ + VALUE_RUN_TOKENS - 1) / VALUE_RUN_TOKENS) * nkv : 0;
    const long long all_blocks = (long long)T_ * blocks_per_token + value_blocks;
    if (all_blocks > 0x7fffffffLL) return ULLM_ERR_SHAPE;
    const int kv_flags = !write_kv ? 0 : (runs ? 1 : 3);   // bit 0: keys, bit 1: values token by token
    dim3 vgrid((unsigned)all_blocks), vblock(256);
#define GOV(TT) hipLaunchKernelGGL(qk_norm_rope_write_vec_kernel<TT>, vgrid, vblock, 0, stream, \
    (const TT*)qkv, qkv_stride, (TT*)q_out, q_out_stride, q_gain, k_gain, eps, cos_sin, table_rows, \
    rot, style, positions, token_entry, block_table, bt_stride, (TT*)k_pool, (TT*)v_pool, page_size, \
    nq, nkv, hd, kv_flags, T_, blocks_per_token, heads_per_thread)
    if (dtype == ULLM_F32) GOV(float);
    else if (dtype == ULLM_BF16) GOV(bf16_t);
    else return ULLM_ERR_DTYPE;
#undef GOV
    ULLM_LAUNCH_CHECK();
  }
  dim3 grid(T_, nq + 2 * nkv), block(WAVE);
#define GO(TT) hipLaunchKernelGGL(qk_norm_rope_write_kernel<TT>, grid, block, 0, stream, \
    (const TT*)qkv, qkv_stride, (TT*)q_out, q_out_stride, q_gain, k_gain, eps, cos_sin, table_rows, \
    rot, style, positions, token_entry, block_table, bt_stride, (TT*)k_pool, (TT*)v_pool, page_size, \
    nq, nkv, hd, write_kv)
  if (dtype == ULLM_F32) GO(float);
  else if (dtype == ULLM_BF16) GO(bf16_t);
  else return ULLM_ERR_DTYPE;
#undef GO
  ULLM_LAUNCH_CHECK();
}
