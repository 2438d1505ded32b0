// Shared helpers of the gfx950 kernels: storage types, 32-bit conversion, wave and block
// reductions with a fixed order (so a row's result never depends on what else is in the batch).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef uint16_t bf16_t;  // bfloat16 as raw bits; all arithmetic is done in float

enum { ULLM_F32 = 0, ULLM_BF16 = 1 };

// error codes of the extern "C" launchers (0 = ok, >0 = hipError_t of the launch)
enum { ULLM_ERR_DTYPE = -1, ULLM_ERR_SHAPE = -2, ULLM_ERR_UNSUPPORTED = -3 };

#define WAVE 64

__device__ __forceinline__ float bf16_bits_to_f32(bf16_t v) {
  return __uint_as_float(((uint32_t)v) << 16);
}

// round to nearest even; NaN stays NaN.  gfx950 converts in hardware (v_cvt_pk_bf16_f32).
__device__ __forceinline__ bf16_t f32_to_bf16_bits(float f) {
  return __builtin_bit_cast(bf16_t, (__bf16)f);
}
typedef __attribute__((ext_vector_type(2))) float ullm_f32x2;
typedef __attribute__((ext_vector_type(2))) __bf16 ullm_bf16x2;
// two values in one instruction: low half = a, high half = b
__device__ __forceinline__ uint32_t pack2_bf16(float a, float b) {
  const ullm_f32x2 v = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, ullm_bf16x2));
}
// silu with the hardware exponential and reciprocal (about 1 ulp each); for results that are rounded
// to bfloat16 afterwards
__device__ __forceinline__ float fast_silu(float g) {
  return g * __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(-1.4426950408889634f * g));
}

__device__ __forceinline__ float ld_f32(const float* p) { return *p; }
__device__ __forceinline__ float ld_f32(const bf16_t* p) { return bf16_bits_to_f32(*p); }
__device__ __forceinline__ void st_f32(float* p, float v) { *p = v; }
__device__ __forceinline__ void st_f32(bf16_t* p, float v) { *p = f32_to_bf16_bits(v); }

// 16 bytes that are read once (a weight matrix streamed through a product): the load carries the
// non-temporal hint, so the lines do not displace what the caches hold for reuse.
__device__ __forceinline__ uint4 ld_stream16(const void* p) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(v.x, v.y, v.z, v.w);
}

// 16 bytes as one vector load / store.  (Copying a uint4 through a cast pointer is a memcpy to the compiler,
// which can keep registers that hold loads in flight in scratch memory; a native vector type is a plain load.)
__device__ __forceinline__ uint4 ld16(const void* p) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 v = *reinterpret_cast<const u32x4*>(p);
  return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ void st16(void* p, const uint4& v) {
  typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;
  const u32x4 t = {v.x, v.y, v.z, v.w};
  *reinterpret_cast<u32x4*>(p) = t;
}

__device__ __forceinline__ uint2 ld_stream8(const void* p) {
  typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
  const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
  return make_uint2(v.x, v.y);
}

// max(v, v of the lane 16 (32) further on or back): the two values change places between rows of 16 (32) lanes
// inside the vector unit (v_permlane16_swap / v_permlane32_swap), without a trip through the LDS crossbar that
// a general lane permutation takes.
__device__ __forceinline__ float max_with_lane_xor16(float v) {
#ifdef __HIP_DEVICE_COMPILE__
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
#else
  return v;
#endif
}
__device__ __forceinline__ float max_with_lane_xor32(float v) {
#ifdef __HIP_DEVICE_COMPILE__
  const unsigned u = __float_as_uint(v);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
#else
  return v;
#endif
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) v += __shfl_xor(v, m, WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int m = WAVE / 2; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, WAVE));
  return v;
}

// Block reductions over up to 1024 threads (16 waves); every thread gets the result.
// `scratch` must hold 16 floats of shared memory; the caller may reuse it after the call.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = 0.f;
  for (int w = 0; w < nwaves; ++w) r += scratch[w];
  return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1), wave = threadIdx.x / WAVE;
  const int nwaves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_max(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < nwaves; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

#define ULLM_LAUNCH_CHECK() return (int)hipGetLastError()
