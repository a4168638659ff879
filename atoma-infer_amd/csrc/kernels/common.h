// Shared device helpers for the gfx950 kernels: bfloat16 bit conversions, wave and block reductions,
// element-type dispatch.  Wavefronts are 64 lanes wide throughout.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace atoma {

constexpr int kWave = 64;

// bfloat16 is carried as its 16 raw bits.
struct bf16_t {
  uint16_t bits;
};

__device__ __host__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
  union { uint32_t u; float f; } v;
  v.u = ((uint32_t)b) << 16;
  return v.f;
}

// round to nearest, ties to even; NaN stays NaN
__device__ __host__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {
  union { uint32_t u; float f; } v;
  v.f = f;
  if ((v.u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((v.u >> 16) | 0x0040u);
  uint32_t lsb = (v.u >> 16) & 1u;
  v.u += 0x7fffu + lsb;
  return (uint16_t)(v.u >> 16);
}

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16_t v) { return bf16_bits_to_f32(v.bits); }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_f32<bf16_t>(float v) {
  bf16_t r;
  r.bits = f32_to_bf16_bits(v);
  return r;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of NWAVES*64 threads; every thread gets the result.  `scratch` holds NWAVES floats.
template <int NWAVES> __device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NWAVES; ++i) t += scratch[i];
  return t;
}

template <int NWAVES> __device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  if (NWAVES == 1) return v;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float t = scratch[0];
#pragma unroll
  for (int i = 1; i < NWAVES; ++i) t = fmaxf(t, scratch[i]);
  return t;
}

// Element type codes of the C interface.
enum DType : int { kF32 = 0, kBF16 = 1 };

}  // namespace atoma

// Error codes of the C interface beyond hipError_t values (which are positive): negative numbers.
#define ATOMA_ERR_DTYPE (-2)
#define ATOMA_ERR_SHAPE (-3)

#define ATOMA_LAUNCH_CHECK()                     \
  do {                                           \
    hipError_t e__ = hipGetLastError();          \
    if (e__ != hipSuccess) return (int)e__;      \
  } while (0)
