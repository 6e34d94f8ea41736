// Shared device helpers for the gfx950 kernels: element types, conversions, wave reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define QVL_WAVE 64

// Error codes returned by the extern "C" launchers (0 = launched).
#define QVL_OK 0
#define QVL_ERR_SHAPE 1
#define QVL_ERR_DTYPE 2
#define QVL_ERR_LAUNCH 3
#define QVL_ERR_LIMIT 4

typedef uint16_t bf16_t;  // bfloat16 as its bit pattern

__device__ __forceinline__ float bf16_to_f32(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// Round to nearest even; NaN stays NaN.
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (bf16_t)((u >> 16) | 0x40u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (bf16_t)(u >> 16);
}

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <> __device__ __forceinline__ float ldf<bf16_t>(const bf16_t* p) { return bf16_to_f32(*p); }

template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void stf<bf16_t>(bf16_t* p, float v) { *p = f32_to_bf16(v); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, QVL_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, QVL_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the total.  `red` holds 17 floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nwaves = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int i = 0; i < nwaves; ++i) t += red[i];
    red[16] = t;
  }
  __syncthreads();
  return red[16];
}

static inline int qvl_launch_status() { return hipGetLastError() == hipSuccess ? QVL_OK : QVL_ERR_LAUNCH; }
