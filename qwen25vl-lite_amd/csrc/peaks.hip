// What this device does at best, measured with the plainest kernels there are: the rates that the
// benchmark's fractions of the published peaks should be read against.
//   read     every thread adds up 16-byte loads of a large buffer (a stream of reads, nothing else)
//   copy     16-byte loads stored elsewhere (reads and writes in equal parts)
//   mfma     v_mfma_f32_16x16x32_bf16 back to back on registers, several independent chains a wave
//   empty    a kernel that does nothing: launched many times in a row it shows what a launch costs
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void peak_read_kernel(const u32x4_t* __restrict__ src, size_t n, uint32_t* __restrict__ out) {
  u32x4_t acc = {0u, 0u, 0u, 0u};
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  for (; i + 3 * stride < n; i += 4 * stride) {   // four loads on their way per thread
    const u32x4_t a = src[i], b = src[i + stride], c = src[i + 2 * stride], d = src[i + 3 * stride];
    acc ^= a ^ b ^ c ^ d;
  }
  for (; i < n; i += stride) acc ^= src[i];
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) out[0] = 1;   // keeps the loads alive
}

// Every block reads all n units (16 bytes each) of a small buffer `reps` times: what the L2 caches deliver
// when everything is found there.
__global__ __launch_bounds__(256) void peak_read_again_kernel(const u32x4_t* __restrict__ src, size_t n, int reps,
                                                              uint32_t* __restrict__ out) {
  u32x4_t acc = {0u, 0u, 0u, 0u};
  for (int r = 0; r < reps; ++r) {
    // blocks start at different places, so that they do not all ask for the same line at once
    size_t i = ((size_t)blockIdx.x * 977 * 256 + threadIdx.x) % n;
    for (size_t done = 0; done + 4 * 256 <= n; done += 4 * 256) {
      const u32x4_t a = src[i], b = src[(i + 256) % n], c = src[(i + 512) % n], d = src[(i + 768) % n];
      acc ^= a ^ b ^ c ^ d;
      i = (i + 1024) % n;
    }
  }
  if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x9e3779b9u) out[0] = 1;
}

__global__ __launch_bounds__(256) void peak_copy_kernel(const u32x4_t* __restrict__ src, u32x4_t* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) dst[i] = src[i];
}

// clocks (may be null): per block, what its first wave's loop took on the shader's own cycle counter
// and on the device's constant 100 MHz clock: their ratio is the clock the shader really ran at, and
// the cycles divided by the instructions a SIMD issued meanwhile say whether a slow rate is a slow
// clock or an instruction that cannot be issued faster.
template <int THREADS>
__global__ __launch_bounds__(THREADS) void peak_mfma_kernel(float* __restrict__ out, int iters,
                                                            unsigned long long* __restrict__ clocks) {
  const u32x4_t one = {0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u};
  const bf16x8_t a = __builtin_bit_cast(bf16x8_t, one), b = a;
  f32x4_t acc[8];
#pragma unroll
  for (int c = 0; c < 8; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const unsigned long long cycles0 = __builtin_readcyclecounter(), wall0 = __builtin_amdgcn_s_memrealtime();
  for (int i = 0; i < iters; ++i) {
#pragma unroll
    for (int c = 0; c < 8; ++c) acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[c], 0, 0, 0);
  }
  asm volatile("s_nop 0" ::"v"(acc[7]));   // the last product has been issued before the clocks are read again
  const unsigned long long cycles1 = __builtin_readcyclecounter(), wall1 = __builtin_amdgcn_s_memrealtime();
  if (clocks && threadIdx.x == 0) {
    clocks[2 * blockIdx.x] = cycles1 - cycles0;
    clocks[2 * blockIdx.x + 1] = wall1 - wall0;
  }
  float s = 0.f;
#pragma unroll
  for (int c = 0; c < 8; ++c) s += acc[c][0] + acc[c][1] + acc[c][2] + acc[c][3];
  if (s == -1.f) out[0] = s;
}

__global__ void peak_empty_kernel() {}

// n: 16-byte units.  blocks: how many blocks of 256 threads.
extern "C" int qvl_peak_read(const void* src, long long n, void* out, int blocks, hipStream_t stream) {
  if (n <= 0 || blocks <= 0) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(peak_read_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)src, (size_t)n, (uint32_t*)out);
  return qvl_launch_status();
}
extern "C" int qvl_peak_read_again(const void* src, long long n, int reps, void* out, int blocks, hipStream_t stream) {
  if (n < 1024 || n % 1024 || reps <= 0 || blocks <= 0) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(peak_read_again_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)src, (size_t)n, reps,
                     (uint32_t*)out);
  return qvl_launch_status();
}
extern "C" int qvl_peak_copy(const void* src, void* dst, long long n, int blocks, hipStream_t stream) {
  if (n <= 0 || blocks <= 0) return QVL_ERR_SHAPE;
  hipLaunchKernelGGL(peak_copy_kernel, dim3(blocks), dim3(256), 0, stream, (const u32x4_t*)src, (u32x4_t*)dst, (size_t)n);
  return qvl_launch_status();
}
// Every wave runs iters * 8 products of 16 x 16 x 32 (2 * 16 * 16 * 32 flops each).
// clocks: null, or 2 * blocks 64-bit counts (see the kernel).  threads: 256 (a wave on each SIMD of
// a compute unit), 512 or 1024 (two or four): the waves of a block are resident together, which
// blocks of a grid larger than the device are not.
extern "C" int qvl_peak_mfma(void* out, int iters, int blocks, int threads, void* clocks, hipStream_t stream) {
  if (iters <= 0 || blocks <= 0) return QVL_ERR_SHAPE;
  unsigned long long* c = (unsigned long long*)clocks;
  if (threads == 256) hipLaunchKernelGGL(peak_mfma_kernel<256>, dim3(blocks), dim3(256), 0, stream, (float*)out, iters, c);
  else if (threads == 512) hipLaunchKernelGGL(peak_mfma_kernel<512>, dim3(blocks), dim3(512), 0, stream, (float*)out, iters, c);
  else if (threads == 1024) hipLaunchKernelGGL(peak_mfma_kernel<1024>, dim3(blocks), dim3(1024), 0, stream, (float*)out, iters, c);
  else return QVL_ERR_SHAPE;
  return qvl_launch_status();
}
extern "C" int qvl_peak_empty(int count, hipStream_t stream) {
  for (int i = 0; i < count; ++i) hipLaunchKernelGGL(peak_empty_kernel, dim3(1), dim3(64), 0, stream);
  return qvl_launch_status();
}
