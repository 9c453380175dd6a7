// Shared device helpers and the C interface's error channel (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef __bf16 bf16_t;

// element types of the C interface
enum { NHV_F32 = 0, NHV_BF16 = 1 };

#define NHV_WAVE 64

// Sets the message that nhv_last_error() returns; always returns 1.
int nhv_fail(const char* fmt, ...);

#define NHV_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) return nhv_fail(__VA_ARGS__); \
  } while (0)

#define NHV_LAUNCH_CHECK(name)                                             \
  do {                                                                     \
    hipError_t e_ = hipGetLastError();                                     \
    if (e_ != hipSuccess) return nhv_fail("%s: launch failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

template <typename T>
__device__ __forceinline__ float to_f32(T v) { return (float)v; }
template <typename T>
__device__ __forceinline__ T from_f32(float v) { return (T)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, NHV_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, NHV_WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// The order of the additions depends on the block size only.
__device__ __forceinline__ float block_sum(float v, float* scratch /* >= 16 floats */) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int nwaves = (blockDim.x + 63) >> 6;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < nwaves; ++i) total += scratch[i];
  return total;
}
