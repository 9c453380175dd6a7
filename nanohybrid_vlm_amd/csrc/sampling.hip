// Sampling of one token per row of float logits [n, V].
// temperature 0: the first index of the largest logit. Otherwise
// argmax_i softmax(logits / T)_i / e_i with e_i ~ Exp(1), which draws i with
// probability softmax_i. The noise is a function of (key[row], i) only, so what a
// request samples does not depend on its batch mates.
#include "nhv_common.h"
#include <math.h>

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__device__ __forceinline__ float exp1_noise(uint64_t key, int i) {
  const uint32_t bits = (uint32_t)(mix64(key ^ (uint64_t)i) >> 40);      // 24 bits
  const float u = (float)(bits + 1u) * (1.0f / 16777216.0f);             // (0, 1]
  return fmaxf(-logf(u), 1e-10f);
}

struct Best {
  float v;
  int i;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}
__device__ __forceinline__ Best block_best(Best b, Best* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    Best other{__shfl_xor(b.v, o, NHV_WAVE), __shfl_xor(b.i, o, NHV_WAVE)};
    b = better(b, other);
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = b;
  __syncthreads();
  Best r = scratch[0];
  for (int w = 1; w < nw; ++w) r = better(r, scratch[w]);
  return r;
}
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float r = scratch[0];
  for (int w = 1; w < nw; ++w) r = fmaxf(r, scratch[w]);
  return r;
}

__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                                                      const uint64_t* __restrict__ keys, int* __restrict__ tokens, int V) {
  __shared__ float fscratch[16];
  __shared__ Best bscratch[16];
  const float* row = logits + (size_t)blockIdx.x * V;
  const float temp = temperatures[blockIdx.x];
  Best best{-INFINITY, 0x7fffffff};
  if (temp <= 0.f) {
    for (int i = threadIdx.x; i < V; i += blockDim.x) best = better(best, Best{row[i], i});
  } else {
    float mx = -INFINITY;
    for (int i = threadIdx.x; i < V; i += blockDim.x) mx = fmaxf(mx, row[i] / temp);
    mx = block_max(mx, fscratch);
    float sum = 0.f;
    for (int i = threadIdx.x; i < V; i += blockDim.x) sum += expf(row[i] / temp - mx);
    sum = block_sum(sum, fscratch);
    const uint64_t key = keys[blockIdx.x];
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
      const float p = expf(row[i] / temp - mx) / sum;
      best = better(best, Best{p / exp1_noise(key, i), i});
    }
  }
  best = block_best(best, bscratch);
  if (threadIdx.x == 0) tokens[blockIdx.x] = best.i;
}

extern "C" int nhv_sample(const void* logits, const void* temperatures, const void* keys, void* tokens, int n, int V,
                          void* stream) {
  NHV_REQUIRE(n > 0 && V > 0, "sample: bad sizes n=%d V=%d", n, V);
  const int threads = V >= 4096 ? 1024 : 256;
  hipLaunchKernelGGL(sample_kernel, dim3(n), dim3(threads), 0, (hipStream_t)stream, (const float*)logits,
                     (const float*)temperatures, (const uint64_t*)keys, (int*)tokens, V);
  NHV_LAUNCH_CHECK("sample");
  return 0;
}
