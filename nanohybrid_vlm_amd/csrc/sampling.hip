// Sampling of one token per row of float logits [n, V].
// temperature 0: the first index of the largest logit. Otherwise
// argmax_i softmax(logits / T)_i / e_i with e_i ~ Exp(1), which draws i with
// probability softmax_i. The noise is a function of (key[row], i) only, so what a
// request samples does not depend on its batch mates.
// Greedy rows are cut into pieces of 4096 logits, one block each (a row of a large
// vocabulary read by one block alone takes ten times as long); a second kernel picks
// among the pieces' winners and does the rows with a temperature, one block a row.
#include "nhv_common.h"
#include <math.h>

__device__ __forceinline__ uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

// Exp(1) noise from 24 random bits: -log(u) with u the middle of the bits' bucket, (bits + 0.5) / 2^24, so that
// the smallest value, 3e-8, is the mean of what a true Exp(1) draw puts into the lowest bucket. (With u = (bits
// + 1) / 2^24 the top pattern gave u = 1 and a noise of 0, held at 1e-10: once in 2^24 draws an index's chance was
// multiplied by 10^10 where 3 * 10^7 is right, and with 150,000 indices a row that is one draw in a hundred.)
// Both halves of the range are computed from numbers that float holds exactly: bits + 0.5 below 2^23, and
// 1 - u = (2^24 - bits - 0.5) / 2^24 above, through log1p. The floor of 1e-10 is the reference's
// (nanovllm/layers/sampler.py:52) and is never met.
__device__ __forceinline__ float exp1_noise_of_bits(uint32_t bits) {
  float e;
  if (bits < (1u << 23)) e = -logf(((float)bits + 0.5f) * (1.0f / 16777216.0f));
  else e = -log1pf(-((float)(16777216u - bits) - 0.5f) * (1.0f / 16777216.0f));
  return fmaxf(e, 1e-10f);
}
__device__ __forceinline__ float exp1_noise(uint64_t key, int i) {
  return exp1_noise_of_bits((uint32_t)(mix64(key ^ (uint64_t)i) >> 40));   // 24 bits
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

constexpr int PIECE = 4096;                 // logits per block of the first kernel

// the best of one piece of a greedy row; rows with a temperature are left to the second kernel
__global__ __launch_bounds__(256) void greedy_pieces_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                                                            float* __restrict__ piece_value, int* __restrict__ piece_index, int V,
                                                            int pieces) {
  __shared__ Best bscratch[16];
  const int r = blockIdx.y, c = blockIdx.x;
  if (temperatures[r] > 0.f) return;
  const float* row = logits + (size_t)r * V;
  const int lo = c * PIECE, hi = min(V, lo + PIECE);
  Best best{-INFINITY, 0x7fffffff};
  if ((((uintptr_t)row) & 15) == 0 && (V & 3) == 0) {
    for (int i = lo + threadIdx.x * 4; i < hi; i += 256 * 4) {       // hi - lo and lo are multiples of 4
      const float4 v = *reinterpret_cast<const float4*>(row + i);
      best = better(best, Best{v.x, i});
      best = better(best, Best{v.y, i + 1});
      best = better(best, Best{v.z, i + 2});
      best = better(best, Best{v.w, i + 3});
    }
  } else {
    for (int i = lo + threadIdx.x; i < hi; i += 256) best = better(best, Best{row[i], i});
  }
  best = block_best(best, bscratch);
  if (threadIdx.x == 0) {
    piece_value[(size_t)r * pieces + c] = best.v;
    piece_index[(size_t)r * pieces + c] = best.i;
  }
}

__global__ __launch_bounds__(1024) void sample_kernel(const float* __restrict__ logits, const float* __restrict__ temperatures,
                                                      const uint64_t* __restrict__ keys, int* __restrict__ tokens, int V,
                                                      const float* __restrict__ piece_value,
                                                      const int* __restrict__ piece_index, int pieces) {
  __shared__ float fscratch[16];
  __shared__ Best bscratch[16];
  const float* row = logits + (size_t)blockIdx.x * V;
  const float temp = temperatures[blockIdx.x];
  Best best{-INFINITY, 0x7fffffff};
  if (temp <= 0.f) {
    for (int c = threadIdx.x; c < pieces; c += blockDim.x)
      best = better(best, Best{piece_value[(size_t)blockIdx.x * pieces + c], piece_index[(size_t)blockIdx.x * pieces + c]});
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

__global__ void noise_of_bits_kernel(const uint32_t* __restrict__ bits, float* __restrict__ out, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) out[i] = exp1_noise_of_bits(bits[i] & 0xFFFFFFu);
}

// the noise that each of n 24-bit patterns gives (for tests of the noise's distribution)
extern "C" int nhv_noise_of_bits(const void* bits, void* out, int n, void* stream) {
  NHV_REQUIRE(n > 0, "noise_of_bits: bad size n=%d", n);
  hipLaunchKernelGGL(noise_of_bits_kernel, dim3((n + 255) / 256), dim3(256), 0, (hipStream_t)stream,
                     (const uint32_t*)bits, (float*)out, n);
  NHV_LAUNCH_CHECK("noise_of_bits");
  return 0;
}

// how many floats (and as many ints) of scratch nhv_sample needs for n rows of V logits
extern "C" int nhv_sample_pieces(int V) { return (V + PIECE - 1) / PIECE; }

// piece_value: float [n, nhv_sample_pieces(V)], piece_index: int of the same shape: scratch of this call
extern "C" int nhv_sample(const void* logits, const void* temperatures, const void* keys, void* tokens, int n, int V,
                          void* piece_value, void* piece_index, void* stream) {
  NHV_REQUIRE(n > 0 && V > 0, "sample: bad sizes n=%d V=%d", n, V);
  NHV_REQUIRE(n <= 65535, "sample: %d rows are beyond this kernel's limit of 65535", n);
  NHV_REQUIRE(piece_value && piece_index, "sample: no scratch");
  const int pieces = (V + PIECE - 1) / PIECE;
  hipLaunchKernelGGL(greedy_pieces_kernel, dim3(pieces, n), dim3(256), 0, (hipStream_t)stream, (const float*)logits,
                     (const float*)temperatures, (float*)piece_value, (int*)piece_index, V, pieces);
  NHV_LAUNCH_CHECK("sample (pieces)");
  const int threads = V >= 4096 ? 1024 : 256;
  hipLaunchKernelGGL(sample_kernel, dim3(n), dim3(threads), 0, (hipStream_t)stream, (const float*)logits,
                     (const float*)temperatures, (const uint64_t*)keys, (int*)tokens, V, (const float*)piece_value,
                     (const int*)piece_index, pieces);
  NHV_LAUNCH_CHECK("sample");
  return 0;
}
