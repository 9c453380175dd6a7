// What the memory gives: a kernel that only reads, for measurements of the bandwidth that the other kernels'
// rates are compared with. Every wave reads one contiguous range, sixteen 16-byte loads a lane in flight.
#include "nhv_common.h"

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__global__ __launch_bounds__(256) void read_ranges_kernel(const floatx4* __restrict__ data, float* __restrict__ sink, size_t chunks) {
  constexpr int IN_FLIGHT = 16;
  const int lane = threadIdx.x & 63;
  const size_t wave = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const size_t nwaves = (size_t)gridDim.x * (blockDim.x >> 6);
  const size_t per = (chunks + nwaves - 1) / nwaves;
  const size_t c0 = wave * per, c1 = c0 + per < chunks ? c0 + per : chunks;
  floatx4 acc = floatx4{0.f, 0.f, 0.f, 0.f};
  for (size_t c = c0; c < c1; c += IN_FLIGHT) {
    floatx4 v[IN_FLIGHT];
#pragma unroll
    for (int u = 0; u < IN_FLIGHT; ++u) v[u] = c + u < c1 ? data[(c + u) * 64 + lane] : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < IN_FLIGHT; ++u) acc += v[u];
  }
  // (the sum is used, so the loads stay; the value it is compared with does not occur)
  if (acc[0] + acc[1] + acc[2] + acc[3] == 12345.678f) sink[0] = 1.f;
}

// Reads `bytes` bytes (a multiple of 1024, 16-byte aligned) once. `sink`: one float that may be written.
extern "C" int nhv_measure_read(const void* data, void* sink, size_t bytes, void* stream) {
  NHV_REQUIRE(data && sink && bytes >= 1024 && bytes % 1024 == 0, "measure_read: %zu bytes (a multiple of 1024 is needed)", bytes);
  NHV_REQUIRE((uintptr_t)data % 16 == 0, "measure_read: the data must be 16-byte aligned");
  hipLaunchKernelGGL(read_ranges_kernel, dim3(2048), dim3(256), 0, (hipStream_t)stream, (const floatx4*)data, (float*)sink,
                     bytes / 1024);
  NHV_LAUNCH_CHECK("measure_read");
  return 0;
}
