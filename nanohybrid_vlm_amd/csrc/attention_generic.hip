// Attention over the paged cache for any head size, page size, number of heads
// and groups, in float or bfloat16 (float scores, running maximum, sum and output).
// One wave per (token, query head): prompt portions and single decoded tokens are
// the same case. The query at position p of request r reads the keys at positions
// lo..p, lo = max(0, p - window + 1) (window 0: lo = 0), of r's block table.
// Keys are taken in blocks of 64 aligned to absolute positions, always in rising
// order, so the result for a position does not depend on the batch or the portion.
// This is the attention of the 32-bit path and the fallback of the bfloat16 path.
#include "nhv_common.h"
#include <math.h>

#define MAX_D_CHUNKS 8   // head sizes up to 512

template <typename T>
__global__ __launch_bounds__(256) void paged_attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache, T* __restrict__ out,
    const int* __restrict__ token_req, const int* __restrict__ positions, const int* __restrict__ block_tables,
    int max_blocks, int n_items, int Hq, int Hkv, int D, int page_size, float scale, int window) {
  extern __shared__ float q_s[];            // 4 waves x D floats
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave;
  const bool live = item < n_items;
  const int t = live ? item / Hq : 0;
  const int h = live ? item % Hq : 0;
  float* qs = q_s + wave * D;
  if (live)
    for (int d = lane; d < D; d += NHV_WAVE) qs[d] = to_f32(q[((size_t)t * Hq + h) * D + d]);
  __syncthreads();
  if (!live) return;

  const int pos = positions[t];
  const int req = token_req[t];
  const int kvh = h / (Hq / Hkv);
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int* bt = block_tables + (size_t)req * max_blocks;

  float m = -INFINITY, l = 0.f;
  float acc[MAX_D_CHUNKS];
#pragma unroll
  for (int i = 0; i < MAX_D_CHUNKS; ++i) acc[i] = 0.f;

  for (int kb = (lo / 64) * 64; kb <= pos; kb += 64) {
    const int kp = kb + lane;
    const bool valid = kp >= lo && kp <= pos;
    float s = -INFINITY;
    int slot = 0;
    if (valid) {
      const int page = bt[kp / page_size];
      slot = page * page_size + kp % page_size;
      const T* kr = k_cache + ((size_t)slot * Hkv + kvh) * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot = fmaf(qs[d], to_f32(kr[d]), dot);
      s = dot * scale;
    }
    const float m_new = fmaxf(m, wave_max(s));     // finite: every block holds at least one visible key
    const float alpha = expf(m - m_new);           // 0 on the first block
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < MAX_D_CHUNKS; ++i) acc[i] *= alpha;
    const int n_here = min(64, pos - kb + 1);
    for (int j = 0; j < n_here; ++j) {
      const float pj = __shfl(p, j, NHV_WAVE);
      const int sj = __shfl(slot, j, NHV_WAVE);
      if (pj == 0.f) continue;                     // same for the whole wave; also skips keys before the window
      const T* vr = v_cache + ((size_t)sj * Hkv + kvh) * D;
#pragma unroll
      for (int i = 0; i < MAX_D_CHUNKS; ++i) {
        const int d = lane + i * NHV_WAVE;
        if (d < D) acc[i] = fmaf(pj, to_f32(vr[d]), acc[i]);
      }
    }
  }
  const float inv = 1.0f / l;
  T* o = out + ((size_t)t * Hq + h) * D;
#pragma unroll
  for (int i = 0; i < MAX_D_CHUNKS; ++i) {
    const int d = lane + i * NHV_WAVE;
    if (d < D) o[d] = from_f32<T>(acc[i] * inv);
  }
}

extern "C" int nhv_paged_attention_generic(const void* q, const void* k_cache, const void* v_cache, void* out,
                                           const void* token_req, const void* positions, const void* block_tables,
                                           int max_blocks, int T, int Hq, int Hkv, int D, int page_size, float scale,
                                           int window, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && Hq > 0 && Hkv > 0 && D > 0 && page_size > 0 && max_blocks > 0,
              "attention: bad sizes T=%d Hq=%d Hkv=%d D=%d page=%d blocks=%d", T, Hq, Hkv, D, page_size, max_blocks);
  NHV_REQUIRE(Hq % Hkv == 0, "attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  NHV_REQUIRE(D <= 64 * MAX_D_CHUNKS, "attention: head size %d is beyond this kernel's limit of %d", D, 64 * MAX_D_CHUNKS);
  NHV_REQUIRE(window >= 0, "attention: negative window");
  const long long n_items = (long long)T * Hq;
  NHV_REQUIRE(n_items < (1ll << 31), "attention: too many (token, head) pairs");
  const unsigned blocks = (unsigned)((n_items + 3) / 4);
  const size_t lds = 4 * (size_t)D * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, dim3(blocks), dim3(256), lds, s, (const float*)q,
                       (const float*)k_cache, (const float*)v_cache, (float*)out, (const int*)token_req,
                       (const int*)positions, (const int*)block_tables, max_blocks, (int)n_items, Hq, Hkv, D, page_size,
                       scale, window);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, dim3(blocks), dim3(256), lds, s, (const bf16_t*)q,
                       (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, (const int*)token_req,
                       (const int*)positions, (const int*)block_tables, max_blocks, (int)n_items, Hq, Hkv, D, page_size,
                       scale, window);
  else
    return nhv_fail("attention: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("paged_attention_generic");
  return 0;
}
