// Attention of single tokens over the paged cache in bfloat16, split over the keys.
// Compiled for one head size: -DNHV_HEAD_DIM=<multiple of 16>.
//
// One wave works on (token, key/value head, split of the keys). The G query heads
// that share the key/value head (G <= 16) are the 16 columns of an MFMA tile:
//   S^T[key, head] = K[key, :] . Q[head, :]   v_mfma_f32_16x16x32_bf16, K rows straight from the cache
// so every lane ends up with four consecutive keys of one head and the running
// maximum needs two shuffles. The probabilities go through LDS to the second half,
// which is plain FMA work: with one token per request the values are read once and
// used by only G heads, so the step is bound by the cache's bandwidth, not by math.
//   O[head, d] += P[head, key] * V[key, d]    lanes own 8 consecutive d of every 64/LPK-th key
// Splits are aligned to absolute key positions. Each split writes its unnormalised
// output with (maximum, sum) in float; a second kernel merges the splits in rising
// order. Keys that are not visible are loaded as zeros (the cache's unused slots
// may hold anything).
#include "nhv_common.h"
#include <math.h>

#ifndef NHV_HEAD_DIM
#error "compile with -DNHV_HEAD_DIM=<head size>"
#endif

constexpr int D = NHV_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 512, "head size must be a multiple of 16 up to 512");
constexpr int DSTEPS = (D + 31) / 32;                       // MFMA steps over the head
constexpr int CHUNKS = D / 8;                               // 16-byte pieces of a row
constexpr int LPK = CHUNKS <= 2 ? 2 : CHUNKS <= 4 ? 4 : CHUNKS <= 8 ? 8 : CHUNKS <= 16 ? 16 : CHUNKS <= 32 ? 32 : 64;
constexpr int KPP = 64 / LPK;                               // keys per pass of the value half
constexpr int RK = 64;                                      // keys per round
constexpr int KT = RK / 16;                                 // MFMA tiles of 16 keys per round
constexpr int PASSES = RK / KPP;                            // passes of the value half per round

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// key position -> slot in the cache; pages whose size is a power of two need no division
__device__ __forceinline__ int slot_of(const int* bt, int key, int page_size, int page_shift) {
  if (page_shift >= 0) return (bt[key >> page_shift] << page_shift) + (key & (page_size - 1));
  return bt[key / page_size] * page_size + key % page_size;
}

template <int GC>
__global__ __launch_bounds__(64) void decode_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    float* __restrict__ part_o, float* __restrict__ part_ml, const int* __restrict__ token_req,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks, int Hq, int Hkv,
    int page_size, int page_shift, float scale, int window, int split_len, int n_splits) {
  __shared__ __attribute__((aligned(16))) float p_s[RK][20];          // [key][head], rows of 16-byte pieces
  __shared__ float alpha_s[16];
  const int lane = threadIdx.x;
  const int split = blockIdx.x, kvh = blockIdx.y, t = blockIdx.z;
  const int G = Hq / Hkv;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int first = max(lo, split * split_len);
  const int last = min(pos, (split + 1) * split_len - 1);
  if (first > last) return;              // this split holds no visible key; the merge knows from pos and lo
  const int* bt = block_tables + (size_t)token_req[t] * max_blocks;
  const int col = lane & 15, grp = lane >> 4;

  // Q^T operand: lane holds 8 entries of head `col`
  bf16x8 qb[DSTEPS];
#pragma unroll
  for (int s = 0; s < DSTEPS; ++s) {
    const int d = s * 32 + grp * 8;
    qb[s] = (col < G && d < D) ? load8(q + ((size_t)t * Hq + kvh * G + col) * D + d) : zero8();
  }

  float m_run = -INFINITY, l_part = 0.f;     // per head `col`; l_part is this lane's share of the sum
  float acc[GC][8];
#pragma unroll
  for (int g = 0; g < GC; ++g)
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[g][e] = 0.f;
  const int ksub = lane / LPK, chunk = lane % LPK;
  const bool chunk_live = chunk * 8 < D;

  for (int kb = (first / RK) * RK; kb <= last; kb += RK) {
    // ---- all keys and values of the round are asked for before anything is computed: 64 keys, 32 KB a wave
    // (pages that are a power of two of at least 64 tokens hold a whole round: one look at the block table)
    const bool one_page = page_shift >= 6;
    const int round_base = one_page ? (bt[kb >> page_shift] << page_shift) : 0;
    bf16x8 ka[KT][DSTEPS];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      const int key = kb + kt * 16 + col;
      const bool ok = key >= first && key <= last;
      int slot = 0;
      if (ok) slot = one_page ? round_base + (key & (page_size - 1)) : slot_of(bt, key, page_size, page_shift);
      const bf16_t* krow = k_cache + ((size_t)slot * Hkv + kvh) * D;
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) {
        const int d = s * 32 + grp * 8;
        ka[kt][s] = (ok && d < D) ? load8(krow + d) : zero8();
      }
    }
    bf16x8 vv[PASSES];
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int key = kb + ps * KPP + ksub;
      const bool ok = chunk_live && key >= first && key <= last;
      int slot = 0;
      if (ok) slot = one_page ? round_base + (key & (page_size - 1)) : slot_of(bt, key, page_size, page_shift);
      vv[ps] = ok ? load8(v_cache + ((size_t)slot * Hkv + kvh) * D + chunk * 8) : zero8();
    }
    // ---- scores
    floatx4 s4[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      s4[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) s4[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[kt][s], qb[s], s4[kt], 0, 0, 0);
    }
    // ---- running softmax for head `col` over keys kb + 16 kt + 4 grp + j
    float m_tile = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + kt * 16 + grp * 4 + j;
        const float v = (key >= first && key <= last) ? s4[kt][j] * scale : -INFINITY;
        s4[kt][j] = v;
        m_tile = fmaxf(m_tile, v);
      }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
    const float m_new = fmaxf(m_run, m_tile);          // finite: every round holds a visible key
    const float alpha = __expf(m_run - m_new);
    float psum = 0.f;
    __syncthreads();                                   // the last round's p_s and alpha_s have been read
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = __expf(s4[kt][j] - m_new);     // exp(-inf) = 0 for keys out of range
        p_s[kt * 16 + grp * 4 + j][col] = p;
        psum += p;
      }
    l_part = l_part * alpha + psum;
    m_run = m_new;
    if (grp == 0) alpha_s[col] = alpha;
    __syncthreads();
    // ---- O += P V
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      const float a = alpha_s[g];
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] *= a;
    }
#pragma unroll
    for (int ps = 0; ps < PASSES; ++ps) {
      const int kl = ps * KPP + ksub;
      float vf[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) vf[e] = (float)vv[ps][e];
      float pg[GC];
      if (GC >= 4) {
#pragma unroll
        for (int g4 = 0; g4 < GC / 4; ++g4) {
          const float4 p4 = *reinterpret_cast<const float4*>(&p_s[kl][g4 * 4]);
          pg[g4 * 4] = p4.x; pg[g4 * 4 + 1] = p4.y; pg[g4 * 4 + 2] = p4.z; pg[g4 * 4 + 3] = p4.w;
        }
      } else {
#pragma unroll
        for (int g = 0; g < GC; ++g) pg[g] = p_s[kl][g];
      }
#pragma unroll
      for (int g = 0; g < GC; ++g)
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[g][e] = fmaf(pg[g], vf[e], acc[g][e]);
    }
  }
  // ---- this split's result: sum over the lanes that hold other keys of the same chunk
#pragma unroll
  for (int off = LPK; off < 64; off <<= 1) {
#pragma unroll
    for (int g = 0; g < GC; ++g)
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[g][e] += __shfl_xor(acc[g][e], off, 64);
  }
  l_part += __shfl_xor(l_part, 16, 64);
  l_part += __shfl_xor(l_part, 32, 64);
  if (lane < 16 && lane < G) {
    float* ml = part_ml + (((size_t)t * Hq + kvh * G + lane) * n_splits + split) * 2;
    ml[0] = m_run;
    ml[1] = l_part;
  }
  if (ksub == 0 && chunk_live) {
#pragma unroll
    for (int g = 0; g < GC; ++g) {
      if (g < G) {
        float* o = part_o + (((size_t)t * Hq + kvh * G + g) * n_splits + split) * D + chunk * 8;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = acc[g][e];
      }
    }
  }
}

// Merges the splits of every (token, head): one wave each. The weights exp(m_s - M) are found with the lanes
// spread over the splits. For the outputs a lane owns four consecutive entries of the head and every
// (64 / lanes per row)-th split, with several loads in flight; the lanes' sums are then added across.
constexpr int MQ = D / 4;                                   // float4 pieces of a row
constexpr int MLPR = MQ <= 4 ? 4 : MQ <= 8 ? 8 : MQ <= 16 ? 16 : MQ <= 32 ? 32 : 64;   // lanes per row
constexpr int MROWS = 64 / MLPR;                            // splits worked on side by side
constexpr int MPIECES = (MQ + MLPR - 1) / MLPR;             // pieces per lane (more than 1 for heads above 256)

__global__ __launch_bounds__(64) void merge_splits_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                          bf16_t* __restrict__ out, const int* __restrict__ positions,
                                                          int window, int split_len, int n_splits, int Hq) {
  const int item = blockIdx.x;               // t * Hq + h
  const int lane = threadIdx.x;
  const int t = item / Hq;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int s0 = lo / split_len, s1 = pos / split_len;
  const float* ml = part_ml + (size_t)item * n_splits * 2;
  float m = -INFINITY;
  for (int s = s0 + lane; s <= s1; s += 64) m = fmaxf(m, ml[s * 2]);
  m = wave_max(m);
  float l = 0.f;
  for (int s = s0 + lane; s <= s1; s += 64) l += ml[s * 2 + 1] * expf(ml[s * 2] - m);
  l = wave_sum(l);
  const float inv = 1.0f / l;
  const float* po = part_o + (size_t)item * n_splits * D;
  const int sub = lane / MLPR, piece = lane % MLPR;
  float4 acc[MPIECES];
#pragma unroll
  for (int i = 0; i < MPIECES; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
  for (int s = s0 + sub; s <= s1; s += MROWS) {
    const float wgt = expf(ml[s * 2] - m);
#pragma unroll
    for (int i = 0; i < MPIECES; ++i) {
      const int qd = piece + i * MLPR;
      if (qd < MQ) {
        const float4 v = *reinterpret_cast<const float4*>(po + (size_t)s * D + qd * 4);
        acc[i].x += v.x * wgt; acc[i].y += v.y * wgt; acc[i].z += v.z * wgt; acc[i].w += v.w * wgt;
      }
    }
  }
#pragma unroll
  for (int off = MLPR; off < 64; off <<= 1) {
#pragma unroll
    for (int i = 0; i < MPIECES; ++i) {
      acc[i].x += __shfl_xor(acc[i].x, off, 64); acc[i].y += __shfl_xor(acc[i].y, off, 64);
      acc[i].z += __shfl_xor(acc[i].z, off, 64); acc[i].w += __shfl_xor(acc[i].w, off, 64);
    }
  }
  if (sub == 0) {
#pragma unroll
    for (int i = 0; i < MPIECES; ++i) {
      const int qd = piece + i * MLPR;
      if (qd < MQ) {
        bf16_t* o = out + (size_t)item * D + qd * 4;
        o[0] = (bf16_t)(acc[i].x * inv); o[1] = (bf16_t)(acc[i].y * inv);
        o[2] = (bf16_t)(acc[i].z * inv); o[3] = (bf16_t)(acc[i].w * inv);
      }
    }
  }
}

extern "C" int nhv_decode_attention_head_dim() { return D; }

// part_o: float [T, Hq, n_splits, D]; part_ml: float [T, Hq, n_splits, 2]; n_splits * split_len must cover
// every context length of the batch (max_context_len).
extern "C" int nhv_decode_attention_bf16(const void* q, const void* k_cache, const void* v_cache, void* out, void* part_o,
                                         void* part_ml, const void* token_req, const void* positions,
                                         const void* block_tables, int max_blocks, int T, int Hq, int Hkv, int page_size,
                                         float scale, int window, int split_len, int n_splits, void* stream) {
  NHV_REQUIRE(T > 0 && Hq > 0 && Hkv > 0 && page_size > 0 && max_blocks > 0, "decode attention: bad sizes");
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  NHV_REQUIRE(Hq % Hkv == 0, "decode attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  const int G = Hq / Hkv;
  NHV_REQUIRE(G <= 16, "decode attention: %d query heads per key head are beyond this kernel's limit of 16", G);
  NHV_REQUIRE(split_len > 0 && split_len % RK == 0, "decode attention: split length %d must be a multiple of %d", split_len, RK);
  NHV_REQUIRE(n_splits > 0 && n_splits <= 65535 && Hkv <= 65535 && T <= 65535, "decode attention: grid too large");
  NHV_REQUIRE(window >= 0, "decode attention: negative window");
  hipStream_t s = (hipStream_t)stream;
  dim3 grid(n_splits, Hkv, T);
#define LAUNCH(GC)                                                                                                    \
  hipLaunchKernelGGL(decode_attention_kernel<GC>, grid, dim3(64), 0, s, (const bf16_t*)q, (const bf16_t*)k_cache,     \
                     (const bf16_t*)v_cache, (float*)part_o, (float*)part_ml, (const int*)token_req,                  \
                     (const int*)positions, (const int*)block_tables, max_blocks, Hq, Hkv, page_size, page_shift, scale,   \
                     window, split_len, n_splits)
  if (G <= 1) LAUNCH(1);
  else if (G <= 2) LAUNCH(2);
  else if (G <= 4) LAUNCH(4);
  else if (G <= 8) LAUNCH(8);
  else LAUNCH(16);
#undef LAUNCH
  NHV_LAUNCH_CHECK("decode_attention");
  hipLaunchKernelGGL(merge_splits_kernel, dim3((unsigned)((size_t)T * Hq)), dim3(64), 0, s, (const float*)part_o,
                     (const float*)part_ml, (bf16_t*)out, (const int*)positions, window, split_len, n_splits, Hq);
  NHV_LAUNCH_CHECK("merge_splits");
  return 0;
}
