// Attention of single tokens over the paged cache in bfloat16, split over the keys.
// Compiled for one head size: -DNHV_HEAD_DIM=<multiple of 16>.
//
// One wave works on (token, key/value head, split of the keys). The G query heads
// that share the key/value head (G <= 16) are the 16 columns of the MFMA tiles:
//   S^T[key, head]  = K[key, :] . Q[head, :]        K rows straight from the cache (v_mfma_f32_16x16x32_bf16)
//   running maximum per head in float (two shuffles), sums kept per lane
//   O^T[d, head]   += V^T[d, key] . P^T[key, head]   V^T from the wave's own LDS tile, P in registers
// Keys are taken 32 a round; all keys and values of a round are asked for from memory
// before anything is computed. The values are written to LDS transposed (four keys,
// 8 bytes, at a time, columns XOR-ed against bank conflicts), which turns the second
// half from 64 x G x D multiply-adds on the vector lanes into 16 matrix instructions.
// The S^T tiles leave every lane with keys of one head in the order in which the second
// product sums them, so P never leaves the registers, and a lane's outputs belong to
// the head of its scores: rescaling needs no exchange. Splits are aligned to absolute
// key positions. Each split writes its unnormalised output with (maximum, sum) in
// float; a second kernel merges the splits in rising order. Keys that are not visible
// are loaded as zeros (the cache's unused slots may hold anything).
#include "nhv_common.h"
#include "nhv_no_alloc.h"
#include <math.h>
#include <mutex>

#ifndef NHV_HEAD_DIM
#error "compile with -DNHV_HEAD_DIM=<head size>"
#endif

constexpr int D = NHV_HEAD_DIM;
static_assert(D % 16 == 0 && D >= 16 && D <= 256, "head size must be a multiple of 16 up to 256");
constexpr int DSTEPS = (D + 31) / 32;                       // MFMA steps over the head in the first product
constexpr int DTILES = D / 16;                              // output tiles of the second product
constexpr int CHUNKS = D / 8;                               // 16-byte pieces of a row
constexpr int LPK = CHUNKS <= 2 ? 2 : CHUNKS <= 4 ? 4 : CHUNKS <= 8 ? 8 : CHUNKS <= 16 ? 16 : 32;   // lanes per key
constexpr int KPP = 64 / LPK;                               // keys per load instruction of the values
constexpr int RK = 32;                                      // keys per round (64 needs 238 registers: one wave per SIMD)
constexpr int KT = RK / 16;                                 // MFMA tiles of 16 keys per round
constexpr int PASSES = RK / KPP;                            // value loads per lane and round: consecutive keys
constexpr int KG = PASSES >= 4 ? 4 : PASSES;                // keys per transposed LDS write
constexpr int VPITCH = RK + 8;                              // elements per row of the V^T tile
constexpr int SWZ_MASK = RK / 4 - 1;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
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

__global__ __launch_bounds__(64) void decode_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    float* __restrict__ part_o, float* __restrict__ part_ml, const int* __restrict__ token_req,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int max_blocks, int Hq, int Hkv,
    int page_size, int page_shift, float scale_log2e, int window, int split_len, int n_splits) {
  __shared__ __attribute__((aligned(16))) bf16_t vt_s[D * VPITCH];
  const int lane = threadIdx.x;
  // blocks go to the eight XCDs in turn by their linear index: with the split as the slowest index every XCD
  // gets the same share of each split (the last splits of a request are short or empty: as the fastest index,
  // four splits a request put all the long ones on half of the chip, 141 us against 108 us at 64 requests)
  // and the key/value head turns with the token and the split: a head's keys are 2 D bytes out of every
  // 2 D Hkv bytes of a page, and an XCD that read one and the same head for every token took 4 to 5 % longer at
  // 32 and 64 requests (116 against 111 us at 64) than one whose blocks go over all heads
  const int t = blockIdx.y, split = blockIdx.z;
  const int kvh = (int)((blockIdx.x + blockIdx.y + blockIdx.z) % gridDim.x);
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

  float m_run = -INFINITY, l_part = 0.f;     // of head `col` (base 2); l_part is this lane's share of the sum
  floatx4 o[DTILES];                          // o[dt][j]: entry dt * 16 + 4 grp + j of head `col`
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int ksub = lane / LPK, chunk = lane % LPK;       // this lane loads piece `chunk` of keys ksub * PASSES + (0..PASSES)
  const bool chunk_live = chunk * 8 < D;

  for (int kb = (first / RK) * RK; kb <= last; kb += RK) {
    // ---- all keys and values of the round are asked for before anything is computed (16 KB a wave at head size 128)
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
      const int key = kb + ksub * PASSES + ps;
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
    // ---- values into LDS, transposed: row d, columns = keys of the round
    __syncthreads();                                   // the last round's tile has been read
    if (chunk_live) {
#pragma unroll
      for (int pg = 0; pg < PASSES / KG; ++pg) {
        const int key0 = ksub * PASSES + pg * KG;      // KG consecutive keys of this lane
        const int vcol = key0 ^ ((chunk & SWZ_MASK) << 2);
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          bf16_t* dst = vt_s + (chunk * 8 + e) * VPITCH + vcol;
          if (KG == 4) {
            bf16x4 four;
#pragma unroll
            for (int k4 = 0; k4 < 4; ++k4) four[k4] = vv[pg * KG + k4][e];
            *reinterpret_cast<bf16x4*>(dst) = four;
          } else {
#pragma unroll
            for (int k4 = 0; k4 < KG; ++k4) dst[k4] = vv[pg * KG + k4][e];
          }
        }
      }
    }
    // ---- running softmax for head `col` over keys kb + 16 kt + 4 grp + j
    float m_tile = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + kt * 16 + grp * 4 + j;
        const float v = (key >= first && key <= last) ? s4[kt][j] * scale_log2e : -INFINITY;
        s4[kt][j] = v;
        m_tile = fmaxf(m_tile, v);
      }
    // the maximum is a reference point only: it moves when some head has grown by more than 2^6 over it, which
    // shows in the lanes' own maxima; the head's maximum over its four lanes is only needed then
    const bool grow = __any(m_tile > m_run + 6.0f);
    if (grow) {
      m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
      m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
    }
    const float m_new = grow ? fmaxf(m_run, m_tile) : m_run;     // finite: every round holds a visible key
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    float psum = 0.f;
    bf16x8 pa[KT / 2];                                 // P of keys (32 a + 4 grp + j) and (32 a + 16 + 4 grp + j)
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = __builtin_amdgcn_exp2f(s4[kt][j] - m_new);   // 0 for keys out of range
        psum += p;
        pa[kt / 2][(kt % 2) * 4 + j] = (__bf16)p;
      }
    l_part = l_part * alpha + psum;
    m_run = m_new;
    __syncthreads();                                   // the tile is written
    // ---- O^T += V^T P^T
    // (the outputs are rescaled only when the reference has moved: a branch of the whole wave; written as a condition
    // inside the loop over the output tiles it became a multiply and a select for every output entry in every round)
    if (grow) {
      asm volatile("" ::: "memory");
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
        for (int j = 0; j < 4; ++j) o[dt][j] *= alpha;
    }
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
      const int drow = dt * 16 + col;
      const int swz = ((drow >> 3) & SWZ_MASK) << 2;
#pragma unroll
      for (int a = 0; a < KT / 2; ++a) {
        const bf16x4 lo4 = *reinterpret_cast<const bf16x4*>(vt_s + drow * VPITCH + ((a * 32 + grp * 4) ^ swz));
        const bf16x4 hi4 = *reinterpret_cast<const bf16x4*>(vt_s + drow * VPITCH + ((a * 32 + 16 + grp * 4) ^ swz));
        bf16x8 va;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          va[j] = lo4[j];
          va[4 + j] = hi4[j];
        }
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pa[a], o[dt], 0, 0, 0);
      }
    }
  }
  // ---- this split's result
  l_part += __shfl_xor(l_part, 16, 64);
  l_part += __shfl_xor(l_part, 32, 64);
  if (col < G) {
    const size_t item = ((size_t)t * Hq + kvh * G + col) * n_splits + split;
    if (grp == 0) {
      part_ml[item * 2] = m_run;
      part_ml[item * 2 + 1] = l_part;
    }
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt)
      *reinterpret_cast<float4*>(part_o + item * D + dt * 16 + grp * 4) = make_float4(o[dt][0], o[dt][1], o[dt][2], o[dt][3]);
  }
}

// Merges the splits of every (token, head): one wave each. The weights exp(m_s - M) are found with the lanes
// spread over the splits. For the outputs a lane owns four consecutive entries of the head and every
// (64 / lanes per row)-th split, with several loads in flight; the lanes' sums are then added across.
constexpr int MQ = D / 4;                                   // float4 pieces of a row
constexpr int MLPR = MQ <= 4 ? 4 : MQ <= 8 ? 8 : MQ <= 16 ? 16 : MQ <= 32 ? 32 : 64;   // lanes per row
constexpr int MROWS = 64 / MLPR;                            // splits worked on side by side
constexpr int MPIECES = (MQ + MLPR - 1) / MLPR;             // pieces per lane (more than 1 for heads above 256)

// W: waves per (token, head); with many splits and few tokens (one request, 30,000 keys: 235 splits) a single
// wave's chain of loads is what the merge takes; four waves take every fourth pair of splits and add up through LDS.
template <int W>
__global__ __launch_bounds__(64 * W) void merge_splits_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                                              bf16_t* __restrict__ out, const int* __restrict__ positions,
                                                              int window, int split_len, int n_splits, int Hq) {
  __shared__ float4 sum_s[W > 1 ? W - 1 : 1][MPIECES][64];
  const int item = blockIdx.x;               // t * Hq + h
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t = item / Hq;
  const int pos = positions[t];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  // (the launch's splits must cover every position; one that they do not cover loses its last keys here rather
  // than reading past the splits' results)
  const int s0 = lo / split_len, s1 = min(pos / split_len, n_splits - 1);
  const float* ml = part_ml + (size_t)item * n_splits * 2;
  float m = -INFINITY;
  for (int s = s0 + lane; s <= s1; s += 64) m = fmaxf(m, ml[s * 2]);
  m = wave_max(m);
  float l = 0.f;
  for (int s = s0 + lane; s <= s1; s += 64) l += ml[s * 2 + 1] * exp2f(ml[s * 2] - m);
  l = wave_sum(l);
  const float inv = 1.0f / l;
  const float* po = part_o + (size_t)item * n_splits * D;
  const int sub = lane / MLPR, piece = lane % MLPR;
  float4 acc[MPIECES];
#pragma unroll
  for (int i = 0; i < MPIECES; ++i) acc[i] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
  for (int s = s0 + wave * MROWS + sub; s <= s1; s += MROWS * W) {
    const float wgt = exp2f(ml[s * 2] - m);
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
  if (W > 1) {                               // the other waves' sums, added in the order of the waves
    if (wave > 0) {
#pragma unroll
      for (int i = 0; i < MPIECES; ++i) sum_s[wave - 1][i][lane] = acc[i];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int wv = 0; wv < W - 1; ++wv)
#pragma unroll
      for (int i = 0; i < MPIECES; ++i) {
        const float4 v = sum_s[wv][i][lane];
        acc[i].x += v.x; acc[i].y += v.y; acc[i].z += v.z; acc[i].w += v.w;
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

// The same merge for launches of few splits (up to MROWS * NL * W): a lane asks for the position and for all the
// numbers of its NL splits at once, whether the position reaches them or not, and only then looks at what has come
// (the kernel above waits for the position, then for the maxima, then for the outputs a few splits at a time). A split that the position does not reach was
// never written: its numbers are set aside by a select, never multiplied. Every wave merges its own splits against
// its own maximum; wave 0 then adds the waves up against the maximum of all, in the order of the waves.
template <int W, int NL>
__global__ __launch_bounds__(64 * W) void merge_splits_at_once_kernel(const float* __restrict__ part_o,
                                                                      const float* __restrict__ part_ml,
                                                                      bf16_t* __restrict__ out, const int* __restrict__ positions,
                                                                      int window, int split_len, int n_splits, int Hq) {
  __shared__ float4 sum_s[W > 1 ? W - 1 : 1][MPIECES][64];
  __shared__ float ml_s[W > 1 ? W - 1 : 1][2];
  const int item = blockIdx.x;               // t * Hq + h
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int sub = lane / MLPR, piece = lane % MLPR;
  const float* ml = part_ml + (size_t)item * n_splits * 2;
  const float* po = part_o + (size_t)item * n_splits * D;
  const int pos = positions[item / Hq];
  float2 mls[NL];
  float4 v[NL][MPIECES];
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int s = (i * W + wave) * MROWS + sub;
    const bool in = s < n_splits;
    mls[i] = in ? *reinterpret_cast<const float2*>(ml + s * 2) : make_float2(-INFINITY, 0.f);
#pragma unroll
    for (int p = 0; p < MPIECES; ++p) {
      const int qd = piece + p * MLPR;
      v[i][p] = (in && qd < MQ) ? *reinterpret_cast<const float4*>(po + (size_t)s * D + qd * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  }
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int s0 = lo / split_len, s1 = min(pos / split_len, n_splits - 1);
  float m = -INFINITY;
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const int s = (i * W + wave) * MROWS + sub;
    if (s < s0 || s > s1) mls[i] = make_float2(-INFINITY, 0.f);
    m = fmaxf(m, mls[i].x);
  }
#pragma unroll
  for (int off = MLPR; off < 64; off <<= 1) m = fmaxf(m, __shfl_xor(m, off, 64));
  const float m_ref = m == -INFINITY ? 0.f : m;          // a wave none of whose splits the position reaches
  float l = 0.f;
  float4 acc[MPIECES];
#pragma unroll
  for (int p = 0; p < MPIECES; ++p) acc[p] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int i = 0; i < NL; ++i) {
    const bool reached = mls[i].x != -INFINITY;
    const float wgt = reached ? exp2f(mls[i].x - m_ref) : 0.f;
    l += reached ? mls[i].y * wgt : 0.f;
#pragma unroll
    for (int p = 0; p < MPIECES; ++p) {
      acc[p].x += reached ? v[i][p].x * wgt : 0.f; acc[p].y += reached ? v[i][p].y * wgt : 0.f;
      acc[p].z += reached ? v[i][p].z * wgt : 0.f; acc[p].w += reached ? v[i][p].w * wgt : 0.f;
    }
  }
#pragma unroll
  for (int off = MLPR; off < 64; off <<= 1) {
    l += __shfl_xor(l, off, 64);
#pragma unroll
    for (int p = 0; p < MPIECES; ++p) {
      acc[p].x += __shfl_xor(acc[p].x, off, 64); acc[p].y += __shfl_xor(acc[p].y, off, 64);
      acc[p].z += __shfl_xor(acc[p].z, off, 64); acc[p].w += __shfl_xor(acc[p].w, off, 64);
    }
  }
  if (W > 1) {
    if (wave > 0) {
#pragma unroll
      for (int p = 0; p < MPIECES; ++p) sum_s[wave - 1][p][lane] = acc[p];
      if (lane == 0) { ml_s[wave - 1][0] = m; ml_s[wave - 1][1] = l; }
    }
    __syncthreads();
    if (wave > 0) return;
    float m_all = m;
#pragma unroll
    for (int wv = 0; wv < W - 1; ++wv) m_all = fmaxf(m_all, ml_s[wv][0]);
    const float own = exp2f(m - m_all);                    // (some split is reached, so m_all is a number)
    l *= own;
#pragma unroll
    for (int p = 0; p < MPIECES; ++p) { acc[p].x *= own; acc[p].y *= own; acc[p].z *= own; acc[p].w *= own; }
#pragma unroll
    for (int wv = 0; wv < W - 1; ++wv) {
      const float theirs = exp2f(ml_s[wv][0] - m_all);
      l += ml_s[wv][1] * theirs;
#pragma unroll
      for (int p = 0; p < MPIECES; ++p) {
        const float4 o = sum_s[wv][p][lane];
        acc[p].x += o.x * theirs; acc[p].y += o.y * theirs; acc[p].z += o.z * theirs; acc[p].w += o.w * theirs;
      }
    }
  }
  if (sub == 0) {
    const float inv = 1.0f / l;
#pragma unroll
    for (int p = 0; p < MPIECES; ++p) {
      const int qd = piece + p * MLPR;
      if (qd < MQ) {
        bf16_t* o = out + (size_t)item * D + qd * 4;
        o[0] = (bf16_t)(acc[p].x * inv); o[1] = (bf16_t)(acc[p].y * inv);
        o[2] = (bf16_t)(acc[p].z * inv); o[3] = (bf16_t)(acc[p].w * inv);
      }
    }
  }
}

extern "C" int nhv_decode_attention_head_dim() { return D; }

// Checks and launches shared by the two entry points.
static int launch_decode_attention(const void* q, const void* k_cache, const void* v_cache, void* out, float* part_o,
                                   float* part_ml, const void* token_req, const void* positions,
                                   const void* block_tables, int max_blocks, int T, int Hq, int Hkv, int page_size,
                                   float scale, int window, int split_len, int n_splits, hipStream_t s) {
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  dim3 grid(Hkv, T, n_splits);
  hipLaunchKernelGGL(decode_attention_kernel, grid, dim3(64), 0, s, (const bf16_t*)q, (const bf16_t*)k_cache,
                     (const bf16_t*)v_cache, part_o, part_ml, (const int*)token_req,
                     (const int*)positions, (const int*)block_tables, max_blocks, Hq, Hkv, page_size, page_shift,
                     scale * 1.4426950408889634f, window, split_len, n_splits);
  NHV_LAUNCH_CHECK("decode_attention");
  const unsigned items = (unsigned)((size_t)T * Hq);
#define NHV_MERGE_ARGS (const float*)part_o, (const float*)part_ml, (bf16_t*)out, (const int*)positions, window, split_len, n_splits, Hq
#define NHV_MERGE_AT_ONCE(W_, NL_) \
  hipLaunchKernelGGL((merge_splits_at_once_kernel<W_, NL_>), dim3(items), dim3(64 * W_), 0, s, NHV_MERGE_ARGS)
  // few splits: everything asked for at once, by four waves from the point where one wave's lanes would take more
  // than four splits each (a decode step of 8 requests of 2,100 keys: 4.28 ms with four waves for its 17 splits, 4.32
  // with one wave, 4.30 with the kernel that waits for one thing after the other)
  if (n_splits <= MROWS * 4) NHV_MERGE_AT_ONCE(1, 4);
  else if (n_splits <= MROWS * 16) NHV_MERGE_AT_ONCE(4, 4);
  else if (n_splits <= MROWS * 32) NHV_MERGE_AT_ONCE(4, 8);
  else if (n_splits <= MROWS * 64) NHV_MERGE_AT_ONCE(4, 16);
  // (beyond that, what decides is the number of splits the launch is made for: inside a graph that is the bound's, but
  // few tokens with a bound of many splits are the case where the four waves pay, and otherwise they cost nothing much)
  else if ((size_t)T * Hq <= 1024)
    hipLaunchKernelGGL(merge_splits_kernel<4>, dim3(items), dim3(256), 0, s, NHV_MERGE_ARGS);
  else
    hipLaunchKernelGGL(merge_splits_kernel<1>, dim3(items), dim3(64), 0, s, NHV_MERGE_ARGS);
#undef NHV_MERGE_AT_ONCE
#undef NHV_MERGE_ARGS
  NHV_LAUNCH_CHECK("merge_splits");
  return 0;
}

static int check_decode_attention(int max_blocks, int T, int Hq, int Hkv, int page_size, int window, int split_len,
                                  int n_splits) {
  NHV_REQUIRE(T > 0 && Hq > 0 && Hkv > 0 && page_size > 0 && max_blocks > 0, "decode attention: bad sizes");
  NHV_REQUIRE(Hq % Hkv == 0, "decode attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  const int G = Hq / Hkv;
  NHV_REQUIRE(G <= 16, "decode attention: %d query heads per key head are beyond this kernel's limit of 16", G);
  NHV_REQUIRE(split_len > 0 && split_len % RK == 0, "decode attention: split length %d must be a multiple of %d", split_len, RK);
  NHV_REQUIRE(n_splits > 0 && n_splits <= 65535 && Hkv <= 65535 && T <= 65535, "decode attention: grid too large");
  NHV_REQUIRE(window >= 0, "decode attention: negative window");
  return 0;
}

// part_o: float [T, Hq, n_splits, D]; part_ml: float [T, Hq, n_splits, 2]; n_splits * split_len must cover
// every context length of the batch (max_context_len).
extern "C" int nhv_decode_attention_bf16(const void* q, const void* k_cache, const void* v_cache, void* out, void* part_o,
                                         void* part_ml, const void* token_req, const void* positions,
                                         const void* block_tables, int max_blocks, int T, int Hq, int Hkv, int page_size,
                                         float scale, int window, int split_len, int n_splits, void* stream) {
  if (check_decode_attention(max_blocks, T, Hq, Hkv, page_size, window, split_len, n_splits)) return 1;
  return launch_decode_attention(q, k_cache, v_cache, out, (float*)part_o, (float*)part_ml, token_req, positions,
                                 block_tables, max_blocks, T, Hq, Hkv, page_size, scale, window, split_len, n_splits,
                                 (hipStream_t)stream);
}

// ---- the entry point that allocates nothing (nhv_no_alloc.h) ----
// The splits' partial results of a call: [T, Hq, n_splits, D] floats, then [T, Hq, n_splits, 2]. Part of the
// library's device image: every GPU that loads the library holds its own copy at its own address.
constexpr size_t SCRATCH_FLOATS = NHV_NO_ALLOC_SCRATCH_BYTES / sizeof(float);
static __device__ __align__(256) float scratch[SCRATCH_FLOATS];

// In host code the array's name stands for a host-side handle, not for device memory: each device's address
// is asked for once, with that device current, and kept.
constexpr int MAX_DEVICES = 64;
static float* scratch_of_device[MAX_DEVICES] = {};
static std::mutex scratch_lock;

static int scratch_address(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  NHV_REQUIRE(e == hipSuccess, "decode attention (no alloc): hipGetDevice failed: %s", hipGetErrorString(e));
  NHV_REQUIRE(device >= 0 && device < MAX_DEVICES, "decode attention (no alloc): device %d is beyond the %d this library keeps track of",
              device, MAX_DEVICES);
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_of_device[device] == nullptr) {
    void* address = nullptr;
    e = hipGetSymbolAddress(&address, HIP_SYMBOL(scratch));
    NHV_REQUIRE(e == hipSuccess && address != nullptr, "decode attention (no alloc): hipGetSymbolAddress failed on device %d: %s",
                device, hipGetErrorString(e));
    scratch_of_device[device] = (float*)address;
  }
  *ptr = scratch_of_device[device];
  return 0;
}

extern "C" size_t nhv_decode_attention_no_alloc_limit() { return NHV_NO_ALLOC_SCRATCH_BYTES; }

extern "C" int nhv_decode_attention_no_alloc_init() {
  float* base = nullptr;
  return scratch_address(&base);
}

extern "C" int nhv_decode_attention_bf16_no_alloc(const void* q, const void* k_cache, const void* v_cache, void* out,
                                                  const void* token_req, const void* positions,
                                                  const void* block_tables, int max_blocks, int T, int Hq, int Hkv,
                                                  int page_size, float scale, int window, int split_len, int n_splits,
                                                  void* stream) {
  if (check_decode_attention(max_blocks, T, Hq, Hkv, page_size, window, split_len, n_splits)) return 1;
  const size_t items = (size_t)T * Hq * n_splits;
  NHV_REQUIRE(items * (D + 2) <= SCRATCH_FLOATS,
              "decode attention (no alloc): %d tokens x %d heads x %d splits need %zu bytes of scratch, the library holds %zu",
              T, Hq, n_splits, items * (D + 2) * sizeof(float), (size_t)NHV_NO_ALLOC_SCRATCH_BYTES);
  float* base = nullptr;
  if (scratch_address(&base)) return 1;
  // a call reads only the entries it has written (the merge looks at the splits that hold a visible key, and
  // those are the splits that write): nothing has to be cleared
  return launch_decode_attention(q, k_cache, v_cache, out, base, base + items * D, token_req, positions, block_tables,
                                 max_blocks, T, Hq, Hkv, page_size, scale, window, split_len, n_splits, (hipStream_t)stream);
}
