// Attention of prompt portions (and of anything else in the batch) over the paged
// cache in bfloat16 on the matrix cores. Compiled for one head size:
// -DNHV_HEAD_DIM=<multiple of 16>.
//
// A block of 4 waves works on one (request, key/value head) and four row tiles; a row
// tile is 16 consecutive tokens of one query head, and the row tiles of a request are
// numbered so that the heads sharing the key/value head come first: with 4 heads per
// key/value head a block is 16 tokens x 4 heads, and every key and value it stages
// in LDS is used by 64 rows. Keys are taken in tiles of 64, in rising order:
//   S^T[key, row] = K[key, :] . Q[row, :]     K tile from LDS, Q in registers (v_mfma_f32_16x16x32_bf16)
//   running maximum and sum per row in float (two shuffles over the lane groups)
//   O[row, d]   += P[row, key] . V[key, d]    P from registers, V^T from LDS (v_mfma_f32_16x16x16_bf16)
// The S^T tile leaves every lane with four consecutive keys of one row, which is the
// operand layout of the second product, so P never goes through memory. V is
// written to LDS transposed, so that its operand is one 8-byte read.
// A query at position p reads keys lo..p (lo = p - window + 1 with a window, else 0).
// Keys outside the block's range are staged as zeros: unused cache slots may hold
// anything, and 0 * NaN would poison the sums.
#include "nhv_common.h"
#include <math.h>

#ifndef NHV_HEAD_DIM
#error "compile with -DNHV_HEAD_DIM=<head size>"
#endif

namespace prefill {

constexpr int D = NHV_HEAD_DIM;
constexpr int DSTEPS = (D + 31) / 32;       // steps of the first product over the head
constexpr int DTILES = D / 16;              // output tiles of the second product
constexpr int CH = D / 8;                   // 16-byte pieces of a row
static_assert(D % 16 == 0 && D >= 16, "head size must be a multiple of 16");
constexpr bool SUPPORTED = D <= 256;        // beyond that the tiles do not fit into 64 KB of LDS
constexpr int BN = D <= 128 ? 64 : 32;      // keys per tile
constexpr int KT = BN / 16;                 // 16-key sub-tiles
constexpr int KPITCH = DSTEPS * 32 + 8;     // elements per row of the K tile (padded against bank conflicts)
constexpr int VPITCH = BN + 8;              // elements per row of the transposed V tile

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

__global__ __launch_bounds__(256) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ cu_seqlens_q, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, int max_blocks, int Hq, int Hkv, int page_size, float scale, int window) {
  constexpr int DL = SUPPORTED ? D : 16;                   // keeps the unsupported sizes compilable; they are never launched
  __shared__ __attribute__((aligned(16))) bf16_t k_s[BN * (SUPPORTED ? KPITCH : 24)];
  __shared__ __attribute__((aligned(16))) bf16_t vt_s[DL * VPITCH];
  if (!SUPPORTED) return;

  const int req = blockIdx.z, kvh = blockIdx.y;
  const int G = Hq / Hkv;
  const int q_begin = cu_seqlens_q[req];
  const int q_len = cu_seqlens_q[req + 1] - q_begin;
  const int ctx = context_lens[req];
  const int start_pos = ctx - q_len;                       // position of the request's first token in this step
  const int n_row_tiles = G * ((q_len + 15) / 16);
  const int first_tile = blockIdx.x * 4;
  if (first_tile >= n_row_tiles) return;                   // the grid is made for the longest portion of the batch

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int my_tile = first_tile + wave;
  const bool wave_live = my_tile < n_row_tiles;
  const int head = kvh * G + (wave_live ? my_tile % G : 0);
  const int tok0 = wave_live ? (my_tile / G) * 16 : 0;     // first token (within the portion) of this wave's rows

  // the block's key range: from the smallest lower bound to the largest position of its rows
  const int last_tile = min(first_tile + 3, n_row_tiles - 1);
  const int blk_tok_lo = (first_tile / G) * 16;
  const int blk_tok_hi = min((last_tile / G) * 16 + 15, q_len - 1);
  const int key_hi = start_pos + blk_tok_hi;
  const int key_lo = window > 0 ? max(0, start_pos + blk_tok_lo - window + 1) : 0;

  // this lane's row in the first product: token tok0 + col
  const int row_tok = tok0 + col;
  const bool row_ok = wave_live && row_tok < q_len;
  const int row_pos = start_pos + min(row_tok, q_len - 1);
  const int row_lo = window > 0 ? max(0, row_pos - window + 1) : 0;
  const int wave_hi = start_pos + min(tok0 + 15, q_len - 1);   // beyond it this wave has nothing to do

  bf16x8 qb[DSTEPS];
#pragma unroll
  for (int s = 0; s < DSTEPS; ++s) {
    const int d = s * 32 + grp * 8;
    qb[s] = (row_ok && d < D) ? *reinterpret_cast<const bf16x8*>(q + ((size_t)(q_begin + row_tok) * Hq + head) * D + d)
                              : zero8();
  }

  float m_run = -INFINITY, l_run = 0.f;                    // of row `col`, the same in all four lane groups
  floatx4 o[DTILES];                                       // o[dt][j]: row 4 grp + j, column dt * 16 + col
#pragma unroll
  for (int dt = 0; dt < DTILES; ++dt) o[dt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int* bt = block_tables + (size_t)req * max_blocks;

  for (int kb = (key_lo / BN) * BN; kb <= key_hi; kb += BN) {
    __syncthreads();                                       // the last tile has been read by every wave
    // ---- stage 64 keys and values
    for (int c = tid; c < BN * CH; c += 256) {
      const int kl = c / CH, dc = c % CH;
      const int key = kb + kl;
      bf16x8 kv8 = zero8(), vv8 = zero8();
      if (key >= key_lo && key <= key_hi) {
        const int slot = bt[key / page_size] * page_size + key % page_size;
        const size_t off = ((size_t)slot * Hkv + kvh) * D + dc * 8;
        kv8 = *reinterpret_cast<const bf16x8*>(k_cache + off);
        vv8 = *reinterpret_cast<const bf16x8*>(v_cache + off);
      }
      *reinterpret_cast<bf16x8*>(k_s + kl * KPITCH + dc * 8) = kv8;
#pragma unroll
      for (int e = 0; e < 8; ++e) vt_s[(dc * 8 + e) * VPITCH + kl] = vv8[e];
    }
    if (D % 32 != 0) {                                     // the padded half step of the first product reads zeros
      for (int c = tid; c < BN * 2; c += 256) *reinterpret_cast<bf16x8*>(k_s + (c / 2) * KPITCH + D + (c % 2) * 8) = zero8();
    }
    __syncthreads();
    if (!wave_live || kb > wave_hi) continue;              // whole wave; it still meets the others at the barriers

    // ---- scores of 64 keys for this wave's 16 rows
    floatx4 s4[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
      s4[kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) {
        const bf16x8 ka = *reinterpret_cast<const bf16x8*>(k_s + (kt * 16 + col) * KPITCH + s * 32 + grp * 8);
        s4[kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[s], s4[kt], 0, 0, 0);
      }
    }
    float m_tile = -INFINITY;
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = kb + kt * 16 + grp * 4 + j;
        const float v = (key <= row_pos && key >= row_lo) ? s4[kt][j] * scale : -INFINITY;
        s4[kt][j] = v;
        m_tile = fmaxf(m_tile, v);
      }
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
    m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
    const float m_new = fmaxf(m_run, m_tile);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // a row that has seen no key yet
    const float alpha = expf(m_run - m_safe);
    float psum = 0.f;
    bf16x4 pa[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float p = expf(s4[kt][j] - m_safe);
        psum += p;
        pa[kt][j] = (__bf16)p;
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l_run = l_run * alpha + psum;
    m_run = m_new;
    // rows of the output tiles are 4 grp + j: fetch their factors from the lanes that own those rows
    float a4[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) a4[j] = __shfl(alpha, grp * 4 + j, 64);
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
      for (int j = 0; j < 4; ++j) o[dt][j] *= a4[j];
#pragma unroll
      for (int kt = 0; kt < KT; ++kt) {
        const bf16x4 vb = *reinterpret_cast<const bf16x4*>(vt_s + (dt * 16 + col) * VPITCH + kt * 16 + grp * 4);
        o[dt] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pa[kt], vb, o[dt], 0, 0, 0);
      }
    }
  }
  if (!wave_live) return;
  float inv4[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) inv4[j] = 1.0f / __shfl(l_run, grp * 4 + j, 64);
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int tok = tok0 + grp * 4 + j;
    if (tok < q_len) {
      bf16_t* dst = out + ((size_t)(q_begin + tok) * Hq + head) * D;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) dst[dt * 16 + col] = (bf16_t)(o[dt][j] * inv4[j]);
    }
  }
}

}  // namespace prefill

extern "C" int nhv_prefill_attention_bf16(const void* q, const void* k_cache, const void* v_cache, void* out,
                                          const void* cu_seqlens_q, const void* context_lens, const void* block_tables,
                                          int max_blocks, int B, int max_q_len, int Hq, int Hkv, int page_size, float scale,
                                          int window, void* stream) {
  NHV_REQUIRE(B > 0 && max_q_len > 0 && Hq > 0 && Hkv > 0 && page_size > 0 && max_blocks > 0, "prefill attention: bad sizes");
  NHV_REQUIRE(Hq % Hkv == 0, "prefill attention: %d query heads are not a multiple of %d key heads", Hq, Hkv);
  NHV_REQUIRE(window >= 0, "prefill attention: negative window");
  NHV_REQUIRE(prefill::SUPPORTED, "prefill attention: head size %d is beyond this kernel's limit of 256", prefill::D);
  const int G = Hq / Hkv;
  const long long row_tiles = (long long)G * ((max_q_len + 15) / 16);
  const long long gx = (row_tiles + 3) / 4;
  NHV_REQUIRE(gx <= 0x7fffffff && Hkv <= 65535 && B <= 65535, "prefill attention: grid too large");
  hipLaunchKernelGGL(prefill::prefill_attention_kernel, dim3((unsigned)gx, Hkv, B), dim3(256), 0, (hipStream_t)stream,
                     (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out,
                     (const int*)cu_seqlens_q, (const int*)context_lens, (const int*)block_tables, max_blocks, Hq, Hkv,
                     page_size, scale, window);
  NHV_LAUNCH_CHECK("prefill_attention");
  return 0;
}
