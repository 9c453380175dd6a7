// Attention of prompt portions (and of anything else in the batch) over the paged
// cache in bfloat16 on the matrix cores. Compiled for one head size:
// -DNHV_HEAD_DIM=<multiple of 16>.
//
// A block of 4 waves works on one (request, key/value head) and four or eight row tiles,
// one or two per wave; a row tile is 16 consecutive tokens of one query head, and the row
// tiles of a request are numbered so that the heads sharing the key/value head come
// first: with 4 heads per key/value head a block is 16 or 32 tokens x 4 heads, and every
// key and value it stages in LDS is used by 64 or 128 rows. With two row tiles a wave
// reads every operand of keys and values from LDS once for both (the reads from LDS are
// what the kernel waits for most); that is taken where the batch still gives every
// compute unit two blocks of that size. Keys are taken in tiles of 64, in rising order:
//   S^T[key, row] = K[key, :] . Q[row, :]      K tile from LDS, Q in registers (v_mfma_f32_16x16x32_bf16)
//   exponentials against a reference point per row that moves only when they have outgrown it (then the row's
//   maximum, two shuffles over the lane groups), sums kept per lane
//   O^T[d, row]  += V^T[d, key] . P^T[key, row]  V^T from LDS, P in registers (v_mfma_f32_16x16x32_bf16)
// An S^T tile leaves every lane with four consecutive keys of one row; two such tiles
// side by side are the eight summation slots of a lane in the second product (the
// order of the slots is free as long as P and V agree), so P never goes through
// memory, and because the second product is taken transposed a lane's output entries
// belong to the same row as its scores: the rescaling needs no exchange between lanes.
//
// Keys and values go from the cache straight into LDS (global_load_lds, 16 bytes a lane,
// no registers in between), row by row as they lie in the cache, into one of two
// buffers: the next tile is on its way while this one is computed, and a tile costs one
// barrier. Such a load puts lane i's piece at the wave's LDS base + 16 i, so the layout
// is linear; bank conflicts are avoided by which piece of the row a lane asks for (the
// piece index XOR-ed with the key's low bits). The V^T operand is read from the
// row-major tile with ds_read_b64_tr_b16: in a group of 16 lanes, lane i receives
// element i % 4 of the 8-byte pieces that lanes i / 4 + 4 j (j = 0..3) point at, so with
// lane r pointing at key r / 4, entries 4 (r % 4).. of the 16-entry block, lane i gets
// entry i of four consecutive keys. A query at position p reads keys lo..p (lo = p -
// window + 1 with a window, else 0). Keys outside the block's range are replaced by the
// nearest key inside it (their P is 0): unused cache slots may hold anything, and 0 * NaN
// would poison the sums.
#include "nhv_common.h"
#include <math.h>
#include <type_traits>

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
constexpr int PIECES = BN * CH;             // 16-byte pieces of a tile of keys (or of values)
constexpr int LOADS = (PIECES + 255) / 256; // direct loads per thread, tile and matrix
constexpr bool CH_POW2 = (CH & (CH - 1)) == 0;
// piece c of key k lies at piece c ^ (k & KSWZ) of its row in the K tile: 16 keys read the same piece at once
constexpr int KSWZ = CH_POW2 ? (CH < 16 ? CH : 16) - 1 : 0;
// and at c ^ ((k & VSWZ) << 1) in the V tile, whose transposed reads take 32 bytes of 8 keys at once
constexpr int VSWZ = CH_POW2 && CH >= 4 ? (CH / 2 < 8 ? CH / 2 : 8) - 1 : 0;
constexpr int MAX_RT = D <= 128 ? 2 : 1;    // row tiles per wave (template argument RT): all of them use every key and value
                                            // that the wave reads from LDS; two need the registers of head sizes up to 128

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(__bf16)))) __bf16 bf16x4;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void* lds_ptr;
typedef const __attribute__((address_space(1))) void* global_ptr;

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

constexpr int BT_LDS = 1024;                // block-table entries that are kept in LDS

template <typename P>
__device__ __forceinline__ int slot_of(P bt, int key, int page_size, int page_shift) {
  if (page_shift >= 0) return (bt[key >> page_shift] << page_shift) + (key & (page_size - 1));
  return bt[key / page_size] * page_size + key % page_size;
}

// BT_IN_LDS: the request's block table (up to the block's last key) is copied into LDS first, so that the
// look-up that every load of a key depends on costs an LDS read instead of a trip to memory.
template <bool BT_IN_LDS, int RT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2))) void prefill_attention_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ k_cache, const bf16_t* __restrict__ v_cache,
    bf16_t* __restrict__ out, const int* __restrict__ cu_seqlens_q, const int* __restrict__ context_lens,
    const int* __restrict__ block_tables, int max_blocks, int Hq, int Hkv, int page_size, int page_shift,
    float scale_log2e, int window) {
  constexpr int DL = SUPPORTED ? D : 16;                   // keeps the unsupported sizes compilable; they are never launched
  constexpr int TILE = SUPPORTED ? BN * DL : 16;           // elements of a tile
  __shared__ __attribute__((aligned(16))) bf16_t k_s0[TILE], k_s1[TILE], v_s0[TILE], v_s1[TILE];
  __shared__ int bt_s[BT_IN_LDS ? BT_LDS : 1];
  if (!SUPPORTED) return;
  constexpr int TPB = 4 * RT;                              // row tiles per block

  // Blocks go to the eight XCDs in turn by their place in the launch order, and each XCD has an L2 of its own:
  // the key/value head is the fastest index of that order, so that (with eight heads) an XCD reads the keys and
  // values of one head only and finds them in its L2 after the first block has asked for them (8,192 new tokens:
  // 833 to 779 us; 2,048 after 6,144: 367 to 360 us; 2,048 alone: the same 82 us).
  const int req = blockIdx.z;
  const int launch_order = blockIdx.x + gridDim.x * blockIdx.y;
  const int kvh = launch_order % gridDim.y;
  const int G = Hq / Hkv;
  const int q_begin = cu_seqlens_q[req];
  const int q_len = cu_seqlens_q[req + 1] - q_begin;
  const int ctx = context_lens[req];
  const int start_pos = ctx - q_len;                       // position of the request's first token in this step
  const int n_row_tiles = G * ((q_len + 15) / 16);
  // Causal work grows with the row tile's place in the portion, and all blocks of a long portion are resident
  // at once, so which blocks share a compute unit decides the kernel's time. Blocks 256 apart in launch order
  // (256 compute units) tend to land on the same unit: the rounds of 256 blocks take their row tiles in rising
  // and in falling order in turn, so that a unit's blocks have long and short key ranges in turn.
  const int per_round = max(1, 256 / (int)gridDim.y);      // row-tile groups in a round of 256 blocks
  const int j = launch_order / (int)gridDim.y;
  const int r = j / per_round;
  const int in_round = min(per_round, (int)gridDim.x - r * per_round);
  const int up = r * per_round + ((r & 1) ? in_round - 1 - (j - r * per_round) : j - r * per_round);
  // and the rounds go from the longest key ranges to the shortest: what is left for the end, when units run empty,
  // is short (4,096 new tokens: 239 to 222 us; 8,192: 803 to 761 us; 2,048 after 6,144: 337 to 319 us)
  const int bx = (int)gridDim.x - 1 - up;
  const int first_tile = bx * TPB;
  if (first_tile >= n_row_tiles) return;                   // the grid is made for the longest portion of the batch

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15, grp = lane >> 4;

  // the block's key range: from the smallest lower bound to the largest position of its rows
  const int last_tile = min(first_tile + TPB - 1, n_row_tiles - 1);
  const int blk_tok_lo = (first_tile / G) * 16;
  const int blk_tok_hi = min((last_tile / G) * 16 + 15, q_len - 1);
  const int key_hi = start_pos + blk_tok_hi;
  const int key_lo = window > 0 ? max(0, start_pos + blk_tok_lo - window + 1) : 0;

  // this wave's row tiles; this lane's row (in both products) is token tok0 + col of the tile's head
  const bool live = first_tile + wave * RT < n_row_tiles;
  int row_pos[RT], row_lo[RT], row_tok[RT], head[RT];
  bool row_ok[RT];
  int wave_lo_pos = 0x7fffffff, wave_hi = -1, wave_max_lo = 0;
  bf16x8 qb[RT][DSTEPS];
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    const int my_tile = first_tile + wave * RT + r;
    const bool tile_live = my_tile < n_row_tiles;
    head[r] = kvh * G + (tile_live ? my_tile % G : 0);
    const int tok0 = tile_live ? (my_tile / G) * 16 : 0;
    row_tok[r] = tok0 + col;
    row_ok[r] = tile_live && row_tok[r] < q_len;
    row_pos[r] = tile_live ? start_pos + min(row_tok[r], q_len - 1) : -1;    // a tile beyond the portion sees no key
    row_lo[r] = window > 0 ? max(0, row_pos[r] - window + 1) : 0;
    if (tile_live) {
      const int hi = start_pos + min(tok0 + 15, q_len - 1);                 // beyond it the tile has nothing to do
      wave_lo_pos = min(wave_lo_pos, start_pos + tok0);                       // the tile's first row sees the fewest keys
      wave_hi = max(wave_hi, hi);
      wave_max_lo = max(wave_max_lo, window > 0 ? max(0, hi - window + 1) : 0);
    }
#pragma unroll
    for (int s = 0; s < DSTEPS; ++s) {
      const int d = s * 32 + grp * 8;
      qb[r][s] = (row_ok[r] && d < D)
                     ? *reinterpret_cast<const bf16x8*>(q + ((size_t)(q_begin + row_tok[r]) * Hq + head[r]) * D + d)
                     : zero8();
    }
  }
  float m_run[RT], l_part[RT];                             // of row `col` (base 2); l_part is this lane's share of the row's sum
  floatx4 o[RT][DTILES];                                   // o[r][dt][j]: entry dt * 16 + 4 grp + j of row `col`
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    m_run[r] = -INFINITY;
    l_part[r] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) o[r][dt] = floatx4{0.f, 0.f, 0.f, 0.f};
  }

  const int* bt_g = block_tables + (size_t)req * max_blocks;
  if (BT_IN_LDS) {
    const int n_entries = min(BT_LDS, key_hi / page_size + 1);
    for (int i = tid; i < n_entries; i += 256) bt_s[i] = bt_g[i];
    __syncthreads();
  }
  // where the key look-ups go: LDS copy or memory
  auto slot = [&](int key) {
    return BT_IN_LDS ? slot_of((const int*)bt_s, key, page_size, page_shift) : slot_of(bt_g, key, page_size, page_shift);
  };

  // memory -> LDS without registers: wave w's load number i brings pieces (4 i + w) * 64 + lane of the tile.
  // With pages that are a power of two and hold whole tiles, a tile inside the block's key range lies in one page
  // at a place that is the same for the whole block: one look-up and scalar arithmetic, and each thread adds
  // offsets that it worked out once. Other tiles (the range's ends, other page sizes) look every key up.
  const bool whole_tiles = page_shift >= 0 && page_size >= BN;
  int k_off[LOADS], v_off[LOADS];
#pragma unroll
  for (int i = 0; i < LOADS; ++i) {
    const int u = (i * 4 + wave) * 64 + lane;
    const int kl = u / CH, piece = u % CH;
    k_off[i] = (kl * Hkv + kvh) * D + (piece ^ (kl & KSWZ)) * 8;
    v_off[i] = (kl * Hkv + kvh) * D + (piece ^ ((kl & VSWZ) << 1)) * 8;
  }
  auto issue = [&](int kb, bf16_t* k_s, bf16_t* v_s) {
    if (whole_tiles && kb >= key_lo && kb + BN - 1 <= key_hi) {
      const int page = __builtin_amdgcn_readfirstlane(BT_IN_LDS ? bt_s[kb >> page_shift] : bt_g[kb >> page_shift]);
      const size_t tile_off = (((size_t)page << page_shift) + (kb & (page_size - 1))) * Hkv * D;
      const bf16_t* k_tile = k_cache + tile_off;
      const bf16_t* v_tile = v_cache + tile_off;
#pragma unroll
      for (int i = 0; i < LOADS; ++i)
        if (PIECES % 256 == 0 || (i * 4 + wave) * 64 + lane < PIECES) {
          __builtin_amdgcn_global_load_lds((global_ptr)(k_tile + k_off[i]), (lds_ptr)(k_s + (i * 4 + wave) * 512), 16, 0, 0);
          __builtin_amdgcn_global_load_lds((global_ptr)(v_tile + v_off[i]), (lds_ptr)(v_s + (i * 4 + wave) * 512), 16, 0, 0);
        }
      return;
    }
#pragma unroll
    for (int i = 0; i < LOADS; ++i) {
      const int u = (i * 4 + wave) * 64 + lane;
      if (PIECES % 256 == 0 || u < PIECES) {
        const int kl = u / CH, piece = u % CH;
        const int key = min(max(kb + kl, key_lo), key_hi);
        const size_t row = ((size_t)slot(key) * Hkv + kvh) * D;
        const size_t koff = row + (piece ^ (kl & KSWZ)) * 8;
        const size_t voff = row + (piece ^ ((kl & VSWZ) << 1)) * 8;
        __builtin_amdgcn_global_load_lds((global_ptr)(k_cache + koff), (lds_ptr)(k_s + (i * 4 + wave) * 512), 16, 0, 0);
        __builtin_amdgcn_global_load_lds((global_ptr)(v_cache + voff), (lds_ptr)(v_s + (i * 4 + wave) * 512), 16, 0, 0);
      }
    }
  };

  // MASKED (a type, so that each call site names a compile-time choice): whether some key of the tile is hidden from
  // some row of the wave. Tiles wholly inside every row's range, which are nearly all, run code without the
  // comparisons: as a run-time flag the test cost three to four instructions for every score in every tile.
  auto compute = [&](auto masked, int kb, const bf16_t* k_s, const bf16_t* v_s) {
    constexpr bool MASKED = decltype(masked)::value;
    // ---- scores of the tile's keys for this wave's rows: every K operand serves all row tiles
    floatx4 s4[RT][KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
      for (int r = 0; r < RT; ++r) s4[r][kt] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < DSTEPS; ++s) {
        const int piece = s * 4 + grp;
        const bf16x8 ka = piece < CH ? *reinterpret_cast<const bf16x8*>(k_s + (kt * 16 + col) * D + (piece ^ (col & KSWZ)) * 8)
                                     : zero8();
#pragma unroll
        for (int r = 0; r < RT; ++r) s4[r][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, qb[r][s], s4[r][kt], 0, 0, 0);
      }
    }
    bf16x8 pa[RT][KT / 2];                                 // P of keys (32 a + 4 grp + j) and (32 a + 16 + 4 grp + j)
    float alpha[RT];
    bool grow[RT];
#pragma unroll
    for (int r = 0; r < RT; ++r) {
      // The reference point of a row's exponentials stays where it is as long as they stay far below float's range:
      // they are taken against it at once, without the tile's maximum, and only a sum that has grown past 2^40 (or is
      // no number: a row that has seen no key yet has no reference) sends the wave to the maximum and a new reference.
      if (MASKED) {
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int key = kb + kt * 16 + grp * 4 + j;
            if (key > row_pos[r] || key < row_lo[r]) s4[r][kt][j] = -INFINITY;
          }
      }
      float psum = 0.f;
#pragma unroll
      for (int kt = 0; kt < KT; ++kt)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s4[r][kt][j], scale_log2e, -m_run[r]));
          psum += p;
          pa[r][kt / 2][(kt % 2) * 4 + j] = (__bf16)p;
        }
      grow[r] = __any(!(psum < 1.0995116e12f));
      alpha[r] = 1.0f;
      if (grow[r]) {
        asm volatile("" ::: "memory");
        float m_tile = -INFINITY;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int j = 0; j < 4; ++j) m_tile = fmaxf(m_tile, s4[r][kt][j]);
        m_tile *= scale_log2e;
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 16, 64));
        m_tile = fmaxf(m_tile, __shfl_xor(m_tile, 32, 64));
        const float m_new = fmaxf(m_run[r], m_tile);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;  // a row that has still seen no key
        alpha[r] = m_run[r] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_run[r] - m_safe);
        psum = 0.f;
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(s4[r][kt][j], scale_log2e, -m_safe));
            psum += p;
            pa[r][kt / 2][(kt % 2) * 4 + j] = (__bf16)p;
          }
        l_part[r] = l_part[r] * alpha[r] + psum;
        m_run[r] = m_new;
      } else {
        l_part[r] += psum;
      }
    }
    // The outputs are rescaled only when a reference has moved: a branch of the whole wave, taken rarely. (Written
    // as a condition inside the loop over the output tiles, the compiler made a multiply and a select of it for
    // every output entry in every tile, 128 instructions a tile; the empty statement keeps the branch a branch.)
#pragma unroll
    for (int r = 0; r < RT; ++r)
      if (grow[r]) {
        asm volatile("" ::: "memory");
#pragma unroll
        for (int dt = 0; dt < DTILES; ++dt)
#pragma unroll
          for (int j = 0; j < 4; ++j) o[r][dt][j] *= alpha[r];
      }
    // this lane points at key 4 grp + col / 4 of a 16-key sub-tile, entries 4 (col % 4).. of the 16-entry block dt
    const int tr_key = grp * 4 + (col >> 2);
    const int tr_piece = (col & 3) >> 1, tr_half = (col & 1) * 4;
#pragma unroll
    for (int dt = 0; dt < DTILES; ++dt) {
#pragma unroll
      for (int a = 0; a < KT / 2; ++a) {
        // this lane's eight summation slots: keys 32 a + 4 grp + (0..3) and 32 a + 16 + 4 grp + (0..3), entry dt * 16 + col
        const int k_lo = a * 32 + tr_key, k_hi = k_lo + 16;
        const bf16_t* p_lo = v_s + k_lo * D + ((dt * 2 + tr_piece) ^ ((k_lo & VSWZ) << 1)) * 8 + tr_half;
        const bf16_t* p_hi = v_s + k_hi * D + ((dt * 2 + tr_piece) ^ ((k_hi & VSWZ) << 1)) * 8 + tr_half;
        const short4_t lo4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)p_lo);
        const short4_t hi4 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) short4_t*)p_hi);
        typedef short short8_t __attribute__((ext_vector_type(8)));
        const short8_t both = __builtin_shufflevector(lo4, hi4, 0, 1, 2, 3, 4, 5, 6, 7);
        const bf16x8 va = __builtin_bit_cast(bf16x8, both);
#pragma unroll
        for (int r = 0; r < RT; ++r) o[r][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pa[r][a], o[r][dt], 0, 0, 0);
      }
    }
  };

  auto run = [&](int kb, const bf16_t* k_s, const bf16_t* v_s) {
    if (kb + BN - 1 > wave_lo_pos || kb < wave_max_lo) compute(std::true_type{}, kb, k_s, v_s);
    else compute(std::false_type{}, kb, k_s, v_s);
  };

  // tiles alternate between the two buffers; the loop is written out for both so that every load and read names
  // its buffer (the compiler then knows that the loads under way do not touch the tile being read)
  const int kb0 = (key_lo / BN) * BN;
  issue(kb0, k_s0, v_s0);
  for (int kb = kb0; kb <= key_hi; kb += 2 * BN) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();                                       // this tile has arrived, the other buffer has been read
    if (kb + BN <= key_hi) issue(kb + BN, k_s1, v_s1);
    if (live && kb <= wave_hi) run(kb, k_s0, v_s0);        // a whole-wave decision; the wave still meets the barriers
    if (kb + BN > key_hi) break;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (kb + 2 * BN <= key_hi) issue(kb + 2 * BN, k_s0, v_s0);
    if (live && kb + BN <= wave_hi) run(kb + BN, k_s1, v_s1);
  }
  if (!live) return;
#pragma unroll
  for (int r = 0; r < RT; ++r) {
    float l = l_part[r];
    l += __shfl_xor(l, 16, 64);
    l += __shfl_xor(l, 32, 64);
    if (row_ok[r]) {
      const float inv = 1.0f / l;
      bf16_t* dst = out + ((size_t)(q_begin + row_tok[r]) * Hq + head[r]) * D;
#pragma unroll
      for (int dt = 0; dt < DTILES; ++dt) {
        bf16x4 four;
#pragma unroll
        for (int j = 0; j < 4; ++j) four[j] = (__bf16)(o[r][dt][j] * inv);
        *reinterpret_cast<bf16x4*>(dst + dt * 16 + grp * 4) = four;
      }
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
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if (page_size == (1 << b)) page_shift = b;
  const int G = Hq / Hkv;
  const long long row_tiles = (long long)G * ((max_q_len + 15) / 16);
  // two row tiles a wave where that still leaves two blocks for every compute unit (1,024 new tokens of 8 kv heads
  // are 256 such blocks: 41 us, and 31 us as 512 blocks of one row tile a wave; after 7,000 keys 259 and 216 us)
  const bool two = prefill::MAX_RT >= 2 && (row_tiles + 7) / 8 * Hkv * B >= 512;
  const int tpb = two ? 8 : 4;
  const long long gx = (row_tiles + tpb - 1) / tpb;
  NHV_REQUIRE(gx <= 0x7fffffff && Hkv <= 65535 && B <= 65535, "prefill attention: grid too large");
#define NHV_PREFILL_LAUNCH(BT, RT_)                                                                                    \
  hipLaunchKernelGGL((prefill::prefill_attention_kernel<BT, RT_>), dim3((unsigned)gx, Hkv, B), dim3(256), 0,         \
                     (hipStream_t)stream, (const bf16_t*)q, (const bf16_t*)k_cache, (const bf16_t*)v_cache, (bf16_t*)out, \
                     (const int*)cu_seqlens_q, (const int*)context_lens, (const int*)block_tables, max_blocks, Hq, Hkv, \
                     page_size, page_shift, scale * 1.4426950408889634f, window)
  const bool bt_in_lds = max_blocks <= prefill::BT_LDS;
  if (two) {
    if (bt_in_lds) NHV_PREFILL_LAUNCH(true, prefill::MAX_RT);
    else NHV_PREFILL_LAUNCH(false, prefill::MAX_RT);
  } else {
    if (bt_in_lds) NHV_PREFILL_LAUNCH(true, 1);
    else NHV_PREFILL_LAUNCH(false, 1);
  }
#undef NHV_PREFILL_LAUNCH
  NHV_LAUNCH_CHECK("prefill_attention");
  return 0;
}
