// y[M, N] = x[M, K] . w[N, K]^T (+ bias), or silu(x . wg^T) * (x . wu^T), in bfloat16 for up to 16
// rows of x: the matrix products of a decoding step, whose time is the time to stream w from memory once.
//
// A block owns NT tiles of 16 rows of w (with GLU also their partners in the second matrix) and all
// of K; its waves take equal, contiguous shares of K, whole cache lines each, and a wave's lanes load
// 16 bytes each straight into the MFMA operand layout (v_mfma_f32_16x16x32_bf16: the w tile as the
// 16 x 32 operand, the rows of x as the 32 x 16 one), several loads in flight before the first is used.
// The waves' sums meet in LDS and are added in the order of the waves, so the result does not depend
// on timing. Rows of x beyond M and columns beyond K read as zero.
//
// Where all rows of x fit into LDS beside the sums (M (K + 8) 2 bytes of the 160 KB) a second kernel is used
// instead: a block copies x into LDS once (straight from memory, global_load_lds) and then walks over
// tiles of w, tile after tile, one or two blocks per compute unit for the whole matrix. The rows of x
// then cross from L2 to a compute unit once per call instead of once per tile: 5 to 25 % less time at
// every size measured, most where N is large (the head: 266 to 221 us at 8 rows). Where x does not
// fit at once and w has at most 256 tiles, a third kernel gives every block one tile and takes x through
// LDS in pieces (the 8B down projection from 7 rows on: 2 to 6 % less time, 12 % with 2,048 outputs). With more
// tiles than that, and x fitting in two pieces, a fourth kernel walks over all of a block's tiles once for each
// piece and keeps the tiles' sums in LDS between the two (16 rows of 5,120 columns: 13 % less time for gate_up).
//
// How many tiles a block takes, how many waves share K and how many loads a wave keeps in flight is
// chosen per call from M, N and K (plan() below): blocks that spread evenly over the compute units
// matter most, two tiles per block halve the reads of x when it has more than a few rows. (Splitting
// K over several blocks, with the last one to arrive adding the parts in order, was measured and never
// won: the fences cost more than the balance gains.)
#include "nhv_common.h"
#include "nhv_gemm_fusion.h"

namespace fewrows {

typedef NhvGemmFusion Fusion;

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// The scales of the rows of an x whose norm is still due (nhv_gemm_fusion.h), in two steps, so that the wait for
// the shares falls where other loads are under way. ask_row_scales: wave w asks for the shares of rows w, w + WAVES,
// ... (M <= 16: SCALE_ROWS<WAVES> rows at most), SCALE_SHARES of them per lane and row. set_row_scales: adds them up
// in a fixed order and leaves the scales in r_s[0..M); the caller's next barrier makes them visible.
constexpr int SCALE_SHARES = 4;              // up to 256 tiles (rows of 4,096) in one go; what is beyond is read when the sums are made
template <int WAVES>
constexpr int SCALE_ROWS = (16 + WAVES - 1) / WAVES;
template <int WAVES>
__device__ __forceinline__ void ask_row_scales(const Fusion& f, float (&share)[SCALE_ROWS<WAVES>][SCALE_SHARES], int M, int wave, int lane) {
  if (f.ss_in == nullptr) return;
#pragma unroll
  for (int i = 0; i < SCALE_ROWS<WAVES>; ++i) {
    const int m = wave + i * WAVES;
#pragma unroll
    for (int j = 0; j < SCALE_SHARES; ++j) {
      const int t = lane + j * 64;
      share[i][j] = (m < M && t < f.tiles_in) ? f.ss_in[(size_t)m * f.tiles_in + t] : 0.f;
    }
  }
}
template <int WAVES>
__device__ __forceinline__ void set_row_scales(const Fusion& f, const float (&share)[SCALE_ROWS<WAVES>][SCALE_SHARES], float* r_s, int M, int K,
                                               int wave, int lane) {
  if (f.ss_in == nullptr) return;
#pragma unroll
  for (int i = 0; i < SCALE_ROWS<WAVES>; ++i) {
    const int m = wave + i * WAVES;
    float sum = 0.f;
#pragma unroll
    for (int j = 0; j < SCALE_SHARES; ++j) sum += share[i][j];
    if (m < M)
      for (int t = lane + SCALE_SHARES * 64; t < f.tiles_in; t += 64) sum += f.ss_in[(size_t)m * f.tiles_in + t];
    sum = wave_sum(sum);
    if (m < M && lane == 0) r_s[m] = 1.0f / sqrtf(sum / (float)K + f.eps);
  }
}

// What the wave that writes a tile adds to and multiplies with, asked for before the tile's weights: the residual's
// entries and the next norm's weights of the lane's four outputs.
__device__ __forceinline__ void read_residual(const Fusion& f, float (&ahead)[8], int col, int grp, int n0, int M, int N) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + grp * 4 + j;
    ahead[4 + j] = 1.0f;
    if (col < M && n < N) {
      const size_t at = (size_t)col * N + n;
      ahead[j] = f.residual_f32 ? reinterpret_cast<const float*>(f.residual)[at] : (float)reinterpret_cast<const bf16_t*>(f.residual)[at];
      if (f.next_w) ahead[4 + j] = f.next_w_f32 ? reinterpret_cast<const float*>(f.next_w)[n] : (float)reinterpret_cast<const bf16_t*>(f.next_w)[n];
    }
  }
}

// A finished tile goes out: lane (col, grp) holds outputs n0 + 4 grp + (0..3) of row col of x. Plain: stored as they
// are. With a residual stream (nhv_gemm_fusion.h): added to it in float, the sum kept there and, times the next
// norm's weight and rounded, in sum_out, and the tile's share of the row's sum of squares (over its 16 outputs, the
// lanes' shares added in a fixed order) in ss_out. `tile` and `tiles` count tiles of 16 outputs over all of N.
// `ahead`: the residual's entries and the next norm's weights where the caller has read them already (read_residual), else null.
template <bool FUSED, typename TOut>
__device__ __forceinline__ void emit_tile(const Fusion& f, const float (&r)[4], TOut* __restrict__ y, int col, int grp, int n0,
                                          int tile, int tiles, int M, int N, const float* ahead = nullptr) {
  if (!FUSED || f.residual == nullptr) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + grp * 4 + j;
      if (col < M && n < N) y[(size_t)col * N + n] = (TOut)r[j];
    }
    return;
  }
  float sq = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + grp * 4 + j;
    if (col < M && n < N) {
      const size_t at = (size_t)col * N + n;
      float sum;
      if (f.residual_f32) {
        float* res = reinterpret_cast<float*>(f.residual);
        sum = r[j] + (ahead ? ahead[j] : res[at]);
        res[at] = sum;
      } else {
        bf16_t* res = reinterpret_cast<bf16_t*>(f.residual);
        sum = r[j] + (ahead ? ahead[j] : (float)res[at]);
        res[at] = (bf16_t)sum;
      }
      float weight = 1.0f;
      if (ahead) weight = ahead[4 + j];
      else if (f.next_w) weight = f.next_w_f32 ? reinterpret_cast<const float*>(f.next_w)[n] : (float)reinterpret_cast<const bf16_t*>(f.next_w)[n];
      f.sum_out[at] = (bf16_t)(sum * weight);
      sq += sum * sum;
    }
  }
  sq += __shfl_xor(sq, 16, 64);
  sq += __shfl_xor(sq, 32, 64);
  if (grp == 0 && col < M) f.ss_out[(size_t)col * tiles + tile] = sq;
}

// NT: tiles of 16 rows of w per block; WAVES: waves that share the block's part of K; UNROLL: loads in
// flight per wave and operand. A step is 32 columns of K (64 bytes of a row).
template <int NT, int WAVES, int UNROLL, bool GLU, bool FUSED, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void gemm_fewrows_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                  const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                                  int M, int N, int K, int steps_per_wave, const Fusion f) {
  constexpr int NA = GLU ? 2 : 1;
  constexpr int TILES = NA * NT;
  static_assert(NT <= WAVES, "wave nt finishes tile nt");
  __shared__ float red[WAVES][TILES][4][64];
  __shared__ float r_s[16];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int n0 = blockIdx.x * 16 * NT;
  float share[SCALE_ROWS<WAVES>][SCALE_SHARES];
  if constexpr (FUSED) ask_row_scales<WAVES>(f, share, M, wave, lane);

  const bf16_t* wrow[TILES];
  bool n_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + nt * 16 + col;
    n_ok[nt] = n < N;
#pragma unroll
    for (int na = 0; na < NA; ++na) wrow[na * NT + nt] = w + ((size_t)na * N + (n_ok[nt] ? n : 0)) * K;
  }
  const bool m_ok = col < M;
  const bf16_t* xrow = x + (size_t)(m_ok ? col : 0) * K;

  floatx4 acc[TILES];
#pragma unroll
  for (int t = 0; t < TILES; ++t) acc[t] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int ksteps = (K + 31) / 32;
  const int first = wave * steps_per_wave;
  const int last = min(first + steps_per_wave, ksteps);
  // a run: UNROLL steps loaded, then multiplied. (Issuing the next run's loads before this run's products was
  // measured too and changed nothing: enough other waves have loads in flight meanwhile.)
  for (int s0 = first; s0 < last; s0 += UNROLL) {
    bf16x8 a[UNROLL][TILES], b[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (s0 + u) * 32 + grp * 8;
      const bool k_ok = (s0 + u < last) && k < K;      // K is a multiple of 8: a piece is inside or outside as a whole
#pragma unroll
      for (int t = 0; t < TILES; ++t) a[u][t] = (n_ok[t % NT] && k_ok) ? load8(wrow[t] + k) : zero8();
      b[u] = (m_ok && k_ok) ? load8(xrow + k) : zero8();
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < TILES; ++t) acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[u], acc[t], 0, 0, 0);
  }
  if constexpr (FUSED) set_row_scales<WAVES>(f, share, r_s, M, K, wave, lane);
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int j = 0; j < 4; ++j) red[wave][t][j][lane] = acc[t][j];
  __syncthreads();
  if (wave >= NT) return;

  // wave nt adds the waves' sums of tile nt (and of its partner) in the order of the waves
  const int nt = wave;
  float v[NA][4];
#pragma unroll
  for (int na = 0; na < NA; ++na)
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float sum = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][na * NT + nt][j][lane];
      v[na][j] = sum;
    }

  const float rs = (FUSED && f.ss_in) ? r_s[col] : 1.0f;           // the row's scale, where x is a sum whose norm is due
  float out[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + nt * 16 + grp * 4 + j;           // the tile's row 4 grp + j is output n, its column is row col of x
    float r = v[0][j] * rs;
    if (bias && n < N) r += (float)bias[n];
    if (GLU) r = r / (1.0f + expf(-r)) * (v[NA - 1][j] * rs);
    out[j] = r;
  }
  emit_tile<FUSED, TOut>(f, out, y, col, grp, n0 + nt * 16, blockIdx.x * NT + nt, (N + 15) / 16, M, N);
}

typedef __attribute__((address_space(3))) void* lds_ptr;
typedef const __attribute__((address_space(1))) void* global_ptr;

// The kernel with x resident in LDS: x_s[m][K + 8] (the 16 bytes between rows spread the rows over the
// banks), then for tile = blockIdx.x, + gridDim.x, ...: waves split K as above, sums meet in one of two
// LDS buffers (one barrier a tile), and the waves take turns in adding them up and writing the result.
// The first weights of a block's first tile are asked for right after x and the wait before the first product is for
// x alone (0.2 to 0.5 us less per call at every shape; asked for before x they made every shape slower, by 0.5 to
// 3 us).
template <int WAVES, int UNROLL, bool GLU, bool FUSED, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void gemm_fewrows_resident_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                           const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                                           int M, int N, int K, int tiles, int steps_per_wave,
                                                                           const Fusion f) {
  constexpr int NA = GLU ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float(*red)[NA][4][64] = reinterpret_cast<float(*)[NA][4][64]>(lds_raw);      // [2 WAVES][NA][4][64]
  bf16_t* x_s = reinterpret_cast<bf16_t*>(lds_raw + 2 * WAVES * NA * 4 * 64 * sizeof(float));
  const int pitch = K + 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  __shared__ float r_s[16];
  // (the rows' scales are wanted when the first tile goes out: their shares are asked for first of all, and the
  // barrier before the tile's sums are added up makes the scales visible)
  float share[SCALE_ROWS<WAVES>][SCALE_SHARES];
  if constexpr (FUSED) ask_row_scales<WAVES>(f, share, M, wave, lane);
  // x into LDS: a wave's load brings 64 consecutive 16-byte pieces of one row
  const int pieces_per_row = K / 8;
  const int loads_per_row = (pieces_per_row + 63) / 64;
  for (int job = wave; job < M * loads_per_row; job += WAVES) {
    const int m = job / loads_per_row, part = job % loads_per_row;
    const int piece = part * 64 + lane;
    if (piece < pieces_per_row)
      __builtin_amdgcn_global_load_lds((global_ptr)(x + (size_t)m * K + piece * 8), (lds_ptr)(x_s + m * pitch + part * 512), 16, 0, 0);
  }
  const int ksteps = (K + 31) / 32;
  const int first = wave * steps_per_wave;
  const int last = min(first + steps_per_wave, ksteps);
  // The first weights of the block's first tile are asked for while x is still on its way: every lane asks (from an
  // address moved into the matrix where it would lie outside), so that exactly UNROLL NA loads are younger than
  // those of x, and the wait below is for x alone.
  asm volatile("" ::: "memory");
  bf16x8 a_first[UNROLL][NA];
  {
    const int n0 = blockIdx.x * 16;
    const bool n_ok = n0 + col < N;
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (first + u) * 32 + grp * 8;
      const int k_in = k + 8 <= K ? k : 0;
#pragma unroll
      for (int na = 0; na < NA; ++na) a_first[u][na] = load8(w + ((size_t)na * N + (n_ok ? n0 + col : 0)) * K + k_in);
    }
  }
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(UNROLL * NA) : "memory");
  __syncthreads();

  const bool m_ok = col < M;
  const bf16_t* xrow_s = x_s + (m_ok ? col : 0) * pitch;
  int parity = 0, turn = 0;
  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x, parity ^= 1, turn = turn + 1 == WAVES ? 0 : turn + 1) {
    const int n0 = tile * 16;
    const bool n_ok = n0 + col < N;
    // the wave that will write this tile asks for the residual's entries it adds to before the tile's weights
    // (the gated product is never added to a residual stream)
    float res_ahead[8] = {0.f, 0.f, 0.f, 0.f, 1.f, 1.f, 1.f, 1.f};
    if constexpr (FUSED && !GLU) if (f.residual != nullptr && wave == turn) read_residual(f, res_ahead, col, grp, n0, M, N);
    const bf16_t* wrow[NA];
#pragma unroll
    for (int na = 0; na < NA; ++na) wrow[na] = w + ((size_t)na * N + (n_ok ? n0 + col : 0)) * K;
    floatx4 acc[NA];
#pragma unroll
    for (int na = 0; na < NA; ++na) acc[na] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = first; s0 < last; s0 += UNROLL) {
      bf16x8 a[UNROLL][NA];
      const bool asked = tile == (int)blockIdx.x && s0 == first;
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int k = (s0 + u) * 32 + grp * 8;
        const bool k_ok = (s0 + u < last) && k < K;
#pragma unroll
        for (int na = 0; na < NA; ++na) {
          if (asked) a[u][na] = (n_ok && k_ok) ? a_first[u][na] : zero8();
          else a[u][na] = (n_ok && k_ok) ? load8(wrow[na] + k) : zero8();
        }
      }
#pragma unroll
      for (int u = 0; u < UNROLL; ++u) {
        const int k = (s0 + u) * 32 + grp * 8;
        const bool k_ok = (s0 + u < last) && k < K;
        const bf16x8 b = (m_ok && k_ok) ? *reinterpret_cast<const bf16x8*>(xrow_s + k) : zero8();
#pragma unroll
        for (int na = 0; na < NA; ++na) acc[na] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][na], b, acc[na], 0, 0, 0);
      }
    }
    if constexpr (FUSED) if (tile == (int)blockIdx.x) set_row_scales<WAVES>(f, share, r_s, M, K, wave, lane);
    float(*my_red)[NA][4][64] = red + parity * WAVES;
#pragma unroll
    for (int na = 0; na < NA; ++na)
#pragma unroll
      for (int j = 0; j < 4; ++j) my_red[wave][na][j][lane] = acc[na][j];
    __syncthreads();                          // the other buffer is the one written in the next tile
    if (wave != turn) continue;
    float v[NA][4];
#pragma unroll
    for (int na = 0; na < NA; ++na)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) sum += my_red[wv][na][j][lane];
        v[na][j] = sum;
      }
    const float rs = (FUSED && f.ss_in) ? r_s[col] : 1.0f;         // the row's scale, where x is a sum whose norm is due
    float out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + grp * 4 + j;
      float r = v[0][j] * rs;
      if (bias && n < N) r += (float)bias[n];
      if (GLU) r = r / (1.0f + expf(-r)) * (v[NA - 1][j] * rs);
      out[j] = r;
    }
    emit_tile<FUSED && !GLU, TOut>(f, out, y, col, grp, n0, tile, tiles, M, N, res_ahead);
  }
}

// Where all of x is too much for LDS: the same with one tile a block and x coming in `nchunks` pieces of
// `chunk_steps` steps of 32 columns, one after the other; the sums run on over the pieces. (A kernel of its own:
// as an option of the one above it cost that one 4 % of its speed.)
template <int WAVES, int UNROLL, bool FUSED, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void gemm_fewrows_pieces_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                           const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                                           int M, int N, int K, int tiles, int nchunks,
                                                                           int chunk_steps, int steps_per_wave, const Fusion f) {
  constexpr int NA = 1;
  constexpr bool GLU = false;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float(*red)[NA][4][64] = reinterpret_cast<float(*)[NA][4][64]>(lds_raw);      // [2 WAVES][NA][4][64]
  bf16_t* x_s = reinterpret_cast<bf16_t*>(lds_raw + 2 * WAVES * NA * 4 * 64 * sizeof(float));
  const int pitch = min(K, chunk_steps * 32) + 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  __shared__ float r_s[16];
  float share[SCALE_ROWS<WAVES>][SCALE_SHARES];
  if constexpr (FUSED) ask_row_scales<WAVES>(f, share, M, wave, lane);
  const int ksteps = (K + 31) / 32;
  const bool m_ok = col < M;
  const bf16_t* xrow_s = x_s + (m_ok ? col : 0) * pitch;
  // columns [32 c0, 32 c_end) of x into LDS: a wave's load brings 64 consecutive 16-byte pieces of one row
  auto load_x = [&](int c0, int c_end) {
    const int col0 = c0 * 32;
    const int pieces_per_row = (min(K, c_end * 32) - col0) / 8;
    const int loads_per_row = (pieces_per_row + 63) / 64;
    for (int job = wave; job < M * loads_per_row; job += WAVES) {
      const int m = job / loads_per_row, part = job % loads_per_row;
      const int piece = part * 64 + lane;
      if (piece < pieces_per_row)
        __builtin_amdgcn_global_load_lds((global_ptr)(x + (size_t)m * K + col0 + piece * 8),
                                         (lds_ptr)(x_s + m * pitch + part * 512), 16, 0, 0);
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
  };
  int parity = 0, turn = 0;
  for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x, parity ^= 1, turn = turn + 1 == WAVES ? 0 : turn + 1) {
    const int n0 = tile * 16;
    const bool n_ok = n0 + col < N;
    const bf16_t* wrow[NA];
#pragma unroll
    for (int na = 0; na < NA; ++na) wrow[na] = w + ((size_t)na * N + (n_ok ? n0 + col : 0)) * K;
    floatx4 acc[NA];
#pragma unroll
    for (int na = 0; na < NA; ++na) acc[na] = floatx4{0.f, 0.f, 0.f, 0.f};
    for (int c = 0; c < nchunks; ++c) {
      const int c0 = c * chunk_steps, c_end = min(c0 + chunk_steps, ksteps);
      if (c > 0) __syncthreads();                        // the piece before has been read by every wave
      load_x(c0, c_end);
      const int first = c0 + wave * steps_per_wave;
      const int last = min(first + steps_per_wave, c_end);
      for (int s0 = first; s0 < last; s0 += UNROLL) {
        bf16x8 a[UNROLL][NA];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int k = (s0 + u) * 32 + grp * 8;
          const bool k_ok = (s0 + u < last) && k < K;
#pragma unroll
          for (int na = 0; na < NA; ++na) a[u][na] = (n_ok && k_ok) ? load8(wrow[na] + k) : zero8();
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int k = (s0 + u) * 32 + grp * 8;
          const bool k_ok = (s0 + u < last) && k < K;
          const bf16x8 b = (m_ok && k_ok) ? *reinterpret_cast<const bf16x8*>(xrow_s + (k - c0 * 32)) : zero8();
#pragma unroll
          for (int na = 0; na < NA; ++na) acc[na] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][na], b, acc[na], 0, 0, 0);
        }
      }
    }
    if constexpr (FUSED) if (tile == (int)blockIdx.x) set_row_scales<WAVES>(f, share, r_s, M, K, wave, lane);
    float(*my_red)[NA][4][64] = red + parity * WAVES;
#pragma unroll
    for (int na = 0; na < NA; ++na)
#pragma unroll
      for (int j = 0; j < 4; ++j) my_red[wave][na][j][lane] = acc[na][j];
    __syncthreads();                          // the other buffer is the one written in the next tile
    if (wave != turn) continue;
    float v[NA][4];
#pragma unroll
    for (int na = 0; na < NA; ++na)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        float sum = 0.f;
#pragma unroll
        for (int wv = 0; wv < WAVES; ++wv) sum += my_red[wv][na][j][lane];
        v[na][j] = sum;
      }
    const float rs = (FUSED && f.ss_in) ? r_s[col] : 1.0f;         // the row's scale, where x is a sum whose norm is due
    float out[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + grp * 4 + j;
      float r = v[0][j] * rs;
      if (bias && n < N) r += (float)bias[n];
      if (GLU) r = r / (1.0f + expf(-r)) * (v[NA - 1][j] * rs);
      out[j] = r;
    }
    emit_tile<FUSED, TOut>(f, out, y, col, grp, n0, tile, tiles, M, N);
  }
}

// Where all of x is too much for LDS and a block has several tiles: x comes in `npasses` pieces of `pass_steps`
// steps of 32 columns; for every piece the block walks over all of its tiles, and a tile's sums over the pieces so
// far wait in LDS (part_s, 1 KB a tile and matrix) for the next piece. The weights are still read once. The
// wave that adds up a tile's sums is the same in every pass, so what it left in part_s it finds again itself.
template <int WAVES, int UNROLL, bool GLU, bool FUSED, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void gemm_fewrows_passes_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                           const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                                           int M, int N, int K, int tiles, int npasses,
                                                                           int pass_steps, int steps_per_wave, int tiles_per_block,
                                                                           const Fusion f) {
  constexpr int NA = GLU ? 2 : 1;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  float(*red)[NA][4][64] = reinterpret_cast<float(*)[NA][4][64]>(lds_raw);      // [2 WAVES][NA][4][64]
  float(*part_s)[NA][4][64] = red + 2 * WAVES;                                   // [tiles_per_block][NA][4][64]
  bf16_t* x_s = reinterpret_cast<bf16_t*>(lds_raw + (size_t)(2 * WAVES + tiles_per_block) * NA * 4 * 64 * sizeof(float));
  const int pitch = min(K, pass_steps * 32) + 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  __shared__ float r_s[16];
  float share[SCALE_ROWS<WAVES>][SCALE_SHARES];
  if constexpr (FUSED) ask_row_scales<WAVES>(f, share, M, wave, lane);
  const int ksteps = (K + 31) / 32;
  const bool m_ok = col < M;
  const bf16_t* xrow_s = x_s + (m_ok ? col : 0) * pitch;
  int parity = 0;
  for (int p = 0; p < npasses; ++p) {
    const int c0 = p * pass_steps, c_end = min(c0 + pass_steps, ksteps);
    // this piece of x into LDS: a wave's load brings 64 consecutive 16-byte pieces of one row
    if (p > 0) __syncthreads();                          // the piece before has been read by every wave
    {
      const int col0 = c0 * 32;
      const int pieces_per_row = (min(K, c_end * 32) - col0) / 8;
      const int loads_per_row = (pieces_per_row + 63) / 64;
      for (int job = wave; job < M * loads_per_row; job += WAVES) {
        const int m = job / loads_per_row, part = job % loads_per_row;
        const int piece = part * 64 + lane;
        if (piece < pieces_per_row)
          __builtin_amdgcn_global_load_lds((global_ptr)(x + (size_t)m * K + col0 + piece * 8),
                                           (lds_ptr)(x_s + m * pitch + part * 512), 16, 0, 0);
      }
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    const int first = c0 + wave * steps_per_wave;
    const int last = min(first + steps_per_wave, c_end);
    int ti = 0, turn = 0;
    for (int tile = blockIdx.x; tile < tiles; tile += gridDim.x, ++ti, parity ^= 1, turn = turn + 1 == WAVES ? 0 : turn + 1) {
      const int n0 = tile * 16;
      const bool n_ok = n0 + col < N;
      const bf16_t* wrow[NA];
#pragma unroll
      for (int na = 0; na < NA; ++na) wrow[na] = w + ((size_t)na * N + (n_ok ? n0 + col : 0)) * K;
      floatx4 acc[NA];
#pragma unroll
      for (int na = 0; na < NA; ++na) acc[na] = floatx4{0.f, 0.f, 0.f, 0.f};
      for (int s0 = first; s0 < last; s0 += UNROLL) {
        bf16x8 a[UNROLL][NA];
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int k = (s0 + u) * 32 + grp * 8;
          const bool k_ok = (s0 + u < last) && k < K;
#pragma unroll
          for (int na = 0; na < NA; ++na) a[u][na] = (n_ok && k_ok) ? load8(wrow[na] + k) : zero8();
        }
#pragma unroll
        for (int u = 0; u < UNROLL; ++u) {
          const int k = (s0 + u) * 32 + grp * 8;
          const bool k_ok = (s0 + u < last) && k < K;
          const bf16x8 b = (m_ok && k_ok) ? *reinterpret_cast<const bf16x8*>(xrow_s + (k - c0 * 32)) : zero8();
#pragma unroll
          for (int na = 0; na < NA; ++na) acc[na] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][na], b, acc[na], 0, 0, 0);
        }
      }
      if constexpr (FUSED) if (p == 0 && ti == 0) set_row_scales<WAVES>(f, share, r_s, M, K, wave, lane);
      float(*my_red)[NA][4][64] = red + parity * WAVES;
#pragma unroll
      for (int na = 0; na < NA; ++na)
#pragma unroll
        for (int j = 0; j < 4; ++j) my_red[wave][na][j][lane] = acc[na][j];
      __syncthreads();                        // the other buffer is the one written for the next tile
      if (wave != turn) continue;
      float v[NA][4];
#pragma unroll
      for (int na = 0; na < NA; ++na)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float sum = p > 0 ? part_s[ti][na][j][lane] : 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) sum += my_red[wv][na][j][lane];
          v[na][j] = sum;
        }
      if (p + 1 < npasses) {
#pragma unroll
        for (int na = 0; na < NA; ++na)
#pragma unroll
          for (int j = 0; j < 4; ++j) part_s[ti][na][j][lane] = v[na][j];
        continue;
      }
      const float rs = (FUSED && f.ss_in) ? r_s[col] : 1.0f;       // the row's scale, where x is a sum whose norm is due
      float out[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + grp * 4 + j;
        float r = v[0][j] * rs;
        if (bias && n < N) r += (float)bias[n];
        if (GLU) r = r / (1.0f + expf(-r)) * (v[NA - 1][j] * rs);
        out[j] = r;
      }
      emit_tile<FUSED, TOut>(f, out, y, col, grp, n0, tile, tiles, M, N);
    }
  }
}

constexpr size_t LDS_BYTES = 160 * 1024 - 64;      // (64 bytes are the rows' scales, which every kernel keeps beside)

// The resident kernel's shape: waves, loads in flight and blocks per compute unit, from the best variants measured
// (same shapes as below), and in how many pieces x comes; waves == 0 when this kernel is not the one to take.
struct ResidentPlan {
  int waves, unroll, blocks_per_cu, nchunks, chunk_steps;
  size_t lds;
};
static ResidentPlan resident_plan(bool glu, int M, int N, int K) {
  const int tiles = (N + 15) / 16, ksteps = (K + 31) / 32;
  auto lds_of = [&](int waves, int steps) {
    const int columns = steps * 32 < K ? steps * 32 : K;
    return (size_t)2 * waves * (glu ? 2 : 1) * 4 * 64 * sizeof(float) + (size_t)M * (columns + 8) * 2;
  };
  int waves, unroll;
  if (glu) {
    waves = M <= 12 ? 8 : 4;
    unroll = M <= 12 ? 2 : 8;
  } else if (M >= 13) {
    waves = 8, unroll = 8;
  } else if (tiles <= 256 || M > 4 || tiles > 2048) {
    waves = 16, unroll = 2;
  } else {
    waves = 8, unroll = 2;
  }
  int nchunks = 1, chunk_steps = ksteps;
  if (lds_of(waves, ksteps) > LDS_BYTES) {      // fewer waves need less room for their sums
    const int fewer = glu ? 4 : 8;
    if (lds_of(fewer, ksteps) <= LDS_BYTES) {
      waves = fewer, unroll = 8;
    } else {
      // x in pieces: only where every block has one tile (the pieces would come again for every tile) and all
      // blocks are on the chip at once, one a compute unit (with 320 tiles it was measured slower by a quarter)
      if (glu || tiles > 256) return {0, 0, 0, 0, 0, 0};
      for (nchunks = 2; nchunks <= 16; ++nchunks) {
        chunk_steps = 2 * waves * ((ksteps + 2 * waves * nchunks - 1) / (2 * waves * nchunks));   // every wave whole lines
        if (lds_of(waves, chunk_steps) <= LDS_BYTES) break;
      }
      if (nchunks > 16) return {0, 0, 0, 0, 0, 0};
      nchunks = (ksteps + chunk_steps - 1) / chunk_steps;
    }
  }
  if (!glu && waves == 8 && unroll == 2 && 2 * lds_of(8, chunk_steps) > LDS_BYTES) {
    // one block a compute unit: eight waves with two loads each are too little in flight
    if (lds_of(16, chunk_steps) <= LDS_BYTES) waves = 16;
    else unroll = 8;
  }
  const size_t lds = lds_of(waves, chunk_steps);
  const int by_lds = (int)(LDS_BYTES / lds), by_waves = 32 / waves;
  const int bpc = by_lds < by_waves ? by_lds : by_waves;
  return {waves, unroll, bpc < 2 ? 1 : 2, nchunks, chunk_steps, lds};
}

template <int WAVES, int UNROLL, bool GLU, bool PIECES, bool FUSED, typename TOut>
static int launch_resident(const ResidentPlan& p, hipStream_t s, const void* x, const void* w, const void* bias, void* y, int M,
                           int N, int K, const Fusion& f) {
  static_assert(!(GLU && PIECES), "x in pieces is not built for the gated kernel");
  const int steps_per_wave = 2 * ((p.chunk_steps + 2 * WAVES - 1) / (2 * WAVES));
  const int tiles = (N + 15) / 16;
  if constexpr (PIECES) {
    auto kernel = gemm_fewrows_pieces_kernel<WAVES, UNROLL, FUSED, TOut>;
    // more than 64 KB of dynamic LDS has to be allowed once per kernel (and per process)
    static const hipError_t allowed =
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
    if (allowed != hipSuccess) return nhv_fail("few-rows gemm: %s", hipGetErrorString(allowed));
    hipLaunchKernelGGL(kernel, dim3(tiles), dim3(64 * WAVES), p.lds, s, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias,
                       (TOut*)y, M, N, K, tiles, p.nchunks, p.chunk_steps, steps_per_wave, f);
  } else {
    auto kernel = gemm_fewrows_resident_kernel<WAVES, UNROLL, GLU, FUSED, TOut>;
    static const hipError_t allowed =
        hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
    if (allowed != hipSuccess) return nhv_fail("few-rows gemm: %s", hipGetErrorString(allowed));
    const int grid = tiles < 256 * p.blocks_per_cu ? tiles : 256 * p.blocks_per_cu;
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(64 * WAVES), p.lds, s, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias,
                       (TOut*)y, M, N, K, tiles, steps_per_wave, f);
  }
  return 0;
}

// The shape of the kernel that takes x in pieces and walks over all of a block's tiles for every piece: one
// block a compute unit; waves == 0 when it does not fit.
struct PassesPlan {
  int waves, unroll, npasses, pass_steps, tiles_per_block, grid;
  size_t lds;
};
static PassesPlan passes_plan(bool glu, int M, int N, int K) {
  const int tiles = (N + 15) / 16, ksteps = (K + 31) / 32;
  const int grid = tiles < 256 ? tiles : 256;
  const int tpb = (tiles + grid - 1) / grid;
  int waves, unroll;
  if (glu) waves = M <= 12 ? 8 : 4, unroll = M <= 12 ? 2 : 8;
  else waves = M >= 13 ? 8 : 16, unroll = M >= 13 ? 8 : 2;
  const int na = glu ? 2 : 1;
  for (int npasses = 2; npasses <= 8; ++npasses) {
    const int pass_steps = 2 * waves * ((ksteps + 2 * waves * npasses - 1) / (2 * waves * npasses));   // every wave whole lines
    const int columns = pass_steps * 32 < K ? pass_steps * 32 : K;
    const size_t lds = (size_t)(2 * waves + tpb) * na * 4 * 64 * sizeof(float) + (size_t)M * (columns + 8) * 2;
    if (lds <= LDS_BYTES) return {waves, unroll, (ksteps + pass_steps - 1) / pass_steps, pass_steps, tpb, grid, lds};
  }
  return {0, 0, 0, 0, 0, 0, 0};
}

template <int WAVES, int UNROLL, bool GLU, bool FUSED, typename TOut>
static int launch_passes(const PassesPlan& p, hipStream_t s, const void* x, const void* w, const void* bias, void* y, int M, int N,
                         int K, const Fusion& f) {
  auto kernel = gemm_fewrows_passes_kernel<WAVES, UNROLL, GLU, FUSED, TOut>;
  // more than 64 KB of dynamic LDS has to be allowed once per kernel (and per process)
  static const hipError_t allowed =
      hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LDS_BYTES);
  if (allowed != hipSuccess) return nhv_fail("few-rows gemm: %s", hipGetErrorString(allowed));
  const int steps_per_wave = 2 * ((p.pass_steps + 2 * WAVES - 1) / (2 * WAVES));
  hipLaunchKernelGGL(kernel, dim3(p.grid), dim3(64 * WAVES), p.lds, s, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias,
                     (TOut*)y, M, N, K, (N + 15) / 16, p.npasses, p.pass_steps, steps_per_wave, p.tiles_per_block, f);
  return 0;
}

struct Plan {
  int nt, waves, unroll;
};

// Chosen from measurements on an MI355X at the layer and head shapes of the 8B, 14B and 32B models
// (N from 4096 to 151936, K from 4096 to 25600, M = 1, 2, 4, 8, 12, 16). The time of a variant followed
//     (1 + M / (16 NT)) * penalty(NT) / evenness(blocks)
// closely: the rows of x are read once per block, so their share falls with NT; two tiles per block cost
// about an eighth for the parallelism they give up; and `evenness` is how full the last of the rounds of
// 256 blocks (one per compute unit) is. Waves and loads in flight were then taken from the best variants.
static Plan plan(bool glu, int M, int N, int K) {
  const int tiles = (N + 15) / 16;
  auto cost = [&](int nt) {
    const int blocks = (tiles + nt - 1) / nt;
    const int rounds = (blocks + 255) / 256;
    const double evenness = (double)blocks / (256.0 * rounds);
    return (1.0 + M / (16.0 * nt)) * (nt == 2 ? 1.13 : 1.0) / evenness;
  };
  const int nt = cost(2) < cost(1) ? 2 : 1;
  if (glu) {
    if (nt == 2) return {2, 8, 4};
    return tiles <= 1024 ? Plan{1, 4, 4} : Plan{1, 8, 4};
  }
  if (nt == 2) return M <= 8 ? Plan{2, 8, 2} : Plan{2, 4, 4};
  if (tiles > 256 && tiles < 512) return M <= 2 ? Plan{1, 4, 8} : Plan{1, 4, 4};
  return {1, 8, 8};
}

template <int NT, int WAVES, int UNROLL, bool GLU>
static void launch(hipStream_t s, const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                   int out_dtype, bool fused, const Fusion& f) {
  const int ksteps = (K + 31) / 32;
  const int steps_per_wave = 2 * ((ksteps + 2 * WAVES - 1) / (2 * WAVES));     // even: whole cache lines of 128 bytes
  const unsigned blocks = (unsigned)((N + 16 * NT - 1) / (16 * NT));
  if (fused)
    hipLaunchKernelGGL((gemm_fewrows_kernel<NT, WAVES, UNROLL, GLU, true, bf16_t>), dim3(blocks), dim3(64 * WAVES), 0, s,
                       (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (bf16_t*)y, M, N, K, steps_per_wave, f);
  else if (out_dtype == NHV_BF16)
    hipLaunchKernelGGL((gemm_fewrows_kernel<NT, WAVES, UNROLL, GLU, false, bf16_t>), dim3(blocks), dim3(64 * WAVES), 0, s,
                       (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (bf16_t*)y, M, N, K, steps_per_wave, f);
  else
    hipLaunchKernelGGL((gemm_fewrows_kernel<NT, WAVES, UNROLL, GLU, false, float>), dim3(blocks), dim3(64 * WAVES), 0, s,
                       (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (float*)y, M, N, K, steps_per_wave, f);
}

}  // namespace fewrows

// The caller has checked sizes, alignment and types (1 <= M <= 16, K a multiple of 8). Returns 0, or 1 with the
// error message set.
int nhv_gemm_fewrows_launch(bool glu, const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                            int out_dtype, hipStream_t s, const NhvGemmFusion& f) {
  using namespace fewrows;
  // a product that takes over work of its neighbours is a kernel of its own kind (more registers): bfloat16 results only
  const bool fused = f.residual != nullptr || f.ss_in != nullptr;
  if (fused && out_dtype != NHV_BF16) return nhv_fail("few-rows gemm: a product that takes over its neighbours' work gives bfloat16");
  const ResidentPlan rp = resident_plan(glu, M, N, K);
#define NHV_RESIDENT_CASE(WV_, UN_, GLU_, PIECES_)                                                                     \
  if (rp.waves == WV_ && rp.unroll == UN_ && glu == GLU_ && (rp.nchunks > 1) == PIECES_)                              \
    return fused                   ? launch_resident<WV_, UN_, GLU_, PIECES_, true, bf16_t>(rp, s, x, w, bias, y, M, N, K, f)  \
           : out_dtype == NHV_BF16 ? launch_resident<WV_, UN_, GLU_, PIECES_, false, bf16_t>(rp, s, x, w, bias, y, M, N, K, f) \
                                   : launch_resident<WV_, UN_, GLU_, PIECES_, false, float>(rp, s, x, w, bias, y, M, N, K, f);
  NHV_RESIDENT_CASE(8, 2, true, false)
  NHV_RESIDENT_CASE(4, 8, true, false)
  NHV_RESIDENT_CASE(16, 2, false, false)
  NHV_RESIDENT_CASE(8, 2, false, false)
  NHV_RESIDENT_CASE(8, 8, false, false)
  NHV_RESIDENT_CASE(4, 8, false, false)
  NHV_RESIDENT_CASE(16, 2, false, true)
  NHV_RESIDENT_CASE(8, 2, false, true)
  NHV_RESIDENT_CASE(8, 8, false, true)
#undef NHV_RESIDENT_CASE
  if (rp.waves == 0) {
    // two pieces of x were faster than the kernel below in all cases but one tie (gate_up at 16 rows of 5,120
    // columns: 97 against 112 us for 17,408 outputs), three and more pieces slower in most
    const PassesPlan pp = passes_plan(glu, M, N, K);
#define NHV_PASSES_CASE(WV_, UN_, GLU_)                                                                  \
  if (pp.npasses == 2 && pp.waves == WV_ && pp.unroll == UN_ && glu == GLU_)                             \
    return fused                   ? launch_passes<WV_, UN_, GLU_, true, bf16_t>(pp, s, x, w, bias, y, M, N, K, f)  \
           : out_dtype == NHV_BF16 ? launch_passes<WV_, UN_, GLU_, false, bf16_t>(pp, s, x, w, bias, y, M, N, K, f) \
                                   : launch_passes<WV_, UN_, GLU_, false, float>(pp, s, x, w, bias, y, M, N, K, f);
    NHV_PASSES_CASE(8, 2, true)
    NHV_PASSES_CASE(4, 8, true)
    NHV_PASSES_CASE(16, 2, false)
    NHV_PASSES_CASE(8, 8, false)
#undef NHV_PASSES_CASE
  }
  const Plan p = plan(glu, M, N, K);
#define NHV_FEWROWS_CASE(NT_, WV_, UN_, GLU_)                                              \
  if (p.nt == NT_ && p.waves == WV_ && p.unroll == UN_ && glu == GLU_) {                   \
    launch<NT_, WV_, UN_, GLU_>(s, x, w, bias, y, M, N, K, out_dtype, fused, f);           \
    return 0;                                                                              \
  }
  NHV_FEWROWS_CASE(1, 8, 8, false)
  NHV_FEWROWS_CASE(1, 4, 8, false)
  NHV_FEWROWS_CASE(1, 4, 4, false)
  NHV_FEWROWS_CASE(2, 8, 2, false)
  NHV_FEWROWS_CASE(2, 4, 4, false)
  NHV_FEWROWS_CASE(1, 4, 4, true)
  NHV_FEWROWS_CASE(1, 8, 4, true)
  NHV_FEWROWS_CASE(2, 8, 4, true)
#undef NHV_FEWROWS_CASE
  return nhv_fail("few-rows gemm: no kernel for the plan (%d, %d, %d)", p.nt, p.waves, p.unroll);
}
