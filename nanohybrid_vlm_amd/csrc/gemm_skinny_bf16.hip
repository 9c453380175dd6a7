// y[M, N] = x[M, K] . w[N, K]^T (+ bias) in bfloat16 for few rows (M <= 64): the entry points of the
// matrix products of a decoding step, and the kernel for 17 to 64 rows. Up to 16 rows go to the kernel in
// gemm_fewrows_bf16.hip.
#include "nhv_common.h"
#include "nhv_gemm_fusion.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

int nhv_gemm_fewrows_launch(bool glu, const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                            int out_dtype, hipStream_t s, const NhvGemmFusion& f);
static const NhvGemmFusion NO_FUSION = {};

__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 sk_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// For 17 to 64 rows of x the rows of x are the larger share of what a wave loads, so here a wave keeps NT
// tiles of 16 rows of w (and with GLU their partners in the second matrix) against the same rows of x:
// every load of x serves NT (2 NT) products. The partial sums of the waves meet in LDS one tile at a time.
template <int MT, int NT, int WAVES, int UNROLL, bool GLU, typename TOut>
__global__ __launch_bounds__(64 * WAVES) void gemm_mid_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                              const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                              int M, int N, int K) {
  constexpr int NA = GLU ? 2 : 1;
  constexpr int TILES = NA * NT;
  static_assert(MT <= WAVES, "each of the first MT waves finishes one tile of rows of x");
  __shared__ float red[WAVES][MT][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int n0 = blockIdx.x * 16 * NT;
  const bf16_t* wrow[TILES];
  bool n_ok[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = n0 + nt * 16 + col;
    n_ok[nt] = n < N;
#pragma unroll
    for (int na = 0; na < NA; ++na) wrow[na * NT + nt] = w + ((size_t)na * N + (n_ok[nt] ? n : 0)) * K;
  }
  const bf16_t* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
    m_ok[mt] = m < M;
    xrow[mt] = x + (size_t)(m_ok[mt] ? m : 0) * K;
  }
  floatx4 acc[TILES][MT];
#pragma unroll
  for (int t = 0; t < TILES; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int ksteps = (K + 31) / 32;
  for (int run = wave; run * UNROLL < ksteps; run += WAVES) {
    bf16x8 a[UNROLL][TILES], b[UNROLL][MT];
#pragma unroll
    for (int u = 0; u < UNROLL; ++u) {
      const int k = (run * UNROLL + u) * 32 + grp * 8;
      const bool k_ok = k < K;
#pragma unroll
      for (int t = 0; t < TILES; ++t) a[u][t] = (n_ok[t % NT] && k_ok) ? sk_load8(wrow[t] + k) : sk_zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (m_ok[mt] && k_ok) ? sk_load8(xrow[mt] + k) : sk_zero8();
    }
#pragma unroll
    for (int u = 0; u < UNROLL; ++u)
#pragma unroll
      for (int t = 0; t < TILES; ++t)
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u][t], b[u][mt], acc[t][mt], 0, 0, 0);
  }
  // wave `mt` adds the waves' partial sums of tile (t, mt) in the order of the waves and writes that tile
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    float v[NA][4];
#pragma unroll
    for (int na = 0; na < NA; ++na) {
      __syncthreads();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
#pragma unroll
        for (int j = 0; j < 4; ++j) red[wave][mt][j][lane] = acc[na * NT + nt][mt][j];
      __syncthreads();
      if (wave < MT) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float sum = 0.f;
#pragma unroll
          for (int wv = 0; wv < WAVES; ++wv) sum += red[wv][wave][j][lane];
          v[na][j] = sum;
        }
      }
    }
    if (wave < MT) {
      const int m = wave * 16 + col;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + nt * 16 + grp * 4 + j;
        if (m < M && n < N) {
          float r = v[0][j];
          if (bias) r += (float)bias[n];
          if (GLU) r = r / (1.0f + expf(-r)) * v[NA - 1][j];
          y[(size_t)m * N + n] = (TOut)r;
        }
      }
    }
  }
}

template <int MT, int NT, bool GLU>
static void mid_launch(hipStream_t s, const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                       int out_dtype) {
  constexpr int WAVES = 8, UNROLL = 2;
  const unsigned blocks = (unsigned)((N + 16 * NT - 1) / (16 * NT));
  if (out_dtype == NHV_BF16)
    hipLaunchKernelGGL((gemm_mid_kernel<MT, NT, WAVES, UNROLL, GLU, bf16_t>), dim3(blocks), dim3(64 * WAVES), 0, s,
                       (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (bf16_t*)y, M, N, K);
  else
    hipLaunchKernelGGL((gemm_mid_kernel<MT, NT, WAVES, UNROLL, GLU, float>), dim3(blocks), dim3(64 * WAVES), 0, s,
                       (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (float*)y, M, N, K);
}

// more than 16 rows: how many tiles of w a wave keeps, by how many blocks that leaves for the chip
template <bool GLU>
static void mid_dispatch(hipStream_t s, const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                         int out_dtype) {
  const int mt = (M + 15) / 16;
  const bool wide = !GLU && N >= 16384;
  if (mt == 2) {
    if (wide) mid_launch<2, 4, GLU>(s, x, w, bias, y, M, N, K, out_dtype);
    else mid_launch<2, 2, GLU>(s, x, w, bias, y, M, N, K, out_dtype);
  } else {
    if (wide) mid_launch<4, 4, GLU>(s, x, w, bias, y, M, N, K, out_dtype);
    else mid_launch<4, 2, GLU>(s, x, w, bias, y, M, N, K, out_dtype);
  }
}

static int sk_check(const char* what, const void* x, const void* w, int M, int N, int K, int out_dtype) {
  NHV_REQUIRE(M > 0 && N > 0 && K > 0, "%s: bad sizes M=%d N=%d K=%d", what, M, N, K);
  NHV_REQUIRE(M <= 64, "%s: %d rows are beyond this kernel's limit of 64", what, M);
  NHV_REQUIRE(K % 8 == 0, "%s: inner size %d must be a multiple of 8", what, K);
  NHV_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "%s: operands must be 16-byte aligned", what);
  NHV_REQUIRE(out_dtype == NHV_BF16 || out_dtype == NHV_F32, "%s: unsupported output type %d", what, out_dtype);
  return 0;
}

extern "C" int nhv_gemm_skinny_bf16(const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                                    int out_dtype, void* stream) {
  if (sk_check("skinny gemm", x, w, M, N, K, out_dtype)) return 1;
  hipStream_t s = (hipStream_t)stream;
  if (M > 16) {
    mid_dispatch<false>(s, x, w, bias, y, M, N, K, out_dtype);
    NHV_LAUNCH_CHECK("gemm_mid_bf16");
    return 0;
  }
  if (nhv_gemm_fewrows_launch(false, x, w, bias, y, M, N, K, out_dtype, s, NO_FUSION)) return 1;
  NHV_LAUNCH_CHECK("gemm_fewrows_bf16");
  return 0;
}

// y[M, N] = silu(x . w[0:N]^T) * (x . w[N:2N]^T): the gated feed-forward's first half in one kernel.
extern "C" int nhv_gemm_skinny_glu_bf16(const void* x, const void* w, void* y, int M, int N, int K, int out_dtype,
                                        void* stream) {
  if (sk_check("skinny gated gemm", x, w, M, N, K, out_dtype)) return 1;
  hipStream_t s = (hipStream_t)stream;
  if (M > 16) {
    mid_dispatch<true>(s, x, w, nullptr, y, M, N, K, out_dtype);
    NHV_LAUNCH_CHECK("gemm_mid_glu_bf16");
    return 0;
  }
  if (nhv_gemm_fewrows_launch(true, x, w, nullptr, y, M, N, K, out_dtype, s, NO_FUSION)) return 1;
  NHV_LAUNCH_CHECK("gemm_fewrows_glu_bf16");
  return 0;
}

// ---- products of up to 16 rows that take over the kernels around them (nhv_gemm_fusion.h) ----
// y = r . (x . w^T) (+ bias), or with glu silu(r . (x . w[0:N]^T)) * (r . (x . w[N:2N]^T)), for 1 <= M <= 16 rows in
// bfloat16. With ss_in: x is a sum (times its norm's weight) whose rows still lack their scales: r per row from ss_in
// [M, tiles_in] (the tiles' shares of the row's sum of squares over its K entries) and eps; without: r = 1.
// With residual: the product is not stored; it is added to residual [M, N] (float or bfloat16, rewritten), the sum
// times next_w [N] (if given), rounded, goes to sum_out [M, N] (bfloat16) and the tiles' shares of its rows' sums of
// squares to ss_out [M, (N + 15) / 16]; y is then not touched (may be null). Not with glu.
extern "C" int nhv_gemm_fewrows_fused_bf16(const void* x, const void* ss_in, int tiles_in, float eps, const void* w,
                                           const void* bias, void* y, int M, int N, int K, int out_dtype, int glu,
                                           void* residual, int residual_dtype, void* sum_out, void* ss_out,
                                           const void* next_w, int next_w_dtype, void* stream) {
  if (sk_check("fused few-rows gemm", x, w, M, N, K, out_dtype)) return 1;
  NHV_REQUIRE(M <= 16, "fused few-rows gemm: %d rows are beyond this kernel's limit of 16", M);
  NhvGemmFusion f = {};
  if (ss_in) {
    NHV_REQUIRE(tiles_in > 0 && eps > 0.f, "fused few-rows gemm: the rows' scales need the tiles' count and eps");
    f.ss_in = (const float*)ss_in;
    f.tiles_in = tiles_in;
    f.eps = eps;
  }
  if (residual) {
    NHV_REQUIRE(!glu, "fused few-rows gemm: the gated product is not added to a residual");
    NHV_REQUIRE(sum_out && ss_out, "fused few-rows gemm: the sum and its squares need a place");
    NHV_REQUIRE(residual_dtype == NHV_F32 || residual_dtype == NHV_BF16, "fused few-rows gemm: residual of unknown type %d", residual_dtype);
    NHV_REQUIRE(!next_w || next_w_dtype == NHV_F32 || next_w_dtype == NHV_BF16, "fused few-rows gemm: norm weight of unknown type %d", next_w_dtype);
    f.residual = residual;
    f.residual_f32 = residual_dtype == NHV_F32;
    f.sum_out = (bf16_t*)sum_out;
    f.ss_out = (float*)ss_out;
    f.next_w = next_w;
    f.next_w_f32 = next_w_dtype == NHV_F32;
  } else {
    NHV_REQUIRE(y != nullptr, "fused few-rows gemm: no place for the result");
  }
  if (nhv_gemm_fewrows_launch(glu != 0, x, w, glu ? nullptr : bias, y, M, N, K, out_dtype, (hipStream_t)stream, f)) return 1;
  NHV_LAUNCH_CHECK("gemm_fewrows_fused_bf16");
  return 0;
}
