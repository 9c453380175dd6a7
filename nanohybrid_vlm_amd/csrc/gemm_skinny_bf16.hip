// y[M, N] = x[M, K] . w[N, K]^T (+ bias) in bfloat16 for few rows (M <= 64): the
// matrix product of a decoding step, where every weight is read once and the
// time is the time to stream w from memory.
//
// A block owns 16 rows of w (16 outputs n) and all M rows of x. Its 8 waves split K
// between them in interleaved steps of 32, so that together they read each row of w
// front to back; a wave's lanes load 16 bytes each straight into the MFMA operand
// layout (v_mfma_f32_16x16x32_bf16: w tile as the 16 x 32 operand, x rows as the
// 32 x 16 one), with several loads in flight before the first is used. The waves'
// partial sums meet in LDS and are added in the order of the waves, so the result
// does not depend on timing. Rows of x beyond M and columns beyond K read as zero.
#include "nhv_common.h"

typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float floatx4;

#define SK_WAVES 8
#define SK_UNROLL 4

__device__ __forceinline__ bf16x8 sk_load8(const bf16_t* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 sk_zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

template <int MT, typename TOut>
__global__ __launch_bounds__(64 * SK_WAVES) void gemm_skinny_kernel(const bf16_t* __restrict__ x, const bf16_t* __restrict__ w,
                                                                    const bf16_t* __restrict__ bias, TOut* __restrict__ y,
                                                                    int M, int N, int K) {
  __shared__ float red[SK_WAVES][MT][4][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int col = lane & 15, grp = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n_a = n0 + col;                          // the row of w that this lane loads
  const bool n_ok = n_a < N;
  const bf16_t* wrow = w + (size_t)(n_ok ? n_a : 0) * K;
  const bf16_t* xrow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
    m_ok[mt] = m < M;
    xrow[mt] = x + (size_t)(m_ok[mt] ? m : 0) * K;
  }
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  const int ksteps = (K + 31) / 32;
  for (int base = wave; base < ksteps; base += SK_WAVES * SK_UNROLL) {
    bf16x8 a[SK_UNROLL], b[SK_UNROLL][MT];
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u) {
      const int k = (base + u * SK_WAVES) * 32 + grp * 8;
      const bool k_ok = k < K;                       // K is a multiple of 8: a piece is inside or outside as a whole
      a[u] = (n_ok && k_ok) ? sk_load8(wrow + k) : sk_zero8();
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[u][mt] = (m_ok[mt] && k_ok) ? sk_load8(xrow[mt] + k) : sk_zero8();
    }
#pragma unroll
    for (int u = 0; u < SK_UNROLL; ++u)
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[u], b[u][mt], acc[mt], 0, 0, 0);
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int j = 0; j < 4; ++j) red[wave][mt][j][lane] = acc[mt][j];
  __syncthreads();
  if (wave != 0) return;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + col;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float v = 0.f;
#pragma unroll
      for (int wv = 0; wv < SK_WAVES; ++wv) v += red[wv][mt][j][lane];
      const int n = n0 + grp * 4 + j;               // the tile's row 4 grp + j is output n, its column is row m of x
      if (m < M && n < N) {
        if (bias) v += (float)bias[n];
        y[(size_t)m * N + n] = (TOut)v;
      }
    }
  }
}

extern "C" int nhv_gemm_skinny_bf16(const void* x, const void* w, const void* bias, void* y, int M, int N, int K,
                                    int out_dtype, void* stream) {
  NHV_REQUIRE(M > 0 && N > 0 && K > 0, "skinny gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  NHV_REQUIRE(M <= 64, "skinny gemm: %d rows are beyond this kernel's limit of 64", M);
  NHV_REQUIRE(K % 8 == 0, "skinny gemm: inner size %d must be a multiple of 8", K);
  NHV_REQUIRE(((uintptr_t)x % 16 == 0) && ((uintptr_t)w % 16 == 0), "skinny gemm: operands must be 16-byte aligned");
  const unsigned blocks = (unsigned)((N + 15) / 16);
  hipStream_t s = (hipStream_t)stream;
  const int mt = (M + 15) / 16;
#define LAUNCH(MT, TO)                                                                                            \
  hipLaunchKernelGGL((gemm_skinny_kernel<MT, TO>), dim3(blocks), dim3(64 * SK_WAVES), 0, s, (const bf16_t*)x,     \
                     (const bf16_t*)w, (const bf16_t*)bias, (TO*)y, M, N, K)
#define BY_MT(TO)                \
  if (mt == 1) LAUNCH(1, TO);    \
  else if (mt == 2) LAUNCH(2, TO); \
  else if (mt == 3) LAUNCH(3, TO); \
  else LAUNCH(4, TO)
  if (out_dtype == NHV_BF16) { BY_MT(bf16_t); }
  else if (out_dtype == NHV_F32) { BY_MT(float); }
  else return nhv_fail("skinny gemm: unsupported output type %d", out_dtype);
#undef BY_MT
#undef LAUNCH
  NHV_LAUNCH_CHECK("gemm_skinny_bf16");
  return 0;
}
