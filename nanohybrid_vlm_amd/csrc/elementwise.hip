// Embedding gather, RMSNorm (+ residual add), SiLU-and-multiply, row gather and
// the fused q/k-norm + rotation + cache-write kernel. All in two element types
// (float, bfloat16); statistics, angles and sums are float.
#include "nhv_common.h"

// ---------------------------------------------------------------- embedding
// scale: the row is multiplied by it in float and rounded once (1: the row is copied as it is)
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, T* __restrict__ out,
                             int H, int V, float scale) {
  const int t = blockIdx.x;
  int id = ids[t];
  const bool ok = id >= 0 && id < V;   // the host checks ids; an id out of range gives a row of zeros, never a wild read
  const T* src = table + (size_t)(ok ? id : 0) * H;
  T* dst = out + (size_t)t * H;
  if (scale == 1.0f) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = ok ? src[i] : from_f32<T>(0.f);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = ok ? from_f32<T>(to_f32(src[i]) * scale) : from_f32<T>(0.f);
  }
}

extern "C" int nhv_embed(const void* ids, const void* table, void* out, int T, int H, int V, int dtype, float scale,
                         void* stream) {
  NHV_REQUIRE(T > 0 && H > 0 && V > 0, "embed: bad sizes T=%d H=%d V=%d", T, H, V);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(T), dim3(256), 0, s, (const int*)ids, (const float*)table, (float*)out, H, V, scale);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(T), dim3(256), 0, s, (const int*)ids, (const bf16_t*)table, (bf16_t*)out, H, V, scale);
  else
    return nhv_fail("embed: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("embed");
  return 0;
}

// ---------------------------------------------------------------- RMSNorm
// y = round(s * rsqrt(mean(s^2) + eps)) * w in float, s = x or x + residual.
// residual_mode 0: no residual. 1: s = x + residual, and s replaces the residual.
// 2: s = x starts a residual (the first norm of a model). The residual may be kept
// in float while the rows are bfloat16: the sum is then carried unrounded from
// layer to layer. The weight is multiplied after rounding to the element type, as
// a separate rounded product.
template <typename T, typename W, typename R>
__global__ void rmsnorm_kernel(const T* __restrict__ x, R* __restrict__ residual, int residual_mode,
                               const W* __restrict__ w, T* __restrict__ y, int H, float eps) {
  extern __shared__ float row[];          // H floats + 16
  float* scratch = row + H;
  const size_t base = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    float v = to_f32(x[base + i]);
    if (residual_mode == 1) v += to_f32(residual[base + i]);
    if (residual_mode != 0) residual[base + i] = from_f32<R>(v);
    row[i] = v;
    ss += v * v;
  }
  const float total = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(total / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const T n = from_f32<T>(row[i] * r);
    y[base + i] = from_f32<T>(to_f32(n) * to_f32(w[i]));
  }
}

// The same for widths that are a multiple of 8: every thread owns up to MAXC pieces of 8 consecutive entries,
// asks for all of them (rows, residual and weight) before it uses any, and keeps the sums in registers.
template <typename V>
__device__ __forceinline__ void load8f(const V* p, float* out) {
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = to_f32(p[e]);
}
template <>
__device__ __forceinline__ void load8f<bf16_t>(const bf16_t* p, float* out) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 v8;
  const v8 v = *reinterpret_cast<const v8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
}
template <>
__device__ __forceinline__ void load8f<float>(const float* p, float* out) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w; out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
template <typename V>
__device__ __forceinline__ void store8f(V* p, const float* in) {
#pragma unroll
  for (int e = 0; e < 8; ++e) p[e] = from_f32<V>(in[e]);
}
template <>
__device__ __forceinline__ void store8f<bf16_t>(bf16_t* p, const float* in) {
  typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 v8;
  v8 v;
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (__bf16)in[e];
  *reinterpret_cast<v8*>(p) = v;
}
template <>
__device__ __forceinline__ void store8f<float>(float* p, const float* in) {
  *reinterpret_cast<float4*>(p) = make_float4(in[0], in[1], in[2], in[3]);
  *reinterpret_cast<float4*>(p + 4) = make_float4(in[4], in[5], in[6], in[7]);
}

template <typename T, typename W, typename R, int MAXC>
__global__ __launch_bounds__(1024) void rmsnorm_vec_kernel(const T* __restrict__ x, R* __restrict__ residual, int residual_mode,
                                                           const W* __restrict__ w, T* __restrict__ y, int H, float eps) {
  __shared__ float scratch[16];
  const size_t base = (size_t)blockIdx.x * H;
  const int nch = H / 8;
  float v[MAXC][8], wv[MAXC][8];
  float ss = 0.f;
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = threadIdx.x + c * blockDim.x;
    if (ch < nch) {
      load8f<T>(x + base + ch * 8, v[c]);
      load8f<W>(w + ch * 8, wv[c]);
      if (residual_mode == 1) {
        float r8[8];
        load8f<R>(residual + base + ch * 8, r8);
#pragma unroll
        for (int e = 0; e < 8; ++e) v[c][e] += r8[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) v[c][e] = 0.f;
    }
  }
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = threadIdx.x + c * blockDim.x;
    if (ch < nch && residual_mode != 0) store8f<R>(residual + base + ch * 8, v[c]);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[c][e] * v[c][e];
  }
  const float total = block_sum(ss, scratch);
  const float r = 1.0f / sqrtf(total / (float)H + eps);
#pragma unroll
  for (int c = 0; c < MAXC; ++c) {
    const int ch = threadIdx.x + c * blockDim.x;
    if (ch < nch) {
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = to_f32(from_f32<T>(v[c][e] * r)) * wv[c][e];
      store8f<T>(y + base + ch * 8, o);
    }
  }
}

extern "C" int nhv_rmsnorm(const void* x, void* residual, int residual_mode, int residual_dtype, const void* w, void* y,
                           int T, int H, float eps, int dtype, int w_dtype, void* stream) {
  NHV_REQUIRE(T > 0 && H > 0, "rmsnorm: bad sizes T=%d H=%d", T, H);
  NHV_REQUIRE(residual_mode >= 0 && residual_mode <= 2, "rmsnorm: bad residual mode %d", residual_mode);
  NHV_REQUIRE((residual_mode == 0) == (residual == nullptr), "rmsnorm: residual and its mode do not agree");
  const size_t lds = ((size_t)H + 16) * sizeof(float);
  NHV_REQUIRE(lds <= 64 * 1024, "rmsnorm: width %d is beyond this kernel's limit of %d", H, (64 * 1024) / 4 - 16);
  hipStream_t s = (hipStream_t)stream;
  if (residual_mode == 0) residual_dtype = NHV_F32;
  // widths that are a multiple of 8 (with rows that then start on 16-byte borders) take the vector kernel
  const bool vec = H % 8 == 0 && ((uintptr_t)x % 16 == 0) && ((uintptr_t)y % 16 == 0) && ((uintptr_t)w % 16 == 0) &&
                   ((uintptr_t)residual % 16 == 0);
  const int nch = H / 8;
  const int vthreads = nch <= 1024 ? ((nch + 63) / 64) * 64 : 1024;
  const int maxc = (nch + vthreads - 1) / vthreads;       // 1 or 2: H <= 16368
  const int threads = H >= 1024 ? 256 : 64;
#define LAUNCH(TT, WW, RR)                                                                                              \
  do {                                                                                                                  \
    if (vec && maxc == 1)                                                                                               \
      hipLaunchKernelGGL((rmsnorm_vec_kernel<TT, WW, RR, 1>), dim3(T), dim3(vthreads), 0, s, (const TT*)x, (RR*)residual, \
                         residual_mode, (const WW*)w, (TT*)y, H, eps);                                                  \
    else if (vec && maxc == 2)                                                                                          \
      hipLaunchKernelGGL((rmsnorm_vec_kernel<TT, WW, RR, 2>), dim3(T), dim3(vthreads), 0, s, (const TT*)x, (RR*)residual, \
                         residual_mode, (const WW*)w, (TT*)y, H, eps);                                                  \
    else                                                                                                                \
      hipLaunchKernelGGL((rmsnorm_kernel<TT, WW, RR>), dim3(T), dim3(threads), lds, s, (const TT*)x, (RR*)residual,     \
                         residual_mode, (const WW*)w, (TT*)y, H, eps);                                                  \
  } while (0)
  if (dtype == NHV_F32 && w_dtype == NHV_F32 && residual_dtype == NHV_F32) LAUNCH(float, float, float);
  else if (dtype == NHV_BF16 && w_dtype == NHV_BF16 && residual_dtype == NHV_F32) LAUNCH(bf16_t, bf16_t, float);
  else if (dtype == NHV_BF16 && w_dtype == NHV_F32 && residual_dtype == NHV_F32) LAUNCH(bf16_t, float, float);
  else if (dtype == NHV_BF16 && w_dtype == NHV_BF16 && residual_dtype == NHV_BF16) LAUNCH(bf16_t, bf16_t, bf16_t);
  else if (dtype == NHV_BF16 && w_dtype == NHV_F32 && residual_dtype == NHV_BF16) LAUNCH(bf16_t, float, bf16_t);
  else return nhv_fail("rmsnorm: unsupported dtypes x=%d w=%d residual=%d", dtype, w_dtype, residual_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("rmsnorm");
  return 0;
}

// ---------------------------------------------------------------- SiLU(gate) * up
// gu: [T, 2I], gate = first I columns, up = last I. Float inside, rounded once.
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / I, i = idx % I;
    const float g = to_f32(gu[t * 2 * I + i]);
    const float u = to_f32(gu[t * 2 * I + I + i]);
    out[idx] = from_f32<T>(g / (1.0f + expf(-g)) * u);
  }
}

// the same, eight entries a thread (widths that are a multiple of 8)
template <typename T>
__global__ void silu_mul_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total8) {
  const int per_row = I / 8;
  for (size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x; idx < total8; idx += (size_t)gridDim.x * blockDim.x) {
    const size_t t = idx / per_row, c = idx % per_row;
    float g[8], u[8], o[8];
    load8f<T>(gu + t * 2 * I + c * 8, g);
    load8f<T>(gu + t * 2 * I + I + c * 8, u);
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = g[e] / (1.0f + expf(-g[e])) * u[e];
    store8f<T>(out + t * I + c * 8, o);
  }
}

extern "C" int nhv_silu_mul(const void* gu, void* out, int T, int I, int dtype, void* stream) {
  NHV_REQUIRE(T > 0 && I > 0, "silu_mul: bad sizes T=%d I=%d", T, I);
  if (I % 8 == 0 && (uintptr_t)gu % 16 == 0 && (uintptr_t)out % 16 == 0) {
    const size_t total8 = (size_t)T * (I / 8);
    const int vblocks = (int)((total8 + 255) / 256 > 65535 * 16 ? 65535 * 16 : (total8 + 255) / 256);
    hipStream_t vs = (hipStream_t)stream;
    if (dtype == NHV_F32)
      hipLaunchKernelGGL(silu_mul_vec_kernel<float>, dim3(vblocks), dim3(256), 0, vs, (const float*)gu, (float*)out, I, total8);
    else if (dtype == NHV_BF16)
      hipLaunchKernelGGL(silu_mul_vec_kernel<bf16_t>, dim3(vblocks), dim3(256), 0, vs, (const bf16_t*)gu, (bf16_t*)out, I, total8);
    else
      return nhv_fail("silu_mul: unknown dtype %d", dtype);
    NHV_LAUNCH_CHECK("silu_mul");
    return 0;
  }
  const size_t total = (size_t)T * I;
  const int blocks = (int)((total + 255) / 256 > 65535 * 4 ? 65535 * 4 : (total + 255) / 256);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gu, (float*)out, I, total);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, dim3(blocks), dim3(256), 0, s, (const bf16_t*)gu, (bf16_t*)out, I, total);
  else
    return nhv_fail("silu_mul: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("silu_mul");
  return 0;
}

// ---------------------------------------------------------------- row gather
template <typename T>
__global__ void gather_rows_kernel(const T* __restrict__ x, const int* __restrict__ rows, T* __restrict__ out,
                                   int H, int T_in) {
  int r = rows[blockIdx.x];
  const bool ok = r >= 0 && r < T_in;
  const T* src = x + (size_t)(ok ? r : 0) * H;
  T* dst = out + (size_t)blockIdx.x * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) dst[i] = ok ? src[i] : from_f32<T>(0.f);
}

extern "C" int nhv_gather_rows(const void* x, const void* rows, void* out, int n, int H, int T_in, int dtype, void* stream) {
  NHV_REQUIRE(n > 0 && H > 0 && T_in > 0, "gather_rows: bad sizes n=%d H=%d T=%d", n, H, T_in);
  hipStream_t s = (hipStream_t)stream;
  if (dtype == NHV_F32)
    hipLaunchKernelGGL(gather_rows_kernel<float>, dim3(n), dim3(256), 0, s, (const float*)x, (const int*)rows, (float*)out, H, T_in);
  else if (dtype == NHV_BF16)
    hipLaunchKernelGGL(gather_rows_kernel<bf16_t>, dim3(n), dim3(256), 0, s, (const bf16_t*)x, (const int*)rows, (bf16_t*)out, H, T_in);
  else
    return nhv_fail("gather_rows: unknown dtype %d", dtype);
  NHV_LAUNCH_CHECK("gather_rows");
  return 0;
}

// ---------------------------------------------------------------- a soft cap on float logits, in place
__global__ void soft_cap_kernel(float* __restrict__ x, size_t n, float cap) {
  const float inv = 1.0f / cap;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv);
}

extern "C" int nhv_soft_cap(void* x, size_t n, float cap, void* stream) {
  NHV_REQUIRE(n > 0 && cap > 0.f, "soft_cap: needs entries and a positive cap (n=%zu, cap=%g)", n, (double)cap);
  const size_t want = (n + 255) / 256;
  hipLaunchKernelGGL(soft_cap_kernel, dim3((unsigned)(want > 65535 * 8 ? 65535 * 8 : want)), dim3(256), 0, (hipStream_t)stream,
                     (float*)x, n, cap);
  NHV_LAUNCH_CHECK("soft_cap");
  return 0;
}

// ---------------------------------------------------------------- q/k norm + rotation + cache write
// One wave per (token, head) of the packed projection qkv[T, (Hq + 2 Hkv) D]
// (+ bias). q and k heads: optional RMSNorm over the head (rounded, then times
// the weight, rounded), then the first `rot` entries are turned pairwise
// (j, j + rot/2) by the angle of the token's position. q goes to q_out[T, Hq, D];
// k and v go into the paged cache at slot_mapping[t] (a negative slot is skipped).
// cos_sin: [max_pos, rot] float, cos in the first rot/2 columns, sin in the rest.
// positions: [axes, T]; pair_axes (may be null: every pair turns by axis 0): [rot/2], the axis whose coordinate
// gives pair j its angle (the table's row is then looked up pair by pair).
template <typename T, typename W>
__global__ void qk_rope_write_kernel(const T* __restrict__ qkv, const T* __restrict__ bias,
                                     const W* __restrict__ q_norm_w, const W* __restrict__ k_norm_w, float eps,
                                     const float* __restrict__ cos_sin, int rot,
                                     const int* __restrict__ positions, const int* __restrict__ pair_axes, int n_tokens,
                                     const int* __restrict__ slot_mapping,
                                     T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache,
                                     int Hq, int Hkv, int D, int heads_per_token) {
  extern __shared__ float head[];          // D floats
  const int t = blockIdx.x / heads_per_token;
  const int h = blockIdx.x % heads_per_token;
  const int lane = threadIdx.x;
  const int width = (Hq + 2 * Hkv) * D;
  const T* src = qkv + (size_t)t * width + (size_t)h * D;
  const bool is_q = h < Hq;
  const bool is_k = !is_q && h < Hq + Hkv;
  const bool is_v = !is_q && !is_k;

  int slot = -1;
  if (!is_q) {
    slot = slot_mapping[t];
    if (slot < 0) return;                  // whole wave leaves together
  }

  float ss = 0.f;
  for (int d = lane; d < D; d += NHV_WAVE) {
    float v = to_f32(src[d]);
    if (bias) v = to_f32(from_f32<T>(v + to_f32(bias[(size_t)h * D + d])));
    head[d] = v;
    ss += v * v;
  }
  if (is_v) {
    T* dst = v_cache + ((size_t)slot * Hkv + (h - Hq - Hkv)) * D;
    __builtin_amdgcn_wave_barrier();
    for (int d = lane; d < D; d += NHV_WAVE) dst[d] = from_f32<T>(head[d]);
    return;
  }
  const W* nw = is_q ? q_norm_w : k_norm_w;
  if (nw) {
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    for (int d = lane; d < D; d += NHV_WAVE) {
      const T n = from_f32<T>(head[d] * r);
      head[d] = to_f32(from_f32<T>(to_f32(n) * to_f32(nw[d])));
    }
  }
  __syncthreads();                          // one wave per block: orders the LDS writes before the paired reads
  T* dst = is_q ? q_out + ((size_t)t * Hq + h) * D : k_cache + ((size_t)slot * Hkv + (h - Hq)) * D;
  const int half = rot / 2;
  for (int d = lane; d < D; d += NHV_WAVE) {
    float out;
    if (d < rot) {
      const int j = d < half ? d : d - half;
      const int axis = pair_axes ? pair_axes[j] : 0;
      const float* cs = cos_sin + (size_t)positions[(size_t)axis * n_tokens + t] * rot;
      out = d < half ? head[d] * cs[j] - head[d + half] * cs[half + j] : head[d] * cs[j] + head[j] * cs[half + j];
    } else {
      out = head[d];
    }
    dst[d] = from_f32<T>(out);
  }
}

// The same for head sizes that are a power of two (and full or no rotation): CH = D / 8 lanes own a head, eight
// consecutive entries each; the norm's sum and the rotation's partner (entry d +- D/2) come by lane shuffles, nothing
// goes through LDS, and a wave works on 64 / CH heads at once.
template <typename T, typename W, int CH>
__global__ __launch_bounds__(256) void qk_rope_write_vec_kernel(
    const T* __restrict__ qkv, const T* __restrict__ bias, const W* __restrict__ q_norm_w, const W* __restrict__ k_norm_w,
    float eps, const float* __restrict__ cos_sin, int rot, const int* __restrict__ positions,
    const int* __restrict__ slot_mapping, T* __restrict__ q_out, T* __restrict__ k_cache, T* __restrict__ v_cache, int Hq,
    int Hkv, int heads_per_token, long long n_items) {
  constexpr int D = CH * 8;
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long item = gid / CH;
  const int c = (int)(gid % CH);
  if (item >= n_items) return;                       // whole heads leave together
  const int t = (int)(item / heads_per_token), h = (int)(item % heads_per_token);
  const int width = (Hq + 2 * Hkv) * D;
  const bool is_q = h < Hq;
  const bool is_k = !is_q && h < Hq + Hkv;
  // everything that does not hang on another load is asked for before anything is looked at (a key's or value's
  // slot used to be waited for before its entries were asked for, one trip to memory after the other)
  float v[8];
  load8f<T>(qkv + (size_t)t * width + (size_t)h * D + c * 8, v);
  const int pos = rot > 0 ? positions[t] : 0;
  int slot = -1;
  if (!is_q) {
    slot = slot_mapping[t];
    if (slot < 0) return;
  }
  constexpr int HALF_LANES = CH / 2 > 0 ? CH / 2 : 1;
  float cs[8], sn[8];
  if (rot > 0 && (is_q || is_k)) {
    const float* row = cos_sin + (size_t)pos * rot;
    const int j = (c % HALF_LANES) * 8;              // index into the table's cosines; sines lie rot / 2 further
    load8f<float>(row + j, cs);
    load8f<float>(row + rot / 2 + j, sn);
  }
  if (bias) {
    float b[8];
    load8f<T>(bias + (size_t)h * D + c * 8, b);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f32(from_f32<T>(v[e] + b[e]));
  }
  if (!is_q && !is_k) {
    store8f<T>(v_cache + ((size_t)slot * Hkv + (h - Hq - Hkv)) * D + c * 8, v);
    return;
  }
  const W* nw = is_q ? q_norm_w : k_norm_w;
  if (nw) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
#pragma unroll
    for (int off = 1; off < CH; off <<= 1) ss += __shfl_xor(ss, off, NHV_WAVE);
    const float r = 1.0f / sqrtf(ss / (float)D + eps);
    float wv[8];
    load8f<W>(nw + c * 8, wv);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = to_f32(from_f32<T>(to_f32(from_f32<T>(v[e] * r)) * wv[e]));
  }
  float o[8];
  if (rot > 0) {
    const bool first_half = c < HALF_LANES;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float partner = __shfl_xor(v[e], HALF_LANES, NHV_WAVE);
      o[e] = first_half ? v[e] * cs[e] - partner * sn[e] : v[e] * cs[e] + partner * sn[e];
    }
  } else {
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = v[e];
  }
  T* dst = is_q ? q_out + ((size_t)t * Hq + h) * D : k_cache + ((size_t)slot * Hkv + (h - Hq)) * D;
  store8f<T>(dst + c * 8, o);
}

extern "C" int nhv_qk_rope_write(const void* qkv, const void* bias, const void* q_norm_w, const void* k_norm_w, float eps,
                                 const void* cos_sin, int rot, int max_pos, const void* positions, const void* pair_axes,
                                 const void* slot_mapping, void* q_out, void* k_cache, void* v_cache, int T, int Hq,
                                 int Hkv, int D, int write_kv, int dtype, int w_dtype, void* stream) {
  NHV_REQUIRE(T > 0 && Hq > 0 && Hkv > 0 && D > 0, "qk_rope_write: bad sizes T=%d Hq=%d Hkv=%d D=%d", T, Hq, Hkv, D);
  NHV_REQUIRE(rot >= 0 && rot <= D && rot % 2 == 0, "qk_rope_write: rotary size %d must be even and at most head size %d", rot, D);
  NHV_REQUIRE(rot == 0 || (cos_sin && max_pos > 0), "qk_rope_write: rotation table missing");
  NHV_REQUIRE(D <= 4096, "qk_rope_write: head size %d is beyond this kernel's limit of 4096", D);
  NHV_REQUIRE((q_norm_w == nullptr) == (k_norm_w == nullptr), "qk_rope_write: q and k norm weights come together");
  NHV_REQUIRE(!write_kv || (slot_mapping && k_cache && v_cache), "qk_rope_write: cache write without cache");
  const int heads = write_kv ? Hq + 2 * Hkv : Hq;
  const size_t lds = (size_t)D * sizeof(float);
  hipStream_t s = (hipStream_t)stream;
  // power-of-two head sizes from 16 to 512 with full (or no) rotation: the shuffle kernel
  const int ch = D / 8;
  const bool pow2 = D % 8 == 0 && ch >= 2 && ch <= 64 && (ch & (ch - 1)) == 0;
  const bool aligned = (uintptr_t)qkv % 16 == 0 && (uintptr_t)q_out % 16 == 0 && (uintptr_t)k_cache % 16 == 0 &&
                       (uintptr_t)v_cache % 16 == 0 && (uintptr_t)bias % 16 == 0 && (uintptr_t)q_norm_w % 16 == 0 &&
                       (uintptr_t)k_norm_w % 16 == 0 && (uintptr_t)cos_sin % 16 == 0;
  if (pow2 && aligned && (rot == D || rot == 0) && pair_axes == nullptr) {
    const long long n_items = (long long)T * heads;
    const long long vblocks = (n_items * ch + 255) / 256;
    NHV_REQUIRE(vblocks <= 0x7fffffff, "qk_rope_write: too many tokens");
#define VLAUNCH(TT, WW, CHN)                                                                                         \
  hipLaunchKernelGGL((qk_rope_write_vec_kernel<TT, WW, CHN>), dim3((unsigned)vblocks), dim3(256), 0, s, (const TT*)qkv, \
                     (const TT*)bias, (const WW*)q_norm_w, (const WW*)k_norm_w, eps, (const float*)cos_sin, rot,     \
                     (const int*)positions, (const int*)slot_mapping, (TT*)q_out, (TT*)k_cache, (TT*)v_cache, Hq, Hkv, \
                     heads, n_items)
#define VBY_CH(TT, WW)                      \
  switch (ch) {                             \
    case 2: VLAUNCH(TT, WW, 2); break;      \
    case 4: VLAUNCH(TT, WW, 4); break;      \
    case 8: VLAUNCH(TT, WW, 8); break;      \
    case 16: VLAUNCH(TT, WW, 16); break;    \
    case 32: VLAUNCH(TT, WW, 32); break;    \
    default: VLAUNCH(TT, WW, 64); break;    \
  }
    if (dtype == NHV_F32 && w_dtype == NHV_F32) { VBY_CH(float, float) }
    else if (dtype == NHV_BF16 && w_dtype == NHV_BF16) { VBY_CH(bf16_t, bf16_t) }
    else if (dtype == NHV_BF16 && w_dtype == NHV_F32) { VBY_CH(bf16_t, float) }
    else return nhv_fail("qk_rope_write: unsupported dtypes x=%d w=%d", dtype, w_dtype);
#undef VBY_CH
#undef VLAUNCH
    NHV_LAUNCH_CHECK("qk_rope_write");
    return 0;
  }
#define LAUNCH(TT, WW)                                                                                              \
  hipLaunchKernelGGL((qk_rope_write_kernel<TT, WW>), dim3((unsigned)((size_t)T * heads)), dim3(NHV_WAVE), lds, s,  \
                     (const TT*)qkv, (const TT*)bias, (const WW*)q_norm_w, (const WW*)k_norm_w, eps,               \
                     (const float*)cos_sin, rot, (const int*)positions, (const int*)pair_axes, T,                  \
                     (const int*)slot_mapping, (TT*)q_out, (TT*)k_cache, (TT*)v_cache, Hq, Hkv, D, heads)
  if (dtype == NHV_F32 && w_dtype == NHV_F32) LAUNCH(float, float);
  else if (dtype == NHV_BF16 && w_dtype == NHV_BF16) LAUNCH(bf16_t, bf16_t);
  else if (dtype == NHV_BF16 && w_dtype == NHV_F32) LAUNCH(bf16_t, float);
  else return nhv_fail("qk_rope_write: unsupported dtypes x=%d w=%d", dtype, w_dtype);
#undef LAUNCH
  NHV_LAUNCH_CHECK("qk_rope_write");
  return 0;
}

// ---------------------------------------------------------------- rows' scales applied on their own
// y[m][k] = round(x[m][k] * r[m]), r[m] = 1 / sqrt(sum over tiles of ss[m][.] / H + eps): what a few-rows product
// does in its own kernel for a sum whose norm is due (nhv_gemm_fusion.h), for a reader that is no such product.
__global__ void scale_rows_kernel(const bf16_t* __restrict__ x, const float* __restrict__ ss, int tiles, float eps,
                                  bf16_t* __restrict__ y, int H) {
  __shared__ float scratch[16];
  const int m = blockIdx.x;
  float sum = 0.f;
  for (int t = threadIdx.x; t < tiles; t += blockDim.x) sum += ss[(size_t)m * tiles + t];
  const float total = block_sum(sum, scratch);
  const float r = 1.0f / sqrtf(total / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += blockDim.x) y[(size_t)m * H + i] = (bf16_t)((float)x[(size_t)m * H + i] * r);
}

extern "C" int nhv_scale_rows(const void* x, const void* ss, int tiles, float eps, void* y, int M, int H, void* stream) {
  NHV_REQUIRE(M > 0 && H > 0 && tiles > 0, "scale_rows: bad sizes M=%d H=%d tiles=%d", M, H, tiles);
  hipLaunchKernelGGL(scale_rows_kernel, dim3(M), dim3(256), 0, (hipStream_t)stream, (const bf16_t*)x, (const float*)ss, tiles,
                     eps, (bf16_t*)y, H);
  NHV_LAUNCH_CHECK("scale_rows");
  return 0;
}
