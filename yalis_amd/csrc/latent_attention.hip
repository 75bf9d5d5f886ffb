// Attention over one latent row per token.  A page row holds [c (kv_rank) | kr (rot_dim)]: the
// normed latent from which every head's keys and values are made, and one rotated key part
// shared by the heads.  The up-projections are applied to the queries and to the attention's
// result instead of to the cached rows:
//   score_h(i, j) = ([W_uk,h^T q_h,i | turn(qr_h,i)] . [c_j | kr_j]) * scale        (float32)
//   o_h,i         = W_uv,h (sum_j softmax_j(score_h(i, .)) c_j)
// so the pages are read as they are, all heads against the same rows.
//
// Three kernels:
//   * latent_prepare: from the stacked down-projection's rows, the normed query latent, and the
//     token's page row (normed latent, rotated key part);
//   * head_linear: per head x[n, h, :in] . W[h] (W [heads][in][out]), with optionally a tail of
//     every head copied behind the product turned by the token's position (queries into the
//     latent's space) or a sigmoid gate per head on the output (values out of it);
//   * latent_attention: a workgroup takes a tile of consecutive tokens of a request and a group
//     of heads (16 pairs at most, four to a wave), walks the keys in blocks staged once in LDS,
//     a lane to a key for the scores and a lane to a latent column for the weighted sum.
#include <algorithm>

#include "common.h"

// --------------------------------------------------------------------------------- prepare
template <typename T, typename TW>
__global__ __launch_bounds__(128) void latent_prepare_kernel(
    const T* __restrict__ proj, int proj_stride, int q_rank, const TW* __restrict__ q_norm, float eps, T* __restrict__ c_q,
    int kv_col, int kv_rank, int rot_dim, const TW* __restrict__ kv_norm, const int32_t* __restrict__ positions,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int interleaved, T* __restrict__ pages,
    T* __restrict__ pages_t, int page_size, const int32_t* __restrict__ slots) {
  __shared__ float scratch[17];
  const size_t n = blockIdx.x;
  const T* row = proj + n * proj_stride;
  float ss = 0.f;
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x) {
    const float v = to_f32<T>(row[c]);
    ss = fmaf(v, v, ss);
  }
  float inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(q_rank) + eps);
  for (int c = threadIdx.x; c < q_rank; c += blockDim.x)
    c_q[n * q_rank + c] = from_f32<T>(to_f32<T>(row[c]) * inv * to_f32<TW>(q_norm[c]));
  if (kv_rank == 0) return;
  const T* kv = row + kv_col;
  ss = 0.f;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const float v = to_f32<T>(kv[c]);
    ss = fmaf(v, v, ss);
  }
  inv = 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(kv_rank) + eps);
  T* dst = pages + static_cast<size_t>(slots[n]) * (kv_rank + rot_dim);
  // pages_t: the latent once more, transposed ([page][column][slot]), for readers that want a column's
  // slots side by side
  const size_t slot = static_cast<size_t>(slots[n]);
  T* dst_t = pages_t == nullptr ? nullptr : pages_t + (slot / page_size) * kv_rank * page_size + slot % page_size;
  for (int c = threadIdx.x; c < kv_rank; c += blockDim.x) {
    const T v = from_f32<T>(to_f32<T>(kv[c]) * inv * to_f32<TW>(kv_norm[c]));
    dst[c] = v;
    if (dst_t != nullptr) dst_t[static_cast<size_t>(c) * page_size] = v;
  }
  const int half = rot_dim / 2;
  const size_t p = static_cast<size_t>(positions[n]);
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const int ia = interleaved ? 2 * i : i, ib = interleaved ? 2 * i + 1 : i + half;
    const float a = to_f32<T>(kv[kv_rank + ia]), b = to_f32<T>(kv[kv_rank + ib]);
    const float c = cos_t[p * half + i], s = sin_t[p * half + i];
    dst[kv_rank + ia] = from_f32<T>(rot_first(a, b, c, s));
    dst[kv_rank + ib] = from_f32<T>(rot_second(a, b, c, s));
  }
}

extern "C" int yk_latent_prepare(const void* proj, int proj_stride, int dtype, int q_rank, const void* q_norm, int w_dtype,
                                 float eps, void* c_q, int kv_col, int kv_rank, int rot_dim, const void* kv_norm,
                                 const int32_t* positions, const float* cos_t, const float* sin_t, int interleaved,
                                 int max_positions, void* pages, void* pages_t, int page_size, const int32_t* slots,
                                 int n_tokens, hipStream_t stream) {
  YK_REQUIRE(pages_t == nullptr || page_size > 0, "latent_prepare: transposed pages need the page size");
  YK_REQUIRE(n_tokens >= 0 && q_rank > 0 && kv_rank >= 0 && rot_dim >= 0 && rot_dim % 2 == 0, "latent_prepare: bad sizes");
  YK_REQUIRE(proj_stride >= q_rank && (kv_rank == 0 || proj_stride >= kv_col + kv_rank + rot_dim),
             "latent_prepare: the projection's rows are shorter than its sections");
  YK_REQUIRE(kv_rank == 0 || (kv_norm != nullptr && pages != nullptr && slots != nullptr && positions != nullptr),
             "latent_prepare: a layer that keeps a cache needs its norm, pages, slots and positions");
  YK_REQUIRE(kv_rank == 0 || rot_dim == 0 || (cos_t != nullptr && sin_t != nullptr && max_positions > 0),
             "latent_prepare: the rotated part needs its tables");
  if (n_tokens == 0) return 0;
#define YK_CASE(D, T, WD, TW)                                                                                         \
  if (dtype == D && w_dtype == WD) {                                                                                  \
    latent_prepare_kernel<T, TW><<<n_tokens, 128, 0, stream>>>(                                                       \
        static_cast<const T*>(proj), proj_stride, q_rank, static_cast<const TW*>(q_norm), eps, static_cast<T*>(c_q),  \
        kv_col, kv_rank, rot_dim, static_cast<const TW*>(kv_norm), positions, cos_t, sin_t, interleaved,              \
        static_cast<T*>(pages), static_cast<T*>(pages_t), page_size, slots);                                          \
    return yk_check_launch("latent_prepare");                                                                         \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("latent_prepare: unsupported dtype combination");
}

// ------------------------------------------------------------------------- per-head products
constexpr int kHeadTokens = 8;   // tokens a workgroup multiplies by one head's matrix
constexpr int kHeadOut = 64;     // output columns a workgroup makes
// SLICES groups of 64 threads divide the input elements among them: four for a handful of tokens (more
// waves on a product that is all latency), one for many (no meeting in LDS, every weight read once a tile)

// out[n, h, o] = sum_i x[n, h, i] w[h][i][o] for a tile of kHeadTokens tokens, one head and kHeadOut
// columns; thread (slice, column) sums every fourth input element, the slices meet in LDS.  TX: the
// input's and TG the gate's element type.
template <typename TX, typename TW, typename TG, typename TO, int kHeadSlices>
__global__ __launch_bounds__(kHeadOut * kHeadSlices) void head_linear_kernel(
    const TX* __restrict__ x, int x_stride, const TW* __restrict__ w, TO* __restrict__ out, int out_stride, int in_dim,
    int out_dim, int tail, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int interleaved, const TG* __restrict__ gate, int gate_stride, int gate_col,
    int gate_elems, int n_tokens) {
  extern __shared__ float xs[];  // [kHeadTokens][in_dim + tail], then [kHeadSlices][kHeadTokens][kHeadOut]
  const int n0 = blockIdx.x * kHeadTokens, h = blockIdx.y, o0 = blockIdx.z * kHeadOut;
  const int count = min(kHeadTokens, n_tokens - n0);
  const int xw = in_dim + tail;
  float* part = xs + kHeadTokens * xw;
  for (int i = threadIdx.x; i < kHeadTokens * xw; i += blockDim.x) {
    const int t = i / xw, c = i % xw;
    xs[i] = t < count ? to_f32<TX>(x[static_cast<size_t>(n0 + t) * x_stride + h * xw + c]) : 0.f;
  }
  __syncthreads();
  const TW* wh = w + static_cast<size_t>(h) * in_dim * out_dim;
  const int ow = out_dim + tail;
  const int slice = threadIdx.x / kHeadOut, o = o0 + threadIdx.x % kHeadOut;
  float acc[kHeadTokens];
#pragma unroll
  for (int t = 0; t < kHeadTokens; ++t) acc[t] = 0.f;
  if (o < out_dim) {
    for (int i0 = slice; i0 < in_dim; i0 += 4 * kHeadSlices) {
      float wv[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = i0 + j * kHeadSlices;
        wv[j] = i < in_dim ? to_f32<TW>(wh[static_cast<size_t>(i) * out_dim + o]) : 0.f;
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int i = min(i0 + j * kHeadSlices, in_dim - 1);
#pragma unroll
        for (int t = 0; t < kHeadTokens; ++t) acc[t] = fmaf(xs[t * xw + i], wv[j], acc[t]);
      }
    }
  }
#pragma unroll
  for (int t = 0; t < kHeadTokens; ++t) part[(slice * kHeadTokens + t) * kHeadOut + threadIdx.x % kHeadOut] = acc[t];
  __syncthreads();
  for (int i = threadIdx.x; i < count * kHeadOut; i += blockDim.x) {
    const int t = i / kHeadOut, oc = i % kHeadOut;
    if (o0 + oc >= out_dim) continue;
    float v = 0.f;
#pragma unroll
    for (int sl = 0; sl < kHeadSlices; ++sl) v += part[(sl * kHeadTokens + t) * kHeadOut + oc];
    if (gate != nullptr)
      v *= 1.f / (1.f + expf(-to_f32<TG>(gate[static_cast<size_t>(n0 + t) * gate_stride + gate_col + h * gate_elems +
                                                  (gate_elems > 1 ? o0 + oc : 0)])));
    out[static_cast<size_t>(n0 + t) * out_stride + h * ow + o0 + oc] = from_f32<TO>(v);
  }
  if (blockIdx.z != 0) return;
  const int half = tail / 2;
  for (int i = threadIdx.x; i < count * half; i += blockDim.x) {
    const int t = i / half, j = i % half;
    const int ia = interleaved ? 2 * j : j, ib = interleaved ? 2 * j + 1 : j + half;
    const float a = xs[t * xw + in_dim + ia], b = xs[t * xw + in_dim + ib];
    const size_t p = static_cast<size_t>(positions[n0 + t]);
    const float c = cos_t[p * half + j], s = sin_t[p * half + j];
    TO* dst = out + static_cast<size_t>(n0 + t) * out_stride + h * ow + out_dim;
    dst[ia] = from_f32<TO>(rot_first(a, b, c, s));
    dst[ib] = from_f32<TO>(rot_second(a, b, c, s));
  }
}

// x, w, gate and out each float32 or bfloat16 (the gate in the output's dtype where the input is float32:
// the way out of the latent; else in the input's)
extern "C" int yk_head_linear(const void* x, int x_stride, int x_dtype, const void* w, int w_dtype, void* out, int out_dtype,
                              int n_heads, int in_dim, int out_dim, int tail, const int32_t* positions, const float* cos_t,
                              const float* sin_t, int interleaved, const void* gate, int gate_dtype, int gate_stride,
                              int gate_col, int gate_elems, int n_tokens, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && in_dim > 0 && out_dim > 0 && tail >= 0 && tail % 2 == 0, "head_linear: bad sizes");
  YK_REQUIRE(gate == nullptr || gate_elems == 1 || gate_elems == out_dim, "head_linear: a gate per head or per output element");
  YK_REQUIRE(x_stride >= n_heads * (in_dim + tail), "head_linear: the input's rows are shorter than its heads");
  YK_REQUIRE(tail == 0 || (positions != nullptr && cos_t != nullptr && sin_t != nullptr), "head_linear: a turned tail needs positions and tables");
  const int slices = 4;
  const size_t lds = sizeof(float) * (static_cast<size_t>(kHeadTokens) * (in_dim + tail) + slices * kHeadTokens * kHeadOut);
  YK_REQUIRE(lds <= 64 * 1024, "head_linear: heads of more than 1,700 input elements do not fit");
  if (n_tokens == 0) return 0;
  dim3 grid((n_tokens + kHeadTokens - 1) / kHeadTokens, n_heads, (out_dim + kHeadOut - 1) / kHeadOut);
  const int out_stride = n_heads * (out_dim + tail);
  if (gate == nullptr) gate_dtype = out_dtype;
#define YK_CASE(XD, TX, WD, TW, GD, TG, OD, TO)                                                                      \
  if (x_dtype == XD && w_dtype == WD && gate_dtype == GD && out_dtype == OD) {                                       \
    if (slices == 1)                                                                                                 \
      head_linear_kernel<TX, TW, TG, TO, 1><<<grid, kHeadOut, lds, stream>>>(                                        \
          static_cast<const TX*>(x), x_stride, static_cast<const TW*>(w), static_cast<TO*>(out), out_stride, in_dim, \
          out_dim, tail, positions, cos_t, sin_t, interleaved, static_cast<const TG*>(gate), gate_stride, gate_col,  \
          gate_elems, n_tokens);                                                                                              \
    else                                                                                                             \
      head_linear_kernel<TX, TW, TG, TO, 4><<<grid, kHeadOut * 4, lds, stream>>>(                                    \
          static_cast<const TX*>(x), x_stride, static_cast<const TW*>(w), static_cast<TO*>(out), out_stride, in_dim, \
          out_dim, tail, positions, cos_t, sin_t, interleaved, static_cast<const TG*>(gate), gate_stride, gate_col,  \
          gate_elems, n_tokens);                                                                                              \
    return yk_check_launch("head_linear");                                                                           \
  }
  YK_CASE(YK_F32, float, YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("head_linear: unsupported dtype combination");
}

// The same products on the matrix cores, for many tokens: bfloat16 weights kept [heads][out][in] (a row of
// the second operand is then 16 bytes of memory a lane), the input bfloat16 or float32 (as two bfloat16
// parts, the rounded value and what the rounding left over, each with its own product).  A wave makes 16 tokens x 64 columns of one head: the first operand is 16 input rows x 32
// elements, loaded as it lies there.  Four waves a workgroup take four token tiles.
typedef __bf16 hl_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float hl_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t hl_u32x4_t __attribute__((ext_vector_type(4)));
union HlFrag {
  hl_u32x4_t u;
  hl_bf16x8_t v;
};

template <typename TX>
__device__ __forceinline__ hl_u32x4_t hl_load8(const TX* p);
template <>
__device__ __forceinline__ hl_u32x4_t hl_load8<bf16_t>(const bf16_t* p) {
  return *reinterpret_cast<const hl_u32x4_t*>(p);
}
template <>
__device__ __forceinline__ hl_u32x4_t hl_load8<float>(const float* p) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  return hl_u32x4_t{pack_bf16x2(a.x, a.y), pack_bf16x2(a.z, a.w), pack_bf16x2(b.x, b.y), pack_bf16x2(b.z, b.w)};
}
// what the rounding of eight floats to bfloat16 left over, itself rounded to bfloat16: a float32 input goes
// through the matrix cores as the sum of the two, so the product sees it to 16 bits of fraction
template <typename TX>
__device__ __forceinline__ hl_u32x4_t hl_rest8(const TX* p, hl_u32x4_t hi);
template <>
__device__ __forceinline__ hl_u32x4_t hl_rest8<bf16_t>(const bf16_t*, hl_u32x4_t) {
  return hl_u32x4_t{0u, 0u, 0u, 0u};
}
__device__ __forceinline__ uint32_t hl_rest2(float x, float y, uint32_t hi) {
  return pack_bf16x2(x - __uint_as_float(hi << 16), y - __uint_as_float(hi & 0xffff0000u));
}
template <>
__device__ __forceinline__ hl_u32x4_t hl_rest8<float>(const float* p, hl_u32x4_t hi) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  return hl_u32x4_t{hl_rest2(a.x, a.y, hi[0]), hl_rest2(a.z, a.w, hi[1]), hl_rest2(b.x, b.y, hi[2]), hl_rest2(b.z, b.w, hi[3])};
}

template <typename TX, typename TG, typename TO>
__global__ __launch_bounds__(256) void head_linear_mfma_kernel(
    const TX* __restrict__ x, int x_stride, const bf16_t* __restrict__ w_t, TO* __restrict__ out, int out_stride, int in_dim,
    int out_dim, int tail, const int32_t* __restrict__ positions, const float* __restrict__ cos_t,
    const float* __restrict__ sin_t, int interleaved, const TG* __restrict__ gate, int gate_stride, int gate_col,
    int gate_elems, int n_tokens) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int r = lane % 16, g = lane / 16;
  const int n0 = (blockIdx.x * 4 + wave) * 16, h = blockIdx.y, o0 = blockIdx.z * 64;
  if (n0 >= n_tokens) return;
  const int xw = in_dim + tail, ow = out_dim + tail;
  const int tok = min(n0 + r, n_tokens - 1);  // (rows past the end repeat the last token and are not stored)
  const TX* xp = x + static_cast<size_t>(tok) * x_stride + h * xw + 8 * g;
  const bf16_t* wp = w_t + (static_cast<size_t>(h) * out_dim + o0 + r) * in_dim + 8 * g;
  hl_f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = hl_f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int n_tiles = min(4, (out_dim - o0) / 16);
  for (int k0 = 0; k0 < in_dim; k0 += 32) {
    HlFrag a, a_rest;
    a.u = hl_load8<TX>(xp + k0);
    a_rest.u = hl_rest8<TX>(xp + k0, a.u);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      if (j < n_tiles) {
        HlFrag b;
        b.u = *reinterpret_cast<const hl_u32x4_t*>(wp + static_cast<size_t>(16 * j) * in_dim + k0);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a.v, b.v, acc[j], 0, 0, 0);
        if (sizeof(TX) == 4) acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_rest.v, b.v, acc[j], 0, 0, 0);
      }
    }
  }
  // acc[j][i]: token n0 + 4 g + i, column o0 + 16 j + r
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = n0 + 4 * g + i;
    if (n >= n_tokens) continue;
    float gv = 1.f;
    const TG* grow = gate == nullptr ? nullptr : gate + static_cast<size_t>(n) * gate_stride + gate_col + h * gate_elems;
    if (gate != nullptr && gate_elems == 1) gv = 1.f / (1.f + expf(-to_f32<TG>(grow[0])));
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (j < n_tiles) {
        if (gate != nullptr && gate_elems > 1) gv = 1.f / (1.f + expf(-to_f32<TG>(grow[o0 + 16 * j + r])));
        out[static_cast<size_t>(n) * out_stride + h * ow + o0 + 16 * j + r] = from_f32<TO>(acc[j][i] * gv);
      }
  }
  if (blockIdx.z != 0 || tail == 0) return;
  const int half = tail / 2;
  for (int i = lane; i < 16 * half; i += kWave) {
    const int t = i / half, j = i % half, n = n0 + t;
    if (n >= n_tokens) break;
    const int ia = interleaved ? 2 * j : j, ib = interleaved ? 2 * j + 1 : j + half;
    const TX* src = x + static_cast<size_t>(n) * x_stride + h * xw + in_dim;
    const float a = to_f32<TX>(src[ia]), b = to_f32<TX>(src[ib]);
    const size_t p = static_cast<size_t>(positions[n]);
    const float c = cos_t[p * half + j], sn = sin_t[p * half + j];
    TO* dst = out + static_cast<size_t>(n) * out_stride + h * ow + out_dim;
    dst[ia] = from_f32<TO>(rot_first(a, b, c, sn));
    dst[ib] = from_f32<TO>(rot_second(a, b, c, sn));
  }
}

extern "C" int yk_head_linear_mfma_ok(int in_dim, int out_dim, int tail) { return in_dim % 32 == 0 && out_dim % 16 == 0 && tail % 8 == 0; }

// w_t: bfloat16 [heads][out_dim][in_dim]; x bfloat16 or float32 with 16-byte aligned rows and heads
extern "C" int yk_head_linear_mfma(const void* x, int x_stride, int x_dtype, const void* w_t, void* out, int out_dtype, int n_heads,
                                   int in_dim, int out_dim, int tail, const int32_t* positions, const float* cos_t,
                                   const float* sin_t, int interleaved, const void* gate, int gate_dtype, int gate_stride,
                                   int gate_col, int gate_elems, int n_tokens, hipStream_t stream) {
  YK_REQUIRE(gate == nullptr || gate_elems == 1 || gate_elems == out_dim, "head_linear_mfma: a gate per head or per output element");
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && yk_head_linear_mfma_ok(in_dim, out_dim, tail), "head_linear_mfma: sizes it is not built for");
  YK_REQUIRE(x_stride >= n_heads * (in_dim + tail) && x_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                 reinterpret_cast<uintptr_t>(w_t) % 16 == 0,
             "head_linear_mfma: the input's rows must be 16-byte aligned");
  YK_REQUIRE(tail == 0 || (positions != nullptr && cos_t != nullptr && sin_t != nullptr), "head_linear_mfma: a turned tail needs positions and tables");
  if (n_tokens == 0) return 0;
  dim3 grid((n_tokens + 63) / 64, n_heads, (out_dim + 63) / 64);
  const int out_stride = n_heads * (out_dim + tail);
  if (gate == nullptr) gate_dtype = out_dtype;
#define YK_CASE(XD, TX, GD, TG, OD, TO)                                                                                 \
  if (x_dtype == XD && gate_dtype == GD && out_dtype == OD) {                                                           \
    head_linear_mfma_kernel<TX, TG, TO><<<grid, 256, 0, stream>>>(                                                      \
        static_cast<const TX*>(x), x_stride, static_cast<const bf16_t*>(w_t), static_cast<TO*>(out), out_stride, in_dim, \
        out_dim, tail, positions, cos_t, sin_t, interleaved, static_cast<const TG*>(gate), gate_stride, gate_col,       \
        gate_elems, n_tokens);                                                                                                      \
    return yk_check_launch("head_linear_mfma");                                                                         \
  }
  YK_CASE(YK_BF16, bf16_t, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("head_linear_mfma: unsupported dtype combination");
}

// --------------------------------------------------------------------------------- attention
constexpr int kLatWaves = 4;       // waves of a workgroup
constexpr int kLatItems = 4;       // (token, head) pairs a wave carries
constexpr int kLatPairs = kLatWaves * kLatItems;

// tiles: rows of (request, first token index in the batch, token count, first position).  Workgroup
// (tile, head group): pair i of it is token i / heads_per_group of the tile and head
// group * heads_per_group + i % heads_per_group; wave w carries the pairs w, w + 4, w + 8, w + 12.
// KB keys are staged per block ([KB][width] in T, rows padded by `pad` elements); RPL latent columns a lane.
template <typename T, int RPL>
__global__ __launch_bounds__(64 * kLatWaves) void latent_attention_kernel(
    const float* __restrict__ q_lat, const T* __restrict__ pages, const int32_t* __restrict__ tiles,
    const int32_t* __restrict__ block_table, int table_width, int page_size, int n_heads, int heads_per_group, int kv_rank,
    int rot_dim, float scale, int KB, int pad, const float* __restrict__ sink, float* __restrict__ out) {
  extern __shared__ unsigned char lds_raw[];
  const int width = kv_rank + rot_dim, row_w = width + pad;
  T* kblock = reinterpret_cast<T*>(lds_raw);                                             // [KB][row_w]
  float* pbuf = reinterpret_cast<float*>(lds_raw + static_cast<size_t>(KB) * row_w * sizeof(T) + 16 -
                                         (static_cast<size_t>(KB) * row_w * sizeof(T)) % 16);  // [kLatPairs][KB]
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int32_t* tile = tiles + 4 * blockIdx.x;
  const int seq = tile[0], tok0 = tile[1], count = tile[2], pos0 = tile[3];
  const int group = blockIdx.y;
  const int n_pairs = count * heads_per_group;
  const int last_pos = pos0 + count - 1;

  // this wave's pairs
  int tok[kLatItems], head[kLatItems], pos[kLatItems];
  bool live[kLatItems];
  float m[kLatItems], l[kLatItems], acc[kLatItems][RPL];
#pragma unroll
  for (int it = 0; it < kLatItems; ++it) {
    const int pair = wave + it * kLatWaves;
    const int t = pair / heads_per_group;
    head[it] = group * heads_per_group + pair % heads_per_group;
    live[it] = pair < n_pairs && head[it] < n_heads;
    tok[it] = tok0 + (live[it] ? t : 0);
    if (!live[it]) head[it] = 0;
    pos[it] = pos0 + (live[it] ? t : 0);
    // a sink is a score without a key: it starts the running maximum and counts once in the sum
    m[it] = sink != nullptr ? sink[head[it]] : -INFINITY;
    l[it] = sink != nullptr ? 1.f : 0.f;
#pragma unroll
    for (int r = 0; r < RPL; ++r) acc[it][r] = 0.f;
  }
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;

  for (int k0 = 0; k0 <= last_pos; k0 += KB) {
    const int nk = min(KB, last_pos + 1 - k0);
    __syncthreads();  // the block before has been read by every wave
    for (int i = threadIdx.x; i < nk * width; i += blockDim.x) {
      const int j = i / width, c = i % width;
      const int key = k0 + j;
      const size_t slot = static_cast<size_t>(bt[key / page_size]) * page_size + key % page_size;
      kblock[j * row_w + c] = pages[slot * width + c];
    }
    __syncthreads();
#pragma unroll
    for (int it = 0; it < kLatItems; ++it) {
      if (!live[it]) continue;  // (uniform over the wave)
      const float* q = q_lat + (static_cast<size_t>(tok[it]) * n_heads + head[it]) * width;
      float* pw = pbuf + (wave + it * kLatWaves) * KB;
      // scores: a lane to a key (KB may exceed 64 never: KB <= 64)
      float s = -INFINITY;
      if (lane < nk && k0 + lane <= pos[it]) {
        const T* kr = kblock + lane * row_w;
        float d = 0.f;
        for (int c = 0; c < width; ++c) d = fmaf(q[c], to_f32<T>(kr[c]), d);
        s = d * scale;
      }
      const float m_new = fmaxf(m[it], wave_max(s));
      const float p = s == -INFINITY ? 0.f : expf(s - m_new);
      const float corr = m[it] == -INFINITY ? 0.f : expf(m[it] - m_new);
      l[it] = l[it] * corr + wave_sum(p);
      m[it] = m_new;
      if (lane < KB) pw[lane] = p;
      // weighted sum of the latent part: a lane to the columns lane, lane + 64, ...
      const int visible = min(nk, pos[it] - k0 + 1);
#pragma unroll
      for (int r = 0; r < RPL; ++r) acc[it][r] *= corr;
      for (int j = 0; j < visible; ++j) {
        const float pj = pw[j];
        const T* kr = kblock + j * row_w;
#pragma unroll
        for (int r = 0; r < RPL; ++r) {
          const int c = lane + r * kWave;
          if (c < kv_rank) acc[it][r] = fmaf(pj, to_f32<T>(kr[c]), acc[it][r]);
        }
      }
    }
  }
#pragma unroll
  for (int it = 0; it < kLatItems; ++it) {
    if (!live[it]) continue;
    const float inv = 1.f / l[it];
    float* o = out + (static_cast<size_t>(tok[it]) * n_heads + head[it]) * kv_rank;
#pragma unroll
    for (int r = 0; r < RPL; ++r) {
      const int c = lane + r * kWave;
      if (c < kv_rank) o[c] = acc[it][r] * inv;
    }
  }
}

extern "C" int yk_latent_tile_tokens(int n_heads) {
  const int hpg = n_heads < kLatItems ? n_heads : kLatItems;
  return kLatPairs / hpg;
}

extern "C" int yk_latent_attention(const float* q_lat, const void* pages, int dtype, const int32_t* tiles, int n_tiles,
                                   const int32_t* block_table, int table_width, int page_size, int n_heads, int kv_rank,
                                   int rot_dim, float scale, const float* sink, float* out, hipStream_t stream) {
  YK_REQUIRE(n_tiles >= 0 && n_heads > 0 && kv_rank > 0 && rot_dim >= 0 && page_size > 0 && table_width > 0,
             "latent_attention: bad sizes");
  YK_REQUIRE(kv_rank <= 16 * kWave, "latent_attention: latents of more than 1,024 elements are not offered");
  if (n_tiles == 0) return 0;
  const int hpg = n_heads < kLatItems ? n_heads : kLatItems;
  const int groups = (n_heads + hpg - 1) / hpg;
  const int width = kv_rank + rot_dim;
  const size_t esz = dtype == YK_BF16 ? 2 : 4;
  // rows a whole number of 32-bit words long and an odd number of them apart: lanes that read the
  // same column of different keys then meet different banks
  int pad = 0;
  while ((static_cast<size_t>(width + pad) * esz) % 4 != 0 || ((static_cast<size_t>(width + pad) * esz) / 4) % 2 == 0) ++pad;
  int KB = 64;
  while (KB > 8 && static_cast<size_t>(KB) * (width + pad) * esz > 96 * 1024) KB /= 2;
  const size_t kbytes = static_cast<size_t>(KB) * (width + pad) * esz;
  YK_REQUIRE(kbytes <= 128 * 1024, "latent_attention: page rows too long for the key block");
  const size_t lds = kbytes + 16 - kbytes % 16 + static_cast<size_t>(kLatPairs) * KB * sizeof(float);
  const int rpl = (kv_rank + kWave - 1) / kWave;
  dim3 grid(n_tiles, groups);
#define YK_LAUNCH(T, R)                                                                                                \
  {                                                                                                                    \
    auto kern = latent_attention_kernel<T, R>;                                                                         \
    if (lds > 64 * 1024 &&                                                                                             \
        hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,          \
                            static_cast<int>(lds)) != hipSuccess)                                                      \
      return yk_fail("latent_attention: the key block does not fit in LDS");                                           \
    kern<<<grid, 64 * kLatWaves, lds, stream>>>(q_lat, static_cast<const T*>(pages), tiles, block_table, table_width,  \
                                                page_size, n_heads, hpg, kv_rank, rot_dim, scale, KB, pad, sink, out);       \
    return yk_check_launch("latent_attention");                                                                        \
  }
#define YK_RPL(T)                      \
  if (rpl <= 1) YK_LAUNCH(T, 1)        \
  if (rpl <= 2) YK_LAUNCH(T, 2)        \
  if (rpl <= 4) YK_LAUNCH(T, 4)        \
  if (rpl <= 8) YK_LAUNCH(T, 8)        \
  YK_LAUNCH(T, 16)
  if (dtype == YK_F32) {
    YK_RPL(float)
  }
  if (dtype == YK_BF16) {
    YK_RPL(bf16_t)
  }
#undef YK_RPL
#undef YK_LAUNCH
  return yk_fail("latent_attention: unsupported dtype");
}

// ------------------------------------------------------------------ attention on the matrix cores
// bfloat16 pages, rows of 32 KS elements of which the first 16 CT are the latent; beside the page
// rows [slot][width] the latent is kept once more transposed, [column][slot], so that both products
// take their first operand from memory as it lies there, 16 bytes a lane:
//   S^T = K . Q^T   (first operand: 16 page rows x 32 elements; second: the queries, in registers)
//   O^T = C^T . P^T (first operand: 16 latent columns x 32 slots of the transposed pages)
// A wave owns 16 columns = (token, head) pairs of one tile: the heads of a token (16 at a time), or
// several tokens' heads where a model has fewer than 16.  It walks the keys in groups of 32; within
// a group the rows of the two score products are assigned to keys so that afterwards lane group g
// holds the probabilities of keys 8g .. 8g + 7 in order (row i is key 8 (i / 4) + i % 4, + 4 for the
// second product), which is the second operand of the other product as it stands.  Each lane keeps
// its column's running maximum and sum.  The four waves of a workgroup take four tiles that follow
// each other, so they ask for the same rows at about the same time.  With n_splits > 1 the groups of
// keys are divided among gridDim.z workgroups, which leave unnormalised sums, maxima and sums of
// weights for a merging kernel.
typedef __bf16 lat_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float lat_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t lat_u32x4_t __attribute__((ext_vector_type(4)));
union LatFrag {
  lat_u32x4_t u;
  lat_bf16x8_t v;
  bf16_t h[8];
};

template <int KS, int CT>
__global__ __launch_bounds__(256, 1) void latent_attention_mfma_kernel(
    const float* __restrict__ q_lat, const bf16_t* __restrict__ kpages, const bf16_t* __restrict__ vpages,
    const int32_t* __restrict__ tiles, int n_tiles, const int32_t* __restrict__ block_table, int table_width, int page_size,
    int n_heads, float scale_log2, int n_splits, const float* __restrict__ sink, float* __restrict__ out, float* __restrict__ ws_o,
    float* __restrict__ ws_ml) {
  constexpr int WIDTH = 32 * KS, RANK = 16 * CT;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave), lane = threadIdx.x % kWave;
  const int tile_i = blockIdx.x * 4 + wave;
  if (tile_i >= n_tiles) return;
  const int r = lane % 16, g = lane / 16;
  const int32_t* tile = tiles + 4 * tile_i;
  const int seq = tile[0], tok0 = tile[1], count = tile[2], pos0 = tile[3];
  const int chunk = blockIdx.y, split = blockIdx.z;
  const int hpt = n_heads < 16 ? n_heads : 16;
  const int tt = r / hpt, hh = r % hpt, head = chunk * 16 + hh;
  const bool col_ok = tt < count && head < n_heads;
  const int my_pos = pos0 + (col_ok ? tt : 0);
  const int last = pos0 + count - 1;

  LatFrag qf[KS];
  {
    const float* qp = q_lat + (static_cast<size_t>(tok0 + (col_ok ? tt : 0)) * n_heads + (col_ok ? head : 0)) * WIDTH + 8 * g;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const float4 a = *reinterpret_cast<const float4*>(qp + 32 * ks), b = *reinterpret_cast<const float4*>(qp + 32 * ks + 4);
      qf[ks].u[0] = col_ok ? pack_bf16x2(a.x, a.y) : 0u;
      qf[ks].u[1] = col_ok ? pack_bf16x2(a.z, a.w) : 0u;
      qf[ks].u[2] = col_ok ? pack_bf16x2(b.x, b.y) : 0u;
      qf[ks].u[3] = col_ok ? pack_bf16x2(b.z, b.w) : 0u;
    }
  }
  const int groups = last / 32 + 1;
  const int per = (groups + n_splits - 1) / n_splits;
  const int g_lo = min(groups, split * per), g_hi = min(groups, g_lo + per);
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;

  float m = -INFINITY, l = 0.f;
  lat_f32x4_t acc[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) acc[ct] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};

  for (int grp = g_lo; grp < g_hi; ++grp) {
    const int k0 = grp * 32;
    const size_t page = static_cast<size_t>(bt[k0 / page_size]);
    const int slot0 = k0 % page_size;
    lat_f32x4_t s[2];
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
      s[sb] = lat_f32x4_t{0.f, 0.f, 0.f, 0.f};
      // the page row behind row r of this product (rows that do not exist yet: the last one that does)
      const int kl = min(8 * (r / 4) + 4 * sb + r % 4, last - k0);
      const bf16_t* krow = kpages + (page * page_size + slot0 + kl) * WIDTH + 8 * g;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks) {
        LatFrag kf;
        kf.u = *reinterpret_cast<const lat_u32x4_t*>(krow + 32 * ks);
        s[sb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf.v, qf[ks].v, s[sb], 0, 0, 0);
      }
    }
    // this lane: column r, keys k0 + 8 g + 4 sb + j
    float tmax = -INFINITY;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int key = k0 + 8 * g + 4 * sb + j;
        s[sb][j] = key <= my_pos ? s[sb][j] * scale_log2 : -INFINITY;
        tmax = fmaxf(tmax, s[sb][j]);
      }
    tmax = column_lanes_max(tmax);
    const float m_new = fmaxf(m, tmax);
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f(m - m_safe);
    float psum = 0.f;
    LatFrag pf;
#pragma unroll
    for (int sb = 0; sb < 2; ++sb) {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        s[sb][j] = __builtin_amdgcn_exp2f(s[sb][j] - m_safe);
        psum += s[sb][j];
      }
      pf.u[2 * sb] = pack_bf16x2(s[sb][0], s[sb][1]);
      pf.u[2 * sb + 1] = pack_bf16x2(s[sb][2], s[sb][3]);
    }
    l = l * alpha + psum;
    m = m_new;
    const bool ragged = k0 + 32 > last + 1;  // slots behind the last key hold whatever was there
    const bf16_t* vcol = vpages + (page * RANK + r) * page_size + slot0 + 8 * g;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      LatFrag vf;
      vf.u = *reinterpret_cast<const lat_u32x4_t*>(vcol + static_cast<size_t>(16 * ct) * page_size);
      if (ragged) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
          if (k0 + 8 * g + e > last) vf.h[e] = 0;
      }
      acc[ct] *= alpha;
      acc[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vf.v, pf.v, acc[ct], 0, 0, 0);
    }
  }
  l = column_lanes_sum(l);
  // acc[ct][j]: latent column 16 ct + 4 g + j of this lane's column r
  if (n_splits == 1) {
    if (!col_ok) return;
    // the sink joins the sum of weights at the end (every column has seen a key: m is finite)
    if (sink != nullptr) l += __builtin_amdgcn_exp2f(sink[head] * 1.4426950408889634f - m);
    const float inv = 1.f / l;
    float* o = out + (static_cast<size_t>(tok0 + tt) * n_heads + head) * RANK + 4 * g;
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
      *reinterpret_cast<float4*>(o + 16 * ct) = make_float4(acc[ct][0] * inv, acc[ct][1] * inv, acc[ct][2] * inv, acc[ct][3] * inv);
    return;
  }
  const size_t part = (static_cast<size_t>(tile_i) * gridDim.y + chunk) * n_splits + split;
  float* o = ws_o + (part * 16 + r) * RANK + 4 * g;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) *reinterpret_cast<float4*>(o + 16 * ct) = make_float4(acc[ct][0], acc[ct][1], acc[ct][2], acc[ct][3]);
  if (g == 0) {
    ws_ml[(part * 16 + r) * 2] = m;
    ws_ml[(part * 16 + r) * 2 + 1] = l;
  }
}

// one workgroup per (tile, head chunk, column): the column's splits merged with weights 2^(m_s - max m), in
// the order of s; the weights are made once, by the first threads, and every thread's loads of a latent
// column's parts are asked for together
__global__ __launch_bounds__(128) void latent_attention_merge_kernel(const float* __restrict__ ws_o, const float* __restrict__ ws_ml,
                                                                     const int32_t* __restrict__ tiles, int n_heads, int rank,
                                                                     int n_splits, const float* __restrict__ sink,
                                                                     float* __restrict__ out) {
  __shared__ float w[256];
  __shared__ float inv_den;
  const int tile_i = blockIdx.x, chunk = blockIdx.y, r = blockIdx.z;
  const int32_t* tile = tiles + 4 * tile_i;
  const int tok0 = tile[1], count = tile[2];
  const int hpt = n_heads < 16 ? n_heads : 16;
  const int tt = r / hpt, head = chunk * 16 + r % hpt;
  if (tt >= count || head >= n_heads) return;
  const size_t part0 = (static_cast<size_t>(tile_i) * gridDim.y + chunk) * n_splits;
  if (threadIdx.x < kWave) {
    float m_max = -INFINITY;
    for (int s = threadIdx.x; s < n_splits; s += kWave) m_max = fmaxf(m_max, ws_ml[((part0 + s) * 16 + r) * 2]);
    m_max = wave_max(m_max);
    float den = 0.f;
    for (int s = threadIdx.x; s < n_splits; s += kWave) {
      const float ws = exp2f(ws_ml[((part0 + s) * 16 + r) * 2] - m_max);
      w[s] = ws;
      den = fmaf(ws, ws_ml[((part0 + s) * 16 + r) * 2 + 1], den);
    }
    den = wave_sum(den);
    if (sink != nullptr) den += exp2f(sink[head] * 1.4426950408889634f - m_max);
    if (threadIdx.x == 0) inv_den = 1.f / den;
  }
  __syncthreads();
  float* o = out + (static_cast<size_t>(tok0 + tt) * n_heads + head) * rank;
  for (int c = 4 * threadIdx.x; c < rank; c += 4 * blockDim.x) {
    float4 num = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int s0 = 0; s0 < n_splits; s0 += 8) {
      float4 v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < n_splits) v[j] = *reinterpret_cast<const float4*>(ws_o + ((part0 + s0 + j) * 16 + r) * rank + c);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        if (s0 + j < n_splits) {
          const float ws = w[s0 + j];
          num.x = fmaf(ws, v[j].x, num.x); num.y = fmaf(ws, v[j].y, num.y);
          num.z = fmaf(ws, v[j].z, num.z); num.w = fmaf(ws, v[j].w, num.w);
        }
    }
    *reinterpret_cast<float4*>(o + c) = make_float4(num.x * inv_den, num.y * inv_den, num.z * inv_den, num.w * inv_den);
  }
}

// sizes the matrix-core form is built for: (page row, latent) = (576, 512), (320, 256), (160, 128), (96, 64), and
// rows that are the latent alone (no rotated part) of 512, 256, 128 or 64 elements
extern "C" int yk_latent_mfma_ok(int kv_rank, int rot_dim, int page_size) {
  const int w = kv_rank + rot_dim;
  const bool size_ok = (w == 576 && kv_rank == 512) || (w == 320 && kv_rank == 256) || (w == 160 && kv_rank == 128) ||
                       (w == 96 && kv_rank == 64) ||
                       (rot_dim == 0 && (kv_rank == 512 || kv_rank == 256 || kv_rank == 128 || kv_rank == 64));
  return size_ok && page_size % 32 == 0 ? 1 : 0;
}

extern "C" int yk_latent_mfma_tile_tokens(int n_heads) { return n_heads >= 16 ? 1 : 16 / n_heads; }

// floats of workspace a launch with these tiles and splits needs
extern "C" size_t yk_latent_mfma_workspace(int n_tiles, int n_heads, int kv_rank, int n_splits) {
  if (n_splits <= 1) return 0;
  const size_t parts = static_cast<size_t>(n_tiles) * ((n_heads + 15) / 16) * n_splits;
  return parts * 16 * (kv_rank + 2);
}

extern "C" int yk_latent_attention_mfma(const float* q_lat, const void* kpages, const void* vpages, const int32_t* tiles,
                                        int n_tiles, const int32_t* block_table, int table_width, int page_size, int n_heads,
                                        int kv_rank, int rot_dim, float scale, int n_splits, const float* sink, float* workspace,
                                        size_t workspace_floats, float* out, hipStream_t stream) {
  YK_REQUIRE(yk_latent_mfma_ok(kv_rank, rot_dim, page_size), "latent_attention_mfma: sizes the matrix-core form is not built for");
  YK_REQUIRE(n_tiles >= 0 && n_heads > 0 && table_width > 0 && n_splits >= 1 && n_splits <= 256, "latent_attention_mfma: bad sizes");
  YK_REQUIRE(workspace_floats >= yk_latent_mfma_workspace(n_tiles, n_heads, kv_rank, n_splits) && (n_splits == 1 || workspace != nullptr),
             "latent_attention_mfma: the workspace is too small");
  if (n_tiles == 0) return 0;
  const int chunks = (n_heads + 15) / 16;
  dim3 grid((n_tiles + 3) / 4, chunks, n_splits);
  const float scale_log2 = scale * 1.4426950408889634f;
  float* ws_o = workspace;
  float* ws_ml = workspace == nullptr ? nullptr : workspace + static_cast<size_t>(n_tiles) * chunks * n_splits * 16 * kv_rank;
#define YK_CASE(KS, CT)                                                                                                      \
  if (kv_rank + rot_dim == 32 * KS && kv_rank == 16 * CT) {                                                                  \
    latent_attention_mfma_kernel<KS, CT><<<grid, 256, 0, stream>>>(                                                          \
        q_lat, static_cast<const bf16_t*>(kpages), static_cast<const bf16_t*>(vpages), tiles, n_tiles, block_table,          \
        table_width, page_size, n_heads, scale_log2, n_splits, sink, out, ws_o, ws_ml);                                            \
    if (yk_check_launch("latent_attention_mfma") != 0) return -1;                                                            \
  }
  YK_CASE(18, 32)
  YK_CASE(10, 16)
  YK_CASE(5, 8)
  YK_CASE(3, 4)
  YK_CASE(16, 32)
  YK_CASE(8, 16)
  YK_CASE(4, 8)
  YK_CASE(2, 4)
#undef YK_CASE
  if (n_splits > 1) {
    latent_attention_merge_kernel<<<dim3(n_tiles, chunks, 16), 128, 0, stream>>>(ws_o, ws_ml, tiles, n_heads, kv_rank, n_splits, sink, out);
    return yk_check_launch("latent_attention_merge");
  }
  return 0;
}
