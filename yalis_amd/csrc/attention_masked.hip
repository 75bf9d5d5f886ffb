// Attention whose heads are prepared, masked and finished in more ways than the plain causal one:
//
//  * yk_qkv_prepare: what happens to a projection's rows [q heads | k heads | v heads | ...]
//    before the scores: an RMS norm per head on queries and keys (a weight of head_dim elements
//    shared by the heads, or none), rotary positions on the first rotary_dim elements of queries
//    and keys, values divided by their root mean square per head, values rotated by their own
//    table over all of value_dim; queries go to a tensor, keys and values into the pages.
//    Every option can be left out; with none of them it is rotary + append.  More options: a float32 bias per
//    column of the projection, added first; values that are the keys as projected (with the bias, before the norm:
//    the projection then has no value columns); the norm over all of a token's query heads at once (and over all
//    its key heads), with weights as wide as the projections, whose inverse root mean square comes from
//  * yk_qk_row_scales: per token, what its queries and its keys are multiplied with as wholes after the weights:
//    that inverse root mean square and / or the queries' temperature 1 + coef ln(floor((p + 1) / every) + 1).
//  * yk_attn_masked: scores q . k * scale, optionally squashed s <- cap * tanh(s / cap); key j
//    is visible to the query at position p iff j <= p and (p - j < window or j < keep_first)
//    (window 0: no window); softmax over the visible keys; keys of head_dim, values of
//    value_dim elements.  One wave per (token, head), float32 arithmetic, any sizes up to 256.
//    Its epilogue can turn the output back by the query's own position (the inverse of the
//    values' rotation) and multiply a head's output by the sigmoid of a gate column of the
//    projection.
//  * yk_attn_finish: that epilogue alone, in place, for outputs that another attention kernel made.
//
// Norms, angles, scores, softmax and the gate are float32; values are rounded once when stored.
#include <algorithm>

#include "common.h"

namespace {

constexpr int kMaxHead = 256;

// Rotate the first `rot` elements of buf[0..len) (float32, in LDS) by the angles of `pos`;
// lane's elements are lane, lane + 64, ...  `sign` -1 turns the other way.
__device__ __forceinline__ float rotated_element(const float* buf, int i, int rot, int interleaved,
                                                 const float* __restrict__ cos_row,
                                                 const float* __restrict__ sin_row, float sign) {
  if (i >= rot) return buf[i];
  if (interleaved) {
    const int m = i / 2;
    const float c = cos_row[m], s = sign * sin_row[m];
    return (i % 2 == 0) ? rot_first(buf[i], buf[i + 1], c, s) : rot_second(buf[i - 1], buf[i], c, s);
  }
  const int half = rot / 2;
  if (i < half) return rot_first(buf[i], buf[i + half], cos_row[i], sign * sin_row[i]);
  return rot_second(buf[i - half], buf[i], cos_row[i - half], sign * sin_row[i - half]);
}

}  // namespace

// A workgroup of four waves takes four heads of a token (a wave a head).
template <typename TS, typename T, typename TW>
__global__ __launch_bounds__(256) void qkv_prepare_kernel(
    const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum, int src_stride,
    T* __restrict__ q_out, int q_stride, int n_heads, int n_kv, int head_dim, int v_dim,
    const int32_t* __restrict__ positions, const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w,
    int qk_norm, float qk_eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rotary_dim,
    int interleaved, int max_pos, int v_norm, float v_eps, const float* __restrict__ v_cos,
    const float* __restrict__ v_sin, int v_interleaved, int v_max_pos, T* __restrict__ k_cache,
    T* __restrict__ v_cache, const int32_t* __restrict__ slots, int page_size, int tiled,
    const float* __restrict__ bias, const float* __restrict__ row_scales, int v_from_k) {
  __shared__ float bufs[4][kMaxHead];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  float* buf = bufs[wave];
  const int n = blockIdx.x, n_slots = n_heads + 2 * n_kv;
  const bool live = blockIdx.y * 4 + wave < n_slots;  // (a wave beyond the heads works on the last one and stores nothing)
  const int slot_y = min(static_cast<int>(blockIdx.y) * 4 + wave, n_slots - 1);
  const int kind = slot_y < n_heads ? 0 : (slot_y < n_heads + n_kv ? 1 : 2);  // q, k, v
  const int len = kind == 2 ? v_dim : head_dim;
  int col0;
  if (kind == 0) col0 = slot_y * head_dim;
  else if (kind == 1) col0 = n_heads * head_dim + (slot_y - n_heads) * head_dim;
  else if (v_from_k) col0 = n_heads * head_dim + (slot_y - n_heads - n_kv) * head_dim;  // the key head's own columns
  else col0 = (n_heads + n_kv) * head_dim + (slot_y - n_heads - n_kv) * v_dim;
  const TS* row = src + static_cast<size_t>(n) * src_stride + col0;
  // the position, this lane's cosines and sines and the token's slot are asked for before the row
  // is: three waits for memory one behind the other (position, table, row) become two side by side
  const int pos = positions[n];
  const float *cr = nullptr, *sr = nullptr;
  int rot = 0, inter = 0;
  if (kind == 2) {
    if (v_cos != nullptr) {
      const int p = min(pos, v_max_pos - 1);
      rot = v_dim, inter = v_interleaved;
      cr = v_cos + static_cast<size_t>(p) * (v_dim / 2);
      sr = v_sin + static_cast<size_t>(p) * (v_dim / 2);
    }
  } else if (rotary_dim > 0) {
    const int p = min(pos, max_pos - 1);
    rot = rotary_dim, inter = interleaved;
    cr = cos_t + static_cast<size_t>(p) * (rotary_dim / 2);
    sr = sin_t + static_cast<size_t>(p) * (rotary_dim / 2);
  }
  float cv[4], sv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    cv[i] = 1.f, sv[i] = 0.f;
    if (d < rot) {
      const int m = inter ? d / 2 : (d < rot / 2 ? d : d - rot / 2);
      cv[i] = cr[m];
      sv[i] = sr[m];
    }
  }
  const int slot = kind != 0 ? slots[n] : 0;
  float val[4];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    float v = 0.f;
    if (d < len) {
      for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(row[s * split_stride + d]);
      v = as_output(v, round_sum);
      if (bias != nullptr) v += bias[col0 + d];
    }
    val[i] = v;
    ss = fmaf(v, v, ss);
  }
  const bool normed = kind == 2 ? v_norm != 0 : qk_norm == 1;
  if (normed) {
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(len) + (kind == 2 ? v_eps : qk_eps));
    const TW* w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < len) val[i] = val[i] * inv * (w != nullptr ? to_f32<TW>(w[d]) : 1.f);
    }
  } else if (kind != 2 && qk_norm == 2) {
    // the norm over the whole projection: weights as wide as the projection; the inverse root mean square over
    // all heads is part of the row's scale below
    const TW* w = kind == 0 ? q_norm_w + col0 : k_norm_w + (col0 - n_heads * head_dim);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < len) val[i] *= to_f32<TW>(w[d]);
    }
  }
  if (kind != 2 && row_scales != nullptr) {
    const float rs = row_scales[2 * static_cast<size_t>(n) + kind];
#pragma unroll
    for (int i = 0; i < 4; ++i) val[i] *= rs;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < len) buf[d] = val[i];
  }
  __syncthreads();
  size_t base = 0;
  int off = 0;
  if (kind != 0) {
    const int page = slot / page_size, g = kind == 1 ? slot_y - n_heads : slot_y - n_heads - n_kv;
    off = slot % page_size;
    base = (static_cast<size_t>(page) * n_kv + g) * page_size * (kind == 1 ? head_dim : v_dim);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d >= len || !live) continue;
    float v = buf[d];
    if (d < rot) {  // the pair's other element from LDS, the angle from the registers
      if (inter)
        v = (d % 2 == 0) ? rot_first(buf[d], buf[d + 1], cv[i], sv[i]) : rot_second(buf[d - 1], buf[d], cv[i], sv[i]);
      else
        v = d < rot / 2 ? rot_first(buf[d], buf[d + rot / 2], cv[i], sv[i]) : rot_second(buf[d - rot / 2], buf[d], cv[i], sv[i]);
    }
    if (kind == 0)
      q_out[static_cast<size_t>(n) * q_stride + col0 + d] = from_f32<T>(v);
    else if (kind == 1)
      k_cache[base + cache_k_offset(tiled, page_size, head_dim, off, d)] = from_f32<T>(v);
    else
      v_cache[base + cache_v_offset(tiled, page_size, v_dim, off, d)] = from_f32<T>(v);
  }
}

// The same for many tokens of bfloat16: a workgroup of eight waves takes one head of eight
// consecutive tokens of the batch (a wave a token), leaves the finished heads in LDS and stores
// them in pieces of 16 bytes: eight elements of a query or key row, and, where the eight tokens'
// slots run on from a multiple of eight within a page, the eight tokens' values of one element as
// one piece of the transposed page (a token at a time stores each value two bytes wide into a
// row of its own, 128 bytes from the next).
template <typename TS, typename TW>
__global__ __launch_bounds__(512) void qkv_prepare8_kernel(
    const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum, int src_stride,
    bf16_t* __restrict__ q_out, int q_stride, int n_heads, int n_kv, int head_dim, int v_dim,
    const int32_t* __restrict__ positions, const TW* __restrict__ q_norm_w, const TW* __restrict__ k_norm_w,
    int qk_norm, float qk_eps, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rotary_dim,
    int interleaved, int max_pos, int v_norm, float v_eps, const float* __restrict__ v_cos,
    const float* __restrict__ v_sin, int v_interleaved, int v_max_pos, bf16_t* __restrict__ k_cache,
    bf16_t* __restrict__ v_cache, const int32_t* __restrict__ slots, int page_size, int tiled, int n_tokens,
    const float* __restrict__ bias, const float* __restrict__ row_scales, int v_from_k) {
  __shared__ float bufs[8][kMaxHead];
  __shared__ __attribute__((aligned(16))) bf16_t outs[8][kMaxHead];
  __shared__ int slot_s[8];
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64;
  float* buf = bufs[wave];
  const int n0 = blockIdx.x * 8, n_live = min(8, n_tokens - n0);
  const int n = min(n0 + wave, n_tokens - 1);  // (a wave beyond the tokens repeats the last one; nothing of it is stored)
  const int slot_y = blockIdx.y;
  const int kind = slot_y < n_heads ? 0 : (slot_y < n_heads + n_kv ? 1 : 2);  // q, k, v: the same for the workgroup
  const int len = kind == 2 ? v_dim : head_dim;
  int col0;
  if (kind == 0) col0 = slot_y * head_dim;
  else if (kind == 1) col0 = n_heads * head_dim + (slot_y - n_heads) * head_dim;
  else if (v_from_k) col0 = n_heads * head_dim + (slot_y - n_heads - n_kv) * head_dim;  // the key head's own columns
  else col0 = (n_heads + n_kv) * head_dim + (slot_y - n_heads - n_kv) * v_dim;
  const TS* row = src + static_cast<size_t>(n) * src_stride + col0;
  const int pos = positions[n];
  const float *cr = nullptr, *sr = nullptr;
  int rot = 0, inter = 0;
  if (kind == 2) {
    if (v_cos != nullptr) {
      const int p = min(pos, v_max_pos - 1);
      rot = v_dim, inter = v_interleaved;
      cr = v_cos + static_cast<size_t>(p) * (v_dim / 2);
      sr = v_sin + static_cast<size_t>(p) * (v_dim / 2);
    }
  } else if (rotary_dim > 0) {
    const int p = min(pos, max_pos - 1);
    rot = rotary_dim, inter = interleaved;
    cr = cos_t + static_cast<size_t>(p) * (rotary_dim / 2);
    sr = sin_t + static_cast<size_t>(p) * (rotary_dim / 2);
  }
  float cv[4], sv[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    cv[i] = 1.f, sv[i] = 0.f;
    if (d < rot) {
      const int m = inter ? d / 2 : (d < rot / 2 ? d : d - rot / 2);
      cv[i] = cr[m];
      sv[i] = sr[m];
    }
  }
  if (lane == 0) slot_s[wave] = kind != 0 ? slots[n] : 0;
  float val[4];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    float v = 0.f;
    if (d < len) {
      for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(row[s * split_stride + d]);
      v = as_output(v, round_sum);
      if (bias != nullptr) v += bias[col0 + d];
    }
    val[i] = v;
    ss = fmaf(v, v, ss);
  }
  const bool normed = kind == 2 ? v_norm != 0 : qk_norm == 1;
  if (normed) {
    ss = wave_sum(ss);
    const float inv = 1.f / sqrtf(ss / static_cast<float>(len) + (kind == 2 ? v_eps : qk_eps));
    const TW* w = kind == 0 ? q_norm_w : (kind == 1 ? k_norm_w : nullptr);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < len) val[i] = val[i] * inv * (w != nullptr ? to_f32<TW>(w[d]) : 1.f);
    }
  } else if (kind != 2 && qk_norm == 2) {
    // the norm over the whole projection: weights as wide as the projection; the inverse root mean square over
    // all heads is part of the row's scale below
    const TW* w = kind == 0 ? q_norm_w + col0 : k_norm_w + (col0 - n_heads * head_dim);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < len) val[i] *= to_f32<TW>(w[d]);
    }
  }
  if (kind != 2 && row_scales != nullptr) {
    const float rs = row_scales[2 * static_cast<size_t>(n) + kind];
#pragma unroll
    for (int i = 0; i < 4; ++i) val[i] *= rs;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < len) buf[d] = val[i];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d >= len) continue;
    float v = buf[d];
    if (d < rot) {
      if (inter)
        v = (d % 2 == 0) ? rot_first(buf[d], buf[d + 1], cv[i], sv[i]) : rot_second(buf[d - 1], buf[d], cv[i], sv[i]);
      else
        v = d < rot / 2 ? rot_first(buf[d], buf[d + rot / 2], cv[i], sv[i]) : rot_second(buf[d - rot / 2], buf[d], cv[i], sv[i]);
    }
    outs[wave][d] = f32_to_bf16(v);
  }
  __syncthreads();
  const int pieces = len / 8;  // (len is a multiple of 8 here)
  if (kind == 0) {
    for (int idx = threadIdx.x; idx < n_live * pieces; idx += blockDim.x) {
      const int t = idx / pieces, p = idx % pieces;
      *reinterpret_cast<uint4*>(q_out + static_cast<size_t>(n0 + t) * q_stride + col0 + 8 * p) =
          *reinterpret_cast<const uint4*>(&outs[t][8 * p]);
    }
    return;
  }
  const int g = kind == 1 ? slot_y - n_heads : slot_y - n_heads - n_kv;
  const size_t slab = static_cast<size_t>(page_size) * len;
  if (kind == 1) {
    for (int idx = threadIdx.x; idx < n_live * pieces; idx += blockDim.x) {
      const int t = idx / pieces, p = idx % pieces;
      const int slot = slot_s[t];
      const size_t base = (static_cast<size_t>(slot / page_size) * n_kv + g) * slab;
      *reinterpret_cast<uint4*>(k_cache + base + cache_k_offset(tiled, page_size, head_dim, slot % page_size, 8 * p)) =
          *reinterpret_cast<const uint4*>(&outs[t][8 * p]);
    }
    return;
  }
  bool together = n_live == 8 && slot_s[0] % 8 == 0;
#pragma unroll
  for (int t = 1; t < 8; ++t) together = together && slot_s[t] == slot_s[0] + t;
  if (together) {
    const int slot = slot_s[0];
    const size_t base = (static_cast<size_t>(slot / page_size) * n_kv + g) * slab;
    for (int d = threadIdx.x; d < v_dim; d += blockDim.x) {
      uint4 w;
      w.x = outs[0][d] | (static_cast<uint32_t>(outs[1][d]) << 16);
      w.y = outs[2][d] | (static_cast<uint32_t>(outs[3][d]) << 16);
      w.z = outs[4][d] | (static_cast<uint32_t>(outs[5][d]) << 16);
      w.w = outs[6][d] | (static_cast<uint32_t>(outs[7][d]) << 16);
      *reinterpret_cast<uint4*>(v_cache + base + cache_v_offset(tiled, page_size, v_dim, slot % page_size, d)) = w;
    }
    return;
  }
  for (int idx = threadIdx.x; idx < n_live * v_dim; idx += blockDim.x) {
    const int t = idx / v_dim, d = idx % v_dim;
    const int slot = slot_s[t];
    const size_t base = (static_cast<size_t>(slot / page_size) * n_kv + g) * slab;
    v_cache[base + cache_v_offset(tiled, page_size, v_dim, slot % page_size, d)] = outs[t][d];
  }
}

extern "C" int yk_qkv_prepare(const void* src, int src_dtype, int n_splits, int round_sum, int src_stride, void* q_out,
                              int act_dtype, int q_stride, int n_tokens, int n_heads, int n_kv, int head_dim, int v_dim,
                              const int32_t* positions, const void* q_norm_w, const void* k_norm_w, int norm_w_dtype,
                              int qk_norm, float qk_eps, const float* cos_t, const float* sin_t, int rotary_dim,
                              int interleaved, int max_pos, int v_norm, float v_eps, const float* v_cos,
                              const float* v_sin, int v_interleaved, int v_max_pos, void* k_cache, void* v_cache,
                              const int32_t* slots, int page_size, int tiled, const float* bias, const float* row_scales,
                              int v_from_k, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv >= 0, "qkv_prepare: bad sizes");
  YK_REQUIRE(qk_norm >= 0 && qk_norm <= 2 && (qk_norm != 2 || (row_scales != nullptr && q_norm_w != nullptr && (n_kv == 0 || k_norm_w != nullptr))),
             "qkv_prepare: a norm over the whole projection takes its weights and the rows' scales");
  YK_REQUIRE(!v_from_k || v_dim == head_dim, "qkv_prepare: values that are the keys are as wide as the keys");
  YK_REQUIRE(head_dim > 0 && head_dim <= kMaxHead && v_dim > 0 && v_dim <= kMaxHead, "qkv_prepare: heads of 1 to 256 elements");
  YK_REQUIRE(rotary_dim >= 0 && rotary_dim <= head_dim && rotary_dim % 2 == 0, "qkv_prepare: rotary_dim must be even and at most head_dim");
  YK_REQUIRE(rotary_dim == 0 || (cos_t != nullptr && sin_t != nullptr && max_pos > 0), "qkv_prepare: rotary tables missing");
  YK_REQUIRE(v_cos == nullptr || (v_sin != nullptr && v_max_pos > 0 && v_dim % 2 == 0), "qkv_prepare: value tables need an even value_dim");
  YK_REQUIRE(n_kv == 0 || (k_cache != nullptr && v_cache != nullptr && slots != nullptr && page_size > 0), "qkv_prepare: no pages to append to");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "qkv_prepare: unreduced slices must be float32");
  YK_REQUIRE(!tiled || (head_dim == v_dim && cache_is_tiled(act_dtype, head_dim, page_size)), "qkv_prepare: these pages cannot be tiled");
  YK_REQUIRE(n_heads + 2 * n_kv <= 65535, "qkv_prepare: too many heads for one launch");
  if (n_tokens == 0) return 0;
  const size_t stride = static_cast<size_t>(n_tokens) * src_stride;
  auto al16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (act_dtype == YK_BF16 && n_tokens >= 16 && head_dim % 8 == 0 && v_dim % 8 == 0 && q_stride % 8 == 0 && page_size % 8 == 0 &&
      al16(q_out) && al16(k_cache) && al16(v_cache) && (norm_w_dtype == YK_BF16 || norm_w_dtype == YK_F32)) {
    dim3 grid8((n_tokens + 7) / 8, n_heads + 2 * n_kv);
#define YK_CASE8(SD, TS, WD, TW)                                                                              \
  if (src_dtype == SD && (norm_w_dtype == WD || (q_norm_w == nullptr && k_norm_w == nullptr && WD == YK_F32))) { \
    qkv_prepare8_kernel<TS, TW><<<grid8, 512, 0, stream>>>(                                                    \
        static_cast<const TS*>(src), n_splits, stride, round_sum, src_stride, static_cast<bf16_t*>(q_out), q_stride, \
        n_heads, n_kv, head_dim, v_dim, positions, static_cast<const TW*>(q_norm_w),                           \
        static_cast<const TW*>(k_norm_w), qk_norm, qk_eps, cos_t, sin_t, rotary_dim, interleaved, max_pos,      \
        v_norm, v_eps, v_cos, v_sin, v_interleaved, v_max_pos, static_cast<bf16_t*>(k_cache),                  \
        static_cast<bf16_t*>(v_cache), slots, page_size, tiled, n_tokens, bias, row_scales, v_from_k);         \
    return yk_check_launch("qkv_prepare (8 tokens)");                                                          \
  }
    YK_CASE8(YK_F32, float, YK_F32, float)
    YK_CASE8(YK_F32, float, YK_BF16, bf16_t)
    YK_CASE8(YK_BF16, bf16_t, YK_F32, float)
    YK_CASE8(YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE8
  }
  dim3 grid(n_tokens, (n_heads + 2 * n_kv + 3) / 4), block(256);
#define YK_CASE(SD, TS, AD, T, WD, TW)                                                                       \
  if (src_dtype == SD && act_dtype == AD && (norm_w_dtype == WD || (q_norm_w == nullptr && k_norm_w == nullptr && WD == YK_F32))) { \
    qkv_prepare_kernel<TS, T, TW><<<grid, block, 0, stream>>>(                                                \
        static_cast<const TS*>(src), n_splits, stride, round_sum, src_stride, static_cast<T*>(q_out), q_stride,  \
        n_heads, n_kv, head_dim, v_dim, positions, static_cast<const TW*>(q_norm_w),                          \
        static_cast<const TW*>(k_norm_w), qk_norm, qk_eps, cos_t, sin_t, rotary_dim, interleaved, max_pos,     \
        v_norm, v_eps, v_cos, v_sin, v_interleaved, v_max_pos, static_cast<T*>(k_cache), static_cast<T*>(v_cache), \
        slots, page_size, tiled, bias, row_scales, v_from_k);                                                 \
    return yk_check_launch("qkv_prepare");                                                                    \
  }
  YK_CASE(YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("qkv_prepare: unsupported dtype combination");
}

// ------------------------------------------------------------------ what scales a token's rows as wholes
// out[n][0] for the queries, out[n][1] for the keys: 1 / sqrt(mean(x^2) + eps) over all n_q_cols query columns (all
// n_k_cols key columns) of the biased projection when `normed`, times, for the queries, the temperature
// 1 + coef * ln(floor((p + 1) / every) + 1) of the token's position p when every > 0.  A workgroup a token.
template <typename TS, bool VEC>
__global__ __launch_bounds__(1024) void qk_row_scales_kernel(
    const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum, int src_stride, int n_q_cols, int n_k_cols,
    const float* __restrict__ bias, int normed, float eps, const int32_t* __restrict__ positions, float temp_coef,
    int temp_every, float* __restrict__ out) {
  __shared__ float part[16][2];
  const int n = blockIdx.x, wave = threadIdx.x / 64, lane = threadIdx.x % 64, n_waves = blockDim.x / 64;
  float sq = 1.f, sk = 1.f;
  if (normed) {
    const TS* row = src + static_cast<size_t>(n) * src_stride;
    const int total = n_q_cols + n_k_cols;
    float ssq = 0.f, ssk = 0.f;
    if (VEC) {
      // bfloat16 rows in pieces of 16 bytes (the launcher checked the alignment and that a piece holds queries or
      // keys, never both)
      for (int c = threadIdx.x * 8; c < total; c += 8 * blockDim.x) {
        const uint4 raw = *reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(row) + c);
        float v[8] = {__uint_as_float(raw.x << 16), __uint_as_float(raw.x & 0xffff0000u), __uint_as_float(raw.y << 16),
                      __uint_as_float(raw.y & 0xffff0000u), __uint_as_float(raw.z << 16), __uint_as_float(raw.z & 0xffff0000u),
                      __uint_as_float(raw.w << 16), __uint_as_float(raw.w & 0xffff0000u)};
        if (bias != nullptr) {
          const float4 b0 = *reinterpret_cast<const float4*>(bias + c), b1 = *reinterpret_cast<const float4*>(bias + c + 4);
          v[0] += b0.x, v[1] += b0.y, v[2] += b0.z, v[3] += b0.w, v[4] += b1.x, v[5] += b1.y, v[6] += b1.z, v[7] += b1.w;
        }
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) ss = fmaf(v[e], v[e], ss);
        if (c < n_q_cols) ssq += ss;
        else ssk += ss;
      }
    } else {
      for (int c = threadIdx.x; c < total; c += blockDim.x) {
        float v = 0.f;
#pragma unroll 8
        for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(row[s * split_stride + c]);
        v = as_output(v, round_sum);
        if (bias != nullptr) v += bias[c];
        if (c < n_q_cols) ssq = fmaf(v, v, ssq);
        else ssk = fmaf(v, v, ssk);
      }
    }
    ssq = wave_sum(ssq);
    ssk = wave_sum(ssk);
    if (lane == 0) part[wave][0] = ssq, part[wave][1] = ssk;
    __syncthreads();
    if (threadIdx.x == 0) {
      ssq = ssk = 0.f;
      for (int w = 0; w < n_waves; ++w) ssq += part[w][0], ssk += part[w][1];
      sq = 1.f / sqrtf(ssq / static_cast<float>(n_q_cols) + eps);
      if (n_k_cols > 0) sk = 1.f / sqrtf(ssk / static_cast<float>(n_k_cols) + eps);
    }
  }
  if (threadIdx.x == 0) {
    if (temp_every > 0) sq *= 1.f + temp_coef * logf(static_cast<float>((positions[n] + 1) / temp_every + 1));
    out[2 * static_cast<size_t>(n)] = sq;
    out[2 * static_cast<size_t>(n) + 1] = sk;
  }
}

extern "C" int yk_qk_row_scales(const void* src, int src_dtype, int n_splits, int round_sum, int src_stride, int n_tokens,
                                int n_q_cols, int n_k_cols, const float* bias, int normed, float eps, const int32_t* positions,
                                float temp_coef, int temp_every, float* out, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_q_cols > 0 && n_k_cols >= 0 && src_stride >= n_q_cols + n_k_cols, "qk_row_scales: bad sizes");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "qk_row_scales: unreduced slices must be float32");
  YK_REQUIRE(temp_every >= 0 && (temp_every == 0 || positions != nullptr) && eps >= 0.f, "qk_row_scales: bad constants");
  if (n_tokens == 0) return 0;
  const size_t stride = static_cast<size_t>(n_tokens) * src_stride;
  // few tokens (single decoded ones, whose projection comes as slices): a token's columns over sixteen waves
  const int grid = n_tokens, block = n_tokens <= 256 ? 1024 : 256;
  const bool vec = src_dtype == YK_BF16 && n_splits == 1 && n_q_cols % 8 == 0 && n_k_cols % 8 == 0 && src_stride % 8 == 0 &&
                   reinterpret_cast<uintptr_t>(src) % 16 == 0 && reinterpret_cast<uintptr_t>(bias) % 16 == 0;
  if (src_dtype == YK_F32)
    qk_row_scales_kernel<float, false><<<grid, block, 0, stream>>>(static_cast<const float*>(src), n_splits, stride, round_sum, src_stride,
                                                                 n_q_cols, n_k_cols, bias, normed, eps, positions, temp_coef,
                                                                 temp_every, out);
  else if (src_dtype == YK_BF16 && vec)
    qk_row_scales_kernel<bf16_t, true><<<grid, block, 0, stream>>>(static_cast<const bf16_t*>(src), n_splits, stride, round_sum, src_stride,
                                                                 n_q_cols, n_k_cols, bias, normed, eps, positions, temp_coef,
                                                                 temp_every, out);
  else if (src_dtype == YK_BF16)
    qk_row_scales_kernel<bf16_t, false><<<grid, block, 0, stream>>>(static_cast<const bf16_t*>(src), n_splits, stride, round_sum, src_stride,
                                                                  n_q_cols, n_k_cols, bias, normed, eps, positions, temp_coef,
                                                                  temp_every, out);
  else
    return yk_fail("qk_row_scales: unsupported dtype");
  return yk_check_launch("qk_row_scales");
}

// ------------------------------------------------------------------------------ the finish
// One head's output `os` [v_dim] (float32, LDS), turned back by the position and gated.
template <typename TG>
__device__ __forceinline__ float head_gate(const TG* __restrict__ gate_src, int gate_splits, size_t gate_split_stride,
                                           int gate_round, size_t index) {
  float g = 0.f;
  for (int s = 0; s < gate_splits; ++s) g += to_f32<TG>(gate_src[s * gate_split_stride + index]);
  g = as_output(g, gate_round);
  return 1.f / (1.f + expf(-g));
}

template <typename T, typename TG>
__global__ __launch_bounds__(64) void attn_masked_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, const T* __restrict__ k_cache,
    const T* __restrict__ v_cache, const int32_t* __restrict__ positions, const int32_t* __restrict__ token_seq,
    const int32_t* __restrict__ block_table, int table_width, int page_size, int head_dim, int v_dim, int n_heads,
    int n_kv, float scale, float softcap, int window, int keep_first, int tiled, const float* __restrict__ v_cos,
    const float* __restrict__ v_sin, int v_interleaved, int v_max_pos, const TG* __restrict__ gate_src,
    int gate_splits, size_t gate_split_stride, int gate_round, int gate_stride, int gate_col0, int gate_elems,
    const float* __restrict__ dist_bias, int bias_rows, const float* __restrict__ sink) {
  const size_t slab_k = static_cast<size_t>(page_size) * head_dim, slab_v = static_cast<size_t>(page_size) * v_dim;
  __shared__ float qs[kMaxHead];
  __shared__ float os[kMaxHead];
  __shared__ float ps[64];
  __shared__ int pbase[64];  // (page * n_kv + kv_head) per key of the tile
  __shared__ int poff[64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int qpk = n_heads / n_kv, g = h / qpk;
  const int pos = positions[n], seq = token_seq[n];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_first = min(keep_first, lo);  // keys below the window that stay visible
  const int total = n_first + (pos + 1 - lo);
  const T* qrow = q + static_cast<size_t>(n) * q_stride + static_cast<size_t>(h) * head_dim;
  for (int d = lane; d < head_dim; d += 64) qs[d] = to_f32<T>(qrow[d]);
  __syncthreads();
  const int32_t* bt = block_table + static_cast<size_t>(seq) * table_width;
  // a sink starts the running maximum and counts once in the sum: exp(sink) in the denominator, with no value
  float m = sink != nullptr ? sink[h] : -INFINITY, l = sink != nullptr ? 1.f : 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  for (int t0 = 0; t0 < total; t0 += 64) {
    const int idx = t0 + lane;
    const bool valid = idx < total;
    float s = -INFINITY;
    int base = 0, off = 0;
    if (valid) {
      const int key = idx < n_first ? idx : lo + (idx - n_first);
      const int page = bt[key / page_size];
      off = key % page_size;
      base = page * n_kv + g;
      const T* kp = k_cache + static_cast<size_t>(base) * slab_k;
      float dot = 0.f;
      for (int d = 0; d < head_dim; ++d)
        dot = fmaf(qs[d], to_f32<T>(kp[cache_k_offset(tiled, page_size, head_dim, off, d)]), dot);
      s = dot * scale;
      if (softcap > 0.f) s = softcap * tanhf(s / softcap);
      // a learned number per (distance, head), added to the scaled score as it is
      if (dist_bias != nullptr) s += dist_bias[static_cast<size_t>(min(pos - key, bias_rows - 1)) * n_heads + h];
    }
    const float m_new = fmaxf(m, wave_max(s));  // finite: the tile holds at least one key
    const float p = valid ? expf(s - m_new) : 0.f;
    const float alpha = expf(m - m_new);  // 0 on the first tile
    l = l * alpha + wave_sum(p);
    m = m_new;
    __syncthreads();  // the previous tile's ps/pbase are no longer read
    ps[lane] = p;
    pbase[lane] = base;
    poff[lane] = off;
    __syncthreads();
    const int count = min(64, total - t0);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < v_dim) {
        float a = acc[i] * alpha;
        for (int j = 0; j < count; ++j) {
          const T* vp = v_cache + static_cast<size_t>(pbase[j]) * slab_v + cache_v_offset(tiled, page_size, v_dim, poff[j], d);
          a = fmaf(ps[j], to_f32<T>(*vp), a);
        }
        acc[i] = a;
      }
    }
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < v_dim) os[d] = acc[i] * inv;
  }
  __syncthreads();
  float gate = 1.f;
  const size_t gate_at = static_cast<size_t>(n) * gate_stride + gate_col0 + static_cast<size_t>(h) * gate_elems;
  if (gate_src != nullptr && gate_elems == 1) gate = head_gate<TG>(gate_src, gate_splits, gate_split_stride, gate_round, gate_at);
  const float *cr = nullptr, *sr = nullptr;
  if (v_cos != nullptr) {
    const int p = min(pos, v_max_pos - 1);
    cr = v_cos + static_cast<size_t>(p) * (v_dim / 2);
    sr = v_sin + static_cast<size_t>(p) * (v_dim / 2);
  }
  T* orow = out + (static_cast<size_t>(n) * n_heads + h) * v_dim;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < v_dim) {
      const float v = cr != nullptr ? rotated_element(os, d, v_dim, v_interleaved, cr, sr, -1.f) : os[d];
      if (gate_src != nullptr && gate_elems > 1) gate = head_gate<TG>(gate_src, gate_splits, gate_split_stride, gate_round, gate_at + d);
      orow[d] = from_f32<T>(v * gate);
    }
  }
}

// gate_elems: 1, a gate per head in column gate_col0 + h, or v_dim, one per output element in column gate_col0 + h *
// v_dim + d.  dist_bias [bias_rows][n_heads] float32 or null: what is added to the score of a key at distance n (the
// last row for every larger distance).  sink [n_heads] float32 or null: exp(sink[h]) joins head h's denominator once.
extern "C" int yk_attn_masked(const void* q, int q_stride, void* out, const void* k_cache, const void* v_cache, int dtype,
                              const int32_t* positions, const int32_t* token_seq, const int32_t* block_table,
                              int table_width, int n_tokens, int page_size, int head_dim, int v_dim, int n_heads, int n_kv,
                              float scale, float softcap, int window, int keep_first, int tiled, const float* v_cos,
                              const float* v_sin, int v_interleaved, int v_max_pos, const void* gate_src, int gate_dtype,
                              int gate_splits, int gate_round, int gate_stride, int gate_col0, int gate_elems,
                              const float* dist_bias, int bias_rows, const float* sink, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0, "attn_masked: bad head counts");
  YK_REQUIRE(gate_src == nullptr || gate_elems == 1 || gate_elems == v_dim, "attn_masked: a gate per head or per output element");
  YK_REQUIRE(dist_bias == nullptr || bias_rows >= 1, "attn_masked: an empty table of biases");
  YK_REQUIRE(head_dim > 0 && head_dim <= kMaxHead && v_dim > 0 && v_dim <= kMaxHead, "attn_masked: heads of 1 to 256 elements");
  YK_REQUIRE(page_size > 0 && table_width > 0, "attn_masked: bad page table");
  YK_REQUIRE(window >= 0 && keep_first >= 0 && softcap >= 0.f, "attn_masked: window, keep_first and softcap must not be negative");
  YK_REQUIRE(n_heads <= 65535, "attn_masked: too many heads for one launch");
  YK_REQUIRE(v_cos == nullptr || (v_sin != nullptr && v_max_pos > 0 && v_dim % 2 == 0), "attn_masked: value tables need an even value_dim");
  YK_REQUIRE(!tiled || (head_dim == v_dim && cache_is_tiled(dtype, head_dim, page_size)), "attn_masked: these pages cannot be tiled");
  YK_REQUIRE(gate_src == nullptr || gate_splits >= 1, "attn_masked: bad gate");
  if (n_tokens == 0) return 0;
  dim3 grid(n_tokens, n_heads), block(64);
  const size_t gstride = static_cast<size_t>(n_tokens) * gate_stride;
#define YK_CASE(D, T, GD, TG)                                                                                 \
  if (dtype == D && (gate_src == nullptr ? GD == D : gate_dtype == GD)) {                                      \
    attn_masked_kernel<T, TG><<<grid, block, 0, stream>>>(                                                     \
        static_cast<const T*>(q), q_stride, static_cast<T*>(out), static_cast<const T*>(k_cache),              \
        static_cast<const T*>(v_cache), positions, token_seq, block_table, table_width, page_size, head_dim,   \
        v_dim, n_heads, n_kv, scale, softcap, window, keep_first, tiled, v_cos, v_sin, v_interleaved, v_max_pos, \
        static_cast<const TG*>(gate_src), gate_splits, gstride, gate_round, gate_stride, gate_col0, gate_elems, \
        dist_bias, bias_rows, sink);                                                                           \
    return yk_check_launch("attn_masked");                                                                     \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("attn_masked: unsupported dtype combination");
}

template <typename T, typename TG>
__global__ __launch_bounds__(64) void attn_finish_kernel(
    T* __restrict__ out, const int32_t* __restrict__ positions, int v_dim, int n_heads, const float* __restrict__ v_cos,
    const float* __restrict__ v_sin, int v_interleaved, int v_max_pos, const TG* __restrict__ gate_src, int gate_splits,
    size_t gate_split_stride, int gate_round, int gate_stride, int gate_col0, int gate_elems) {
  __shared__ float os[kMaxHead];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  T* orow = out + (static_cast<size_t>(n) * n_heads + h) * v_dim;
  for (int d = lane; d < v_dim; d += 64) os[d] = to_f32<T>(orow[d]);
  __syncthreads();
  float gate = 1.f;
  const size_t gate_at = static_cast<size_t>(n) * gate_stride + gate_col0 + static_cast<size_t>(h) * gate_elems;
  if (gate_src != nullptr && gate_elems == 1) gate = head_gate<TG>(gate_src, gate_splits, gate_split_stride, gate_round, gate_at);
  const float *cr = nullptr, *sr = nullptr;
  if (v_cos != nullptr) {
    const int p = min(positions[n], v_max_pos - 1);
    cr = v_cos + static_cast<size_t>(p) * (v_dim / 2);
    sr = v_sin + static_cast<size_t>(p) * (v_dim / 2);
  }
  for (int d = lane; d < v_dim; d += 64) {
    const float v = cr != nullptr ? rotated_element(os, d, v_dim, v_interleaved, cr, sr, -1.f) : os[d];
    if (gate_src != nullptr && gate_elems > 1) gate = head_gate<TG>(gate_src, gate_splits, gate_split_stride, gate_round, gate_at + d);
    orow[d] = from_f32<T>(v * gate);
  }
}

extern "C" int yk_attn_finish(void* out, int dtype, const int32_t* positions, int n_tokens, int v_dim, int n_heads,
                              const float* v_cos, const float* v_sin, int v_interleaved, int v_max_pos,
                              const void* gate_src, int gate_dtype, int gate_splits, int gate_round, int gate_stride,
                              int gate_col0, int gate_elems, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && n_heads <= 65535 && v_dim > 0 && v_dim <= kMaxHead, "attn_finish: bad sizes");
  YK_REQUIRE(gate_src == nullptr || gate_elems == 1 || gate_elems == v_dim, "attn_finish: a gate per head or per output element");
  YK_REQUIRE(v_cos == nullptr || (v_sin != nullptr && v_max_pos > 0 && v_dim % 2 == 0), "attn_finish: value tables need an even value_dim");
  if (n_tokens == 0 || (v_cos == nullptr && gate_src == nullptr)) return 0;
  dim3 grid(n_tokens, n_heads), block(64);
  const size_t gstride = static_cast<size_t>(n_tokens) * gate_stride;
#define YK_CASE(D, T, GD, TG)                                                                          \
  if (dtype == D && (gate_src == nullptr ? GD == D : gate_dtype == GD)) {                               \
    attn_finish_kernel<T, TG><<<grid, block, 0, stream>>>(static_cast<T*>(out), positions, v_dim, n_heads, v_cos, v_sin, \
                                                          v_interleaved, v_max_pos, static_cast<const TG*>(gate_src),   \
                                                          gate_splits, gstride, gate_round, gate_stride, gate_col0,     \
                                                          gate_elems);                                                  \
    return yk_check_launch("attn_finish");                                                              \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("attn_finish: unsupported dtype combination");
}
