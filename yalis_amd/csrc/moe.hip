// A mixture of small gated feed-forward experts over a ragged batch of tokens.
//
// Which experts a token uses is decided before these kernels (by a table over token ids here;
// a learned router would write the same arrays): `choice` [tokens, top] names them.  A (token,
// k-th choice) is a "pair", numbered token * top + k.
//   * moe_route: sorts the pairs by expert (a counting sort in one workgroup) and cuts every
//     expert's run into tiles of `tile_rows` pairs: order [pairs], slot_expert [pairs], and a
//     tile list (expert, first sorted slot, count).  The order of the pairs inside a run is
//     whatever the atomics gave; every pair's row is computed on its own, so no result depends
//     on it.
//   * moe_gate_up: for the pair in sorted slot i with expert e, y[i, :] = gated_pair(x[token] .
//     Wg_e^T, x[token] . Wu_e^T); the weights of all experts are one tensor [experts][2][ff][hidden].
//   * moe_down: rows[pair, :] = y[i, :] . Wd_e^T in float32, stored in pair order (token-major), so
//     that whoever adds a token's rows finds them side by side (the norm that follows does).
// Each product has a float32 FMA form for any sizes and dtypes, and a matrix-core form for
// bfloat16 with K a multiple of 32: a wave multiplies 16 * FT weight rows (the A operand, straight
// from memory) with 16 * MT pairs (the B operand, gathered rows of x), so an expert's weights are
// read once per tile of pairs.
#include <algorithm>

#include "common.h"

// ------------------------------------------------------------------------------- routing
__global__ __launch_bounds__(1024) void moe_route_kernel(
    const int32_t* __restrict__ token_ids, const int32_t* __restrict__ table, int vocab, int top, int n_experts,
    int n_pairs, int tile_rows, int32_t* __restrict__ order, int32_t* __restrict__ slot_expert,
    int32_t* __restrict__ tiles, int32_t* __restrict__ n_tiles_out, int max_tiles) {
  extern __shared__ int lds[];  // [n_experts] counts, then cursors; [n_experts + 1] first tile of each expert
  int* cnt = lds;
  int* tile0 = lds + n_experts;
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    int id = token_ids != nullptr ? token_ids[i / top] : i / top;  // (no ids: the table has a row per token of the step)
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int e = table[static_cast<size_t>(id) * top + i % top];
    atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0, t = 0;
    for (int e = 0; e < n_experts; ++e) {
      const int c = cnt[e];
      tile0[e] = t;
      t += (c + tile_rows - 1) / tile_rows;
      cnt[e] = run;  // becomes the cursor
      run += c;
    }
    tile0[n_experts] = t;
    *n_tiles_out = t < max_tiles ? t : max_tiles;
  }
  __syncthreads();
  // the tiles of every expert, from the run starts that the cursors still hold
  for (int e = threadIdx.x; e < n_experts; e += blockDim.x) {
    const int first = cnt[e];
    const int n_t = tile0[e + 1] - tile0[e];
    const int len = (e + 1 < n_experts ? cnt[e + 1] : n_pairs) - first;  // starts are running sums
    for (int k = 0; k < n_t; ++k) {
      const int t = tile0[e] + k;
      if (t < max_tiles) {
        tiles[3 * t] = e;
        tiles[3 * t + 1] = first + k * tile_rows;
        tiles[3 * t + 2] = min(tile_rows, len - k * tile_rows);
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n_pairs; i += blockDim.x) {
    int id = token_ids != nullptr ? token_ids[i / top] : i / top;  // (no ids: the table has a row per token of the step)
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    const int e = table[static_cast<size_t>(id) * top + i % top];
    const int at = atomicAdd(&cnt[e], 1);
    order[at] = i;
    slot_expert[at] = e;
  }
}

extern "C" int yk_moe_max_tiles(int n_pairs, int n_experts, int tile_rows) {
  return (n_pairs + tile_rows - 1) / tile_rows + n_experts;
}

extern "C" int yk_moe_route(const int32_t* token_ids, const int32_t* table, int vocab, int top, int n_experts,
                            int n_tokens, int tile_rows, int32_t* order, int32_t* slot_expert, int32_t* tiles,
                            int32_t* n_tiles, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && top >= 1 && n_experts >= 1 && vocab >= 1 && tile_rows >= 1, "moe_route: bad sizes");
  YK_REQUIRE(n_experts <= 4096, "moe_route: more than 4,096 experts");
  if (n_tokens == 0) return 0;
  const int n_pairs = n_tokens * top;
  const size_t lds = (2 * static_cast<size_t>(n_experts) + 1) * sizeof(int);
  moe_route_kernel<<<1, 1024, lds, stream>>>(token_ids, table, vocab, top, n_experts, n_pairs, tile_rows, order,
                                             slot_expert, tiles, n_tiles, yk_moe_max_tiles(n_pairs, n_experts, tile_rows));
  return yk_check_launch("moe_route");
}

// ------------------------------------------------------------------------ a learned router
// Per token: the `top` experts with the largest logits (ties: the lower number), their numbers into choice
// [tokens][top], and the token's row once per chosen expert, multiplied by that expert's score sigmoid(logit), into xs
// [tokens * top][hidden]: the score weighs what the expert reads, not what it returns.  A workgroup a token; its
// first wave chooses.  bias [n_experts] (or null) joins the logits before the choice.  With `weights` (float32 [tokens][top])
// in place of xs, the chosen experts' weights are written instead: the softmax over the chosen logits alone (they weigh
// what the experts return; nothing is copied).
template <typename T>
__global__ __launch_bounds__(256) void moe_router_topk_kernel(const float* __restrict__ logits, int logits_stride, int n_experts, int top,
                                                              const T* __restrict__ x, int x_stride, int hidden,
                                                              int32_t* __restrict__ choice, T* __restrict__ xs,
                                                              const float* __restrict__ bias, float* __restrict__ weights, int n_tokens) {
  extern __shared__ float sel_all[];  // per choosing wave: [top] scores, then [top] numbers (as ints)
  // with weights every wave of the workgroup chooses for a token of its own (there is nothing to copy afterwards)
  const bool per_wave = weights != nullptr;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  float* sel = sel_all + (per_wave ? wave * 2 * top : 0);
  int* sel_e = reinterpret_cast<int*>(sel + top);
  const int n = per_wave ? min(static_cast<int>(blockIdx.x) * 4 + wave, n_tokens - 1) : blockIdx.x;
  const float* row = logits + static_cast<size_t>(n) * logits_stride;
  if (per_wave || threadIdx.x < kWave) {
    for (int k = 0; k < top; ++k) {
      float best = -INFINITY;
      int best_e = 0x7fffffff;
      for (int e = lane; e < n_experts; e += kWave) {
        bool taken = false;
        for (int j = 0; j < k; ++j) taken |= sel_e[j] == e;
        const float v = bias != nullptr ? row[e] + bias[e] : row[e];
        // (a NaN is never larger: such a row falls back on the lowest free numbers)
        if (!taken && (v > best || (best_e == 0x7fffffff) || (v == best && e < best_e))) {
          best = v;
          best_e = e;
        }
      }
      // the wave's best: the largest value, among equals the lowest number
      for (int off = kWave / 2; off > 0; off /= 2) {
        const float ov = __shfl_xor(best, off, kWave);
        const int oe = __shfl_xor(best_e, off, kWave);
        if (oe != 0x7fffffff && (best_e == 0x7fffffff || ov > best || (ov == best && oe < best_e))) {
          best = ov;
          best_e = oe;
        }
      }
      if (lane == 0) {
        sel_e[k] = best_e;
        sel[k] = weights != nullptr ? best : 1.f / (1.f + expf(-best));
        choice[static_cast<size_t>(n) * top + k] = best_e;
      }
      __builtin_amdgcn_wave_barrier();
      __threadfence_block();
    }
    if (weights != nullptr && lane == 0) {  // sel[0] is the largest
      float sum = 0.f;
      for (int k = 0; k < top; ++k) sum += expf(sel[k] - sel[0]);
      for (int k = 0; k < top; ++k) weights[static_cast<size_t>(n) * top + k] = expf(sel[k] - sel[0]) / sum;
    }
  }
  if (weights != nullptr) return;
  __syncthreads();
  const T* src = x + static_cast<size_t>(n) * x_stride;
  for (int c = threadIdx.x; c < hidden; c += blockDim.x) {
    const float v = to_f32<T>(src[c]);
    for (int k = 0; k < top; ++k) xs[(static_cast<size_t>(n) * top + k) * hidden + c] = from_f32<T>(v * sel[k]);
  }
}

extern "C" int yk_moe_router_topk(const float* logits, int logits_stride, int n_experts, int top, const void* x, int x_stride, int dtype,
                                  int hidden, int32_t* choice, void* xs, int n_tokens, const float* bias, float* weights,
                                  hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_experts >= 1 && top >= 1 && top <= n_experts && top <= 64 && logits_stride >= n_experts,
             "moe_router_topk: bad sizes (up to 64 experts a token)");
  YK_REQUIRE((weights != nullptr) != (xs != nullptr), "moe_router_topk: weights for the outputs, or scaled copies of the inputs");
  YK_REQUIRE(weights != nullptr || (x != nullptr && hidden > 0 && x_stride >= hidden), "moe_router_topk: bad input rows");
  if (n_tokens == 0) return 0;
  const size_t lds = 2 * static_cast<size_t>(top) * sizeof(float);
  if (weights != nullptr)  // a wave chooses and weighs for a token, four tokens a workgroup; there is nothing to copy
    moe_router_topk_kernel<float><<<(n_tokens + 3) / 4, 256, 4 * lds, stream>>>(logits, logits_stride, n_experts, top, nullptr, 0, 0, choice,
                                                                                nullptr, bias, weights, n_tokens);
  else if (dtype == YK_F32)
    moe_router_topk_kernel<float><<<n_tokens, 256, lds, stream>>>(logits, logits_stride, n_experts, top, static_cast<const float*>(x), x_stride,
                                                                  hidden, choice, static_cast<float*>(xs), bias, nullptr, n_tokens);
  else if (dtype == YK_BF16)
    moe_router_topk_kernel<bf16_t><<<n_tokens, 256, lds, stream>>>(logits, logits_stride, n_experts, top, static_cast<const bf16_t*>(x), x_stride,
                                                                   hidden, choice, static_cast<bf16_t*>(xs), bias, nullptr, n_tokens);
  else
    return yk_fail("moe_router_topk: unsupported dtype");
  return yk_check_launch("moe_router_topk");
}

// out[n, :] = dense[n, :] (a tensor, a product's unreduced slices, or nothing) + weight * the sum of the token's `top`
// rows of rows [tokens * top][width] (each times its own entry of row_weights [tokens * top] where given): what a mixture adds to
// the stream, as one float32 tensor
template <typename TD>
__global__ void moe_combine_kernel(const TD* __restrict__ dense, int n_splits, size_t split_stride, int round_sum,
                                   const float* __restrict__ rows, int top, float weight, float* __restrict__ out, int width,
                                   size_t total, const float* __restrict__ row_weights) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const size_t n = i / width;
    const int c = static_cast<int>(i % width);
    float d = 0.f;
    if (dense != nullptr) {
      for (int s = 0; s < n_splits; ++s) d += to_f32<TD>(dense[s * split_stride + i]);
      d = as_output(d, round_sum);
    }
    float e = 0.f;
    if (row_weights != nullptr)  // every row has a weight of its own
      for (int k = 0; k < top; ++k) e = fmaf(row_weights[n * top + k], rows[(n * top + k) * width + c], e);
    else
      for (int k = 0; k < top; ++k) e += rows[(n * top + k) * width + c];
    out[i] = fmaf(weight, e, d);
  }
}

extern "C" int yk_moe_combine(const void* dense, int dense_dtype, int n_splits, int round_sum, const float* rows, int top,
                              float weight, float* out, int n_tokens, int width, const float* row_weights, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && width > 0 && top >= 1 && n_splits >= 1 && (n_splits == 1 || dense_dtype == YK_F32), "moe_combine: bad sizes");
  if (n_tokens == 0) return 0;
  const size_t total = static_cast<size_t>(n_tokens) * width;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 1 << 20));
  if (dense == nullptr || dense_dtype == YK_F32)
    moe_combine_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(dense), n_splits, total, round_sum, rows, top,
                                                        weight, out, width, total, row_weights);
  else if (dense_dtype == YK_BF16)
    moe_combine_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(dense), n_splits, total, round_sum, rows, top,
                                                         weight, out, width, total, row_weights);
  else
    return yk_fail("moe_combine: unsupported dtype");
  return yk_check_launch("moe_combine");
}

// ---------------------------------------------------------------- float32 FMA products
template <typename T, typename TW>
__global__ __launch_bounds__(256) void moe_gate_up_fma_kernel(
    const T* __restrict__ x, int x_stride, const TW* __restrict__ w, const int32_t* __restrict__ order,
    const int32_t* __restrict__ slot_expert, int top, int hidden, int ff, int kind, float p0, float p1,
    T* __restrict__ y, int gated) {
  extern __shared__ float xs[];  // [hidden]
  const int i = blockIdx.x;
  const int token = order[i] / top, e = slot_expert[i];
  for (int k = threadIdx.x; k < hidden; k += blockDim.x) xs[k] = to_f32<T>(x[static_cast<size_t>(token) * x_stride + k]);
  __syncthreads();
  if (!gated) {  // an expert without a gate: act(up x), the weights [experts][ff][hidden]
    for (int j = blockIdx.y * blockDim.x + threadIdx.x; j < ff; j += gridDim.y * blockDim.x) {
      const TW* wu = w + (static_cast<size_t>(e) * ff + j) * hidden;
      float u = 0.f;
      for (int k = 0; k < hidden; ++k) u = fmaf(to_f32<TW>(wu[k]), xs[k], u);
      y[static_cast<size_t>(i) * ff + j] = from_f32<T>(act_plain(u, kind));
    }
    return;
  }
  for (int j = blockIdx.y * blockDim.x + threadIdx.x; j < ff; j += gridDim.y * blockDim.x) {
    const TW* wg = w + (static_cast<size_t>(e) * 2 * ff + j) * hidden;
    const TW* wu = wg + static_cast<size_t>(ff) * hidden;
    float g = 0.f, u = 0.f;
    for (int k = 0; k < hidden; ++k) {
      g = fmaf(to_f32<TW>(wg[k]), xs[k], g);
      u = fmaf(to_f32<TW>(wu[k]), xs[k], u);
    }
    y[static_cast<size_t>(i) * ff + j] = from_f32<T>(gated_pair(g, u, kind, p0, p1));
  }
}

template <typename T, typename TW>
__global__ __launch_bounds__(256) void moe_down_fma_kernel(
    const T* __restrict__ y, const TW* __restrict__ w, const int32_t* __restrict__ order,
    const int32_t* __restrict__ slot_expert, int hidden, int ff, float* __restrict__ rows) {
  extern __shared__ float ys[];  // [ff]
  const int i = blockIdx.x;
  const int pair = order[i], e = slot_expert[i];
  for (int k = threadIdx.x; k < ff; k += blockDim.x) ys[k] = to_f32<T>(y[static_cast<size_t>(i) * ff + k]);
  __syncthreads();
  for (int h = blockIdx.y * blockDim.x + threadIdx.x; h < hidden; h += gridDim.y * blockDim.x) {
    const TW* wd = w + (static_cast<size_t>(e) * hidden + h) * ff;
    float acc = 0.f;
    for (int k = 0; k < ff; ++k) acc = fmaf(to_f32<TW>(wd[k]), ys[k], acc);
    rows[static_cast<size_t>(pair) * hidden + h] = acc;
  }
}

// ---------------------------------------------------------------- matrix-core products
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
union MoeFrag {
  u32x4_t u;
  bf16x8_t v;
};

// Operands of v_mfma_f32_16x16x32_bf16 (r = lane % 16, g = lane / 16): A lane holds A[r][8g..8g+7],
// B lane holds B[8g..8g+7][r], C lane holds C[4g..4g+3][r].  A = 16 weight rows, B = 16 pairs'
// rows of x: C[i][r] = (pair r, feature 4g + i).
// A wave owns FT tiles of 16 features and MT tiles of 16 pairs; the fragments of the next step
// of 32 along K are asked for before the products of this one are issued (two register sets by
// turns), so that loads and matrix cores overlap.
//
// A workgroup has 4 * WR waves: four side by side over the features, WR one above the other over
// the tile's pairs (16 * MT each).  Workgroups are numbered so that those that share a tile's pairs
// (one per group of features) come one behind the other on one die (numbers 8 apart), whose L2 then
// holds the tile's rows of x for all of them; every weight row is read once per tile.
__device__ __forceinline__ void moe_tile_of(int n_groups, int& tile, int& group) {
  const int die = blockIdx.x % 8, slot = blockIdx.x / 8;
  tile = (slot / n_groups) * 8 + die;
  group = slot % n_groups;
}

// KS: the four waves of a workgroup share one set of features and divide K between them (their
// sums meet in LDS): steps of few pairs have few tiles, and this way four times the waves pull on
// an expert's weights.
// GATED false: experts without a gate, act(up x) with a plain activation; the weights are [experts][ff][hidden] and only
// the `u` half of everything below is computed.
template <int MT, int FT, int WR, bool KS, bool GATED>
__global__ __launch_bounds__(256 * WR) void moe_gate_up_mfma_kernel(
    const bf16_t* __restrict__ x, int x_stride, const bf16_t* __restrict__ w, const int32_t* __restrict__ order,
    const int32_t* __restrict__ tiles, const int32_t* __restrict__ n_tiles, int top, int hidden, int ff, int kind,
    float p0, float p1, bf16_t* __restrict__ y, int n_groups) {
  int t, group;
  moe_tile_of(n_groups, t, group);
  if (t >= *n_tiles) return;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, r = lane % 16, g = lane / 16;
  const int e = tiles[3 * t], row0 = 16 * MT * (wave / 4);
  const int first = tiles[3 * t + 1] + row0, count = tiles[3 * t + 2] - row0;
  const int f0 = (KS ? group : group * 4 + wave % 4) * 16 * FT;
  if (f0 >= ff || count <= 0) return;
  const int k_quarter = ((hidden / 32 + 3) / 4) * 32;
  const int k_begin = KS ? wave * k_quarter : 0, k_end = KS ? min(hidden, k_begin + k_quarter) : hidden;
  const bf16_t *wg[FT], *wu[FT];
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    const int row = min(f0 + 16 * f + r, ff - 1);  // (tiles beyond the width repeat its last row and are not stored)
    wg[f] = w + (static_cast<size_t>(e) * (GATED ? 2 : 1) * ff + row) * hidden + 8 * g;
    wu[f] = GATED ? wg[f] + static_cast<size_t>(ff) * hidden : wg[f];
  }
  const bf16_t* xr[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int slot = first + min(16 * m + r, count - 1);  // rows beyond the tile repeat its last pair and are not stored
    xr[m] = x + static_cast<size_t>(order[slot] / top) * x_stride + 8 * g;
  }
  f32x4_t ag[FT][MT], au[FT][MT];
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int m = 0; m < MT; ++m) ag[f][m] = au[f][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  MoeFrag a0[2][FT], b0[MT], a1[2][FT], b1[MT];
#define MOE_LOAD(A, B, K0)                                                                  \
  {                                                                                         \
    _Pragma("unroll") for (int f = 0; f < FT; ++f) {                                        \
      if (GATED) A[0][f].u = *reinterpret_cast<const u32x4_t*>(wg[f] + (K0));               \
      A[1][f].u = *reinterpret_cast<const u32x4_t*>(wu[f] + (K0));                          \
    }                                                                                       \
    _Pragma("unroll") for (int m = 0; m < MT; ++m) B[m].u = *reinterpret_cast<const u32x4_t*>(xr[m] + (K0)); \
  }
#define MOE_MMA(A, B)                                                                       \
  {                                                                                         \
    _Pragma("unroll") for (int f = 0; f < FT; ++f)                                          \
    _Pragma("unroll") for (int m = 0; m < MT; ++m) {                                        \
      if (GATED) ag[f][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[0][f].v, B[m].v, ag[f][m], 0, 0, 0); \
      au[f][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[1][f].v, B[m].v, au[f][m], 0, 0, 0); \
    }                                                                                       \
  }
  if (k_begin < k_end) MOE_LOAD(a0, b0, k_begin)
  for (int k0 = k_begin; k0 < k_end; k0 += 64) {
    const bool second = k0 + 32 < k_end;
    if (second) MOE_LOAD(a1, b1, k0 + 32)
    MOE_MMA(a0, b0)
    if (k0 + 64 < k_end) MOE_LOAD(a0, b0, k0 + 64)
    if (second) MOE_MMA(a1, b1)
  }
#undef MOE_LOAD
#undef MOE_MMA
  if (KS) {
    __shared__ f32x4_t part[3][2 * FT * MT][64];
    if (wave > 0) {
#pragma unroll
      for (int f = 0; f < FT; ++f)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          if (GATED) part[wave - 1][(2 * f) * MT + m][lane] = ag[f][m];
          part[wave - 1][(2 * f + 1) * MT + m][lane] = au[f][m];
        }
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w2 = 0; w2 < 3; ++w2)
#pragma unroll
      for (int f = 0; f < FT; ++f)
#pragma unroll
        for (int m = 0; m < MT; ++m) {
          if (GATED) ag[f][m] += part[w2][(2 * f) * MT + m][lane];
          au[f][m] += part[w2][(2 * f + 1) * MT + m][lane];
        }
  }
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    if (f0 + 16 * f >= ff) continue;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (16 * m + r < count) {
        uint32_t o[2];
        if (GATED) {
          o[0] = pack_bf16x2(gated_pair(ag[f][m][0], au[f][m][0], kind, p0, p1), gated_pair(ag[f][m][1], au[f][m][1], kind, p0, p1));
          o[1] = pack_bf16x2(gated_pair(ag[f][m][2], au[f][m][2], kind, p0, p1), gated_pair(ag[f][m][3], au[f][m][3], kind, p0, p1));
        } else {
          o[0] = pack_bf16x2(act_plain(au[f][m][0], kind), act_plain(au[f][m][1], kind));
          o[1] = pack_bf16x2(act_plain(au[f][m][2], kind), act_plain(au[f][m][3], kind));
        }
        *reinterpret_cast<uint2*>(y + static_cast<size_t>(first + 16 * m + r) * ff + f0 + 16 * f + 4 * g) = make_uint2(o[0], o[1]);
      }
    }
  }
}

template <int MT, int FT, int WR, bool KS>
__global__ __launch_bounds__(256 * WR) void moe_down_mfma_kernel(
    const bf16_t* __restrict__ y, const bf16_t* __restrict__ w, const int32_t* __restrict__ order,
    const int32_t* __restrict__ tiles, const int32_t* __restrict__ n_tiles, int hidden, int ff,
    float* __restrict__ rows, int n_groups) {
  int t, group;
  moe_tile_of(n_groups, t, group);
  if (t >= *n_tiles) return;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, r = lane % 16, g = lane / 16;
  const int e = tiles[3 * t], row0 = 16 * MT * (wave / 4);
  const int first = tiles[3 * t + 1] + row0, count = tiles[3 * t + 2] - row0;
  const int h0 = (KS ? group : group * 4 + wave % 4) * 16 * FT;
  if (h0 >= hidden || count <= 0) return;
  const int k_quarter = ((ff / 32 + 3) / 4) * 32;
  const int k_begin = KS ? wave * k_quarter : 0, k_end = KS ? min(ff, k_begin + k_quarter) : ff;
  const bf16_t* wd[FT];
#pragma unroll
  for (int f = 0; f < FT; ++f)
    wd[f] = w + (static_cast<size_t>(e) * hidden + min(h0 + 16 * f + r, hidden - 1)) * ff + 8 * g;
  const bf16_t* yr[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) yr[m] = y + static_cast<size_t>(first + min(16 * m + r, count - 1)) * ff + 8 * g;
  f32x4_t acc[FT][MT];
#pragma unroll
  for (int f = 0; f < FT; ++f)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[f][m] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  MoeFrag a0[FT], b0[MT], a1[FT], b1[MT];
#define MOE_LOAD(A, B, K0)                                                                  \
  {                                                                                         \
    _Pragma("unroll") for (int f = 0; f < FT; ++f) A[f].u = *reinterpret_cast<const u32x4_t*>(wd[f] + (K0)); \
    _Pragma("unroll") for (int m = 0; m < MT; ++m) B[m].u = *reinterpret_cast<const u32x4_t*>(yr[m] + (K0)); \
  }
#define MOE_MMA(A, B)                                                                       \
  {                                                                                         \
    _Pragma("unroll") for (int f = 0; f < FT; ++f)                                          \
    _Pragma("unroll") for (int m = 0; m < MT; ++m)                                          \
      acc[f][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A[f].v, B[m].v, acc[f][m], 0, 0, 0); \
  }
  if (k_begin < k_end) MOE_LOAD(a0, b0, k_begin)
  for (int k0 = k_begin; k0 < k_end; k0 += 64) {
    const bool second = k0 + 32 < k_end;
    if (second) MOE_LOAD(a1, b1, k0 + 32)
    MOE_MMA(a0, b0)
    if (k0 + 64 < k_end) MOE_LOAD(a0, b0, k0 + 64)
    if (second) MOE_MMA(a1, b1)
  }
#undef MOE_LOAD
#undef MOE_MMA
  if (KS) {
    __shared__ f32x4_t part[3][FT * MT][64];
    if (wave > 0) {
#pragma unroll
      for (int f = 0; f < FT; ++f)
#pragma unroll
        for (int m = 0; m < MT; ++m) part[wave - 1][f * MT + m][lane] = acc[f][m];
    }
    __syncthreads();
    if (wave > 0) return;
#pragma unroll
    for (int w2 = 0; w2 < 3; ++w2)
#pragma unroll
      for (int f = 0; f < FT; ++f)
#pragma unroll
        for (int m = 0; m < MT; ++m) acc[f][m] += part[w2][f * MT + m][lane];
  }
#pragma unroll
  for (int f = 0; f < FT; ++f) {
    if (h0 + 16 * f >= hidden) continue;
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      if (16 * m + r < count) {
        const int pair = order[first + 16 * m + r];
        *reinterpret_cast<float4*>(rows + static_cast<size_t>(pair) * hidden + h0 + 16 * f + 4 * g) =
            make_float4(acc[f][m][0], acc[f][m][1], acc[f][m][2], acc[f][m][3]);
      }
    }
  }
}

// Whether the matrix-core forms take these sizes (bfloat16 everywhere is the caller's to check).
extern "C" int yk_moe_mfma_ok(int hidden, int ff, int x_stride) {
  return hidden % 32 == 0 && ff % 32 == 0 && x_stride % 8 == 0;
}

static bool aligned16(const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; }

extern "C" int yk_moe_gate_up(const void* x, int x_stride, int dtype, const void* w, int w_dtype, const int32_t* order,
                              const int32_t* slot_expert, const int32_t* tiles, const int32_t* n_tiles, int tile_rows,
                              int max_tiles, int n_pairs, int top, int hidden, int ff, int kind, float p0, float p1,
                              void* y, int gated, hipStream_t stream) {
  YK_REQUIRE(n_pairs >= 0 && top >= 1 && hidden > 0 && ff > 0 && x_stride >= hidden, "moe_gate_up: bad sizes");
  YK_REQUIRE(kind >= 0 && kind < (gated ? YK_GATED_KINDS : YK_PLAIN_KINDS), "moe_gate_up: unknown activation");
  if (n_pairs == 0) return 0;
  if (dtype == YK_BF16 && w_dtype == YK_BF16 && yk_moe_mfma_ok(hidden, ff, x_stride) && aligned16(x) && aligned16(w) &&
      aligned16(y) && (tile_rows == 16 || tile_rows == 64 || tile_rows == 128)) {
    constexpr int FT = 2;  // feature tiles of 16 a wave
    const int n_groups = tile_rows == 16 ? (ff + 16 * FT - 1) / (16 * FT) : (ff + 64 * FT - 1) / (64 * FT);
    const long long n_wg = static_cast<long long>((max_tiles + 7) / 8 * 8) * n_groups;
    YK_REQUIRE(n_wg <= 0x7fffffffLL, "moe_gate_up: too many tiles for one launch");
    dim3 grid(static_cast<unsigned>(n_wg));
#define YK_MOE_GU(MT, WR, KS)                                                                                   \
  if (gated)                                                                                                     \
    moe_gate_up_mfma_kernel<MT, FT, WR, KS, true><<<grid, 256 * WR, 0, stream>>>(                                     \
        static_cast<const bf16_t*>(x), x_stride, static_cast<const bf16_t*>(w), order, tiles, n_tiles, top, hidden, ff, \
        kind, p0, p1, static_cast<bf16_t*>(y), n_groups);                                                         \
  else                                                                                                           \
    moe_gate_up_mfma_kernel<MT, FT, WR, KS, false><<<grid, 256 * WR, 0, stream>>>(                                    \
        static_cast<const bf16_t*>(x), x_stride, static_cast<const bf16_t*>(w), order, tiles, n_tiles, top, hidden, ff, \
        kind, p0, p1, static_cast<bf16_t*>(y), n_groups)
    if (tile_rows == 16) { YK_MOE_GU(1, 1, true); }
    else if (tile_rows == 64) { YK_MOE_GU(4, 1, false); }
    else { YK_MOE_GU(4, 2, false); }
#undef YK_MOE_GU
    return yk_check_launch("moe_gate_up (matrix cores)");
  }
  YK_REQUIRE(hidden <= 15 * 1024, "moe_gate_up: rows of more than 15,360 elements do not fit");
  dim3 grid(n_pairs, std::min((ff + 255) / 256, 64)), block(256);
  const size_t lds = static_cast<size_t>(hidden) * sizeof(float);
#define YK_CASE(D, T, WD, TW)                                                                                     \
  if (dtype == D && w_dtype == WD) {                                                                               \
    moe_gate_up_fma_kernel<T, TW><<<grid, block, lds, stream>>>(static_cast<const T*>(x), x_stride, static_cast<const TW*>(w), \
                                                                order, slot_expert, top, hidden, ff, kind, p0, p1,            \
                                                                static_cast<T*>(y), gated);                                   \
    return yk_check_launch("moe_gate_up");                                                                         \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("moe_gate_up: unsupported dtype combination");
}

extern "C" int yk_moe_down(const void* y, int dtype, const void* w, int w_dtype, const int32_t* order,
                           const int32_t* slot_expert, const int32_t* tiles, const int32_t* n_tiles, int tile_rows,
                           int max_tiles, int n_pairs, int hidden, int ff, float* rows, hipStream_t stream) {
  YK_REQUIRE(n_pairs >= 0 && hidden > 0 && ff > 0, "moe_down: bad sizes");
  if (n_pairs == 0) return 0;
  if (dtype == YK_BF16 && w_dtype == YK_BF16 && yk_moe_mfma_ok(ff, hidden, ff) && aligned16(y) && aligned16(w) &&
      aligned16(rows) && (tile_rows == 16 || tile_rows == 64 || tile_rows == 128)) {
    constexpr int FT = 4;
    const int n_groups = tile_rows == 16 ? (hidden + 16 * FT - 1) / (16 * FT) : (hidden + 64 * FT - 1) / (64 * FT);
    const long long n_wg = static_cast<long long>((max_tiles + 7) / 8 * 8) * n_groups;
    YK_REQUIRE(n_wg <= 0x7fffffffLL, "moe_down: too many tiles for one launch");
    dim3 grid(static_cast<unsigned>(n_wg));
#define YK_MOE_DN(MT, WR, KS)                                                                                   \
  moe_down_mfma_kernel<MT, FT, WR, KS><<<grid, 256 * WR, 0, stream>>>(static_cast<const bf16_t*>(y), static_cast<const bf16_t*>(w), \
                                                                  order, tiles, n_tiles, hidden, ff, rows, n_groups)
    if (tile_rows == 16) YK_MOE_DN(1, 1, true);
    else if (tile_rows == 64) YK_MOE_DN(4, 1, false);
    else YK_MOE_DN(4, 2, false);
#undef YK_MOE_DN
    return yk_check_launch("moe_down (matrix cores)");
  }
  YK_REQUIRE(ff <= 15 * 1024, "moe_down: rows of more than 15,360 elements do not fit");
  dim3 grid(n_pairs, std::min((hidden + 255) / 256, 64)), block(256);
  const size_t lds = static_cast<size_t>(ff) * sizeof(float);
#define YK_CASE(D, T, WD, TW)                                                                                    \
  if (dtype == D && w_dtype == WD) {                                                                              \
    moe_down_fma_kernel<T, TW><<<grid, block, lds, stream>>>(static_cast<const T*>(y), static_cast<const TW*>(w), order, \
                                                             slot_expert, hidden, ff, rows);                            \
    return yk_check_launch("moe_down");                                                                           \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("moe_down: unsupported dtype combination");
}
