// Recurrences whose memory is a matrix per head, S [dim][vdim] float32 in the request's state slot:
//
//   S <- diag(a_t) S                       a_t: one decay for the head, or one per key channel (row of S)
//   u  = v_t                               plain write
//   u  = beta_t (v_t - S^T k_t)            delta rule
//   u  = dt_t v_t                          a write as strong as the token's step (state-space duality: with the head's
//                                          decay exp(-exp(A_log) dt_t), dt_t = softplus(x + dt_bias), q = C, k = B)
//   S <- S + k_t u^T,   o_t = S^T q_t      (the read-out sees the token's own write; + skip_h v_t where a skip is given)
//
// The columns of S never meet: column e needs k_t, q_t, a_t, beta_t and its own v_t[e] only.  So a
// column lives in the registers of a group of TPC lanes (lane s of the group holds the rows s,
// 16 s .. 16 s + 15), the two sums over rows are exchanges inside the group, and a workgroup walks a
// request's span token by token with k, q and the decays of the next 32 tokens staged in LDS (a wave
// per token and vector makes the unit norm while it stages), read back 16 bytes at a time.  Decays, write strengths and unit norms are made here, in float32, from the
// projections' raw outputs:
//   decay per head:     exp(-exp(A_log[h]) * softplus(x[n, h] + dt_bias[h]))
//   decay per channel:  sigmoid(z[n, h, i] + bias[h, i]) ^ (1 / tau)  =  exp(logsigmoid(.) / tau)
//   beta:               sigmoid(x[n, h])
//   unit vectors:       q / sqrt(sum q^2 + eps), k likewise (with unit_eps >= 0), then q * q_scale
// A span cut anywhere gives the same S bit for bit: every token's step is made alone.
//
// Beside it: the read-out's norm and gate (each head's o divided by its root mean square, times a
// weight shared by the heads, times silu of a gate column), and the shift of a convolution's kept
// inputs by a span.
#include <algorithm>

#include "common.h"

constexpr int kScanRowsMax = 16;  // rows of S a lane holds at the most (template R: 8 or 16): sub * R .. sub * R + R - 1 of its column
constexpr int kScanTokens = 32;  // tokens staged at a time (fewer where LDS would not hold them)

__device__ __forceinline__ float scan_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// the sum over the TPC lanes of a column (lanes that differ in their low bits), in all of them.  Inside
// a row of 16 lanes the exchanges are register moves (quad permutations, then rotations of the row by 4
// and by 8: after the quads' sums, s_j = Q_j + Q_(j+1) and s_j + s_(j+2) is the row's sum); wider groups
// go on through the LDS pipe.
__device__ __forceinline__ float dpp_add(float v, int ctrl_xor1_2_ror4_8) {
  const int x = __float_as_int(v);
  int y;
  switch (ctrl_xor1_2_ror4_8) {
    case 0: y = __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xf, 0xf, false); break;   // quad_perm [1,0,3,2]
    case 1: y = __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xf, 0xf, false); break;   // quad_perm [2,3,0,1]
    case 2: y = __builtin_amdgcn_update_dpp(0, x, 0x124, 0xf, 0xf, false); break;  // row_ror:4
    default: y = __builtin_amdgcn_update_dpp(0, x, 0x128, 0xf, 0xf, false); break; // row_ror:8
  }
  return v + __int_as_float(y);
}
template <int TPC>
__device__ __forceinline__ float column_sum(float v) {
  if (TPC >= 2) v = dpp_add(v, 0);
  if (TPC >= 4) v = dpp_add(v, 1);
  if (TPC == 8) {
    // two quads a column: each takes the other's sum (quads 0 and 2 from four lanes up, 1 and 3 from four down)
    const int x = __float_as_int(v);
    int y = __builtin_amdgcn_update_dpp(0, x, 0x104, 0xf, 0x5, false);  // row_shl:4 into quads 0 and 2
    y = __builtin_amdgcn_update_dpp(y, x, 0x114, 0xf, 0xa, false);      // row_shr:4 into quads 1 and 3
    v += __int_as_float(y);
  }
  if (TPC >= 16) {
    v = dpp_add(v, 2);
    v = dpp_add(v, 3);
  }
  if (TPC >= 32) {  // lanes r and r + 16
    const auto a = __builtin_amdgcn_permlane16_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  }
  if (TPC >= 64) {  // and the other half of the wave
    const auto b = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
    v = __uint_as_float(b[0]) + __uint_as_float(b[1]);
  }
  return v;
}

// eight consecutive elements (16-byte aligned where T is bfloat16, 32 where float) as floats
template <typename T>
__device__ __forceinline__ void scan_load8(const T* p, float* out);
template <>
__device__ __forceinline__ void scan_load8<float>(const float* p, float* out) {
  const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
  out[0] = a.x; out[1] = a.y; out[2] = a.z; out[3] = a.w; out[4] = b.x; out[5] = b.y; out[6] = b.z; out[7] = b.w;
}
template <>
__device__ __forceinline__ void scan_load8<bf16_t>(const bf16_t* p, float* out) {
  const uint4 w = *reinterpret_cast<const uint4*>(p);
  out[0] = __uint_as_float(w.x << 16); out[1] = __uint_as_float(w.x & 0xffff0000u);
  out[2] = __uint_as_float(w.y << 16); out[3] = __uint_as_float(w.y & 0xffff0000u);
  out[4] = __uint_as_float(w.z << 16); out[5] = __uint_as_float(w.z & 0xffff0000u);
  out[6] = __uint_as_float(w.w << 16); out[7] = __uint_as_float(w.w & 0xffff0000u);
}

// LDS per staged token: k and q padded to TPC * 16 floats each (rows past dim are zeros, so nobody
// asks whether a row exists), the per-channel decays likewise where there are any
template <typename T, int TPC, int kScanRows, bool VEC>
__global__ __launch_bounds__(256) void linear_state_scan_kernel(
    const T* __restrict__ qkv, int qkv_stride, int n_heads, int n_kv, int dim, int vdim, float* __restrict__ state,
    const int32_t* __restrict__ seq_qstart, const int32_t* __restrict__ seq_qlen, const int32_t* __restrict__ state_slots,
    float q_scale, float unit_eps, int decay_mode, const float* __restrict__ decay, int decay_stride, int decay_col,
    const float* __restrict__ decay_p0, const float* __restrict__ decay_p1, float tau, const float* __restrict__ beta,
    int beta_stride, int beta_col, int chunk, float* __restrict__ out, int q_col, int k_col, int v_col, int write_mode,
    const float* __restrict__ skip) {
  extern __shared__ float lds[];
  constexpr int DP = TPC * kScanRows;  // padded key channels
  constexpr int DS = DP + 4;           // a staged row's stride: rows of different tokens then start in different banks
  const int cols_per_block = blockDim.x / TPC;
  float* ks = lds;                                        // [chunk][DS]
  float* qs = ks + chunk * DS;                            // [chunk][DS]
  float* as = qs + chunk * DS;                            // [chunk][DS] (per channel) or [chunk]
  float* vs = as + chunk * (decay_mode == 1 ? DS : 1);    // [chunk][cols_per_block]
  float* bs = vs + chunk * cols_per_block;                // [chunk]
  float* kqs = bs + chunk;                                // [chunk]: k . q of every token, as they enter the recurrence

  const int seq = blockIdx.x, h = blockIdx.y, kvh = h / (n_heads / n_kv);
  const int col0 = blockIdx.z * cols_per_block;
  const int sub = threadIdx.x % TPC, col_local = threadIdx.x / TPC, col = col0 + col_local;
  const bool has_col = col < vdim;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave, n_waves = blockDim.x / kWave;
  const int q0 = seq_qstart[seq], ql = seq_qlen[seq];
  float* S_head = state + (static_cast<size_t>(state_slots[seq]) * n_heads + h) * dim * vdim;
  const bool delta = write_mode == 1;
  const float skip_h = skip != nullptr ? skip[h] : 0.f;

  float S[kScanRows];
#pragma unroll
  for (int r = 0; r < kScanRows; ++r) {
    const int i = sub * kScanRows + r;
    S[r] = has_col && i < dim ? S_head[static_cast<size_t>(i) * vdim + col] : 0.f;
  }
  for (int t0 = 0; t0 < ql; t0 += chunk) {
    const int nt = min(chunk, ql - t0);
    __syncthreads();  // the chunk before has been read
    if constexpr (VEC) {
      // Everything the chunk needs is asked for at once, 16 bytes a load, before anything is used: q and
      // k (eight elements a piece), the decays' logits and biases (four), v, the scalars.  One round
      // trip to memory a chunk; one after the other the loads cost a round trip each, which was most
      // of the kernel's time.
      constexpr int P8 = DP / 8 > 0 ? DP / 8 : 1;  // pieces of a padded row (DP >= 16: at least two)
      const float q_mul = unit_eps >= 0.f ? 1.f : q_scale;
      const int n_qk = 2 * nt * (DP / 8);
      float qk[8][8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int v = threadIdx.x + j * 256;
        const int item = v / P8, c = 8 * (v % P8), t = item >> 1, is_k = item & 1;
        if (v < n_qk && c < dim)
          scan_load8<T>(qkv + static_cast<size_t>(q0 + t0 + t) * qkv_stride + (is_k ? k_col : q_col) + kvh * dim + c, qk[j]);
        else {
#pragma unroll
          for (int e = 0; e < 8; ++e) qk[j][e] = 0.f;
        }
      }
      constexpr int P4 = DP / 4;
      const int n_dec = decay_mode == 1 ? nt * P4 : 0;
      float4 dz[8], db[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int v = threadIdx.x + j * 256;
        const int t = v / P4, c = 4 * (v % P4);
        dz[j] = db[j] = make_float4(0.f, 0.f, 0.f, 0.f);
        if (v < n_dec && c < dim) {
          dz[j] = *reinterpret_cast<const float4*>(decay + static_cast<size_t>(q0 + t0 + t) * decay_stride + decay_col + h * dim + c);
          db[j] = *reinterpret_cast<const float4*>(decay_p0 + h * dim + c);
        }
      }
      const int n_v = nt * cols_per_block;
      float vv[8];
      for (int i0 = 0; i0 < n_v; i0 += 8 * 256) {  // (one pass unless a column is a single lane's)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + threadIdx.x + j * 256;
          const int t = i / cols_per_block, c = col0 + i % cols_per_block;
          vv[j] = i < n_v && c < vdim ? to_f32<T>(qkv[static_cast<size_t>(q0 + t0 + t) * qkv_stride + v_col + h * vdim + c]) : 0.f;
        }
        if (i0 + 8 * 256 < n_v) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int i = i0 + threadIdx.x + j * 256;
            if (i < n_v) vs[i] = vv[j];
          }
        }
      }
      float s_dec = 0.f, s_beta = 0.f;
      if (threadIdx.x < nt) {
        const size_t n = static_cast<size_t>(q0 + t0 + threadIdx.x);
        if (decay_mode == 0) s_dec = decay[n * decay_stride + decay_col + h];
        if (delta) s_beta = beta[n * beta_stride + beta_col + h];
      }
      // ---- everything is on its way; now the stores
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int v = threadIdx.x + j * 256;
        if (v < n_qk) {
          const int item = v / P8, c = 8 * (v % P8), t = item >> 1, is_k = item & 1;
          const float mul = is_k ? 1.f : q_mul;
          float* dst = (is_k ? ks : qs) + t * DS + c;
          *reinterpret_cast<float4*>(dst) = make_float4(qk[j][0] * mul, qk[j][1] * mul, qk[j][2] * mul, qk[j][3] * mul);
          *reinterpret_cast<float4*>(dst + 4) = make_float4(qk[j][4] * mul, qk[j][5] * mul, qk[j][6] * mul, qk[j][7] * mul);
        }
      }
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const int v = threadIdx.x + j * 256;
        if (v < n_dec) {
          const int c = 4 * (v % P4);
          // sigmoid(z)^(1/tau); channels past dim decay to nothing (their rows of S are zeros anyway)
          float4 a = make_float4(0.f, 0.f, 0.f, 0.f);
          if (c < dim)
            a = make_float4(expf(-scan_softplus(-(dz[j].x + db[j].x)) / tau), expf(-scan_softplus(-(dz[j].y + db[j].y)) / tau),
                            expf(-scan_softplus(-(dz[j].z + db[j].z)) / tau), expf(-scan_softplus(-(dz[j].w + db[j].w)) / tau));
          *reinterpret_cast<float4*>(as + (v / P4) * DS + c) = a;
        }
      }
      {
        const int i0 = (n_v - 1) / (8 * 256) * (8 * 256);  // the last pass's values are still in registers
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + threadIdx.x + j * 256;
          if (i < n_v) vs[i] = vv[j];
        }
      }
      if (threadIdx.x < nt) {
        const float step = decay_mode == 0 ? scan_softplus(s_dec + decay_p1[h]) : 1.f;
        if (decay_mode == 0) as[threadIdx.x] = expf(-expf(decay_p0[h]) * step);
        bs[threadIdx.x] = delta ? 1.f / (1.f + expf(-s_beta)) : (write_mode == 2 ? step : 1.f);
      }
    } else {
    // q and k of the chunk's tokens to LDS, every load of a thread asked for before the first is used
    // (one after the other they cost a round trip to memory each)
    {
      const float q_mul = unit_eps >= 0.f ? 1.f : q_scale;
      const int total = 2 * nt * DP;
      for (int i0 = threadIdx.x; i0 < total; i0 += 8 * blockDim.x) {
        float x[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + j * blockDim.x;
          const int item = i / DP, c = i % DP, t = item >> 1, is_k = item & 1;
          x[j] = i < total && c < dim
                     ? to_f32<T>(qkv[static_cast<size_t>(q0 + t0 + t) * qkv_stride + (is_k ? k_col : q_col) + kvh * dim + c])
                     : 0.f;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + j * blockDim.x;
          if (i < total) {
            const int item = i / DP, c = i % DP, t = item >> 1, is_k = item & 1;
            ((is_k ? ks : qs) + t * DS)[c] = is_k ? x[j] : x[j] * q_mul;
          }
        }
      }
    }
    if (decay_mode == 1) {
      const int total = nt * DP;
      for (int i0 = threadIdx.x; i0 < total; i0 += 8 * blockDim.x) {
        float z[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + j * blockDim.x;
          const int t = i / DP, c = i % DP;
          z[j] = i < total && c < dim
                     ? decay[static_cast<size_t>(q0 + t0 + t) * decay_stride + decay_col + h * dim + c] + decay_p0[h * dim + c]
                     : INFINITY;
        }
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int i = i0 + j * blockDim.x;
          // sigmoid(z)^(1/tau); channels past dim decay to nothing (their rows of S are zeros anyway)
          if (i < total) as[(i / DP) * DS + i % DP] = i % DP < dim ? expf(-scan_softplus(-z[j]) / tau) : 0.f;
        }
      }
    }
    for (int i = threadIdx.x; i < nt * cols_per_block; i += blockDim.x) {
      const int t = i / cols_per_block, c = col0 + i % cols_per_block;
      vs[i] = c < vdim ? to_f32<T>(qkv[static_cast<size_t>(q0 + t0 + t) * qkv_stride + v_col + h * vdim + c]) : 0.f;
    }
    for (int t = threadIdx.x; t < nt; t += blockDim.x) {
      const size_t n = static_cast<size_t>(q0 + t0 + t);
      const float step = decay_mode == 0 ? scan_softplus(decay[n * decay_stride + decay_col + h] + decay_p1[h]) : 1.f;
      if (decay_mode == 0) as[t] = expf(-expf(decay_p0[h]) * step);
      bs[t] = delta ? 1.f / (1.f + expf(-beta[n * beta_stride + beta_col + h])) : (write_mode == 2 ? step : 1.f);
    }
    }
    __syncthreads();
    // eight lanes a token: unit norms (the rows scaled where they lie) and k . q, which the read-out needs;
    // the sums over a token's eight lanes are register exchanges
    for (int t = threadIdx.x / 8; t < nt; t += blockDim.x / 8) {
      const int s8 = threadIdx.x % 8;
      float* qrow = qs + t * DS;
      float* krow = ks + t * DS;
      float ssq = 0.f, ssk = 0.f, dot = 0.f;
      for (int c = 4 * s8; c < DP; c += 32) {
        const float4 a = *reinterpret_cast<const float4*>(qrow + c), b = *reinterpret_cast<const float4*>(krow + c);
        ssq = fmaf(a.x, a.x, fmaf(a.y, a.y, fmaf(a.z, a.z, fmaf(a.w, a.w, ssq))));
        ssk = fmaf(b.x, b.x, fmaf(b.y, b.y, fmaf(b.z, b.z, fmaf(b.w, b.w, ssk))));
        dot = fmaf(a.x, b.x, fmaf(a.y, b.y, fmaf(a.z, b.z, fmaf(a.w, b.w, dot))));
      }
      dot = column_sum<8>(dot);
      if (unit_eps >= 0.f) {
        const float mq = q_scale / sqrtf(column_sum<8>(ssq) + unit_eps), mk = 1.f / sqrtf(column_sum<8>(ssk) + unit_eps);
        for (int c = 4 * s8; c < DP; c += 32) {
          float4 a = *reinterpret_cast<const float4*>(qrow + c), b = *reinterpret_cast<const float4*>(krow + c);
          a.x *= mq; a.y *= mq; a.z *= mq; a.w *= mq;
          b.x *= mk; b.y *= mk; b.z *= mk; b.w *= mk;
          *reinterpret_cast<float4*>(qrow + c) = a;
          *reinterpret_cast<float4*>(krow + c) = b;
        }
        dot *= mq * mk;
      }
      if (s8 == 0) kqs[t] = dot;
    }
    __syncthreads();
    // the walk; a token's k, q and decays are read from LDS while the token before is worked on
    // (the token's scalars come with them: read where they are used, each costs the single wave of a SIMD a
    // round trip to LDS that nothing hides)
    float kn[kScanRows], qn[kScanRows], an[kScanRows];
    float a_n = 1.f, v_n = 0.f, b_n = 1.f, kq_n = 0.f;
    auto fetch = [&](int t) {
      if (decay_mode != 1) a_n = as[t];
      v_n = vs[t * cols_per_block + col_local];
      b_n = bs[t];
      kq_n = kqs[t];
      const float4* kt = reinterpret_cast<const float4*>(ks + t * DS + sub * kScanRows);
      const float4* qt = reinterpret_cast<const float4*>(qs + t * DS + sub * kScanRows);
#pragma unroll
      for (int r4 = 0; r4 < kScanRows / 4; ++r4) {
        const float4 k4 = kt[r4], q4 = qt[r4];
        kn[4 * r4] = k4.x; kn[4 * r4 + 1] = k4.y; kn[4 * r4 + 2] = k4.z; kn[4 * r4 + 3] = k4.w;
        qn[4 * r4] = q4.x; qn[4 * r4 + 1] = q4.y; qn[4 * r4 + 2] = q4.z; qn[4 * r4 + 3] = q4.w;
      }
      if (decay_mode == 1) {
        const float4* at = reinterpret_cast<const float4*>(as + t * DS + sub * kScanRows);
#pragma unroll
        for (int r4 = 0; r4 < kScanRows / 4; ++r4) {
          const float4 a4 = at[r4];
          an[4 * r4] = a4.x; an[4 * r4 + 1] = a4.y; an[4 * r4 + 2] = a4.z; an[4 * r4 + 3] = a4.w;
        }
      }
    };
    fetch(0);
#pragma unroll 2
    for (int t = 0; t < nt; ++t) {
      float kr[kScanRows], qr[kScanRows];
#pragma unroll
      for (int r = 0; r < kScanRows; ++r) {
        kr[r] = kn[r];
        qr[r] = qn[r];
      }
      if (decay_mode == 1) {
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) S[r] *= an[r];
      } else {
        const float a = a_n;
#pragma unroll
        for (int r = 0; r < kScanRows; ++r) S[r] *= a;
      }
      const float v_t = v_n, b_t = b_n, kq_t = kq_n;
      if (t + 1 < nt) fetch(t + 1);
      // both sums over the decayed S at once: S^T k for the write, S^T q for the read-out, which sees the
      // token's own write through q . (k u^T) = u (k . q)
      float pk[4] = {0.f, 0.f, 0.f, 0.f}, pq[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int r = 0; r < kScanRows; ++r) {
        pk[r % 4] = fmaf(S[r], kr[r], pk[r % 4]);
        pq[r % 4] = fmaf(S[r], qr[r], pq[r % 4]);
      }
      const float sq = column_sum<TPC>((pq[0] + pq[1]) + (pq[2] + pq[3]));
      float u = v_t;
      if (delta) u = b_t * (u - column_sum<TPC>((pk[0] + pk[1]) + (pk[2] + pk[3])));
      else u *= b_t;  // (1 for plain writes)
      const float so = fmaf(skip_h, v_t, fmaf(u, kq_t, sq));
#pragma unroll
      for (int r = 0; r < kScanRows; ++r) S[r] = fmaf(kr[r], u, S[r]);
      if (has_col && sub == 0) out[(static_cast<size_t>(q0 + t0 + t) * n_heads + h) * vdim + col] = so;
    }
  }
#pragma unroll
  for (int r = 0; r < kScanRows; ++r) {
    const int i = sub * kScanRows + r;
    if (has_col && i < dim) S_head[static_cast<size_t>(i) * vdim + col] = S[r];
  }
}

// decay_mode 0: one decay per head from decay[n, decay_col + h], p0 = A_log [heads], p1 = dt_bias [heads];
// decay_mode 1: one per key channel from decay[n, decay_col + h * dim + i], p0 = bias [heads * dim], tau.
// write_mode 0: plain writes; 1: the delta rule with beta = sigmoid(beta[n, beta_col + h]); 2: u = dt v with the
// step dt = softplus(decay[n, decay_col + h] + p1[h]) that the head's decay is made of (decay_mode 0 only).
// unit_eps < 0: q and k are taken as they are.  q_col, k_col, v_col: where the kv_heads' queries and keys and the
// heads' values start in a row of qkv.  skip [heads] or null: o += skip[h] v.
extern "C" int yk_linear_state_scan(const void* qkv, int qkv_stride, int dtype, int n_heads, int n_kv, int dim, int vdim,
                                    float* state, const int32_t* seq_qstart, const int32_t* seq_qlen,
                                    const int32_t* state_slots, int n_seqs, int n_tokens, float q_scale, float unit_eps, int decay_mode,
                                    const float* decay, int decay_stride, int decay_col, const float* decay_p0,
                                    const float* decay_p1, float tau, const float* beta, int beta_stride, int beta_col,
                                    float* out, int q_col, int k_col, int v_col, int write_mode, const float* skip,
                                    hipStream_t stream) {
  YK_REQUIRE(n_seqs >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && dim > 0 && vdim > 0, "linear_state_scan: bad sizes");
  YK_REQUIRE(q_col >= 0 && k_col >= 0 && v_col >= 0 && qkv_stride >= std::max(std::max(q_col, k_col) + n_kv * dim, v_col + n_heads * vdim),
             "linear_state_scan: rows shorter than q, k and v");
  YK_REQUIRE(write_mode == 0 || (write_mode == 1 && beta != nullptr) || (write_mode == 2 && decay_mode == 0),
             "linear_state_scan: the delta rule needs beta, a write by the step the decay per head");
  YK_REQUIRE(decay_mode == 0 || decay_mode == 1, "linear_state_scan: unknown kind of decay");
  YK_REQUIRE(decay != nullptr && decay_p0 != nullptr && (decay_mode == 1 || decay_p1 != nullptr), "linear_state_scan: the decay's inputs are missing");
  YK_REQUIRE(decay_mode == 0 || tau > 0.f, "linear_state_scan: tau must be positive");
  YK_REQUIRE(dim <= kScanRowsMax * kWave, "linear_state_scan: heads of more than 1,024 key channels are not offered");
  if (n_seqs == 0) return 0;
  // eight rows a lane while that leaves a column inside a wave (a wave's instructions per token are what
  // the walk costs: fewer rows a lane, more lanes a column), sixteen beyond
  // (steps of single tokens are all staging and no walk: there the fewer, larger workgroups of sixteen rows
  // a lane stage less twice)
  const int rows = dim <= 8 * kWave && n_tokens > 4 * n_seqs ? 8 : 16;
  int tpc = 1;
  while (tpc * rows < dim) tpc *= 2;
  // (always 256 threads: columns a workgroup has no use for idle in the walk but help to stage)
  const int threads = 256;
  const int cols = threads / tpc;
  dim3 grid(n_seqs, n_heads, (vdim + cols - 1) / cols);
  const size_t dp = static_cast<size_t>(tpc) * rows;
  int chunk = kScanTokens;
  const size_t per_token = sizeof(float) * (2 * (dp + 4) + (decay_mode == 1 ? dp + 4 : 1) + cols + 2);
  while (chunk > 4 && (chunk * per_token > 110 * 1024 || chunk * dp > 8192)) chunk /= 2;
  const size_t lds = chunk * per_token;
  YK_REQUIRE(lds <= 128 * 1024, "linear_state_scan: the staged tokens do not fit in LDS");
  auto al16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = dim % 8 == 0 && qkv_stride % 8 == 0 && q_col % 8 == 0 && k_col % 8 == 0 && al16(qkv) && chunk * dp <= 8192 &&
                   (decay_mode == 0 || (decay_stride % 4 == 0 && decay_col % 4 == 0 && al16(decay) && al16(decay_p0)));
#define YK_LAUNCH(T, TPC)                                                                                                       \
  {                                                                                                                             \
    auto kern = rows == 8 ? (vec ? linear_state_scan_kernel<T, TPC, 8, true> : linear_state_scan_kernel<T, TPC, 8, false>)      \
                          : (vec ? linear_state_scan_kernel<T, TPC, 16, true> : linear_state_scan_kernel<T, TPC, 16, false>);   \
    if (lds > 64 * 1024 && hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, \
                                               static_cast<int>(lds)) != hipSuccess)                                            \
      return yk_fail("linear_state_scan: the staged tokens do not fit in LDS");                                                 \
    kern<<<grid, threads, lds, stream>>>(static_cast<const T*>(qkv), qkv_stride, n_heads, n_kv, dim, vdim, state, seq_qstart,   \
                                         seq_qlen, state_slots, q_scale, unit_eps, decay_mode, decay, decay_stride, decay_col,  \
                                         decay_p0, decay_p1, tau, beta, beta_stride, beta_col, chunk, out, q_col, k_col,       \
                                         v_col, write_mode, skip);                                                              \
    return yk_check_launch("linear_state_scan");                                                                                \
  }
#define YK_TPC(T)                   \
  switch (tpc) {                    \
    case 1: YK_LAUNCH(T, 1)         \
    case 2: YK_LAUNCH(T, 2)         \
    case 4: YK_LAUNCH(T, 4)         \
    case 8: YK_LAUNCH(T, 8)         \
    case 16: YK_LAUNCH(T, 16)       \
    case 32: YK_LAUNCH(T, 32)       \
    default: YK_LAUNCH(T, 64)       \
  }
  if (dtype == YK_F32) YK_TPC(float)
  if (dtype == YK_BF16) YK_TPC(bf16_t)
#undef YK_TPC
#undef YK_LAUNCH
  return yk_fail("linear_state_scan: unsupported dtype");
}

// --------------------------------------------------------------- the read-out's norm and gate
// a wave per (token, part of vdim elements): y = o / sqrt(mean(o^2) + eps) * w * silu(gate), or, gate_first, the gate
// before the norm: y = g / sqrt(mean(g^2) + eps) * w with g = o * silu(gate).  w_stride 0: one weight of vdim elements
// for every part; vdim: a weight of n_heads * vdim elements.
template <typename TW, typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, const TW* __restrict__ w, float eps,
                                                              const TG* __restrict__ gate, int gate_stride, int gate_col,
                                                              int n_heads, int vdim, TO* __restrict__ out, size_t total,
                                                              int w_stride, int gate_first) {
  const size_t item = blockIdx.x * static_cast<size_t>(blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= total) return;
  const int lane = threadIdx.x % kWave;
  const size_t n = item / n_heads;
  const int h = static_cast<int>(item % n_heads);
  const float* row = o + item * vdim;
  const TG* g = gate + n * gate_stride + gate_col + h * vdim;
  const TW* wp = w + static_cast<size_t>(h) * w_stride;
  float ss = 0.f;
  if (gate_first) {
    for (int c = lane; c < vdim; c += kWave) {
      const float v = row[c] * act_silu(to_f32<TG>(g[c]));
      ss = fmaf(v, v, ss);
    }
    const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
    for (int c = lane; c < vdim; c += kWave)
      out[item * vdim + c] = from_f32<TO>(row[c] * act_silu(to_f32<TG>(g[c])) * inv * to_f32<TW>(wp[c]));
    return;
  }
  for (int c = lane; c < vdim; c += kWave) ss = fmaf(row[c], row[c], ss);
  const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
  for (int c = lane; c < vdim; c += kWave)
    out[item * vdim + c] = from_f32<TO>(row[c] * inv * to_f32<TW>(wp[c]) * act_silu(to_f32<TG>(g[c])));
}

extern "C" int yk_gated_head_norm(const float* o, const void* w, int w_dtype, float eps, const void* gate, int gate_dtype,
                                  int gate_stride, int gate_col, int n_heads, int vdim, void* out, int out_dtype, int n_tokens,
                                  int w_per_part, int gate_first, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && vdim > 0 && gate_stride >= gate_col + n_heads * vdim, "gated_head_norm: bad sizes");
  YK_REQUIRE(gate_dtype == out_dtype, "gated_head_norm: the gate comes in the output's dtype");
  if (n_tokens == 0) return 0;
  const size_t total = static_cast<size_t>(n_tokens) * n_heads;
  const int grid = static_cast<int>((total + 3) / 4);
  const int w_stride = w_per_part ? vdim : 0;
#define YK_CASE(WD, TW, OD, TO)                                                                                       \
  if (w_dtype == WD && out_dtype == OD) {                                                                             \
    gated_head_norm_kernel<TW, TO, TO><<<grid, 256, 0, stream>>>(o, static_cast<const TW*>(w), eps,                   \
                                                                 static_cast<const TO*>(gate), gate_stride, gate_col, \
                                                                 n_heads, vdim, static_cast<TO*>(out), total, w_stride, \
                                                                 gate_first);                                         \
    return yk_check_launch("gated_head_norm");                                                                        \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("gated_head_norm: unsupported dtype combination");
}

// ------------------------------------------------------------ a convolution's kept inputs
// state [slots][keep][channels] holds a request's last `keep` inputs, oldest first; after a span of
// ql tokens it holds the last `keep` of (old state, the span's inputs).  A thread per (request, channel).
template <typename T>
__global__ void conv_state_push_kernel(const T* __restrict__ x, int x_stride, T* __restrict__ state,
                                       const int32_t* __restrict__ seq_qstart, const int32_t* __restrict__ seq_qlen,
                                       const int32_t* __restrict__ state_slots, int keep, int channels, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const int seq = static_cast<int>(i / channels), c = static_cast<int>(i % channels);
    const int q0 = seq_qstart[seq], ql = seq_qlen[seq];
    T* st = state + static_cast<size_t>(state_slots[seq]) * keep * channels + c;
    // new[j] = old[j + ql] while that exists, else the span's input ql - keep + j; ascending j reads
    // old rows before they are overwritten (j + ql > j)
    for (int j = 0; j < keep; ++j) {
      const int from = j + ql;
      st[static_cast<size_t>(j) * channels] =
          from < keep ? st[static_cast<size_t>(from) * channels] : x[static_cast<size_t>(q0 + from - keep) * x_stride + c];
    }
  }
}

extern "C" int yk_conv_state_push(const void* x, int x_stride, int dtype, void* state, const int32_t* seq_qstart,
                                  const int32_t* seq_qlen, const int32_t* state_slots, int n_seqs, int keep, int channels,
                                  hipStream_t stream) {
  YK_REQUIRE(n_seqs >= 0 && keep >= 0 && channels > 0 && x_stride >= channels, "conv_state_push: bad sizes");
  if (n_seqs == 0 || keep == 0) return 0;
  const size_t total = static_cast<size_t>(n_seqs) * channels;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 1 << 20));
  if (dtype == YK_F32)
    conv_state_push_kernel<float><<<grid, 256, 0, stream>>>(static_cast<const float*>(x), x_stride, static_cast<float*>(state),
                                                            seq_qstart, seq_qlen, state_slots, keep, channels, total);
  else if (dtype == YK_BF16)
    conv_state_push_kernel<bf16_t><<<grid, 256, 0, stream>>>(static_cast<const bf16_t*>(x), x_stride, static_cast<bf16_t*>(state),
                                                             seq_qstart, seq_qlen, state_slots, keep, channels, total);
  else
    return yk_fail("conv_state_push: unsupported dtype");
  return yk_check_launch("conv_state_push");
}
