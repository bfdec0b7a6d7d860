// Recurrences whose memory is a matrix per head, S [dim][vdim] float32 in the request's state slot:
//
//   S <- diag(a_t) S                       a_t: one decay for the head, or one per key channel (row of S)
//   u  = v_t                               plain write
//   u  = beta_t (v_t - S^T k_t)            delta rule
//   S <- S + k_t u^T,   o_t = S^T q_t      (the read-out sees the token's own write)
//
// The columns of S never meet: column e needs k_t, q_t, a_t, beta_t and its own v_t[e] only.  So a
// column lives in the registers of a group of TPC lanes (lane s of the group holds the rows s,
// s + TPC, s + 2 TPC, ...; 16 rows a lane), the two sums over rows are exchanges inside the group,
// and a workgroup walks a request's span token by token with k, q and the decays of the next few
// tokens staged in LDS.  Decays, write strengths and unit norms are made here, in float32, from the
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

constexpr int kScanRows = 16;    // rows of S a lane holds
constexpr int kScanTokens = 16;  // tokens staged at a time

__device__ __forceinline__ float scan_softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

template <typename T>
__global__ __launch_bounds__(256) void linear_state_scan_kernel(
    const T* __restrict__ qkv, int qkv_stride, int n_heads, int n_kv, int dim, int vdim, float* __restrict__ state,
    const int32_t* __restrict__ seq_qstart, const int32_t* __restrict__ seq_qlen, const int32_t* __restrict__ state_slots,
    float q_scale, float unit_eps, int decay_mode, const float* __restrict__ decay, int decay_stride, int decay_col,
    const float* __restrict__ decay_p0, const float* __restrict__ decay_p1, float tau, const float* __restrict__ beta,
    int beta_stride, int beta_col, int tpc, float* __restrict__ out) {
  extern __shared__ float lds[];
  // [kScanTokens] x (k[dim], q[dim], a[dim or 1]), v[kScanTokens][cols], beta[kScanTokens], inv_k, inv_q
  const int cols_per_block = blockDim.x / tpc;
  float* ks = lds;
  float* qs = ks + kScanTokens * dim;
  float* as = qs + kScanTokens * dim;
  const int a_w = decay_mode == 1 ? dim : 1;
  float* vs = as + kScanTokens * a_w;
  float* bs = vs + kScanTokens * cols_per_block;
  float* inv = bs + kScanTokens;  // [kScanTokens][2]

  const int seq = blockIdx.x, h = blockIdx.y, kvh = h / (n_heads / n_kv);
  const int col0 = blockIdx.z * cols_per_block;
  const int sub = threadIdx.x % tpc, col_local = threadIdx.x / tpc, col = col0 + col_local;
  const bool has_col = col < vdim;
  const int q0 = seq_qstart[seq], ql = seq_qlen[seq];
  float* S_head = state + (static_cast<size_t>(state_slots[seq]) * n_heads + h) * dim * vdim;

  float S[kScanRows];
#pragma unroll
  for (int r = 0; r < kScanRows; ++r) {
    const int i = r * tpc + sub;
    S[r] = has_col && i < dim ? S_head[static_cast<size_t>(i) * vdim + col] : 0.f;
  }
  const int kd = n_kv * dim;
  for (int t0 = 0; t0 < ql; t0 += kScanTokens) {
    const int nt = min(kScanTokens, ql - t0);
    __syncthreads();
    for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) {
      const int t = i / dim, c = i % dim;
      const T* row = qkv + static_cast<size_t>(q0 + t0 + t) * qkv_stride;
      qs[i] = to_f32<T>(row[kvh * dim + c]);
      ks[i] = to_f32<T>(row[kd + kvh * dim + c]);
      if (decay_mode == 1) {
        const float z = decay[static_cast<size_t>(q0 + t0 + t) * decay_stride + decay_col + h * dim + c] + decay_p0[h * dim + c];
        as[i] = expf(-scan_softplus(-z) / tau);  // sigmoid(z)^(1/tau)
      }
    }
    for (int i = threadIdx.x; i < nt * cols_per_block; i += blockDim.x) {
      const int t = i / cols_per_block, c = col0 + i % cols_per_block;
      vs[i] = c < vdim ? to_f32<T>(qkv[static_cast<size_t>(q0 + t0 + t) * qkv_stride + 2 * kd + h * vdim + c]) : 0.f;
    }
    for (int t = threadIdx.x; t < nt; t += blockDim.x) {
      const size_t n = static_cast<size_t>(q0 + t0 + t);
      if (decay_mode == 0)
        as[t] = expf(-expf(decay_p0[h]) * scan_softplus(decay[n * decay_stride + decay_col + h] + decay_p1[h]));
      bs[t] = beta != nullptr ? 1.f / (1.f + expf(-beta[n * beta_stride + beta_col + h])) : 1.f;
    }
    __syncthreads();
    if (unit_eps >= 0.f) {
      // a thread per (token, q or k): the sum of squares in the order of the elements
      for (int i = threadIdx.x; i < 2 * nt; i += blockDim.x) {
        const float* x = (i & 1 ? ks : qs) + (i >> 1) * dim;
        float ss = 0.f;
        for (int c = 0; c < dim; ++c) ss = fmaf(x[c], x[c], ss);
        inv[i] = 1.f / sqrtf(ss + unit_eps);
      }
      __syncthreads();
      for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) {
        const int t = i / dim;
        qs[i] = qs[i] * inv[2 * t] * q_scale;
        ks[i] *= inv[2 * t + 1];
      }
    } else {
      for (int i = threadIdx.x; i < nt * dim; i += blockDim.x) qs[i] *= q_scale;
    }
    __syncthreads();
    for (int t = 0; t < nt; ++t) {
      const float* kt = ks + t * dim;
      const float* qt = qs + t * dim;
      const float* at = as + t * a_w;
      float kr[kScanRows];
      float sk = 0.f;
#pragma unroll
      for (int r = 0; r < kScanRows; ++r) {
        const int i = r * tpc + sub;
        const bool in = i < dim;
        kr[r] = in ? kt[i] : 0.f;
        const float a = decay_mode == 1 ? (in ? at[i] : 0.f) : at[0];
        S[r] *= a;
        sk = fmaf(S[r], kr[r], sk);
      }
      float u = vs[t * cols_per_block + col_local];
      if (beta != nullptr) {
        for (int o = tpc / 2; o > 0; o >>= 1) sk += __shfl_xor(sk, o, kWave);
        u = bs[t] * (u - sk);
      }
      float so = 0.f;
#pragma unroll
      for (int r = 0; r < kScanRows; ++r) {
        const int i = r * tpc + sub;
        S[r] = fmaf(kr[r], u, S[r]);
        so = fmaf(S[r], i < dim ? qt[i] : 0.f, so);
      }
      for (int o = tpc / 2; o > 0; o >>= 1) so += __shfl_xor(so, o, kWave);
      if (has_col && sub == 0) out[(static_cast<size_t>(q0 + t0 + t) * n_heads + h) * vdim + col] = so;
    }
  }
#pragma unroll
  for (int r = 0; r < kScanRows; ++r) {
    const int i = r * tpc + sub;
    if (has_col && i < dim) S_head[static_cast<size_t>(i) * vdim + col] = S[r];
  }
}

// decay_mode 0: one decay per head from decay[n, decay_col + h], p0 = A_log [heads], p1 = dt_bias [heads];
// decay_mode 1: one per key channel from decay[n, decay_col + h * dim + i], p0 = bias [heads * dim], tau.
// beta null: plain writes; else the delta rule with beta = sigmoid(beta[n, beta_col + h]).  unit_eps < 0: q
// and k are taken as they are.
extern "C" int yk_linear_state_scan(const void* qkv, int qkv_stride, int dtype, int n_heads, int n_kv, int dim, int vdim,
                                    float* state, const int32_t* seq_qstart, const int32_t* seq_qlen,
                                    const int32_t* state_slots, int n_seqs, float q_scale, float unit_eps, int decay_mode,
                                    const float* decay, int decay_stride, int decay_col, const float* decay_p0,
                                    const float* decay_p1, float tau, const float* beta, int beta_stride, int beta_col,
                                    float* out, hipStream_t stream) {
  YK_REQUIRE(n_seqs >= 0 && n_heads > 0 && n_kv > 0 && n_heads % n_kv == 0 && dim > 0 && vdim > 0, "linear_state_scan: bad sizes");
  YK_REQUIRE(qkv_stride >= 2 * n_kv * dim + n_heads * vdim, "linear_state_scan: rows shorter than q, k and v");
  YK_REQUIRE(decay_mode == 0 || decay_mode == 1, "linear_state_scan: unknown kind of decay");
  YK_REQUIRE(decay != nullptr && decay_p0 != nullptr && (decay_mode == 1 || decay_p1 != nullptr), "linear_state_scan: the decay's inputs are missing");
  YK_REQUIRE(decay_mode == 0 || tau > 0.f, "linear_state_scan: tau must be positive");
  YK_REQUIRE(dim <= kScanRows * kWave, "linear_state_scan: heads of more than 1,024 key channels are not offered");
  if (n_seqs == 0) return 0;
  int tpc = 1;
  while (tpc * kScanRows < dim) tpc *= 2;
  int threads = vdim * tpc;
  threads = std::min(256, (threads + kWave - 1) / kWave * kWave);
  const int cols = threads / tpc;
  dim3 grid(n_seqs, n_heads, (vdim + cols - 1) / cols);
  const size_t lds = sizeof(float) * (static_cast<size_t>(kScanTokens) * (2 * dim + (decay_mode == 1 ? dim : 1) + cols + 3));
  YK_REQUIRE(lds <= 64 * 1024, "linear_state_scan: the staged tokens do not fit in LDS");
  if (dtype == YK_F32)
    linear_state_scan_kernel<float><<<grid, threads, lds, stream>>>(
        static_cast<const float*>(qkv), qkv_stride, n_heads, n_kv, dim, vdim, state, seq_qstart, seq_qlen, state_slots, q_scale,
        unit_eps, decay_mode, decay, decay_stride, decay_col, decay_p0, decay_p1, tau, beta, beta_stride, beta_col, tpc, out);
  else if (dtype == YK_BF16)
    linear_state_scan_kernel<bf16_t><<<grid, threads, lds, stream>>>(
        static_cast<const bf16_t*>(qkv), qkv_stride, n_heads, n_kv, dim, vdim, state, seq_qstart, seq_qlen, state_slots, q_scale,
        unit_eps, decay_mode, decay, decay_stride, decay_col, decay_p0, decay_p1, tau, beta, beta_stride, beta_col, tpc, out);
  else
    return yk_fail("linear_state_scan: unsupported dtype");
  return yk_check_launch("linear_state_scan");
}

// --------------------------------------------------------------- the read-out's norm and gate
// a wave per (token, head): y = o / sqrt(mean(o^2) + eps) * w * silu(gate)
template <typename TW, typename TG, typename TO>
__global__ __launch_bounds__(256) void gated_head_norm_kernel(const float* __restrict__ o, const TW* __restrict__ w, float eps,
                                                              const TG* __restrict__ gate, int gate_stride, int gate_col,
                                                              int n_heads, int vdim, TO* __restrict__ out, size_t total) {
  const size_t item = blockIdx.x * static_cast<size_t>(blockDim.x / kWave) + threadIdx.x / kWave;
  if (item >= total) return;
  const int lane = threadIdx.x % kWave;
  const size_t n = item / n_heads;
  const int h = static_cast<int>(item % n_heads);
  const float* row = o + item * vdim;
  float ss = 0.f;
  for (int c = lane; c < vdim; c += kWave) ss = fmaf(row[c], row[c], ss);
  const float inv = 1.f / sqrtf(wave_sum(ss) / static_cast<float>(vdim) + eps);
  const TG* g = gate + n * gate_stride + gate_col + h * vdim;
  for (int c = lane; c < vdim; c += kWave)
    out[item * vdim + c] = from_f32<TO>(row[c] * inv * to_f32<TW>(w[c]) * act_silu(to_f32<TG>(g[c])));
}

extern "C" int yk_gated_head_norm(const float* o, const void* w, int w_dtype, float eps, const void* gate, int gate_dtype,
                                  int gate_stride, int gate_col, int n_heads, int vdim, void* out, int out_dtype, int n_tokens,
                                  hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && n_heads > 0 && vdim > 0 && gate_stride >= gate_col + n_heads * vdim, "gated_head_norm: bad sizes");
  YK_REQUIRE(gate_dtype == out_dtype, "gated_head_norm: the gate comes in the output's dtype");
  if (n_tokens == 0) return 0;
  const size_t total = static_cast<size_t>(n_tokens) * n_heads;
  const int grid = static_cast<int>((total + 3) / 4);
#define YK_CASE(WD, TW, OD, TO)                                                                                       \
  if (w_dtype == WD && out_dtype == OD) {                                                                             \
    gated_head_norm_kernel<TW, TO, TO><<<grid, 256, 0, stream>>>(o, static_cast<const TW*>(w), eps,                   \
                                                                 static_cast<const TO*>(gate), gate_stride, gate_col, \
                                                                 n_heads, vdim, static_cast<TO*>(out), total);        \
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
