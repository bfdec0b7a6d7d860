// A gated linear recurrence with a short causal convolution in front (the recurrent block of
// Griffin, De et al. 2024: a real-gated linear recurrent unit), over a ragged batch: every
// request brings a span of tokens and carries its state from step to step in a slot.
//
//   u_t = bias + sum_j w[c, j] * x_(t - (taps - 1 - j))          per channel c, zeros before the start
//   r_t = sigmoid(Ra[b] u_t[b] + ba), i_t = sigmoid(Ri[b] u_t[b] + bi)   per block b of channels
//   log a_t = -rate * r_t * softplus(lam),  a_t = exp(log a_t)
//   S_t = a_t * S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t
//   out_t = S_t * gelu_tanh(y_t)                                  (y the other branch, before its activation)
//
// State per request: S [channels] float32, and the last taps - 1 inputs x of the convolution
// [taps - 1, channels] in the activation dtype.  Three kernels:
//   * causal_conv: u for every token of the step (reads the state, does not change it);
//   * rglru_gates: a_t and b_t = sqrt(1 - a_t^2) i_t u_t for tiles of tokens, float32;
//   * rglru_scan: one thread per (request, channel) walks its span, writes the outputs and
//     leaves both states as the span's last token leaves them.
// The recurrence, its gates, decays and logarithms are float32; a span cut anywhere gives the
// same S bit for bit, since S is carried exactly and every token's a and b are made alone.
#include <algorithm>

#include "common.h"

template <typename T, typename TW>
__global__ void causal_conv_kernel(const T* __restrict__ x, int x_stride, const TW* __restrict__ w,
                                   const TW* __restrict__ bias, const T* __restrict__ state,
                                   const int32_t* __restrict__ token_seq, const int32_t* __restrict__ seq_qstart,
                                   const int32_t* __restrict__ state_slots, T* __restrict__ out, int channels,
                                   int taps, int act, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    const int n = static_cast<int>(i / channels), c = static_cast<int>(i % channels);
    const int seq = token_seq[n];
    const int t = n - seq_qstart[seq];  // the token's place in its span
    const T* hist = state + static_cast<size_t>(state_slots[seq]) * (taps - 1) * channels;
    float acc = bias != nullptr ? to_f32<TW>(bias[c]) : 0.f;
    for (int j = 0; j < taps; ++j) {
      const int back = taps - 1 - j;
      float v;
      if (t - back >= 0)
        v = to_f32<T>(x[static_cast<size_t>(n - back) * x_stride + c]);
      else  // before the span: the state's row (taps - 1) + (t - back), counted from its oldest
        v = to_f32<T>(hist[static_cast<size_t>(taps - 1 + t - back) * channels + c]);
      acc = fmaf(to_f32<TW>(w[static_cast<size_t>(c) * taps + j]), v, acc);
    }
    out[i] = from_f32<T>(act == 1 ? act_silu(acc) : acc);
  }
}

// act: 0 none, 1 silu on the convolution's output
extern "C" int yk_causal_conv(const void* x, int x_stride, int dtype, const void* w, const void* bias, int w_dtype,
                              const void* state, const int32_t* token_seq, const int32_t* seq_qstart,
                              const int32_t* state_slots, void* out, int n_tokens, int channels, int taps, int act,
                              hipStream_t stream) {
  YK_REQUIRE(act == 0 || act == 1, "causal_conv: unknown activation");
  YK_REQUIRE(n_tokens >= 0 && channels > 0 && taps >= 1 && x_stride >= channels, "causal_conv: bad sizes");
  YK_REQUIRE(taps == 1 || state != nullptr, "causal_conv: a convolution of several taps needs its state");
  if (n_tokens == 0) return 0;
  const size_t total = static_cast<size_t>(n_tokens) * channels;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 1 << 20));
#define YK_CASE(D, T, WD, TW)                                                                                   \
  if (dtype == D && w_dtype == WD) {                                                                             \
    causal_conv_kernel<T, TW><<<grid, 256, 0, stream>>>(static_cast<const T*>(x), x_stride, static_cast<const TW*>(w), \
                                                        static_cast<const TW*>(bias), static_cast<const T*>(state),     \
                                                        token_seq, seq_qstart, state_slots, static_cast<T*>(out),       \
                                                        channels, taps, act, total);                                    \
    return yk_check_launch("causal_conv");                                                                       \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("causal_conv: unsupported dtype combination");
}

// --------------------------------------------------------------------------------- gates
constexpr int kGateTokens = 16;  // tokens a workgroup takes through one block's two matrices

__device__ __forceinline__ float softplus_f32(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// Weights come transposed, [block][in][out], so that the threads of a workgroup (one per output
// channel of the block) read consecutive addresses at every step of the sum.
template <typename T, typename TW>
__global__ __launch_bounds__(256) void rglru_gates_kernel(
    const T* __restrict__ u, const TW* __restrict__ wa_t, const TW* __restrict__ ba, const TW* __restrict__ wi_t,
    const TW* __restrict__ bi, const TW* __restrict__ lam, float rate, float* __restrict__ a_out,
    float* __restrict__ b_out, int n_tokens, int channels, int block_size) {
  extern __shared__ float us[];  // [kGateTokens][block_size]
  const int n0 = blockIdx.x * kGateTokens, b = blockIdx.y;
  const int count = min(kGateTokens, n_tokens - n0);
  for (int i = threadIdx.x; i < kGateTokens * block_size; i += blockDim.x) {
    const int t = i / block_size, k = i % block_size;
    us[i] = t < count ? to_f32<T>(u[static_cast<size_t>(n0 + t) * channels + b * block_size + k]) : 0.f;
  }
  __syncthreads();
  const size_t mat = static_cast<size_t>(b) * block_size * block_size;
  for (int o = threadIdx.x; o < block_size; o += blockDim.x) {
    float ra[kGateTokens], ri[kGateTokens];
#pragma unroll
    for (int t = 0; t < kGateTokens; ++t) ra[t] = ri[t] = 0.f;
    for (int k = 0; k < block_size; ++k) {
      const float wa = to_f32<TW>(wa_t[mat + static_cast<size_t>(k) * block_size + o]);
      const float wi = to_f32<TW>(wi_t[mat + static_cast<size_t>(k) * block_size + o]);
#pragma unroll
      for (int t = 0; t < kGateTokens; ++t) {
        const float uv = us[t * block_size + k];
        ra[t] = fmaf(wa, uv, ra[t]);
        ri[t] = fmaf(wi, uv, ri[t]);
      }
    }
    const int c = b * block_size + o;
    const float bav = to_f32<TW>(ba[c]), biv = to_f32<TW>(bi[c]);
    const float decay = rate * softplus_f32(to_f32<TW>(lam[c]));
#pragma unroll
    for (int t = 0; t < kGateTokens; ++t) {
      if (t < count) {
        const float r = 1.f / (1.f + expf(-(ra[t] + bav)));
        const float ig = 1.f / (1.f + expf(-(ri[t] + biv)));
        const float log_a = -decay * r;
        const float a = expf(log_a);
        const float root = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f));  // sqrt(1 - a^2)
        const size_t idx = static_cast<size_t>(n0 + t) * channels + c;
        a_out[idx] = a;
        b_out[idx] = root * ig * us[t * block_size + o];
      }
    }
  }
}


// The same gates on the matrix cores, for bfloat16 branches and weights with blocks of a multiple
// of 32 channels: the products u_b . Ra[b]^T and u_b . Ri[b]^T are bfloat16 x bfloat16 with float32
// accumulation (every product of two bfloat16 numbers is exact in float32, so only the order of
// the sum differs from the kernel above); sigmoids, decays and roots are float32 as there.
// A wave owns 16 output channels of a block and 64 tokens; the weights come in the checkpoint's
// own layout [block][out][in], whose rows are the A operand as they lie.
typedef __bf16 rg_bf16x8_t __attribute__((ext_vector_type(8)));
typedef float rg_f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t rg_u32x4_t __attribute__((ext_vector_type(4)));
union RgFrag {
  rg_u32x4_t u;
  rg_bf16x8_t v;
};

__global__ __launch_bounds__(256) void rglru_gates_mfma_kernel(
    const bf16_t* __restrict__ u, const bf16_t* __restrict__ wa, const bf16_t* __restrict__ ba,
    const bf16_t* __restrict__ wi, const bf16_t* __restrict__ bi, const bf16_t* __restrict__ lam, float rate,
    float* __restrict__ a_out, float* __restrict__ b_out, int n_tokens, int channels, int block_size) {
  constexpr int MT = 4;
  const int wave = threadIdx.x / 64, lane = threadIdx.x % 64, r = lane % 16, g = lane / 16;
  const int n0 = blockIdx.x * 16 * MT, b = blockIdx.y;
  const int o0 = (blockIdx.z * 4 + wave) * 16;  // first output channel of the wave within the block
  if (o0 >= block_size) return;
  const size_t mat = static_cast<size_t>(b) * block_size * block_size;
  const bf16_t* wa_row = wa + mat + static_cast<size_t>(o0 + r) * block_size + 8 * g;
  const bf16_t* wi_row = wi + mat + static_cast<size_t>(o0 + r) * block_size + 8 * g;
  const bf16_t* ur[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m)
    ur[m] = u + static_cast<size_t>(min(n0 + 16 * m + r, n_tokens - 1)) * channels + b * block_size + 8 * g;
  rg_f32x4_t acc_a[MT], acc_i[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) acc_a[m] = acc_i[m] = rg_f32x4_t{0.f, 0.f, 0.f, 0.f};
  for (int k0 = 0; k0 < block_size; k0 += 32) {
    RgFrag fa, fi, fu[MT];
    fa.u = *reinterpret_cast<const rg_u32x4_t*>(wa_row + k0);
    fi.u = *reinterpret_cast<const rg_u32x4_t*>(wi_row + k0);
#pragma unroll
    for (int m = 0; m < MT; ++m) fu[m].u = *reinterpret_cast<const rg_u32x4_t*>(ur[m] + k0);
#pragma unroll
    for (int m = 0; m < MT; ++m) {
      acc_a[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa.v, fu[m].v, acc_a[m], 0, 0, 0);
      acc_i[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fi.v, fu[m].v, acc_i[m], 0, 0, 0);
    }
  }
  // lane (r, g) holds, for token 16m + r, the channels o0 + 4g .. 4g + 3
  const int c0 = b * block_size + o0 + 4 * g;
  float bav[4], biv[4], decay[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    bav[i] = bf16_to_f32(ba[c0 + i]);
    biv[i] = bf16_to_f32(bi[c0 + i]);
    decay[i] = rate * softplus_f32(bf16_to_f32(lam[c0 + i]));
  }
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    const int n = n0 + 16 * m + r;
    if (n >= n_tokens) continue;
    const uint2 uw = *reinterpret_cast<const uint2*>(u + static_cast<size_t>(n) * channels + c0);
    const float uv[4] = {__uint_as_float(uw.x << 16), __uint_as_float(uw.x & 0xffff0000u), __uint_as_float(uw.y << 16),
                         __uint_as_float(uw.y & 0xffff0000u)};
    float av[4], bv[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const float rg = 1.f / (1.f + expf(-(acc_a[m][i] + bav[i])));
      const float ig = 1.f / (1.f + expf(-(acc_i[m][i] + biv[i])));
      const float log_a = -decay[i] * rg;
      av[i] = expf(log_a);
      bv[i] = sqrtf(fmaxf(-expm1f(2.f * log_a), 0.f)) * ig * uv[i];
    }
    *reinterpret_cast<float4*>(a_out + static_cast<size_t>(n) * channels + c0) = make_float4(av[0], av[1], av[2], av[3]);
    *reinterpret_cast<float4*>(b_out + static_cast<size_t>(n) * channels + c0) = make_float4(bv[0], bv[1], bv[2], bv[3]);
  }
}

// wa, wi: the matrices in the checkpoint's layout [block][out][in] (may be null: then the float32 form runs)
extern "C" int yk_rglru_gates_mfma_ok(int channels, int blocks) {
  return blocks > 0 && channels % blocks == 0 && (channels / blocks) % 32 == 0 && channels % 8 == 0;
}

extern "C" int yk_rglru_gates(const void* u, int dtype, const void* wa_t, const void* ba, const void* wi_t, const void* bi,
                              const void* lam, int w_dtype, float rate, float* a_out, float* b_out, int n_tokens,
                              int channels, int blocks, const void* wa, const void* wi, hipStream_t stream) {
  YK_REQUIRE(n_tokens >= 0 && channels > 0 && blocks > 0 && channels % blocks == 0, "rglru_gates: channels must divide into the blocks");
  YK_REQUIRE(blocks <= 65535, "rglru_gates: too many blocks for one launch");
  const int block_size = channels / blocks;
  const size_t lds = static_cast<size_t>(kGateTokens) * block_size * sizeof(float);
  if (n_tokens == 0) return 0;
  if (dtype == YK_BF16 && w_dtype == YK_BF16 && wa != nullptr && wi != nullptr && yk_rglru_gates_mfma_ok(channels, blocks) &&
      reinterpret_cast<uintptr_t>(u) % 16 == 0 && reinterpret_cast<uintptr_t>(wa) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(wi) % 16 == 0 && reinterpret_cast<uintptr_t>(a_out) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(b_out) % 16 == 0) {
    dim3 mgrid((n_tokens + 63) / 64, blocks, (block_size + 63) / 64);
    YK_REQUIRE(mgrid.z <= 65535, "rglru_gates: blocks too wide for one launch");
    rglru_gates_mfma_kernel<<<mgrid, 256, 0, stream>>>(
        static_cast<const bf16_t*>(u), static_cast<const bf16_t*>(wa), static_cast<const bf16_t*>(ba),
        static_cast<const bf16_t*>(wi), static_cast<const bf16_t*>(bi), static_cast<const bf16_t*>(lam), rate, a_out, b_out,
        n_tokens, channels, block_size);
    return yk_check_launch("rglru_gates (matrix cores)");
  }
  YK_REQUIRE(lds <= 150 * 1024, "rglru_gates: blocks of more than 2,400 channels do not fit the float32 form");
  if (lds > 48 * 1024) {  // more than the default limit of dynamic LDS: raised once per kernel form
    static bool raised = false;
    if (!raised) {
      bool ok = hipFuncSetAttribute(reinterpret_cast<const void*>(&rglru_gates_kernel<float, float>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
      ok = ok && hipFuncSetAttribute(reinterpret_cast<const void*>(&rglru_gates_kernel<bf16_t, bf16_t>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
      ok = ok && hipFuncSetAttribute(reinterpret_cast<const void*>(&rglru_gates_kernel<bf16_t, float>), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
      if (!ok) return yk_fail("rglru_gates: cannot raise the LDS limit");
      raised = true;
    }
  }
  dim3 grid((n_tokens + kGateTokens - 1) / kGateTokens, blocks);
  const int threads = std::min(256, (block_size + 63) / 64 * 64);
#define YK_CASE(D, T, WD, TW)                                                                                  \
  if (dtype == D && w_dtype == WD) {                                                                            \
    rglru_gates_kernel<T, TW><<<grid, threads, lds, stream>>>(                                                  \
        static_cast<const T*>(u), static_cast<const TW*>(wa_t), static_cast<const TW*>(ba),                     \
        static_cast<const TW*>(wi_t), static_cast<const TW*>(bi), static_cast<const TW*>(lam), rate, a_out, b_out, \
        n_tokens, channels, block_size);                                                                        \
    return yk_check_launch("rglru_gates");                                                                      \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("rglru_gates: unsupported dtype combination");
}

// ---------------------------------------------------------------------------------- scan
template <typename T>
__global__ void rglru_scan_kernel(const float* __restrict__ a, const float* __restrict__ b, const T* __restrict__ y,
                                  int y_stride, const T* __restrict__ x, int x_stride, float* __restrict__ s_state,
                                  T* __restrict__ conv_state, const int32_t* __restrict__ seq_qstart,
                                  const int32_t* __restrict__ seq_qlen, const int32_t* __restrict__ state_slots,
                                  T* __restrict__ out, int channels, int taps) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int q0 = seq_qstart[seq], ql = seq_qlen[seq], slot = state_slots[seq];
  float S = s_state[static_cast<size_t>(slot) * channels + c];
  for (int t = 0; t < ql; ++t) {
    const size_t idx = static_cast<size_t>(q0 + t) * channels + c;
    S = fmaf(a[idx], S, b[idx]);
    const float yv = to_f32<T>(y[static_cast<size_t>(q0 + t) * y_stride + c]);
    out[idx] = from_f32<T>(S * act_gelu_tanh(yv));
  }
  s_state[static_cast<size_t>(slot) * channels + c] = S;
  // the convolution's last taps - 1 inputs, oldest first: what is left of the old ones, then the span's
  const int keep = taps - 1;
  if (keep > 0) {
    T* hist = conv_state + static_cast<size_t>(slot) * keep * channels;
    if (ql >= keep) {
      for (int i = 0; i < keep; ++i) hist[static_cast<size_t>(i) * channels + c] = x[static_cast<size_t>(q0 + ql - keep + i) * x_stride + c];
    } else {
      for (int i = 0; i < keep - ql; ++i) hist[static_cast<size_t>(i) * channels + c] = hist[static_cast<size_t>(i + ql) * channels + c];
      for (int i = 0; i < ql; ++i) hist[static_cast<size_t>(keep - ql + i) * channels + c] = x[static_cast<size_t>(q0 + i) * x_stride + c];
    }
  }
}

extern "C" int yk_rglru_scan(const float* a, const float* b, const void* y, int y_stride, const void* x, int x_stride,
                             int dtype, float* s_state, void* conv_state, const int32_t* seq_qstart,
                             const int32_t* seq_qlen, const int32_t* state_slots, void* out, int n_seqs, int channels,
                             int taps, hipStream_t stream) {
  YK_REQUIRE(n_seqs >= 0 && channels > 0 && taps >= 1, "rglru_scan: bad sizes");
  YK_REQUIRE(n_seqs <= 65535, "rglru_scan: too many requests for one launch");
  YK_REQUIRE(taps == 1 || conv_state != nullptr, "rglru_scan: the convolution's state is missing");
  if (n_seqs == 0) return 0;
  dim3 grid((channels + 63) / 64, n_seqs), block(64);
  if (dtype == YK_F32)
    rglru_scan_kernel<float><<<grid, block, 0, stream>>>(a, b, static_cast<const float*>(y), y_stride,
                                                        static_cast<const float*>(x), x_stride, s_state,
                                                        static_cast<float*>(conv_state), seq_qstart, seq_qlen,
                                                        state_slots, static_cast<float*>(out), channels, taps);
  else if (dtype == YK_BF16)
    rglru_scan_kernel<bf16_t><<<grid, block, 0, stream>>>(a, b, static_cast<const bf16_t*>(y), y_stride,
                                                         static_cast<const bf16_t*>(x), x_stride, s_state,
                                                         static_cast<bf16_t*>(conv_state), seq_qstart, seq_qlen,
                                                         state_slots, static_cast<bf16_t*>(out), channels, taps);
  else
    return yk_fail("rglru_scan: unsupported dtype");
  return yk_check_launch("rglru_scan");
}


// -------------------------------------------------------------------- the scan in chunks
// A long span walked by one thread per channel is a long chain of dependent steps with few
// threads.  Spans are cut into chunks (`chunks` rows of (request, first token of the batch,
// count); `seq_chunk0` [requests + 1] the first chunk of every request):
//   reduce: every chunk alone, from nothing: P = product of its a, Q = its last S started at 0;
//   carry:  per request and channel over its chunks in order: the S each chunk starts from
//           (S <- P S + Q), the request's S afterwards, and the convolution's state;
//   apply:  every chunk again from the S it starts from, writing the outputs.
// What a token gets depends on where its chunk starts only through rounding (P S + Q against
// the same steps taken one by one).
__global__ void rglru_chunk_reduce_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                          const int32_t* __restrict__ chunks, float* __restrict__ pq, int channels) {
  const int ch = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t0 = chunks[3 * ch + 1], n = chunks[3 * ch + 2];
  float P = 1.f, Q = 0.f;
  for (int t = 0; t < n; ++t) {
    const size_t idx = static_cast<size_t>(t0 + t) * channels + c;
    const float av = a[idx];
    Q = fmaf(av, Q, b[idx]);
    P *= av;
  }
  pq[(static_cast<size_t>(ch) * 2) * channels + c] = P;
  pq[(static_cast<size_t>(ch) * 2 + 1) * channels + c] = Q;
}

template <typename T>
__global__ void rglru_chunk_carry_kernel(float* __restrict__ pq, const int32_t* __restrict__ seq_chunk0,
                                         const T* __restrict__ x, int x_stride, float* __restrict__ s_state,
                                         T* __restrict__ conv_state, const int32_t* __restrict__ seq_qstart,
                                         const int32_t* __restrict__ seq_qlen, const int32_t* __restrict__ state_slots,
                                         int channels, int taps) {
  const int seq = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = state_slots[seq];
  float S = s_state[static_cast<size_t>(slot) * channels + c];
  for (int ch = seq_chunk0[seq]; ch < seq_chunk0[seq + 1]; ++ch) {
    const size_t at = (static_cast<size_t>(ch) * 2) * channels + c;
    const float P = pq[at], Q = pq[at + channels];
    pq[at] = S;  // what the chunk starts from
    S = fmaf(P, S, Q);
  }
  s_state[static_cast<size_t>(slot) * channels + c] = S;
  const int keep = taps - 1, q0 = seq_qstart[seq], ql = seq_qlen[seq];
  if (keep > 0) {
    T* hist = conv_state + static_cast<size_t>(slot) * keep * channels;
    if (ql >= keep) {
      for (int i = 0; i < keep; ++i) hist[static_cast<size_t>(i) * channels + c] = x[static_cast<size_t>(q0 + ql - keep + i) * x_stride + c];
    } else {
      for (int i = 0; i < keep - ql; ++i) hist[static_cast<size_t>(i) * channels + c] = hist[static_cast<size_t>(i + ql) * channels + c];
      for (int i = 0; i < ql; ++i) hist[static_cast<size_t>(keep - ql + i) * channels + c] = x[static_cast<size_t>(q0 + i) * x_stride + c];
    }
  }
}

template <typename T>
__global__ void rglru_chunk_apply_kernel(const float* __restrict__ a, const float* __restrict__ b, const T* __restrict__ y,
                                         int y_stride, const int32_t* __restrict__ chunks, const float* __restrict__ pq,
                                         T* __restrict__ out, int channels) {
  const int ch = blockIdx.y, c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int t0 = chunks[3 * ch + 1], n = chunks[3 * ch + 2];
  float S = pq[(static_cast<size_t>(ch) * 2) * channels + c];
  for (int t = 0; t < n; ++t) {
    const size_t idx = static_cast<size_t>(t0 + t) * channels + c;
    S = fmaf(a[idx], S, b[idx]);
    const float yv = to_f32<T>(y[static_cast<size_t>(t0 + t) * y_stride + c]);
    out[idx] = from_f32<T>(S * act_gelu_tanh(yv));
  }
}

// pq: float32 scratch [n_chunks][2][channels]
extern "C" int yk_rglru_scan_chunked(const float* a, const float* b, const void* y, int y_stride, const void* x, int x_stride,
                                     int dtype, float* s_state, void* conv_state, const int32_t* seq_qstart,
                                     const int32_t* seq_qlen, const int32_t* state_slots, const int32_t* chunks, int n_chunks,
                                     const int32_t* seq_chunk0, float* pq, void* out, int n_seqs, int channels, int taps,
                                     hipStream_t stream) {
  YK_REQUIRE(n_seqs >= 0 && n_chunks >= n_seqs && channels > 0 && taps >= 1, "rglru_scan_chunked: bad sizes");
  YK_REQUIRE(n_seqs <= 65535 && n_chunks <= 65535, "rglru_scan_chunked: too many requests or chunks for one launch");
  YK_REQUIRE(taps == 1 || conv_state != nullptr, "rglru_scan_chunked: the convolution's state is missing");
  YK_REQUIRE(dtype == YK_F32 || dtype == YK_BF16, "rglru_scan_chunked: unsupported dtype");
  if (n_seqs == 0) return 0;
  dim3 block(64), cgrid((channels + 63) / 64, n_chunks), sgrid((channels + 63) / 64, n_seqs);
  rglru_chunk_reduce_kernel<<<cgrid, block, 0, stream>>>(a, b, chunks, pq, channels);
  if (yk_check_launch("rglru_chunk_reduce")) return -1;
  if (dtype == YK_F32) {
    rglru_chunk_carry_kernel<float><<<sgrid, block, 0, stream>>>(pq, seq_chunk0, static_cast<const float*>(x), x_stride, s_state,
                                                                static_cast<float*>(conv_state), seq_qstart, seq_qlen,
                                                                state_slots, channels, taps);
    if (yk_check_launch("rglru_chunk_carry")) return -1;
    rglru_chunk_apply_kernel<float><<<cgrid, block, 0, stream>>>(a, b, static_cast<const float*>(y), y_stride, chunks, pq,
                                                                static_cast<float*>(out), channels);
  } else {
    rglru_chunk_carry_kernel<bf16_t><<<sgrid, block, 0, stream>>>(pq, seq_chunk0, static_cast<const bf16_t*>(x), x_stride, s_state,
                                                                 static_cast<bf16_t*>(conv_state), seq_qstart, seq_qlen,
                                                                 state_slots, channels, taps);
    if (yk_check_launch("rglru_chunk_carry")) return -1;
    rglru_chunk_apply_kernel<bf16_t><<<cgrid, block, 0, stream>>>(a, b, static_cast<const bf16_t*>(y), y_stride, chunks, pq,
                                                                 static_cast<bf16_t*>(out), channels);
  }
  return yk_check_launch("rglru_chunk_apply");
}
