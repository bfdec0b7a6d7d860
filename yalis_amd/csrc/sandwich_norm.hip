// Norms on both sides of a branch, in one pass over a row of the residual stream:
//
//   t        = post(branch[n, :])            (or branch[n, :] itself without a post-norm)
//   r        = residual[row, :] + scale * t  (written back unless rows are gathered)
//   out[n,:] = pre(r)                        (left out when nobody reads the stream next)
//
// post and pre are norms with weight and optional bias:
//   centred:   (x - mean) / sqrt(mean((x - mean)^2) + eps) * w + b      (a layer norm)
//   otherwise:  x / sqrt(mean(x^2) + eps) * w + b                       (an RMS norm)
// Mean and variance are taken in two passes over the row, which is parked in LDS; everything is
// float32, the output rounded once.  The branch may be a tensor in the activation dtype or
// float32, or the unreduced K slices of a product (float32 [slices, rows, width], summed in
// order and, with round_sum, rounded as the product's own output would have been).  Without a
// residual the kernel is the plain norm of the branch's rows.  `rows` (one index per output
// row) picks rows of residual and branch and leaves the residual as it is: the final norm on
// the rows whose logits are wanted.
//
// Beside it: an elementwise activation of a product's output (relu squared, silu, gelu) and the
// multiplication of float32 rows by a constant.
#include <algorithm>

#include "common.h"

struct NormStats {
  float mean, inv;
};

// mean (0 when not centred) and 1 / sqrt(variance + eps) of row[0 .. width), every thread its own columns
__device__ __forceinline__ NormStats row_stats(const float* row, int width, int center, float eps, float* scratch) {
  float mean = 0.f;
  if (center) {
    float s = 0.f;
    for (int c = threadIdx.x; c < width; c += blockDim.x) s += row[c];
    mean = block_sum(s, scratch) / static_cast<float>(width);
  }
  float ss = 0.f;
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float d = row[c] - mean;
    ss = fmaf(d, d, ss);
  }
  const float var = block_sum(ss, scratch) / static_cast<float>(width);
  return {mean, 1.f / sqrtf(var + eps)};
}

template <typename TS, typename TW, typename TO>
__global__ __launch_bounds__(256) void sandwich_norm_kernel(
    float* __restrict__ residual, const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum,
    const TW* __restrict__ wa, const TW* __restrict__ ba, float eps_a, int center_a, int has_post, float scale,
    const TW* __restrict__ wb, const TW* __restrict__ bb, float eps_b, int center_b, int has_pre,
    const int32_t* __restrict__ rows, TO* __restrict__ out, int width) {
  extern __shared__ float row[];  // [width], then 17 floats of scratch
  float* scratch = row + width;
  const size_t n = blockIdx.x;
  const size_t r = rows != nullptr ? static_cast<size_t>(rows[n]) : n;
  if (src != nullptr) {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float v = 0.f;
      for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(src[s * split_stride + r * width + c]);
      row[c] = as_output(v, round_sum);
    }
    if (has_post) {
      const NormStats st = row_stats(row, width, center_a, eps_a, scratch);
      for (int c = threadIdx.x; c < width; c += blockDim.x) {
        float t = (row[c] - st.mean) * st.inv * to_f32<TW>(wa[c]);
        if (ba != nullptr) t += to_f32<TW>(ba[c]);
        row[c] = t;
      }
    }
  }
  if (residual != nullptr) {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float v = residual[r * width + c];
      if (src != nullptr) {
        v = fmaf(scale, row[c], v);
        if (rows == nullptr) residual[r * width + c] = v;
      }
      row[c] = v;
    }
  }
  if (!has_pre) return;
  const NormStats st = row_stats(row, width, center_b, eps_b, scratch);
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    float t = (row[c] - st.mean) * st.inv * to_f32<TW>(wb[c]);
    if (bb != nullptr) t += to_f32<TW>(bb[c]);
    out[n * width + c] = from_f32<TO>(t);
  }
}

// The same for rows of up to 4,096 elements in 16-byte pieces, a thread holding up to four of them in
// registers: everything a thread reads (the branch's slices, the residual, both norms' weights and
// biases) is asked for before the first reduction, one round trip to memory instead of six.
template <typename T>
__device__ __forceinline__ float4 sn_load4(const T* p);
template <>
__device__ __forceinline__ float4 sn_load4<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 sn_load4<bf16_t>(const bf16_t* p) {
  const uint2 w = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                     __uint_as_float(w.y & 0xffff0000u));
}
template <typename T>
__device__ __forceinline__ void sn_store4(T* p, float4 v);
template <>
__device__ __forceinline__ void sn_store4<float>(float* p, float4 v) {
  *reinterpret_cast<float4*>(p) = v;
}
template <>
__device__ __forceinline__ void sn_store4<bf16_t>(bf16_t* p, float4 v) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pack_bf16x2(v.x, v.y), pack_bf16x2(v.z, v.w));
}

constexpr int kSnPieces = 4;

__device__ __forceinline__ NormStats piece_stats(const float4* v, const bool* has, int width, int center, float eps, float* scratch) {
  float mean = 0.f;
  if (center) {
    float s = 0.f;
#pragma unroll
    for (int k = 0; k < kSnPieces; ++k)
      if (has[k]) s += (v[k].x + v[k].y) + (v[k].z + v[k].w);
    mean = block_sum(s, scratch) / static_cast<float>(width);
  }
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < kSnPieces; ++k)
    if (has[k]) {
      const float a = v[k].x - mean, b = v[k].y - mean, c = v[k].z - mean, d = v[k].w - mean;
      ss = fmaf(a, a, fmaf(b, b, fmaf(c, c, fmaf(d, d, ss))));
    }
  return {mean, 1.f / sqrtf(block_sum(ss, scratch) / static_cast<float>(width) + eps)};
}

__device__ __forceinline__ float4 piece_norm(float4 v, NormStats st, float4 w, float4 b) {
  return make_float4(fmaf((v.x - st.mean) * st.inv, w.x, b.x), fmaf((v.y - st.mean) * st.inv, w.y, b.y),
                     fmaf((v.z - st.mean) * st.inv, w.z, b.z), fmaf((v.w - st.mean) * st.inv, w.w, b.w));
}

template <typename TS, typename TW, typename TO>
__global__ __launch_bounds__(256) void sandwich_norm_vec_kernel(
    float* __restrict__ residual, const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum,
    const TW* __restrict__ wa, const TW* __restrict__ ba, float eps_a, int center_a, int has_post, float scale,
    const TW* __restrict__ wb, const TW* __restrict__ bb, float eps_b, int center_b, int has_pre,
    const int32_t* __restrict__ rows, TO* __restrict__ out, int width) {
  __shared__ float scratch[17];
  const size_t n = blockIdx.x;
  const size_t r = rows != nullptr ? static_cast<size_t>(rows[n]) : n;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 br[kSnPieces], rs[kSnPieces], fwa[kSnPieces], fba[kSnPieces], fwb[kSnPieces], fbb[kSnPieces];
  bool has[kSnPieces];
#pragma unroll
  for (int k = 0; k < kSnPieces; ++k) {
    const int c = 4 * (threadIdx.x + 256 * k);
    has[k] = c < width;
    br[k] = rs[k] = fba[k] = fbb[k] = zero;
    fwa[k] = fwb[k] = zero;
    if (!has[k]) continue;
    if (src != nullptr) {
      for (int s0 = 0; s0 < n_splits; s0 += 8) {
        float4 t[8];
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < n_splits) t[j] = sn_load4<TS>(src + (s0 + j) * split_stride + r * width + c);
#pragma unroll
        for (int j = 0; j < 8; ++j)
          if (s0 + j < n_splits) {
            br[k].x += t[j].x; br[k].y += t[j].y; br[k].z += t[j].z; br[k].w += t[j].w;
          }
      }
      br[k] = make_float4(as_output(br[k].x, round_sum), as_output(br[k].y, round_sum), as_output(br[k].z, round_sum),
                          as_output(br[k].w, round_sum));
    }
    if (residual != nullptr) rs[k] = *reinterpret_cast<const float4*>(residual + r * width + c);
    if (has_post) {
      fwa[k] = sn_load4<TW>(wa + c);
      if (ba != nullptr) fba[k] = sn_load4<TW>(ba + c);
    }
    if (has_pre) {
      fwb[k] = sn_load4<TW>(wb + c);
      if (bb != nullptr) fbb[k] = sn_load4<TW>(bb + c);
    }
  }
  if (src != nullptr && has_post) {
    const NormStats st = piece_stats(br, has, width, center_a, eps_a, scratch);
#pragma unroll
    for (int k = 0; k < kSnPieces; ++k) br[k] = piece_norm(br[k], st, fwa[k], fba[k]);
  }
  if (residual != nullptr) {
#pragma unroll
    for (int k = 0; k < kSnPieces; ++k) {
      if (src != nullptr) {
        rs[k] = make_float4(fmaf(scale, br[k].x, rs[k].x), fmaf(scale, br[k].y, rs[k].y), fmaf(scale, br[k].z, rs[k].z),
                            fmaf(scale, br[k].w, rs[k].w));
        if (rows == nullptr && has[k]) *reinterpret_cast<float4*>(residual + r * width + 4 * (threadIdx.x + 256 * k)) = rs[k];
      }
    }
  } else {
#pragma unroll
    for (int k = 0; k < kSnPieces; ++k) rs[k] = br[k];
  }
  if (!has_pre) return;
  const NormStats st = piece_stats(rs, has, width, center_b, eps_b, scratch);
#pragma unroll
  for (int k = 0; k < kSnPieces; ++k)
    if (has[k]) sn_store4<TO>(out + n * width + 4 * (threadIdx.x + 256 * k), piece_norm(rs[k], st, fwb[k], fbb[k]));
}

// src_rows: rows of residual and of every slice of src (the stride between slices); n_rows: rows of out.
extern "C" int yk_sandwich_norm(float* residual, const void* src, int src_dtype, int n_splits, int round_sum, int src_rows,
                                const void* wa, const void* ba, float eps_a, int center_a, float scale, const void* wb,
                                const void* bb, float eps_b, int center_b, int w_dtype, const int32_t* rows, void* out,
                                int out_dtype, int n_rows, int width, hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && width > 0 && src_rows >= 0, "sandwich_norm: bad sizes");
  YK_REQUIRE(residual != nullptr || src != nullptr, "sandwich_norm: neither a residual nor a branch");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "sandwich_norm: unreduced slices must be float32");
  YK_REQUIRE(width <= 15 * 1024, "sandwich_norm: rows of more than 15,360 elements do not fit the row buffer");
  YK_REQUIRE((wb != nullptr) == (out != nullptr), "sandwich_norm: an output needs a norm, and a norm an output");
  YK_REQUIRE(wa == nullptr || src != nullptr, "sandwich_norm: a branch's norm needs the branch");
  if (n_rows == 0) return 0;
  const size_t stride = static_cast<size_t>(src_rows) * width;
  const size_t lds = (static_cast<size_t>(width) + 17) * sizeof(float);
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = width % 4 == 0 && width <= 4 * 256 * kSnPieces && al(residual) && al(src) && al(wa) && al(ba) && al(wb) &&
                   al(bb) && al(out);
#define YK_CASE(SD, TS, WD, TW, OD, TO)                                                                           \
  if ((src == nullptr || src_dtype == SD) && w_dtype == WD && (out == nullptr || out_dtype == OD)) {              \
    if (vec)                                                                                                      \
      sandwich_norm_vec_kernel<TS, TW, TO><<<n_rows, 256, 0, stream>>>(                                           \
          residual, static_cast<const TS*>(src), n_splits, stride, round_sum, static_cast<const TW*>(wa),         \
          static_cast<const TW*>(ba), eps_a, center_a, wa != nullptr, scale, static_cast<const TW*>(wb),          \
          static_cast<const TW*>(bb), eps_b, center_b, wb != nullptr, rows, static_cast<TO*>(out), width);        \
    else                                                                                                          \
    sandwich_norm_kernel<TS, TW, TO><<<n_rows, 256, lds, stream>>>(                                               \
        residual, static_cast<const TS*>(src), n_splits, stride, round_sum, static_cast<const TW*>(wa),           \
        static_cast<const TW*>(ba), eps_a, center_a, wa != nullptr, scale, static_cast<const TW*>(wb),            \
        static_cast<const TW*>(bb), eps_b, center_b, wb != nullptr, rows, static_cast<TO*>(out), width);          \
    return yk_check_launch("sandwich_norm");                                                                      \
  }
  YK_CASE(YK_F32, float, YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t, YK_F32, float)
#undef YK_CASE
  return yk_fail("sandwich_norm: unsupported dtype combination");
}

// ------------------------------------------------------------------------------ activation
// kinds: 0 silu, 1 gelu (tanh form), 2 the square of relu
template <typename TS, typename TO>
__global__ void activation_kernel(const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum, int kind,
                                  TO* __restrict__ out, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x) {
    float v = 0.f;
    for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(src[s * split_stride + i]);
    v = as_output(v, round_sum);
    float y;
    if (kind == 2) {
      const float p = fmaxf(v, 0.f);
      y = p * p;
    } else {
      y = act_apply(v, kind);
    }
    out[i] = from_f32<TO>(y);
  }
}

extern "C" int yk_activation(const void* src, int src_dtype, int n_splits, int round_sum, int kind, void* out, int out_dtype,
                             size_t total, hipStream_t stream) {
  YK_REQUIRE(kind >= 0 && kind <= 2, "activation: unknown kind");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "activation: unreduced slices must be float32");
  if (total == 0) return 0;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 1 << 20));
#define YK_CASE(SD, TS, OD, TO)                                                                                    \
  if (src_dtype == SD && out_dtype == OD) {                                                                        \
    activation_kernel<TS, TO><<<grid, 256, 0, stream>>>(static_cast<const TS*>(src), n_splits, total, round_sum, kind, \
                                                        static_cast<TO*>(out), total);                             \
    return yk_check_launch("activation");                                                                          \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("activation: unsupported dtype combination");
}

__global__ void scale_rows_kernel(float* __restrict__ x, float s, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    x[i] *= s;
}

extern "C" int yk_scale_rows(float* x, float s, size_t total, hipStream_t stream) {
  if (total == 0) return 0;
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 1 << 20));
  scale_rows_kernel<<<grid, 256, 0, stream>>>(x, s, total);
  return yk_check_launch("scale_rows");
}
