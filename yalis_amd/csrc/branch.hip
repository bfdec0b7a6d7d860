// A branch's output joins the residual stream through a norm of its own:
//   residual[n, :] += branch[n, :] / sqrt(mean(branch[n, :]^2) + eps) * w'      (w' = w or 1 + w)
// and, where the engine's activations are narrower than the float32 residual, the new residual
// rounded to the activation dtype is written beside it: the next branch reads the stream itself,
// not a normed copy, so this is the only pass over the row between two branches.
//
// The branch may come as
//   * a tensor [rows, width] in the activation dtype or float32,
//   * the unreduced K slices of a product (float32 [slices, rows, width]; summed in the order of
//     the slices and, with round_sum, rounded as the product's own output would have been),
//   * and / or the rows of a mixture of experts before they are combined: float32
//     [rows * top, width], of which row n takes pair_weight * (the sum of its `top` rows, in
//     order).
// Everything is float32 arithmetic; one workgroup a row, the row parked in LDS between the
// sum of squares and the update.
#include <algorithm>

#include "common.h"

// Four consecutive elements of a row of T as floats (16-byte aligned rows of a multiple of four).
template <typename T>
__device__ __forceinline__ float4 na_load4(const T* p);
template <>
__device__ __forceinline__ float4 na_load4<float>(const float* p) {
  return *reinterpret_cast<const float4*>(p);
}
template <>
__device__ __forceinline__ float4 na_load4<bf16_t>(const bf16_t* p) {
  const uint2 w = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(w.x << 16), __uint_as_float(w.x & 0xffff0000u), __uint_as_float(w.y << 16),
                     __uint_as_float(w.y & 0xffff0000u));
}

// VEC: four columns a thread with 16-byte accesses, and the slices (or a token's expert rows) of a
// column asked for eight at a time before any is added: with one element a thread and one load
// behind the other, eight rows of 2,048 took 17 us of waiting.  The sums keep the order of the slices.
template <typename TS, typename TW, typename TO, bool VEC>
__global__ __launch_bounds__(256) void norm_add_kernel(
    float* __restrict__ residual, const TS* __restrict__ src, int n_splits, size_t split_stride, int round_sum,
    const float* __restrict__ pairs, int top, float pair_weight, const TW* __restrict__ w, int unit_offset,
    float eps, TO* __restrict__ out, int width) {
  extern __shared__ float row[];  // [width], then 17 floats of scratch
  float* scratch = row + width;
  const size_t n = blockIdx.x;
  float ss = 0.f;
  if (VEC) {
    for (int c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (src != nullptr) {
        for (int s0 = 0; s0 < n_splits; s0 += 8) {
          float4 t[8];
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (s0 + j < n_splits) t[j] = na_load4<TS>(src + (s0 + j) * split_stride + n * width + c);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (s0 + j < n_splits) {
              v.x += t[j].x; v.y += t[j].y; v.z += t[j].z; v.w += t[j].w;
            }
        }
        v.x = as_output(v.x, round_sum); v.y = as_output(v.y, round_sum);
        v.z = as_output(v.z, round_sum); v.w = as_output(v.w, round_sum);
      }
      if (pairs != nullptr) {
        float4 e = make_float4(0.f, 0.f, 0.f, 0.f);
        for (int k0 = 0; k0 < top; k0 += 8) {
          float4 t[8];
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (k0 + j < top) t[j] = *reinterpret_cast<const float4*>(pairs + (n * top + k0 + j) * width + c);
#pragma unroll
          for (int j = 0; j < 8; ++j)
            if (k0 + j < top) {
              e.x += t[j].x; e.y += t[j].y; e.z += t[j].z; e.w += t[j].w;
            }
        }
        v.x = fmaf(pair_weight, e.x, v.x); v.y = fmaf(pair_weight, e.y, v.y);
        v.z = fmaf(pair_weight, e.z, v.z); v.w = fmaf(pair_weight, e.w, v.w);
      }
      *reinterpret_cast<float4*>(row + c) = v;
      ss = fmaf(v.x, v.x, fmaf(v.y, v.y, fmaf(v.z, v.z, fmaf(v.w, v.w, ss))));
    }
  } else {
    for (int c = threadIdx.x; c < width; c += blockDim.x) {
      float v = 0.f;
      if (src != nullptr) {
        for (int s = 0; s < n_splits; ++s) v += to_f32<TS>(src[s * split_stride + n * width + c]);
        v = as_output(v, round_sum);
      }
      if (pairs != nullptr) {
        float e = 0.f;
        for (int k = 0; k < top; ++k) e += pairs[(n * top + k) * width + c];
        v = fmaf(pair_weight, e, v);
      }
      row[c] = v;
      ss = fmaf(v, v, ss);
    }
  }
  const float total = block_sum(ss, scratch);
  const float inv = 1.f / sqrtf(total / static_cast<float>(width) + eps);
  if (VEC) {
    for (int c = 4 * threadIdx.x; c < width; c += 4 * blockDim.x) {
      const float4 wv = na_load4<TW>(w + c), b = *reinterpret_cast<const float4*>(row + c);
      const float off = unit_offset ? 1.f : 0.f;
      float4 r = *reinterpret_cast<const float4*>(residual + n * width + c);
      r.x += b.x * inv * (wv.x + off); r.y += b.y * inv * (wv.y + off);
      r.z += b.z * inv * (wv.z + off); r.w += b.w * inv * (wv.w + off);
      *reinterpret_cast<float4*>(residual + n * width + c) = r;
      if (out != nullptr)
        *reinterpret_cast<uint2*>(out + n * width + c) = make_uint2(pack_bf16x2(r.x, r.y), pack_bf16x2(r.z, r.w));
    }
    return;
  }
  for (int c = threadIdx.x; c < width; c += blockDim.x) {
    const float wv = to_f32<TW>(w[c]) + (unit_offset ? 1.f : 0.f);
    const float r = residual[n * width + c] + row[c] * inv * wv;
    residual[n * width + c] = r;
    if (out != nullptr) out[n * width + c] = from_f32<TO>(r);
  }
}

// rows of a float32 stream rounded to the activation dtype (what the first branch of a model reads)
template <typename TO>
__global__ void round_rows_kernel(const float* __restrict__ x, TO* __restrict__ out, size_t total) {
  for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < total;
       i += static_cast<size_t>(gridDim.x) * blockDim.x)
    out[i] = from_f32<TO>(x[i]);
}

extern "C" int yk_round_rows(const float* x, void* out, int out_dtype, size_t total, hipStream_t stream) {
  if (total == 0) return 0;
  YK_REQUIRE(out_dtype == YK_BF16, "round_rows: the narrow dtype is bfloat16");
  const int grid = static_cast<int>(std::min<size_t>((total + 255) / 256, 65535));
  round_rows_kernel<bf16_t><<<grid, 256, 0, stream>>>(x, static_cast<bf16_t*>(out), total);
  return yk_check_launch("round_rows");
}

extern "C" int yk_norm_add(float* residual, const void* src, int src_dtype, int n_splits, int round_sum,
                           const float* pairs, int top, float pair_weight, const void* w, int w_dtype,
                           int unit_offset, float eps, void* out, int out_dtype, int n_rows, int width,
                           hipStream_t stream) {
  YK_REQUIRE(n_rows >= 0 && width > 0, "norm_add: bad sizes");
  YK_REQUIRE(src != nullptr || pairs != nullptr, "norm_add: no branch given");
  YK_REQUIRE(n_splits >= 1 && (n_splits == 1 || src_dtype == YK_F32), "norm_add: unreduced slices must be float32");
  YK_REQUIRE(pairs == nullptr || top >= 1, "norm_add: expert rows need a count per token");
  YK_REQUIRE(width <= 15 * 1024, "norm_add: rows of more than 15,360 elements do not fit the row buffer");
  YK_REQUIRE(out == nullptr || out_dtype == YK_BF16, "norm_add: the rounded copy is bfloat16");
  if (n_rows == 0) return 0;
  const size_t stride = static_cast<size_t>(n_rows) * width;
  const size_t lds = (static_cast<size_t>(width) + 17) * sizeof(float);
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = width % 4 == 0 && al(residual) && al(src) && al(pairs) && al(w) && al(out);
#define YK_CASE(SD, TS, WD, TW)                                                                            \
  if ((src == nullptr || src_dtype == SD) && w_dtype == WD) {                                                \
    if (vec)                                                                                                 \
      norm_add_kernel<TS, TW, bf16_t, true><<<n_rows, 256, lds, stream>>>(                                   \
          residual, static_cast<const TS*>(src), n_splits, stride, round_sum, pairs, top, pair_weight,       \
          static_cast<const TW*>(w), unit_offset, eps, static_cast<bf16_t*>(out), width);                    \
    else                                                                                                     \
      norm_add_kernel<TS, TW, bf16_t, false><<<n_rows, 256, lds, stream>>>(                                  \
          residual, static_cast<const TS*>(src), n_splits, stride, round_sum, pairs, top, pair_weight,       \
          static_cast<const TW*>(w), unit_offset, eps, static_cast<bf16_t*>(out), width);                    \
    return yk_check_launch("norm_add");                                                                      \
  }
  YK_CASE(YK_F32, float, YK_F32, float)
  YK_CASE(YK_F32, float, YK_BF16, bf16_t)
  YK_CASE(YK_BF16, bf16_t, YK_F32, float)
  YK_CASE(YK_BF16, bf16_t, YK_BF16, bf16_t)
#undef YK_CASE
  return yk_fail("norm_add: unsupported dtype combination");
}
