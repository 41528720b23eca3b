// A norm on a sublayer's output, added into the residual stream:
//
//   y_j   = A_j + B_j                           (up to two addends, each a sum of parts, see below)
//   res_j += m * y_j / sqrt(mean_j(y_j^2) + eps) * (w_j  or  1 + w_j)                       (RMS norm), or
//   res_j += m * ((y_j - mean(y)) / sqrt(mean_j((y_j - mean(y))^2) + eps) * w_j + b_j)        (`center`: layer norm; b optional)
//   act_j = res_j rounded to the activation type  (what the next sublayer reads; optional)
//
// m is one number of the model (1 where it has none).
//
// An addend is a float32 tensor [T, W], or parts that are added in ascending order: the float32 partial products of
// a matrix product whose K was split (part p of row t at p * part_stride + t * row_stride), or the outputs of the
// experts that a token chose, [T, n, W] with a weight per (token, part).  The sums, the statistics, the weight and
// the residual are 32-bit.  A row's arithmetic depends on nothing but the row.
#include "common.h"

namespace arle {

constexpr int kPostThreads = 256;
constexpr int kPostWaves = kPostThreads / kWave;

struct Addend {
  const float* p;         // null: no addend
  int parts;              // parts added in order (>= 1)
  long long part_stride;  // elements between parts of one row
  long long row_stride;   // elements between rows
  const float* weights;   // [T, parts] factors, or null
};

// Four consecutive entries of an addend's row: its parts added in ascending order (weighted where it has weights).
// Every load is typed and stands under no condition on data, so the parts' loads are in flight together.
template <bool VEC>
__device__ __forceinline__ float4 addend_at(const Addend& a, int64_t row, int i) {
  const float* base = a.p + row * a.row_stride + i;
  auto get = [&](int p) {
    if (VEC) return *reinterpret_cast<const float4*>(base + p * a.part_stride);
    return float4{base[p * a.part_stride], 0.f, 0.f, 0.f};
  };
  float4 sum = get(0);
  if (a.weights) {
    const float f = a.weights[row * a.parts];
    sum.x *= f; sum.y *= f; sum.z *= f; sum.w *= f;
  }
  for (int p = 1; p < a.parts; ++p) {
    const float4 v = get(p);
    if (a.weights) {
      const float f = a.weights[row * a.parts + p];
      sum.x = fmaf(f, v.x, sum.x); sum.y = fmaf(f, v.y, sum.y); sum.z = fmaf(f, v.z, sum.z); sum.w = fmaf(f, v.w, sum.w);
    } else {
      sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
    }
  }
  return sum;
}

// VEC: width a multiple of 4 and every pointer and stride 16-byte aligned; a thread takes four entries at a time.
template <typename TAct, typename TW, bool VEC>
__global__ __launch_bounds__(kPostThreads) void norm_add_kernel(float* __restrict__ residual, const Addend a,
                                                                const Addend b, const TW* __restrict__ w,
                                                                int one_plus, int center, const TW* __restrict__ bias,
                                                                float mult, TAct* __restrict__ act, int width,
                                                                float eps) {
  extern __shared__ float ys[];  // [width]
  __shared__ float lds[kPostWaves];
  const int64_t r = blockIdx.x;
  constexpr int kStep = VEC ? 4 : 1;
  float ss = 0.f, sum = 0.f;
  for (int i = kStep * threadIdx.x; i < width; i += kStep * kPostThreads) {
    float4 y = addend_at<VEC>(a, r, i);
    if (b.p) {
      const float4 z = addend_at<VEC>(b, r, i);
      y.x += z.x; y.y += z.y; y.z += z.z; y.w += z.w;
    }
    if (VEC) {
      *reinterpret_cast<float4*>(ys + i) = y;
      ss = fmaf(y.x, y.x, ss); ss = fmaf(y.y, y.y, ss); ss = fmaf(y.z, y.z, ss); ss = fmaf(y.w, y.w, ss);
      sum += (y.x + y.y) + (y.z + y.w);
    } else {
      ys[i] = y.x;
      ss = fmaf(y.x, y.x, ss);
      sum += y.x;
    }
  }
  float mean = 0.f;
  if (center) {   // the squares of the deviations from the mean, each thread over the entries it wrote itself
    mean = block_sum<kPostWaves>(sum, lds) / static_cast<float>(width);
    ss = 0.f;
    for (int i = kStep * threadIdx.x; i < width; i += kStep * kPostThreads) {
      if (VEC) {
        float4 y = *reinterpret_cast<const float4*>(ys + i);
        y.x -= mean; y.y -= mean; y.z -= mean; y.w -= mean;
        *reinterpret_cast<float4*>(ys + i) = y;
        ss = fmaf(y.x, y.x, ss); ss = fmaf(y.y, y.y, ss); ss = fmaf(y.z, y.z, ss); ss = fmaf(y.w, y.w, ss);
      } else {
        const float y = ys[i] - mean;
        ys[i] = y;
        ss = fmaf(y, y, ss);
      }
    }
  }
  const float total = block_sum<kPostWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  float* res = residual + r * width;
  const float one = one_plus ? 1.0f : 0.0f;
  const bool plain_add = mult == 1.0f && !bias;
  for (int i = kStep * threadIdx.x; i < width; i += kStep * kPostThreads) {
    if (VEC) {
      const float4 g = ld4<TW>(w + i), y = *reinterpret_cast<const float4*>(ys + i);
      const float4 c = bias ? ld4<TW>(bias + i) : float4{0.f, 0.f, 0.f, 0.f};
      float4 v = *reinterpret_cast<const float4*>(res + i);
      if (plain_add) {   // no factor and no bias: one fused multiply-add an entry, rounded once
        v.x = fmaf(y.x * inv, one + g.x, v.x); v.y = fmaf(y.y * inv, one + g.y, v.y);
        v.z = fmaf(y.z * inv, one + g.z, v.z); v.w = fmaf(y.w * inv, one + g.w, v.w);
      } else {
        v.x = fmaf(mult, fmaf(y.x * inv, one + g.x, c.x), v.x); v.y = fmaf(mult, fmaf(y.y * inv, one + g.y, c.y), v.y);
        v.z = fmaf(mult, fmaf(y.z * inv, one + g.z, c.z), v.z); v.w = fmaf(mult, fmaf(y.w * inv, one + g.w, c.w), v.w);
      }
      *reinterpret_cast<float4*>(res + i) = v;
      if (act) st4<TAct>(act + r * width + i, v);
    } else {
      const float v = plain_add ? fmaf(ys[i] * inv, one + to_float(w[i]), res[i])
                                : fmaf(mult, fmaf(ys[i] * inv, one + to_float(w[i]), bias ? to_float(bias[i]) : 0.f), res[i]);
      res[i] = v;
      if (act) act[r * width + i] = from_float<TAct>(v);
    }
  }
}

}  // namespace arle

using namespace arle;

// residual float32 [rows, width], updated in place.  Addends are float32.  act: [rows, width] of act_dtype, or null.
// center != 0: the layer norm; bias: [width] of the weight's type, or null; mult: the factor on what is added.
extern "C" int arle_norm_add(float* residual, const float* a, int a_parts, long long a_part_stride,
                             long long a_row_stride, const float* a_weights, const float* b, int b_parts,
                             long long b_part_stride, long long b_row_stride, const float* b_weights,
                             const void* w, int w_dtype, int one_plus, int center, const void* bias, float mult,
                             void* act, int act_dtype, int rows, int width, float eps, void* stream) {
  if (rows == 0) return 0;
  if (!a || a_parts < 1 || (b && b_parts < 1) || width < 1 || width > 16384) return static_cast<int>(hipErrorInvalidValue);
  const Addend A{a, a_parts, a_part_stride, a_row_stride, a_weights};
  const Addend B{b, b_parts, b_part_stride, b_row_stride, b_weights};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = static_cast<size_t>(width) * sizeof(float);
  auto al = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  const bool vec = width % 4 == 0 && al(residual) && al(a) && a_part_stride % 4 == 0 && a_row_stride % 4 == 0 &&
                   (!b || (al(b) && b_part_stride % 4 == 0 && b_row_stride % 4 == 0)) && al(w) && al(act) && al(bias);
#define ARLE_POST_V(TA, TWT, V)                                                                                \
  do {                                                                                                         \
    static bool raised = false;                                                                                \
    if (!raised && lds > 48 * 1024) {                                                                          \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&norm_add_kernel<TA, TWT, V>),    \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);         \
      if (e != hipSuccess) return static_cast<int>(e);                                                         \
      raised = true;                                                                                           \
    }                                                                                                          \
    norm_add_kernel<TA, TWT, V><<<rows, kPostThreads, lds, s>>>(residual, A, B, static_cast<const TWT*>(w),    \
                                                                one_plus, center, static_cast<const TWT*>(bias), \
                                                                mult, static_cast<TA*>(act), width, eps);      \
  } while (0)
#define ARLE_POST(TA, TWT)                     \
  do {                                         \
    if (vec) ARLE_POST_V(TA, TWT, true);       \
    else ARLE_POST_V(TA, TWT, false);          \
  } while (0)
  if (act_dtype == kF32) {
    if (w_dtype == kF32) ARLE_POST(float, float); else ARLE_POST(float, bf16);
  } else {
    if (w_dtype == kF32) ARLE_POST(bf16, float); else ARLE_POST(bf16, bf16);
  }
#undef ARLE_POST
#undef ARLE_POST_V
  return launch_status();
}
