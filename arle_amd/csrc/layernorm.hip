// Layer norm over rows (its own bias optional), with the residual adds of a parallel block fused in and one or two
// outputs from one pass.
//
//   x      = residual + (term_0 + bias_0) + (term_1 + bias_1)         (32-bit, written back)
//   mu     = mean_j x_j;   var = mean_j (x_j - mu)^2                   (two passes over registers)
//   out_a  = (x - mu) / sqrt(var + eps) * w_a + c_a;   out_b likewise with w_b, c_b (optional; c: the norm's own bias,
//            of the weight's type, optional)
//
// A block whose mixer and feed-forward both read the same residual hands on two deltas, each of which may be
// a stack of float32 partial products (added in the order of the stack) and may carry the bias of the
// projection that made it; the next block's two norms are of that same sum, so they share the statistics.
// With `rows` given (the final norm before the head) the rows named there are read for the last time and
// the sum is not written back.
#include "common.h"

namespace arle {

constexpr int kLnThreads = 256;
constexpr int kLnWaves = kLnThreads / kWave;

struct LnTerm {
  const void* data;     // [n_stack][T][width], or null
  int n_stack;
  long long stack_stride;
  int dtype;
  const void* bias;     // [width] or null
  int bias_dtype;
};

// PER elements a thread (width <= kLnThreads * PER), the row stays in registers.
template <int PER>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(
    float* __restrict__ residual, LnTerm t0, LnTerm t1, const void* __restrict__ wa, const void* __restrict__ wb,
    int w_dtype, void* __restrict__ out_a, void* __restrict__ out_b, int out_dtype, const int* __restrict__ rows,
    int width, float eps, const void* __restrict__ ca, const void* __restrict__ cb) {
  __shared__ float lds[kLnWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  float* res = residual + src * width;
  float x[PER];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    float v = 0.f;
    if (i < width) {
      v = res[i];
      if (t0.data) {
        float d = load_as_float(t0.data, t0.dtype, src * width + i);
        for (int s = 1; s < t0.n_stack; ++s) d += load_as_float(t0.data, t0.dtype, s * t0.stack_stride + src * width + i);
        if (t0.bias) d += load_as_float(t0.bias, t0.bias_dtype, i);
        v += d;
      }
      if (t1.data) {
        float d = load_as_float(t1.data, t1.dtype, src * width + i);
        for (int s = 1; s < t1.n_stack; ++s) d += load_as_float(t1.data, t1.dtype, s * t1.stack_stride + src * width + i);
        if (t1.bias) d += load_as_float(t1.bias, t1.bias_dtype, i);
        v += d;
      }
      if (!rows && (t0.data || t1.data)) res[i] = v;
    }
    x[k] = v;
    sum += v;
  }
  const float mu = block_sum<kLnWaves>(sum, lds) / static_cast<float>(width);
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    const float d = i < width ? x[k] - mu : 0.f;
    x[k] = d;
    sq += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum<kLnWaves>(sq, lds) / static_cast<float>(width) + eps);
  const int64_t o = static_cast<int64_t>(r) * width;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    if (i < width) {
      const float n = x[k] * inv;
      store_from_float(out_a, out_dtype, o + i, fmaf(n, load_as_float(wa, w_dtype, i), ca ? load_as_float(ca, w_dtype, i) : 0.f));
      if (out_b) store_from_float(out_b, out_dtype, o + i, fmaf(n, load_as_float(wb, w_dtype, i), cb ? load_as_float(cb, w_dtype, i) : 0.f));
    }
  }
}

// The same for the usual types: terms that are float32 (a projection's 32-bit output or its stack of partial
// products), biases, weights and outputs of one type TA, a width that is a multiple of 4.  Four elements a lane and
// access, every load of a row issued without a condition on data, before anything is stored.
template <typename TA, int PER4>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_vec_kernel(
    float* __restrict__ residual, const float* __restrict__ t0, int n0, long long s0, const TA* __restrict__ b0,
    const float* __restrict__ t1, int n1, long long s1, const TA* __restrict__ b1, const TA* __restrict__ wa,
    const TA* __restrict__ wb, TA* __restrict__ out_a, TA* __restrict__ out_b, const int* __restrict__ rows, int width,
    float eps, const TA* __restrict__ ca, const TA* __restrict__ cb) {
  __shared__ float lds[kLnWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  const int64_t base = src * width;
  const int last = width - 4, tid = threadIdx.x;
  float4 x[PER4];
#pragma unroll
  for (int k = 0; k < PER4; ++k) x[k] = ld4<float>(residual + base + min((tid + k * kLnThreads) * 4, last));
  auto add_term = [&](const float* t, int n, long long stride, const TA* bias) {
    float4 d[PER4];
#pragma unroll
    for (int k = 0; k < PER4; ++k) d[k] = ld4<float>(t + base + min((tid + k * kLnThreads) * 4, last));
    // the parts of a stack are fetched several at a time (eight for rows up to 4,096 wide) without a condition (a part past the last is the last one
    // again, fetched and dropped), so that their loads are in flight together; they are added in the stack's order
    constexpr int G = PER4 <= 4 ? 8 : (PER4 <= 8 ? 4 : 2);
    for (int s0 = 1; s0 < n; s0 += G) {
      float4 e[G][PER4];
#pragma unroll
      for (int j = 0; j < G; ++j) {
        const long long at = min(s0 + j, n - 1) * stride + base;
#pragma unroll
        for (int k = 0; k < PER4; ++k) e[j][k] = ld4<float>(t + at + min((tid + k * kLnThreads) * 4, last));
      }
#pragma unroll
      for (int j = 0; j < G; ++j) {
        if (s0 + j < n) {
#pragma unroll
          for (int k = 0; k < PER4; ++k) {
            d[k].x += e[j][k].x; d[k].y += e[j][k].y; d[k].z += e[j][k].z; d[k].w += e[j][k].w;
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < PER4; ++k) {
      if (bias) {
        const float4 e = ld4<TA>(bias + min((tid + k * kLnThreads) * 4, last));
        d[k].x += e.x; d[k].y += e.y; d[k].z += e.z; d[k].w += e.w;
      }
      x[k].x += d[k].x; x[k].y += d[k].y; x[k].z += d[k].z; x[k].w += d[k].w;
    }
  };
  // the norm weights are fetched now, not behind the two reductions that their use waits for
  float4 w_a[PER4], w_b[PER4], c_a[PER4], c_b[PER4];
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    w_a[k] = ld4<TA>(wa + min((tid + k * kLnThreads) * 4, last));
    w_b[k] = ld4<TA>((wb ? wb : wa) + min((tid + k * kLnThreads) * 4, last));
    // (a bias that is absent is the weight again, fetched and dropped)
    c_a[k] = ld4<TA>((ca ? ca : wa) + min((tid + k * kLnThreads) * 4, last));
    c_b[k] = ld4<TA>((cb ? cb : wa) + min((tid + k * kLnThreads) * 4, last));
    if (!ca) c_a[k] = float4{0.f, 0.f, 0.f, 0.f};
    if (!cb) c_b[k] = float4{0.f, 0.f, 0.f, 0.f};
  }
  if (t0) add_term(t0, n0, s0, b0);
  if (t1) add_term(t1, n1, s1, b1);
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    const int i = (tid + k * kLnThreads) * 4;
    if (i < width) {
      if (!rows && (t0 || t1)) st4<float>(residual + base + i, x[k]);
      sum += (x[k].x + x[k].y) + (x[k].z + x[k].w);
    }
  }
  const float mu = block_sum<kLnWaves>(sum, lds) / static_cast<float>(width);
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    const int i = (tid + k * kLnThreads) * 4;
    x[k].x -= mu; x[k].y -= mu; x[k].z -= mu; x[k].w -= mu;
    if (i < width) sq += (x[k].x * x[k].x + x[k].y * x[k].y) + (x[k].z * x[k].z + x[k].w * x[k].w);
  }
  const float inv = 1.0f / sqrtf(block_sum<kLnWaves>(sq, lds) / static_cast<float>(width) + eps);
  const int64_t o = static_cast<int64_t>(r) * width;
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    const int i = (tid + k * kLnThreads) * 4;
    if (i < width) {
      const float4 w = w_a[k], c = c_a[k];
      st4<TA>(out_a + o + i, float4{fmaf(x[k].x * inv, w.x, c.x), fmaf(x[k].y * inv, w.y, c.y), fmaf(x[k].z * inv, w.z, c.z),
                                    fmaf(x[k].w * inv, w.w, c.w)});
      if (out_b) {
        const float4 v = w_b[k], e = c_b[k];
        st4<TA>(out_b + o + i, float4{fmaf(x[k].x * inv, v.x, e.x), fmaf(x[k].y * inv, v.y, e.y), fmaf(x[k].z * inv, v.z, e.z),
                                      fmaf(x[k].w * inv, v.w, e.w)});
      }
    }
  }
}

template <typename TA>
static int launch_ln_vec(float* residual, const LnTerm& t0, const LnTerm& t1, const void* wa, const void* wb, void* out_a,
                         void* out_b, const int* rows, int n_rows, int width, float eps, const void* ca, const void* cb,
                         hipStream_t s) {
#define ARLE_LNV(PER4)                                                                                              \
  add_layernorm_vec_kernel<TA, PER4><<<n_rows, kLnThreads, 0, s>>>(                                                  \
      residual, static_cast<const float*>(t0.data), t0.n_stack, t0.stack_stride, static_cast<const TA*>(t0.bias),  \
      static_cast<const float*>(t1.data), t1.n_stack, t1.stack_stride, static_cast<const TA*>(t1.bias),            \
      static_cast<const TA*>(wa), static_cast<const TA*>(wb), static_cast<TA*>(out_a), static_cast<TA*>(out_b), rows, \
      width, eps, static_cast<const TA*>(ca), static_cast<const TA*>(cb))
  if (width <= kLnThreads * 4) {
    ARLE_LNV(1);
  } else if (width <= kLnThreads * 8) {
    ARLE_LNV(2);
  } else if (width <= kLnThreads * 16) {
    ARLE_LNV(4);
  } else if (width <= kLnThreads * 32) {
    ARLE_LNV(8);
  } else {
    ARLE_LNV(16);
  }
#undef ARLE_LNV
  return launch_status();
}

}  // namespace arle

using namespace arle;

// residual float32 [T, width] contiguous.  term*: null, [T, width] (n_stack 1) or a stack; bias*: null or [width].
// out_a, out_b (out_b and wb may be null): [n_rows, width] contiguous of out_dtype.  width <= 16384.
// norm_bias_a, norm_bias_b: the norms' own biases, [width] of the weights' type, or null.
extern "C" int arle_add_layernorm(float* residual, const void* term0, int n0, long long stride0, int dtype0,
                                  const void* bias0, int bias_dtype0, const void* term1, int n1, long long stride1,
                                  int dtype1, const void* bias1, int bias_dtype1, const void* wa, const void* wb,
                                  int w_dtype, void* out_a, void* out_b, int out_dtype, const int* rows, int n_rows,
                                  int width, float eps, const void* norm_bias_a, const void* norm_bias_b, void* stream) {
  if (n_rows == 0) return 0;
  if (width <= 0 || width > kLnThreads * 64) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const LnTerm t0{term0, n0, stride0, dtype0, bias0, bias_dtype0};
  const LnTerm t1{term1, n1, stride1, dtype1, bias1, bias_dtype1};
  // the usual case: float32 terms, everything else of the output's type, whole groups of four
  const auto fits = [&](const LnTerm& t) { return !t.data || (t.dtype == kF32 && (!t.bias || t.bias_dtype == out_dtype)); };
  if (width % 4 == 0 && fits(t0) && fits(t1) && w_dtype == out_dtype) {
    return out_dtype == kF32 ? launch_ln_vec<float>(residual, t0, t1, wa, wb, out_a, out_b, rows, n_rows, width, eps, norm_bias_a, norm_bias_b, s)
                             : launch_ln_vec<bf16>(residual, t0, t1, wa, wb, out_a, out_b, rows, n_rows, width, eps, norm_bias_a, norm_bias_b, s);
  }
#define ARLE_LN(PER)                                                                                          \
  add_layernorm_kernel<PER><<<n_rows, kLnThreads, 0, s>>>(residual, t0, t1, wa, wb, w_dtype, out_a, out_b, \
                                                          out_dtype, rows, width, eps, norm_bias_a, norm_bias_b)
  if (width <= kLnThreads * 4) {
    ARLE_LN(4);
  } else if (width <= kLnThreads * 16) {
    ARLE_LN(16);
  } else {
    ARLE_LN(64);
  }
#undef ARLE_LN
  return launch_status();
}
