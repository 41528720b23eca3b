// Residual streams with learned connections (hyper-connections), and the norm-and-average of two mixers that
// run side by side.
//
// `hyper_step`: instead of one residual a token has S streams x_1..x_S, float32 [T, S, W].  A sublayer with the
// connection (a[S], b[S], M[S, S]) reads  N(sum_s a_s x_s)  and its output y is written as
//     x_t <- sum_s M[s, t] x_s + b_t y        (all streams at once from the old ones).
// One launch does the write of the sublayer before and the read of the next one, a workgroup a token (256 threads
// where the step has rows enough to fill the chip, else up to 1,024, so that a decoded row's columns are loaded in one
// round instead of several that wait for each other):
//     x' = write(x, y; M, b)   (y null: x' = x);   u = sum_t a_t x'_t   (a null: the plain sum);
//     out = u / sqrt(mean(u^2) + eps) * w   in the activation type.
// The input streams may be one row for all streams (stream stride 0: every stream starts as a copy of the
// embedding's output).  With `rows` only those tokens are read and nothing is written (the norm in front of the
// output head).  y is a tensor [T, W] of type TY or a float32 stack [P, T, W] of partial sums, added in order.
// Every sum runs in a fixed order (streams ascending), so a token's result does not depend on its neighbours.
//
// `pair_norm`: out = coef * (a / rms(a) * wa + b / rms(b) * wb), float32, a and b tensors or float32 stacks.
#include "common.h"

namespace arle {

constexpr int kHyThreads = 256;

template <typename TY, int VEC>
__device__ __forceinline__ void load_y(const TY* y, int parts, int64_t part_stride, int64_t at, float (&v)[VEC]) {
  if constexpr (VEC == 4) {
    float4 s = ld4<TY>(y + at);
    for (int p = 1; p < parts; ++p) {
      const float4 n = ld4<TY>(y + p * part_stride + at);
      s = float4{s.x + n.x, s.y + n.y, s.z + n.z, s.w + n.w};
    }
    v[0] = s.x;
    if (VEC > 1) { v[1 % VEC] = s.y; v[2 % VEC] = s.z; v[3 % VEC] = s.w; }
  } else {
    float s = to_float(y[at]);
    for (int p = 1; p < parts; ++p) s += to_float(y[p * part_stride + at]);
    v[0] = s;
  }
}

template <typename TY, typename TA, int SMAX, int VEC, int THREADS>
__global__ __launch_bounds__(THREADS) void hyper_step_kernel(
    const float* x_in, long long in_row_stride, long long in_stream_stride, float* x_out,   // may be the same memory
    const TY* __restrict__ y, long long y_stride, int y_parts, long long y_part_stride, const float* __restrict__ mix,
    const float* __restrict__ out_w, const float* __restrict__ in_w, const float* __restrict__ norm_w, float eps,
    const int* __restrict__ rows, TA* __restrict__ out, long long out_stride, int S, int W) {
  extern __shared__ float u_lds[];      // [W] and the reduction's scratch behind it
  float* red = u_lds + W;
  const int64_t t = rows ? rows[blockIdx.x] : blockIdx.x;
  const float* src = x_in + t * in_row_stride;
  float* dst = (x_out && !rows) ? x_out + t * static_cast<int64_t>(S) * W : nullptr;
  float ss = 0.f;
  for (int c = threadIdx.x * VEC; c < W; c += THREADS * VEC) {
    float x[SMAX][VEC];
#pragma unroll
    for (int s = 0; s < SMAX; ++s) {
      if (s < S) {
        if constexpr (VEC == 4) {
          const float4 v = *reinterpret_cast<const float4*>(src + s * in_stream_stride + c);
          x[s][0] = v.x; x[s][1 % VEC] = v.y; x[s][2 % VEC] = v.z; x[s][3 % VEC] = v.w;
        } else {
          x[s][0] = src[s * in_stream_stride + c];
        }
      }
    }
    float u[VEC];
#pragma unroll
    for (int e = 0; e < VEC; ++e) u[e] = 0.f;
    if (y) {
      float yv[VEC];
      load_y<TY, VEC>(y, y_parts, y_part_stride, t * y_stride + c, yv);
#pragma unroll
      for (int to = 0; to < SMAX; ++to) {
        if (to < S) {
          float n[VEC];
#pragma unroll
          for (int e = 0; e < VEC; ++e) n[e] = mix[to] * x[0][e];
#pragma unroll
          for (int s = 1; s < SMAX; ++s) {
            if (s < S) {
              const float m = mix[s * S + to];
#pragma unroll
              for (int e = 0; e < VEC; ++e) n[e] = fmaf(m, x[s][e], n[e]);
            }
          }
          const float b = out_w[to], a = in_w ? in_w[to] : 1.0f;
#pragma unroll
          for (int e = 0; e < VEC; ++e) {
            n[e] = fmaf(b, yv[e], n[e]);
            u[e] = fmaf(a, n[e], u[e]);
          }
          if (dst) {
            if constexpr (VEC == 4) {
              *reinterpret_cast<float4*>(dst + static_cast<int64_t>(to) * W + c) = float4{n[0], n[1 % VEC], n[2 % VEC], n[3 % VEC]};
            } else {
              dst[static_cast<int64_t>(to) * W + c] = n[0];
            }
          }
        }
      }
    } else {
#pragma unroll
      for (int s = 0; s < SMAX; ++s) {
        if (s < S) {
          const float a = in_w ? in_w[s] : 1.0f;
#pragma unroll
          for (int e = 0; e < VEC; ++e) u[e] = fmaf(a, x[s][e], u[e]);
          if (dst && dst + static_cast<int64_t>(s) * W != src + s * in_stream_stride) {
            if constexpr (VEC == 4) {
              *reinterpret_cast<float4*>(dst + static_cast<int64_t>(s) * W + c) = float4{x[s][0], x[s][1 % VEC], x[s][2 % VEC], x[s][3 % VEC]};
            } else {
              dst[static_cast<int64_t>(s) * W + c] = x[s][0];
            }
          }
        }
      }
    }
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      u_lds[c + e] = u[e];
      ss = fmaf(u[e], u[e], ss);
    }
  }
  const float inv = 1.0f / sqrtf(block_sum<THREADS / kWave>(ss, red) / static_cast<float>(W) + eps);
  TA* o = out + static_cast<int64_t>(blockIdx.x) * out_stride;
  for (int c = threadIdx.x * VEC; c < W; c += THREADS * VEC) {
    if constexpr (VEC == 4) {
      const float4 w = *reinterpret_cast<const float4*>(norm_w + c);
      st4<TA>(o + c, float4{u_lds[c] * inv * w.x, u_lds[c + 1] * inv * w.y, u_lds[c + 2] * inv * w.z, u_lds[c + 3] * inv * w.w});
    } else {
      o[c] = from_float<TA>(u_lds[c] * inv * norm_w[c]);
    }
  }
}

// One workgroup a token; a and b are read twice (the second time from the caches).
template <typename TY, int VEC>
__global__ __launch_bounds__(kHyThreads) void pair_norm_kernel(
    const TY* __restrict__ a, long long a_stride, int a_parts, long long a_part_stride, const TY* __restrict__ b,
    long long b_stride, int b_parts, long long b_part_stride, const float* __restrict__ wa,
    const float* __restrict__ wb, float eps, float coef, float* __restrict__ out, int W) {
  __shared__ float red[kHyThreads / kWave];
  const int64_t t = blockIdx.x;
  float sa = 0.f, sb = 0.f;
  for (int c = threadIdx.x * VEC; c < W; c += kHyThreads * VEC) {
    float va[VEC], vb[VEC];
    load_y<TY, VEC>(a, a_parts, a_part_stride, t * a_stride + c, va);
    load_y<TY, VEC>(b, b_parts, b_part_stride, t * b_stride + c, vb);
#pragma unroll
    for (int e = 0; e < VEC; ++e) {
      sa = fmaf(va[e], va[e], sa);
      sb = fmaf(vb[e], vb[e], sb);
    }
  }
  const float ia = 1.0f / sqrtf(block_sum<kHyThreads / kWave>(sa, red) / static_cast<float>(W) + eps);
  const float ib = 1.0f / sqrtf(block_sum<kHyThreads / kWave>(sb, red) / static_cast<float>(W) + eps);
  for (int c = threadIdx.x * VEC; c < W; c += kHyThreads * VEC) {
    float va[VEC], vb[VEC];
    load_y<TY, VEC>(a, a_parts, a_part_stride, t * a_stride + c, va);
    load_y<TY, VEC>(b, b_parts, b_part_stride, t * b_stride + c, vb);
#pragma unroll
    for (int e = 0; e < VEC; ++e) out[t * W + c + e] = coef * (va[e] * ia * wa[c + e] + vb[e] * ib * wb[c + e]);
  }
}

template <typename TY, typename TA, int VEC>
int launch_hyper(const float* x_in, long long in_row_stride, long long in_stream_stride, float* x_out, const void* y,
                 long long y_stride, int y_parts, long long y_part_stride, const float* mix, const float* out_w,
                 const float* in_w, const float* norm_w, float eps, const int* rows, void* out, long long out_stride,
                 int grid, int S, int W, hipStream_t s) {
  const size_t lds = (static_cast<size_t>(W) + 1024 / kWave) * sizeof(float);
  // few rows: as many threads a row as its columns ask for, up to 1,024 (S <= 4 only: more streams are more registers)
  // (bfloat16 steps only: in float32 a row's sums run in one order whatever else the step holds)
  const bool wide = sizeof(TA) == 2 && grid < 512 && S <= 4 && W > kHyThreads * VEC;
#define ARLE_HYPER_T(SMAX, THREADS)                                                                                  \
  hyper_step_kernel<TY, TA, SMAX, VEC, THREADS><<<grid, THREADS, lds, s>>>(                                          \
      x_in, in_row_stride, in_stream_stride, x_out, static_cast<const TY*>(y), y_stride, y_parts, y_part_stride, mix, \
      out_w, in_w, norm_w, eps, rows, static_cast<TA*>(out), out_stride, S, W)
#define ARLE_HYPER(SMAX)                                                                                             \
  do {                                                                                                               \
    if (wide && SMAX <= 4) ARLE_HYPER_T(SMAX <= 4 ? SMAX : 4, 1024); else ARLE_HYPER_T(SMAX, kHyThreads);            \
  } while (0)
  if (S <= 2) ARLE_HYPER(2); else if (S <= 4) ARLE_HYPER(4); else if (S <= 8) ARLE_HYPER(8); else ARLE_HYPER(16);
#undef ARLE_HYPER_T
#undef ARLE_HYPER
  return launch_status();
}

}  // namespace arle

using namespace arle;

// x_in float32 streams (row and stream strides in elements; stream stride 0: one row for every stream); x_out float32
// [T, S, W] or null; y null, a [T, W] tensor of y_dtype, or (y_parts > 1, float32) a stack; mix [S, S], out_w [S],
// in_w [S] or null, norm_w [W], all float32; rows int32 [grid] or null; out [grid, W] of out_dtype.
extern "C" int arle_hyper_step(const void* x_in, long long in_row_stride, long long in_stream_stride, void* x_out,
                               const void* y, int y_dtype, long long y_stride, int y_parts, long long y_part_stride,
                               const void* mix, const void* out_w, const void* in_w, const void* norm_w, float eps,
                               const int* rows, void* out, int out_dtype, long long out_stride, int grid, int S, int W,
                               int vec, void* stream) {
  if (grid == 0 || W == 0) return 0;
  if (S < 1 || S > 16 || W > 16000 || (y_parts > 1 && y_dtype != kF32)) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float* xi = static_cast<const float*>(x_in);
  float* xo = static_cast<float*>(x_out);
  const float *m = static_cast<const float*>(mix), *ow = static_cast<const float*>(out_w),
              *iw = static_cast<const float*>(in_w), *nw = static_cast<const float*>(norm_w);
#define ARLE_GO(TY, TA, VEC)                                                                                        \
  return launch_hyper<TY, TA, VEC>(xi, in_row_stride, in_stream_stride, xo, y, y_stride, y_parts, y_part_stride, m, \
                                   ow, iw, nw, eps, rows, out, out_stride, grid, S, W, s)
  const bool yf = !y || y_dtype == kF32;
  if (vec) {
    if (yf && out_dtype == kF32) ARLE_GO(float, float, 4);
    if (yf) ARLE_GO(float, bf16, 4);
    if (out_dtype == kF32) ARLE_GO(bf16, float, 4);
    ARLE_GO(bf16, bf16, 4);
  }
  if (yf && out_dtype == kF32) ARLE_GO(float, float, 1);
  if (yf) ARLE_GO(float, bf16, 1);
  if (out_dtype == kF32) ARLE_GO(bf16, float, 1);
  ARLE_GO(bf16, bf16, 1);
#undef ARLE_GO
}

extern "C" int arle_pair_norm(const void* a, long long a_stride, int a_parts, long long a_part_stride, const void* b,
                              long long b_stride, int b_parts, long long b_part_stride, int dtype, const void* wa,
                              const void* wb, float eps, float coef, void* out, int tokens, int W, int vec,
                              void* stream) {
  if (tokens == 0 || W == 0) return 0;
  if ((a_parts > 1 || b_parts > 1) && dtype != kF32) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ARLE_PAIR(TY, VEC)                                                                                         \
  pair_norm_kernel<TY, VEC><<<tokens, kHyThreads, 0, s>>>(                                                         \
      static_cast<const TY*>(a), a_stride, a_parts, a_part_stride, static_cast<const TY*>(b), b_stride, b_parts,   \
      b_part_stride, static_cast<const float*>(wa), static_cast<const float*>(wb), eps, coef, static_cast<float*>(out), W)
  if (dtype == kF32) {
    if (vec) ARLE_PAIR(float, 4); else ARLE_PAIR(float, 1);
  } else {
    if (vec) ARLE_PAIR(bf16, 4); else ARLE_PAIR(bf16, 1);
  }
#undef ARLE_PAIR
  return launch_status();
}
