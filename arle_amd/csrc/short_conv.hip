// A short causal convolution over time on every channel of the rows of a packed step, continued across
// steps through a per-request state of the last taps-1 inputs.
//
//   y_t[c] = (ADD ? u_t[c] : 0) + sum_{j < taps} w[c][j] * u_(t - taps + 1 + j)[c],    u := input (+ bias)
//   (SILU: y <- y / (1 + exp(-y)) on the way out.  The entry point's `add_input` holds both: bit 0 ADD, bit 1 SILU.)
//
// The rows of one request are consecutive in the step; an input further back than the request's first row of
// this step comes from its state [slots][taps-1][channels] (the most recent input last), which is all zeros
// when the request starts, so inputs before position 0 count as zero without a test.  The sums are 32-bit.
// `conv_state_update` then shifts each request's state by the rows it brought.  The update is a kernel of its
// own because the convolution of a step reads the old state of every request.
#include "common.h"

namespace arle {

constexpr int kConvMaxTaps = 16;
constexpr int kConvAdd = 1, kConvSilu = 2;

__device__ __forceinline__ float conv_out(float y, int flags) { return (flags & kConvSilu) ? y / (1.0f + expf(-y)) : y; }

__global__ void causal_conv_kernel(const void* __restrict__ u, long long u_stride, int u_dtype,
                                   const void* __restrict__ bias, int bias_dtype, const void* __restrict__ w,
                                   int w_dtype, const void* __restrict__ state, int state_dtype,
                                   const int* __restrict__ slot_of_token, void* __restrict__ out,
                                   long long out_stride, int out_dtype, int channels, int taps, int add_input) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = slot_of_token[t];
  const float b = bias ? load_as_float(bias, bias_dtype, c) : 0.f;
  const float now = load_as_float(u, u_dtype, t * u_stride + c) + b;
  if (!w) {   // no convolution: the input with its bias
    store_from_float(out, out_dtype, t * out_stride + c, now);
    return;
  }
  // rows of the same request right before this one in the step (at most taps-1 matter)
  int mine = 0;
  while (mine < taps - 1 && t - mine - 1 >= 0 && slot_of_token[t - mine - 1] == slot) ++mine;
  float acc = (add_input & kConvAdd) ? now : 0.f;
  acc = fmaf(load_as_float(w, w_dtype, static_cast<int64_t>(c) * taps + taps - 1), now, acc);
  for (int back = 1; back < taps; ++back) {
    float v;
    if (back <= mine) {
      v = load_as_float(u, u_dtype, (t - back) * u_stride + c) + b;
    } else {  // state row taps-1 - (back - mine): the (back - mine)-th most recent input before the step
      const int64_t row = static_cast<int64_t>(slot) * (taps - 1) + (taps - 1 - (back - mine));
      v = load_as_float(state, state_dtype, row * channels + c);
    }
    acc = fmaf(load_as_float(w, w_dtype, static_cast<int64_t>(c) * taps + taps - 1 - back), v, acc);
  }
  store_from_float(out, out_dtype, t * out_stride + c, conv_out(acc, add_input));
}

// One element type T throughout and channels in whole groups of four: a lane takes four channels of a row with one
// access each for the input, the taps - 1 rows before it (the step's, or the state's) and the weights; none of the
// loads stands under a condition on data (which rows are the step's is the same for the whole workgroup).
template <typename T, int TAPS>
__global__ void causal_conv_vec_kernel(const T* __restrict__ u, long long u_stride, const T* __restrict__ bias,
                                       const T* __restrict__ w, const T* __restrict__ state,
                                       const int* __restrict__ slot_of_token, T* __restrict__ out, long long out_stride,
                                       int channels, int add_input) {
  const int t = blockIdx.x;
  const int c = (blockIdx.y * blockDim.x + threadIdx.x) * 4;
  if (c >= channels) return;
  const int slot = slot_of_token[t];
  int mine = 0;
  while (mine < TAPS - 1 && t - mine - 1 >= 0 && slot_of_token[t - mine - 1] == slot) ++mine;
  const float4 b = bias ? ld4<T>(bias + c) : float4{0.f, 0.f, 0.f, 0.f};
  float4 in[TAPS];     // in[back]: the input `back` rows before this one
#pragma unroll
  for (int back = 0; back < TAPS; ++back) {
    if (back <= mine) {
      const float4 v = ld4<T>(u + (t - back) * u_stride + c);
      in[back] = float4{v.x + b.x, v.y + b.y, v.z + b.z, v.w + b.w};
    } else {
      const int64_t row = static_cast<int64_t>(slot) * (TAPS - 1) + (TAPS - 1 - (back - mine));
      in[back] = ld4<T>(state + row * channels + c);
    }
  }
  float wt[4][TAPS];   // four channels' taps are 4 * TAPS consecutive elements
#pragma unroll
  for (int j = 0; j < TAPS; ++j) {
    const float4 v = ld4<T>(w + static_cast<int64_t>(c) * TAPS + 4 * j);
    const float e[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) wt[(4 * j + i) / TAPS][(4 * j + i) % TAPS] = e[i];
  }
  float acc[4];
  const float now[4] = {in[0].x, in[0].y, in[0].z, in[0].w};
#pragma unroll
  for (int i = 0; i < 4; ++i) acc[i] = fmaf(wt[i][TAPS - 1], now[i], (add_input & kConvAdd) ? now[i] : 0.f);
#pragma unroll
  for (int back = 1; back < TAPS; ++back) {
    const float v[4] = {in[back].x, in[back].y, in[back].z, in[back].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = fmaf(wt[i][TAPS - 1 - back], v[i], acc[i]);
  }
  st4<T>(out + t * out_stride + c, float4{conv_out(acc[0], add_input), conv_out(acc[1], add_input), conv_out(acc[2], add_input),
                                         conv_out(acc[3], add_input)});
}

// One thread a (segment, channel): the new state is the last taps-1 of (old state, this step's inputs).
__global__ void conv_state_update_kernel(const void* __restrict__ u, long long u_stride, int u_dtype,
                                         const void* __restrict__ bias, int bias_dtype, void* __restrict__ state,
                                         int state_dtype, const int* __restrict__ seg_row0,
                                         const int* __restrict__ seg_slot, int channels, int taps) {
  const int seg = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int row0 = seg_row0[seg], len = seg_row0[seg + 1] - row0;
  const int keep = taps - 1;
  const int64_t base = static_cast<int64_t>(seg_slot[seg]) * keep;
  const float b = bias ? load_as_float(bias, bias_dtype, c) : 0.f;
  float fresh[kConvMaxTaps];
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j) {
    if (j < keep) {
      const int at = len - keep + j;   // place among this step's rows; negative: still in the old state
      fresh[j] = at >= 0 ? load_as_float(u, u_dtype, (row0 + at) * u_stride + c) + b
                         : load_as_float(state, state_dtype, (base + j + len) * channels + c);
    }
  }
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j)
    if (j < keep) store_from_float(state, state_dtype, (base + j) * channels + c, fresh[j]);
}

}  // namespace arle

using namespace arle;

// u [T, channels] rows u_stride apart; out likewise; w [channels, taps] or null (then out = u + bias);
// state [slots, taps-1, channels]; slot_of_token int32 [T].
extern "C" int arle_causal_conv(const void* u, long long u_stride, int u_dtype, const void* bias, int bias_dtype,
                                const void* w, int w_dtype, const void* state, int state_dtype,
                                const int* slot_of_token, void* out, long long out_stride, int out_dtype, int tokens,
                                int channels, int taps, int add_input, void* stream) {
  if (tokens == 0 || channels == 0) return 0;
  if (w && (taps < 1 || taps > kConvMaxTaps)) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const auto at16 = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (w && taps >= 2 && taps <= 4 && channels % 4 == 0 && u_stride % 4 == 0 && out_stride % 4 == 0 && at16(u) && at16(out) &&
      at16(state) && u_dtype == out_dtype && w_dtype == out_dtype && state_dtype == out_dtype &&
      (!bias || bias_dtype == out_dtype)) {
    dim3 vgrid(tokens, (channels / 4 + 255) / 256);
#define ARLE_CONV(T, TAPS)                                                                                          \
  causal_conv_vec_kernel<T, TAPS><<<vgrid, 256, 0, s>>>(static_cast<const T*>(u), u_stride, static_cast<const T*>(bias), \
                                                        static_cast<const T*>(w), static_cast<const T*>(state),       \
                                                        slot_of_token, static_cast<T*>(out), out_stride, channels,    \
                                                        add_input)
    if (out_dtype == kF32) {
      if (taps == 2) ARLE_CONV(float, 2); else if (taps == 3) ARLE_CONV(float, 3); else ARLE_CONV(float, 4);
    } else {
      if (taps == 2) ARLE_CONV(bf16, 2); else if (taps == 3) ARLE_CONV(bf16, 3); else ARLE_CONV(bf16, 4);
    }
#undef ARLE_CONV
    return launch_status();
  }
  dim3 grid(tokens, (channels + 255) / 256);
  causal_conv_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      u, u_stride, u_dtype, bias, bias_dtype, w, w_dtype, state, state_dtype, slot_of_token, out, out_stride,
      out_dtype, channels, taps, add_input);
  return launch_status();
}

extern "C" int arle_conv_state_update(const void* u, long long u_stride, int u_dtype, const void* bias,
                                      int bias_dtype, void* state, int state_dtype, const int* seg_row0,
                                      const int* seg_slot, int segments, int channels, int taps, void* stream) {
  if (segments == 0 || channels == 0 || taps <= 1) return 0;
  if (taps > kConvMaxTaps) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid(segments, (channels + 255) / 256);
  conv_state_update_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      u, u_stride, u_dtype, bias, bias_dtype, state, state_dtype, seg_row0, seg_slot, channels, taps);
  return launch_status();
}
