// Embedding gather and the SiLU-gated product.
//
// embed_gather: out[t, :] = float(table[ids[t], :]) * scale   (residual stream is 32-bit; scale 1 for most models)
//   reference counterpart: crates/cuda-kernels/csrc/misc/elementwise_basic.cu:186-211
// silu_mul:     out[t, j] = silu(gate[t, j]) * up[t, j], silu(z) = z / (1 + exp(-z))
//   reference counterpart: crates/cuda-kernels/csrc/misc/elementwise_basic.cu:18-24,34-95
// tanh_cap:     x <- cap * tanh(x / cap) in place on float32 (soft-capped logits)
#include "common.h"

namespace arle {

__global__ void tanh_cap_kernel(float* __restrict__ x, int64_t count, float cap, float inv_cap) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < count) x[i] = cap * tanhf(x[i] * inv_cap);
}

template <typename TT>
__global__ void embed_gather_kernel(const TT* __restrict__ table, const int* __restrict__ ids,
                                    float* __restrict__ out, int hidden, float scale) {
  const int t = blockIdx.x;
  const TT* src = table + static_cast<int64_t>(ids[t]) * hidden;
  float* dst = out + static_cast<int64_t>(t) * hidden;
  for (int i = threadIdx.x; i < hidden; i += blockDim.x) dst[i] = to_float(src[i]) * scale;
}

// block == 0: gate and up are two [T, width] views.  block > 0: one buffer whose columns alternate
// between `block` gate columns and the `block` matching up columns (gate is its first column).
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                int64_t in_stride, T* __restrict__ out, int width, int block, int act_code) {
  const int t = blockIdx.x;
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j >= width) return;
  const int64_t row = static_cast<int64_t>(t) * in_stride;
  const int64_t gi = block > 0 ? row + (j / block) * 2 * block + j % block : row + j;
  const float g = to_float(gate[gi]);
  const float u = to_float(block > 0 ? gate[gi + block] : up[gi]);
  const float act = gate_act(g, act_code);
  out[static_cast<int64_t>(t) * width + j] = from_float<T>(act * u);
}

// bfloat16, eight columns a thread: two 16-byte loads, one 16-byte store.  width, block (if any) and
// in_stride are multiples of 8 and the pointers 16-byte aligned (the launcher checks).
__global__ void silu_mul_bf16x8_kernel(const uint16_t* __restrict__ gate, const uint16_t* __restrict__ up,
                                       int64_t in_stride, uint16_t* __restrict__ out, int width, int block,
                                       int64_t chunks, int act_code) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (c >= chunks) return;
  const int per_row = width / 8;
  const int64_t t = c / per_row;
  const int j = static_cast<int>(c % per_row) * 8;
  const int64_t row = t * in_stride;
  const int64_t gi = block > 0 ? row + (j / block) * 2 * block + j % block : row + j;
  const uint4 g4 = *reinterpret_cast<const uint4*>(gate + gi);
  const uint4 u4 = *reinterpret_cast<const uint4*>(block > 0 ? gate + gi + block : up + gi);
  const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  uint32_t ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    ow[i] = pack_bf16x2(gate_act(g0, act_code) * u0, gate_act(g1, act_code) * u1);
  }
  *reinterpret_cast<uint4*>(out + t * width + j) = uint4{ow[0], ow[1], ow[2], ow[3]};
}

// out[i] = parts[0][i] + parts[1][i] + ..., added in that order: the sum of the float32 partial
// products that a matrix product with K split over workgroups leaves behind.
template <typename TOut>
__global__ void sum_partials_kernel(const float* __restrict__ parts, int n_parts, int64_t stride,
                                    TOut* __restrict__ out, int64_t count) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= count) return;
  float v = parts[i];
  for (int sp = 1; sp < n_parts; ++sp) v += parts[sp * stride + i];
  out[i] = from_float<TOut>(v);
}

// Four elements a thread, eight parts in flight at a time (loads without a condition: past the last part the
// last one is fetched again and not added).  count, stride % 4 == 0 and 16-byte aligned pointers.
template <typename TOut>
__global__ __launch_bounds__(256) void sum_partials_x4_kernel(const float* __restrict__ parts, int n_parts, int64_t stride,
                                                              TOut* __restrict__ out, int64_t groups) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const float* p = parts + 4 * i;
  float4 acc = {0.f, 0.f, 0.f, 0.f};
  for (int base = 0; base < n_parts; base += 8) {
    float4 e[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) e[u] = *reinterpret_cast<const float4*>(p + static_cast<int64_t>(min(base + u, n_parts - 1)) * stride);
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const bool in = base + u < n_parts;
      acc.x += in ? e[u].x : 0.f;
      acc.y += in ? e[u].y : 0.f;
      acc.z += in ? e[u].z : 0.f;
      acc.w += in ? e[u].w : 0.f;
    }
  }
  if constexpr (sizeof(TOut) == 4) {
    *reinterpret_cast<float4*>(out + 4 * i) = acc;
  } else {
    *reinterpret_cast<uint2*>(out + 4 * i) = uint2{pack_bf16x2(acc.x, acc.y), pack_bf16x2(acc.z, acc.w)};
  }
}

}  // namespace arle

using namespace arle;

extern "C" int arle_embed_gather(const void* table, int table_dtype, const int* ids, float* out,
                                 int tokens, int hidden, float scale, void* stream) {
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (table_dtype == kF32) {
    embed_gather_kernel<float><<<tokens, 256, 0, s>>>(static_cast<const float*>(table), ids, out, hidden, scale);
  } else {
    embed_gather_kernel<bf16><<<tokens, 256, 0, s>>>(static_cast<const bf16*>(table), ids, out, hidden, scale);
  }
  return launch_status();
}

// gate and up are two columns blocks of rows with a common row stride (in
// elements), so one fused [T, 2I] buffer and two separate buffers both fit.
// act: kActSilu or kActGeluTanh.
extern "C" int arle_act_mul(const void* gate, const void* up, long long in_stride, void* out,
                            int dtype, int tokens, int width, int block, int act, void* stream) {
  if (tokens == 0 || width == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (dtype == kBF16 && width % 8 == 0 && block % 8 == 0 && in_stride % 8 == 0 && aligned(gate) &&
      (block > 0 || aligned(up)) && aligned(out)) {
    const int64_t chunks = static_cast<int64_t>(tokens) * (width / 8);
    silu_mul_bf16x8_kernel<<<static_cast<unsigned>((chunks + 255) / 256), 256, 0, s>>>(
        static_cast<const uint16_t*>(gate), static_cast<const uint16_t*>(up), in_stride,
        static_cast<uint16_t*>(out), width, block, chunks, act);
    return launch_status();
  }
  dim3 grid(tokens, (width + 255) / 256);
  if (dtype == kF32) {
    silu_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate),
                                                static_cast<const float*>(up), in_stride,
                                                static_cast<float*>(out), width, block, act);
  } else {
    silu_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gate),
                                               static_cast<const bf16*>(up), in_stride,
                                               static_cast<bf16*>(out), width, block, act);
  }
  return launch_status();
}

extern "C" int arle_silu_mul(const void* gate, const void* up, long long in_stride, void* out,
                             int dtype, int tokens, int width, int block, void* stream) {
  return arle_act_mul(gate, up, in_stride, out, dtype, tokens, width, block, kActSilu, stream);
}

// parts [n_parts][count] float32 (stride elements apart) -> out [count] float32 or bfloat16.
extern "C" int arle_sum_partials(const float* parts, int n_parts, long long stride, void* out, int out_dtype,
                                 long long count, void* stream) {
  if (count == 0) return 0;
  if (n_parts < 1) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (count % 4 == 0 && stride % 4 == 0 && reinterpret_cast<uintptr_t>(parts) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(out) % 16 == 0) {
    const int64_t groups = count / 4;
    const unsigned blocks = static_cast<unsigned>((groups + 255) / 256);
    if (out_dtype == kF32)
      sum_partials_x4_kernel<float><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<float*>(out), groups);
    else
      sum_partials_x4_kernel<bf16><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<bf16*>(out), groups);
    return launch_status();
  }
  const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
  if (out_dtype == kF32)
    sum_partials_kernel<float><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<float*>(out), count);
  else
    sum_partials_kernel<bf16><<<blocks, 256, 0, s>>>(parts, n_parts, stride, static_cast<bf16*>(out), count);
  return launch_status();
}

namespace arle {

// out[t, j] = act(gate[t, j]) * x[t, j] for two views with row strides of their own; out is contiguous [T, width].
template <typename T>
__global__ void gate_mul_kernel(const T* __restrict__ gate, int64_t gate_stride, const T* __restrict__ x,
                                int64_t x_stride, T* __restrict__ out, int width, int act_code) {
  const int64_t t = blockIdx.x;
  const int j = blockIdx.y * blockDim.x + threadIdx.x;
  if (j >= width) return;
  out[t * width + j] = from_float<T>(gate_act(to_float(gate[t * gate_stride + j]), act_code) * to_float(x[t * x_stride + j]));
}

// bfloat16, eight columns a thread; width and both strides multiples of 8, pointers 16-byte aligned.
__global__ void gate_mul_bf16x8_kernel(const uint16_t* __restrict__ gate, int64_t gate_stride,
                                       const uint16_t* __restrict__ x, int64_t x_stride, uint16_t* __restrict__ out,
                                       int width, int64_t chunks, int act_code) {
  const int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (c >= chunks) return;
  const int per_row = width / 8;
  const int64_t t = c / per_row;
  const int j = static_cast<int>(c % per_row) * 8;
  const uint4 g4 = *reinterpret_cast<const uint4*>(gate + t * gate_stride + j);
  const uint4 u4 = *reinterpret_cast<const uint4*>(x + t * x_stride + j);
  const uint32_t gw[4] = {g4.x, g4.y, g4.z, g4.w}, uw[4] = {u4.x, u4.y, u4.z, u4.w};
  uint32_t ow[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    ow[i] = pack_bf16x2(gate_act(g0, act_code) * u0, gate_act(g1, act_code) * u1);
  }
  *reinterpret_cast<uint4*>(out + t * width + j) = uint4{ow[0], ow[1], ow[2], ow[3]};
}

// out[t, j] = act(z[t, j]) * table[ids[t], first + j]: a gate on a slice of a second embedding's row.
template <typename T, typename TT>
__global__ void token_gate_kernel(const T* __restrict__ z, int64_t z_stride, const TT* __restrict__ table,
                                  int64_t table_stride, int first, const int* __restrict__ ids, T* __restrict__ out,
                                  int width, int act_code) {
  const int64_t t = blockIdx.x;
  const TT* row = table + static_cast<int64_t>(ids[t]) * table_stride + first;
  for (int j = threadIdx.x; j < width; j += blockDim.x)
    out[t * width + j] = from_float<T>(gate_act(to_float(z[t * z_stride + j]), act_code) * to_float(row[j]));
}

}  // namespace arle

// gate, x: [T, width] views of `dtype` with row strides in elements; out contiguous [T, width].  act: a kAct code.
extern "C" int arle_gate_mul(const void* gate, long long gate_stride, const void* x, long long x_stride, void* out,
                             int dtype, int tokens, int width, int act, void* stream) {
  if (tokens == 0 || width == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % 16 == 0; };
  if (dtype == kBF16 && width % 8 == 0 && gate_stride % 8 == 0 && x_stride % 8 == 0 && aligned(gate) && aligned(x) &&
      aligned(out)) {
    const int64_t chunks = static_cast<int64_t>(tokens) * (width / 8);
    gate_mul_bf16x8_kernel<<<static_cast<unsigned>((chunks + 255) / 256), 256, 0, s>>>(
        static_cast<const uint16_t*>(gate), gate_stride, static_cast<const uint16_t*>(x), x_stride,
        static_cast<uint16_t*>(out), width, chunks, act);
    return launch_status();
  }
  dim3 grid(tokens, (width + 255) / 256);
  if (dtype == kF32)
    gate_mul_kernel<float><<<grid, 256, 0, s>>>(static_cast<const float*>(gate), gate_stride, static_cast<const float*>(x),
                                                x_stride, static_cast<float*>(out), width, act);
  else
    gate_mul_kernel<bf16><<<grid, 256, 0, s>>>(static_cast<const bf16*>(gate), gate_stride, static_cast<const bf16*>(x),
                                               x_stride, static_cast<bf16*>(out), width, act);
  return launch_status();
}

// z [T, width] of `dtype` (row stride in elements), table [rows, table_stride] of `table_dtype`, ids int32 [T] (checked
// by the caller to lie in the table); out contiguous [T, width] of `dtype`.
extern "C" int arle_token_gate(const void* z, long long z_stride, int dtype, const void* table, long long table_stride,
                               int table_dtype, int first, const int* ids, void* out, int tokens, int width, int act,
                               void* stream) {
  if (tokens == 0 || width == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int threads = width <= 64 ? 64 : 256;
#define ARLE_TG(T, TT)                                                                                             \
  token_gate_kernel<T, TT><<<tokens, threads, 0, s>>>(static_cast<const T*>(z), z_stride, static_cast<const TT*>(table), \
                                                      table_stride, first, ids, static_cast<T*>(out), width, act)
  if (dtype == kF32) {
    if (table_dtype == kF32) ARLE_TG(float, float); else ARLE_TG(float, bf16);
  } else {
    if (table_dtype == kF32) ARLE_TG(bf16, float); else ARLE_TG(bf16, bf16);
  }
#undef ARLE_TG
  return launch_status();
}

// x float32 [count], in place.
extern "C" int arle_tanh_cap(float* x, long long count, float cap, void* stream) {
  if (count == 0) return 0;
  if (!(cap > 0.f)) return static_cast<int>(hipErrorInvalidValue);
  const unsigned blocks = static_cast<unsigned>((count + 255) / 256);
  tanh_cap_kernel<<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(x, count, cap, 1.0f / cap);
  return launch_status();
}
