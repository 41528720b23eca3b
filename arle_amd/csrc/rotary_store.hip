// Preparation of the operands of an attention with rotary positions: per-head norms of q and k in front of or
// behind the rotation, the rotation itself in either pairing, and the write of keys and values into the pages.
//
// For every head of q and k of a row at position p (D entries, of which the first R rotate):
//   before:  x <- x / sqrt(mean(x^2) + eps) * w        (w given: one weight of D for all heads of q, one for k)
//   rotate:  the pair (u, v) = (x[i], x[i + R/2])  (halves)  or  (x[2i], x[2i + 1])  (interleaved), i < R/2,
//            becomes (u c - v s, v c + u s) with c = cos[p][i], s = sin[p][i] from float32 tables [positions, R/2]
//            (a scaling of the frequencies and a factor on both are part of the tables)
//   after:   x <- x / sqrt(mean(x^2) + eps)             (unit_after)
// q is changed in place, k goes to pages [page, nkv, slot, Dk], v as it is to pages [page, nkv, Dv, slot].
// One wave a (row, head); the head lies in LDS between the steps so that a lane finds its partner.  All of it is
// 32-bit arithmetic on the values as the projection left them.
#include "common.h"

namespace arle {

constexpr int kRotMaxD = 1024;

template <typename T>
__global__ __launch_bounds__(kWave) void rotary_qkv_store_kernel(
    T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_dtype, float eps,
    int unit_after, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int R, int interleaved,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, const int* __restrict__ block_table,
    int table_stride, T* __restrict__ k_pages, T* __restrict__ v_pages, int nq, int nkv, int Dk, int Dv,
    int page_size) {
  __shared__ float head[kRotMaxD];
  const int64_t t = blockIdx.x;
  const int y = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  if (y >= nq + nkv) {
    const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
    const int g = y - nq - nkv;
    T* dst = v_pages + (static_cast<int64_t>(page) * nkv + g) * Dv * page_size + pos % page_size;
    for (int d = lane; d < Dv; d += kWave) dst[static_cast<int64_t>(d) * page_size] = v[t * v_stride + g * Dv + d];
    return;
  }
  const bool is_q = y < nq;
  const int g = is_q ? y : y - nq;
  const T* src = is_q ? q + t * q_stride + g * Dk : k + t * k_stride + g * Dk;
  const void* weight = is_q ? q_weight : k_weight;
  float x[kRotMaxD / kWave];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < kRotMaxD / kWave; ++j) {
    const int d = lane + j * kWave;
    if (j * kWave < Dk) {
      x[j] = to_float(src[min(d, Dk - 1)]);
      if (d < Dk) ss = fmaf(x[j], x[j], ss);
    }
  }
  if (weight) {
    const float f = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dk) + eps);
#pragma unroll
    for (int j = 0; j < kRotMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < Dk) x[j] = x[j] * f * load_as_float(weight, w_dtype, min(d, Dk - 1));
    }
  }
  if (R > 0) {
#pragma unroll
    for (int j = 0; j < kRotMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < Dk && d < Dk) head[d] = x[j];
    }
    __syncthreads();
    const int half = R / 2;
    const float* c_row = cos_t + static_cast<int64_t>(pos) * half;
    const float* s_row = sin_t + static_cast<int64_t>(pos) * half;
#pragma unroll
    for (int j = 0; j < kRotMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < R && d < R) {
        const bool first = interleaved ? (d % 2 == 0) : (d < half);
        const int i = interleaved ? d / 2 : (first ? d : d - half);
        const int partner = interleaved ? (d ^ 1) : (first ? d + half : d - half);
        const float c = c_row[i], s = s_row[i], other = head[partner];
        x[j] = first ? x[j] * c - other * s : x[j] * c + other * s;
      }
    }
  }
  float f = 1.0f;
  if (unit_after) {
    ss = 0.f;
#pragma unroll
    for (int j = 0; j < kRotMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < Dk && d < Dk) ss = fmaf(x[j], x[j], ss);
    }
    f = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dk) + eps);
  }
  T* dst;
  if (is_q) {
    dst = q + t * q_stride + g * Dk;
  } else {
    const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
    dst = k_pages + ((static_cast<int64_t>(page) * nkv + g) * page_size + pos % page_size) * Dk;
  }
#pragma unroll
  for (int j = 0; j < kRotMaxD / kWave; ++j) {
    const int d = lane + j * kWave;
    if (j * kWave < Dk && d < Dk) dst[d] = from_float<T>(x[j] * f);
  }
}

}  // namespace arle

using namespace arle;

extern "C" int arle_rotary_qkv_store(void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                                     long long v_stride, int dtype, const void* q_weight, const void* k_weight,
                                     int w_dtype, float eps, int unit_after, const void* cos_t, const void* sin_t,
                                     int rotary_dim, int interleaved, const int* positions, const int* slot_of_token,
                                     const int* block_table, int table_stride, void* k_pages, void* v_pages, int tokens,
                                     int nq, int nkv, int Dk, int Dv, int page_size, void* stream) {
  if (tokens == 0) return 0;
  if (Dk > kRotMaxD || rotary_dim > Dk || rotary_dim % 2) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid(tokens, nq + 2 * nkv);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) {
    rotary_qkv_store_kernel<float><<<grid, kWave, 0, s>>>(
        static_cast<float*>(q), q_stride, static_cast<const float*>(k), k_stride, static_cast<const float*>(v), v_stride,
        q_weight, k_weight, w_dtype, eps, unit_after, static_cast<const float*>(cos_t), static_cast<const float*>(sin_t),
        rotary_dim, interleaved, positions, slot_of_token, block_table, table_stride, static_cast<float*>(k_pages),
        static_cast<float*>(v_pages), nq, nkv, Dk, Dv, page_size);
  } else {
    rotary_qkv_store_kernel<bf16><<<grid, kWave, 0, s>>>(
        static_cast<bf16*>(q), q_stride, static_cast<const bf16*>(k), k_stride, static_cast<const bf16*>(v), v_stride,
        q_weight, k_weight, w_dtype, eps, unit_after, static_cast<const float*>(cos_t), static_cast<const float*>(sin_t),
        rotary_dim, interleaved, positions, slot_of_token, block_table, table_stride, static_cast<bf16*>(k_pages),
        static_cast<bf16*>(v_pages), nq, nkv, Dk, Dv, page_size);
  }
  return launch_status();
}
