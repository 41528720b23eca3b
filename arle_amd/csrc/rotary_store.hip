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
// `rotary_qkv_store_kernel`: one wave a (row, head); the head lies in LDS between the steps so that a lane finds its
// partner.  `rotary_qkv_store_x8_kernel` (bfloat16, head sizes that are multiples of 8, at most 512, and for the
// halves pairing R / 2 a multiple of 8): a lane takes eight consecutive entries by one 16-byte access, the 1 to 64
// lanes of a head add their squares by lane exchanges, a partner of the halves pairing is eight entries of another
// lane, one of the interleaved pairing lies in the lane itself; a wave is then several heads, and a row of a model
// of ordinary widths a dozen waves where the first kernel takes half a hundred, each a chain of dependent loads.
// All of it is 32-bit arithmetic on the values as the projection left them, the same for a row wherever it stands.
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

// LPH: lanes of a head (a power of two, 8 LPH >= Dk).  A row's lanes: (nq + nkv) LPH for q and k, then Dv / 8 for
// every head of v.
template <int LPH>
__global__ __launch_bounds__(256) void rotary_qkv_store_x8_kernel(
    bf16* __restrict__ q, long long q_stride, const bf16* __restrict__ k, long long k_stride, const bf16* __restrict__ v,
    long long v_stride, const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_dtype, float eps,
    int unit_after, const float* __restrict__ cos_t, const float* __restrict__ sin_t, int R, int interleaved,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, const int* __restrict__ block_table,
    int table_stride, bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int nq, int nkv, int Dk, int Dv,
    int page_size) {
  const int64_t t = blockIdx.x;
  const int idx = blockIdx.y * 256 + threadIdx.x, lane = threadIdx.x % kWave;
  const int qk_lanes = (nq + nkv) * LPH, qk_padded = (qk_lanes + kWave - 1) / kWave * kWave, v_units = Dv / 8;
  const int pos = positions[t];
  const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
  if (idx >= qk_padded) {   // whole waves: the values' lanes begin with a wave
    const int e = idx - qk_padded;
    if (e >= nkv * v_units) return;
    const int g = e / v_units, u = e % v_units;
    const uint4 raw = *reinterpret_cast<const uint4*>(v + t * v_stride + g * Dv + 8 * u);
    uint16_t* dst = reinterpret_cast<uint16_t*>(v_pages) +
                    ((static_cast<int64_t>(page) * nkv + g) * Dv + 8 * u) * page_size + pos % page_size;
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 8; ++i) dst[static_cast<int64_t>(i) * page_size] = static_cast<uint16_t>(w[i / 2] >> (16 * (i % 2)));
    return;
  }
  // lanes behind the last head of k fill its wave: they exchange with the others and load and store nothing of their own
  const int y = min(idx / LPH, nq + nkv - 1), u = idx % LPH;
  const bool is_q = y < nq, live = idx < qk_lanes && 8 * u < Dk;
  const int g = is_q ? y : y - nq;
  const bf16* src = is_q ? q + t * q_stride + g * Dk : k + t * k_stride + g * Dk;
  const void* weight = is_q ? q_weight : k_weight;
  float x[8];
  {
    const uint4 raw = *reinterpret_cast<const uint4*>(src + (live ? 8 * u : 0));
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      x[2 * i] = live ? __uint_as_float(w[i] << 16) : 0.f;
      x[2 * i + 1] = live ? __uint_as_float(w[i] & 0xffff0000u) : 0.f;
    }
  }
  auto head_sum_sq = [&]() {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) ss = fmaf(x[i], x[i], ss);
#pragma unroll
    for (int off = LPH / 2; off > 0; off >>= 1) ss += __shfl_xor(ss, off, kWave);
    return ss;
  };
  if (weight) {
    const float f = 1.0f / sqrtf(head_sum_sq() / static_cast<float>(Dk) + eps);
#pragma unroll
    for (int i = 0; i < 8; ++i) x[i] = x[i] * f * load_as_float(weight, w_dtype, live ? 8 * u + i : 0);
  }
  if (R > 0) {
    const int half = R / 2;
    const float* c_row = cos_t + static_cast<int64_t>(pos) * half;
    const float* s_row = sin_t + static_cast<int64_t>(pos) * half;
    if (interleaved) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int e = 4 * u + i;   // the pair's number
        if (e < half) {
          const float c = c_row[e], s = s_row[e], a = x[2 * i], b = x[2 * i + 1];
          x[2 * i] = a * c - b * s;
          x[2 * i + 1] = b * c + a * s;
        }
      }
    } else {
      const int hu = half / 8;   // lanes of a half
      const bool first = u < hu, turns = u < 2 * hu;
      const int partner = turns ? (first ? lane + hu : lane - hu) : lane;
      float other[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) other[i] = __shfl(x[i], partner, kWave);
      if (turns) {
        const int e0 = 8 * (first ? u : u - hu);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float c = c_row[e0 + i], s = s_row[e0 + i];
          x[i] = first ? x[i] * c - other[i] * s : x[i] * c + other[i] * s;
        }
      }
    }
  }
  float f = 1.0f;
  if (unit_after) f = 1.0f / sqrtf(head_sum_sq() / static_cast<float>(Dk) + eps);
  if (!live) return;
  bf16* dst = is_q ? q + t * q_stride + g * Dk + 8 * u
                   : k_pages + ((static_cast<int64_t>(page) * nkv + g) * page_size + pos % page_size) * Dk + 8 * u;
  uint4 raw;
  raw.x = pack_bf16x2(x[0] * f, x[1] * f);
  raw.y = pack_bf16x2(x[2] * f, x[3] * f);
  raw.z = pack_bf16x2(x[4] * f, x[5] * f);
  raw.w = pack_bf16x2(x[6] * f, x[7] * f);
  *reinterpret_cast<uint4*>(dst) = raw;
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
  hipStream_t s = static_cast<hipStream_t>(stream);
  const auto aligned = [](const void* p, long long stride) { return reinterpret_cast<uintptr_t>(p) % 16 == 0 && stride % 8 == 0; };
  if (dtype != kF32 && Dk % 8 == 0 && Dk <= 512 && Dv % 8 == 0 && (interleaved || rotary_dim % 16 == 0) &&
      aligned(q, q_stride) && aligned(k, k_stride) && aligned(v, v_stride) && aligned(k_pages, 8)) {
    int lph = 1;
    while (8 * lph < Dk) lph *= 2;
    // a head's lanes lie in one wave (lph divides 64); the values' lanes start at the next multiple of 64
    const int lanes = ((nq + nkv) * lph + 63) / 64 * 64 + nkv * (Dv / 8);
    if ((lanes + 255) / 256 <= 65535) {
      const dim3 grid(tokens, (lanes + 255) / 256);
#define ARLE_ROT_X8(LPH)                                                                                             \
  rotary_qkv_store_x8_kernel<LPH><<<grid, 256, 0, s>>>(                                                              \
      static_cast<bf16*>(q), q_stride, static_cast<const bf16*>(k), k_stride, static_cast<const bf16*>(v), v_stride, \
      q_weight, k_weight, w_dtype, eps, unit_after, static_cast<const float*>(cos_t),                                \
      static_cast<const float*>(sin_t), rotary_dim, interleaved, positions, slot_of_token, block_table,              \
      table_stride, static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), nq, nkv, Dk, Dv, page_size)
      switch (lph) {
        case 1: ARLE_ROT_X8(1); break;
        case 2: ARLE_ROT_X8(2); break;
        case 4: ARLE_ROT_X8(4); break;
        case 8: ARLE_ROT_X8(8); break;
        case 16: ARLE_ROT_X8(16); break;
        case 32: ARLE_ROT_X8(32); break;
        default: ARLE_ROT_X8(64); break;
      }
#undef ARLE_ROT_X8
      return launch_status();
    }
  }
  dim3 grid(tokens, nq + 2 * nkv);
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
