// Operands of a latent attention: every token caches one compressed vector c (C numbers) from which all heads'
// keys and values are linear maps, and one rotated key part (R numbers) shared by the heads.  With the maps folded
// into the query and the output, the attention itself is a multi-query attention over keys [c | k_rot] of C + R
// numbers and values c:
//
//   score_h = (W_uk,h^T q_h) . c + q_rot,h . k_rot,        out_h = W_uv,h (sum_j p_j c_j)
//
// `latent_prep`: RMS norm of the first C entries of the down projection (plain weight, eps inside the root), the
// rotation of the R entries behind them and of every head's rotated query part, and the write of [c | k_rot] into
// the key pages and of c (d-major) into the value pages.  The rotation pairs entry 2i with 2i + 1 over the first
// `rot` entries (or, with `halves`, entry i with i + rot / 2), by a table of cos and sin per position; entries past
// `rot` pass unchanged.
// `head_proj`: out[t, h, :] = in[t, h, :] . Wt[h] for a matrix of its own per head, Wt[h] stored [K, N]; the sum over
// k is one chain of fused multiply-adds in ascending k for every output, whatever else the launch holds.
// Norm, angles and sums are 32-bit.
#include "common.h"

namespace arle {

constexpr int kLatentThreads = 256;

template <typename T>
__global__ __launch_bounds__(kLatentThreads) void latent_prep_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ dkv, long long dkv_stride,
    T* __restrict__ q_full, long long qf_stride, const void* __restrict__ c_weight, int w_dtype, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, const int* __restrict__ positions,
    const int* __restrict__ slot_of_token, const int* __restrict__ block_table, int table_stride,
    T* __restrict__ k_pages, T* __restrict__ v_pages, int heads, int D, int R, int C, int page_size, int halves) {
  __shared__ float lds[kLatentThreads / kWave];
  const int64_t t = blockIdx.x;
  const int pos = positions[t];
  const int half = rot / 2;
  const float* cs = cos_t + static_cast<int64_t>(pos) * half;
  const float* sn = sin_t + static_cast<int64_t>(pos) * half;
  // entry i (< rot) of a rotated vector x: x_i cos a -+ x_partner sin a, minus for the first of a pair
  auto turned = [&](const T* x, int i) {
    const int partner = halves ? (i < half ? i + half : i - half) : (i ^ 1);
    const int pair = halves ? (i < half ? i : i - half) : i / 2;
    const bool second = halves ? i >= half : (i & 1);
    const float v = to_float(x[i]), other = to_float(x[partner]), c = cs[pair], sv = sn[pair];
    return second ? fmaf(v, c, other * sv) : fmaf(v, c, -other * sv);
  };
  if (blockIdx.y == 0) {
    const T* row = dkv + t * dkv_stride;
    float ss = 0.f;
    for (int i = threadIdx.x; i < C; i += kLatentThreads) {
      const float x = to_float(row[i]);
      ss = fmaf(x, x, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum<kLatentThreads / kWave>(ss, lds) / static_cast<float>(C) + eps);
    const int64_t page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
    const int in_page = pos % page_size;
    T* krow = k_pages + (page * page_size + in_page) * (C + R);
    T* vcol = v_pages + page * C * page_size + in_page;
    for (int i = threadIdx.x; i < C; i += kLatentThreads) {
      const T c = from_float<T>(to_float(row[i]) * inv * load_as_float(c_weight, w_dtype, i));
      krow[i] = c;
      vcol[static_cast<int64_t>(i) * page_size] = c;
    }
    for (int i = threadIdx.x; i < R; i += kLatentThreads) {
      krow[C + i] = from_float<T>(i < rot ? turned(row + C, i) : to_float(row[C + i]));
    }
    return;
  }
  const int h = blockIdx.y - 1;
  const T* src = q + t * q_stride + static_cast<int64_t>(h) * (D + R) + D;
  T* dst = q_full + t * qf_stride + static_cast<int64_t>(h) * (C + R) + C;
  for (int i = threadIdx.x; i < R; i += kLatentThreads) {
    dst[i] = from_float<T>(i < rot ? turned(src, i) : to_float(src[i]));
  }
}

constexpr int kProjRows = 16;
constexpr int kProjThreads = 256;

// grid (row tiles of 16, heads, column tiles of 256).  in [T, .] with head h at h * in_head elements, K numbers; Wt
// [heads, K, N]; out [T, .] with head h at h * out_head elements, N numbers.
template <typename T>
__global__ __launch_bounds__(kProjThreads) void head_proj_kernel(const T* __restrict__ in, long long in_stride,
                                                                 int in_head, const T* __restrict__ wt,
                                                                 T* __restrict__ out, long long out_stride,
                                                                 int out_head, int rows, int K, int N) {
  extern __shared__ float xs[];  // [kProjRows][K]
  const int row0 = blockIdx.x * kProjRows, h = blockIdx.y;
  const int n = blockIdx.z * kProjThreads + threadIdx.x;
  for (int i = threadIdx.x; i < kProjRows * K; i += kProjThreads) {
    const int r = i / K, k = i % K;
    xs[i] = row0 + r < rows ? to_float(in[static_cast<int64_t>(row0 + r) * in_stride + static_cast<int64_t>(h) * in_head + k]) : 0.f;
  }
  __syncthreads();
  if (n >= N) return;
  float acc[kProjRows];
#pragma unroll
  for (int r = 0; r < kProjRows; ++r) acc[r] = 0.f;
  const T* w = wt + static_cast<int64_t>(h) * K * N + n;
  for (int k = 0; k < K; ++k) {
    const float wv = to_float(w[static_cast<int64_t>(k) * N]);
#pragma unroll
    for (int r = 0; r < kProjRows; ++r) acc[r] = fmaf(xs[r * K + k], wv, acc[r]);
  }
#pragma unroll
  for (int r = 0; r < kProjRows; ++r)
    if (row0 + r < rows)
      out[static_cast<int64_t>(row0 + r) * out_stride + static_cast<int64_t>(h) * out_head + n] = from_float<T>(acc[r]);
}

// ---- matrix-core form (bfloat16) -----------------------------------------------------------------
// The same product with every head's matrix stored [N, K] (K-major), so that both operands of
// `v_mfma_f32_16x16x32_bf16` are sixteen consecutive bytes a lane, straight from memory: a head's matrix is a few
// dozen kilobytes and stays in the caches.  A wave takes sixteen rows and sixty-four columns of one head; the four
// waves of a workgroup take sixty-four rows.  K a multiple of 8, heads' offsets multiples of 8, rows 16-byte aligned.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void head_proj_mfma_kernel(const bf16* __restrict__ in, long long in_stride, int in_head,
                                                             const bf16* __restrict__ wnk, bf16* __restrict__ out,
                                                             long long out_stride, int out_head, int rows, int K, int N) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n = lane % 16, g = lane / 16;
  const int h = blockIdx.y, n0 = blockIdx.z * 64;
  const int row0 = blockIdx.x * 64 + wave * 16;
  if (row0 >= rows) return;
  const bf16* arow = in + static_cast<int64_t>(min(row0 + n, rows - 1)) * in_stride + static_cast<int64_t>(h) * in_head;
  const bf16* wh = wnk + static_cast<int64_t>(h) * N * K;
  const bf16* wrow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) wrow[j] = wh + static_cast<int64_t>(min(n0 + 16 * j + n, N - 1)) * K;
  f32x4_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const u32x4_t zero = {0, 0, 0, 0};
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int k = min(k0 + 8 * g, K - 8);      // a piece past K is the last piece again, and zeroed
    const bool in_k = k0 + 8 * g < K;
    const u32x4_t a_raw = *reinterpret_cast<const u32x4_t*>(arow + k);
    u32x4_t b_raw[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) b_raw[j] = *reinterpret_cast<const u32x4_t*>(wrow[j] + k);
    const bf16x8_t a_op = __builtin_bit_cast(bf16x8_t, in_k ? a_raw : zero);
#pragma unroll
    for (int j = 0; j < 4; ++j)
      acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, __builtin_bit_cast(bf16x8_t, b_raw[j]), acc[j], 0, 0, 0);
  }
  // acc[j][i]: row 4 g + i of the wave's sixteen, column 16 j + n of the tile
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + 4 * g + i;
    if (r >= rows) continue;
    bf16* orow = out + static_cast<int64_t>(r) * out_stride + static_cast<int64_t>(h) * out_head;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int col = n0 + 16 * j + n;
      if (col < N) orow[col] = from_float<bf16>(acc[j][i]);
    }
  }
}

}  // namespace arle

using namespace arle;

// bfloat16; wnk [heads, N, K].
extern "C" int arle_head_proj_mfma(const void* in, long long in_stride, int in_head, const void* wnk, void* out,
                                   long long out_stride, int out_head, int rows, int heads, int K, int N, void* stream) {
  if (rows == 0) return 0;
  if (heads < 1 || heads > 65535 || K < 8 || K % 8 || in_head % 8 || in_stride % 8 || N < 1 || (N + 63) / 64 > 65535 ||
      reinterpret_cast<uintptr_t>(in) % 16 || reinterpret_cast<uintptr_t>(wnk) % 16)
    return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid((rows + 63) / 64, heads, (N + 63) / 64);
  head_proj_mfma_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      static_cast<const bf16*>(in), in_stride, in_head, static_cast<const bf16*>(wnk), static_cast<bf16*>(out), out_stride,
      out_head, rows, K, N);
  return launch_status();
}

// q [T, heads*(D+R)], dkv [T, C+R] and q_full [T, heads*(C+R)] of `dtype`, as the pages: k_pages
// [pages, 1, page_size, C+R], v_pages [pages, 1, C, page_size].  cos, sin: float32 [positions, rot/2].
extern "C" int arle_latent_prep(const void* q, long long q_stride, const void* dkv, long long dkv_stride, void* q_full,
                                long long qf_stride, int dtype, const void* c_weight, int w_dtype, float eps,
                                const float* cos_t, const float* sin_t, int rot, const int* positions,
                                const int* slot_of_token, const int* block_table, int table_stride, void* k_pages,
                                void* v_pages, int tokens, int heads, int D, int R, int C, int page_size, int halves,
                                void* stream) {
  if (tokens == 0) return 0;
  if (heads < 1 || heads > 65534 || D < 1 || R < 0 || C < 1 || rot < 0 || rot > R || rot % 2 || page_size < 1 ||
      (rot > 0 && (!cos_t || !sin_t)))
    return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(tokens, 1 + heads);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) {
    latent_prep_kernel<float><<<grid, kLatentThreads, 0, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<const float*>(dkv), dkv_stride, static_cast<float*>(q_full),
        qf_stride, c_weight, w_dtype, eps, cos_t, sin_t, rot, positions, slot_of_token, block_table, table_stride,
        static_cast<float*>(k_pages), static_cast<float*>(v_pages), heads, D, R, C, page_size, halves);
  } else {
    latent_prep_kernel<bf16><<<grid, kLatentThreads, 0, s>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<const bf16*>(dkv), dkv_stride, static_cast<bf16*>(q_full),
        qf_stride, c_weight, w_dtype, eps, cos_t, sin_t, rot, positions, slot_of_token, block_table, table_stride,
        static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), heads, D, R, C, page_size, halves);
  }
  return launch_status();
}

extern "C" int arle_head_proj(const void* in, long long in_stride, int in_head, const void* wt, void* out,
                              long long out_stride, int out_head, int dtype, int rows, int heads, int K, int N,
                              void* stream) {
  if (rows == 0) return 0;
  if (heads < 1 || heads > 65535 || K < 1 || K > 1024 || N < 1) return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid((rows + kProjRows - 1) / kProjRows, heads, (N + kProjThreads - 1) / kProjThreads);
  const size_t lds = static_cast<size_t>(kProjRows) * K * sizeof(float);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ARLE_PROJ(TT)                                                                                              \
  do {                                                                                                             \
    static bool raised = false;                                                                                    \
    if (!raised && lds > 48 * 1024) {                                                                              \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&head_proj_kernel<TT>),               \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, kProjRows * 1024 * 4);  \
      if (e != hipSuccess) return static_cast<int>(e);                                                             \
      raised = true;                                                                                               \
    }                                                                                                              \
    head_proj_kernel<TT><<<grid, kProjThreads, lds, s>>>(static_cast<const TT*>(in), in_stride, in_head,           \
                                                         static_cast<const TT*>(wt), static_cast<TT*>(out),        \
                                                         out_stride, out_head, rows, K, N);                        \
  } while (0)
  if (dtype == kF32) ARLE_PROJ(float); else ARLE_PROJ(bf16);
#undef ARLE_PROJ
  return launch_status();
}
