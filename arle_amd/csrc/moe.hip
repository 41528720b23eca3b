// A mixture of experts: the router, and the experts' products over the tokens that chose them.
//
//   z = W_r h (32-bit sums),  s = sigmoid(z) or softmax(z) over all router outputs;  the `top` experts with the largest
//   s + correction are chosen (ties: the lower index), where the experts form `groups` equal groups of neighbours among
//   the `keep` groups with the largest such number in them only (the others count as minus infinity);  weight of a
//   chosen expert = s / (sum of the chosen s + 1e-20) * scale, or without the division s * scale.
//   expert e: down_e (silu(gate_e h) * (up_e h)).  Router outputs past the experts that have tensors stand for experts
//   that hand back their input (`moe_identity` writes their rows).
//
// `moe_route`: one workgroup a token.  `moe_expert`: a workgroup takes one expert, 64 consecutive rows of the step and 64
// output columns; it lists the rows of its 64 that chose the expert (in row order) and multiplies only those, so no
// step sorts anything and a launch's shape follows the number of rows alone.  The result of (token t, its k-th
// choice) lies at row t * top + k: the gate|up pass leaves the activation there, the down pass the expert's output,
// which the consumer weighs and adds in the order of k.  Every output is summed in one fixed order over K (chains
// of 16, added in ascending order), whatever else the step holds.  bfloat16 runs the matrix-core form further down.
#include "common.h"

namespace arle {

constexpr int kMaxExpertsPerLane = 16;   // experts <= 64 * 16

struct Best {
  float v;
  int i;
};

__device__ __forceinline__ Best wave_best(Best b) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ov = __shfl_xor(b.v, off, kWave);
    const int oi = __shfl_xor(b.i, off, kWave);
    if (ov > b.v || (ov == b.v && oi < b.i)) {
      b.v = ov;
      b.i = oi;
    }
  }
  return b;
}

constexpr int kRouteThreads = 256;

// One workgroup a token: the row goes to LDS as floats once; wave w computes the logits of experts w, w + 4, ...
// (eight consecutive entries a lane and step where the width allows, one otherwise: an order that depends on the
// width alone); then the first wave picks the `top` experts one after the other.
struct RouteRule {
  int softmax;     // 0: s = sigmoid(z); 1: s = softmax(z)
  int groups;      // equal groups of neighbouring experts (1: no groups)
  int keep;        // groups among which the choice is made
  int normalize;   // 1: the chosen scores are divided by their sum
  float scale;
};

template <typename T, typename TW, bool VEC>
__global__ __launch_bounds__(kRouteThreads) void moe_route_kernel(const T* __restrict__ x, long long x_stride,
                                                                  const TW* __restrict__ w, const void* __restrict__ correction,
                                                                  int c_dtype, int* __restrict__ ids, float* __restrict__ weights,
                                                                  int width, int experts, int top, const RouteRule rule) {
  extern __shared__ float route_lds[];   // [width] the row, then [experts] the scores, [experts] the choice numbers, [groups]
  float* xs = route_lds;
  float* score = route_lds + width;
  float* pick = score + experts;
  float* group_best = pick + experts;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const T* row = x + t * x_stride;
  for (int i = threadIdx.x; i < width; i += kRouteThreads) xs[i] = to_float(row[i]);
  __syncthreads();
  for (int e = wave; e < experts; e += kRouteThreads / kWave) {
    const TW* we = w + static_cast<int64_t>(e) * width;
    float dot = 0.f;
    if (VEC) {
      for (int i = 8 * lane; i < width; i += 8 * kWave) {
        const float4 lo = ld4<TW>(we + i), hi = ld4<TW>(we + i + 4);
        dot = fmaf(xs[i], lo.x, dot); dot = fmaf(xs[i + 1], lo.y, dot); dot = fmaf(xs[i + 2], lo.z, dot); dot = fmaf(xs[i + 3], lo.w, dot);
        dot = fmaf(xs[i + 4], hi.x, dot); dot = fmaf(xs[i + 5], hi.y, dot); dot = fmaf(xs[i + 6], hi.z, dot); dot = fmaf(xs[i + 7], hi.w, dot);
      }
    } else {
      for (int i = lane; i < width; i += kWave) dot = fmaf(xs[i], to_float(we[i]), dot);
    }
    dot = wave_sum(dot);
    if (lane == 0) score[e] = rule.softmax ? dot : 1.0f / (1.0f + expf(-dot));
  }
  __syncthreads();
  // From here on the first wave works alone; the others only keep the barriers' count.
  float s[kMaxExpertsPerLane], choice[kMaxExpertsPerLane];
  if (wave == 0) {
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      const int e = lane + j * kWave;
      s[j] = e < experts ? score[e] : (rule.softmax ? -INFINITY : 0.f);
    }
    if (rule.softmax) {   // over all router outputs, in 32 bits: the largest logit taken off, one sum in a fixed order
      float top_z = -INFINITY;
#pragma unroll
      for (int j = 0; j < kMaxExpertsPerLane; ++j) top_z = fmaxf(top_z, s[j]);
      top_z = wave_max(top_z);
      float sum = 0.f;
#pragma unroll
      for (int j = 0; j < kMaxExpertsPerLane; ++j) {
        s[j] = lane + j * kWave < experts ? expf(s[j] - top_z) : 0.f;
        sum += s[j];
      }
      const float inv = 1.0f / wave_sum(sum);
#pragma unroll
      for (int j = 0; j < kMaxExpertsPerLane; ++j) s[j] *= inv;
    }
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      const int e = lane + j * kWave;
      choice[j] = e < experts ? s[j] + (correction ? load_as_float(correction, c_dtype, e) : 0.f) : -INFINITY;
      if (e < experts) pick[e] = choice[j];
    }
  }
  if (rule.groups > 1) {   // (the same for every thread of the launch)
    __syncthreads();
    const int per = experts / rule.groups;
    if (wave == 0) {
      // a group's number is the largest choice number in it; lane l looks after the groups l, l + 64, ...
      float best[kMaxExpertsPerLane];
#pragma unroll
      for (int j = 0; j < kMaxExpertsPerLane; ++j) {
        const int g = lane + j * kWave;
        float b = -INFINITY;
        if (g < rule.groups)
          for (int i = 0; i < per; ++i) b = fmaxf(b, pick[g * per + i]);
        best[j] = b;
        if (g < rule.groups) group_best[g] = 0.f;   // 1 once the group is kept
      }
      for (int k = 0; k < rule.keep; ++k) {
        Best b{-INFINITY, 0x7fffffff};
#pragma unroll
        for (int j = 0; j < kMaxExpertsPerLane; ++j) {
          const int g = lane + j * kWave;
          if (g < rule.groups && best[j] != INFINITY && (best[j] > b.v || (best[j] == b.v && g < b.i))) {
            b.v = best[j];
            b.i = g;
          }
        }
        b = wave_best(b);
#pragma unroll
        for (int j = 0; j < kMaxExpertsPerLane; ++j) {
          if (b.i == lane + j * kWave) {
            best[j] = INFINITY;   // taken
            group_best[b.i] = 1.f;
          }
        }
      }
    }
    __syncthreads();
    if (wave == 0) {
#pragma unroll
      for (int j = 0; j < kMaxExpertsPerLane; ++j) {
        const int e = lane + j * kWave;
        if (e < experts && group_best[e / per] == 0.f) choice[j] = -INFINITY;
      }
    }
  }
  if (wave != 0) return;
  float sum = 0.f, mine = 0.f;   // lane k keeps the k-th chosen score (top <= 64)
  int mine_id = 0;
  for (int k = 0; k < top; ++k) {
    Best b{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < experts && s[j] >= 0.f && (choice[j] > b.v || (choice[j] == b.v && e < b.i))) {
        b.v = choice[j];
        b.i = e;
      }
    }
    b = wave_best(b);
    float sv = 0.f;
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      if (b.i == lane + j * kWave) {
        sv = s[j];
        choice[j] = -INFINITY;
        s[j] = -1.0f;   // taken: a score is never negative, so this marks it whatever its choice number was
      }
    }
    sv = __shfl(sv, b.i % kWave, kWave);
    sum += sv;
    if (lane == k) {
      mine = sv;
      mine_id = b.i;
    }
  }
  if (lane < top) {
    ids[t * top + lane] = mine_id;
    weights[t * top + lane] = (rule.normalize ? mine / (sum + 1e-20f) : mine) * rule.scale;
  }
}

// The rows of experts without tensors: where token t's k-th choice is a router output from `first` on, row t * top + k
// of out (float32 [T * top, width]) is the token's input itself.  One workgroup a token: it reads the row once and
// writes it for each such choice (most tokens have none, and their workgroups leave after reading `top` numbers).
template <typename T>
__global__ __launch_bounds__(256) void moe_identity_kernel(const T* __restrict__ x, long long x_stride,
                                                           const int* __restrict__ ids, float* __restrict__ out, int top,
                                                           int width, int first) {
  const int64_t t = blockIdx.x;
  unsigned long long which = 0;   // bit k: the k-th choice is such an expert (top <= 64)
  for (int k = 0; k < top; ++k) which |= static_cast<unsigned long long>(ids[t * top + k] >= first) << k;
  if (!which) return;
  const T* row = x + t * x_stride;
  for (int i = threadIdx.x; i < width; i += 256) {
    const float v = to_float(row[i]);
    for (unsigned long long left = which; left; left &= left - 1)
      out[(t * top + __builtin_ctzll(left)) * width + i] = v;
  }
}

constexpr int kEM = 64, kEN = 64, kEK = 16;
constexpr int kExpertThreads = 256;

// GATE_UP: w [experts, 2 N, K] (gate rows, then up rows), rows of x are tokens, out[(t top + k), n] = silu(g) u of
// type T.  Else: w [experts, N, K], rows of x are t top + k, out float32 [(t top + k), n].
template <typename T, bool GATE_UP>
__global__ __launch_bounds__(kExpertThreads) void moe_expert_kernel(const T* __restrict__ x, long long x_stride,
                                                                    const T* __restrict__ w, const int* __restrict__ ids,
                                                                    void* __restrict__ out, int tokens, int top, int N,
                                                                    int K) {
  __shared__ int list_t[kEM], list_k[kEM];
  __shared__ int count;
  __shared__ float as[kEK][kEM + 4];
  __shared__ float ws[kEK][kEN + 4];
  __shared__ float us[GATE_UP ? kEK : 1][kEN + 4];
  const int e = blockIdx.z;
  const int n0 = blockIdx.y * kEN;
  if (threadIdx.x < kWave) {
    const int t = blockIdx.x * kEM + threadIdx.x;
    int slot = -1;
    if (t < tokens)
      for (int k = 0; k < top; ++k)
        if (ids[static_cast<int64_t>(t) * top + k] == e) slot = k;
    const unsigned long long chose = __ballot(slot >= 0);
    if (slot >= 0) {
      const int rank = __popcll(chose & ((1ull << threadIdx.x) - 1ull));
      list_t[rank] = t;
      list_k[rank] = slot;
    }
    if (threadIdx.x == 0) count = __popcll(chose);
  }
  __syncthreads();
  const int rows = count;
  if (rows == 0) return;
  const T* we = w + static_cast<int64_t>(e) * (GATE_UP ? 2 : 1) * N * K;
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  float acc[4][4] = {}, acc_u[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += kEK) {
#pragma unroll
    for (int i = 0; i < (kEM * kEK) / kExpertThreads; ++i) {
      const int idx = threadIdx.x + i * kExpertThreads;
      const int r = idx / kEK, c = idx % kEK;
      const int gk = k0 + c, gn = n0 + r;
      float av = 0.f;
      if (r < rows && gk < K) {
        const int64_t src = GATE_UP ? list_t[r] : static_cast<int64_t>(list_t[r]) * top + list_k[r];
        av = to_float(x[src * x_stride + gk]);
      }
      as[c][r] = av;
      const bool in = gn < N && gk < K;
      ws[c][r] = in ? to_float(we[static_cast<int64_t>(gn) * K + gk]) : 0.f;
      if (GATE_UP) us[c][r] = in ? to_float(we[static_cast<int64_t>(N + gn) * K + gk]) : 0.f;
    }
    __syncthreads();
    float part[4][4] = {}, part_u[4][4] = {};
#pragma unroll
    for (int kk = 0; kk < kEK; ++kk) {
      float av[4], wv[4], uv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = as[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        wv[j] = ws[kk][tx * 4 + j];
        if (GATE_UP) uv[j] = us[kk][tx * 4 + j];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          part[i][j] = fmaf(av[i], wv[j], part[i][j]);
          if (GATE_UP) part_u[i][j] = fmaf(av[i], uv[j], part_u[i][j]);
        }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[i][j] += part[i][j];
        if (GATE_UP) acc_u[i][j] += part_u[i][j];
      }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = ty * 4 + i;
    if (r >= rows) continue;
    const int64_t dst = (static_cast<int64_t>(list_t[r]) * top + list_k[r]) * N;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      if (GATE_UP) {
        const float g = acc[i][j];
        static_cast<T*>(out)[dst + n] = from_float<T>(g / (1.0f + expf(-g)) * acc_u[i][j]);
      } else {
        static_cast<float*>(out)[dst + n] = acc[i][j];
      }
    }
  }
}

// ---- matrix-core form (bfloat16) -----------------------------------------------------------------
// A workgroup of four waves takes one expert, 256 consecutive rows of the step and a tile of output columns (64 gate
// and the 64 matching up columns, or 128 columns of down).  It lists the rows of its 256 that chose the expert, in row
// order, and walks them 64 at a time: wave w multiplies rows 16 w .. 16 w + 15 of the 64 by the whole column tile
// with `v_mfma_f32_16x16x32_bf16`.  The weight tile of a k step (128 rows of 32) goes through LDS once for the four
// waves; a wave's own rows come straight from memory, sixteen bytes a lane, which is the A operand as it lies.  The
// next k step's loads are in flight while this one's products run.  K a multiple of 8; rows 16-byte aligned.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kMoeChunk = 256;     // rows of the step a workgroup looks through
constexpr int kMoeCols = 128;      // weight rows of a tile (gate|up: 64 + 64)
constexpr int kMoeLdsRow = 40;     // bfloat16 a weight row of 32 takes in LDS (80 bytes: no two lanes of a read on one bank)

template <bool GATE_UP>
__global__ __launch_bounds__(256) void moe_expert_mfma_kernel(const bf16* __restrict__ x, long long x_stride,
                                                              const bf16* __restrict__ w, const int* __restrict__ ids,
                                                              void* __restrict__ out, int tokens, int top, int N, int K) {
  __shared__ int list_src[kMoeChunk], list_dst[kMoeChunk];
  __shared__ int wave_count[4];
  __shared__ __attribute__((aligned(16))) bf16 wt[kMoeCols * kMoeLdsRow];
  const int e = blockIdx.z;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n = lane % 16, g = lane / 16;
  {
    const int t = blockIdx.x * kMoeChunk + threadIdx.x;
    int slot = -1;
    if (t < tokens)
      for (int k = 0; k < top; ++k)
        if (ids[static_cast<int64_t>(t) * top + k] == e) slot = k;
    const unsigned long long chose = __ballot(slot >= 0);
    if (lane == 0) wave_count[wave] = __popcll(chose);
    __syncthreads();
    int before = 0;
    for (int i = 0; i < wave; ++i) before += wave_count[i];
    if (slot >= 0) {
      const int rank = before + __popcll(chose & ((1ull << lane) - 1ull));
      list_src[rank] = GATE_UP ? t : t * top + slot;
      list_dst[rank] = t * top + slot;
    }
    __syncthreads();
  }
  const int rows = wave_count[0] + wave_count[1] + wave_count[2] + wave_count[3];
  if (rows == 0) return;
  const int cols = GATE_UP ? kMoeCols / 2 : kMoeCols;     // output columns of the tile
  const int n0 = blockIdx.y * cols;
  const bf16* we = w + static_cast<int64_t>(e) * (GATE_UP ? 2 : 1) * N * K;
  // the weight row this thread copies into LDS (two pieces of 8 of a row of 32), or none past N
  const int wr = threadIdx.x / 2, wpiece = (threadIdx.x % 2) * 16;
  const int wcol = GATE_UP ? (wr < 64 ? n0 + wr : n0 + wr - 64) : n0 + wr;
  const bool w_in = wcol < N;
  const bf16* wsrc = we + static_cast<int64_t>(GATE_UP && wr >= 64 ? N + wcol : wcol) * K;
  const u32x4_t zero = {0, 0, 0, 0};
  for (int sub = 0; sub * 64 < rows; ++sub) {
    const int r = sub * 64 + wave * 16 + n;
    const bf16* arow = x + static_cast<int64_t>(list_src[min(r, rows - 1)]) * x_stride;
    f32x4_t acc[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) acc[j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    u32x4_t a_next, w_next[2];
    auto fetch = [&](int k0) {
      const int ka = k0 + 8 * g;
      a_next = ka < K ? *reinterpret_cast<const u32x4_t*>(arow + ka) : zero;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int kw = k0 + wpiece + 8 * h;
        w_next[h] = (w_in && kw < K) ? *reinterpret_cast<const u32x4_t*>(wsrc + kw) : zero;
      }
    };
    fetch(0);
    for (int k0 = 0; k0 < K; k0 += 32) {
      const u32x4_t a_now = a_next;
      __syncthreads();      // the tile before has been read by every wave
#pragma unroll
      for (int h = 0; h < 2; ++h) *reinterpret_cast<u32x4_t*>(&wt[wr * kMoeLdsRow + wpiece + 8 * h]) = w_next[h];
      __syncthreads();
      if (k0 + 32 < K) fetch(k0 + 32);
      const bf16x8_t a_op = __builtin_bit_cast(bf16x8_t, a_now);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const u32x4_t b = *reinterpret_cast<const u32x4_t*>(&wt[(16 * j + n) * kMoeLdsRow + 8 * g]);
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op, __builtin_bit_cast(bf16x8_t, b), acc[j], 0, 0, 0);
      }
    }
    // acc[j][i] is the product of row 4 g + i of the wave's sixteen and weight row 16 j + n of the tile
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int rr = sub * 64 + wave * 16 + 4 * g + i;
      if (rr >= rows) continue;
      const int64_t dst = static_cast<int64_t>(list_dst[rr]) * N;
      if (GATE_UP) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const int col = n0 + 16 * j + n;
          const float gt = acc[j][i];
          if (col < N) static_cast<bf16*>(out)[dst + col] = from_float<bf16>(gt / (1.0f + expf(-gt)) * acc[j + 4][i]);
        }
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int col = n0 + 16 * j + n;
          if (col < N) static_cast<float*>(out)[dst + col] = acc[j][i];
        }
      }
    }
    __syncthreads();        // before the next 64 rows overwrite the tile
  }
}

// ---- the same for many rows --------------------------------------------------------------------
// With a few hundred rows an expert the form above reads every weight fragment from LDS once for sixteen rows, and
// what a launch waits for is the passes over the weights: every workgroup streams its weight tile over all of K.  Here
// a workgroup of RG x 4 waves (RG 1 or 2) looks through RG x 256 rows of the step and takes RG x 64 listed rows and 256 weight rows
// (128 gate and the 128 matching up columns, or 256 columns of down) a k step, both through LDS: the weight tile is
// fetched once for all RG groups of 64 rows, and a wave multiplies the 64 rows of its group by 64 weight rows (32
// gate and their 32 up columns): sixteen products for four row and four weight fragments, twice a k step of 64.  Two
// k steps of loads are in flight; sixteen rows that hold no listed row are not multiplied.  (A k step of 64 instead
// of 32, with half the barriers a product: 4,647 instead of 5,228 us for the sixteen launches of a 2,048-token prefill
// at the Qwen3-4B widths.)
constexpr int kBigCols = 256;       // weight rows of a tile
constexpr int kBigRows = 64;        // listed rows of a group of four waves

template <bool GATE_UP, int RG, int BK>
__global__ __launch_bounds__(256 * RG) void moe_expert_tiles_kernel(const bf16* __restrict__ x, long long x_stride,
                                                                    const bf16* __restrict__ w, const int* __restrict__ ids,
                                                                    void* __restrict__ out, int tokens, int top, int N,
                                                                    int K) {
  constexpr int kThreads = 256 * RG, kWaves = 4 * RG, kRows = kBigRows * RG;
  constexpr int kLdsRow = BK + 8;                 // bfloat16 a row of BK takes in LDS (no two lanes of a read on one bank)
  constexpr int kLanesRow = BK / 8;               // lanes that copy one row of a tile, a piece of 8 each (whole lines)
  constexpr int kPass = kThreads / kLanesRow;     // rows that the workgroup copies in one go
  constexpr int kWPieces = kBigCols / kPass, kAPieces = kRows / kPass;
  __shared__ int list_src[kThreads], list_dst[kThreads];
  __shared__ int wave_count[kWaves];
  __shared__ __attribute__((aligned(16))) bf16 wt[kBigCols * kLdsRow];
  __shared__ __attribute__((aligned(16))) bf16 at[kRows * kLdsRow];
  const int e = blockIdx.z;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n = lane % 16, g = lane / 16;
  const int rg = wave / 4, cw = wave % 4;     // the wave's group of 64 rows, and its 64 weight rows of the tile
  {
    const int t = blockIdx.x * kThreads + threadIdx.x;
    int slot = -1;
    if (t < tokens)
      for (int k = 0; k < top; ++k)
        if (ids[static_cast<int64_t>(t) * top + k] == e) slot = k;
    const unsigned long long chose = __ballot(slot >= 0);
    if (lane == 0) wave_count[wave] = __popcll(chose);
    __syncthreads();
    int before = 0;
    for (int i = 0; i < wave; ++i) before += wave_count[i];
    if (slot >= 0) {
      const int rank = before + __popcll(chose & ((1ull << lane) - 1ull));
      list_src[rank] = GATE_UP ? t : t * top + slot;
      list_dst[rank] = t * top + slot;
    }
    __syncthreads();
  }
  int rows = 0;
#pragma unroll
  for (int i = 0; i < kWaves; ++i) rows += wave_count[i];
  if (rows == 0) return;
  const int cols = GATE_UP ? kBigCols / 2 : kBigCols;     // output columns of the tile
  const int n0 = blockIdx.y * cols;
  const bf16* we = w + static_cast<int64_t>(e) * (GATE_UP ? 2 : 1) * N * K;
  // the weight rows of which this thread copies one piece of 8 into LDS: LDS row r belongs to column wave r / 64; of
  // its 64 rows the first 32 are gate columns, the last 32 the matching up columns
  const int piece = (static_cast<int>(threadIdx.x) % kLanesRow) * 8, prow = static_cast<int>(threadIdx.x) / kLanesRow;
  const bf16* wsrc[kWPieces];
  bool w_in[kWPieces];
#pragma unroll
  for (int h = 0; h < kWPieces; ++h) {
    const int r = kPass * h + prow;
    int wcol, wrow_global;
    if (GATE_UP) {
      const int within = r % 64;
      wcol = n0 + (r / 64) * 32 + within % 32;
      wrow_global = within < 32 ? wcol : N + wcol;
    } else {
      wcol = n0 + r;
      wrow_global = wcol;
    }
    w_in[h] = wcol < N;
    wsrc[h] = we + static_cast<int64_t>(w_in[h] ? wrow_global : 0) * K + piece;
  }
  const u32x4_t zero = {0, 0, 0, 0};
  for (int sub = 0; sub * kRows < rows; ++sub) {
    const bf16* asrc[kAPieces];
#pragma unroll
    for (int h = 0; h < kAPieces; ++h)
      asrc[h] = x + static_cast<int64_t>(list_src[min(sub * kRows + kPass * h + prow, rows - 1)]) * x_stride + piece;
    f32x4_t acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    const int first = sub * kRows + kBigRows * rg;        // the first listed row of this wave's group
    const int live = max(0, min(4, (rows - first + 15) / 16));
    // two k steps are in flight: the loads of step k + 2 are sent while step k is multiplied
    u32x4_t a_set[2][kAPieces], w_set[2][kWPieces];
    auto fetch = [&](int k0, u32x4_t (&a_to)[kAPieces], u32x4_t (&w_to)[kWPieces]) {
#pragma unroll
      for (int h = 0; h < kAPieces; ++h)
        a_to[h] = k0 + piece < K ? *reinterpret_cast<const u32x4_t*>(asrc[h] + k0) : zero;
#pragma unroll
      for (int h = 0; h < kWPieces; ++h)
        w_to[h] = (w_in[h] && k0 + piece < K) ? *reinterpret_cast<const u32x4_t*>(wsrc[h] + k0) : zero;
    };
    auto step = [&](int k0, u32x4_t (&a_reg)[kAPieces], u32x4_t (&w_reg)[kWPieces]) {
      __syncthreads();      // the tiles before have been read by every wave
#pragma unroll
      for (int h = 0; h < kAPieces; ++h) *reinterpret_cast<u32x4_t*>(&at[(kPass * h + prow) * kLdsRow + piece]) = a_reg[h];
#pragma unroll
      for (int h = 0; h < kWPieces; ++h) *reinterpret_cast<u32x4_t*>(&wt[(kPass * h + prow) * kLdsRow + piece]) = w_reg[h];
      __syncthreads();
      if (k0 + 2 * BK < K) fetch(k0 + 2 * BK, a_reg, w_reg);
      if (live == 0) return;
#pragma unroll
      for (int kk = 0; kk < BK; kk += 32) {
        bf16x8_t a_op[4], b_op[4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          a_op[i] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&at[(kBigRows * rg + 16 * i + n) * kLdsRow + kk + 8 * g]));
#pragma unroll
        for (int j = 0; j < 4; ++j)
          b_op[j] = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const u32x4_t*>(&wt[(64 * cw + 16 * j + n) * kLdsRow + kk + 8 * g]));
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (i < live) {       // sixteen rows of the 64 that hold no listed row are not multiplied
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a_op[i], b_op[j], acc[i][j], 0, 0, 0);
          }
      }
    };
    fetch(0, a_set[0], w_set[0]);
    if (BK < K) fetch(BK, a_set[1], w_set[1]);
    for (int k0 = 0; k0 < K; k0 += 2 * BK) {
      step(k0, a_set[0], w_set[0]);
      if (k0 + BK < K) step(k0 + BK, a_set[1], w_set[1]);
    }
    // acc[i][j][c]: listed row 16 i + 4 g + c of the group's 64, weight row 16 j + n of the wave's 64
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int rr = first + 16 * i + 4 * g + c;
        if (rr >= rows) continue;
        const int64_t dst = static_cast<int64_t>(list_dst[rr]) * N;
        if (GATE_UP) {
#pragma unroll
          for (int j = 0; j < 2; ++j) {
            const int col = n0 + cw * 32 + 16 * j + n;
            const float gt = acc[i][j][c];
            if (col < N) static_cast<bf16*>(out)[dst + col] = from_float<bf16>(gt / (1.0f + expf(-gt)) * acc[i][j + 2][c]);
          }
        } else {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int col = n0 + cw * 64 + 16 * j + n;
            if (col < N) static_cast<float*>(out)[dst + col] = acc[i][j][c];
          }
        }
      }
    }
    __syncthreads();        // before the next rows overwrite the tiles
  }
}

}  // namespace arle

using namespace arle;

// x [T, width] of x_dtype, w [experts, width] of w_dtype, correction [experts] or null; ids int32 [T, top], weights
// float32 [T, top].
extern "C" int arle_moe_route(const void* x, long long x_stride, int x_dtype, const void* w, int w_dtype,
                              const void* correction, int c_dtype, int* ids, float* weights, int tokens, int width,
                              int experts, int top, float scale, int softmax, int groups, int keep, int normalize,
                              void* stream) {
  if (tokens == 0) return 0;
  if (experts < 1 || experts > kWave * kMaxExpertsPerLane || top < 1 || top > experts || top > kWave || groups < 1 ||
      experts % groups || keep < 1 || keep > groups || top > keep * (experts / groups))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const RouteRule rule{softmax, groups, keep, normalize, scale};
  const size_t lds = static_cast<size_t>(width + 2 * experts + groups) * sizeof(float);
  if (lds > 60 * 1024) return static_cast<int>(hipErrorInvalidValue);
  const bool vec = width % 8 == 0 && reinterpret_cast<uintptr_t>(w) % 16 == 0;
#define ARLE_ROUTE_V(TX, TWT, V)                                                                                   \
  do {                                                                                                             \
    static bool raised = false;                                                                                    \
    if (!raised && lds > 48 * 1024) {                                                                              \
      const hipError_t err = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_route_kernel<TX, TWT, V>),     \
                                                 hipFuncAttributeMaxDynamicSharedMemorySize, 60 * 1024);           \
      if (err != hipSuccess) return static_cast<int>(err);                                                         \
      raised = true;                                                                                               \
    }                                                                                                              \
    moe_route_kernel<TX, TWT, V><<<tokens, kRouteThreads, lds, s>>>(static_cast<const TX*>(x), x_stride,           \
                                                                    static_cast<const TWT*>(w), correction, c_dtype, \
                                                                    ids, weights, width, experts, top, rule);       \
  } while (0)
#define ARLE_ROUTE(TX, TWT)                          \
  do {                                               \
    if (vec) ARLE_ROUTE_V(TX, TWT, true);            \
    else ARLE_ROUTE_V(TX, TWT, false);               \
  } while (0)
  if (x_dtype == kF32) {
    if (w_dtype == kF32) ARLE_ROUTE(float, float); else ARLE_ROUTE(float, bf16);
  } else {
    if (w_dtype == kF32) ARLE_ROUTE(bf16, float); else ARLE_ROUTE(bf16, bf16);
  }
#undef ARLE_ROUTE
#undef ARLE_ROUTE_V
  return launch_status();
}

// x [T, width] of `dtype`, ids int32 [T * top], out float32 [T * top, width]: see moe_identity_kernel.
extern "C" int arle_moe_identity(const void* x, long long x_stride, int dtype, const int* ids, void* out, int tokens,
                                 int top, int width, int first, void* stream) {
  if (tokens == 0) return 0;
  if (top < 1 || top > 64 || width < 1 || first < 0) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const unsigned items = static_cast<unsigned>(tokens);
  if (dtype == kF32)
    moe_identity_kernel<float><<<items, 256, 0, s>>>(static_cast<const float*>(x), x_stride, ids, static_cast<float*>(out), top, width, first);
  else
    moe_identity_kernel<bf16><<<items, 256, 0, s>>>(static_cast<const bf16*>(x), x_stride, ids, static_cast<float*>(out), top, width, first);
  return launch_status();
}

// gate_up != 0: x [T, K], w [experts, 2 N, K], out [T * top, N] of `dtype`.  Else: x [T * top, K], w [experts, N, K],
// out float32 [T * top, N].
extern "C" int arle_moe_expert(const void* x, long long x_stride, const void* w, const int* ids, void* out, int dtype,
                               int gate_up, int tokens, int experts, int top, int N, int K, void* stream) {
  if (tokens == 0) return 0;
  if (experts < 1 || experts > 65535 || top < 1 || N < 1 || K < 1 || (N + kEN - 1) / kEN > 65535)
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kBF16 && K % 8 == 0 && x_stride % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w) % 16 == 0) {
    if (tokens > 64) {      // rows enough that an expert's list fills tiles of 64
      const int bcols = gate_up ? kBigCols / 2 : kBigCols;
      const bf16* xb = static_cast<const bf16*>(x);
      const bf16* wb = static_cast<const bf16*>(w);
#define ARLE_TILES(GU, RGS)                                                                                      \
  moe_expert_tiles_kernel<GU, RGS, 64><<<dim3((tokens + 256 * RGS - 1) / (256 * RGS), (N + bcols - 1) / bcols, experts), \
                                         256 * RGS, 0, s>>>(xb, x_stride, wb, ids, out, tokens, top, N, K)
      // two groups of 64 rows a weight tile once the step has rows for them: a tile's fetch is what the launch waits
      // for (all sixteen launches of a 2,048-token prefill at the Qwen3-4B widths: one group 6,508 us, two 5,219 us,
      // four, which leaves a wave 128 registers, 5,456 us)
      if (tokens > 256) {
        if (gate_up) ARLE_TILES(true, 2); else ARLE_TILES(false, 2);
      } else {
        if (gate_up) ARLE_TILES(true, 1); else ARLE_TILES(false, 1);
      }
#undef ARLE_TILES
      return launch_status();
    }
    const int cols = gate_up ? kMoeCols / 2 : kMoeCols;
    const dim3 mgrid((tokens + kMoeChunk - 1) / kMoeChunk, (N + cols - 1) / cols, experts);
    if (gate_up)
      moe_expert_mfma_kernel<true><<<mgrid, 256, 0, s>>>(static_cast<const bf16*>(x), x_stride, static_cast<const bf16*>(w), ids, out, tokens, top, N, K);
    else
      moe_expert_mfma_kernel<false><<<mgrid, 256, 0, s>>>(static_cast<const bf16*>(x), x_stride, static_cast<const bf16*>(w), ids, out, tokens, top, N, K);
    return launch_status();
  }
  const dim3 grid((tokens + kEM - 1) / kEM, (N + kEN - 1) / kEN, experts);
#define ARLE_EXPERT(TT, GU)                                                                                         \
  moe_expert_kernel<TT, GU><<<grid, kExpertThreads, 0, s>>>(static_cast<const TT*>(x), x_stride,                    \
                                                            static_cast<const TT*>(w), ids, out, tokens, top, N, K)
  if (dtype == kF32) {
    if (gate_up) ARLE_EXPERT(float, true); else ARLE_EXPERT(float, false);
  } else {
    if (gate_up) ARLE_EXPERT(bf16, true); else ARLE_EXPERT(bf16, false);
  }
#undef ARLE_EXPERT
  return launch_status();
}
