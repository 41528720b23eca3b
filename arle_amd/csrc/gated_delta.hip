// The gated delta rule, token by token, for the rows of a packed step, continued across steps through a
// per-request state S [heads, D, Dv] in 32-bit floats.
//
// Per head, with q and k of D entries (head h reads q/k head h / (H / G)) and v of Dv:
//   q <- q / sqrt(sum q^2 + 1e-6) * D^(-1/2),   k <- k / sqrt(sum k^2 + 1e-6)
//   beta = sigmoid(b),   g = exp(-exp(A_log_h) * softplus(a + dt_bias_h))
//   S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q
// CHANNEL: a decay for every head and key entry, g_d = exp(-exp(A_log_h) * softplus(a_hd + dt_bias_hd)), on the rows of
// S (S <- diag(g) S); the decays' pre-activations are then a [T, H, D], and dt_bias [H, D].
// A column of S (one entry of v) never meets another, so the columns spread over workgroups: a workgroup a
// (request, head, 16 columns), four columns a wave, a sixteenth of D a lane.  Rows go through LDS in blocks of
// 32; the block's unit norms, gates and the dot products k . q are made there, a row by eight threads, always
// the same entries in the same order.  The chain of a row is one pass over the lane's share of the old S for both
// S^T k and S^T q (o = g S_old^T q + u (k . q), which is S_new^T q), one exchange over the sixteen shares, and the
// update.  Two layouts of a wave, which add the sixteen shares in the same tree and so give the same bits.  ROWS
// (steps with portions): the sixteen shares of a column are the sixteen lanes of a row of the wave, and the exchange
// is four data-parallel-primitive moves inside the vector unit (neighbours, pairs, the mirrored half, the mirrored
// row), never through LDS, whose unit the rows' reads of q and k keep busy.  Otherwise (steps of decoded rows, whose
// time is the state's way in and out): the four columns of a wave are four neighbouring lanes, so that a load of the
// state is sixteen bytes for every four lanes, and the shares exchange through lane reads four, eight, sixteen and
// 32 lanes away.  `gated_delta_output` divides each head's o by its root mean square, multiplies by the norm's weight and
// by silu (or sigmoid) of the gate's projection.
#include "common.h"

namespace arle {

constexpr int kGdWaves = 4;
constexpr int kGdThreads = kGdWaves * kWave;
constexpr int kGdWaveCols = 4;
constexpr int kGdParts = kWave / kGdWaveCols;     // shares of D
constexpr int kGdCols = kGdWaves * kGdWaveCols;   // columns of a workgroup
constexpr int kGdRows = 32;                       // rows staged at a time
constexpr int kGdRowThreads = kGdThreads / kGdRows;   // threads that prepare a row

__device__ __forceinline__ float softplus(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

// The sum of v over the sixteen lanes of a row, in every lane of the row, the same bits in each: lane i adds lane
// i ^ 1, then i ^ 2 (afterwards the four lanes of a quad agree), then the lane mirrored in its half (the other quad's
// sum), then the lane mirrored in its row (the other half's sum).
template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xf, 0xf, true));
}
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_move<0xB1>(v);    // quad_perm [1, 0, 3, 2]
  v += dpp_move<0x4E>(v);    // quad_perm [2, 3, 0, 1]
  v += dpp_move<0x141>(v);   // row_half_mirror
  v += dpp_move<0x140>(v);   // row_mirror
  return v;
}

template <typename T, int DS, bool ROWS, bool CHANNEL>
__global__ __launch_bounds__(kGdThreads) void gated_delta_scan_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const float* __restrict__ beta_in /* [T, H] */, long long beta_stride,
    const float* __restrict__ decay_in /* [T, H], CHANNEL: [T, H * D] */, long long decay_stride,
    const float* __restrict__ a_log, const float* __restrict__ dt_bias, float unit_eps, float* __restrict__ s_state,
    const int* __restrict__ seg_row0, const int* __restrict__ seg_slot, float* __restrict__ out /* [T, H * Dv] */,
    int H, int G, int D, int Dv) {
  constexpr int DP = kGdParts * DS;   // padded D: what lies past D is zero in LDS and in the registers
  constexpr int RS = ROWS ? kGdRows : 1;   // rows staged at a time: a decoded row's segment is that one row
  __shared__ __attribute__((aligned(16))) float q_lds[RS][DP];
  __shared__ __attribute__((aligned(16))) float k_lds[RS][DP];
  __shared__ __attribute__((aligned(16))) float g_lds[CHANNEL ? RS : 1][DP];   // CHANNEL: the decays of the key entries
  __shared__ float v_lds[RS][kGdCols];
  __shared__ float c_lds[RS][4];   // decay (of the head), beta, k . q
  const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int kvh = h / (H / G);
  static_assert(kGdParts == 16, "a column's shares are the lanes of one row of sixteen");
  const int col_in = wave * kGdWaveCols + (ROWS ? lane / kGdParts : lane % kGdWaveCols);
  const int col = blockIdx.z * kGdCols + col_in;
  const int part = ROWS ? lane % kGdParts : lane / kGdWaveCols;
  const bool live = col < Dv;
  const int row0 = seg_row0[seg], rows = ROWS ? seg_row0[seg + 1] - row0 : 1;
  float* s_ptr = s_state + (static_cast<int64_t>(seg_slot[seg]) * H + h) * D * Dv;
  const float rate = expf(a_log[h]), bias = CHANNEL ? 0.f : dt_bias[h], q_scale = 1.0f / sqrtf(static_cast<float>(D));

  float S[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    S[i] = (live && d < D) ? s_ptr[static_cast<int64_t>(d) * Dv + col] : 0.f;
  }
  // A block's rows are fetched from memory into registers while the chain of the block before runs, and go on to LDS
  // (with their norms and gates) when it has ended.
  constexpr int kMine = DP / kGdRowThreads;                      // entries of a row's q (and k) a thread prepares
  constexpr int kValues = (RS * kGdCols + kGdThreads - 1) / kGdThreads;   // entries of the block's v a thread moves
  const int r = tid / kGdRowThreads, sub = tid % kGdRowThreads;   // a row by kGdRowThreads threads
  float q_next[kMine], k_next[kMine], v_next[kValues], b_next = 0.f, a_next = 0.f;
  // CHANNEL: a_hd of the row and dt_bias_hd.  With portions a row's eight threads take the entries they prepare of q
  // and k; a decoded row's entries go one a thread (entry `tid`), so that the exponentials are one deep, not sixteen.
  constexpr int kDecays = ROWS ? kMine : 1;
  float g_next[CHANNEL ? kDecays : 1], g_bias[CHANNEL ? kDecays : 1];
  if constexpr (CHANNEL) {
#pragma unroll
    for (int j = 0; j < kDecays; ++j) {
      const int d = ROWS ? sub + j * kGdRowThreads : tid;
      g_bias[j] = d < D ? dt_bias[h * D + d] : 0.f;
    }
  }
  auto fetch = [&](int base) {
    const int n = min(kGdRows, rows - base);   // <= 0 behind the last block: nothing is loaded
    const int64_t t = row0 + base + min(r, max(n, 1) - 1);
    const T* qr = q + t * q_stride + kvh * D;
    const T* kr = k + t * k_stride + kvh * D;
#pragma unroll
    for (int j = 0; j < kMine; ++j) {
      const int d = sub + j * kGdRowThreads;
      const bool there = r < n && d < D;
      q_next[j] = there ? to_float(qr[d]) : 0.f;
      k_next[j] = there ? to_float(kr[d]) : 0.f;
      if constexpr (CHANNEL && ROWS) g_next[j] = there ? decay_in[t * decay_stride + h * D + d] : 0.f;
    }
    if constexpr (CHANNEL && !ROWS) g_next[0] = (n > 0 && tid < D) ? decay_in[(row0 + base) * decay_stride + h * D + tid] : 0.f;
    if (sub == 0 && r < n) {
      b_next = beta_in[t * beta_stride + h];
      if constexpr (!CHANNEL) a_next = decay_in[t * decay_stride + h];
    }
#pragma unroll
    for (int j = 0; j < kValues; ++j) {
      const int e = tid + j * kGdThreads, rr = e / kGdCols, cc = e % kGdCols;
      const int c_abs = min(static_cast<int>(blockIdx.z) * kGdCols + cc, Dv - 1);
      v_next[j] = (rr < n && e < RS * kGdCols) ? to_float(v[(row0 + base + rr) * v_stride + h * Dv + c_abs]) : 0.f;
    }
  };
  fetch(0);
  for (int base = 0; base < rows; base += kGdRows) {
    const int n = min(kGdRows, rows - base);
    __syncthreads();   // the block before has been read
    if (r < n) {   // (the threads of a row leave or stay together; a decoded row's block is one row)
      float sq = 0.f, sk = 0.f, kq = 0.f;
#pragma unroll
      for (int j = 0; j < kMine; ++j) {
        sq = fmaf(q_next[j], q_next[j], sq);
        sk = fmaf(k_next[j], k_next[j], sk);
        kq = fmaf(k_next[j], q_next[j], kq);
      }
#pragma unroll
      for (int off = kGdRowThreads / 2; off > 0; off >>= 1) {
        sq += __shfl_xor(sq, off, kWave);
        sk += __shfl_xor(sk, off, kWave);
        kq += __shfl_xor(kq, off, kWave);
      }
      const float fq = q_scale / sqrtf(sq + unit_eps), fk = 1.0f / sqrtf(sk + unit_eps);
#pragma unroll
      for (int j = 0; j < kMine; ++j) {
        if constexpr (CHANNEL && ROWS)   // (past D: some decay on zeros)
          g_lds[r][sub + j * kGdRowThreads] = expf(-rate * softplus(g_next[j] + g_bias[j]));
        q_lds[r][sub + j * kGdRowThreads] = q_next[j] * fq;
        k_lds[r][sub + j * kGdRowThreads] = k_next[j] * fk;
      }
      if (sub == 0) {
        c_lds[r][0] = CHANNEL ? 1.0f : expf(-rate * softplus(a_next + bias));
        c_lds[r][1] = 1.0f / (1.0f + expf(-b_next));
        c_lds[r][2] = kq * fq * fk;
      }
    }
    if constexpr (CHANNEL && !ROWS) {
      if (tid < DP) g_lds[0][tid] = expf(-rate * softplus(g_next[0] + g_bias[0]));
    }
#pragma unroll
    for (int j = 0; j < kValues; ++j) {
      const int e = tid + j * kGdThreads;
      if (e < RS * kGdCols) v_lds[e / kGdCols][e % kGdCols] = v_next[j];
    }
    __syncthreads();
    fetch(base + kGdRows);
    for (int r = 0; r < n; ++r) {
      const float g = c_lds[r][0], beta = c_lds[r][1], kq = c_lds[r][2];
      float kk[DS], dk = 0.f, dq = 0.f;
      if constexpr (CHANNEL) {   // the decayed state diag(g) S first, in the registers: everything below reads it
        if constexpr (DS % 4 == 0) {
          const float4* g4 = reinterpret_cast<const float4*>(&g_lds[r][part * DS]);
#pragma unroll
          for (int i = 0; i < DS / 4; ++i) {
            const float4 gv = g4[i];
            S[4 * i] *= gv.x; S[4 * i + 1] *= gv.y; S[4 * i + 2] *= gv.z; S[4 * i + 3] *= gv.w;
          }
        } else {
#pragma unroll
          for (int i = 0; i < DS; ++i) S[i] *= g_lds[r][part * DS + i];
        }
      }
      if constexpr (DS % 4 == 0) {
        const float4* k4 = reinterpret_cast<const float4*>(&k_lds[r][part * DS]);
        const float4* q4 = reinterpret_cast<const float4*>(&q_lds[r][part * DS]);
#pragma unroll
        for (int i = 0; i < DS / 4; ++i) {
          const float4 kv = k4[i], qv = q4[i];
          kk[4 * i] = kv.x; kk[4 * i + 1] = kv.y; kk[4 * i + 2] = kv.z; kk[4 * i + 3] = kv.w;

          dq = fmaf(S[4 * i], qv.x, dq); dq = fmaf(S[4 * i + 1], qv.y, dq);
          dq = fmaf(S[4 * i + 2], qv.z, dq); dq = fmaf(S[4 * i + 3], qv.w, dq);
        }
      } else {
#pragma unroll
        for (int i = 0; i < DS; ++i) {
          kk[i] = k_lds[r][part * DS + i];
          dq = fmaf(S[i], q_lds[r][part * DS + i], dq);
        }
      }
#pragma unroll
      for (int i = 0; i < DS; ++i) dk = fmaf(S[i], kk[i], dk);
      if constexpr (ROWS) {   // over the shares of D: with share p ^ 1, then p ^ 2, p ^ 4, p ^ 8
        dk = row16_sum(dk);
        dq = row16_sum(dq);
      } else {
#pragma unroll
        for (int off = kGdWaveCols; off < kWave; off <<= 1) {
          dk += __shfl_xor(dk, off, kWave);
          dq += __shfl_xor(dq, off, kWave);
        }
      }
      const float u = beta * (v_lds[r][col_in] - g * dk);
#pragma unroll
      for (int i = 0; i < DS; ++i) S[i] = fmaf(kk[i], u, CHANNEL ? S[i] : g * S[i]);
      if (part == 0 && live) out[static_cast<int64_t>(row0 + base + r) * (H * Dv) + h * Dv + col] = fmaf(u, kq, g * dq);
    }
  }
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    if (live && d < D) s_ptr[static_cast<int64_t>(d) * Dv + col] = S[i];
  }
}

// One wave a (row, head): o / rms(o) * w * act(gate), act silu or sigmoid (a kAct code).
template <typename T>
__global__ __launch_bounds__(kWave) void gated_delta_output_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                                   long long gate_stride, const void* __restrict__ weight,
                                                                   int w_dtype, float eps, T* __restrict__ out, int H,
                                                                   int Dv, int act) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* row = o + (t * H + h) * Dv;
  float ss = 0.f;
  for (int d = lane; d < Dv; d += kWave) ss = fmaf(row[d], row[d], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dv) + eps);
  for (int d = lane; d < Dv; d += kWave) {
    const float z = to_float(gate[t * gate_stride + h * Dv + d]);
    out[(t * H + h) * Dv + d] = from_float<T>(row[d] * inv * load_as_float(weight, w_dtype, d) * gate_act(z, act));
  }
}

}  // namespace arle

using namespace arle;

extern "C" int arle_gated_delta_scan(const void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                                     long long v_stride, int dtype, const void* beta_in, long long beta_stride,
                                     const void* decay_in, long long decay_stride, const void* a_log, const void* dt_bias, float unit_eps, void* s_state,
                                     const int* seg_row0, const int* seg_slot, int segments, int single_rows, void* out,
                                     int H, int G, int D, int Dv, int channel, void* stream) {
  if (segments == 0) return 0;
  if (D < 1 || D > 256 || H % G) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid(segments, H, (Dv + kGdCols - 1) / kGdCols);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ARLE_GD(T, DS)                                                                                               \
  do {                                                                                                               \
    if (channel) ARLE_GD_R(T, DS, true); else ARLE_GD_R(T, DS, false);                                               \
  } while (0)
#define ARLE_GD_R(T, DS, CH)                                                                                         \
  do {                                                                                                               \
    if (single_rows) ARLE_GD_L(T, DS, false, CH); else ARLE_GD_L(T, DS, true, CH);                                   \
  } while (0)
#define ARLE_GD_L(T, DS, ROWS, CH)                                                                                   \
  gated_delta_scan_kernel<T, DS, ROWS, CH><<<grid, kGdThreads, 0, s>>>(                                                \
      static_cast<const T*>(q), q_stride, static_cast<const T*>(k), k_stride, static_cast<const T*>(v), v_stride,    \
      static_cast<const float*>(beta_in), beta_stride, static_cast<const float*>(decay_in), decay_stride,            \
      static_cast<const float*>(a_log),                                                                              \
      static_cast<const float*>(dt_bias), unit_eps, static_cast<float*>(s_state), seg_row0, seg_slot,                \
      static_cast<float*>(out), H, G, D, Dv)
#define ARLE_GD_T(T)                                                                                                 \
  if (D <= 32) ARLE_GD(T, 2); else if (D <= 64) ARLE_GD(T, 4); else if (D <= 128) ARLE_GD(T, 8); else ARLE_GD(T, 16)
  if (dtype == kF32) { ARLE_GD_T(float); } else { ARLE_GD_T(bf16); }
#undef ARLE_GD_T
#undef ARLE_GD_L
#undef ARLE_GD_R
#undef ARLE_GD
  return launch_status();
}

extern "C" int arle_gated_delta_output(const void* o, const void* gate, long long gate_stride, int dtype,
                                       const void* weight, int w_dtype, float eps, void* out, int tokens, int H, int Dv,
                                       int act, void* stream) {
  if (tokens == 0) return 0;
  dim3 grid(tokens, H);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) {
    gated_delta_output_kernel<float><<<grid, kWave, 0, s>>>(static_cast<const float*>(o), static_cast<const float*>(gate),
                                                            gate_stride, weight, w_dtype, eps, static_cast<float*>(out), H, Dv, act);
  } else {
    gated_delta_output_kernel<bf16><<<grid, kWave, 0, s>>>(static_cast<const float*>(o), static_cast<const bf16*>(gate),
                                                           gate_stride, weight, w_dtype, eps, static_cast<bf16*>(out), H, Dv, act);
  }
  return launch_status();
}
