// Windowed causal attention over a paged cache whose scores are soft-capped and carry a logarithmic distance
// penalty, with key and value heads of different sizes, and the preparation of its operands.
//
//   s_ij = scale (q_i . k_j);   s <- cap tanh(s / cap)  (cap > 0);   s <- s - r1_h ln(1 + r2_h (i - j))  (r1 given)
//   o_i  = sum_j softmax_j(s_ij) v_j     over  max(0, i - window + 1) <= j <= i   (window 0: every earlier key)
//
// Two further options: `chunk` > 0 lets row i see only the keys of its own chunk, floor(i / chunk) chunk <= j <= i
// (chunks are counted from position 0 of the request); `sink` [heads] adds exp(sink_h) to the softmax's denominator,
// a term without key or value.  `wide_norm_store` prepares the operands of an attention whose q and k are RMS-normed
// over the whole projection (all heads at once) and whose values may be mixed with another layer's.
//
// q head h reads kv head h / (nq / nkv).  Keys lie in pages [page, nkv, slot, Dk], values d-major
// [page, nkv, Dv, slot].  Scores, the cap, the penalty, probabilities and sums are 32-bit.
//
// `qkv_norm_store`: per-head RMS norm of q and k (one weight of Dk for all heads, eps inside the root), the
// query temperature q <- q (1 + coef ln(floor((p + 1) / every) + 1)) at position p, and the write of k and v
// into the request's pages.  `attn_softcap_simt`: one wave a (row, q head), keys in tiles of 64 aligned to
// the absolute key index and walked in ascending order, so that a row's arithmetic depends on its position
// and window only: the true 32-bit path, and the plain counterpart of the matrix-core kernel below.
#include "common.h"

namespace arle {

constexpr int kCapMaxD = 1024;   // the widest head: a latent attention's keys are its latent and its rotated part together

// One wave a (row, head of q, k or v).  T: the element type of q, k, v and the pages; the loads of a head are typed and
// unconditional (an element past the head's size reads the head's last one and is dropped).
template <typename T>
__global__ __launch_bounds__(kWave) void qkv_norm_store_kernel(
    T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const void* __restrict__ q_weight, const void* __restrict__ k_weight, int w_dtype, float eps,
    float temp_coef, int temp_every, const int* __restrict__ positions, const int* __restrict__ slot_of_token,
    const int* __restrict__ block_table, int table_stride, T* __restrict__ k_pages, T* __restrict__ v_pages, int nq,
    int nkv, int Dk, int Dv, int page_size) {
  const int64_t t = blockIdx.x;
  const int y = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  if (y < nq + nkv) {
    const bool is_q = y < nq;
    const int g = is_q ? y : y - nq;
    const T* src = is_q ? q + t * q_stride + g * Dk : k + t * k_stride + g * Dk;
    const void* weight = is_q ? q_weight : k_weight;
    float x[kCapMaxD / kWave], w[kCapMaxD / kWave];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < Dk) {
        x[j] = to_float(src[min(d, Dk - 1)]);
        w[j] = weight ? load_as_float(weight, w_dtype, min(d, Dk - 1)) : 1.0f;
        if (d < Dk) ss = fmaf(x[j], x[j], ss);
      }
    }
    float f = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dk) + eps);
    T* dst;
    if (is_q) {
      if (temp_coef != 0.f) f *= 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every + 1));
      dst = q + t * q_stride + g * Dk;
    } else {
      const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
      dst = k_pages + ((static_cast<int64_t>(page) * nkv + g) * page_size + pos % page_size) * Dk;
    }
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (j * kWave < Dk && d < Dk) dst[d] = from_float<T>(x[j] * f * w[j]);
    }
    return;
  }
  const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
  const int g = y - nq - nkv;
  T* dst = v_pages + (static_cast<int64_t>(page) * nkv + g) * Dv * page_size + pos % page_size;
  for (int d = lane; d < Dv; d += kWave) dst[static_cast<int64_t>(d) * page_size] = v[t * v_stride + g * Dv + d];
}

template <typename T>
__global__ __launch_bounds__(kWave) void attn_softcap_simt_kernel(
    const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t o_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ block_table, int table_stride,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, int nq, int nkv, int Dk, int Dv,
    int page_size, float scale, float cap, const void* __restrict__ r1, const void* __restrict__ r2, int r_dtype,
    int window, int chunk, const void* __restrict__ sink, int sink_dtype, int keep_first) {
  extern __shared__ float qs[];  // [Dk]
  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int lane = threadIdx.x;
  const int kvh = h / (nq / nkv);
  const int pos = positions[t];
  const int* table = block_table + static_cast<int64_t>(slot_of_token[t]) * table_stride;
  const float pen1 = r1 ? load_as_float(r1, r_dtype, h) : 0.f;
  const float pen2 = r1 ? load_as_float(r2, r_dtype, h) : 0.f;
  const float inv_cap = cap > 0.f ? 1.0f / cap : 0.f;

  const T* qr = q + static_cast<int64_t>(t) * q_stride + h * Dk;
  for (int d = lane; d < Dk; d += kWave) qs[d] = to_float(qr[d]);
  __syncthreads();

  int first = window > 0 ? max(0, pos - window + 1) : 0;
  // the first `kept` keys of the request stay visible when the window has passed them (the chunk rule still holds)
  const int chunk_first = chunk > 0 ? pos / chunk * chunk : 0;
  first = max(first, chunk_first);
  const int kept = min(keep_first, first);              // keys [chunk_first, kept) and [first, pos] are seen
  const bool head_part = kept > chunk_first;
  const int64_t k_page = static_cast<int64_t>(nkv) * page_size * Dk, v_page = static_cast<int64_t>(nkv) * page_size * Dv;
  const int64_t k_head = static_cast<int64_t>(kvh) * page_size * Dk, v_head = static_cast<int64_t>(kvh) * page_size * Dv;

  float m = -INFINITY, l = 0.f;
  float acc[kCapMaxD / kWave];
#pragma unroll
  for (int i = 0; i < kCapMaxD / kWave; ++i) acc[i] = 0.f;

  for (int tile = head_part ? chunk_first / kWave : first / kWave; tile * kWave <= pos; ++tile) {
    if (head_part && tile * kWave >= kept && (tile + 1) * kWave <= first) {   // a tile between the two parts
      tile = first / kWave - 1;
      continue;
    }
    const int c = tile * kWave + lane;
    const bool valid = c <= pos && (c >= first || (head_part && c >= chunk_first && c < kept));
    float s = -INFINITY;
    if (valid) {
      const int page = table[c / page_size];
      const T* kr = k_pages + page * k_page + k_head + static_cast<int64_t>(c % page_size) * Dk;
      float dot = 0.f;
      for (int d = 0; d < Dk; ++d) dot = fmaf(qs[d], to_float(kr[d]), dot);
      s = dot * scale;
      if (cap > 0.f) s = cap * tanhf(s * inv_cap);
      if (r1) s -= pen1 * log1pf(pen2 * static_cast<float>(pos - c));
    }
    const float m_new = fmaxf(m, wave_max(s));  // the tile holds at least one visible key
    const float alpha = expf(m - m_new);        // 0 on the first tile (m = -inf)
    const float p = valid ? expf(s - m_new) : 0.f;
    l = l * alpha + wave_sum(p);
#pragma unroll
    for (int i = 0; i < kCapMaxD / kWave; ++i) acc[i] *= alpha;

    const int j_lo = max((head_part ? chunk_first : first) - tile * kWave, 0);
    const int j_hi = min(pos - tile * kWave, kWave - 1);
    for (int j = j_lo; j <= j_hi; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int cj = tile * kWave + j;
      if (cj < first && cj >= kept) continue;   // between the parts: a page that may have been given back
      const int page = table[cj / page_size];
      const T* vr = v_pages + page * v_page + v_head + (cj % page_size);  // [d][slot in page]
#pragma unroll
      for (int i = 0; i < kCapMaxD / kWave; ++i) {
        const int d = lane + i * kWave;
        if (d < Dv) acc[i] = fmaf(pj, to_float(vr[static_cast<int64_t>(d) * page_size]), acc[i]);
      }
    }
    m = m_new;
  }

  T* o = out + static_cast<int64_t>(t) * o_stride + h * Dv;
  float keep = 1.0f;
  if (sink) {  // one more term in the denominator, with no value behind it
    const float sk = load_as_float(sink, sink_dtype, h);
    const float m_all = fmaxf(m, sk);
    keep = expf(m - m_all);
    l = l * keep + expf(sk - m_all);
  }
  const float inv_l = keep / l;
#pragma unroll
  for (int i = 0; i < kCapMaxD / kWave; ++i) {
    const int d = lane + i * kWave;
    if (d < Dv) o[d] = from_float<T>(acc[i] * inv_l);
  }
}

// Operands of an attention that norms q and k over the whole projection.  One workgroup a (row, one of q, k, v):
//   q <- q / rms(q) * wq  in place over all nq * Dk entries (wq null: q stays as it is);
//   k likewise over all nkv * Dk entries, into the pages;
//   v <- (1 - lambda) v + lambda v_first (v_first given), into the pages (d-major).
// lambda is one number in memory, so that a captured launch reads the checkpoint's value.
constexpr int kWideThreads = 256;
template <typename T>
__global__ __launch_bounds__(kWideThreads) void wide_norm_store_kernel(
    T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const T* __restrict__ v_first, long long vf_stride, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int w_dtype, const void* __restrict__ lambda, int lambda_dtype, float eps,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, const int* __restrict__ block_table,
    int table_stride, T* __restrict__ k_pages, T* __restrict__ v_pages, int nq, int nkv, int Dk, int Dv, int page_size,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int halves) {
  extern __shared__ float staged[];   // [max(nq, nkv) * Dk] with a rotation, else nothing
  __shared__ float lds[kWideThreads / kWave];
  const int64_t t = blockIdx.x;
  const int what = blockIdx.y;
  const int pos = positions[t];
  // With a rotation the normed row waits in LDS, so that an entry's partner is read as it was before anything is
  // written: entry d < rot of a head turns with entry d ^ 1 (or, with `halves`, d +- rot / 2) by the angle of its pair.
  const int half = rot / 2;
  const float* cs = rot ? cos_t + static_cast<int64_t>(pos) * half : nullptr;
  const float* sn = rot ? sin_t + static_cast<int64_t>(pos) * half : nullptr;
  auto turned = [&](const float* head, int d) {
    const int partner = halves ? (d < half ? d + half : d - half) : (d ^ 1);
    const int pair = halves ? (d < half ? d : d - half) : d / 2;
    const bool second = halves ? d >= half : (d & 1);
    const float c = cs[pair], sv = sn[pair];
    return second ? fmaf(head[d], c, head[partner] * sv) : fmaf(head[d], c, -head[partner] * sv);
  };
  auto stage = [&](const T* row, int width, const void* weight) {   // the row, normed where it has a weight, into LDS
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kWideThreads) {
      const float x = to_float(row[i]);
      staged[i] = x;
      ss = fmaf(x, x, ss);
    }
    const float total = block_sum<kWideThreads / kWave>(ss, lds);   // (its barriers also order the writes above)
    if (weight) {
      const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
      for (int i = threadIdx.x; i < width; i += kWideThreads) staged[i] = staged[i] * inv * load_as_float(weight, w_dtype, i);
    }
    __syncthreads();
  };
  if (what == 0) {
    if (!q_weight && !rot) return;
    const int width = nq * Dk;
    T* row = q + t * q_stride;
    if (rot) {
      stage(row, width, q_weight);
      for (int i = threadIdx.x; i < width; i += kWideThreads) {
        const int d = i % Dk;
        row[i] = from_float<T>(d < rot ? turned(staged + (i - d), d) : staged[i]);
      }
      return;
    }
    float ss = 0.f;
    for (int i = threadIdx.x; i < width; i += kWideThreads) {
      const float x = to_float(row[i]);
      ss = fmaf(x, x, ss);
    }
    const float inv = 1.0f / sqrtf(block_sum<kWideThreads / kWave>(ss, lds) / static_cast<float>(width) + eps);
    for (int i = threadIdx.x; i < width; i += kWideThreads)
      row[i] = from_float<T>(to_float(row[i]) * inv * load_as_float(q_weight, w_dtype, i));
    return;
  }
  const int64_t page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
  const int in_page = pos % page_size;
  if (what == 1) {
    const int width = nkv * Dk;
    const T* row = k + t * k_stride;
    if (rot) {
      stage(row, width, k_weight);
      for (int i = threadIdx.x; i < width; i += kWideThreads) {
        const int g = i / Dk, d = i % Dk;
        k_pages[((page * nkv + g) * page_size + in_page) * Dk + d] =
            from_float<T>(d < rot ? turned(staged + (i - d), d) : staged[i]);
      }
      return;
    }
    float inv = 1.0f;
    if (k_weight) {
      float ss = 0.f;
      for (int i = threadIdx.x; i < width; i += kWideThreads) {
        const float x = to_float(row[i]);
        ss = fmaf(x, x, ss);
      }
      inv = 1.0f / sqrtf(block_sum<kWideThreads / kWave>(ss, lds) / static_cast<float>(width) + eps);
    }
    for (int i = threadIdx.x; i < width; i += kWideThreads) {
      const int g = i / Dk, d = i % Dk;
      const float x = to_float(row[i]);
      k_pages[((page * nkv + g) * page_size + in_page) * Dk + d] =
          k_weight ? from_float<T>(x * inv * load_as_float(k_weight, w_dtype, i)) : row[i];
    }
    return;
  }
  const int width = nkv * Dv;
  const float lam = v_first ? load_as_float(lambda, lambda_dtype, 0) : 0.f;
  for (int i = threadIdx.x; i < width; i += kWideThreads) {
    const int g = i / Dv, d = i % Dv;
    T x = v[t * v_stride + i];
    if (v_first) x = from_float<T>((1.0f - lam) * to_float(x) + lam * to_float(v_first[t * vf_stride + i]));
    v_pages[((page * nkv + g) * Dv + d) * page_size + in_page] = x;
  }
}

}  // namespace arle

using namespace arle;

// q [T, nq*Dk] is normed and scaled in place; k [T, nkv*Dk] and v [T, nkv*Dv] go to the pages (nkv 0: a layer
// that reads another layer's pages and only prepares q).  q_weight, k_weight: [Dk] or null.
extern "C" int arle_qkv_norm_store(void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                                   long long v_stride, int dtype, const void* q_weight, const void* k_weight,
                                   int w_dtype, float eps, float temp_coef, int temp_every, const int* positions,
                                   const int* slot_of_token, const int* block_table, int table_stride, void* k_pages,
                                   void* v_pages, int tokens, int nq, int nkv, int Dk, int Dv, int page_size,
                                   void* stream) {
  if (tokens == 0) return 0;
  if (Dk > kCapMaxD || Dk < 1 || nq + 2 * nkv > 65535 || (temp_coef != 0.f && temp_every < 1))
    return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(tokens, nq + 2 * nkv);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kF32) {
    qkv_norm_store_kernel<float><<<grid, kWave, 0, s>>>(
        static_cast<float*>(q), q_stride, static_cast<const float*>(k), k_stride, static_cast<const float*>(v), v_stride,
        q_weight, k_weight, w_dtype, eps, temp_coef, temp_every, positions, slot_of_token, block_table, table_stride,
        static_cast<float*>(k_pages), static_cast<float*>(v_pages), nq, nkv, Dk, Dv, page_size);
  } else {
    qkv_norm_store_kernel<bf16><<<grid, kWave, 0, s>>>(
        static_cast<bf16*>(q), q_stride, static_cast<const bf16*>(k), k_stride, static_cast<const bf16*>(v), v_stride,
        q_weight, k_weight, w_dtype, eps, temp_coef, temp_every, positions, slot_of_token, block_table, table_stride,
        static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), nq, nkv, Dk, Dv, page_size);
  }
  return launch_status();
}

// q [T, nq*Dk], out [T, nq*Dv] of `dtype`, as the pages.  cap 0: no soft cap.  r1, r2: [nq] or null.
extern "C" int arle_attn_softcap_simt(const void* q, long long q_stride, void* out, long long o_stride,
                                      const void* k_pages, const void* v_pages, int dtype, const int* block_table,
                                      int table_stride, const int* positions, const int* slot_of_token, int tokens,
                                      int nq, int nkv, int Dk, int Dv, int page_size, float scale, float cap,
                                      const void* r1, const void* r2, int r_dtype, int window, int chunk,
                                      const void* sink, int sink_dtype, int keep_first, void* stream) {
  if (tokens == 0) return 0;
  if (Dk > kCapMaxD || Dv > kCapMaxD || nkv < 1 || nq % nkv != 0 || nq > 65535 || window < 0 || chunk < 0 ||
      keep_first < 0 || (keep_first > 0 && window == 0))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(tokens, nq);
  const size_t lds = static_cast<size_t>(Dk) * sizeof(float);
  if (dtype == kF32) {
    attn_softcap_simt_kernel<float><<<grid, kWave, lds, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out), o_stride, static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), block_table, table_stride, positions, slot_of_token, nq, nkv, Dk, Dv,
        page_size, scale, cap, r1, r2, r_dtype, window, chunk, sink, sink_dtype, keep_first);
  } else {
    attn_softcap_simt_kernel<bf16><<<grid, kWave, lds, s>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), o_stride, static_cast<const bf16*>(k_pages),
        static_cast<const bf16*>(v_pages), block_table, table_stride, positions, slot_of_token, nq, nkv, Dk, Dv,
        page_size, scale, cap, r1, r2, r_dtype, window, chunk, sink, sink_dtype, keep_first);
  }
  return launch_status();
}

// q [T, nq*Dk] is normed in place over the whole row (q_weight [nq*Dk] or null); k [T, nkv*Dk] is normed likewise
// (k_weight [nkv*Dk] or null) and goes to the pages; v [T, nkv*Dv], mixed with v_first by *lambda where v_first is
// given, goes to the pages.  rot > 0: behind the norm the first `rot` entries of every head of q and k turn by the
// angles of float32 tables cos, sin [positions, rot / 2]; halves != 0 pairs entry i with i + rot / 2, else 2i with 2i + 1.
extern "C" int arle_wide_norm_store(void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                                    long long v_stride, const void* v_first, long long vf_stride, int dtype,
                                    const void* q_weight, const void* k_weight, int w_dtype, const void* lambda,
                                    int lambda_dtype, float eps, const int* positions, const int* slot_of_token,
                                    const int* block_table, int table_stride, void* k_pages, void* v_pages, int tokens,
                                    int nq, int nkv, int Dk, int Dv, int page_size, const float* cos_t,
                                    const float* sin_t, int rot, int halves, void* stream) {
  if (tokens == 0) return 0;
  if (nq < 1 || nkv < 1 || Dk < 1 || Dv < 1 || page_size < 1 || (v_first && !lambda) || rot < 0 || rot > Dk || rot % 2 ||
      (rot && (!cos_t || !sin_t)))
    return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid(tokens, 3);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t staged_bytes = rot ? static_cast<size_t>(nq > nkv ? nq : nkv) * Dk * sizeof(float) : 0;
  if (staged_bytes > 64 * 1024) return static_cast<int>(hipErrorInvalidValue);
  if (staged_bytes > 48 * 1024) {
    static bool raised = false;
    if (!raised) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&wide_norm_store_kernel<float>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
      if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void*>(&wide_norm_store_kernel<bf16>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
      if (e != hipSuccess) return static_cast<int>(e);
      raised = true;
    }
  }
  if (dtype == kF32) {
    wide_norm_store_kernel<float><<<grid, kWideThreads, staged_bytes, s>>>(
        static_cast<float*>(q), q_stride, static_cast<const float*>(k), k_stride, static_cast<const float*>(v), v_stride,
        static_cast<const float*>(v_first), vf_stride, q_weight, k_weight, w_dtype, lambda, lambda_dtype, eps, positions,
        slot_of_token, block_table, table_stride, static_cast<float*>(k_pages), static_cast<float*>(v_pages), nq, nkv, Dk,
        Dv, page_size, cos_t, sin_t, rot, halves);
  } else {
    wide_norm_store_kernel<bf16><<<grid, kWideThreads, staged_bytes, s>>>(
        static_cast<bf16*>(q), q_stride, static_cast<const bf16*>(k), k_stride, static_cast<const bf16*>(v), v_stride,
        static_cast<const bf16*>(v_first), vf_stride, q_weight, k_weight, w_dtype, lambda, lambda_dtype, eps, positions,
        slot_of_token, block_table, table_stride, static_cast<bf16*>(k_pages), static_cast<bf16*>(v_pages), nq, nkv, Dk,
        Dv, page_size, cos_t, sin_t, rot, halves);
  }
  return launch_status();
}

// ---- matrix-core kernel (bfloat16) ------------------------------------------------------------
// One wave a work item of sixteen queries that share a kv head: sixteen consecutive rows of one request for one
// q head (prompt portions), or one decoded row for the up to sixteen q heads of a kv head.  The scores are
// computed transposed, S^T[key][query] = K . Q^T with `v_mfma_f32_16x16x32_bf16`, so that a lane holds, for its
// query (lane % 16), the keys 4g..4g+3 (g = lane / 16) of each sixteen-key half of a tile of 32 keys: the cap, the
// penalty, the mask and the running softmax are per-lane arithmetic plus two lane exchanges, and the eight
// probabilities of a lane are, as they lie, the B operand of the second product O^T += V^T . P^T once the keys of
// the tile are taken in the order (4g..4g+3 of the first half, 4g..4g+3 of the second) on the V side too, which is
// two 8-byte loads from the d-major value pages.  A half tile is sixteen slots of one page (page sizes are
// multiples of 16).  Pages that a window has passed (entry -1) and slots beyond the newest key are never visible;
// their keys are masked by a select and their values replaced by zeros, so that stale bits cannot reach a sum.
namespace arle {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));

// tanh through one exponential and the hardware's reciprocal (a division in full would be a dozen instructions a score)
__device__ __forceinline__ float fast_tanh(float x) {
  return fmaf(-2.0f, __builtin_amdgcn_rcpf(1.0f + __expf(2.0f * x)), 1.0f);
}

// Portions do not fetch a tile ahead: with thousands of waves, more of them a SIMD hide the loads better than a second
// set of registers (2,048 rows behind a window of 1,024: 213 us a layer without, 288 with).
constexpr bool kCapRowsAhead = false;

struct CapArgs {
  const bf16* q; long long q_stride;
  bf16* out; long long o_stride;
  const bf16* k_pages; const bf16* v_pages;
  const int* block_table; int table_stride;
  const int* seg_row0; const int* seg_slot; const int* seg_start;
  int segments, nq, nkv, Dk, Dv, page_size;
  float scale, cap;
  const void* r1; const void* r2; int r_dtype;
  int window;
  int chunk;                          // 0: none; else a row sees only the keys of its own chunk of so many positions
  const void* sink; int sink_dtype;   // [nq] or null: exp(sink_h) joins the softmax's denominator
  int merge_floats;   // floats of dynamic LDS in front of the page ids
  int keep_first;     // with a window: the request's first so many keys stay visible behind it (0: none)
};

// KC: chunks of 32 of the key size held (Dk <= 32 KC); VC: chunks of 16 of the value size (Dv <= 16 VC).
// HEADS: a work item is one row (a segment of one row) and the q heads of a kv head, and the WAVES waves of the
// workgroup take its tiles of keys in turn and add their sums through LDS; else an item is sixteen rows of one q head,
// and the waves of a workgroup are WAVES q heads of one kv head on the same rows, so that they fetch the same tiles.
// (Portions of heads up to 128 are asked to fit three waves a SIMD: the kernel waits for its loads, and 163 registers
// hold what 202 held; with larger heads, or four waves, the compiler would spill.)
template <int KC, int VC, bool HEADS, int WAVES>
__global__ __launch_bounds__(WAVES * kWave) __attribute__((amdgpu_waves_per_eu(!HEADS && KC <= 4 && VC <= 8 ? 3 : 1)))
void attn_softcap_mfma_kernel(const CapArgs a) {
  extern __shared__ float merge_lds[];   // HEADS: [WAVES][n_vc][64 lanes][4], then m [WAVES][16], l [WAVES][16]; then page ids
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave, n = lane % 16, g = lane / 16;
  const int group = a.nq / a.nkv;
  int seg, row, head, kvh, first_row, last_row;
  bool live;
  if (HEADS) {
    // a kv head with more than sixteen q heads is taken by several workgroups, sixteen q heads each
    const int parts = (group + 15) / 16, part = blockIdx.y % parts;
    seg = blockIdx.x;
    kvh = blockIdx.y / parts;
    row = first_row = last_row = a.seg_row0[seg];
    head = kvh * group + min(16 * part + n, group - 1);
    live = 16 * part + n < group;
  } else {
    // Workgroups go to the chip's eight dies in turn (the launch order is blockIdx.x fastest), and every die has a
    // level-two cache of its own: with the head groups a multiple of eight, die i takes the head groups i, i + 8, ...
    // with all their row blocks, so that it keeps the keys and values of its own kv heads and not everybody's.
    int bx = blockIdx.x, by = blockIdx.y;
    if (gridDim.y % 8 == 0) {
      const unsigned linear = blockIdx.y * gridDim.x + blockIdx.x, die = linear % 8, within = linear / 8;
      by = die + 8 * (within / gridDim.x);
      bx = within % gridDim.x;
    }
    // the bx-th block of sixteen rows, counted through the segments
    int left = bx, found = -1;
    for (int s = 0; s < a.segments; ++s) {
      const int blocks = (a.seg_row0[s + 1] - a.seg_row0[s] + 15) / 16;
      if (left < blocks) {
        found = s;
        break;
      }
      left -= blocks;
    }
    if (found < 0) return;
    seg = found;
    head = by * WAVES + wave;
    kvh = head / group;
    const int end = a.seg_row0[seg + 1];
    first_row = a.seg_row0[seg] + left * 16;
    last_row = min(first_row + 15, end - 1);
    live = first_row + n < end;
    row = min(first_row + n, end - 1);
  }
  const int seg_first = a.seg_row0[seg];
  const int pos = a.seg_start[seg] + (row - seg_first);
  // keys that any query of the item sees: from the first row's window to the last row's own position
  const int pos_lo = a.seg_start[seg] + (first_row - seg_first);
  const int pos_hi = a.seg_start[seg] + (last_row - seg_first);
  auto first_seen = [&](int p) {
    int lo = a.window > 0 ? max(0, p - a.window + 1) : 0;
    if (a.chunk > 0) lo = max(lo, p / a.chunk * a.chunk);
    return lo;
  };
  const int key_lo = first_seen(pos_lo);
  const int my_lo = first_seen(pos);
  // The request's first `keep` keys stay visible to rows whose window has passed them.  Their tiles of 32 keys that
  // lie wholly in front of the first tile of the windows are `head_tiles` tiles of their own, walked first; the walk
  // counts tiles through both parts (`walk` 0 .. walk_last), and `tile_of` gives the tile of keys behind a count.
  const int keep = a.keep_first;
  const int head_tiles = min((keep + 31) / 32, key_lo / 32);
  const int main_first = key_lo / 32;
  auto tile_of = [&](int walk) { return walk < head_tiles ? walk : walk - head_tiles + main_first; };
  const float sink = a.sink ? load_as_float(a.sink, a.sink_dtype, head) : -INFINITY;
  const int* table = a.block_table + static_cast<int64_t>(a.seg_slot[seg]) * a.table_stride;
  const float pen1 = a.r1 ? load_as_float(a.r1, a.r_dtype, head) : 0.f;
  const float pen2 = a.r1 ? load_as_float(a.r2, a.r_dtype, head) : 0.f;
  const float inv_cap = a.cap > 0.f ? 1.0f / a.cap : 0.f;
  const int n_kc = (a.Dk + 31) / 32, n_vc = a.Dv / 16;

  // Q^T operand: for chunk c, Q[row][32 c + 8 g .. + 7]
  bf16x8_t qreg[KC];
  const bf16* qr = a.q + static_cast<int64_t>(row) * a.q_stride + head * a.Dk;
#pragma unroll
  for (int c = 0; c < KC; ++c) {
    const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(qr + min(32 * c + 8 * g, a.Dk - 8));
    qreg[c] = __builtin_bit_cast(bf16x8_t, 32 * c + 8 * g < a.Dk ? raw : u32x4_t{0, 0, 0, 0});
  }
  f32x4_t acc[VC];
#pragma unroll
  for (int c = 0; c < VC; ++c) acc[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;

  const int64_t k_page = static_cast<int64_t>(a.nkv) * a.page_size * a.Dk, v_page = static_cast<int64_t>(a.nkv) * a.page_size * a.Dv;
  const int64_t k_head = static_cast<int64_t>(kvh) * a.page_size * a.Dk, v_head = static_cast<int64_t>(kvh) * a.page_size * a.Dv;
  const int tile_step = HEADS ? WAVES : 1;
  const int tile_first = HEADS ? wave : 0;                                   // counts of the walk
  const int tile_last = head_tiles + pos_hi / 32 - main_first, last_entry = a.table_stride - 1;

  // Every load of a tile (K rows, V columns, after the two page ids) is sent a tile ahead, while the tile before it
  // is worked through; a tile past the last is the last one again, fetched and dropped.
  // The ids of the pages that the item sees are put into LDS once: a tile's loads then follow no load of a page id,
  // and the reads of LDS are counted apart from the loads from memory, so they disturb no wait for those.
  const int page_first = (key_lo / 32 * 32) / a.page_size;   // the page of the first tile's first key, which may lie in front of key_lo's
  // (the ids of the head tiles' pages, the request's first ones, lie in front of them)
  const int head_pages = head_tiles > 0 ? (head_tiles * 32 + a.page_size - 1) / a.page_size : 0;
  int* head_lds = reinterpret_cast<int*>(merge_lds) + a.merge_floats;
  int* page_lds = head_lds + head_pages;
  for (int i = threadIdx.x; i < head_pages; i += WAVES * kWave) head_lds[i] = table[min(i, last_entry)];
  for (int i = threadIdx.x; i <= (pos_hi / 32 * 32 + 31) / a.page_size - page_first; i += WAVES * kWave)
    page_lds[i] = table[min(page_first + i, last_entry)];
  __syncthreads();
  auto load_tile = [&](int walk, u32x4_t (&kraw)[2][KC], u32x4_t (&vraw)[VC]) {
    const int at = min(walk, tile_last);
    const int key0 = tile_of(at) * 32;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      const int kb = key0 + 16 * half;
      const int64_t page = max(at < head_tiles ? head_lds[kb / a.page_size] : page_lds[max(kb / a.page_size - page_first, 0)], 0);
      const int in_page = kb % a.page_size;
      const bf16* kr = a.k_pages + page * k_page + k_head + static_cast<int64_t>(in_page + n) * a.Dk;
      // no load stands under a condition (one would make every later wait a wait for all loads in flight): a piece
      // past the head's size is the head's last piece again, zeroed or left unused afterwards
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const u32x4_t raw = *reinterpret_cast<const u32x4_t*>(kr + min(32 * c + 8 * g, a.Dk - 8));
        kraw[half][c] = 32 * c + 8 * g < a.Dk ? raw : u32x4_t{0, 0, 0, 0};
      }
#pragma unroll
      for (int c = 0; c < VC; ++c) {
        const bf16* vr = a.v_pages + page * v_page + v_head + static_cast<int64_t>(min(16 * c + n, a.Dv - 1)) * a.page_size +
                         in_page + 4 * g;
        const u32x2_t two = *reinterpret_cast<const u32x2_t*>(vr);
        vraw[c][2 * half] = two[0];
        vraw[c][2 * half + 1] = two[1];
      }
    }
  };

  auto work_tile = [&](int walk, const u32x4_t (&kraw)[2][KC], const u32x4_t (&vraw)[VC]) {
    const int key0 = tile_of(walk) * 32;
    float s[8];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      // S^T half tile: A = K[key kb + n][32 c + 8 g ..], B = Q^T
      f32x4_t z = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; ++c)
        if (c < n_kc) z = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, kraw[half][c]), qreg[c], z, 0, 0, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = key0 + 16 * half + 4 * g + i;
        float v = z[i] * a.scale;
        if (a.cap > 0.f) v = a.cap * fast_tanh(v * inv_cap);
        if (a.r1) v -= pen1 * __logf(1.0f + pen2 * static_cast<float>(pos - key));
        s[4 * half + i] = ((key >= my_lo || key < keep) && key <= pos) ? v : -INFINITY;
      }
    }
    float m_new = m_run;
#pragma unroll
    for (int i = 0; i < 8; ++i) m_new = fmaxf(m_new, s[i]);
    m_new = fmaxf(m_new, __shfl_xor(m_new, 16, kWave));
    m_new = fmaxf(m_new, __shfl_xor(m_new, 32, kWave));
    // a query whose window begins behind this tile has seen nothing yet: keep its sums at zero without 0 * inf
    const float m_safe = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __expf(m_run - m_safe);
    float p[8], sum = 0.f;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      p[i] = __expf(s[i] - m_safe);
      sum += p[i];
    }
    sum += __shfl_xor(sum, 16, kWave);
    sum += __shfl_xor(sum, 32, kWave);
    l_run = l_run * alpha + sum;
    m_run = m_new;
    u32x4_t pb;
    pb[0] = pack_bf16x2(p[0], p[1]);
    pb[1] = pack_bf16x2(p[2], p[3]);
    pb[2] = pack_bf16x2(p[4], p[5]);
    pb[3] = pack_bf16x2(p[6], p[7]);
    const bf16x8_t pop = __builtin_bit_cast(bf16x8_t, pb);
    // which of this lane's eight key slots hold written keys (those between the item's first and last key, and the
    // kept first ones)
    const bool edge = key0 < key_lo || key0 + 31 > pos_hi;
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      if (c < n_vc) {
        u32x4_t vr = vraw[c];
        if (edge) {
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            const int key = key0 + 16 * (j / 4) + 4 * g + j % 4;
            if ((key < key_lo && key >= keep) || key > pos_hi) vr[j / 2] &= (j % 2) ? 0x0000ffffu : 0xffff0000u;
          }
        }
        f32x4_t o = acc[c];
        o[0] *= alpha; o[1] *= alpha; o[2] *= alpha; o[3] *= alpha;
        acc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, vr), pop, o, 0, 0, 0);
      }
    }
  };

  // (with keys of more than 128 and values of more than 128 a second set of tile registers no longer fits a wave's
  // registers: a decoded row behind 1,024 keys of 256 took 144 us with it)
  if ((HEADS || kCapRowsAhead) && 2 * KC + VC <= 24) {
    // a decoded row's waves are few and each walks a chain of tiles: the next tile's loads fly while this one is worked
    u32x4_t k_even[2][KC], v_even[VC], k_odd[2][KC], v_odd[VC];
    if (tile_first <= tile_last) load_tile(tile_first, k_even, v_even);
    for (int tile = tile_first; tile <= tile_last; tile += 2 * tile_step) {
      load_tile(tile + tile_step, k_odd, v_odd);
      work_tile(tile, k_even, v_even);
      if (tile + tile_step > tile_last) break;
      load_tile(tile + 2 * tile_step, k_even, v_even);
      work_tile(tile + tile_step, k_odd, v_odd);
    }
  } else {
    u32x4_t k_now[2][KC], v_now[VC];
    for (int tile = tile_first; tile <= tile_last; tile += tile_step) {
      load_tile(tile, k_now, v_now);
      work_tile(tile, k_now, v_now);
    }
  }

  if (HEADS && WAVES > 1) {
    // the waves' sums meet in LDS; wave w then finishes the chunks w, w + WAVES, ... of the value size
    f32x4_t* part = reinterpret_cast<f32x4_t*>(merge_lds);
    float* part_m = merge_lds + WAVES * n_vc * kWave * 4;
    float* part_l = part_m + WAVES * 16;
#pragma unroll
    for (int c = 0; c < VC; ++c)
      if (c < n_vc) part[(wave * n_vc + c) * kWave + lane] = acc[c];
    if (g == 0) {
      part_m[wave * 16 + n] = m_run;
      part_l[wave * 16 + n] = l_run;
    }
    __syncthreads();
    float m_all = sink;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) m_all = fmaxf(m_all, part_m[w * 16 + n]);
    float l_all = a.sink ? __expf(sink - m_all) : 0.f, f[WAVES];
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      f[w] = __expf(part_m[w * 16 + n] - m_all);
      l_all += part_l[w * 16 + n] * f[w];
    }
    if (!live) return;
    const float inv_l = 1.0f / l_all;
    bf16* orow = a.out + static_cast<int64_t>(row) * a.o_stride + head * a.Dv;
    for (int c = wave; c < n_vc; c += WAVES) {
      f32x4_t o = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        const f32x4_t t = part[(w * n_vc + c) * kWave + lane];
        o[0] += t[0] * f[w]; o[1] += t[1] * f[w]; o[2] += t[2] * f[w]; o[3] += t[3] * f[w];
      }
      u32x2_t packed;
      packed[0] = pack_bf16x2(o[0] * inv_l, o[1] * inv_l);
      packed[1] = pack_bf16x2(o[2] * inv_l, o[3] * inv_l);
      *reinterpret_cast<u32x2_t*>(orow + 16 * c + 4 * g) = packed;
    }
    return;
  }
  if (!live) return;
  float inv_l = 1.0f / l_run;
  if (a.sink) {
    const float m_all = fmaxf(m_run, sink), keep = __expf(m_run - m_all);
    inv_l = keep / (l_run * keep + __expf(sink - m_all));
  }
  bf16* orow = a.out + static_cast<int64_t>(row) * a.o_stride + head * a.Dv;
#pragma unroll
  for (int c = 0; c < VC; ++c) {
    if (c < n_vc) {
      u32x2_t packed;
      packed[0] = pack_bf16x2(acc[c][0] * inv_l, acc[c][1] * inv_l);
      packed[1] = pack_bf16x2(acc[c][2] * inv_l, acc[c][3] * inv_l);
      *reinterpret_cast<u32x2_t*>(orow + 16 * c + 4 * g) = packed;
    }
  }
}

constexpr int kCapSplitWaves = 8;   // waves that share the keys of a decoded row
constexpr int kCapLdsMost = 160 * 1024;   // LDS of a gfx950 compute unit: no workgroup can ask for more

// What a workgroup may ask for on this device (never more than kCapLdsMost), asked once.
inline int cap_lds_limit() {
  static int limit = 0;
  if (limit == 0) {
    int dev = 0, value = 0;
    if (hipGetDevice(&dev) == hipSuccess &&
        hipDeviceGetAttribute(&value, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && value > 0)
      limit = value < kCapLdsMost ? value : kCapLdsMost;
    else
      limit = 64 * 1024;
  }
  return limit;
}

}  // namespace arle

// Bytes of LDS that a workgroup of the matrix-core kernel may use on this device (the return value, not an error code).
extern "C" int arle_attn_softcap_lds_limit() { return cap_lds_limit(); }

// bfloat16 only.  Dk a multiple of 8 up to 256, Dv a multiple of 16 up to 256, page_size a multiple of 16, rows of
// q and out 16-byte aligned (strides multiples of 8).  heads_mode: every segment is one row.
// row_blocks: an upper bound of the sixteen-row blocks of all segments (blocks past the last one return).
extern "C" int arle_attn_softcap_mfma(const void* q, long long q_stride, void* out, long long o_stride,
                                      const void* k_pages, const void* v_pages, const int* block_table,
                                      int table_stride, const int* seg_row0, const int* seg_slot, const int* seg_start,
                                      int segments, int row_blocks, int heads_mode, int nq, int nkv, int Dk, int Dv,
                                      int page_size, float scale, float cap, const void* r1, const void* r2,
                                      int r_dtype, int window, int chunk, const void* sink, int sink_dtype,
                                      int keep_first, void* stream) {
  if (segments == 0) return 0;
  // (kept first keys go with a window alone: under the chunk rule a row's chunk would have to hold them)
  if (Dk % 8 || Dk > 256 || Dv % 16 || Dv > 256 || page_size % 16 || nkv < 1 || nq % nkv || nq > 65535 ||
      window < 0 || chunk < 0 || keep_first < 0 || (keep_first > 0 && (window == 0 || chunk > 0)))
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const CapArgs a{static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), o_stride,
                  static_cast<const bf16*>(k_pages), static_cast<const bf16*>(v_pages), block_table, table_stride,
                  seg_row0, seg_slot, seg_start, segments, nq, nkv, Dk, Dv, page_size, scale, cap, r1, r2, r_dtype, window,
                  chunk, sink, sink_dtype, heads_mode ? kCapSplitWaves * ((Dv / 16) * kWave * 4 + 32) : 0, keep_first};
  // pages an item can see: its rows' windows (or everything the block table maps) and the tiles' rounding to 32 keys;
  // nothing of a step's lengths, so that a captured launch holds for every later step of its shape
  const long long mapped = static_cast<long long>(table_stride) * page_size;
  const int span = window > 0 && chunk > 0 ? (window < chunk ? window : chunk) : (window > 0 ? window : chunk);
  const long long keys_seen = (span > 0 && span + 16 < mapped ? span + 16 : mapped) + 64;
  const size_t page_bytes = (static_cast<size_t>(keys_seen) / page_size + 2 + (keep_first + 31) / page_size + 2) * sizeof(int);
  if (page_bytes > 48 * 1024) return static_cast<int>(hipErrorInvalidValue);
  const int size = (Dk + 1) / 2 > Dv ? (Dk + 1) / 2 : Dv;   // Dk counts half: a chunk of keys is 32 wide, of values 16
  const int group = nq / nkv;
  const int head_waves = group % 4 == 0 ? 4 : (group % 2 == 0 ? 2 : 1);   // q heads of one kv head that share a workgroup
  const size_t merge_bytes = static_cast<size_t>(kCapSplitWaves) * ((Dv / 16) * kWave * 4 + 32) * sizeof(float) + page_bytes;
  if (heads_mode && merge_bytes > static_cast<size_t>(cap_lds_limit())) return static_cast<int>(hipErrorInvalidValue);
#define ARLE_CAP(KC, VC)                                                                                           \
  do {                                                                                                             \
    if (heads_mode) {                                                                                              \
      static bool raised = false;   /* more LDS than a launch gets unasked: said once for the kernel */            \
      if (!raised && merge_bytes > 48 * 1024) {                                                                    \
        const int most = kCapSplitWaves * (VC * kWave * 4 + 32) * 4 + 48 * 1024;                                   \
        const hipError_t e = hipFuncSetAttribute(                                                                  \
            reinterpret_cast<const void*>(&attn_softcap_mfma_kernel<KC, VC, true, kCapSplitWaves>),                \
            hipFuncAttributeMaxDynamicSharedMemorySize, most < cap_lds_limit() ? most : cap_lds_limit());              \
        if (e != hipSuccess) return static_cast<int>(e);                                                           \
        raised = true;                                                                                             \
      }                                                                                                            \
      attn_softcap_mfma_kernel<KC, VC, true, kCapSplitWaves>                                                       \
          <<<dim3(segments, nkv * ((group + 15) / 16)), kCapSplitWaves * kWave, merge_bytes, s>>>(a);                                    \
    }                                                                                                              \
    else if (head_waves == 4)                                                                                      \
      attn_softcap_mfma_kernel<KC, VC, false, 4><<<dim3(row_blocks, nq / 4), 4 * kWave, page_bytes, s>>>(a);                \
    else if (head_waves == 2)                                                                                      \
      attn_softcap_mfma_kernel<KC, VC, false, 2><<<dim3(row_blocks, nq / 2), 2 * kWave, page_bytes, s>>>(a);                \
    else                                                                                                           \
      attn_softcap_mfma_kernel<KC, VC, false, 1><<<dim3(row_blocks, nq), kWave, page_bytes, s>>>(a);                        \
  } while (0)
  if (size <= 64) {
    ARLE_CAP(4, 4);
  } else if (Dk <= 128 && Dv <= 128) {
    ARLE_CAP(4, 8);
  } else if (size <= 128) {
    ARLE_CAP(8, 8);
  } else if (Dv <= 192) {
    ARLE_CAP(8, 12);
  } else {
    ARLE_CAP(8, 16);
  }
#undef ARLE_CAP
  return launch_status();
}
