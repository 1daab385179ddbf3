// Windowed causal attention over a paged cache whose scores are soft-capped and carry a logarithmic distance
// penalty, with key and value heads of different sizes, and the preparation of its operands.
//
//   s_ij = scale (q_i . k_j);   s <- cap tanh(s / cap)  (cap > 0);   s <- s - r1_h ln(1 + r2_h (i - j))  (r1 given)
//   o_i  = sum_j softmax_j(s_ij) v_j     over  max(0, i - window + 1) <= j <= i   (window 0: every earlier key)
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

constexpr int kCapMaxD = 512;

__global__ __launch_bounds__(kWave) void qkv_norm_store_kernel(
    void* __restrict__ q, long long q_stride, const void* __restrict__ k, long long k_stride,
    const void* __restrict__ v, long long v_stride, int dtype, const void* __restrict__ q_weight,
    const void* __restrict__ k_weight, int w_dtype, float eps, float temp_coef, int temp_every,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, const int* __restrict__ block_table,
    int table_stride, void* __restrict__ k_pages, void* __restrict__ v_pages, int nq, int nkv, int Dk, int Dv,
    int page_size) {
  const int64_t t = blockIdx.x;
  const int y = blockIdx.y, lane = threadIdx.x;
  const int pos = positions[t];
  if (y < nq) {
    float x[kCapMaxD / kWave];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      x[j] = d < Dk ? load_as_float(q, dtype, t * q_stride + y * Dk + d) : 0.f;
      ss = fmaf(x[j], x[j], ss);
    }
    float f = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dk) + eps);
    const float temp = temp_coef != 0.f ? 1.0f + temp_coef * logf(static_cast<float>((pos + 1) / temp_every + 1)) : 1.0f;
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (d < Dk) {
        const float w = q_weight ? load_as_float(q_weight, w_dtype, d) : 1.0f;
        store_from_float(q, dtype, t * q_stride + y * Dk + d, x[j] * f * w * temp);
      }
    }
    return;
  }
  const int page = block_table[static_cast<int64_t>(slot_of_token[t]) * table_stride + pos / page_size];
  const int in_page = pos % page_size;
  if (y < nq + nkv) {
    const int g = y - nq;
    float x[kCapMaxD / kWave];
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      x[j] = d < Dk ? load_as_float(k, dtype, t * k_stride + g * Dk + d) : 0.f;
      ss = fmaf(x[j], x[j], ss);
    }
    const float f = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dk) + eps);
    const int64_t base = ((static_cast<int64_t>(page) * nkv + g) * page_size + in_page) * Dk;
#pragma unroll
    for (int j = 0; j < kCapMaxD / kWave; ++j) {
      const int d = lane + j * kWave;
      if (d < Dk) {
        const float w = k_weight ? load_as_float(k_weight, w_dtype, d) : 1.0f;
        store_from_float(k_pages, dtype, base + d, x[j] * f * w);
      }
    }
    return;
  }
  const int g = y - nq - nkv;
  const int64_t base = (static_cast<int64_t>(page) * nkv + g) * Dv * page_size + in_page;
  for (int d = lane; d < Dv; d += kWave)
    store_from_float(v_pages, dtype, base + static_cast<int64_t>(d) * page_size,
                     load_as_float(v, dtype, t * v_stride + g * Dv + d));
}

template <typename T>
__global__ __launch_bounds__(kWave) void attn_softcap_simt_kernel(
    const T* __restrict__ q, int64_t q_stride, T* __restrict__ out, int64_t o_stride, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, const int* __restrict__ block_table, int table_stride,
    const int* __restrict__ positions, const int* __restrict__ slot_of_token, int nq, int nkv, int Dk, int Dv,
    int page_size, float scale, float cap, const void* __restrict__ r1, const void* __restrict__ r2, int r_dtype,
    int window) {
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

  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  const int64_t k_page = static_cast<int64_t>(nkv) * page_size * Dk, v_page = static_cast<int64_t>(nkv) * page_size * Dv;
  const int64_t k_head = static_cast<int64_t>(kvh) * page_size * Dk, v_head = static_cast<int64_t>(kvh) * page_size * Dv;

  float m = -INFINITY, l = 0.f;
  float acc[kCapMaxD / kWave];
#pragma unroll
  for (int i = 0; i < kCapMaxD / kWave; ++i) acc[i] = 0.f;

  for (int tile = first / kWave; tile * kWave <= pos; ++tile) {
    const int c = tile * kWave + lane;
    const bool valid = c >= first && c <= pos;
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

    const int j_lo = max(first - tile * kWave, 0);
    const int j_hi = min(pos - tile * kWave, kWave - 1);
    for (int j = j_lo; j <= j_hi; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int cj = tile * kWave + j;
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
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int i = 0; i < kCapMaxD / kWave; ++i) {
    const int d = lane + i * kWave;
    if (d < Dv) o[d] = from_float<T>(acc[i] * inv_l);
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
  qkv_norm_store_kernel<<<dim3(tokens, nq + 2 * nkv), kWave, 0, static_cast<hipStream_t>(stream)>>>(
      q, q_stride, k, k_stride, v, v_stride, dtype, q_weight, k_weight, w_dtype, eps, temp_coef, temp_every, positions,
      slot_of_token, block_table, table_stride, k_pages, v_pages, nq, nkv, Dk, Dv, page_size);
  return launch_status();
}

// q [T, nq*Dk], out [T, nq*Dv] of `dtype`, as the pages.  cap 0: no soft cap.  r1, r2: [nq] or null.
extern "C" int arle_attn_softcap_simt(const void* q, long long q_stride, void* out, long long o_stride,
                                      const void* k_pages, const void* v_pages, int dtype, const int* block_table,
                                      int table_stride, const int* positions, const int* slot_of_token, int tokens,
                                      int nq, int nkv, int Dk, int Dv, int page_size, float scale, float cap,
                                      const void* r1, const void* r2, int r_dtype, int window, void* stream) {
  if (tokens == 0) return 0;
  if (Dk > kCapMaxD || Dv > kCapMaxD || nkv < 1 || nq % nkv != 0 || nq > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  dim3 grid(tokens, nq);
  const size_t lds = static_cast<size_t>(Dk) * sizeof(float);
  if (dtype == kF32) {
    attn_softcap_simt_kernel<float><<<grid, kWave, lds, s>>>(
        static_cast<const float*>(q), q_stride, static_cast<float*>(out), o_stride, static_cast<const float*>(k_pages),
        static_cast<const float*>(v_pages), block_table, table_stride, positions, slot_of_token, nq, nkv, Dk, Dv,
        page_size, scale, cap, r1, r2, r_dtype, window);
  } else {
    attn_softcap_simt_kernel<bf16><<<grid, kWave, lds, s>>>(
        static_cast<const bf16*>(q), q_stride, static_cast<bf16*>(out), o_stride, static_cast<const bf16*>(k_pages),
        static_cast<const bf16*>(v_pages), block_table, table_stride, positions, slot_of_token, nq, nkv, Dk, Dv,
        page_size, scale, cap, r1, r2, r_dtype, window);
  }
  return launch_status();
}
