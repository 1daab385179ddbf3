// The mLSTM matrix memory, token by token, for the rows of a packed step, continued across steps through a
// per-request state in 32-bit floats: S [heads, D, Dv], n [heads, D] and the running maximum m [heads].
//
//   i_t = cap tanh((gi_t + bi) / cap)                      log input gate
//   f_t = logsigmoid(cap tanh((gf_t + bf) / cap))          log forget gate
//   m_t = max(f_t + m_(t-1), i_t);  keep = exp(f_t + m_(t-1) - m_t);  take = exp(i_t - m_t)
//   S_t = keep S_(t-1) + take k_t v_t^T;   n_t = keep n_(t-1) + take k_t
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),   q_t = (W_q h_t) D^(-1/2)
//
// Three kernels.  `mlstm_gates` owns n and m: one wave a (request, head) walks the request's rows, leaves
// (keep, take, 1/denominator) for every (row, head) and updates n and m.  `mlstm_memory` owns S: a workgroup a
// (request, head, 64 columns of Dv) holds its part of S in registers, sixteen columns a wave and a quarter of D
// a lane, walks the rows with q, k and v staged through LDS in blocks of rows, and writes o.  The two share
// nothing that both write, so columns can be spread over as many workgroups as Dv gives.  `mlstm_output`
// divides each head's o by its root mean square, and multiplies by the norm weight and by sigmoid(gate).
// Every sum runs in the same order for a row whether it comes in a portion or alone.
#include "common.h"

namespace arle {

constexpr int kGateMaxPer = 8;   // D <= 512
constexpr int kGateBlock = 8;    // rows fetched together by the gates kernel

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__global__ __launch_bounds__(kWave) void mlstm_gates_kernel(
    const void* __restrict__ q, long long q_stride, const void* __restrict__ k, long long k_stride, int qk_dtype,
    const float* __restrict__ gates, long long gates_stride, const void* __restrict__ bias_i,
    const void* __restrict__ bias_f, int bias_dtype, float cap, float q_scale, float* __restrict__ n_state,
    float* __restrict__ m_state, const int* __restrict__ seg_row0, const int* __restrict__ seg_slot,
    float* __restrict__ coefs /* [T, H, 3] */, int H, int D) {
  const int seg = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int row0 = seg_row0[seg], rows = seg_row0[seg + 1] - row0;
  const int slot = seg_slot[seg];
  float* n_ptr = n_state + (static_cast<int64_t>(slot) * H + h) * D;
  float n[kGateMaxPer];
#pragma unroll
  for (int j = 0; j < kGateMaxPer; ++j) {
    const int d = lane + j * kWave;
    n[j] = d < D ? n_ptr[d] : 0.f;
  }
  float m = m_state[static_cast<int64_t>(slot) * H + h];
  const float bi = load_as_float(bias_i, bias_dtype, h), bf = load_as_float(bias_f, bias_dtype, h);
  const float inv_cap = 1.0f / cap;

  for (int base = 0; base < rows; base += kGateBlock) {
    float kk[kGateBlock][kGateMaxPer], qq[kGateBlock][kGateMaxPer], gi[kGateBlock], gf[kGateBlock];
#pragma unroll
    for (int b = 0; b < kGateBlock; ++b) {      // all loads of the block go out before any is used
      const int64_t t = row0 + min(base + b, rows - 1);
      gi[b] = gates[t * gates_stride + h];
      gf[b] = gates[t * gates_stride + H + h];
#pragma unroll
      for (int j = 0; j < kGateMaxPer; ++j) {
        const int d = lane + j * kWave;
        if (j * kWave < D) {
          const int dd = min(d, D - 1);
          kk[b][j] = load_as_float(k, qk_dtype, t * k_stride + h * D + dd);
          qq[b][j] = load_as_float(q, qk_dtype, t * q_stride + h * D + dd);
        }
      }
    }
#pragma unroll
    for (int b = 0; b < kGateBlock; ++b) {
      if (base + b < rows) {
        const float it = cap * tanhf((gi[b] + bi) * inv_cap);
        const float ft = log_sigmoid(cap * tanhf((gf[b] + bf) * inv_cap));
        const float m_new = fmaxf(ft + m, it);
        const float keep = expf(ft + m - m_new), take = expf(it - m_new);
        float dot = 0.f;
#pragma unroll
        for (int j = 0; j < kGateMaxPer; ++j) {
          const int d = lane + j * kWave;
          if (j * kWave < D && d < D) {
            n[j] = fmaf(keep, n[j], take * kk[b][j]);
            dot = fmaf(n[j], qq[b][j] * q_scale, dot);
          }
        }
        dot = wave_sum(dot);
        m = m_new;
        if (lane == 0) {
          float* c = coefs + (static_cast<int64_t>(row0 + base + b) * H + h) * 3;
          c[0] = keep;
          c[1] = take;
          c[2] = 1.0f / (fmaxf(fabsf(dot), expf(-m_new)) + 1e-6f);
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < kGateMaxPer; ++j) {
    const int d = lane + j * kWave;
    if (d < D) n_ptr[d] = n[j];
  }
  if (lane == 0) m_state[static_cast<int64_t>(slot) * H + h] = m;
}

constexpr int kMemThreads = 256;       // four waves, sixteen columns each
constexpr int kMemCols = 64;
constexpr int kMemRows = 8;            // rows staged in LDS at a time

// DS: elements of D a lane holds (D <= 4 * DS).
template <int DS>
__global__ __launch_bounds__(kMemThreads) void mlstm_memory_kernel(
    const void* __restrict__ q, long long q_stride, const void* __restrict__ k, long long k_stride,
    const void* __restrict__ v, long long v_stride, int dtype, const float* __restrict__ coefs, float q_scale,
    float* __restrict__ s_state, const int* __restrict__ seg_row0, const int* __restrict__ seg_slot,
    float* __restrict__ out /* [T, H * Dv] */, int H, int D, int Dv) {
  constexpr int DP = 4 * DS;   // padded D: what lies past D is zero in LDS and in the registers
  __shared__ float q_lds[kMemRows][DP];
  __shared__ float k_lds[kMemRows][DP];
  __shared__ float v_lds[kMemRows][kMemCols];
  __shared__ float c_lds[kMemRows][4];
  const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const int col = blockIdx.z * kMemCols + wave * 16 + lane % 16;
  const int part = lane / 16;              // which quarter of D
  const bool live = col < Dv;
  const int row0 = seg_row0[seg], rows = seg_row0[seg + 1] - row0;
  float* s_ptr = s_state + (static_cast<int64_t>(seg_slot[seg]) * H + h) * D * Dv;

  float S[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    S[i] = (live && d < D) ? s_ptr[static_cast<int64_t>(d) * Dv + col] : 0.f;
  }

  for (int base = 0; base < rows; base += kMemRows) {
    const int n = min(kMemRows, rows - base);
    __syncthreads();   // the block before has been read
    for (int e = tid; e < kMemRows * DP; e += kMemThreads) {
      const int r = e / DP, d = e % DP;
      float qv = 0.f, kv = 0.f;
      if (r < n && d < D) {
        const int64_t t = row0 + base + r;
        qv = load_as_float(q, dtype, t * q_stride + h * D + d) * q_scale;
        kv = load_as_float(k, dtype, t * k_stride + h * D + d);
      }
      q_lds[r][d] = qv;
      k_lds[r][d] = kv;
    }
    for (int e = tid; e < kMemRows * kMemCols; e += kMemThreads) {
      const int r = e / kMemCols, c = blockIdx.z * kMemCols + e % kMemCols;
      v_lds[r][e % kMemCols] = (r < n && c < Dv) ? load_as_float(v, dtype, (row0 + base + r) * v_stride + h * Dv + c) : 0.f;
    }
    if (tid < kMemRows * 3) {
      const int r = tid / 3;
      c_lds[r][tid % 3] = r < n ? coefs[(static_cast<int64_t>(row0 + base + r) * H + h) * 3 + tid % 3] : 0.f;
    }
    __syncthreads();
    for (int r = 0; r < n; ++r) {
      const float keep = c_lds[r][0], take = c_lds[r][1], inv_den = c_lds[r][2];
      const float tv = take * v_lds[r][wave * 16 + lane % 16];
      float acc = 0.f;
#pragma unroll
      for (int i = 0; i < DS; ++i) {
        S[i] = fmaf(keep, S[i], tv * k_lds[r][part * DS + i]);
        acc = fmaf(S[i], q_lds[r][part * DS + i], acc);
      }
      acc += __shfl_xor(acc, 16, kWave);
      acc += __shfl_xor(acc, 32, kWave);
      if (part == 0 && live) out[static_cast<int64_t>(row0 + base + r) * H * Dv + h * Dv + col] = acc * inv_den;
    }
  }
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    if (live && d < D) s_ptr[static_cast<int64_t>(d) * Dv + col] = S[i];
  }
}

// One wave a (row, head): o / rms(o) * weight * sigmoid(gate).
__global__ __launch_bounds__(kWave) void mlstm_output_kernel(const float* __restrict__ o, const void* __restrict__ gate,
                                                             long long gate_stride, int gate_dtype,
                                                             const void* __restrict__ weight, int w_dtype,
                                                             void* __restrict__ out, int out_dtype, int H, int Dv,
                                                             float eps) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* row = o + (t * H + h) * Dv;
  float ss = 0.f;
  for (int c = lane; c < Dv; c += kWave) ss = fmaf(row[c], row[c], ss);
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dv) + eps);
  for (int c = lane; c < Dv; c += kWave) {
    const float g = load_as_float(gate, gate_dtype, t * gate_stride + h * Dv + c);
    const float y = row[c] * inv * load_as_float(weight, w_dtype, h * Dv + c) / (1.0f + expf(-g));
    store_from_float(out, out_dtype, (t * H + h) * Dv + c, y);
  }
}

}  // namespace arle

using namespace arle;

// q, k [T, H*D], v, gate [T, H*Dv]: rows with their own strides, of `dtype`.  gates float32 [T, >= 2H] (input gate
// pre-activations of the heads first, then the forget gate's).  coefs float32 [T, H, 3] and o float32 [T, H*Dv]
// are scratch of the call.  n_state [slots, H, D], m_state [slots, H], s_state [slots, H, D, Dv] float32.
extern "C" int arle_mlstm_scan(const void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                               long long v_stride, int dtype, const float* gates, long long gates_stride,
                               const void* bias_i, const void* bias_f, int bias_dtype, float cap, float* s_state,
                               float* n_state, float* m_state, const int* seg_row0, const int* seg_slot,
                               int segments, float* coefs, float* o, int H, int D, int Dv, void* stream) {
  if (segments == 0) return 0;
  if (D < 1 || D > 256 || Dv < 1 || H < 1 || H > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float q_scale = 1.0f / sqrtf(static_cast<float>(D));
  mlstm_gates_kernel<<<dim3(segments, H), kWave, 0, s>>>(q, q_stride, k, k_stride, dtype, gates, gates_stride, bias_i,
                                                         bias_f, bias_dtype, cap, q_scale, n_state, m_state, seg_row0,
                                                         seg_slot, coefs, H, D);
  const dim3 grid(segments, H, (Dv + kMemCols - 1) / kMemCols);
#define ARLE_MEM(DS)                                                                                               \
  mlstm_memory_kernel<DS><<<grid, kMemThreads, 0, s>>>(q, q_stride, k, k_stride, v, v_stride, dtype, coefs, q_scale, \
                                                       s_state, seg_row0, seg_slot, o, H, D, Dv)
  if (D <= 32) {
    ARLE_MEM(8);
  } else if (D <= 64) {
    ARLE_MEM(16);
  } else if (D <= 128) {
    ARLE_MEM(32);
  } else {
    ARLE_MEM(64);
  }
#undef ARLE_MEM
  return launch_status();
}

extern "C" int arle_mlstm_output(const float* o, const void* gate, long long gate_stride, int gate_dtype,
                                 const void* weight, int w_dtype, void* out, int out_dtype, int tokens, int H, int Dv,
                                 float eps, void* stream) {
  if (tokens == 0) return 0;
  mlstm_output_kernel<<<dim3(tokens, H), kWave, 0, static_cast<hipStream_t>(stream)>>>(
      o, gate, gate_stride, gate_dtype, weight, w_dtype, out, out_dtype, H, Dv, eps);
  return launch_status();
}
