// The mLSTM matrix memory, token by token, for the rows of a packed step, continued across steps through a
// per-request state in 32-bit floats: S [heads, D, Dv], n [heads, D] and the running maximum m [heads].
//
//   i_t = cap tanh((gi_t + bi) / cap)                      log input gate
//   f_t = logsigmoid(cap tanh((gf_t + bf) / cap))          log forget gate
//   m_t = max(f_t + m_(t-1), i_t);  keep = exp(f_t + m_(t-1) - m_t);  take = exp(i_t - m_t)
//   S_t = keep S_(t-1) + take k_t v_t^T;   n_t = keep n_(t-1) + take k_t
//   o_t = S_t^T q_t / (max(|n_t . q_t|, exp(-m_t)) + 1e-6),   q_t = (W_q h_t) D^(-1/2)
//
// Three kernels.  `mlstm_gates` owns m: one wave a (request, head) takes the request's rows 64 at a time, a row a lane
// for the gates' tanh, logsigmoid and exponentials, and walks the one dependent chain m_t = max(f_t + m_(t-1), i_t)
// lane by lane; it leaves (keep, take, m_t) for every (row, head).  `mlstm_memory` owns S and n: a workgroup a
// (request, head, 16 columns of Dv) holds its part of S in registers, four columns a wave and a sixteenth of D a lane;
// a fifth wave holds n, which is the column that S would have for a value of 1.  The rows' q, k and v go through LDS in
// blocks of 32 rows, fetched a block ahead; the kernel writes the numerators S_t^T q_t and n_t . q_t.  Columns
// share nothing that both write, so they spread over as many workgroups as Dv gives.  `mlstm_output` divides by the
// denominator, then each head's o by its root mean square, and multiplies by the norm weight and by sigmoid(gate).
// Every sum runs in the same order for a row whether it comes in a portion or alone.
#include "common.h"

namespace arle {

__device__ __forceinline__ float log_sigmoid(float x) { return fminf(x, 0.f) - log1pf(expf(-fabsf(x))); }

__global__ __launch_bounds__(kWave) void mlstm_gates_kernel(const float* __restrict__ gates, long long gates_stride,
                                                            const float* __restrict__ bias_i,
                                                            const float* __restrict__ bias_f, float cap,
                                                            float* __restrict__ m_state, const int* __restrict__ seg_row0,
                                                            const int* __restrict__ seg_slot,
                                                            float* __restrict__ coefs /* [T, H, 3] */, int H) {
  const int seg = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int row0 = seg_row0[seg], rows = seg_row0[seg + 1] - row0;
  float* m_ptr = m_state + static_cast<int64_t>(seg_slot[seg]) * H + h;
  float m = *m_ptr;
  const float bi = bias_i[h], bf = bias_f[h], inv_cap = 1.0f / cap;
  for (int base = 0; base < rows; base += kWave) {
    const int count = min(kWave, rows - base);
    const int64_t t = row0 + base + min(lane, count - 1);
    const float it = cap * tanhf((gates[t * gates_stride + h] + bi) * inv_cap);
    const float ft = log_sigmoid(cap * tanhf((gates[t * gates_stride + H + h] + bf) * inv_cap));
    float m_before = 0.f, m_mine = 0.f;
    for (int j = 0; j < count; ++j) {      // the one chain that is serial: two operations a row
      // row j's gates, read from lane j into scalars (j is the same in all lanes)
      const float fj = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(ft), j));
      const float ij = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(it), j));
      const float m_new = fmaxf(fj + m, ij);
      if (lane == j) {
        m_before = m;
        m_mine = m_new;
      }
      m = m_new;
    }
    if (lane < count) {
      float* c = coefs + (t * H + h) * 3;
      c[0] = expf(ft + m_before - m_mine);
      c[1] = expf(it - m_mine);
      c[2] = m_mine;
    }
  }
  if (lane == 0) *m_ptr = m;
}

// A row's work is one dependent chain a wave (LDS reads, the lane's share of D, the sum over the shares), and a wave
// has its SIMD to itself, so the chain is kept short: a lane holds a sixteenth of D for one column, a wave four columns.
constexpr int kMemColWaves = 4;                          // waves that hold columns of S, four each
constexpr int kMemThreads = (kMemColWaves + 1) * kWave;  // and one that holds n
constexpr int kMemWaveCols = 4;
constexpr int kMemParts = kWave / kMemWaveCols;          // shares of D
constexpr int kMemCols = kMemColWaves * kMemWaveCols;
constexpr int kMemRows = 32;                             // rows staged in LDS at a time

// DS: elements of D a lane holds (D <= 16 * DS).  VEC: D is a multiple of 4 and the rows of q, k, v are 16-byte
// aligned, so the staging fetches four elements at a time.
template <typename T, int DS, bool VEC>
__global__ __launch_bounds__(kMemThreads) void mlstm_memory_kernel(
    const T* __restrict__ q, long long q_stride, const T* __restrict__ k, long long k_stride, const T* __restrict__ v,
    long long v_stride, const float* __restrict__ coefs, float q_scale, float* __restrict__ s_state,
    float* __restrict__ n_state, const int* __restrict__ seg_row0, const int* __restrict__ seg_slot,
    float* __restrict__ num /* [T, H * Dv] */, float* __restrict__ nq /* [T, H] */, int H, int D, int Dv) {
  constexpr int DP = kMemParts * DS;   // padded D: what lies past D is zero in LDS and in the registers
  constexpr int W = VEC ? 4 : 1;                                    // elements a staging access
  constexpr int QK_PER = (kMemRows * DP / W + kMemThreads - 1) / kMemThreads;
  constexpr int V_PER = (kMemRows * kMemCols / W + kMemThreads - 1) / kMemThreads;
  __shared__ __attribute__((aligned(16))) float q_lds[kMemRows][DP];
  __shared__ __attribute__((aligned(16))) float k_lds[kMemRows][DP];
  __shared__ __attribute__((aligned(16))) float v_lds[kMemRows][kMemCols];
  __shared__ float c_lds[kMemRows][2];
  const int seg = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int lane = tid % kWave, wave = tid / kWave;
  const bool n_wave = wave == kMemColWaves;           // holds n; only the first workgroup of a head writes it
  const int col = blockIdx.z * kMemCols + wave * kMemWaveCols + lane % kMemWaveCols;
  const int part = lane / kMemWaveCols;               // which share of D
  const bool live = n_wave ? (blockIdx.z == 0 && lane % kMemWaveCols == 0) : col < Dv;
  const int row0 = seg_row0[seg], rows = seg_row0[seg + 1] - row0;
  const int64_t slot = seg_slot[seg];
  float* s_ptr = s_state + (slot * H + h) * D * Dv;
  float* n_ptr = n_state + (slot * H + h) * D;

  float S[DS];
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    S[i] = 0.f;
    if (d < D) {
      if (n_wave) {
        S[i] = n_ptr[d];
      } else if (live) {
        S[i] = s_ptr[static_cast<int64_t>(d) * Dv + col];
      }
    }
  }
  for (int e = tid; e < kMemRows * DP; e += kMemThreads) {
    q_lds[e / DP][e % DP] = 0.f;
    k_lds[e / DP][e % DP] = 0.f;
  }

  // what a thread fetches of a block of rows: its shares of q, k, v and the rows' coefficients
  const int per_row = D / W, v_cols = min(kMemCols, Dv - static_cast<int>(blockIdx.z) * kMemCols);
  float4 fq[QK_PER], fk[QK_PER], fv[V_PER];
  float fc = 0.f;
  auto fetch = [&](int base) {
    const int n = min(kMemRows, rows - base);
#pragma unroll
    for (int x = 0; x < QK_PER; ++x) {
      const int e = tid + x * kMemThreads;
      const int r = min(e / per_row, n - 1), d = (e % per_row) * W;
      const int64_t t = row0 + base + r;
      if (VEC) {
        fq[x] = ld4<T>(q + t * q_stride + h * D + d);
        fk[x] = ld4<T>(k + t * k_stride + h * D + d);
      } else {
        fq[x].x = to_float(q[t * q_stride + h * D + d]);
        fk[x].x = to_float(k[t * k_stride + h * D + d]);
      }
    }
#pragma unroll
    for (int x = 0; x < V_PER; ++x) {
      const int e = tid + x * kMemThreads;
      const int r = min(e / (kMemCols / W), n - 1), c = (e % (kMemCols / W)) * W;
      const int64_t t = row0 + base + r;
      const int cc = blockIdx.z * kMemCols + min(c, max(v_cols - W, 0));
      if (VEC) {
        fv[x] = ld4<T>(v + t * v_stride + h * Dv + cc);
      } else {
        fv[x].x = to_float(v[t * v_stride + h * Dv + cc]);
      }
    }
    if (tid < kMemRows * 2) fc = coefs[(static_cast<int64_t>(row0 + base + min(tid / 2, n - 1)) * H + h) * 3 + tid % 2];
  };
  auto park = [&]() {
#pragma unroll
    for (int x = 0; x < QK_PER; ++x) {
      const int e = tid + x * kMemThreads;
      if (e < kMemRows * per_row) {
        const int r = e / per_row, d = (e % per_row) * W;
        if (VEC) {
          *reinterpret_cast<float4*>(&q_lds[r][d]) = float4{fq[x].x * q_scale, fq[x].y * q_scale, fq[x].z * q_scale, fq[x].w * q_scale};
          *reinterpret_cast<float4*>(&k_lds[r][d]) = fk[x];
        } else {
          q_lds[r][d] = fq[x].x * q_scale;
          k_lds[r][d] = fk[x].x;
        }
      }
    }
#pragma unroll
    for (int x = 0; x < V_PER; ++x) {
      const int e = tid + x * kMemThreads;
      if (e < kMemRows * kMemCols / W) {
        const int r = e / (kMemCols / W), c = (e % (kMemCols / W)) * W;
        if (VEC) {
          *reinterpret_cast<float4*>(&v_lds[r][c]) = fv[x];
        } else {
          v_lds[r][c] = fv[x].x;
        }
      }
    }
    if (tid < kMemRows * 2) c_lds[tid / 2][tid % 2] = fc;
  };

  fetch(0);
  for (int base = 0; base < rows; base += kMemRows) {
    const int n = min(kMemRows, rows - base);
    __syncthreads();   // the block before has been read (and, the first time, the padding is zero)
    park();
    __syncthreads();
    if (base + kMemRows < rows) fetch(base + kMemRows);   // in flight while this block is worked through
#pragma unroll 2
    for (int r = 0; r < n; ++r) {
      const float keep = c_lds[r][0], take = c_lds[r][1];
      const float tv = n_wave ? take : take * v_lds[r][wave * kMemWaveCols + lane % kMemWaveCols];
      float part_sum[4] = {0.f, 0.f, 0.f, 0.f};
      if (DS % 4 == 0) {   // 16-byte reads
        const float4* k4 = reinterpret_cast<const float4*>(&k_lds[r][part * DS]);
        const float4* q4 = reinterpret_cast<const float4*>(&q_lds[r][part * DS]);
#pragma unroll
        for (int i = 0; i < DS / 4; ++i) {
          const float4 kv = k4[i], qv = q4[i];
          const float ke[4] = {kv.x, kv.y, kv.z, kv.w}, qe[4] = {qv.x, qv.y, qv.z, qv.w};
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            S[4 * i + j] = fmaf(keep, S[4 * i + j], tv * ke[j]);
            part_sum[j] = fmaf(S[4 * i + j], qe[j], part_sum[j]);
          }
        }
      } else {
#pragma unroll
        for (int i = 0; i < DS; ++i) {
          S[i] = fmaf(keep, S[i], tv * k_lds[r][part * DS + i]);
          part_sum[i % 4] = fmaf(S[i], q_lds[r][part * DS + i], part_sum[i % 4]);
        }
      }
      float acc = (part_sum[0] + part_sum[1]) + (part_sum[2] + part_sum[3]);
#pragma unroll
      for (int off = kMemWaveCols; off < kWave; off <<= 1) acc += __shfl_xor(acc, off, kWave);
      if (part == 0 && live) {
        const int64_t t = row0 + base + r;
        if (n_wave) {
          nq[t * H + h] = acc;
        } else {
          num[t * H * Dv + h * Dv + col] = acc;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < DS; ++i) {
    const int d = part * DS + i;
    if (live && d < D) {
      if (n_wave) {
        n_ptr[d] = S[i];
      } else {
        s_ptr[static_cast<int64_t>(d) * Dv + col] = S[i];
      }
    }
  }
}

// One wave a (row, head): o = numerator / (max(|n . q|, exp(-m)) + 1e-6), then o / rms(o) * weight * sigmoid(gate).
__global__ __launch_bounds__(kWave) void mlstm_output_kernel(const float* __restrict__ num, const float* __restrict__ nq,
                                                             const float* __restrict__ coefs, const void* __restrict__ gate,
                                                             long long gate_stride, int gate_dtype,
                                                             const void* __restrict__ weight, int w_dtype,
                                                             void* __restrict__ out, int out_dtype, int H, int Dv,
                                                             float eps) {
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, lane = threadIdx.x;
  const float* row = num + (t * H + h) * Dv;
  const float inv_den = 1.0f / (fmaxf(fabsf(nq[t * H + h]), expf(-coefs[(t * H + h) * 3 + 2])) + 1e-6f);
  float ss = 0.f;
  for (int c = lane; c < Dv; c += kWave) {
    const float o = row[c] * inv_den;
    ss = fmaf(o, o, ss);
  }
  const float inv = 1.0f / sqrtf(wave_sum(ss) / static_cast<float>(Dv) + eps);
  for (int c = lane; c < Dv; c += kWave) {
    const float g = load_as_float(gate, gate_dtype, t * gate_stride + h * Dv + c);
    const float y = row[c] * inv_den * inv * load_as_float(weight, w_dtype, h * Dv + c) / (1.0f + expf(-g));
    store_from_float(out, out_dtype, (t * H + h) * Dv + c, y);
  }
}

template <typename T>
static int launch_memory(const void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                         long long v_stride, const float* coefs, float q_scale, float* s_state, float* n_state,
                         const int* seg_row0, const int* seg_slot, int segments, float* num, float* nq, int H, int D, int Dv,
                         hipStream_t s) {
  const dim3 grid(segments, H, (Dv + kMemCols - 1) / kMemCols);
  const auto aligned = [](const void* p) { return reinterpret_cast<uintptr_t>(p) % (4 * sizeof(T)) == 0; };
  const bool vec = D % 4 == 0 && Dv % 4 == 0 && q_stride % 4 == 0 && k_stride % 4 == 0 && v_stride % 4 == 0 && aligned(q) &&
                   aligned(k) && aligned(v);
#define ARLE_MEM(DS, VEC)                                                                                              \
  mlstm_memory_kernel<T, DS, VEC><<<grid, kMemThreads, 0, s>>>(static_cast<const T*>(q), q_stride,                     \
                                                               static_cast<const T*>(k), k_stride,                     \
                                                               static_cast<const T*>(v), v_stride, coefs, q_scale,     \
                                                               s_state, n_state, seg_row0, seg_slot, num, nq, H, D, Dv)
#define ARLE_MEM_DS(DS) \
  do {                  \
    if (vec)            \
      ARLE_MEM(DS, true); \
    else                \
      ARLE_MEM(DS, false); \
  } while (0)
  if (D <= 32) {
    ARLE_MEM_DS(2);
  } else if (D <= 64) {
    ARLE_MEM_DS(4);
  } else if (D <= 128) {
    ARLE_MEM_DS(8);
  } else {
    ARLE_MEM_DS(16);
  }
#undef ARLE_MEM_DS
#undef ARLE_MEM
  return launch_status();
}

}  // namespace arle

using namespace arle;

// q, k [T, H*D], v, gate [T, H*Dv]: rows with their own strides, of `dtype`.  gates float32 [T, >= 2H] (input gate
// pre-activations of the heads first, then the forget gate's); bias_i, bias_f float32 [H].  coefs float32 [T, H, 3]
// (keep, take, m), num float32 [T, H*Dv] and nq float32 [T, H] are outputs for `arle_mlstm_output`.
// n_state [slots, H, D], m_state [slots, H], s_state [slots, H, D, Dv] float32.
extern "C" int arle_mlstm_scan(const void* q, long long q_stride, const void* k, long long k_stride, const void* v,
                               long long v_stride, int dtype, const float* gates, long long gates_stride,
                               const float* bias_i, const float* bias_f, float cap, float* s_state, float* n_state,
                               float* m_state, const int* seg_row0, const int* seg_slot, int segments, float* coefs,
                               float* num, float* nq, int H, int D, int Dv, void* stream) {
  if (segments == 0) return 0;
  if (D < 1 || D > 256 || Dv < 1 || H < 1 || H > 65535) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float q_scale = 1.0f / sqrtf(static_cast<float>(D));
  mlstm_gates_kernel<<<dim3(segments, H), kWave, 0, s>>>(gates, gates_stride, bias_i, bias_f, cap, m_state, seg_row0,
                                                         seg_slot, coefs, H);
  return dtype == kF32 ? launch_memory<float>(q, q_stride, k, k_stride, v, v_stride, coefs, q_scale, s_state, n_state,
                                              seg_row0, seg_slot, segments, num, nq, H, D, Dv, s)
                       : launch_memory<bf16>(q, q_stride, k, k_stride, v, v_stride, coefs, q_scale, s_state, n_state,
                                             seg_row0, seg_slot, segments, num, nq, H, D, Dv, s);
}

extern "C" int arle_mlstm_output(const float* num, const float* nq, const float* coefs, const void* gate,
                                 long long gate_stride, int gate_dtype, const void* weight, int w_dtype, void* out,
                                 int out_dtype, int tokens, int H, int Dv, float eps, void* stream) {
  if (tokens == 0) return 0;
  mlstm_output_kernel<<<dim3(tokens, H), kWave, 0, static_cast<hipStream_t>(stream)>>>(
      num, nq, coefs, gate, gate_stride, gate_dtype, weight, w_dtype, out, out_dtype, H, Dv, eps);
  return launch_status();
}
