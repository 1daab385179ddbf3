// A mixture of experts: the router, and the experts' products over the tokens that chose them.
//
//   z = W_r h (32-bit sums),  s = sigmoid(z);  the `top` experts with the largest s + correction are chosen (ties: the
//   lower index);  weight of a chosen expert = s / (sum of the chosen s + 1e-20) * scale.
//   expert e: down_e (silu(gate_e h) * (up_e h)).
//
// `moe_route`: one wave a token.  `moe_expert`: a workgroup takes one expert, 64 consecutive rows of the step and 64
// output columns; it lists the rows of its 64 that chose the expert (in row order) and multiplies only those, so no
// step sorts anything and a launch's shape follows the number of rows alone.  The result of (token t, its k-th
// choice) lies at row t * top + k: the gate|up pass leaves the activation there, the down pass the expert's output,
// which the consumer weighs and adds in the order of k.  Every output is summed in one fixed order over K (chains
// of 16, added in ascending order), whatever else the step holds.
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

template <typename T, typename TW>
__global__ __launch_bounds__(kWave) void moe_route_kernel(const T* __restrict__ x, long long x_stride,
                                                          const TW* __restrict__ w, const void* __restrict__ correction,
                                                          int c_dtype, int* __restrict__ ids, float* __restrict__ weights,
                                                          int width, int experts, int top, float scale) {
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x;
  const T* row = x + t * x_stride;
  float s[kMaxExpertsPerLane], choice[kMaxExpertsPerLane];
#pragma unroll
  for (int j = 0; j < kMaxExpertsPerLane; ++j) {
    s[j] = 0.f;
    choice[j] = -INFINITY;
  }
  for (int e = 0; e < experts; ++e) {
    const TW* we = w + static_cast<int64_t>(e) * width;
    float dot = 0.f;
    for (int i = lane; i < width; i += kWave) dot = fmaf(to_float(row[i]), to_float(we[i]), dot);
    dot = wave_sum(dot);
    const float sg = 1.0f / (1.0f + expf(-dot));
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      if (e == lane + j * kWave) {
        s[j] = sg;
        choice[j] = sg + (correction ? load_as_float(correction, c_dtype, e) : 0.f);
      }
    }
  }
  float sum = 0.f, mine = 0.f;   // lane k keeps the k-th chosen score (top <= 64)
  int mine_id = 0;
  for (int k = 0; k < top; ++k) {
    Best b{-INFINITY, 0x7fffffff};
#pragma unroll
    for (int j = 0; j < kMaxExpertsPerLane; ++j) {
      const int e = lane + j * kWave;
      if (e < experts && (choice[j] > b.v || (choice[j] == b.v && e < b.i))) {
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
    weights[t * top + lane] = mine / (sum + 1e-20f) * scale;
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

}  // namespace arle

using namespace arle;

// x [T, width] of x_dtype, w [experts, width] of w_dtype, correction [experts] or null; ids int32 [T, top], weights
// float32 [T, top].
extern "C" int arle_moe_route(const void* x, long long x_stride, int x_dtype, const void* w, int w_dtype,
                              const void* correction, int c_dtype, int* ids, float* weights, int tokens, int width,
                              int experts, int top, float scale, void* stream) {
  if (tokens == 0) return 0;
  if (experts < 1 || experts > kWave * kMaxExpertsPerLane || top < 1 || top > experts || top > kWave)
    return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ARLE_ROUTE(TX, TWT)                                                                                       \
  moe_route_kernel<TX, TWT><<<tokens, kWave, 0, s>>>(static_cast<const TX*>(x), x_stride, static_cast<const TWT*>(w), \
                                                     correction, c_dtype, ids, weights, width, experts, top, scale)
  if (x_dtype == kF32) {
    if (w_dtype == kF32) ARLE_ROUTE(float, float); else ARLE_ROUTE(float, bf16);
  } else {
    if (w_dtype == kF32) ARLE_ROUTE(bf16, float); else ARLE_ROUTE(bf16, bf16);
  }
#undef ARLE_ROUTE
  return launch_status();
}

// gate_up != 0: x [T, K], w [experts, 2 N, K], out [T * top, N] of `dtype`.  Else: x [T * top, K], w [experts, N, K],
// out float32 [T * top, N].
extern "C" int arle_moe_expert(const void* x, long long x_stride, const void* w, const int* ids, void* out, int dtype,
                               int gate_up, int tokens, int experts, int top, int N, int K, void* stream) {
  if (tokens == 0) return 0;
  if (experts < 1 || experts > 65535 || top < 1 || N < 1 || K < 1 || (N + kEN - 1) / kEN > 65535)
    return static_cast<int>(hipErrorInvalidValue);
  const dim3 grid((tokens + kEM - 1) / kEM, (N + kEN - 1) / kEN, experts);
  hipStream_t s = static_cast<hipStream_t>(stream);
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
