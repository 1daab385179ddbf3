// Layer norm without bias over rows, with the residual adds of a parallel block fused in and one or two
// outputs from one pass.
//
//   x      = residual + (term_0 + bias_0) + (term_1 + bias_1)         (32-bit, written back)
//   mu     = mean_j x_j;   var = mean_j (x_j - mu)^2                   (two passes over registers)
//   out_a  = (x - mu) / sqrt(var + eps) * w_a;   out_b likewise with w_b (optional)
//
// A block whose mixer and feed-forward both read the same residual hands on two deltas, each of which may be
// a stack of float32 partial products (added in the order of the stack) and may carry the bias of the
// projection that made it; the next block's two norms are of that same sum, so they share the statistics.
// With `rows` given (the final norm before the head) the rows named there are read for the last time and
// the sum is not written back.
#include "common.h"

namespace arle {

constexpr int kLnThreads = 256;
constexpr int kLnWaves = kLnThreads / kWave;

struct LnTerm {
  const void* data;     // [n_stack][T][width], or null
  int n_stack;
  long long stack_stride;
  int dtype;
  const void* bias;     // [width] or null
  int bias_dtype;
};

// PER elements a thread (width <= kLnThreads * PER), the row stays in registers.
template <int PER>
__global__ __launch_bounds__(kLnThreads) void add_layernorm_kernel(
    float* __restrict__ residual, LnTerm t0, LnTerm t1, const void* __restrict__ wa, const void* __restrict__ wb,
    int w_dtype, void* __restrict__ out_a, void* __restrict__ out_b, int out_dtype, const int* __restrict__ rows,
    int width, float eps) {
  __shared__ float lds[kLnWaves];
  const int r = blockIdx.x;
  const int64_t src = rows ? rows[r] : r;
  float* res = residual + src * width;
  float x[PER];
  float sum = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    float v = 0.f;
    if (i < width) {
      v = res[i];
      if (t0.data) {
        float d = load_as_float(t0.data, t0.dtype, src * width + i);
        for (int s = 1; s < t0.n_stack; ++s) d += load_as_float(t0.data, t0.dtype, s * t0.stack_stride + src * width + i);
        if (t0.bias) d += load_as_float(t0.bias, t0.bias_dtype, i);
        v += d;
      }
      if (t1.data) {
        float d = load_as_float(t1.data, t1.dtype, src * width + i);
        for (int s = 1; s < t1.n_stack; ++s) d += load_as_float(t1.data, t1.dtype, s * t1.stack_stride + src * width + i);
        if (t1.bias) d += load_as_float(t1.bias, t1.bias_dtype, i);
        v += d;
      }
      if (!rows && (t0.data || t1.data)) res[i] = v;
    }
    x[k] = v;
    sum += v;
  }
  const float mu = block_sum<kLnWaves>(sum, lds) / static_cast<float>(width);
  float sq = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    const float d = i < width ? x[k] - mu : 0.f;
    x[k] = d;
    sq += d * d;
  }
  const float inv = 1.0f / sqrtf(block_sum<kLnWaves>(sq, lds) / static_cast<float>(width) + eps);
  const int64_t o = static_cast<int64_t>(r) * width;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kLnThreads;
    if (i < width) {
      const float n = x[k] * inv;
      store_from_float(out_a, out_dtype, o + i, n * load_as_float(wa, w_dtype, i));
      if (out_b) store_from_float(out_b, out_dtype, o + i, n * load_as_float(wb, w_dtype, i));
    }
  }
}

}  // namespace arle

using namespace arle;

// residual float32 [T, width] contiguous.  term*: null, [T, width] (n_stack 1) or a stack; bias*: null or [width].
// out_a, out_b (out_b and wb may be null): [n_rows, width] contiguous of out_dtype.  width <= 16384.
extern "C" int arle_add_layernorm(float* residual, const void* term0, int n0, long long stride0, int dtype0,
                                  const void* bias0, int bias_dtype0, const void* term1, int n1, long long stride1,
                                  int dtype1, const void* bias1, int bias_dtype1, const void* wa, const void* wb,
                                  int w_dtype, void* out_a, void* out_b, int out_dtype, const int* rows, int n_rows,
                                  int width, float eps, void* stream) {
  if (n_rows == 0) return 0;
  if (width <= 0 || width > kLnThreads * 64) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const LnTerm t0{term0, n0, stride0, dtype0, bias0, bias_dtype0};
  const LnTerm t1{term1, n1, stride1, dtype1, bias1, bias_dtype1};
#define ARLE_LN(PER)                                                                                          \
  add_layernorm_kernel<PER><<<n_rows, kLnThreads, 0, s>>>(residual, t0, t1, wa, wb, w_dtype, out_a, out_b, \
                                                          out_dtype, rows, width, eps)
  if (width <= kLnThreads * 4) {
    ARLE_LN(4);
  } else if (width <= kLnThreads * 16) {
    ARLE_LN(16);
  } else {
    ARLE_LN(64);
  }
#undef ARLE_LN
  return launch_status();
}
