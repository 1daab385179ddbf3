// PolyNorm activation over the rows of a feed-forward's hidden layer:
//
//   z = u + bias;   N(y) = y / sqrt(mean_j(y_j^2) + eps)   (over the row)
//   out = a N(z) + b N(z^2) + c N(z^3) + e                 (powers element by element)
//
// so a row needs the means of z^2, z^4 and z^6; they, the roots and the sum are 32-bit.  The row stays in
// registers between the reduction and the output.  (a, b, c, e) are read from the checkpoint's tensor on
// the GPU.
#include "common.h"

namespace arle {

constexpr int kPnThreads = 256;
constexpr int kPnWaves = kPnThreads / kWave;

template <int PER>
__global__ __launch_bounds__(kPnThreads) void polynorm_kernel(const void* __restrict__ u, long long u_stride,
                                                              int u_dtype, const void* __restrict__ bias,
                                                              int bias_dtype, const void* __restrict__ coef,
                                                              int coef_dtype, void* __restrict__ out, int out_dtype,
                                                              int width, float eps) {
  __shared__ float lds[kPnWaves];
  const int64_t r = blockIdx.x;
  float z[PER];
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kPnThreads;
    float v = 0.f;
    if (i < width) {
      v = load_as_float(u, u_dtype, r * u_stride + i);
      if (bias) v += load_as_float(bias, bias_dtype, i);
    }
    z[k] = v;
    const float q = v * v;
    s2 += q;
    s4 += q * q;
    s6 += q * q * q;
  }
  const float n = static_cast<float>(width);
  const float i1 = 1.0f / sqrtf(block_sum<kPnWaves>(s2, lds) / n + eps);
  const float i2 = 1.0f / sqrtf(block_sum<kPnWaves>(s4, lds) / n + eps);
  const float i3 = 1.0f / sqrtf(block_sum<kPnWaves>(s6, lds) / n + eps);
  const float a = load_as_float(coef, coef_dtype, 0) * i1, b = load_as_float(coef, coef_dtype, 1) * i2,
              c = load_as_float(coef, coef_dtype, 2) * i3, e = load_as_float(coef, coef_dtype, 3);
#pragma unroll
  for (int k = 0; k < PER; ++k) {
    const int i = threadIdx.x + k * kPnThreads;
    if (i < width) {
      const float v = z[k];
      store_from_float(out, out_dtype, r * width + i, fmaf(v, fmaf(v, fmaf(v, c, b), a), e));
    }
  }
}

}  // namespace arle

using namespace arle;

// u [T, width] rows u_stride apart; bias [width] or null; coef [4]; out [T, width] contiguous.  width <= 24576.
extern "C" int arle_polynorm(const void* u, long long u_stride, int u_dtype, const void* bias, int bias_dtype,
                             const void* coef, int coef_dtype, void* out, int out_dtype, int tokens, int width,
                             float eps, void* stream) {
  if (tokens == 0) return 0;
  if (width <= 0 || width > kPnThreads * 96) return static_cast<int>(hipErrorInvalidValue);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define ARLE_PN(PER)                                                                                              \
  polynorm_kernel<PER><<<tokens, kPnThreads, 0, s>>>(u, u_stride, u_dtype, bias, bias_dtype, coef, coef_dtype, out, \
                                                     out_dtype, width, eps)
  if (width <= kPnThreads * 8) {
    ARLE_PN(8);
  } else if (width <= kPnThreads * 32) {
    ARLE_PN(32);
  } else {
    ARLE_PN(96);
  }
#undef ARLE_PN
  return launch_status();
}
