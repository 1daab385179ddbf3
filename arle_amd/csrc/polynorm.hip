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

// One element type T for input, bias, coefficients and output, a width that is a multiple of 4: four elements a lane
// and access, all loads of the row issued together.
template <typename T, int PER4>
__global__ __launch_bounds__(kPnThreads) void polynorm_vec_kernel(const T* __restrict__ u, long long u_stride,
                                                                  const T* __restrict__ bias, const T* __restrict__ coef,
                                                                  T* __restrict__ out, int width, float eps) {
  __shared__ float lds[kPnWaves];
  const int64_t r = blockIdx.x;
  const int last = width - 4, tid = threadIdx.x;
  float4 z[PER4];
#pragma unroll
  for (int k = 0; k < PER4; ++k) z[k] = ld4<T>(u + r * u_stride + min((tid + k * kPnThreads) * 4, last));
  if (bias) {
#pragma unroll
    for (int k = 0; k < PER4; ++k) {
      const float4 b = ld4<T>(bias + min((tid + k * kPnThreads) * 4, last));
      z[k].x += b.x; z[k].y += b.y; z[k].z += b.z; z[k].w += b.w;
    }
  }
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    if ((tid + k * kPnThreads) * 4 < width) {
      const float e[4] = {z[k].x, z[k].y, z[k].z, z[k].w};
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const float q = e[j] * e[j];
        s2 += q;
        s4 += q * q;
        s6 += q * q * q;
      }
    }
  }
  const float n = static_cast<float>(width);
  const float i1 = 1.0f / sqrtf(block_sum<kPnWaves>(s2, lds) / n + eps);
  const float i2 = 1.0f / sqrtf(block_sum<kPnWaves>(s4, lds) / n + eps);
  const float i3 = 1.0f / sqrtf(block_sum<kPnWaves>(s6, lds) / n + eps);
  const float a = to_float(coef[0]) * i1, b = to_float(coef[1]) * i2, c = to_float(coef[2]) * i3, e = to_float(coef[3]);
  auto poly = [&](float v) { return fmaf(v, fmaf(v, fmaf(v, c, b), a), e); };
#pragma unroll
  for (int k = 0; k < PER4; ++k) {
    const int i = (tid + k * kPnThreads) * 4;
    if (i < width) st4<T>(out + r * width + i, float4{poly(z[k].x), poly(z[k].y), poly(z[k].z), poly(z[k].w)});
  }
}

template <typename T>
static int launch_pn_vec(const void* u, long long u_stride, const void* bias, const void* coef, void* out, int tokens,
                         int width, float eps, hipStream_t s) {
#define ARLE_PNV(PER4)                                                                                                 \
  polynorm_vec_kernel<T, PER4><<<tokens, kPnThreads, 0, s>>>(static_cast<const T*>(u), u_stride,                       \
                                                             static_cast<const T*>(bias), static_cast<const T*>(coef), \
                                                             static_cast<T*>(out), width, eps)
  if (width <= kPnThreads * 8) {
    ARLE_PNV(2);
  } else if (width <= kPnThreads * 16) {
    ARLE_PNV(4);
  } else if (width <= kPnThreads * 32) {
    ARLE_PNV(8);
  } else if (width <= kPnThreads * 48) {
    ARLE_PNV(12);
  } else {
    ARLE_PNV(24);
  }
#undef ARLE_PNV
  return launch_status();
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
  const bool aligned = reinterpret_cast<uintptr_t>(u) % 16 == 0 && u_stride % 4 == 0;
  if (width % 4 == 0 && aligned && u_dtype == out_dtype && coef_dtype == out_dtype && (!bias || bias_dtype == out_dtype)) {
    return out_dtype == kF32 ? launch_pn_vec<float>(u, u_stride, bias, coef, out, tokens, width, eps, s)
                             : launch_pn_vec<bf16>(u, u_stride, bias, coef, out, tokens, width, eps, s);
  }
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
