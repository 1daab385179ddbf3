// A norm on a sublayer's output, added into the residual stream:
//
//   y_j   = A_j + B_j                           (up to two addends, each a sum of parts, see below)
//   res_j += y_j / sqrt(mean_j(y_j^2) + eps) * (w_j  or  1 + w_j)
//   act_j = res_j rounded to the activation type  (what the next sublayer reads; optional)
//
// An addend is a tensor [T, W], or parts that are added in ascending order: the float32 partial products of a
// matrix product whose K was split (part p of row t at p * part_stride + t * row_stride), or the outputs of the
// experts that a token chose, [T, n, W] with a weight per (token, part).  The sums, the statistics, the weight and
// the residual are 32-bit.  A row's arithmetic depends on nothing but the row.
#include "common.h"

namespace arle {

constexpr int kPostThreads = 256;
constexpr int kPostWaves = kPostThreads / kWave;

struct Addend {
  const void* p;          // null: no addend
  int parts;              // parts added in order (>= 1)
  long long part_stride;  // elements between parts of one row
  long long row_stride;   // elements between rows
  int dtype;              // kF32 / kBF16
  const float* weights;   // [T, parts] factors, or null
};

__device__ __forceinline__ float addend_at(const Addend& a, int64_t row, int i) {
  const int64_t base = row * a.row_stride + i;
  float sum = load_as_float(a.p, a.dtype, base);
  if (a.weights) sum *= a.weights[row * a.parts];
  for (int p = 1; p < a.parts; ++p) {
    const float v = load_as_float(a.p, a.dtype, base + p * a.part_stride);
    sum = a.weights ? fmaf(a.weights[row * a.parts + p], v, sum) : sum + v;
  }
  return sum;
}

template <typename TAct, typename TW>
__global__ __launch_bounds__(kPostThreads) void norm_add_kernel(float* __restrict__ residual, const Addend a,
                                                                const Addend b, const TW* __restrict__ w,
                                                                int one_plus, TAct* __restrict__ act, int width,
                                                                float eps) {
  extern __shared__ float ys[];  // [width]
  __shared__ float lds[kPostWaves];
  const int64_t r = blockIdx.x;
  float ss = 0.f;
  for (int i = threadIdx.x; i < width; i += kPostThreads) {
    float y = addend_at(a, r, i);
    if (b.p) y += addend_at(b, r, i);
    ys[i] = y;
    ss = fmaf(y, y, ss);
  }
  const float total = block_sum<kPostWaves>(ss, lds);
  const float inv = 1.0f / sqrtf(total / static_cast<float>(width) + eps);
  float* res = residual + r * width;
  for (int i = threadIdx.x; i < width; i += kPostThreads) {
    const float g = one_plus ? 1.0f + to_float(w[i]) : to_float(w[i]);
    const float v = res[i] + ys[i] * inv * g;
    res[i] = v;
    if (act) act[r * width + i] = from_float<TAct>(v);
  }
}

}  // namespace arle

using namespace arle;

// residual float32 [rows, width], updated in place.  act: [rows, width] of act_dtype, or null.
extern "C" int arle_norm_add(float* residual, const void* a, int a_parts, long long a_part_stride,
                             long long a_row_stride, int a_dtype, const float* a_weights, const void* b, int b_parts,
                             long long b_part_stride, long long b_row_stride, int b_dtype, const float* b_weights,
                             const void* w, int w_dtype, int one_plus, void* act, int act_dtype, int rows, int width,
                             float eps, void* stream) {
  if (rows == 0) return 0;
  if (!a || a_parts < 1 || (b && b_parts < 1) || width < 1 || width > 16384) return static_cast<int>(hipErrorInvalidValue);
  const Addend A{a, a_parts, a_part_stride, a_row_stride, a_dtype, a_weights};
  const Addend B{b, b_parts, b_part_stride, b_row_stride, b_dtype, b_weights};
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t lds = static_cast<size_t>(width) * sizeof(float);
#define ARLE_POST(TA, TWT)                                                                                     \
  do {                                                                                                         \
    static bool raised = false;                                                                                \
    if (!raised && lds > 48 * 1024) {                                                                          \
      const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&norm_add_kernel<TA, TWT>),       \
                                               hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);         \
      if (e != hipSuccess) return static_cast<int>(e);                                                         \
      raised = true;                                                                                           \
    }                                                                                                          \
    norm_add_kernel<TA, TWT><<<rows, kPostThreads, lds, s>>>(residual, A, B, static_cast<const TWT*>(w), one_plus, \
                                                             static_cast<TA*>(act), width, eps);               \
  } while (0)
  if (act_dtype == kF32) {
    if (w_dtype == kF32) ARLE_POST(float, float); else ARLE_POST(float, bf16);
  } else {
    if (w_dtype == kF32) ARLE_POST(bf16, float); else ARLE_POST(bf16, bf16);
  }
#undef ARLE_POST
  return launch_status();
}
