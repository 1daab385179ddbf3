// A short causal convolution over time on every channel of the rows of a packed step, continued across
// steps through a per-request state of the last taps-1 inputs.
//
//   y_t[c] = (ADD ? u_t[c] : 0) + sum_{j < taps} w[c][j] * u_(t - taps + 1 + j)[c],    u := input (+ bias)
//
// The rows of one request are consecutive in the step; an input further back than the request's first row of
// this step comes from its state [slots][taps-1][channels] (the most recent input last), which is all zeros
// when the request starts, so inputs before position 0 count as zero without a test.  The sums are 32-bit.
// `conv_state_update` then shifts each request's state by the rows it brought.  The update is a kernel of its
// own because the convolution of a step reads the old state of every request.
#include "common.h"

namespace arle {

constexpr int kConvMaxTaps = 16;

__global__ void causal_conv_kernel(const void* __restrict__ u, long long u_stride, int u_dtype,
                                   const void* __restrict__ bias, int bias_dtype, const void* __restrict__ w,
                                   int w_dtype, const void* __restrict__ state, int state_dtype,
                                   const int* __restrict__ slot_of_token, void* __restrict__ out,
                                   long long out_stride, int out_dtype, int channels, int taps, int add_input) {
  const int t = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int slot = slot_of_token[t];
  const float b = bias ? load_as_float(bias, bias_dtype, c) : 0.f;
  const float now = load_as_float(u, u_dtype, t * u_stride + c) + b;
  if (!w) {   // no convolution: the input with its bias
    store_from_float(out, out_dtype, t * out_stride + c, now);
    return;
  }
  // rows of the same request right before this one in the step (at most taps-1 matter)
  int mine = 0;
  while (mine < taps - 1 && t - mine - 1 >= 0 && slot_of_token[t - mine - 1] == slot) ++mine;
  float acc = add_input ? now : 0.f;
  acc = fmaf(load_as_float(w, w_dtype, static_cast<int64_t>(c) * taps + taps - 1), now, acc);
  for (int back = 1; back < taps; ++back) {
    float v;
    if (back <= mine) {
      v = load_as_float(u, u_dtype, (t - back) * u_stride + c) + b;
    } else {  // state row taps-1 - (back - mine): the (back - mine)-th most recent input before the step
      const int64_t row = static_cast<int64_t>(slot) * (taps - 1) + (taps - 1 - (back - mine));
      v = load_as_float(state, state_dtype, row * channels + c);
    }
    acc = fmaf(load_as_float(w, w_dtype, static_cast<int64_t>(c) * taps + taps - 1 - back), v, acc);
  }
  store_from_float(out, out_dtype, t * out_stride + c, acc);
}

// One thread a (segment, channel): the new state is the last taps-1 of (old state, this step's inputs).
__global__ void conv_state_update_kernel(const void* __restrict__ u, long long u_stride, int u_dtype,
                                         const void* __restrict__ bias, int bias_dtype, void* __restrict__ state,
                                         int state_dtype, const int* __restrict__ seg_row0,
                                         const int* __restrict__ seg_slot, int channels, int taps) {
  const int seg = blockIdx.x;
  const int c = blockIdx.y * blockDim.x + threadIdx.x;
  if (c >= channels) return;
  const int row0 = seg_row0[seg], len = seg_row0[seg + 1] - row0;
  const int keep = taps - 1;
  const int64_t base = static_cast<int64_t>(seg_slot[seg]) * keep;
  const float b = bias ? load_as_float(bias, bias_dtype, c) : 0.f;
  float fresh[kConvMaxTaps];
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j) {
    if (j < keep) {
      const int at = len - keep + j;   // place among this step's rows; negative: still in the old state
      fresh[j] = at >= 0 ? load_as_float(u, u_dtype, (row0 + at) * u_stride + c) + b
                         : load_as_float(state, state_dtype, (base + j + len) * channels + c);
    }
  }
#pragma unroll
  for (int j = 0; j < kConvMaxTaps; ++j)
    if (j < keep) store_from_float(state, state_dtype, (base + j) * channels + c, fresh[j]);
}

}  // namespace arle

using namespace arle;

// u [T, channels] rows u_stride apart; out likewise; w [channels, taps] or null (then out = u + bias);
// state [slots, taps-1, channels]; slot_of_token int32 [T].
extern "C" int arle_causal_conv(const void* u, long long u_stride, int u_dtype, const void* bias, int bias_dtype,
                                const void* w, int w_dtype, const void* state, int state_dtype,
                                const int* slot_of_token, void* out, long long out_stride, int out_dtype, int tokens,
                                int channels, int taps, int add_input, void* stream) {
  if (tokens == 0 || channels == 0) return 0;
  if (w && (taps < 1 || taps > kConvMaxTaps)) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid(tokens, (channels + 255) / 256);
  causal_conv_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      u, u_stride, u_dtype, bias, bias_dtype, w, w_dtype, state, state_dtype, slot_of_token, out, out_stride,
      out_dtype, channels, taps, add_input);
  return launch_status();
}

extern "C" int arle_conv_state_update(const void* u, long long u_stride, int u_dtype, const void* bias,
                                      int bias_dtype, void* state, int state_dtype, const int* seg_row0,
                                      const int* seg_slot, int segments, int channels, int taps, void* stream) {
  if (segments == 0 || channels == 0 || taps <= 1) return 0;
  if (taps > kConvMaxTaps) return static_cast<int>(hipErrorInvalidValue);
  dim3 grid(segments, (channels + 255) / 256);
  conv_state_update_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream)>>>(
      u, u_stride, u_dtype, bias, bias_dtype, state, state_dtype, seg_row0, seg_slot, channels, taps);
  return launch_status();
}
