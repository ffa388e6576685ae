// A gated linear recurrence with fixed-size state per request, and the short causal
// convolution in front of it.
//
// Per channel c and token t: u = conv(x) (a few taps back, continued across steps from the
// inputs the state saved), two gates r, i = sigmoid(block-diagonal products of u, computed by
// the per-head product kernel), log a = decay[c] * r, S <- a S + sqrt(1 - a^2) i u, and the
// output is S times the other branch, gelu_tanh(y). Everything that enters the recurrence
// is float, whatever the activation type: the gates, the decay and its exponential, the step
// size sqrt(1 - a^2) (taken as sqrt(-expm1(2 log a)), which keeps its digits when a is near
// one), the state. A step continues from state[slot] and leaves the new state there; the
// runner hands a request that starts at position 0 a zeroed slot.

#include "api.h"
#include "common.h"

namespace psamd {

constexpr int kMaxTaps = 16;

template <typename A>
__global__ __launch_bounds__(256) void causal_conv_kernel(
    const A* __restrict__ in, int64_t in_row, const float* __restrict__ in_bias, const float* __restrict__ conv_w,
    const float* __restrict__ conv_b, float* __restrict__ u, const float* __restrict__ state, int64_t state_row,
    const int32_t* __restrict__ tok_item, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots,
    int width, int taps) {
  const int64_t t = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const int item = tok_item[t];
  const int64_t s0 = item_start[item];
  const int li = static_cast<int>(t - s0);
  const float* saved = state + static_cast<int64_t>(slots[item]) * state_row;
  const float b = in_bias[c];
  float acc = conv_b[c];
  for (int j = 0; j < taps; ++j) {                     // oldest input first, the token's own last
    const int src = li - (taps - 1) + j;
    const float v = src >= 0 ? to_float<A>(in[(s0 + src) * in_row + c]) + b
                             : saved[static_cast<int64_t>(taps - 1 + src) * width + c];
    acc = fmaf(conv_w[static_cast<int64_t>(c) * taps + j], v, acc);
  }
  u[t * width + c] = acc;
}

__device__ __forceinline__ float sigmoid_f(float z) { return 1.f / (1.f + expf(-z)); }

template <typename A>
__global__ __launch_bounds__(256) void gated_scan_kernel(
    const float* __restrict__ gates, const float* __restrict__ gate_b, const float* __restrict__ u,
    const float* __restrict__ decay, const A* __restrict__ y, const A* __restrict__ x, int64_t in_row,
    const float* __restrict__ y_bias, const float* __restrict__ x_bias, A* __restrict__ out, float* __restrict__ state,
    int64_t state_row, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots, int width, int blocks,
    int taps) {
  const int item = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const int bw = width / blocks;
  const int b = c / bw, cb = c - b * bw;
  const int64_t s0 = item_start[item], s1 = item_start[item + 1];
  float* st = state + static_cast<int64_t>(slots[item]) * state_row;
  const int64_t g_off = static_cast<int64_t>(b) * 2 * bw + cb;
  const float br = gate_b[g_off], bi = gate_b[g_off + bw];
  const float dec = decay[c], yb = y_bias[c];
  float S = st[static_cast<int64_t>(taps - 1) * width + c];
  for (int64_t t = s0; t < s1; ++t) {
    const float r = sigmoid_f(gates[t * 2 * width + g_off] + br);
    const float g = sigmoid_f(gates[t * 2 * width + g_off + bw] + bi);
    const float la = dec * r;
    const float a = expf(la);
    const float step = sqrtf(-expm1f(2.f * la));
    S = fmaf(a, S, step * g * u[t * width + c]);
    out[t * width + c] = from_float<A>(S * gelu_tanh_f(to_float<A>(y[t * in_row + c]) + yb));
  }
  st[static_cast<int64_t>(taps - 1) * width + c] = S;
  // The inputs the next step's convolution reaches back to: the last taps - 1 of (saved, then this step's).
  const int n = static_cast<int>(s1 - s0), keep = taps - 1;
  const float xb = x_bias[c];
  float next[kMaxTaps];
#pragma unroll
  for (int k = 0; k < kMaxTaps; ++k) {
    if (k < keep) {
      const int li = n - keep + k;
      next[k] = li >= 0 ? to_float<A>(x[(s0 + li) * in_row + c]) + xb : st[static_cast<int64_t>(k + n) * width + c];
    }
  }
#pragma unroll
  for (int k = 0; k < kMaxTaps; ++k)
    if (k < keep) st[static_cast<int64_t>(k) * width + c] = next[k];
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_causal_conv(void* stream, const void* in, int act_dtype, int64_t in_row, const float* in_bias,
                                 const float* conv_w, const float* conv_b, float* u, const float* state,
                                 int64_t state_row, const int32_t* tok_item, const int32_t* item_start,
                                 const int32_t* slots, int64_t tokens, int width, int taps) {
  PSAMD_REQUIRE(tokens >= 0 && width > 0 && taps >= 1 && taps <= kMaxTaps, "bad sizes (at most 16 taps)");
  PSAMD_REQUIRE(in_row >= width && state_row >= static_cast<int64_t>(taps) * width, "rows too short");
  PSAMD_REQUIRE(tokens <= 2147483647LL && ceil_div(width, 256) <= 65535, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(tokens), static_cast<unsigned>(ceil_div(width, 256)));
  if (act_dtype == kBF16) {
    causal_conv_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(in), in_row, in_bias, conv_w, conv_b, u,
                                                         state, state_row, tok_item, item_start, slots, width, taps);
  } else if (act_dtype == kF32) {
    causal_conv_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(in), in_row, in_bias, conv_w, conv_b, u,
                                                        state, state_row, tok_item, item_start, slots, width, taps);
  } else {
    return fail("psamd_causal_conv: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_causal_conv");
}

extern "C" int psamd_gated_scan(void* stream, const float* gates, const float* gate_b, const float* u, const float* decay,
                                const void* y, const void* x, int act_dtype, int64_t in_row, const float* y_bias,
                                const float* x_bias, void* out, float* state, int64_t state_row,
                                const int32_t* item_start, const int32_t* slots, int items, int width, int blocks,
                                int taps) {
  PSAMD_REQUIRE(items >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "bad sizes");
  PSAMD_REQUIRE(taps >= 1 && taps <= kMaxTaps, "at most 16 taps");
  PSAMD_REQUIRE(in_row >= width && state_row >= static_cast<int64_t>(taps) * width, "rows too short");
  PSAMD_REQUIRE(ceil_div(width, 256) <= 65535, "too large for one launch");
  if (items == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(items), static_cast<unsigned>(ceil_div(width, 256)));
  if (act_dtype == kBF16) {
    gated_scan_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(gates, gate_b, u, decay, static_cast<const bf16_t*>(y),
                                                        static_cast<const bf16_t*>(x), in_row, y_bias, x_bias,
                                                        static_cast<bf16_t*>(out), state, state_row, item_start, slots,
                                                        width, blocks, taps);
  } else if (act_dtype == kF32) {
    gated_scan_kernel<float><<<grid, dim3(256), 0, s>>>(gates, gate_b, u, decay, static_cast<const float*>(y),
                                                       static_cast<const float*>(x), in_row, y_bias, x_bias,
                                                       static_cast<float*>(out), state, state_row, item_start, slots,
                                                       width, blocks, taps);
  } else {
    return fail("psamd_gated_scan: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_gated_scan");
}
