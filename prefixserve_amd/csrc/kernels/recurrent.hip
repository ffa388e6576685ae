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

// One token of the recurrence: the decay a and what flows in, from the gates' sums.
__device__ __forceinline__ void scan_terms(float gr, float gi, float dec, float u, float& a, float& inflow) {
  const float r = sigmoid_f(gr), g = sigmoid_f(gi);
  const float la = dec * r;
  a = expf(la);
  inflow = sqrtf(-expm1f(2.f * la)) * g * u;
}

// The state's saved inputs after an item's step: the last taps - 1 of (saved before, then this step's).
template <typename A>
__device__ __forceinline__ void save_inputs(float* st, const A* x, int64_t in_row, int64_t s0, int n, int taps, int width,
                                            int c, float xb) {
  const int keep = taps - 1;
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

// The whole of each listed item, token after token: a thread per (item, channel). For items of one
// token (decoding), where there is nothing to share out. `list` (or NULL: every item) names the items.
template <typename A>
__global__ __launch_bounds__(256) void gated_scan_kernel(
    const float* __restrict__ gates, const float* __restrict__ gate_b, const float* __restrict__ u,
    const float* __restrict__ decay, const A* __restrict__ y, const A* __restrict__ x, int64_t in_row,
    const float* __restrict__ y_bias, const float* __restrict__ x_bias, A* __restrict__ out, float* __restrict__ state,
    int64_t state_row, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ list, int width, int blocks, int taps) {
  const int item = list != nullptr ? list[blockIdx.x] : blockIdx.x;
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
    float a, inflow;
    scan_terms(gates[t * 2 * width + g_off] + br, gates[t * 2 * width + g_off + bw] + bi, dec, u[t * width + c], a, inflow);
    S = fmaf(a, S, inflow);
    out[t * width + c] = from_float<A>(S * gelu_tanh_f(to_float<A>(y[t * in_row + c]) + yb));
  }
  st[static_cast<int64_t>(taps - 1) * width + c] = S;
  save_inputs<A>(st, x, in_row, s0, static_cast<int>(s1 - s0), taps, width, c, x_bias[c]);
}

// Items of more than one token, cut into the step's tiles of `tile` tokens (tiles[k] = (item, first
// token of the tile within the item); the tiles of an item follow each other): a thread per (tile,
// channel). The recurrence S <- a S + b is linear in S, so a tile can be summed up from S = 0 as the
// pair (product of its a, its own sum): pass 0 leaves that pair per tile and channel, and the state the
// item started from; pass 1 folds the pairs of the tiles in front of its own (in order, from the
// item's starting state), runs its tile from there and writes the outputs; the item's last tile
// leaves the new state in the slot.
template <typename A, int PASS>
__global__ __launch_bounds__(256) void gated_scan_tiles_kernel(
    const float* __restrict__ gates, const float* __restrict__ gate_b, const float* __restrict__ u,
    const float* __restrict__ decay, const A* __restrict__ y, const A* __restrict__ x, int64_t in_row,
    const float* __restrict__ y_bias, const float* __restrict__ x_bias, A* __restrict__ out, float* __restrict__ state,
    int64_t state_row, const int32_t* __restrict__ item_start, const int32_t* __restrict__ slots,
    const int32_t* __restrict__ tiles, int tile, float* __restrict__ carry, int n_tiles, int width, int blocks, int taps) {
  const int k = blockIdx.x;
  const int c = blockIdx.y * 256 + threadIdx.x;
  if (c >= width) return;
  const int item = tiles[2 * k], q0 = tiles[2 * k + 1];
  const int bw = width / blocks;
  const int b = c / bw, cb = c - b * bw;
  const int64_t s0 = item_start[item];
  const int len = static_cast<int>(item_start[item + 1] - s0);
  const int n = min(tile, len - q0);
  const int64_t g_off = static_cast<int64_t>(b) * 2 * bw + cb;
  const float br = gate_b[g_off], bi = gate_b[g_off + bw];
  const float dec = decay[c];
  float* st = state + static_cast<int64_t>(slots[item]) * state_row;
  float* prod = carry;                                          // [n_tiles][width]
  float* sum = carry + static_cast<int64_t>(n_tiles) * width;   // [n_tiles][width]
  float* begin = carry + 2LL * n_tiles * width;                 // [n_tiles][width]: the item's starting state, at its first tile
  if (PASS == 0) {
    float P = 1.f, B = 0.f;
    // Eight tokens' operands are asked for together (they do not depend on the sums), then folded in order.
    for (int64_t t8 = s0 + q0; t8 < s0 + q0 + n; t8 += 8) {
      float gr[8], gi[8], uu[8];
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const int64_t t = min(t8 + i, s0 + q0 + n - 1);
        gr[i] = gates[t * 2 * width + g_off];
        gi[i] = gates[t * 2 * width + g_off + bw];
        uu[i] = u[t * width + c];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (t8 + i < s0 + q0 + n) {
          float a, inflow;
          scan_terms(gr[i] + br, gi[i] + bi, dec, uu[i], a, inflow);
          B = fmaf(a, B, inflow);
          P *= a;
        }
      }
    }
    prod[static_cast<int64_t>(k) * width + c] = P;
    sum[static_cast<int64_t>(k) * width + c] = B;
    if (q0 == 0) begin[static_cast<int64_t>(k) * width + c] = st[static_cast<int64_t>(taps - 1) * width + c];
    return;
  }
  const int first = k - q0 / tile;
  float S = begin[static_cast<int64_t>(first) * width + c];
  for (int j = first; j < k; ++j) S = fmaf(prod[static_cast<int64_t>(j) * width + c], S, sum[static_cast<int64_t>(j) * width + c]);
  const float yb = y_bias[c];
  for (int64_t t8 = s0 + q0; t8 < s0 + q0 + n; t8 += 8) {
    float gr[8], gi[8], uu[8], yy[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int64_t t = min(t8 + i, s0 + q0 + n - 1);
      gr[i] = gates[t * 2 * width + g_off];
      gi[i] = gates[t * 2 * width + g_off + bw];
      uu[i] = u[t * width + c];
      yy[i] = to_float<A>(y[t * in_row + c]);
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (t8 + i < s0 + q0 + n) {
        float a, inflow;
        scan_terms(gr[i] + br, gi[i] + bi, dec, uu[i], a, inflow);
        S = fmaf(a, S, inflow);
        out[(t8 + i) * width + c] = from_float<A>(S * gelu_tanh_f(yy[i] + yb));
      }
    }
  }
  if (q0 + n == len) {
    st[static_cast<int64_t>(taps - 1) * width + c] = S;
    save_inputs<A>(st, x, in_row, s0, len, taps, width, c, x_bias[c]);
  }
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

template <typename A>
static int launch_scan(hipStream_t s, const float* gates, const float* gate_b, const float* u, const float* decay,
                       const void* y, const void* x, int64_t in_row, const float* y_bias, const float* x_bias, void* out,
                       float* state, int64_t state_row, const int32_t* item_start, const int32_t* slots, int items,
                       const int32_t* tiles, int n_tiles, int tile, const int32_t* singles, int n_singles, float* carry,
                       int width, int blocks, int taps) {
  const unsigned cb = static_cast<unsigned>(ceil_div(width, 256));
  const A* yp = static_cast<const A*>(y);
  const A* xp = static_cast<const A*>(x);
  A* op = static_cast<A*>(out);
  if (tiles == nullptr) {       // every item whole, token after token
    gated_scan_kernel<A><<<dim3(items, cb), dim3(256), 0, s>>>(gates, gate_b, u, decay, yp, xp, in_row, y_bias, x_bias, op, state,
                                                            state_row, item_start, slots, nullptr, width, blocks, taps);
    return check_launch("psamd_gated_scan");
  }
  if (n_tiles > 0) {
    gated_scan_tiles_kernel<A, 0><<<dim3(n_tiles, cb), dim3(256), 0, s>>>(gates, gate_b, u, decay, yp, xp, in_row, y_bias, x_bias,
                                                                      op, state, state_row, item_start, slots, tiles, tile,
                                                                      carry, n_tiles, width, blocks, taps);
    gated_scan_tiles_kernel<A, 1><<<dim3(n_tiles, cb), dim3(256), 0, s>>>(gates, gate_b, u, decay, yp, xp, in_row, y_bias, x_bias,
                                                                      op, state, state_row, item_start, slots, tiles, tile,
                                                                      carry, n_tiles, width, blocks, taps);
  }
  if (n_singles > 0)
    gated_scan_kernel<A><<<dim3(n_singles, cb), dim3(256), 0, s>>>(gates, gate_b, u, decay, yp, xp, in_row, y_bias, x_bias, op,
                                                                state, state_row, item_start, slots, singles, width, blocks, taps);
  return check_launch("psamd_gated_scan");
}

extern "C" int psamd_gated_scan(void* stream, const float* gates, const float* gate_b, const float* u, const float* decay,
                                const void* y, const void* x, int act_dtype, int64_t in_row, const float* y_bias,
                                const float* x_bias, void* out, float* state, int64_t state_row,
                                const int32_t* item_start, const int32_t* slots, int items, const int32_t* tiles,
                                int n_tiles, int tile, const int32_t* singles, int n_singles, float* carry, int width,
                                int blocks, int taps) {
  PSAMD_REQUIRE(items >= 0 && width > 0 && blocks > 0 && width % blocks == 0, "bad sizes");
  PSAMD_REQUIRE(taps >= 1 && taps <= kMaxTaps, "at most 16 taps");
  PSAMD_REQUIRE(in_row >= width && state_row >= static_cast<int64_t>(taps) * width, "rows too short");
  PSAMD_REQUIRE(ceil_div(width, 256) <= 65535, "too large for one launch");
  PSAMD_REQUIRE(tiles == nullptr || (n_tiles >= 0 && n_singles >= 0 && tile >= 1 && (n_tiles == 0 || carry != nullptr) &&
                                     (n_singles == 0 || singles != nullptr)), "tiles need their size, the singles' list and room for the carries");
  if (items == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (act_dtype == kBF16)
    return launch_scan<bf16_t>(s, gates, gate_b, u, decay, y, x, in_row, y_bias, x_bias, out, state, state_row, item_start, slots,
                               items, tiles, n_tiles, tile, singles, n_singles, carry, width, blocks, taps);
  if (act_dtype == kF32)
    return launch_scan<float>(s, gates, gate_b, u, decay, y, x, in_row, y_bias, x_bias, out, state, state_row, item_start, slots,
                              items, tiles, n_tiles, tile, singles, n_singles, carry, width, blocks, taps);
  return fail("psamd_gated_scan: activation dtype must be float32 or bfloat16");
}
