// Mixture-of-experts feed-forward: the router, and the experts one (token, choice) pair at a
// time. The pair form reads an expert's matrices once per pair, which is what a decode step
// needs (a handful of tokens, each with its own experts) and what the 32-bit path uses at every
// size; it is templated on the element type (bfloat16 or float) and sums in float.
//
// Router: score = sigmoid(x . w_r[e]) in float; the `top` largest are taken, the lower index
// among equals. Expert: with h = weight * x, g = min(gate h, limit), u = clamp(up h, -limit, limit),
// act = g * sigmoid(gate_alpha * g) * (u + up_shift), out = down act. The weight multiplies the
// expert's input, so it cannot be pulled out of the clamps.

#include <algorithm>

#include "api.h"
#include "common.h"

namespace psamd {

// Dot product of a row of n elements with a float vector in LDS, dealt out over the 64 lanes;
// every lane returns the whole sum. bfloat16 rows whose length is a multiple of 8 are read in
// 16-byte pieces.
template <typename W>
__device__ __forceinline__ float wave_dot(const W* __restrict__ row, const float* __restrict__ xs, int n, int lane) {
  float acc = 0.f;
  if (sizeof(W) == 2 && (n & 7) == 0 && (reinterpret_cast<uintptr_t>(row) & 15) == 0) {
    const int chunks = n >> 3;
    for (int c = lane; c < chunks; c += kWave) {
      const uint4 q = *reinterpret_cast<const uint4*>(reinterpret_cast<const bf16_t*>(row) + 8 * c);
      const uint32_t w4[4] = {q.x, q.y, q.z, q.w};
      const float* xp = xs + 8 * c;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        acc = fmaf(__uint_as_float(w4[i] << 16), xp[2 * i], acc);
        acc = fmaf(__uint_as_float(w4[i] & 0xffff0000u), xp[2 * i + 1], acc);
      }
    }
  } else {
    for (int i = lane; i < n; i += kWave) acc = fmaf(to_float<W>(row[i]), xs[i], acc);
  }
  return wave_sum(acc);
}

// ------------------------------------------------------------------ router

// One block of four waves per token: the waves share the experts' dot products, then wave 0
// picks the `top` largest scores one after the other (each pick: a strided scan and a wave
// reduction that prefers the lower index among equals).
template <typename A>
__global__ __launch_bounds__(256) void moe_route_kernel(const A* __restrict__ x, const float* __restrict__ w_router,
                                                        int32_t* __restrict__ chosen, float* __restrict__ weight,
                                                        int K, int experts, int top) {
  extern __shared__ __align__(16) float route_smem[];    // xs[K], score[experts]
  float* xs = route_smem;
  float* score = route_smem + K;
  const int64_t t = blockIdx.x;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  for (int i = threadIdx.x; i < K; i += blockDim.x) xs[i] = to_float<A>(x[t * K + i]);
  __syncthreads();
  for (int e = wave; e < experts; e += 4) {
    const float z = wave_dot<float>(w_router + static_cast<int64_t>(e) * K, xs, K, lane);
    if (lane == 0) score[e] = 1.f / (1.f + expf(-z));
  }
  __syncthreads();
  if (wave != 0) return;
  for (int j = 0; j < top; ++j) {
    float best = -1.f;                                   // scores lie in [0, 1]; taken ones are set to -2
    int at = 0x7fffffff;
    for (int e = lane; e < experts; e += kWave) {
      const float s = score[e];
      if (s > best) {                                    // ascending e: the first of equals stays
        best = s;
        at = e;
      }
    }
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, kWave);
      const int oa = __shfl_xor(at, o, kWave);
      if (ob > best || (ob == best && oa < at)) {
        best = ob;
        at = oa;
      }
    }
    if (lane == 0) {
      chosen[t * top + j] = at;
      weight[t * top + j] = best;
      score[at] = -2.f;
    }
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
  }
}

// ------------------------------------------------------------------ experts, pair by pair

constexpr int kRowsPerWave = 4;
constexpr int kRowsPerBlock = 4 * kRowsPerWave;

// grid (pairs, ceil(F / 16)): the block stages h = weight * x[t] in LDS and each wave computes
// kRowsPerWave activations of the pair's expert.
template <typename A>
__global__ __launch_bounds__(256) void moe_gate_up_rows_kernel(
    const A* __restrict__ x, const int32_t* __restrict__ chosen, const float* __restrict__ weight,
    const A* __restrict__ w_gate_up, A* __restrict__ act, int K, int F, int experts, int top, float gate_alpha,
    float limit, float up_shift) {
  extern __shared__ __align__(16) float rows_smem[];     // h[K]
  const int64_t pair = blockIdx.x;
  const int64_t t = pair / top;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int e = min(max(chosen[pair], 0), experts - 1);
  const float wgt = weight[pair];
  for (int i = threadIdx.x; i < K; i += blockDim.x) rows_smem[i] = wgt * to_float<A>(x[t * K + i]);
  __syncthreads();
  const A* we = w_gate_up + static_cast<int64_t>(e) * 2 * F * K;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int f = static_cast<int>(blockIdx.y) * kRowsPerBlock + wave * kRowsPerWave + r;
    if (f >= F) break;
    float g = wave_dot<A>(we + static_cast<int64_t>(f) * K, rows_smem, K, lane);
    float u = wave_dot<A>(we + static_cast<int64_t>(F + f) * K, rows_smem, K, lane);
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
    if (lane == 0) act[pair * F + f] = from_float<A>(g / (1.f + expf(-gate_alpha * g)) * (u + up_shift));
  }
}

// grid (pairs, ceil(K / 16)): out[j][t][k] = down[e][k] . act[pair].
template <typename A>
__global__ __launch_bounds__(256) void moe_down_rows_kernel(
    const A* __restrict__ act, const int32_t* __restrict__ chosen, const A* __restrict__ w_down,
    float* __restrict__ out, int64_t tokens, int K, int F, int experts, int top) {
  extern __shared__ __align__(16) float rows_smem[];     // act[F]
  const int64_t pair = blockIdx.x;
  const int64_t t = pair / top;
  const int j = static_cast<int>(pair - t * top);
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x >> 6;
  const int e = min(max(chosen[pair], 0), experts - 1);
  for (int i = threadIdx.x; i < F; i += blockDim.x) rows_smem[i] = to_float<A>(act[pair * F + i]);
  __syncthreads();
  const A* we = w_down + static_cast<int64_t>(e) * K * F;
  float* o = out + (static_cast<int64_t>(j) * tokens + t) * K;
#pragma unroll
  for (int r = 0; r < kRowsPerWave; ++r) {
    const int k = static_cast<int>(blockIdx.y) * kRowsPerBlock + wave * kRowsPerWave + r;
    if (k >= K) break;
    const float v = wave_dot<A>(we + static_cast<int64_t>(k) * F, rows_smem, F, lane);
    if (lane == 0) o[k] = v;
  }
}

template <typename A>
static int launch_experts_rows(hipStream_t s, const void* x, const int32_t* chosen, const float* weight,
                               const void* w_gate_up, const void* w_down, void* act, float* out, int64_t tokens, int K,
                               int F, int experts, int top, float gate_alpha, float limit, float up_shift) {
  const unsigned pairs = static_cast<unsigned>(tokens * top);
  moe_gate_up_rows_kernel<A><<<dim3(pairs, static_cast<unsigned>(ceil_div(F, kRowsPerBlock))), dim3(256),
                               sizeof(float) * K, s>>>(
      static_cast<const A*>(x), chosen, weight, static_cast<const A*>(w_gate_up), static_cast<A*>(act), K, F, experts, top,
      gate_alpha, limit, up_shift);
  if (check_launch("psamd_moe_experts_rows (gate/up)")) return 1;
  moe_down_rows_kernel<A><<<dim3(pairs, static_cast<unsigned>(ceil_div(K, kRowsPerBlock))), dim3(256), sizeof(float) * F,
                            s>>>(static_cast<const A*>(act), chosen, static_cast<const A*>(w_down), out, tokens, K, F,
                                 experts, top);
  return check_launch("psamd_moe_experts_rows (down)");
}

}  // namespace psamd

using namespace psamd;

extern "C" {

int psamd_moe_route(void* stream, const void* x, int x_dtype, const float* w_router, int32_t* chosen, float* weight,
                    int64_t tokens, int K, int experts, int top) {
  PSAMD_REQUIRE(tokens >= 0 && K > 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * (static_cast<size_t>(K) + experts) <= 64 * 1024, "row and scores do not fit in LDS");
  PSAMD_REQUIRE(tokens <= 2147483647LL, "too many tokens for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const size_t smem = sizeof(float) * (static_cast<size_t>(K) + experts);
  const dim3 grid(static_cast<unsigned>(tokens));
  if (x_dtype == kBF16) {
    moe_route_kernel<bf16_t><<<grid, dim3(256), smem, s>>>(static_cast<const bf16_t*>(x), w_router, chosen, weight, K,
                                                          experts, top);
  } else if (x_dtype == kF32) {
    moe_route_kernel<float><<<grid, dim3(256), smem, s>>>(static_cast<const float*>(x), w_router, chosen, weight, K,
                                                         experts, top);
  } else {
    return fail("psamd_moe_route: x must be float32 or bfloat16");
  }
  return check_launch("psamd_moe_route");
}

int psamd_moe_experts_rows(void* stream, const void* x, const int32_t* chosen, const float* weight,
                           const void* w_gate_up, const void* w_down, void* act, float* out, int dtype,
                           int64_t tokens, int K, int F, int experts, int top, float gate_alpha, float limit,
                           float up_shift) {
  PSAMD_REQUIRE(tokens >= 0 && K > 0 && F > 0 && experts > 0 && top >= 1 && top <= experts, "bad sizes");
  PSAMD_REQUIRE(sizeof(float) * static_cast<size_t>(std::max(K, F)) <= 64 * 1024, "a row does not fit in LDS");
  PSAMD_REQUIRE(tokens * top <= 2147483647LL && ceil_div(std::max(K, F), kRowsPerBlock) <= 65535, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (dtype == kBF16)
    return launch_experts_rows<bf16_t>(s, x, chosen, weight, w_gate_up, w_down, act, out, tokens, K, F, experts, top,
                                       gate_alpha, limit, up_shift);
  if (dtype == kF32)
    return launch_experts_rows<float>(s, x, chosen, weight, w_gate_up, w_down, act, out, tokens, K, F, experts, top,
                                      gate_alpha, limit, up_shift);
  return fail("psamd_moe_experts_rows: dtype must be float32 or bfloat16");
}

}  // extern "C"
