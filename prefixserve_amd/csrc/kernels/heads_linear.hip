// One small matrix product per head: out[t, h, n] = sum_k x[t, h, k] * w[h, n, k].
//
// What latent attention needs twice (a head's query folded into the compressed space, and the
// compressed result unfolded into the head's values) and what a recurrence with block-diagonal
// gate matrices needs once. Rows of x and out are strided, so that a head's operand may sit
// inside a wider row and its result may land inside another.
//
// Two forms. LDS-tiled FMA with float accumulation for any element types, the 32-bit path's
// product: k is summed in ascending order whatever the number of tokens, so a token's 32-bit
// result does not depend on what else is in the step. And, for bfloat16 operands whose rows start
// on 16-byte boundaries, v_mfma_f32_16x16x32_bf16 with both operands straight from memory (they
// are small: a head's matrix stays in L2 for all its tokens): a wave owns 16 tokens and NT tiles
// of 16 output columns, so the tokens' fragment serves NT matrix instructions.

#include "api.h"
#include "common.h"

namespace psamd {

template <typename TX, typename TW, typename TO>
__global__ __launch_bounds__(256) void heads_linear_kernel(const TX* __restrict__ x, int64_t x_row, int x_head,
                                                           const TW* __restrict__ w, TO* __restrict__ out, int64_t o_row,
                                                           int o_head, int64_t M, int N, int K) {
  constexpr int BM = 64, BN = 64, BK = 16;
  __shared__ float xs[BK][BM + 1];
  __shared__ float wsm[BK][BN + 1];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int h = blockIdx.z;
  const int64_t m0 = static_cast<int64_t>(blockIdx.y) * BM;
  const int n0 = blockIdx.x * BN;
  x += static_cast<int64_t>(h) * x_head;
  w += static_cast<int64_t>(h) * N * K;
  out += static_cast<int64_t>(h) * o_head;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int e = tid + i * 256;
      const int r = e / BK, k = e % BK;
      const bool kin = k0 + k < K;
      xs[k][r] = (kin && m0 + r < M) ? to_float<TX>(x[(m0 + r) * x_row + k0 + k]) : 0.f;
      wsm[k][r] = (kin && n0 + r < N) ? to_float<TW>(w[static_cast<int64_t>(n0 + r) * K + k0 + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = wsm[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int64_t m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) out[m * o_row + n] = from_float<TO>(acc[i][j]);
    }
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

// Operand layout of the instruction: lane l supplies row l % 16, k = 8 * (l / 16) + [0, 8) of both
// operands and receives C[4 * (l / 16) + v][l % 16]; C's rows are rows of w, its columns tokens.
template <int NT>
__global__ __launch_bounds__(256) void heads_linear_mfma_kernel(const bf16_t* __restrict__ x, int64_t x_row, int x_head,
                                                                const bf16_t* __restrict__ w, bf16_t* __restrict__ out,
                                                                int64_t o_row, int o_head, int64_t M, int N, int K) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int h = blockIdx.z;
  const int64_t m0 = (static_cast<int64_t>(blockIdx.y) * 4 + wave) * 16;
  if (m0 >= M) return;
  const int n0 = blockIdx.x * NT * 16;
  const bf16_t* xr = x + static_cast<int64_t>(h) * x_head + min(m0 + r, M - 1) * x_row + 8 * g;
  const bf16_t* wr[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    wr[nt] = w + (static_cast<int64_t>(h) * N + min(n0 + nt * 16 + r, N - 1)) * K + 8 * g;
  f32x4 acc[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) acc[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = static_cast<__bf16>(0.f);
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool in = k0 + 8 * g < K;                   // K is a multiple of 8: a piece is inside or outside
    const bf16x8 b = in ? *reinterpret_cast<const bf16x8*>(xr + k0) : zero;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const bf16x8 a = in ? *reinterpret_cast<const bf16x8*>(wr[nt] + k0) : zero;
      acc[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[nt], 0, 0, 0);
    }
  }
  const int64_t m = m0 + r;
  if (m >= M) return;
  bf16_t* o = out + static_cast<int64_t>(h) * o_head + m * o_row;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int n = n0 + nt * 16 + 4 * g + v;
      if (n < N) o[n] = float_to_bf16(acc[nt][v]);
    }
}

template <typename T>
static int launch_heads(hipStream_t s, const void* x, int64_t x_row, int x_head, const void* w, void* out, int64_t o_row,
                        int o_head, int64_t M, int H, int N, int K) {
  const dim3 grid(static_cast<unsigned>(ceil_div(N, 64)), static_cast<unsigned>(ceil_div(M, 64)), static_cast<unsigned>(H));
  heads_linear_kernel<T, T, T><<<grid, dim3(256), 0, s>>>(static_cast<const T*>(x), x_row, x_head, static_cast<const T*>(w),
                                                          static_cast<T*>(out), o_row, o_head, M, N, K);
  return check_launch("psamd_heads_linear");
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_heads_linear(void* stream, const void* x, int x_dtype, int64_t x_row, int x_head, const void* w,
                                  int w_dtype, void* out, int out_dtype, int64_t out_row, int out_head, int64_t M, int H,
                                  int N, int K) {
  PSAMD_REQUIRE(M >= 0 && H > 0 && N > 0 && K > 0, "bad sizes");
  PSAMD_REQUIRE(H <= 65535 && ceil_div(M, 64) <= 65535, "too large for one launch");
  PSAMD_REQUIRE(x_head >= 0 && out_head >= 0 && x_row >= static_cast<int64_t>(H - 1) * x_head + K &&
                out_row >= static_cast<int64_t>(H - 1) * out_head + N, "rows too short for their heads");
  PSAMD_REQUIRE(x_dtype == w_dtype && x_dtype == out_dtype, "x, w and out must have one dtype");
  if (M == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (x_dtype == kBF16 && K % 8 == 0 && x_row % 8 == 0 && x_head % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
      reinterpret_cast<uintptr_t>(w) % 16 == 0 && ceil_div(M, 64) <= 65535) {
    constexpr int NT = 4;
    const dim3 grid(static_cast<unsigned>(ceil_div(N, 16 * NT)), static_cast<unsigned>(ceil_div(M, 64)), static_cast<unsigned>(H));
    heads_linear_mfma_kernel<NT><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(x), x_row, x_head,
                                                           static_cast<const bf16_t*>(w), static_cast<bf16_t*>(out), out_row,
                                                           out_head, M, N, K);
    return check_launch("psamd_heads_linear");
  }
  if (x_dtype == kBF16) return launch_heads<bf16_t>(s, x, x_row, x_head, w, out, out_row, out_head, M, H, N, K);
  if (x_dtype == kF32) return launch_heads<float>(s, x, x_row, x_head, w, out, out_row, out_head, M, H, N, K);
  return fail("psamd_heads_linear: dtype must be float32 or bfloat16");
}
