// Latent attention's step between its input product and the attention itself: the token's
// compressed vector is normalized and, with the rotated key part all heads share, written to
// the token's place in the paged cache; every head's rotated query part is laid into the query
// the attention kernels read.
//
// The cache holds one "head" per token, `slots` wide: the key is [compressed (rank) | rotated
// part (rot) | zeros], the value (transposed in the page, as for every attention here) is
// [compressed | zeros]. A head's query is [its un-rotated part folded into the compressed
// space (rank, written by the product that follows) | its rotated part | zeros], so that
// query . key is the head's whole score and the weighted sum of values is the weighted sum of
// compressed vectors, which a product per head then unfolds.
//
// The rotation pairs neighbours, (2i, 2i + 1); statistics, rotation and norm are float.

#include "api.h"
#include "common.h"

namespace psamd {

template <typename A>
__global__ __launch_bounds__(256) void latent_kv_append_kernel(
    const A* __restrict__ in, int64_t in_row, A* __restrict__ q_lat, int hq, int dim, int rot, int rank, int slots,
    const int32_t* __restrict__ positions, const float2* __restrict__ table, const float* __restrict__ norm_w, float eps,
    A* __restrict__ kv, const int32_t* __restrict__ write_slot) {
  __shared__ float scratch[4];
  const int64_t t = blockIdx.x;
  const int tid = threadIdx.x;
  const A* row = in + t * in_row;
  const A* low = row + static_cast<int64_t>(hq) * (dim + rot);      // [rank | rot]
  const int pos = positions[t];
  const int pairs = rot >> 1;
  const float2* cs = table + static_cast<int64_t>(pos) * pairs;

  float ss = 0.f;
  for (int i = tid; i < rank; i += 256) {
    const float v = to_float<A>(low[i]);
    ss += v * v;
  }
  ss = block_sum(ss, scratch, 4);
  const float inv = rsqrtf(ss / static_cast<float>(rank) + eps);

  if (kv != nullptr) {
    const int slot = write_slot[t];
    const int64_t page = slot / kPage;
    const int off = slot % kPage;
    A* kpage = kv + page * (2LL * kPage * slots) + static_cast<int64_t>(off) * slots;      // [16][slots]
    A* vpage = kv + page * (2LL * kPage * slots) + static_cast<int64_t>(kPage) * slots + off;   // [slots][16]
    for (int i = tid; i < slots; i += 256) {
      A key = from_float<A>(0.f), val = from_float<A>(0.f);
      if (i < rank) {
        key = val = from_float<A>(to_float<A>(low[i]) * inv * norm_w[i]);
      } else if (i < rank + rot) {
        const int p = (i - rank) >> 1;
        const float u = to_float<A>(low[rank + 2 * p]), v = to_float<A>(low[rank + 2 * p + 1]);
        const float2 c = cs[p];
        key = from_float<A>(((i - rank) & 1) ? v * c.x + u * c.y : u * c.x - v * c.y);
      }
      kpage[i] = key;
      vpage[static_cast<int64_t>(i) * kPage] = val;
    }
  }

  // Every head's rotated query part and the zeros behind it.
  const int tail = slots - rank;
  A* q_out = q_lat + t * (static_cast<int64_t>(hq) * slots);
  for (int e = tid; e < hq * tail; e += 256) {
    const int h = e / tail, i = e - h * tail;
    A val = from_float<A>(0.f);
    if (i < rot) {
      const A* q = row + static_cast<int64_t>(h) * (dim + rot) + dim;
      const int p = i >> 1;
      const float u = to_float<A>(q[2 * p]), v = to_float<A>(q[2 * p + 1]);
      const float2 c = cs[p];
      val = from_float<A>((i & 1) ? v * c.x + u * c.y : u * c.x - v * c.y);
    }
    q_out[static_cast<int64_t>(h) * slots + rank + i] = val;
  }
}

}  // namespace psamd

using namespace psamd;

extern "C" int psamd_latent_kv_append(void* stream, const void* in, int64_t in_row, void* q_lat, int act_dtype,
                                      int64_t tokens, int hq, int dim, int rot, int rank, int slots,
                                      const int32_t* positions, const float* table, const float* norm_w, float eps,
                                      void* kv, const int32_t* write_slot) {
  PSAMD_REQUIRE(tokens >= 0 && hq > 0 && dim >= 0 && rank > 0 && rot >= 0 && rot % 2 == 0, "bad sizes");
  PSAMD_REQUIRE(slots >= rank + rot, "a slot must hold the compressed vector and the rotated part");
  PSAMD_REQUIRE(in_row >= static_cast<int64_t>(hq) * (dim + rot) + rank + rot, "input rows too short");
  PSAMD_REQUIRE(rot == 0 || table != nullptr, "a rotated part needs its table");
  PSAMD_REQUIRE(positions != nullptr && norm_w != nullptr, "positions and the norm's weight are needed");
  PSAMD_REQUIRE(kv == nullptr || write_slot != nullptr, "a cache needs write slots");
  PSAMD_REQUIRE(tokens <= 2147483647LL, "too large for one launch");
  if (tokens == 0) return 0;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float2* tab = reinterpret_cast<const float2*>(table);
  const dim3 grid(static_cast<unsigned>(tokens));
  if (act_dtype == kBF16) {
    latent_kv_append_kernel<bf16_t><<<grid, dim3(256), 0, s>>>(static_cast<const bf16_t*>(in), in_row,
                                                              static_cast<bf16_t*>(q_lat), hq, dim, rot, rank, slots,
                                                              positions, tab, norm_w, eps, static_cast<bf16_t*>(kv), write_slot);
  } else if (act_dtype == kF32) {
    latent_kv_append_kernel<float><<<grid, dim3(256), 0, s>>>(static_cast<const float*>(in), in_row,
                                                             static_cast<float*>(q_lat), hq, dim, rot, rank, slots,
                                                             positions, tab, norm_w, eps, static_cast<float*>(kv), write_slot);
  } else {
    return fail("psamd_latent_kv_append: activation dtype must be float32 or bfloat16");
  }
  return check_launch("psamd_latent_kv_append");
}
