// On-device random tensors: uniform, normal, log-normal and Bernoulli draws
// from the counter-based generator Philox4x32-10 (Salmon, Moraes, Dror, Shaw:
// "Parallel Random Numbers: As Easy as 1, 2, 3", SC'11).  The generator has no
// state in memory: element i of a call takes word i%4 of the 128-bit block
// whose counter is offset + i/4 under the 64-bit key `seed`, so a tensor is
// filled by one streaming kernel, the result depends only on (seed, offset, i),
// and a prefix of a longer draw equals the shorter draw.
#include "phip_pointwise.h"

namespace phip {
namespace {

using namespace pointwise;

struct Block { uint32_t w[4]; };

__device__ inline Block philox4x32_10(uint64_t counter, uint64_t key) {
  uint32_t c0 = (uint32_t)counter, c1 = (uint32_t)(counter >> 32), c2 = 0, c3 = 0;
  uint32_t k0 = (uint32_t)key, k1 = (uint32_t)(key >> 32);
#pragma unroll
  for (int round = 0; round < 10; ++round) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    c1 = (uint32_t)p1;
    c3 = (uint32_t)p0;
    c0 = n0;
    c2 = n2;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  return {{c0, c1, c2, c3}};
}

// 24 random bits -> (0, 1]: every value is a multiple of 2^-24 and exact in fp32.
__device__ inline float unit_interval(uint32_t w) { return (float)((w >> 8) + 1u) * 5.9604644775390625e-8f; }

enum class Draw { Uniform, Bernoulli, Normal, LogNormal };

// Element e (0..3) of a block for the requested distribution.
template <Draw DRAW>
__device__ inline float draw(const Block &b, int e, float p0, float p1) {
  if constexpr (DRAW == Draw::Uniform) {
    return fmaf(unit_interval(b.w[e]), p1 - p0, p0);                // (lower, upper], one rounding
  } else if constexpr (DRAW == Draw::Bernoulli) {
    return unit_interval(b.w[e]) <= p0 ? 1.f : 0.f;
  } else {
    // Box-Muller on the word pair (0,1) or (2,3): cosine for the even element, sine for the odd
    const float u = unit_interval(b.w[e & 2]), v = unit_interval(b.w[(e & 2) + 1]);
    const float r = sqrtf(-2.f * logf(u));
    const float t = 6.283185307179586f * v;
    const float z = fmaf(r * ((e & 1) ? sinf(t) : cosf(t)), p1, p0);
    return DRAW == Draw::LogNormal ? expf(z) : z;
  }
}

template <typename T, Draw DRAW>
__global__ __launch_bounds__(kBlock) void random_kernel(T *y, size_t n, uint64_t seed, uint64_t offset, float p0,
                                                         float p1) {
  const size_t blocks = (n + 3) / 4;
  const bool aligned = reinterpret_cast<uintptr_t>(y) % (4 * sizeof(T)) == 0;
  for (size_t q = (size_t)blockIdx.x * kBlock + threadIdx.x; q < blocks; q += (size_t)gridDim.x * kBlock) {
    const Block b = philox4x32_10(offset + q, seed);
    // a block's four results leave as one store (y is aligned to four elements); the last block may be short
    struct alignas(4 * sizeof(T)) Quad {
      T v[4];
    } out;
#pragma unroll
    for (int e = 0; e < 4; ++e) out.v[e] = from_f32<T>(draw<DRAW>(b, e, p0, p1));
    if (q * 4 + 4 <= n && aligned) {
      *reinterpret_cast<Quad *>(y + q * 4) = out;
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (q * 4 + e < n) y[q * 4 + e] = out.v[e];
    }
  }
}

template <typename T, Draw DRAW>
int launch(phip_ctx *ctx, uint64_t seed, uint64_t offset, float p0, float p1, void *y, size_t n) {
  PHIP_ENTER(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(y != nullptr, "null pointer");
  hipLaunchKernelGGL((random_kernel<T, DRAW>), dim3(blocks_for((n + 3) / 4, ctx)), dim3(kBlock), 0, ctx->stream,
                     static_cast<T *>(y), n, seed, offset, p0, p1);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_RANDOM(SUF, T, PTR)                                                                          \
  int phip_random_uniform_##SUF(phip_ctx *ctx, uint64_t seed, uint64_t offset, float lower, float upper, PTR y,  \
                                size_t n) {                                                                      \
    return launch<T, Draw::Uniform>(ctx, seed, offset, lower, upper, y, n);                                      \
  }                                                                                                              \
  int phip_random_bernoulli_##SUF(phip_ctx *ctx, uint64_t seed, uint64_t offset, float p, PTR y, size_t n) {     \
    return launch<T, Draw::Bernoulli>(ctx, seed, offset, p, 0.f, y, n);                                          \
  }                                                                                                              \
  int phip_random_normal_##SUF(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd, PTR y,       \
                               size_t n) {                                                                       \
    return launch<T, Draw::Normal>(ctx, seed, offset, mean, sd, y, n);                                           \
  }                                                                                                              \
  int phip_random_log_normal_##SUF(phip_ctx *ctx, uint64_t seed, uint64_t offset, float mean, float sd, PTR y,   \
                                   size_t n) {                                                                   \
    return launch<T, Draw::LogNormal>(ctx, seed, offset, mean, sd, y, n);                                        \
  }

PHIP_EXPORT_RANDOM(f32, float, float *)
PHIP_EXPORT_RANDOM(f16, f16_t, void *)
PHIP_EXPORT_RANDOM(bf16, bf16_t, void *)

#undef PHIP_EXPORT_RANDOM

}  // extern "C"
