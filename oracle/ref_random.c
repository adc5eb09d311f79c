/*
 * CPU oracle for the on-device random tensors.  TEST INFRASTRUCTURE ONLY: the
 * checker the GPU library is compared against; never part of the shipped GPU
 * path, and nothing in the product may call it.
 *
 * The reference's GPU device draws from cuRAND (primitiv/devices/cuda/ops/
 * random_{bernoulli,uniform,normal,log_normal}.cu), a third-party library that
 * is not in the reference tree; its streams cannot be restated, so the
 * reference's seeded vectors (test/cuda_device_test.cc:107-240) do not apply
 * and PARITY WITH THE REFERENCE'S STREAMS IS UNPINNED.  What is restated here
 * is the reference's use of the draws - uniform values in (0, 1] scaled to
 * (lower, upper] (random_uniform.cu:9-27), Bernoulli as (u <= p)
 * (random_bernoulli.cu:9-25), normal and log-normal with (mean, sd) - on top of
 * the published generator Philox4x32-10 (Salmon et al., SC'11), which is pinned
 * by the known-answer vectors of that paper's reference implementation
 * (Random123 kat_vectors) in tests/test_oracle_random.py.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

void ref_philox4x32_10(const uint32_t ctr[4], const uint32_t key[2], uint32_t out[4]) {
  uint32_t c0 = ctr[0], c1 = ctr[1], c2 = ctr[2], c3 = ctr[3];
  uint32_t k0 = key[0], k1 = key[1];
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
  out[0] = c0;
  out[1] = c1;
  out[2] = c2;
  out[3] = c3;
}

static float unit_interval(uint32_t w) { return (float)((w >> 8) + 1u) * 5.9604644775390625e-8f; }

enum { D_UNIFORM, D_BERNOULLI, D_NORMAL, D_LOG_NORMAL };

/* Element i takes word i%4 of the block with counter offset + i/4, key = seed. */
int ref_random(int kind, uint64_t seed, uint64_t offset, float p0, float p1, float *y, size_t n) {
  if (kind < D_UNIFORM || kind > D_LOG_NORMAL) return -1;
  for (size_t i = 0; i < n; ++i) {
    const uint64_t counter = offset + i / 4;
    const uint32_t ctr[4] = {(uint32_t)counter, (uint32_t)(counter >> 32), 0, 0};
    const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
    uint32_t w[4];
    ref_philox4x32_10(ctr, key, w);
    const int e = (int)(i % 4);
    if (kind == D_UNIFORM) {
      y[i] = fmaf(unit_interval(w[e]), p1 - p0, p0);
    } else if (kind == D_BERNOULLI) {
      y[i] = unit_interval(w[e]) <= p0 ? 1.f : 0.f;
    } else {
      const float u = unit_interval(w[e & 2]), v = unit_interval(w[(e & 2) + 1]);
      const float r = sqrtf(-2.f * logf(u));
      const float t = 6.283185307179586f * v;
      const float z = fmaf(r * ((e & 1) ? sinf(t) : cosf(t)), p1, p0);
      y[i] = kind == D_LOG_NORMAL ? expf(z) : z;
    }
  }
  return 0;
}
