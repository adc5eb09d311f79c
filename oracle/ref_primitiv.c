/*
 * CPU oracle for the primitiv matmul path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file restates, in plain C, what primitiv's Eigen CPU device computes
 * for the functions on the matmul hot path.  It is the checker the GPU
 * library is compared against and the CPU baseline that the benchmark times;
 * it is never part of the shipped GPU path and nothing in the product may
 * call it.
 *
 * The arithmetic of the reference lives in Eigen 3.3 (`Map<MatrixXf>`
 * products; external, un-vendored, required by the reference's top-level
 * CMakeLists.txt:32-34).  Its published semantics are those of a dense
 * column-major single-precision GEMM; only Eigen's internal summation order
 * is not reproduced, which moves fp32 results by ~1e-6 relative.
 *
 * Functions and the reference lines they follow:
 *   ref_shape_matmul      primitiv/core/shape_ops.cc:152-160,
 *                         primitiv/core/shape.h:55,136-138,156
 *   ref_matmul_fw         primitiv/devices/eigen/ops/matmul.cc:9-38
 *   ref_matmul_bw         primitiv/devices/eigen/ops/matmul.cc:40-79
 *   ref_matmul_fw_f64 /
 *   ref_matmul_bw_f64     same rules, plain triple loops accumulating in
 *                         double (the brute-force check of the fast routines)
 *   ref_inplace_add       primitiv/devices/eigen/ops/inplace_add.cc:9-23
 *   ref_batch_sum         primitiv/devices/eigen/ops/batch_sum.cc:9-22
 *   ref_pool_block_size   primitiv/core/memory_pool.cc:35-52,
 *                         primitiv/core/numeric_utils.h:16-37
 *
 * Parity status: every function above is pinned by the reference's own
 * golden vectors (test/tensor_forward_test.cc:1798-1927,
 * test/tensor_backward_test.cc:1599-1668, test/operator_impl_test.cc:1132-1144,
 * test/tensor_test.cc:541-631, test/tensor_forward_test.cc:2920-2934,
 * test/cuda_memory_pool_test.cc:106-167, test/shape_ops_test.cc:330-358) and
 * by float64 library products; see tests/test_oracle.py.
 *
 * All matrices are dense column-major (leading dimension = rows); the
 * minibatch is the outermost index with stride rows*cols, or stride 0 for an
 * operand whose batch size is 1.
 */
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

/* ------------------------------------------------------------------------ */
/* Blocked single-precision GEMM:  C[m x n] (ldc) += A * B, where the        */
/* operands are addressed through (row stride, column stride) pairs so that  */
/* plain and transposed uses share one routine.  fp32 accumulation.          */
/* ------------------------------------------------------------------------ */

enum { MR = 16, NR = 6, MC = 192, KC = 384, NC = 3072 };

typedef float v8f __attribute__((vector_size(32), aligned(4)));

static void micro_16x6(int kc, const float *ap, const float *bp, float *acc) {
  v8f c[NR][2];
  for (int j = 0; j < NR; ++j) {
    c[j][0] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
    c[j][1] = (v8f){0, 0, 0, 0, 0, 0, 0, 0};
  }
  for (int p = 0; p < kc; ++p) {
    const v8f a0 = *(const v8f *)(ap + p * MR);
    const v8f a1 = *(const v8f *)(ap + p * MR + 8);
    const float *b = bp + p * NR;
    for (int j = 0; j < NR; ++j) {
      const float s = b[j];
      const v8f bj = (v8f){s, s, s, s, s, s, s, s};
      c[j][0] += a0 * bj;
      c[j][1] += a1 * bj;
    }
  }
  for (int j = 0; j < NR; ++j) {
    memcpy(acc + j * MR, &c[j][0], 32);
    memcpy(acc + j * MR + 8, &c[j][1], 32);
  }
}

static void pack_a(int mc, int kc, const float *a, ptrdiff_t rs, ptrdiff_t cs,
                   float *dst) {
  for (int i0 = 0; i0 < mc; i0 += MR) {
    const int mr = mc - i0 < MR ? mc - i0 : MR;
    for (int p = 0; p < kc; ++p) {
      for (int i = 0; i < mr; ++i) dst[i] = a[(i0 + i) * rs + p * cs];
      for (int i = mr; i < MR; ++i) dst[i] = 0.0f;
      dst += MR;
    }
  }
}

static void pack_b(int kc, int nc, const float *b, ptrdiff_t rs, ptrdiff_t cs,
                   float *dst) {
  for (int j0 = 0; j0 < nc; j0 += NR) {
    const int nr = nc - j0 < NR ? nc - j0 : NR;
    for (int p = 0; p < kc; ++p) {
      for (int j = 0; j < nr; ++j) dst[j] = b[p * rs + (j0 + j) * cs];
      for (int j = nr; j < NR; ++j) dst[j] = 0.0f;
      dst += NR;
    }
  }
}

static void sgemm_acc(int m, int n, int k,
                      const float *a, ptrdiff_t rsa, ptrdiff_t csa,
                      const float *b, ptrdiff_t rsb, ptrdiff_t csb,
                      float *c, ptrdiff_t ldc, int threads) {
  if (m <= 0 || n <= 0 || k <= 0) return;
  if (threads < 1) threads = 1;
  float *bpack = (float *)aligned_alloc(64, sizeof(float) * KC * (NC + NR));
  float *apack_all =
      (float *)aligned_alloc(64, sizeof(float) * (size_t)threads * KC * (MC + MR));
  for (int jc = 0; jc < n; jc += NC) {
    const int nc = n - jc < NC ? n - jc : NC;
    for (int pc = 0; pc < k; pc += KC) {
      const int kc = k - pc < KC ? k - pc : KC;
      pack_b(kc, nc, b + pc * rsb + jc * csb, rsb, csb, bpack);
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads)
#endif
      for (int ic = 0; ic < m; ic += MC) {
        const int mc = m - ic < MC ? m - ic : MC;
#ifdef _OPENMP
        float *apack = apack_all + (size_t)omp_get_thread_num() * KC * (MC + MR);
#else
        float *apack = apack_all;
#endif
        float acc[MR * NR];
        pack_a(mc, kc, a + ic * rsa + pc * csa, rsa, csa, apack);
        for (int jr = 0; jr < nc; jr += NR) {
          const int nr = nc - jr < NR ? nc - jr : NR;
          for (int ir = 0; ir < mc; ir += MR) {
            const int mr = mc - ir < MR ? mc - ir : MR;
            micro_16x6(kc, apack + (size_t)ir * kc, bpack + (size_t)jr * kc, acc);
            float *cc = c + (ic + ir) + (ptrdiff_t)(jc + jr) * ldc;
            for (int j = 0; j < nr; ++j)
              for (int i = 0; i < mr; ++i) cc[i + j * ldc] += acc[i + j * MR];
          }
        }
      }
    }
  }
  free(apack_all);
  free(bpack);
}

/* ------------------------------------------------------------------------ */
/* Shape rule                                                                */
/* ------------------------------------------------------------------------ */

/*
 * A shape is (dims[0..depth), batch); dimensions past `depth` read as 1 and
 * trailing 1s are not counted in `depth`.  Returns 0 and fills out[0..2] =
 * {rows, cols, batch} of the product, or -1 when the reference would throw.
 */
int ref_shape_matmul(const uint32_t *ldims, uint32_t ldepth, uint32_t lbatch,
                     const uint32_t *rdims, uint32_t rdepth, uint32_t rbatch,
                     uint32_t *out) {
  while (ldepth > 0 && ldims[ldepth - 1] == 1) --ldepth;
  while (rdepth > 0 && rdims[rdepth - 1] == 1) --rdepth;
  const uint32_t l0 = ldepth > 0 ? ldims[0] : 1, l1 = ldepth > 1 ? ldims[1] : 1;
  const uint32_t r0 = rdepth > 0 ? rdims[0] : 1, r1 = rdepth > 1 ? rdims[1] : 1;
  if (ldepth > 2 || rdepth > 2) return -1;
  if (l1 != r0) return -1;
  if (!(lbatch == rbatch || lbatch == 1 || rbatch == 1)) return -1;
  out[0] = l0;
  out[1] = r1;
  out[2] = lbatch > rbatch ? lbatch : rbatch;
  return 0;
}

/* ------------------------------------------------------------------------ */
/* matmul forward / backward, fp32                                           */
/* ------------------------------------------------------------------------ */

/* y = a . b.  a: [di x dj] x ba, b: [dj x dk] x bb, y: [di x dk] x max. */
void ref_matmul_fw(const float *a, const float *b, float *y,
                   uint32_t di, uint32_t dj, uint32_t dk,
                   uint32_t ba, uint32_t bb, int threads) {
  if (ba > 1) {
    /* one product per sample; b advances only when it has a minibatch */
    const size_t a_skip = (size_t)di * dj;
    const size_t b_skip = (bb > 1) ? (size_t)dj * dk : 0;
    const size_t y_skip = (size_t)di * dk;
    for (uint32_t n = 0; n < ba; ++n) {
      float *yy = y + n * y_skip;
      memset(yy, 0, sizeof(float) * y_skip);
      sgemm_acc(di, dk, dj, a + n * a_skip, 1, di, b + n * b_skip, 1, dj, yy, di,
                threads);
    }
  } else {
    /* minibatch of b folded into the columns of one combined matrix */
    const size_t dkb = (size_t)dk * bb;
    memset(y, 0, sizeof(float) * di * dkb);
    sgemm_acc(di, (int)dkb, dj, a, 1, di, b, 1, dj, y, di, threads);
  }
}

/* ga += gy . b^T ;  gb += a^T . gy   (both accumulate). */
void ref_matmul_bw(const float *a, const float *b, const float *gy,
                   float *ga, float *gb,
                   uint32_t di, uint32_t dj, uint32_t dk,
                   uint32_t ba, uint32_t bb, int threads) {
  if (ba > 1) {
    const size_t a_skip = (size_t)di * dj;
    const size_t b_skip = (bb > 1) ? (size_t)dj * dk : 0;
    const size_t y_skip = (size_t)di * dk;
    for (uint32_t n = 0; n < ba; ++n) {
      const float *aa = a + n * a_skip, *bbp = b + n * b_skip;
      const float *gyy = gy + n * y_skip;
      /* gaa[di x dj] += gyy[di x dk] . bb^T[dk x dj] */
      sgemm_acc(di, dj, dk, gyy, 1, di, bbp, dj, 1, ga + n * a_skip, di, threads);
      /* gbb[dj x dk] += aa^T[dj x di] . gyy[di x dk]; gb does not advance
         when b is shared, so every sample lands in the same block */
      sgemm_acc(dj, dk, di, aa, di, 1, gyy, 1, di, gb + n * b_skip, dj, threads);
    }
  } else {
    const size_t dkb = (size_t)dk * bb;
    sgemm_acc(di, dj, (int)dkb, gy, 1, di, b, dj, 1, ga, di, threads);
    sgemm_acc(dj, (int)dkb, di, a, di, 1, gy, 1, di, gb, dj, threads);
  }
}

/* ------------------------------------------------------------------------ */
/* The same rules as brute-force loops with double accumulation.             */
/* ------------------------------------------------------------------------ */

void ref_matmul_fw_f64(const float *a, const float *b, float *y,
                       uint32_t di, uint32_t dj, uint32_t dk,
                       uint32_t ba, uint32_t bb) {
  const uint32_t bs = ba > bb ? ba : bb;
  const size_t sa = ba > 1 ? (size_t)di * dj : 0, sb = bb > 1 ? (size_t)dj * dk : 0;
  for (uint32_t n = 0; n < bs; ++n)
    for (uint32_t k = 0; k < dk; ++k)
      for (uint32_t i = 0; i < di; ++i) {
        double s = 0.0;
        for (uint32_t j = 0; j < dj; ++j)
          s += (double)a[n * sa + i + (size_t)j * di] *
               (double)b[n * sb + j + (size_t)k * dj];
        y[(size_t)n * di * dk + i + (size_t)k * di] = (float)s;
      }
}

void ref_matmul_bw_f64(const float *a, const float *b, const float *gy,
                       float *ga, float *gb,
                       uint32_t di, uint32_t dj, uint32_t dk,
                       uint32_t ba, uint32_t bb) {
  const uint32_t bs = ba > bb ? ba : bb;
  const size_t sa = ba > 1 ? (size_t)di * dj : 0, sb = bb > 1 ? (size_t)dj * dk : 0;
  const size_t sy = (size_t)di * dk;
  /* ga[n or 0][i,j] += sum over (samples sharing it) sum_k gy[n][i,k] b[n][j,k] */
  const uint32_t ga_blocks = ba > 1 ? ba : 1, gb_blocks = bb > 1 ? bb : 1;
  for (uint32_t g = 0; g < ga_blocks; ++g)
    for (uint32_t j = 0; j < dj; ++j)
      for (uint32_t i = 0; i < di; ++i) {
        double s = 0.0;
        for (uint32_t n = (ba > 1 ? g : 0); n < (ba > 1 ? g + 1 : bs); ++n)
          for (uint32_t k = 0; k < dk; ++k)
            s += (double)gy[n * sy + i + (size_t)k * di] *
                 (double)b[n * sb + j + (size_t)k * dj];
        float *p = &ga[g * (size_t)di * dj + i + (size_t)j * di];
        *p = (float)((double)*p + s);
      }
  for (uint32_t g = 0; g < gb_blocks; ++g)
    for (uint32_t k = 0; k < dk; ++k)
      for (uint32_t j = 0; j < dj; ++j) {
        double s = 0.0;
        for (uint32_t n = (bb > 1 ? g : 0); n < (bb > 1 ? g + 1 : bs); ++n)
          for (uint32_t i = 0; i < di; ++i)
            s += (double)a[n * sa + i + (size_t)j * di] *
                 (double)gy[n * sy + i + (size_t)k * di];
        float *p = &gb[g * (size_t)dj * dk + j + (size_t)k * dj];
        *p = (float)((double)*p + s);
      }
}

/* ------------------------------------------------------------------------ */
/* Helpers around the path                                                   */
/* ------------------------------------------------------------------------ */

/* y += x with either side's minibatch broadcast: bs = max(bx, by); a side
   with batch 1 does not advance, so by == 1 sums x over the minibatch. */
void ref_inplace_add(const float *x, float *y, uint32_t volume, uint32_t bx,
                     uint32_t by) {
  const uint32_t bs = bx > by ? bx : by;
  const size_t skip_x = bx > 1 ? volume : 0, skip_y = by > 1 ? volume : 0;
  for (uint32_t n = 0; n < bs; ++n) {
    for (uint32_t i = 0; i < volume; ++i) y[i] += x[i];
    y += skip_y;
    x += skip_x;
  }
}

/* y[i] = x[0][i] + x[1][i] + ... in sample order. */
void ref_batch_sum(const float *x, float *y, uint32_t volume, uint32_t bs) {
  for (uint32_t i = 0; i < volume; ++i) y[i] = x[i];
  for (uint32_t n = 1; n < bs; ++n) {
    x += volume;
    for (uint32_t i = 0; i < volume; ++i) y[i] += x[i];
  }
}

/* Size of the pool block that serves a request of `size` bytes: at least
   `minimum`, rounded up to a power of two; 0 stays 0. */
uint64_t ref_pool_block_size(uint64_t size, uint64_t minimum) {
  if (size == 0) return 0;
  if (size < minimum) size = minimum;
  uint64_t s = 1;
  while (s < size) s <<= 1;
  return s;
}

int ref_num_threads_available(void) {
#ifdef _OPENMP
  return omp_get_max_threads();
#else
  return 1;
#endif
}
