/*
 * CPU oracle for the elementwise operations around the matmul path.
 * TEST INFRASTRUCTURE ONLY: the checker the GPU library is compared against;
 * never part of the shipped GPU path, and nothing in the product may call it.
 *
 * Restates, expression for expression (including which subexpressions the
 * reference evaluates in double because of a double literal), the loops of
 * primitiv's plain CPU device:
 *   ref_unary_fw / _bw     primitiv/devices/naive/ops/{negate,abs,sqrt,exp,log,
 *                          tanh,sigmoid,softplus,sin,cos,tan}.cc through
 *                          CPUDEV_FW_X / CPUDEV_BW_X (naive/ops/common.h:12-29)
 *   ref_const_fw / _bw     naive/ops/{add,subtract,multiply,divide,pow,prelu,
 *                          elu}.cc through CPUDEV_FW_X_CONST / CPUDEV_BW_X_CONST
 *                          (common.h:31-49)
 *   ref_pown_fw / _bw      naive/ops/pown.cc:12-46
 *   ref_scalar_fw          CPUDEV_FW_X_SCALAR (common.h:51-66) as used in
 *                          add.cc, subtract.cc, multiply.cc, divide.cc, pow.cc
 *   ref_binary_fw          CPUDEV_FW_AB (common.h:68-83)
 *   ref_binary_bw          add_bw_impl ... pow_bw_impl in the same five files
 *   ref_inplace_subtract   naive/ops/inplace_subtract.cc:11-27
 *   ref_inplace_multiply_const  naive/ops/inplace_multiply_const.cc:9-13
 *   ref_identity           naive/ops/identity.cc:9-14
 * Operation codes are the oracle's own (listed in the enums below).
 *
 * Parity status: every operation code is pinned by the reference's own golden
 * vectors (test/tensor_forward_test.cc:92-112,572-1502,1929-2304;
 * test/tensor_backward_test.cc:369-773,1201-1597; test/tensor_test.cc:467-540,
 * 633-722), which tests/test_oracle_pointwise.py checks with the reference's
 * ULP bounds, and by float64 library routines on random inputs.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>

enum { U_NEGATE, U_ABS, U_SQRT, U_EXP, U_LOG, U_TANH, U_SIGMOID, U_SOFTPLUS, U_SIN, U_COS, U_TAN };
enum { C_ADD, C_SUB_R, C_SUB_L, C_MUL, C_DIV_R, C_DIV_L, C_POW_R, C_POW_L, C_PRELU, C_ELU };
enum { B_ADD, B_SUB, B_MUL, B_DIV, B_POW };

int ref_unary_fw(int op, const float *src, float *dest, size_t size) {
  for (size_t i = 0; i < size; ++i) {
    switch (op) {
      case U_NEGATE: dest[i] = -src[i]; break;
      case U_ABS: dest[i] = fabsf(src[i]); break;
      case U_SQRT: dest[i] = sqrtf(src[i]); break;
      case U_EXP: dest[i] = expf(src[i]); break;
      case U_LOG: dest[i] = logf(src[i]); break;
      case U_TANH: dest[i] = tanhf(src[i]); break;
      case U_SIGMOID: dest[i] = .5 + .5 * tanh(.5 * src[i]); break;
      case U_SOFTPLUS:
        dest[i] = src[i] > 0 ? src[i] + logf(1 + expf(-src[i])) : logf(1 + expf(src[i]));
        break;
      case U_SIN: dest[i] = sinf(src[i]); break;
      case U_COS: dest[i] = cosf(src[i]); break;
      case U_TAN: dest[i] = tanf(src[i]); break;
      default: return -1;
    }
  }
  return 0;
}

int ref_unary_bw(int op, const float *px, const float *py, const float *pgy, float *pgx, size_t size) {
  for (size_t i = 0; i < size; ++i) {
    switch (op) {
      case U_ABS: pgx[i] += ((px[i] > 0) - (px[i] < 0)) * pgy[i]; break;
      case U_SQRT: pgx[i] += .5 * pgy[i] / py[i]; break;
      case U_EXP: pgx[i] += py[i] * pgy[i]; break;
      case U_LOG: pgx[i] += pgy[i] / px[i]; break;
      case U_TANH: pgx[i] += (1. - py[i] * py[i]) * pgy[i]; break;
      case U_SIGMOID: pgx[i] += py[i] * (1. - py[i]) * pgy[i]; break;
      case U_SOFTPLUS: pgx[i] += (.5 + .5 * tanh(.5 * px[i])) * pgy[i]; break;
      case U_SIN: pgx[i] += cosf(px[i]) * pgy[i]; break;
      case U_COS: pgx[i] += -sinf(px[i]) * pgy[i]; break;
      case U_TAN: pgx[i] += (1 + py[i] * py[i]) * pgy[i]; break;
      default: return -1;
    }
  }
  return 0;
}

int ref_const_fw(int op, const float *src, float k, float *dest, size_t size) {
  for (size_t i = 0; i < size; ++i) {
    switch (op) {
      case C_ADD: dest[i] = src[i] + k; break;
      case C_SUB_R: dest[i] = src[i] - k; break;
      case C_SUB_L: dest[i] = k - src[i]; break;
      case C_MUL: dest[i] = src[i] * k; break;
      case C_DIV_R: dest[i] = src[i] / k; break;
      case C_DIV_L: dest[i] = k / src[i]; break;
      case C_POW_R: dest[i] = powf(src[i], k); break;
      case C_POW_L: dest[i] = powf(k, src[i]); break;
      case C_PRELU: dest[i] = src[i] * ((src[i] > 0) + k * (src[i] <= 0)); break;
      case C_ELU: dest[i] = src[i] * (src[i] > 0) + k * (expf(src[i] * (src[i] <= 0)) - 1); break;
      default: return -1;
    }
  }
  return 0;
}

int ref_const_bw(int op, const float *px, const float *py, const float *pgy, float k, float *pgx, size_t size) {
  for (size_t i = 0; i < size; ++i) {
    switch (op) {
      case C_ADD: pgx[i] += pgy[i]; break;
      case C_SUB_R: pgx[i] += pgy[i]; break;
      case C_SUB_L: pgx[i] += -pgy[i]; break;
      case C_MUL: pgx[i] += k * pgy[i]; break;
      case C_DIV_R: pgx[i] += pgy[i] / k; break;
      case C_DIV_L: pgx[i] += -py[i] * pgy[i] / px[i]; break;
      case C_POW_R: pgx[i] += k * pgy[i] * py[i] / px[i]; break;
      case C_POW_L: pgx[i] += logf(k) * pgy[i] * py[i]; break;
      case C_PRELU: pgx[i] += pgy[i] * ((px[i] > 0) + k * (px[i] <= 0)); break;
      case C_ELU: pgx[i] += pgy[i] * ((px[i] > 0) + (py[i] + k) * (px[i] <= 0)); break;
      default: return -1;
    }
  }
  return 0;
}

void ref_pown_fw(const float *src, int32_t k, float *dest, size_t size) {
  const uint32_t abs_k = k < 0 ? 0u - (uint32_t)k : (uint32_t)k;
  for (size_t i = 0; i < size; ++i) {
    float ret = 1.;
    float factor = src[i];
    uint32_t remain = abs_k;
    while (remain) {
      if (remain & 1) ret *= factor;
      factor *= factor;
      remain >>= 1;
    }
    dest[i] = k >= 0 ? ret : 1. / ret;
  }
}

void ref_pown_bw(const float *px, const float *py, const float *pgy, int32_t k, float *pgx, size_t size) {
  for (size_t i = 0; i < size; ++i) pgx[i] += k * pgy[i] * py[i] / px[i];
}

static float binary_value(int op, float a, float b) {
  switch (op) {
    case B_ADD: return a + b;
    case B_SUB: return a - b;
    case B_MUL: return a * b;
    case B_DIV: return a / b;
    default: return powf(a, b);
  }
}

/* dest = x op k (or k op x when k_on_left) with one scalar per sample. */
int ref_scalar_fw(int op, int k_on_left, const float *src_x, const float *src_k, float *dest, uint32_t size,
                  uint32_t bx, uint32_t bk) {
  if (op < B_ADD || op > B_POW) return -1;
  const uint32_t bs = bx > bk ? bx : bk;
  const size_t skip_x = bx > 1 ? size : 0, skip_k = bk > 1 ? 1 : 0;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    for (uint32_t i = 0; i < size; ++i)
      dest[i] = k_on_left ? binary_value(op, *src_k, src_x[i]) : binary_value(op, src_x[i], *src_k);
    dest += size;
    src_x += skip_x;
    src_k += skip_k;
  }
  return 0;
}

int ref_binary_fw(int op, const float *src_a, const float *src_b, float *dest, uint32_t size, uint32_t ba,
                  uint32_t bb) {
  if (op < B_ADD || op > B_POW) return -1;
  const uint32_t bs = ba > bb ? ba : bb;
  const size_t skip_a = ba > 1 ? size : 0, skip_b = bb > 1 ? size : 0;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    for (uint32_t i = 0; i < size; ++i) dest[i] = binary_value(op, src_a[i], src_b[i]);
    dest += size;
    src_a += skip_a;
    src_b += skip_b;
  }
  return 0;
}

/* ga += dy/da * gy, gb += dy/db * gy; a gradient whose batch is 1 does not
   advance, so it collects every sample. */
int ref_binary_bw(int op, const float *pa, const float *pb, const float *py, const float *pgy, float *pga,
                  float *pgb, uint32_t size, uint32_t ba, uint32_t bb) {
  if (op < B_ADD || op > B_POW) return -1;
  const uint32_t bs = ba > bb ? ba : bb;
  const size_t skip_a = ba > 1 ? size : 0, skip_b = bb > 1 ? size : 0;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    for (uint32_t i = 0; i < size; ++i) {
      switch (op) {
        case B_ADD: {
          const float k = pgy[i];
          pga[i] += k;
          pgb[i] += k;
          break;
        }
        case B_SUB: {
          const float k = pgy[i];
          pga[i] += k;
          pgb[i] -= k;
          break;
        }
        case B_MUL: {
          const float k = pgy[i];
          pga[i] += k * pb[i];
          pgb[i] += k * pa[i];
          break;
        }
        case B_DIV: {
          const float k = pgy[i] / pb[i];
          pga[i] += k;
          pgb[i] -= k * py[i];
          break;
        }
        default: {
          const float a = pgy[i] * py[i];
          pga[i] += a * pb[i] / pa[i];
          pgb[i] += a * logf(pa[i]);
          break;
        }
      }
    }
    if (pa) pa += skip_a;
    if (pb) pb += skip_b;
    if (py) py += size;
    pgy += size;
    pga += skip_a;
    pgb += skip_b;
  }
  return 0;
}

void ref_inplace_subtract(const float *src, float *dest, uint32_t size, uint32_t bx, uint32_t by) {
  const uint32_t bs = bx > by ? bx : by;
  const size_t b_skip_d = by > 1 ? size : 0, b_skip_s = bx > 1 ? size : 0;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    for (uint32_t i = 0; i < size; ++i) dest[i] -= src[i];
    dest += b_skip_d;
    src += b_skip_s;
  }
}

void ref_inplace_multiply_const(float k, float *dest, size_t size) {
  for (size_t i = 0; i < size; ++i) dest[i] *= k;
}

void ref_identity(float *dest, uint32_t size) {
  for (size_t i = 0; i < (size_t)size * size; ++i) dest[i] = 0;
  for (uint32_t i = 0; i < size; ++i) dest[(size_t)i * (size + 1)] = 1;
}
