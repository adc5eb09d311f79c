/*
 * CPU oracle for the data-movement and reduction operations between the
 * matmuls.  TEST INFRASTRUCTURE ONLY: the checker the GPU library is compared
 * against; never part of the shipped GPU path, and nothing in the product may
 * call it.
 *
 * Restates the loops of primitiv's plain CPU device on whole tensors, taking
 * the shape as (dims, depth, batch) the way the reference's Shape holds it:
 *   ref_slice_fw / _bw        primitiv/devices/naive/ops/slice.cc:11-56
 *   ref_concat_fw             naive/ops/concat.cc:11-37
 *   ref_pick_fw / _bw         naive/ops/pick.cc:11-52
 *   ref_batch_pick_fw / _bw   naive/ops/batch_pick.cc:11-34
 *   ref_batch_slice_fw / _bw  naive/ops/batch_slice.cc:11-28
 *   ref_batch_concat_fw       naive/ops/batch_concat.cc:11-22
 *   ref_transpose_fw / _bw    naive/ops/transpose.cc:11-39
 *   ref_permute_dims_fw / _bw naive/ops/permute_dims.cc:11-84
 *   ref_flip_fw / _bw         naive/ops/flip.cc:9-40
 *   ref_sum_fw                naive/ops/sum.cc:9-27
 *   ref_logsumexp_fw          naive/ops/logsumexp.cc:11-35
 *   ref_broadcast_fw          naive/ops/broadcast.cc:9-27
 *   ref_max_fw / ref_min_fw,
 *   ref_max_bw / ref_min_bw   naive/ops/max.cc:9-55, min.cc
 *   ref_argmax / ref_argmin   naive/ops/argmax.cc:11-36, argmin.cc
 *   lower_volume              primitiv/core/shape.h:100-104
 *
 * Parity status: pinned by the reference's golden vectors
 * (test/tensor_forward_test.cc: CheckPickNN :121, CheckSlice :193, CheckConcat*
 * :349-476, CheckTranspose* :1530-1584, CheckFlip* :1592-1690, CheckPermuteDims*
 * :1692-1786, CheckMaxDims/CheckMinDims :2306,2357, CheckSum :2408,
 * CheckLogSumExp :2455, CheckBroadcast :2623, CheckBatchPickNN :2709,
 * CheckBatchSlice :2766, CheckBatchConcat :2853; test/tensor_backward_test.cc:
 * CheckSlice* :41-154, CheckPick* :212-320, CheckMaxDims :775, CheckBatchPick*
 * :1670-1749; test/tensor_test.cc CheckArgMaxDims :744), replayed by
 * tests/test_oracle_indexing.py, and by numpy's indexing routines
 * (take, concatenate, transpose, flip, sum, max, argmax) on random shapes.
 */
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <string.h>

typedef struct {
  const uint32_t *dims;
  uint32_t depth;
  uint32_t batch;
} shape_t;

static uint32_t dim_at(shape_t s, uint32_t i) { return i < s.depth ? s.dims[i] : 1; }
static uint32_t lower_volume(shape_t s, uint32_t dim) {
  uint32_t v = 1;
  for (uint32_t i = 0; i < dim && i < s.depth; ++i) v *= s.dims[i];
  return v;
}
static uint32_t volume(shape_t s) { return lower_volume(s, s.depth); }

/* y = x[..., offset : offset + ny, ...] along dim; ydims = xdims with dims[dim] = ny */
void ref_slice_fw(const float *x, const uint32_t *xdims, uint32_t depth, uint32_t batch, uint32_t dim,
                  uint32_t offset, uint32_t ny, float *y) {
  const shape_t sx = {xdims, depth, batch};
  const uint32_t base = lower_volume(sx, dim);
  const uint32_t span = base * ny;
  const uint32_t skip = base * dim_at(sx, dim);
  const uint32_t ysize = volume(sx) / dim_at(sx, dim) * ny * batch;
  const uint32_t repeat = ysize / span;
  const float *src = x + base * offset;
  for (uint32_t i = 0; i < repeat; ++i) {
    for (uint32_t j = 0; j < span; ++j) *y++ = src[j];
    src += skip;
  }
}

/* gx[..., offset : offset + ny, ...] += gy with either minibatch broadcast */
void ref_slice_bw(const float *gy, uint32_t by, uint32_t ny, const uint32_t *xdims, uint32_t depth, uint32_t bx,
                  uint32_t dim, uint32_t offset, float *gx) {
  const shape_t sx = {xdims, depth, bx};
  const uint32_t base = lower_volume(sx, dim);
  const uint32_t span = base * ny;
  const uint32_t skip = base * dim_at(sx, dim);
  const uint32_t repeat = volume(sx) / skip;
  const uint32_t bs = bx > by ? bx : by;
  const uint32_t b_skip_d = bx > 1 ? volume(sx) : 0;
  const uint32_t b_skip_s = by > 1 ? span * repeat : 0;
  float *dest = gx + base * offset;
  const float *src = gy;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    float *dp = dest;
    const float *sp = src;
    for (uint32_t i = 0; i < repeat; ++i) {
      for (uint32_t j = 0; j < span; ++j) dp[j] += *sp++;
      dp += skip;
    }
    dest += b_skip_d;
    src += b_skip_s;
  }
}

/* One input of a concatenation: x (its extent along dim is nx, batch bx) goes
   to position `offset` (in elements of dim) of y (ydims, batch by). */
void ref_concat_fw_one(const float *x, uint32_t nx, uint32_t bx, const uint32_t *ydims, uint32_t depth, uint32_t by,
                       uint32_t dim, uint32_t offset, float *y) {
  const shape_t sy = {ydims, depth, by};
  const uint32_t base = lower_volume(sy, dim);
  const uint32_t skip = base * dim_at(sy, dim);
  const uint32_t repeat = volume(sy) / skip;
  const uint32_t span = base * nx;
  const uint32_t b_skip = bx > 1 ? span * repeat : 0;
  float *dest = y + base * offset;
  const float *src = x;
  for (uint32_t batch = 0; batch < by; ++batch) {
    const float *sp = src;
    for (uint32_t i = 0; i < repeat; ++i) {
      for (uint32_t j = 0; j < span; ++j) dest[j] = *sp++;
      dest += skip;
    }
    src += b_skip;
  }
}

void ref_pick_fw(const float *x, const uint32_t *xdims, uint32_t depth, uint32_t bx, const uint32_t *ids,
                 uint32_t n_ids, uint32_t dim, float *y) {
  const shape_t sx = {xdims, depth, bx};
  const uint32_t bs = bx > n_ids ? bx : n_ids;
  const uint32_t skip_x = bx > 1 ? volume(sx) : 0;
  const uint32_t skip_i = n_ids > 1;
  const uint32_t base = lower_volume(sx, dim);
  const uint32_t skip = base * dim_at(sx, dim);
  const uint32_t repeat = volume(sx) / skip;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    const float *src = x + batch * skip_x + base * ids[batch * skip_i];
    for (uint32_t i = 0; i < repeat; ++i) {
      for (uint32_t j = 0; j < base; ++j) *y++ = src[j];
      src += skip;
    }
  }
}

void ref_pick_bw(const float *gy, const uint32_t *xdims, uint32_t depth, uint32_t bx, const uint32_t *ids,
                 uint32_t n_ids, uint32_t dim, float *gx) {
  const shape_t sx = {xdims, depth, bx};
  const uint32_t bs = bx > n_ids ? bx : n_ids;
  const uint32_t skip_x = bx > 1 ? volume(sx) : 0;
  const uint32_t skip_i = n_ids > 1;
  const uint32_t base = lower_volume(sx, dim);
  const uint32_t skip = base * dim_at(sx, dim);
  const uint32_t repeat = volume(sx) / skip;
  for (uint32_t batch = 0; batch < bs; ++batch) {
    float *dest = gx + batch * skip_x + base * ids[batch * skip_i];
    for (uint32_t i = 0; i < repeat; ++i) {
      for (uint32_t j = 0; j < base; ++j) dest[j] += *gy++;
      dest += skip;
    }
  }
}

void ref_batch_pick_fw(const float *x, uint32_t span, const uint32_t *ids, uint32_t n_ids, float *y) {
  for (uint32_t batch = 0; batch < n_ids; ++batch) {
    memcpy(y, x + (size_t)span * ids[batch], sizeof(float) * span);
    y += span;
  }
}

void ref_batch_pick_bw(const float *gy, uint32_t span, const uint32_t *ids, uint32_t n_ids, float *gx) {
  for (uint32_t batch = 0; batch < n_ids; ++batch) {
    float *dest = gx + (size_t)span * ids[batch];
    for (uint32_t i = 0; i < span; ++i) dest[i] += *gy++;
  }
}

void ref_batch_slice_fw(const float *x, uint32_t vol, uint32_t offset, uint32_t by, float *y) {
  memcpy(y, x + (size_t)vol * offset, sizeof(float) * vol * by);
}

void ref_batch_slice_bw(const float *gy, uint32_t vol, uint32_t offset, uint32_t by, float *gx) {
  float *dest = gx + (size_t)vol * offset;
  for (size_t i = 0; i < (size_t)vol * by; ++i) dest[i] += gy[i];
}

void ref_transpose_fw(const float *x, uint32_t d1, uint32_t d2, uint32_t bs, float *y) {
  const uint32_t ms = d1 * d2;
  for (uint32_t k = 0; k < bs; ++k) {
    float *pd = y;
    for (uint32_t j = 0; j < d2; ++j) {
      float *ppd = pd;
      for (uint32_t i = 0; i < d1; ++i) {
        *ppd = *x++;
        ppd += d2;
      }
      ++pd;
    }
    y += ms;
  }
}

/* gx (d1 x d2) += transpose of gy (d2 x d1) */
void ref_transpose_bw(const float *gy, uint32_t d1, uint32_t d2, uint32_t bs, float *gx) {
  for (uint32_t k = 0; k < bs; ++k) {
    for (uint32_t j = 0; j < d2; ++j)
      for (uint32_t i = 0; i < d1; ++i) gx[i + (size_t)j * d1] += gy[j + (size_t)i * d2];
    gx += (size_t)d1 * d2;
    gy += (size_t)d1 * d2;
  }
}

static void permute_strides(const uint32_t *xdims, const uint32_t *perm, uint32_t ndims, uint32_t *x_strides,
                            uint32_t *y_strides) {
  uint32_t x_stride_tmp = 1, y_stride_tmp = 1;
  for (uint32_t i = 0; i < ndims; ++i) {
    x_strides[ndims - i - 1] = x_stride_tmp;
    y_strides[ndims - perm[i] - 1] = y_stride_tmp;
    x_stride_tmp *= xdims[i];
    y_stride_tmp *= xdims[perm[i]];   /* y.shape()[i] */
  }
}

void ref_permute_dims_fw(const float *x, const uint32_t *xdims, uint32_t ndims, const uint32_t *perm, uint32_t bs,
                         float *y) {
  uint32_t xs[8], ys[8], vol = 1;
  permute_strides(xdims, perm, ndims, xs, ys);
  for (uint32_t i = 0; i < ndims; ++i) vol *= xdims[i];
  for (uint32_t k = 0; k < bs; ++k) {
    for (uint32_t i = 0; i < vol; ++i) {
      uint32_t tmp = i, j = 0;
      for (uint32_t d = 0; d < ndims; ++d) {
        const uint32_t p = tmp / xs[d];
        tmp -= p * xs[d];
        j += p * ys[d];
      }
      y[j] = x[i];
    }
    x += vol;
    y += vol;
  }
}

void ref_permute_dims_bw(const float *gy, const uint32_t *xdims, uint32_t ndims, const uint32_t *perm, uint32_t bs,
                         float *gx) {
  uint32_t xs[8], ys[8], vol = 1;
  permute_strides(xdims, perm, ndims, xs, ys);
  for (uint32_t i = 0; i < ndims; ++i) vol *= xdims[i];
  for (uint32_t k = 0; k < bs; ++k) {
    for (uint32_t i = 0; i < vol; ++i) {
      uint32_t tmp = i, j = 0;
      for (uint32_t d = 0; d < ndims; ++d) {
        const uint32_t p = tmp / xs[d];
        tmp -= p * xs[d];
        j += p * ys[d];
      }
      gx[i] += gy[j];
    }
    gx += vol;
    gy += vol;
  }
}

/* y (=, or += when accumulate) x flipped along dim */
void ref_flip(const float *x, const uint32_t *dims, uint32_t depth, uint32_t batch, uint32_t dim, int accumulate,
              float *y) {
  const shape_t s = {dims, depth, batch};
  const uint32_t n = dim_at(s, dim);
  const uint32_t skip = lower_volume(s, dim);
  const uint32_t r = volume(s) * batch / n;
  for (uint32_t j = 0; j < n; ++j) {
    for (uint32_t i = 0; i < r; ++i) {
      const uint32_t offset = i * n - i % skip * (n - 1);
      if (accumulate) y[offset + j * skip] += x[offset + (n - j - 1) * skip];
      else y[offset + j * skip] = x[offset + (n - j - 1) * skip];
    }
  }
}

enum { R_SUM, R_LOGSUMEXP, R_MAX, R_MIN };

/* y = reduction of x along dim (ydims = xdims with dims[dim] = 1) */
int ref_reduce_fw(int op, const float *src, const uint32_t *dims, uint32_t depth, uint32_t batch, uint32_t dim,
                  float *dest) {
  const shape_t s = {dims, depth, batch};
  const uint32_t n = dim_at(s, dim);
  const uint32_t repeat = volume(s) * batch / n;
  const uint32_t skip1 = lower_volume(s, dim);
  const uint32_t skip2 = skip1 * n;
  for (uint32_t i = 0; i < repeat; ++i) {
    uint32_t offset = i % skip1 + (i / skip1) * skip2;
    float tmp;
    switch (op) {
      case R_SUM:
        tmp = 0;
        for (uint32_t j = 0; j < n; ++j) {
          tmp += src[offset];
          offset += skip1;
        }
        break;
      case R_LOGSUMEXP:
        tmp = src[offset];
        for (uint32_t j = 1; j < n; ++j) {
          offset += skip1;
          const float arg = src[offset];
          tmp = tmp > arg ? tmp + log(1. + exp(arg - tmp)) : arg + log(1. + exp(tmp - arg));
        }
        break;
      case R_MAX:
      case R_MIN:
        tmp = src[offset];
        for (uint32_t j = 0; j < n; ++j) {
          if (op == R_MAX ? src[offset] > tmp : src[offset] < tmp) tmp = src[offset];
          offset += skip1;
        }
        break;
      default:
        return -1;
    }
    dest[i] = tmp;
  }
  return 0;
}

/* gx[first position along dim whose value equals y] += gy */
void ref_extremum_bw(const float *px, const float *py, const float *pgy, const uint32_t *dims, uint32_t depth,
                     uint32_t batch, uint32_t dim, float *pgx) {
  const shape_t s = {dims, depth, batch};
  const uint32_t n = dim_at(s, dim);
  const uint32_t repeat = volume(s) * batch / n;
  const uint32_t skip1 = lower_volume(s, dim);
  const uint32_t skip2 = skip1 * n;
  for (uint32_t i = 0; i < repeat; ++i) {
    const float val = py[i];
    uint32_t offset = i % skip1 + (i / skip1) * skip2;
    for (uint32_t j = 0; j < n; ++j) {
      if (px[offset] == val) {
        pgx[offset] += pgy[i];
        break;
      }
      offset += skip1;
    }
  }
}

void ref_arg_extremum(int want_max, const float *src, const uint32_t *dims, uint32_t depth, uint32_t batch,
                      uint32_t dim, uint32_t *ret) {
  const shape_t s = {dims, depth, batch};
  const uint32_t n = dim_at(s, dim);
  const uint32_t repeat = volume(s) * batch / n;
  const uint32_t skip1 = lower_volume(s, dim);
  const uint32_t skip2 = skip1 * n;
  for (uint32_t i = 0; i < repeat; ++i) {
    uint32_t offset = i % skip1 + (i / skip1) * skip2;
    float best = src[offset];
    uint32_t arg = 0;
    for (uint32_t j = 1; j < n; ++j) {
      offset += skip1;
      if (want_max ? src[offset] > best : src[offset] < best) {
        best = src[offset];
        arg = j;
      }
    }
    ret[i] = arg;
  }
}

/* y = x repeated `size` times along dim (x's extent along dim is 1) */
void ref_broadcast_fw(const float *src, const uint32_t *xdims, uint32_t depth, uint32_t batch, uint32_t dim,
                      uint32_t size, float *dest) {
  const shape_t s = {xdims, depth, batch};
  const uint32_t repeat = volume(s) * batch;
  const uint32_t skip1 = lower_volume(s, dim);
  const uint32_t skip2 = skip1 * size;
  for (uint32_t i = 0; i < repeat; ++i) {
    uint32_t offset = i % skip1 + (i / skip1) * skip2;
    const float tmp = src[i];
    for (uint32_t j = 0; j < size; ++j) {
      dest[offset] = tmp;
      offset += skip1;
    }
  }
}
