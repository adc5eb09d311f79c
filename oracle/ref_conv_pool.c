/*
 * CPU oracle for 2-D convolution and max pooling.  TEST INFRASTRUCTURE ONLY:
 * the checker the GPU library is compared against; never part of the shipped
 * GPU path, and nothing in the product may call it.
 *
 * Restates the loops of primitiv's plain CPU device:
 *   ref_conv2d_fw / _bw      primitiv/devices/naive/ops/conv2d.cc:9-151
 *   ref_max_pool2d_fw / _bw  primitiv/devices/naive/ops/max_pool2d.cc:9-113
 *   ref_shape_conv2d         primitiv/core/shape_ops.cc:162-187
 *   ref_shape_pool2d         primitiv/core/shape_ops.cc:189-213
 * x is H x W x C per sample (H contiguous), w is KH x KW x C x OC, y is
 * OH x OW x OC; bx / bw are the minibatch sizes of x and w (1 = shared).
 * Sums run in double and are rounded once, so that the oracle is the better
 * value when a device result is compared with it.
 *
 * Parity status: pinned by the reference's golden vectors
 * (test/tensor_forward_test.cc CheckConv2D_* :3110-3632, CheckMaxPool2D_*
 * :3708-4025; test/tensor_backward_test.cc CheckConv2D_* :1939-2598,
 * CheckMaxPool2D_* :2614-2952; test/shape_ops_test.cc CheckConv2D / CheckPool2D
 * and their invalid cases), replayed by tests/test_oracle_conv_pool.py, and by
 * scipy.signal.convolve2d / correlate2d and numpy window maxima on random
 * inputs there.
 */
#include <float.h>
#include <stddef.h>
#include <stdint.h>

/* Output extent along one axis, or 0 when the arguments are invalid. */
static uint32_t conv_extent(uint32_t x, uint32_t w, uint32_t pad, uint32_t str, uint32_t dil) {
  if (str == 0 || dil == 0 || w == 0) return 0;
  const uint64_t e = (uint64_t)x + 2ull * pad, k = (uint64_t)(w - 1) * dil + 1;
  if (e < k) return 0;
  return (uint32_t)((e - k) / str + 1);
}

/* dims[3] = {OH, OW, OC}; returns 0 on success, 1 for arguments the reference rejects.
 * The caller passes dims padded with ones (depth checks are the caller's). */
int ref_shape_conv2d(uint32_t x0, uint32_t x1, uint32_t xc, uint32_t bx, uint32_t w0, uint32_t w1, uint32_t wc,
                     uint32_t oc, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1,
                     uint32_t dil0, uint32_t dil1, uint32_t *dims, uint32_t *batch) {
  const uint32_t oh = conv_extent(x0, w0, pad0, str0, dil0), ow = conv_extent(x1, w1, pad1, str1, dil1);
  if (oh == 0 || ow == 0 || xc != wc || !(bx == bw || bx == 1 || bw == 1)) return 1;
  dims[0] = oh; dims[1] = ow; dims[2] = oc;
  *batch = bx > bw ? bx : bw;
  return 0;
}

int ref_shape_pool2d(uint32_t x0, uint32_t x1, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1,
                     uint32_t str0, uint32_t str1, uint32_t *dims) {
  const uint32_t oh = conv_extent(x0, win0, pad0, str0, 1), ow = conv_extent(x1, win1, pad1, str1, 1);
  if (oh == 0 || ow == 0) return 1;
  dims[0] = oh; dims[1] = ow;
  return 0;
}

typedef struct {
  uint32_t H, W, C, KH, KW, OC, OH, OW;
  uint32_t pad0, pad1, str0, str1, dil0, dil1;
} conv_t;

static conv_t conv_of(uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t pad0,
                      uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1) {
  conv_t g = {x0, x1, c, w0, w1, oc, conv_extent(x0, w0, pad0, str0, dil0), conv_extent(x1, w1, pad1, str1, dil1),
              pad0, pad1, str0, str1, dil0, dil1};
  return g;
}

/* conv2d.cc:38-76 */
void ref_conv2d_fw(const float *x, const float *w, float *y, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0,
                   uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0,
                   uint32_t str1, uint32_t dil0, uint32_t dil1) {
  const conv_t g = conv_of(x0, x1, c, w0, w1, oc, pad0, pad1, str0, str1, dil0, dil1);
  const uint32_t bs = bx > bw ? bx : bw;
  const size_t xs = (bx > 1) * (size_t)g.H * g.W * g.C, ws = (bw > 1) * (size_t)g.KH * g.KW * g.C * g.OC;
  const size_t ys = (size_t)g.OH * g.OW * g.OC;
#pragma omp parallel for collapse(2) schedule(static)
  for (uint32_t b = 0; b < bs; ++b)
    for (uint32_t yc = 0; yc < g.OC; ++yc) {
      const float *px = x + b * xs, *pw = w + b * ws;
      float *py = y + b * ys;
      for (uint32_t yx = 0; yx < g.OW; ++yx)
        for (uint32_t yy = 0; yy < g.OH; ++yy) {
          double sum = 0.0;
          for (uint32_t xc = 0; xc < g.C; ++xc)
            for (uint32_t wx = 0; wx < g.KW; ++wx)
              for (uint32_t wy = 0; wy < g.KH; ++wy) {
                const int64_t xy = -(int64_t)g.pad0 + (int64_t)yy * g.str0 + (int64_t)wy * g.dil0;
                const int64_t xx = -(int64_t)g.pad1 + (int64_t)yx * g.str1 + (int64_t)wx * g.dil1;
                if (xy < 0 || xy >= g.H || xx < 0 || xx >= g.W) continue;
                const size_t xa = ((size_t)xc * g.W + xx) * g.H + xy;
                const size_t wa = (((size_t)yc * g.C + xc) * g.KW + (g.KW - 1 - wx)) * g.KH + (g.KH - 1 - wy);
                sum += (double)px[xa] * pw[wa];
              }
          py[((size_t)yc * g.OW + yx) * g.OH + yy] = (float)sum;
        }
    }
}

/* conv2d.cc:107-148: gx and gw are added to; a shared operand's gradient collects every sample */
void ref_conv2d_bw(const float *x, const float *w, const float *gy, float *gx, float *gw, uint32_t x0, uint32_t x1,
                   uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0,
                   uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1) {
  const conv_t g = conv_of(x0, x1, c, w0, w1, oc, pad0, pad1, str0, str1, dil0, dil1);
  const uint32_t bs = bx > bw ? bx : bw;
  const size_t xv = (size_t)g.H * g.W * g.C, wv = (size_t)g.KH * g.KW * g.C * g.OC;
  const size_t xs = (bx > 1) * xv, ws = (bw > 1) * wv, ys = (size_t)g.OH * g.OW * g.OC;
  /* gradient of x: one output element at a time, all its contributions in double */
#pragma omp parallel for schedule(static)
  for (size_t e = 0; e < (bx > 1 ? bs : 1) * xv; ++e) {
    const size_t bq = e / xv, r = e % xv;
    const uint32_t xy = (uint32_t)(r % g.H), xx = (uint32_t)((r / g.H) % g.W), xc = (uint32_t)(r / ((size_t)g.H * g.W));
    double sum = 0.0;
    for (uint32_t b = (bx > 1 ? (uint32_t)bq : 0); b < (bx > 1 ? (uint32_t)bq + 1 : bs); ++b) {
      const float *pw = w + b * ws, *pgy = gy + b * ys;
      for (uint32_t yc = 0; yc < g.OC; ++yc)
        for (uint32_t wx = 0; wx < g.KW; ++wx)
          for (uint32_t wy = 0; wy < g.KH; ++wy) {
            const int64_t ty = (int64_t)xy + g.pad0 - (int64_t)wy * g.dil0;
            const int64_t tx = (int64_t)xx + g.pad1 - (int64_t)wx * g.dil1;
            if (ty < 0 || tx < 0 || ty % g.str0 || tx % g.str1) continue;
            const int64_t yy = ty / g.str0, yx = tx / g.str1;
            if (yy >= g.OH || yx >= g.OW) continue;
            const size_t wa = (((size_t)yc * g.C + xc) * g.KW + (g.KW - 1 - wx)) * g.KH + (g.KH - 1 - wy);
            sum += (double)pgy[((size_t)yc * g.OW + yx) * g.OH + yy] * pw[wa];
          }
    }
    gx[e] = (float)(gx[e] + sum);
  }
  /* gradient of w */
#pragma omp parallel for schedule(static)
  for (size_t e = 0; e < (bw > 1 ? bs : 1) * wv; ++e) {
    const size_t bq = e / wv, r = e % wv;
    const uint32_t wyi = (uint32_t)(r % g.KH), wxi = (uint32_t)((r / g.KH) % g.KW);
    const uint32_t xc = (uint32_t)((r / ((size_t)g.KH * g.KW)) % g.C), yc = (uint32_t)(r / ((size_t)g.KH * g.KW * g.C));
    const uint32_t wy = g.KH - 1 - wyi, wx = g.KW - 1 - wxi;
    double sum = 0.0;
    for (uint32_t b = (bw > 1 ? (uint32_t)bq : 0); b < (bw > 1 ? (uint32_t)bq + 1 : bs); ++b) {
      const float *px = x + b * xs, *pgy = gy + b * ys;
      for (uint32_t yx = 0; yx < g.OW; ++yx)
        for (uint32_t yy = 0; yy < g.OH; ++yy) {
          const int64_t xy = -(int64_t)g.pad0 + (int64_t)yy * g.str0 + (int64_t)wy * g.dil0;
          const int64_t xx = -(int64_t)g.pad1 + (int64_t)yx * g.str1 + (int64_t)wx * g.dil1;
          if (xy < 0 || xy >= g.H || xx < 0 || xx >= g.W) continue;
          sum += (double)pgy[((size_t)yc * g.OW + yx) * g.OH + yy] * px[((size_t)xc * g.W + xx) * g.H + xy];
        }
    }
    gw[e] = (float)(gw[e] + sum);
  }
}

/* max_pool2d.cc:31-56; `repeat` planes of H x W */
void ref_max_pool2d_fw(const float *x, float *y, uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0,
                       uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1) {
  const uint32_t oh = conv_extent(x0, win0, pad0, str0, 1), ow = conv_extent(x1, win1, pad1, str1, 1);
#pragma omp parallel for schedule(static)
  for (uint32_t r = 0; r < repeat; ++r) {
    const float *px = x + (size_t)r * x0 * x1;
    float *py = y + (size_t)r * oh * ow;
    for (uint32_t yx = 0; yx < ow; ++yx)
      for (uint32_t yy = 0; yy < oh; ++yy) {
        float best = -FLT_MAX;
        for (uint32_t wx = 0; wx < win1; ++wx) {
          const int64_t xx = -(int64_t)pad1 + (int64_t)yx * str1 + wx;
          if (xx < 0 || xx >= x1) continue;
          for (uint32_t wy = 0; wy < win0; ++wy) {
            const int64_t xy = -(int64_t)pad0 + (int64_t)yy * str0 + wy;
            if (xy < 0 || xy >= x0) continue;
            const float v = px[xx * x0 + xy];
            if (v > best) best = v;
          }
        }
        py[(size_t)yx * oh + yy] = best;
      }
  }
}

/* max_pool2d.cc:84-112: the first element of the window equal to y receives gy */
void ref_max_pool2d_bw(const float *x, const float *y, const float *gy, float *gx, uint32_t x0, uint32_t x1,
                       uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,
                       uint32_t str1) {
  const uint32_t oh = conv_extent(x0, win0, pad0, str0, 1), ow = conv_extent(x1, win1, pad1, str1, 1);
#pragma omp parallel for schedule(static)
  for (uint32_t r = 0; r < repeat; ++r) {
    const float *px = x + (size_t)r * x0 * x1;
    const float *py = y + (size_t)r * oh * ow, *pgy = gy + (size_t)r * oh * ow;
    float *pgx = gx + (size_t)r * x0 * x1;
    for (uint32_t yx = 0; yx < ow; ++yx)
      for (uint32_t yy = 0; yy < oh; ++yy) {
        const float target = py[(size_t)yx * oh + yy];
        int next = 1;
        for (uint32_t wx = 0; next && wx < win1; ++wx) {
          const int64_t xx = -(int64_t)pad1 + (int64_t)yx * str1 + wx;
          if (xx < 0 || xx >= x1) continue;
          for (uint32_t wy = 0; next && wy < win0; ++wy) {
            const int64_t xy = -(int64_t)pad0 + (int64_t)yy * str0 + wy;
            if (xy < 0 || xy >= x0) continue;
            if (px[xx * x0 + xy] == target) {
              pgx[xx * x0 + xy] += pgy[(size_t)yx * oh + yy];
              next = 0;
            }
          }
        }
      }
  }
}
