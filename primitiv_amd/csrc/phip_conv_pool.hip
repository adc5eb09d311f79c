// 2-D convolution and max pooling of primitiv tensors.
//
// Layouts (column-major, first dimension contiguous): x is H x W x C per
// sample, w is KH x KW x C x OC, y is OH x OW x OC.  conv2d is a true
// convolution: output (oy, ox) pairs tap (wy, wx), counted from the window's
// origin, with the kernel element (KH-1-wy, KW-1-wx)
// (primitiv/devices/naive/ops/conv2d.cc:38-76).
//
// The convolution runs on the matrix cores through the GEMM layer of this
// library.  With n = ox*OH + oy (a position of y's plane, in memory order) and
// k = (c*KW + (KW-1-wx))*KH + (KH-1-wy) (a position inside one output
// channel's kernel, in memory order):
//   col[k][n]   = x at the tap (c, wy, wx) of output n, 0 outside the image,
//   y   (N x OC) = col^T (N x K) . w (K x OC)            forward
//   gcol(N x K ) = gy (N x OC) . w^T (OC x K)            backward, then
//   gx          += the taps of gcol that land on each element of x,
//   gw  (K x OC)+= col (K x N) . gy (N x OC)             (summed over the
//                                                         minibatch when w is shared)
// so that w and y are used in place as GEMM operands and only col / gcol are
// scratch (pool memory, a bounded number of samples at a time).  A 1 x 1
// kernel with unit stride and no padding needs no col at all: col == x.
//
// Max pooling: one thread per output scans its window; the gradient goes to
// the FIRST element of the window (wx outer, wy inner) equal to y
// (naive/ops/max_pool2d.cc:88-104).  Backward first records that element's
// position per output, then every element of gx gathers from the windows that
// contain it: no atomics, the same bits on every run, any storage type.
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

constexpr int kBlock = 256;
constexpr uint32_t kNoPosition = 0xffffffffu;
// col / gcol scratch per group of samples (elements)
constexpr long kScratchElements = 128L << 20;

struct ConvGeom {
  int H, W, C;      // x
  int KH, KW, OC;   // w
  int OH, OW;       // y
  int pad0, pad1, str0, str1, dil0, dil1;
};

// col[z][k][n] for the samples of x.  A thread owns one output position n of
// one channel c (blockIdx.y) of one sample (blockIdx.z) and walks the KH x KW
// taps: per tap one load and one store that are contiguous across the
// wavefront, and everything but n's two coordinates is uniform.
template <typename T>
__global__ __launch_bounds__(kBlock) void im2col_kernel(const T *x, T *col, const ConvGeom g, long x_stride) {
  const int N = g.OH * g.OW;
  const int n = blockIdx.x * kBlock + threadIdx.x;
  if (n >= N) return;
  const int c = blockIdx.y, z = blockIdx.z;
  const long K = (long)g.C * g.KW * g.KH;
  const T *xs = x + z * x_stride + (long)c * g.W * g.H;
  T *dst = col + ((long)z * K + (long)c * g.KW * g.KH) * N + n;
  const int ox = n / g.OH, oy = n - ox * g.OH;
  const int y0 = oy * g.str0 - g.pad0, x0 = ox * g.str1 - g.pad1;
  for (int wx = 0; wx < g.KW; ++wx) {
    const int xx = x0 + wx * g.dil1;
    const bool in_x = xx >= 0 && xx < g.W;
    const T *xc = xs + (long)xx * g.H;
    T *dc = dst + (long)(g.KW - 1 - wx) * g.KH * N;
    for (int wy = 0; wy < g.KH; ++wy) {
      const int xy = y0 + wy * g.dil0;
      const bool in = in_x && xy >= 0 && xy < g.H;
      dc[(long)(g.KH - 1 - wy) * N] = in ? xc[xy] : from_f32<T>(0.0f);
    }
  }
}

// gx[zx] += the taps of gcol[z] that land on each of its elements; `fold`
// samples of gcol go into every sample of gx (all of them when x is shared).
// A thread owns one position of one channel (blockIdx.y) of one sample of gx
// (blockIdx.z).
template <typename T>
__global__ __launch_bounds__(kBlock) void col2im_kernel(const T *gcol, T *gx, const ConvGeom g, int fold) {
  const int plane = g.H * g.W;
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p >= plane) return;
  const int c = blockIdx.y;
  const long zx = blockIdx.z;
  const long K = (long)g.C * g.KW * g.KH;
  const long N = (long)g.OH * g.OW;
  const int xx = p / g.H, xy = p - xx * g.H;
  float sum = 0.0f;
  for (int f = 0; f < fold; ++f) {
    const T *src = gcol + ((zx * fold + f) * K + (long)c * g.KW * g.KH) * N;
    for (int wx = 0; wx < g.KW; ++wx) {
      const int px = xx + g.pad1 - wx * g.dil1;
      if (px < 0) continue;
      const int ox = g.str1 == 1 ? px : px / g.str1;
      if (ox >= g.OW || ox * g.str1 != px) continue;
      const T *sc = src + (long)(g.KW - 1 - wx) * g.KH * N + (long)ox * g.OH;
      for (int wy = 0; wy < g.KH; ++wy) {
        const int py = xy + g.pad0 - wy * g.dil0;
        if (py < 0) continue;
        const int oy = g.str0 == 1 ? py : py / g.str0;
        if (oy >= g.OH || oy * g.str0 != py) continue;
        sum += to_f32(sc[(long)(g.KH - 1 - wy) * N + oy]);
      }
    }
  }
  T *dst = gx + (zx * g.C + c) * plane + p;
  *dst = from_f32<T>(to_f32(*dst) + sum);
}

template <typename T>
int run_gemm(phip_ctx *ctx, const Gemm &p) {
  if constexpr (sizeof(T) == 4) return gemm_f32(ctx, p);
  else if constexpr (__is_same(T, f16_t)) return gemm_h16(ctx, p, Elem::F16);
  else return gemm_h16(ctx, p, Elem::BF16);
}

struct ConvArgs {
  uint32_t x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1;
};

int conv_geometry(const ConvArgs &a, ConvGeom *g) {
  PHIP_REQUIRE(a.x0 >= 1 && a.x1 >= 1 && a.c >= 1 && a.w0 >= 1 && a.w1 >= 1 && a.oc >= 1, "empty operand");
  PHIP_REQUIRE(a.str0 >= 1 && a.str1 >= 1 && a.dil0 >= 1 && a.dil1 >= 1, "stride and dilation must be positive");
  PHIP_REQUIRE(a.bx >= 1 && a.bw >= 1 && (a.bx == a.bw || a.bx == 1 || a.bw == 1),
               "Invalid arguments to calculate a convolution: batch sizes %u and %u", a.bx, a.bw);
  const uint64_t lim = 1u << 30;
  PHIP_REQUIRE(a.x0 < lim && a.x1 < lim && a.c < lim && a.w0 < lim && a.w1 < lim && a.oc < lim && a.pad0 < lim &&
               a.pad1 < lim && a.str0 < lim && a.str1 < lim && a.dil0 < lim && a.dil1 < lim, "argument out of range");
  const uint64_t e0 = (uint64_t)a.x0 + 2ull * a.pad0, e1 = (uint64_t)a.x1 + 2ull * a.pad1;
  const uint64_t k0 = (uint64_t)(a.w0 - 1) * a.dil0 + 1, k1 = (uint64_t)(a.w1 - 1) * a.dil1 + 1;
  PHIP_REQUIRE(e0 >= k0 && e1 >= k1, "Invalid arguments to calculate a convolution: the kernel exceeds the padded image");
  const uint64_t oh = (e0 - k0) / a.str0 + 1, ow = (e1 - k1) / a.str1 + 1;
  const uint64_t n = oh * ow, k = (uint64_t)a.c * a.w0 * a.w1;
  PHIP_REQUIRE(n < (1ull << 31) && k < (1ull << 31) && n * k < (1ull << 40) &&
               (uint64_t)a.x0 * a.x1 * a.c < (1ull << 31), "convolution too large");
  g->H = a.x0; g->W = a.x1; g->C = a.c;
  g->KH = a.w0; g->KW = a.w1; g->OC = a.oc;
  g->OH = (int)oh; g->OW = (int)ow;
  g->pad0 = a.pad0; g->pad1 = a.pad1; g->str0 = a.str0; g->str1 = a.str1; g->dil0 = a.dil0; g->dil1 = a.dil1;
  return PHIP_OK;
}

bool col_is_x(const ConvGeom &g) {
  return g.KH == 1 && g.KW == 1 && g.pad0 == 0 && g.pad1 == 0 && g.str0 == 1 && g.str1 == 1;
}

template <typename T>
int launch_im2col(phip_ctx *ctx, const T *x, T *col, const ConvGeom &g, long x_stride, int samples) {
  const long K = (long)g.C * g.KW * g.KH;
  const long N = (long)g.OH * g.OW;
  PHIP_REQUIRE(g.C <= 65535, "%d channels exceed what one launch covers", g.C);
  for (int z0 = 0; z0 < samples; z0 += 65535) {
    const int zs = samples - z0 < 65535 ? samples - z0 : 65535;
    hipLaunchKernelGGL(im2col_kernel<T>, dim3((unsigned)((N + kBlock - 1) / kBlock), (unsigned)g.C, (unsigned)zs),
                       dim3(kBlock), 0, ctx->stream, x + (long)z0 * x_stride, col + (long)z0 * K * N, g, x_stride);
    PHIP_LAUNCH_CHECK();
  }
  return PHIP_OK;
}

// gx (`samples` of them) += gcol, `fold` samples of gcol per sample of gx
template <typename T>
int launch_col2im(phip_ctx *ctx, const T *gcol, T *gx, const ConvGeom &g, int samples, int fold) {
  const long K = (long)g.C * g.KW * g.KH;
  const long N = (long)g.OH * g.OW;
  const long plane = (long)g.H * g.W;
  PHIP_REQUIRE(g.C <= 65535, "%d channels exceed what one launch covers", g.C);
  for (int z0 = 0; z0 < samples; z0 += 65535) {
    const int zs = samples - z0 < 65535 ? samples - z0 : 65535;
    hipLaunchKernelGGL(col2im_kernel<T>, dim3((unsigned)((plane + kBlock - 1) / kBlock), (unsigned)g.C, (unsigned)zs),
                       dim3(kBlock), 0, ctx->stream, gcol + (long)z0 * fold * K * N, gx + (long)z0 * plane * g.C, g,
                       fold);
    PHIP_LAUNCH_CHECK();
  }
  return PHIP_OK;
}

// samples per group so that col (and gcol) stay within the scratch bound
int group_size(const ConvGeom &g, int bs) {
  const long per = (long)g.C * g.KW * g.KH * g.OH * g.OW;
  long n = kScratchElements / per;
  if (n < 1) n = 1;
  return (int)(n < bs ? n : bs);
}

template <typename T>
int conv2d_fw(phip_ctx *ctx, const void *xv, const void *wv, void *yv, const ConvArgs &a) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(xv != nullptr && wv != nullptr && yv != nullptr, "null tensor pointer");
  ConvGeom g;
  int rc = conv_geometry(a, &g);
  if (rc != PHIP_OK) return rc;
  const T *x = static_cast<const T *>(xv);
  const T *w = static_cast<const T *>(wv);
  T *y = static_cast<T *>(yv);
  const int bs = (int)(a.bx > a.bw ? a.bx : a.bw);
  const int K = g.C * g.KW * g.KH;
  const long N = (long)g.OH * g.OW;
  const long x_vol = (long)g.H * g.W * g.C, w_vol = (long)K * g.OC, y_vol = N * g.OC;

  Gemm p;
  p.M = (int)N; p.N = g.OC; p.K = K;
  p.lda = N; p.ldb = K; p.ldc = N;
  p.a_kmajor = false;
  p.b_kmajor = true;
  p.accumulate = false;
  p.sB = a.bw > 1 ? w_vol : 0;
  p.sC = y_vol;
  if (col_is_x(g)) {
    p.A = x; p.B = w; p.C = y;
    p.sA = a.bx > 1 ? x_vol : 0;
    p.batch = bs;
    return run_gemm<T>(ctx, p);
  }
  // a shared x has one col for all samples
  const int col_samples = a.bx > 1 ? group_size(g, bs) : 1;
  void *block = nullptr;
  rc = phip_pool_alloc(ctx, sizeof(T) * (size_t)col_samples * K * N, &block, nullptr);
  if (rc != PHIP_OK) return rc;
  T *col = static_cast<T *>(block);
  const int step = a.bx > 1 ? col_samples : bs;
  for (int z0 = 0; z0 < bs && rc == PHIP_OK; z0 += step) {
    const int zs = step < bs - z0 ? step : bs - z0;
    rc = launch_im2col<T>(ctx, x + (a.bx > 1 ? z0 * x_vol : 0), col, g, x_vol, a.bx > 1 ? zs : 1);
    if (rc != PHIP_OK) break;
    p.A = col;
    p.B = w + (a.bw > 1 ? z0 * w_vol : 0);
    p.C = y + z0 * y_vol;
    p.sA = a.bx > 1 ? (long)K * N : 0;
    p.batch = zs;
    rc = run_gemm<T>(ctx, p);
  }
  phip_pool_free(ctx, block);  // the stream is in order: reusable behind these launches
  return rc;
}

template <typename T>
int conv2d_bw(phip_ctx *ctx, const void *xv, const void *wv, const void *gyv, void *gxv, void *gwv,
              const ConvArgs &a) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(xv != nullptr && wv != nullptr && gyv != nullptr && gxv != nullptr && gwv != nullptr,
               "null tensor pointer");
  ConvGeom g;
  int rc = conv_geometry(a, &g);
  if (rc != PHIP_OK) return rc;
  const T *x = static_cast<const T *>(xv);
  const T *w = static_cast<const T *>(wv);
  const T *gy = static_cast<const T *>(gyv);
  T *gx = static_cast<T *>(gxv);
  T *gw = static_cast<T *>(gwv);
  const int bs = (int)(a.bx > a.bw ? a.bx : a.bw);
  const int K = g.C * g.KW * g.KH;
  const long N = (long)g.OH * g.OW;
  const long x_vol = (long)g.H * g.W * g.C, w_vol = (long)K * g.OC, y_vol = N * g.OC;
  const bool direct = col_is_x(g);

  // gcol = gy . w^T (for a 1 x 1 kernel: straight into gx); gw += col . gy
  Gemm pg;
  pg.M = (int)N; pg.N = K; pg.K = g.OC;
  pg.lda = N; pg.ldb = K; pg.ldc = N;
  pg.a_kmajor = false;
  pg.b_kmajor = false;
  pg.sA = y_vol;
  pg.sB = a.bw > 1 ? w_vol : 0;
  Gemm pw;
  pw.M = K; pw.N = g.OC; pw.K = (int)N;
  pw.lda = N; pw.ldb = N; pw.ldc = K;
  pw.a_kmajor = true;
  pw.b_kmajor = true;
  pw.accumulate = true;

  const int group = group_size(g, bs);
  void *col_block = nullptr, *gcol_block = nullptr;
  if (!direct) {
    rc = phip_pool_alloc(ctx, sizeof(T) * (size_t)(a.bx > 1 ? group : 1) * K * N, &col_block, nullptr);
    if (rc != PHIP_OK) return rc;
  }
  if (!direct || a.bx == 1) {
    // a shared x collects every sample's gcol: they are summed by the gather below
    rc = phip_pool_alloc(ctx, sizeof(T) * (size_t)group * K * N, &gcol_block, nullptr);
    if (rc != PHIP_OK) {
      if (col_block) phip_pool_free(ctx, col_block);
      return rc;
    }
  }
  T *col = static_cast<T *>(col_block);
  T *gcol = static_cast<T *>(gcol_block);
  if (!direct && a.bx == 1) rc = launch_im2col<T>(ctx, x, col, g, x_vol, 1);

  for (int z0 = 0; z0 < bs && rc == PHIP_OK; z0 += group) {
    const int zs = group < bs - z0 ? group : bs - z0;
    if (!direct && a.bx > 1) {
      rc = launch_im2col<T>(ctx, x + z0 * x_vol, col, g, x_vol, zs);
      if (rc != PHIP_OK) break;
    }
    // gradient of x
    pg.A = gy + z0 * y_vol;
    pg.B = w + (a.bw > 1 ? z0 * w_vol : 0);
    pg.batch = zs;
    if (direct && a.bx > 1) {
      pg.C = gx + z0 * x_vol;
      pg.sC = x_vol;
      pg.accumulate = true;
      rc = run_gemm<T>(ctx, pg);
    } else {
      pg.C = gcol;
      pg.sC = (long)K * N;
      pg.accumulate = false;
      rc = run_gemm<T>(ctx, pg);
      if (rc != PHIP_OK) break;
      rc = a.bx > 1 ? launch_col2im<T>(ctx, gcol, gx + z0 * x_vol, g, zs, 1) : launch_col2im<T>(ctx, gcol, gx, g, 1, zs);
    }
    if (rc != PHIP_OK) break;
    // gradient of w
    const T *cz = direct ? x + (a.bx > 1 ? z0 * x_vol : 0) : col;
    const long c_stride = a.bx > 1 ? (direct ? x_vol : (long)K * N) : 0;
    pw.A = cz;
    pw.B = gy + z0 * y_vol;
    if (a.bw > 1) {
      pw.C = gw + z0 * w_vol;
      pw.batch = zs;
      pw.rbatch = 1;
      pw.sA = c_stride; pw.sB = y_vol; pw.sC = w_vol;
      pw.rA = pw.rB = 0;
    } else {
      pw.C = gw;
      pw.batch = 1;
      pw.rbatch = zs;
      pw.rA = c_stride; pw.rB = y_vol;
      pw.sA = pw.sB = pw.sC = 0;
    }
    rc = run_gemm<T>(ctx, pw);
  }
  if (gcol_block) phip_pool_free(ctx, gcol_block);
  if (col_block) phip_pool_free(ctx, col_block);
  return rc;
}

// ---- max pooling ------------------------------------------------------------------

struct PoolGeom {
  int H, W, OH, OW;
  int win0, win1, pad0, pad1, str0, str1;
};

template <typename T>
__global__ __launch_bounds__(kBlock) void max_pool2d_fw_kernel(const T *x, T *y, const PoolGeom g) {
  const long plane_y = (long)g.OH * g.OW, plane_x = (long)g.H * g.W;
  const int n = blockIdx.x * kBlock + threadIdx.x;
  if (n < plane_y) {
    const long r = blockIdx.y + (long)blockIdx.z * gridDim.y;
    const long i = r * plane_y + n;
    const int ox = n / g.OH, oy = n - ox * g.OH;
    const T *xs = x + r * plane_x;
    float best = -3.402823466e+38f;  // the lowest finite float, as std::numeric_limits<float>::lowest()
    for (int wx = 0; wx < g.win1; ++wx) {
      const int xx = ox * g.str1 - g.pad1 + wx;
      if (xx < 0 || xx >= g.W) continue;
      for (int wy = 0; wy < g.win0; ++wy) {
        const int xy = oy * g.str0 - g.pad0 + wy;
        if (xy < 0 || xy >= g.H) continue;
        const float v = to_f32(xs[(long)xx * g.H + xy]);
        if (v > best) best = v;
      }
    }
    y[i] = from_f32<T>(best);
  }
}

// position (inside x's plane) of the first element of each window equal to y
template <typename T>
__global__ __launch_bounds__(kBlock) void max_pool2d_where_kernel(const T *x, const T *y, uint32_t *where,
                                                                 const PoolGeom g) {
  const long plane_y = (long)g.OH * g.OW, plane_x = (long)g.H * g.W;
  const int n = blockIdx.x * kBlock + threadIdx.x;
  if (n < plane_y) {
    const long r = blockIdx.y + (long)blockIdx.z * gridDim.y;
    const long i = r * plane_y + n;
    const int ox = n / g.OH, oy = n - ox * g.OH;
    const T *xs = x + r * plane_x;
    const float target = to_f32(y[i]);
    uint32_t pos = kNoPosition;
    for (int wx = 0; wx < g.win1 && pos == kNoPosition; ++wx) {
      const int xx = ox * g.str1 - g.pad1 + wx;
      if (xx < 0 || xx >= g.W) continue;
      for (int wy = 0; wy < g.win0; ++wy) {
        const int xy = oy * g.str0 - g.pad0 + wy;
        if (xy < 0 || xy >= g.H) continue;
        if (to_f32(xs[(long)xx * g.H + xy]) == target) {
          pos = (uint32_t)(xx * g.H + xy);
          break;
        }
      }
    }
    where[i] = pos;
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void max_pool2d_bw_kernel(const T *gy, const uint32_t *where, T *gx,
                                                              const PoolGeom g) {
  const long plane_y = (long)g.OH * g.OW, plane_x = (long)g.H * g.W;
  const int p = blockIdx.x * kBlock + threadIdx.x;
  if (p < plane_x) {
    const long r = blockIdx.y + (long)blockIdx.z * gridDim.y;
    const long i = r * plane_x + p;
    const int xx = p / g.H, xy = p - xx * g.H;
    // windows (oy, ox) that contain (xy, xx): o*str - pad <= x < o*str - pad + win
    const int ty = xy + g.pad0, tx = xx + g.pad1;
    int oy_lo = ty - g.win0 + 1 > 0 ? (ty - g.win0 + g.str0) / g.str0 : 0;
    int ox_lo = tx - g.win1 + 1 > 0 ? (tx - g.win1 + g.str1) / g.str1 : 0;
    int oy_hi = ty / g.str0, ox_hi = tx / g.str1;
    if (oy_hi >= g.OH) oy_hi = g.OH - 1;
    if (ox_hi >= g.OW) ox_hi = g.OW - 1;
    float sum = 0.0f;
    bool any = false;
    for (int ox = ox_lo; ox <= ox_hi; ++ox)
      for (int oy = oy_lo; oy <= oy_hi; ++oy) {
        const long o = r * plane_y + (long)ox * g.OH + oy;
        if (where[o] == (uint32_t)p) {
          sum += to_f32(gy[o]);
          any = true;
        }
      }
    if (any) gx[i] = from_f32<T>(to_f32(gx[i]) + sum);
  }
}

// Windows that do not overlap (stride >= window on both axes): every element of
// gx belongs to at most one window, so the thread that owns an output finds the
// first element equal to y and adds gy to it directly - one launch, no scratch.
template <typename T>
__global__ __launch_bounds__(kBlock) void max_pool2d_bw_disjoint_kernel(const T *x, const T *y, const T *gy, T *gx,
                                                                       const PoolGeom g) {
  const int plane_y = g.OH * g.OW;
  const int n = blockIdx.x * kBlock + threadIdx.x;
  if (n >= plane_y) return;
  const long r = blockIdx.y + (long)blockIdx.z * gridDim.y;
  const long plane_x = (long)g.H * g.W;
  const int ox = n / g.OH, oy = n - ox * g.OH;
  const T *xs = x + r * plane_x;
  const float target = to_f32(y[r * plane_y + n]);
  for (int wx = 0; wx < g.win1; ++wx) {
    const int xx = ox * g.str1 - g.pad1 + wx;
    if (xx < 0 || xx >= g.W) continue;
    for (int wy = 0; wy < g.win0; ++wy) {
      const int xy = oy * g.str0 - g.pad0 + wy;
      if (xy < 0 || xy >= g.H) continue;
      const long p = (long)xx * g.H + xy;
      if (to_f32(xs[p]) == target) {
        T *dst = gx + r * plane_x + p;
        *dst = from_f32<T>(to_f32(*dst) + to_f32(gy[r * plane_y + n]));
        return;
      }
    }
  }
}

// Calls launch(first_plane, grid_y, grid_z) until `repeat` planes are covered;
// a kernel finds its plane as first_plane + blockIdx.y + blockIdx.z * gridDim.y.
template <typename F>
int for_plane_grids(uint32_t repeat, F launch) {
  const unsigned wide = repeat < 65535u ? repeat : 65535u;
  for (uint32_t r0 = 0; r0 < repeat;) {
    const uint32_t left = repeat - r0;
    unsigned gz = left / wide;
    if (gz > 65535u) gz = 65535u;
    const unsigned yd = gz == 0 ? left : wide, zd = gz == 0 ? 1u : gz;
    launch(r0, yd, zd);
    PHIP_LAUNCH_CHECK();
    r0 += yd * zd;
  }
  return PHIP_OK;
}

struct PoolArgs {
  uint32_t x0, x1, repeat, win0, win1, pad0, pad1, str0, str1;
};

int pool_geometry(const PoolArgs &a, PoolGeom *g) {
  PHIP_REQUIRE(a.x0 >= 1 && a.x1 >= 1, "empty operand");
  PHIP_REQUIRE(a.win0 >= 1 && a.win1 >= 1 && a.str0 >= 1 && a.str1 >= 1, "window and stride must be positive");
  const uint64_t lim = 1u << 30;
  PHIP_REQUIRE(a.x0 < lim && a.x1 < lim && a.win0 < lim && a.win1 < lim && a.pad0 < lim && a.pad1 < lim &&
               a.str0 < lim && a.str1 < lim, "argument out of range");
  const uint64_t e0 = (uint64_t)a.x0 + 2ull * a.pad0, e1 = (uint64_t)a.x1 + 2ull * a.pad1;
  PHIP_REQUIRE(e0 >= a.win0 && e1 >= a.win1, "Invalid arguments to calculate a pooling: the window exceeds the padded image");
  PHIP_REQUIRE((uint64_t)a.x0 * a.x1 < (1ull << 31), "image plane too large");
  g->H = a.x0; g->W = a.x1;
  g->OH = (int)((e0 - a.win0) / a.str0 + 1);
  g->OW = (int)((e1 - a.win1) / a.str1 + 1);
  g->win0 = a.win0; g->win1 = a.win1; g->pad0 = a.pad0; g->pad1 = a.pad1; g->str0 = a.str0; g->str1 = a.str1;
  return PHIP_OK;
}

template <typename T>
int max_pool2d_fw(phip_ctx *ctx, const void *x, void *y, const PoolArgs &a) {
  PHIP_ENTER(ctx);
  if (a.repeat == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null tensor pointer");
  PoolGeom g;
  const int rc = pool_geometry(a, &g);
  if (rc != PHIP_OK) return rc;
  const long px = (long)g.H * g.W, py = (long)g.OH * g.OW;
  return for_plane_grids(a.repeat, [&](uint32_t r0, unsigned yd, unsigned zd) {
    hipLaunchKernelGGL(max_pool2d_fw_kernel<T>, dim3((unsigned)((py + kBlock - 1) / kBlock), yd, zd), dim3(kBlock), 0,
                       ctx->stream, static_cast<const T *>(x) + r0 * px, static_cast<T *>(y) + r0 * py, g);
  });
}

template <typename T>
int max_pool2d_bw(phip_ctx *ctx, const void *x, const void *y, const void *gy, void *gx, const PoolArgs &a) {
  PHIP_ENTER(ctx);
  if (a.repeat == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr && gy != nullptr && gx != nullptr, "null tensor pointer");
  PoolGeom g;
  int rc = pool_geometry(a, &g);
  if (rc != PHIP_OK) return rc;
  const long px = (long)g.H * g.W, py = (long)g.OH * g.OW;
  const T *xp = static_cast<const T *>(x), *yp = static_cast<const T *>(y), *gyp = static_cast<const T *>(gy);
  T *gxp = static_cast<T *>(gx);
  if (g.str0 >= g.win0 && g.str1 >= g.win1) {
    return for_plane_grids(a.repeat, [&](uint32_t r0, unsigned yd, unsigned zd) {
      hipLaunchKernelGGL(max_pool2d_bw_disjoint_kernel<T>, dim3((unsigned)((py + kBlock - 1) / kBlock), yd, zd),
                         dim3(kBlock), 0, ctx->stream, xp + r0 * px, yp + r0 * py, gyp + r0 * py, gxp + r0 * px, g);
    });
  }
  void *block = nullptr;
  rc = phip_pool_alloc(ctx, sizeof(uint32_t) * (size_t)py * a.repeat, &block, nullptr);
  if (rc != PHIP_OK) return rc;
  uint32_t *where = static_cast<uint32_t *>(block);
  rc = for_plane_grids(a.repeat, [&](uint32_t r0, unsigned yd, unsigned zd) {
    hipLaunchKernelGGL(max_pool2d_where_kernel<T>, dim3((unsigned)((py + kBlock - 1) / kBlock), yd, zd), dim3(kBlock),
                       0, ctx->stream, xp + r0 * px, yp + r0 * py, where + r0 * py, g);
  });
  if (rc == PHIP_OK)
    rc = for_plane_grids(a.repeat, [&](uint32_t r0, unsigned yd, unsigned zd) {
      hipLaunchKernelGGL(max_pool2d_bw_kernel<T>, dim3((unsigned)((px + kBlock - 1) / kBlock), yd, zd), dim3(kBlock), 0,
                         ctx->stream, gyp + r0 * py, where + r0 * py, gxp + r0 * px, g);
    });
  phip_pool_free(ctx, block);  // the stream is in order: reusable behind these launches
  return rc;
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_CONV_POOL(SUF, T, CPTR, PTR)                                                                   \
  int phip_conv2d_fw_##SUF(phip_ctx *ctx, CPTR x, CPTR w, PTR y, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, \
                           uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1,        \
                           uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1) {                            \
    const ConvArgs a = {x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1};                         \
    return conv2d_fw<T>(ctx, x, w, y, a);                                                                           \
  }                                                                                                                \
  int phip_conv2d_bw_##SUF(phip_ctx *ctx, CPTR x, CPTR w, CPTR gy, PTR gx, PTR gw, uint32_t x0, uint32_t x1,        \
                           uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw,             \
                           uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0,               \
                           uint32_t dil1) {                                                                         \
    const ConvArgs a = {x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1};                         \
    return conv2d_bw<T>(ctx, x, w, gy, gx, gw, a);                                                                  \
  }                                                                                                                \
  int phip_max_pool2d_fw_##SUF(phip_ctx *ctx, CPTR x, PTR y, uint32_t x0, uint32_t x1, uint32_t repeat,             \
                               uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,           \
                               uint32_t str1) {                                                                     \
    const PoolArgs a = {x0, x1, repeat, win0, win1, pad0, pad1, str0, str1};                                        \
    return max_pool2d_fw<T>(ctx, x, y, a);                                                                          \
  }                                                                                                                \
  int phip_max_pool2d_bw_##SUF(phip_ctx *ctx, CPTR x, CPTR y, CPTR gy, PTR gx, uint32_t x0, uint32_t x1,            \
                               uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1,         \
                               uint32_t str0, uint32_t str1) {                                                      \
    const PoolArgs a = {x0, x1, repeat, win0, win1, pad0, pad1, str0, str1};                                        \
    return max_pool2d_bw<T>(ctx, x, y, gy, gx, a);                                                                  \
  }

PHIP_EXPORT_CONV_POOL(f32, float, const float *, float *)
PHIP_EXPORT_CONV_POOL(f16, f16_t, const void *, void *)
PHIP_EXPORT_CONV_POOL(bf16, bf16_t, const void *, void *)

#undef PHIP_EXPORT_CONV_POOL

}  // extern "C"
