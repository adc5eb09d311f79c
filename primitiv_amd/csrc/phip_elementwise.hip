// Streaming helpers around the matmul path: fill, storage conversion,
// broadcasting in-place add / subtract and minibatch sum.  All are HBM-bound; each
// element is read once and written once.
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {

static constexpr int kBlock = 256;

static inline unsigned grid_for(size_t n, int per_thread, const phip_ctx *ctx) {
  const size_t blocks = (n + (size_t)kBlock * per_thread - 1) / ((size_t)kBlock * per_thread);
  const size_t cap = (size_t)ctx->prop.multiProcessorCount * 16;
  return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

template <typename T>
__global__ __launch_bounds__(kBlock) void fill_kernel(T *p, float value, size_t n) {
  const T v = from_f32<T>(value);
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    p[i] = v;
  }
}

template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void cvt_kernel(const S *__restrict__ src, D *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    dst[i] = from_f32<D>(to_f32(src[i]));
  }
}

// y[n][i] += sign * x[n or 0][i]   (by == bs; x advances only when it has a batch)
template <typename T>
__global__ __launch_bounds__(kBlock) void add_same_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                          size_t volume, size_t total, bool x_batched, float sign) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < total; i += (size_t)gridDim.x * kBlock) {
    const size_t xi = x_batched ? i : i % volume;
    y[i] = from_f32<T>(to_f32(y[i]) + sign * to_f32(x[xi]));
  }
}

// y[i] (+)= sign * sum_n x[n][i]; one thread owns one output element, so the
// reduction needs no atomics and its order is fixed.
template <typename T, bool kAccumulate>
__global__ __launch_bounds__(kBlock) void batch_reduce_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                              size_t volume, uint32_t bs, float sign) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < volume; i += (size_t)gridDim.x * kBlock) {
    float s = kAccumulate ? to_f32(y[i]) : 0.0f;
    const T *px = x + i;
    for (uint32_t n = 0; n < bs; ++n) {
      s += sign * to_f32(*px);
      px += volume;
    }
    y[i] = from_f32<T>(s);
  }
}

template <typename T>
static int fill_impl(phip_ctx *ctx, void *p, float value, size_t n) {
  PHIP_ENTER_HOST(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(p != nullptr, "null pointer");
  // A fill is the one operation that sits between the matrix products of a backward pass (every
  // gradient is reset before products are added into it) and it names its memory as they do: it
  // takes a lane like a product instead of releasing the lanes (phip_lanes.hip).
  // (fp32 only: the products of 16-bit storage never leave the main lane.)
  if (sizeof(T) == sizeof(float)) {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
    const phip::MemRange written = {lo, lo + n * sizeof(T), true};
    const int rc = phip::lanes_place(ctx, &written, 1, n * sizeof(T) <= ((size_t)64 << 20), &ctx);
    if (rc != PHIP_OK) return rc;
  } else if (ctx->lanes != nullptr) {
    const int rc = phip::lanes_join(ctx);
    if (rc != PHIP_OK) return rc;
  }
  hipLaunchKernelGGL(fill_kernel<T>, dim3(grid_for(n, 4, ctx)), dim3(kBlock), 0, ctx->stream,
                     static_cast<T *>(p), value, n);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename S, typename D>
static int cvt_impl(phip_ctx *ctx, const void *src, void *dst, size_t n) {
  PHIP_ENTER(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  hipLaunchKernelGGL((cvt_kernel<S, D>), dim3(grid_for(n, 4, ctx)), dim3(kBlock), 0, ctx->stream,
                     static_cast<const S *>(src), static_cast<D *>(dst), n);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
static int inplace_add_impl(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx,
                            uint32_t by, float sign) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(bx >= 1 && by >= 1 && (bx == by || bx == 1 || by == 1),
               "incompatible batch sizes: %u, %u", bx, by);
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  if (by == 1 && bx > 1) {
    hipLaunchKernelGGL((batch_reduce_kernel<T, true>), dim3(grid_for(volume, 1, ctx)), dim3(kBlock), 0,
                       ctx->stream, static_cast<const T *>(x), static_cast<T *>(y), (size_t)volume, bx, sign);
  } else {
    const size_t total = (size_t)volume * by;
    hipLaunchKernelGGL(add_same_kernel<T>, dim3(grid_for(total, 4, ctx)), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(x), static_cast<T *>(y), (size_t)volume, total, bx > 1, sign);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
static int batch_sum_impl(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(bs >= 1, "batch size must be positive");
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  hipLaunchKernelGGL((batch_reduce_kernel<T, false>), dim3(grid_for(volume, 1, ctx)), dim3(kBlock), 0,
                     ctx->stream, static_cast<const T *>(x), static_cast<T *>(y), (size_t)volume, bs, 1.0f);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace phip

using namespace phip;

extern "C" {

int phip_fill_f32(phip_ctx *ctx, float *p, float v, size_t n) { return fill_impl<float>(ctx, p, v, n); }
int phip_fill_f16(phip_ctx *ctx, void *p, float v, size_t n) { return fill_impl<f16_t>(ctx, p, v, n); }
int phip_fill_bf16(phip_ctx *ctx, void *p, float v, size_t n) { return fill_impl<bf16_t>(ctx, p, v, n); }

int phip_cvt_f32_to_f16(phip_ctx *ctx, const float *s, void *d, size_t n) { return cvt_impl<float, f16_t>(ctx, s, d, n); }
int phip_cvt_f16_to_f32(phip_ctx *ctx, const void *s, float *d, size_t n) { return cvt_impl<f16_t, float>(ctx, s, d, n); }
int phip_cvt_f32_to_bf16(phip_ctx *ctx, const float *s, void *d, size_t n) { return cvt_impl<float, bf16_t>(ctx, s, d, n); }
int phip_cvt_bf16_to_f32(phip_ctx *ctx, const void *s, float *d, size_t n) { return cvt_impl<bf16_t, float>(ctx, s, d, n); }

int phip_inplace_add_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<float>(ctx, x, y, volume, bx, by, 1.0f);
}
int phip_inplace_add_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<f16_t>(ctx, x, y, volume, bx, by, 1.0f);
}
int phip_inplace_add_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<bf16_t>(ctx, x, y, volume, bx, by, 1.0f);
}

int phip_inplace_subtract_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<float>(ctx, x, y, volume, bx, by, -1.0f);
}
int phip_inplace_subtract_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<f16_t>(ctx, x, y, volume, bx, by, -1.0f);
}
int phip_inplace_subtract_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  return inplace_add_impl<bf16_t>(ctx, x, y, volume, bx, by, -1.0f);
}

int phip_batch_sum_f32(phip_ctx *ctx, const float *x, float *y, uint32_t volume, uint32_t bs) {
  return batch_sum_impl<float>(ctx, x, y, volume, bs);
}
int phip_batch_sum_f16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs) {
  return batch_sum_impl<f16_t>(ctx, x, y, volume, bs);
}
int phip_batch_sum_bf16(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs) {
  return batch_sum_impl<bf16_t>(ctx, x, y, volume, bs);
}

}  // extern "C"
