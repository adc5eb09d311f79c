// Streaming helpers around the matmul path: fill, storage conversion,
// broadcasting in-place add / subtract and minibatch sum.  All are HBM-bound; each
// element is read once and written once.
#include <cmath>
#include <type_traits>

#include "phip_internal.h"
#include "phip_types.h"

namespace phip {

static constexpr int kBlock = 256;

static inline unsigned grid_for(size_t n, int per_thread, const phip_ctx *ctx) {
  const size_t blocks = (n + (size_t)kBlock * per_thread - 1) / ((size_t)kBlock * per_thread);
  const size_t cap = (size_t)ctx->prop.multiProcessorCount * 16;
  return (unsigned)(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

// 16 bytes of T: what one lane moves per load / store instruction.
template <typename T>
struct alignas(16) Pack16 {
  static constexpr int N = 16 / sizeof(T);
  T v[N];
};

// p[i] = value.  With VEC, p is 16-byte aligned and every lane stores 16 bytes; the last n % N elements
// are written one by one.
template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void fill_kernel(T *p, float value, size_t n) {
  const T v = from_f32<T>(value);
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x, stride = (size_t)gridDim.x * kBlock;
  if constexpr (VEC) {
    constexpr int N = Pack16<T>::N;
    Pack16<T> pack;
#pragma unroll
    for (int e = 0; e < N; ++e) pack.v[e] = v;
    const size_t packs = n / N;
    for (size_t i = first; i < packs; i += stride) reinterpret_cast<Pack16<T> *>(p)[i] = pack;
    const size_t t = packs * N + first;
    if (t < n) p[t] = v;
  } else {
    for (size_t i = first; i < n; i += stride) p[i] = v;
  }
}

template <typename S, typename D>
__global__ __launch_bounds__(kBlock) void cvt_kernel(const S *__restrict__ src, D *__restrict__ dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock) {
    dst[i] = from_f32<D>(to_f32(src[i]));
  }
}

// y[s][i] (+)= sign * x[s or 0][i] for i < volume, s < bs (grid y walks the samples; x advances only
// when it has a batch).  `accumulate` off: y's old value counts as zero and is not read.  With VEC,
// x, y and (when bs > 1) volume are multiples of 16 bytes.
template <typename T, bool VEC>
__global__ __launch_bounds__(kBlock) void add_same_kernel(const T *__restrict__ x, T *__restrict__ y, size_t volume,
                                                          uint32_t bs, size_t x_stride, float sign, bool accumulate) {
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x, stride = (size_t)gridDim.x * kBlock;
  for (uint32_t s = blockIdx.y; s < bs; s += gridDim.y) {
    const T *px = x + s * x_stride;
    T *py = y + (size_t)s * volume;
    auto one = [&](size_t i) {
      const float old = accumulate ? to_f32(py[i]) : 0.0f;
      py[i] = from_f32<T>(old + sign * to_f32(px[i]));
    };
    if constexpr (VEC) {
      constexpr int N = Pack16<T>::N;
      const size_t packs = volume / N;
      for (size_t p = first; p < packs; p += stride) {
        const Pack16<T> vx = reinterpret_cast<const Pack16<T> *>(px)[p];
        Pack16<T> vy;
        if (accumulate) vy = reinterpret_cast<const Pack16<T> *>(py)[p];
#pragma unroll
        for (int e = 0; e < N; ++e) vy.v[e] = from_f32<T>((accumulate ? to_f32(vy.v[e]) : 0.0f) + sign * to_f32(vx.v[e]));
        reinterpret_cast<Pack16<T> *>(py)[p] = vy;
      }
      const size_t t = packs * N + first;
      if (t < volume) one(t);
    } else {
      for (size_t i = first; i < volume; i += stride) one(i);
    }
  }
}

// y[i] (+)= sign * sum_n x[n][i]; one thread owns one output element, so the
// reduction needs no atomics and its order is fixed.  kAccumulate with
// `accumulate` off: y's old value counts as zero and is not read.
template <typename T, bool kAccumulate>
__global__ __launch_bounds__(kBlock) void batch_reduce_kernel(const T *__restrict__ x, T *__restrict__ y,
                                                              size_t volume, uint32_t bs, float sign,
                                                              bool accumulate = true) {
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < volume; i += (size_t)gridDim.x * kBlock) {
    float s = kAccumulate && accumulate ? to_f32(y[i]) : 0.0f;
    const T *px = x + i;
    for (uint32_t n = 0; n < bs; ++n) {
      s += sign * to_f32(*px);
      px += volume;
    }
    y[i] = from_f32<T>(s);
  }
}

template <typename T>
static constexpr int elem_code() {
  return sizeof(T) == 4 ? 0 : std::is_same<T, f16_t>::value ? 1 : 2;
}

// Launches a fill (the device is current, the arguments are checked).
template <typename T>
static int fill_now(phip_ctx *ctx, void *p, float value, size_t n) {
  // A fill is the one operation that sits between the matrix products of a backward pass (every
  // gradient is reset before products are added into it) and it names its memory as they do: it
  // takes a lane like a product instead of releasing the lanes (phip_lanes.hip).
  {
    const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
    const phip::MemRange written = {lo, lo + n * sizeof(T), true};
    const int rc = phip::lanes_place(ctx, &written, 1, n * sizeof(T) <= ((size_t)64 << 20), &ctx);
    if (rc != PHIP_OK) return rc;
  }
  if (reinterpret_cast<uintptr_t>(p) % 16 == 0) {
    hipLaunchKernelGGL((fill_kernel<T, true>), dim3(grid_for(n / Pack16<T>::N + Pack16<T>::N, 2, ctx)), dim3(kBlock), 0,
                       ctx->stream, static_cast<T *>(p), value, n);
  } else {
    hipLaunchKernelGGL((fill_kernel<T, false>), dim3(grid_for(n, 4, ctx)), dim3(kBlock), 0, ctx->stream,
                       static_cast<T *>(p), value, n);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// At most this many zero fills are noted at a time (a backward step of primitiv's graph resets one
// or two gradients and then calls the operator that adds into them).
static constexpr size_t kMaxNotedZeros = 8;

template <typename T>
static int fill_impl(phip_ctx *ctx, void *p, float value, size_t n) {
  PHIP_ENTER_HOST(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(p != nullptr, "null pointer");
  const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
  const size_t bytes = n * sizeof(T);
  {
    // a fill replaces every noted fill that it covers; one that it only overlaps is launched first
    bool overlap_left = false;
    {
      std::lock_guard<std::mutex> lock(ctx->mutex);
      size_t kept = 0;
      for (const PendingZero &z : ctx->zeros) {
        const bool covered = z.lo >= lo && z.lo + z.bytes <= lo + bytes;
        if (!covered && z.lo < lo + bytes && lo < z.lo + z.bytes) overlap_left = true;
        if (!covered) ctx->zeros[kept++] = z;
      }
      ctx->zeros.resize(kept);
      ctx->zeros_count.store((int)kept, std::memory_order_relaxed);
    }
    if (overlap_left) PHIP_FLUSH_ZEROS(ctx);
  }
  if (value == 0.0f && !std::signbit(value) && ctx->defer_zero_fills && !ctx->fixed_mode) {
    bool full;
    {
      std::lock_guard<std::mutex> lock(ctx->mutex);
      full = ctx->zeros.size() >= kMaxNotedZeros;
    }
    if (full) PHIP_FLUSH_ZEROS(ctx);
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->zeros.push_back(PendingZero{lo, bytes, elem_code<T>()});
    ctx->zeros_count.store((int)ctx->zeros.size(), std::memory_order_relaxed);
    return PHIP_OK;
  }
  return fill_now<T>(ctx, p, value, n);
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
  PHIP_ENTER_KEEP_ZEROS(ctx);
  PHIP_REQUIRE(bx >= 1 && by >= 1 && (bx == by || bx == 1 || by == 1),
               "incompatible batch sizes: %u, %u", bx, by);
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  // y noted as zero and not yet filled: write instead of add
  const size_t ybytes = (size_t)volume * by * sizeof(T);
  const bool accumulate = shares_memory(y, ybytes, x, (size_t)volume * bx * sizeof(T)) || !zeros_take(ctx, y, ybytes);
  PHIP_FLUSH_ZEROS(ctx);
  if (by == 1 && bx > 1) {
    hipLaunchKernelGGL((batch_reduce_kernel<T, true>), dim3(grid_for(volume, 1, ctx)), dim3(kBlock), 0,
                       ctx->stream, static_cast<const T *>(x), static_cast<T *>(y), (size_t)volume, bx, sign, accumulate);
  } else {
    // same batch on both sides: one long sample; a shared x is re-read per sample of y
    size_t vol = volume;
    uint32_t bs = by;
    size_t x_stride = 0;
    if (bx == by) {
      vol *= by;
      bs = 1;
    }
    constexpr int N = Pack16<T>::N;
    // 16-byte packs pay for 16-bit elements (64 Mi of them: 67 -> 60 us); with fp32 the same loop runs 3 - 5 %
    // slower than 4 bytes per lane (167 against 160 us, 8-byte packs 164), so fp32 keeps the narrow form
    const bool vec = sizeof(T) == 2 && reinterpret_cast<uintptr_t>(x) % 16 == 0 &&
                     reinterpret_cast<uintptr_t>(y) % 16 == 0 && (bs == 1 || vol % N == 0);
    const unsigned gx = grid_for(vec ? vol / N + N : vol, vec ? 2 : 4, ctx);
    const unsigned cap = (unsigned)ctx->prop.multiProcessorCount * 16;
    unsigned gy = gx >= cap ? 1 : cap / gx;
    if (gy > bs) gy = bs;
    if (gy > 65535u) gy = 65535u;
    if (vec) {
      hipLaunchKernelGGL((add_same_kernel<T, true>), dim3(gx, gy), dim3(kBlock), 0, ctx->stream, static_cast<const T *>(x),
                         static_cast<T *>(y), vol, bs, x_stride, sign, accumulate);
    } else {
      hipLaunchKernelGGL((add_same_kernel<T, false>), dim3(gx, gy), dim3(kBlock), 0, ctx->stream,
                         static_cast<const T *>(x), static_cast<T *>(y), vol, bs, x_stride, sign, accumulate);
    }
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// Launches every noted zero fill, in the order they were asked for.
int zeros_flush(phip_ctx *ctx) {
  PendingZero list[kMaxNotedZeros + 1];
  size_t n = 0;
  {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    for (const PendingZero &z : ctx->zeros) {
      if (n < kMaxNotedZeros + 1) list[n++] = z;
    }
    ctx->zeros.clear();
    ctx->zeros_count.store(0, std::memory_order_relaxed);
  }
  for (size_t i = 0; i < n; ++i) {
    void *p = reinterpret_cast<void *>(list[i].lo);
    int rc;
    if (list[i].elem == 0) rc = fill_now<float>(ctx, p, 0.0f, list[i].bytes / 4);
    else if (list[i].elem == 1) rc = fill_now<f16_t>(ctx, p, 0.0f, list[i].bytes / 2);
    else rc = fill_now<bf16_t>(ctx, p, 0.0f, list[i].bytes / 2);
    if (rc != PHIP_OK) return rc;
  }
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
