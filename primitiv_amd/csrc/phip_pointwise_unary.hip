// One-operand elementwise families: y = f(x), y = f(x, k) with a host constant
// (float or integer), their gradients gx += f'(x, y) * gy, and the in-place
// scaling x *= k.  Each kernel streams its operands once with 16-byte
// accesses per lane (4 fp32 or 8 16-bit values) and computes in fp32; a
// backward kernel loads only those of x and y that its formula uses.
#include "phip_pointwise.h"

namespace phip {
namespace {

using namespace pointwise;

// ---- formulas ---------------------------------------------------------------
// fw(x) is the forward value; bw(x, y, gy) the amount added to gx.  kX / kY
// say whether bw reads x / y.

struct Negate {
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return -x; }
  __device__ float bw(float, float, float gy) const { return -gy; }
};
struct Abs {
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return fabsf(x); }
  __device__ float bw(float x, float, float gy) const { return (float)((x > 0.f) - (x < 0.f)) * gy; }
};
struct Sqrt {
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return sqrtf(x); }
  __device__ float bw(float, float y, float gy) const { return .5f * gy / y; }
};
struct Exp {
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return expf(x); }
  __device__ float bw(float, float y, float gy) const { return y * gy; }
};
struct Log {
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return logf(x); }
  __device__ float bw(float x, float, float gy) const { return gy / x; }
};
struct Tanh {
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return tanhf(x); }
  __device__ float bw(float, float y, float gy) const { return (1.f - y * y) * gy; }
};
struct Sigmoid {
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return .5f + .5f * tanhf(.5f * x); }
  __device__ float bw(float, float y, float gy) const { return y * (1.f - y) * gy; }
};
struct Softplus {
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return fmaxf(x, 0.f) + logf(1.f + expf(-fabsf(x))); }
  __device__ float bw(float x, float, float gy) const { return (.5f + .5f * tanhf(.5f * x)) * gy; }
};
struct Sin {
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return sinf(x); }
  __device__ float bw(float x, float, float gy) const { return cosf(x) * gy; }
};
struct Cos {
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return cosf(x); }
  __device__ float bw(float x, float, float gy) const { return -sinf(x) * gy; }
};
struct Tan {
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return tanf(x); }
  __device__ float bw(float, float y, float gy) const { return (1.f + y * y) * gy; }
};

struct AddConst {
  float k;
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return x + k; }
  __device__ float bw(float, float, float gy) const { return gy; }
};
struct SubtractConstR {
  float k;
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return x - k; }
  __device__ float bw(float, float, float gy) const { return gy; }
};
struct SubtractConstL {
  float k;
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return k - x; }
  __device__ float bw(float, float, float gy) const { return -gy; }
};
struct MultiplyConst {
  float k;
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return x * k; }
  __device__ float bw(float, float, float gy) const { return k * gy; }
};
struct DivideConstR {
  float k;
  static constexpr bool kX = false, kY = false;
  __device__ float fw(float x) const { return x / k; }
  __device__ float bw(float, float, float gy) const { return gy / k; }
};
struct DivideConstL {
  float k;
  static constexpr bool kX = true, kY = true;
  __device__ float fw(float x) const { return k / x; }
  __device__ float bw(float x, float y, float gy) const { return -y * gy / x; }
};
struct PowConstR {
  float k;
  static constexpr bool kX = true, kY = true;
  __device__ float fw(float x) const { return powf(x, k); }
  __device__ float bw(float x, float y, float gy) const { return k * gy * y / x; }
};
struct PowConstL {
  float k;
  static constexpr bool kX = false, kY = true;
  __device__ float fw(float x) const { return powf(k, x); }
  __device__ float bw(float, float y, float gy) const { return logf(k) * gy * y; }
};
struct PRelu {
  float k;
  static constexpr bool kX = true, kY = false;
  __device__ float fw(float x) const { return fmaxf(x, 0.f) + k * fminf(x, 0.f); }
  __device__ float bw(float x, float, float gy) const { return gy * ((float)(x > 0.f) + k * (float)(x <= 0.f)); }
};
struct Elu {
  float k;
  static constexpr bool kX = true, kY = true;
  __device__ float fw(float x) const { return fmaxf(x, 0.f) + k * (expf(fminf(x, 0.f)) - 1.f); }
  __device__ float bw(float x, float y, float gy) const {
    return gy * ((float)(x > 0.f) + (y + k) * (float)(x <= 0.f));
  }
};
// x ^ k by repeated squaring; |k| is taken in unsigned arithmetic so that the
// most negative k is handled.
struct Pown {
  int32_t k;
  static constexpr bool kX = true, kY = true;
  __device__ float fw(float x) const {
    uint32_t remain = k < 0 ? 0u - (uint32_t)k : (uint32_t)k;
    float ret = 1.f, factor = x;
    while (remain) {
      if (remain & 1u) ret *= factor;
      factor *= factor;
      remain >>= 1;
    }
    return k >= 0 ? ret : 1.f / ret;
  }
  __device__ float bw(float x, float y, float gy) const { return (float)k * gy * y / x; }
};

// ---- kernels ----------------------------------------------------------------

// y[i] = f.fw(x[i]).  x and y may be the same array.
template <typename T, typename F, bool VEC>
__global__ __launch_bounds__(kBlock) void map_fw_kernel(const F f, const T *x, T *y, size_t n) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  if constexpr (VEC) {
    constexpr int N = Pack<T>::N;
    const size_t packs = n / N;
    for (size_t p = first; p < packs; p += stride) {
      const Pack<T> in = load_pack(x + p * N);
      Pack<T> out;
#pragma unroll
      for (int e = 0; e < N; ++e) out.v[e] = from_f32<T>(f.fw(to_f32(in.v[e])));
      store_pack(y + p * N, out);
    }
    const size_t t = packs * N + first;  // the last n % N elements
    if (t < n) y[t] = from_f32<T>(f.fw(to_f32(x[t])));
  } else {
    for (size_t i = first; i < n; i += stride) y[i] = from_f32<T>(f.fw(to_f32(x[i])));
  }
}

// gx[i] += f.bw(x[i], y[i], gy[i]).  `accumulate` off: gx's old value counts as zero and is not read.
template <typename T, typename F, bool VEC>
__global__ __launch_bounds__(kBlock) void map_bw_kernel(const F f, const T *x, const T *y, const T *gy, T *gx,
                                                         size_t n, bool accumulate) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  auto one = [&](size_t i) {
    const float xv = F::kX ? to_f32(x[i]) : 0.f;
    const float yv = F::kY ? to_f32(y[i]) : 0.f;
    gx[i] = from_f32<T>((accumulate ? to_f32(gx[i]) : 0.f) + f.bw(xv, yv, to_f32(gy[i])));
  };
  if constexpr (VEC) {
    constexpr int N = Pack<T>::N;
    const size_t packs = n / N;
    for (size_t p = first; p < packs; p += stride) {
      Pack<T> px, py;
      if constexpr (F::kX) px = load_pack(x + p * N);
      if constexpr (F::kY) py = load_pack(y + p * N);
      const Pack<T> pg = load_pack(gy + p * N);
      Pack<T> acc;
      if (accumulate) acc = load_pack(gx + p * N);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        float xv = 0.f, yv = 0.f;
        if constexpr (F::kX) xv = to_f32(px.v[e]);
        if constexpr (F::kY) yv = to_f32(py.v[e]);
        acc.v[e] = from_f32<T>((accumulate ? to_f32(acc.v[e]) : 0.f) + f.bw(xv, yv, to_f32(pg.v[e])));
      }
      store_pack(gx + p * N, acc);
    }
    const size_t t = packs * N + first;
    if (t < n) one(t);
  } else {
    for (size_t i = first; i < n; i += stride) one(i);
  }
}

// y[i] = (i is on the diagonal of a rows x rows matrix)
template <typename T>
__global__ __launch_bounds__(kBlock) void identity_kernel(T *y, uint32_t rows, size_t n) {
  const T one = from_f32<T>(1.f), zero = from_f32<T>(0.f);
  for (size_t i = (size_t)blockIdx.x * kBlock + threadIdx.x; i < n; i += (size_t)gridDim.x * kBlock)
    y[i] = (i % ((size_t)rows + 1)) == 0 ? one : zero;
}

// ---- launchers --------------------------------------------------------------

template <typename T, typename F>
int launch_fw(phip_ctx *ctx, const F &f, const void *x, void *y, size_t n) {
  PHIP_ENTER(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  const T *px = static_cast<const T *>(x);
  T *py = static_cast<T *>(y);
  if (aligned16(x) && aligned16(y)) {
    hipLaunchKernelGGL((map_fw_kernel<T, F, true>), dim3(blocks_for(n / Pack<T>::N + Pack<T>::N, ctx)),
                       dim3(kBlock), 0, ctx->stream, f, px, py, n);
  } else {
    hipLaunchKernelGGL((map_fw_kernel<T, F, false>), dim3(blocks_for(n, ctx)), dim3(kBlock), 0, ctx->stream, f,
                       px, py, n);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T, typename F>
int launch_bw(phip_ctx *ctx, const F &f, const void *x, const void *y, const void *gy, void *gx, size_t n) {
  PHIP_ENTER_KEEP_ZEROS(ctx);
  if (n == 0) return PHIP_OK;
  PHIP_REQUIRE(gy != nullptr && gx != nullptr, "null pointer");
  PHIP_REQUIRE(!F::kX || x != nullptr, "this gradient needs x");
  PHIP_REQUIRE(!F::kY || y != nullptr, "this gradient needs y");
  // gx noted as zero and not yet filled: write instead of add
  const size_t bytes = n * sizeof(T);
  const bool read_too = shares_memory(gx, bytes, gy, bytes) || (F::kX && shares_memory(gx, bytes, x, bytes)) ||
                        (F::kY && shares_memory(gx, bytes, y, bytes));
  const bool accumulate = read_too || !zeros_take(ctx, gx, bytes);
  PHIP_FLUSH_ZEROS(ctx);
  const T *px = static_cast<const T *>(x);
  const T *py = static_cast<const T *>(y);
  const T *pgy = static_cast<const T *>(gy);
  T *pgx = static_cast<T *>(gx);
  const bool vec = aligned16(gy) && aligned16(gx) && (!F::kX || aligned16(x)) && (!F::kY || aligned16(y));
  if (vec) {
    hipLaunchKernelGGL((map_bw_kernel<T, F, true>), dim3(blocks_for(n / Pack<T>::N + Pack<T>::N, ctx)),
                       dim3(kBlock), 0, ctx->stream, f, px, py, pgy, pgx, n, accumulate);
  } else {
    hipLaunchKernelGGL((map_bw_kernel<T, F, false>), dim3(blocks_for(n, ctx)), dim3(kBlock), 0, ctx->stream, f,
                       px, py, pgy, pgx, n, accumulate);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// Calls `call(formula)` for the formula an operation code names.
template <typename Call>
int with_unary(int op, bool backward, Call &&call) {
  switch (op) {
    case PHIP_NEGATE:
      if (backward) return fail(PHIP_ERR_INVALID_ARGUMENT, "negate has no backward operation");
      return call(Negate{});
    case PHIP_ABS: return call(Abs{});
    case PHIP_SQRT: return call(Sqrt{});
    case PHIP_EXP: return call(Exp{});
    case PHIP_LOG: return call(Log{});
    case PHIP_TANH: return call(Tanh{});
    case PHIP_SIGMOID: return call(Sigmoid{});
    case PHIP_SOFTPLUS: return call(Softplus{});
    case PHIP_SIN: return call(Sin{});
    case PHIP_COS: return call(Cos{});
    case PHIP_TAN: return call(Tan{});
    default: return fail(PHIP_ERR_INVALID_ARGUMENT, "unknown unary operation %d", op);
  }
}

template <typename Call>
int with_const(int op, float k, Call &&call) {
  switch (op) {
    case PHIP_ADD_CONST: return call(AddConst{k});
    case PHIP_SUBTRACT_CONST_R: return call(SubtractConstR{k});
    case PHIP_SUBTRACT_CONST_L: return call(SubtractConstL{k});
    case PHIP_MULTIPLY_CONST: return call(MultiplyConst{k});
    case PHIP_DIVIDE_CONST_R: return call(DivideConstR{k});
    case PHIP_DIVIDE_CONST_L: return call(DivideConstL{k});
    case PHIP_POW_CONST_R: return call(PowConstR{k});
    case PHIP_POW_CONST_L: return call(PowConstL{k});
    case PHIP_PRELU: return call(PRelu{k});
    case PHIP_ELU: return call(Elu{k});
    default: return fail(PHIP_ERR_INVALID_ARGUMENT, "unknown constant operation %d", op);
  }
}

template <typename T>
int unary_fw(phip_ctx *ctx, int op, const void *x, void *y, size_t n) {
  return with_unary(op, false, [&](auto f) { return launch_fw<T>(ctx, f, x, y, n); });
}
template <typename T>
int unary_bw(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx, size_t n) {
  return with_unary(op, true, [&](auto f) { return launch_bw<T>(ctx, f, x, y, gy, gx, n); });
}
template <typename T>
int const_fw(phip_ctx *ctx, int op, const void *x, float k, void *y, size_t n) {
  return with_const(op, k, [&](auto f) { return launch_fw<T>(ctx, f, x, y, n); });
}
template <typename T>
int const_bw(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, float k, void *gx, size_t n) {
  return with_const(op, k, [&](auto f) { return launch_bw<T>(ctx, f, x, y, gy, gx, n); });
}

template <typename T>
int identity(phip_ctx *ctx, void *y, uint32_t rows) {
  PHIP_ENTER(ctx);
  if (rows == 0) return PHIP_OK;
  PHIP_REQUIRE(y != nullptr, "null pointer");
  const size_t n = (size_t)rows * rows;
  hipLaunchKernelGGL(identity_kernel<T>, dim3(blocks_for(n, ctx)), dim3(kBlock), 0, ctx->stream,
                     static_cast<T *>(y), rows, n);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_UNARY(SUF, T, CPTR, PTR)                                                                      \
  int phip_unary_fw_##SUF(phip_ctx *ctx, int op, CPTR x, PTR y, size_t n) { return unary_fw<T>(ctx, op, x, y, n); } \
  int phip_unary_bw_##SUF(phip_ctx *ctx, int op, CPTR x, CPTR y, CPTR gy, PTR gx, size_t n) {                     \
    return unary_bw<T>(ctx, op, x, y, gy, gx, n);                                                                 \
  }                                                                                                               \
  int phip_const_fw_##SUF(phip_ctx *ctx, int op, CPTR x, float k, PTR y, size_t n) {                              \
    return const_fw<T>(ctx, op, x, k, y, n);                                                                      \
  }                                                                                                               \
  int phip_const_bw_##SUF(phip_ctx *ctx, int op, CPTR x, CPTR y, CPTR gy, float k, PTR gx, size_t n) {            \
    return const_bw<T>(ctx, op, x, y, gy, k, gx, n);                                                              \
  }                                                                                                               \
  int phip_pown_fw_##SUF(phip_ctx *ctx, CPTR x, int32_t k, PTR y, size_t n) {                                     \
    return launch_fw<T>(ctx, Pown{k}, x, y, n);                                                                   \
  }                                                                                                               \
  int phip_pown_bw_##SUF(phip_ctx *ctx, CPTR x, CPTR y, CPTR gy, int32_t k, PTR gx, size_t n) {                   \
    return launch_bw<T>(ctx, Pown{k}, x, y, gy, gx, n);                                                           \
  }                                                                                                               \
  int phip_inplace_multiply_const_##SUF(phip_ctx *ctx, float k, PTR x, size_t n) {                                \
    return launch_fw<T>(ctx, MultiplyConst{k}, x, x, n);                                                          \
  }                                                                                                               \
  int phip_identity_##SUF(phip_ctx *ctx, PTR y, uint32_t rows) { return identity<T>(ctx, y, rows); }

PHIP_EXPORT_UNARY(f32, float, const float *, float *)
PHIP_EXPORT_UNARY(f16, f16_t, const void *, void *)
PHIP_EXPORT_UNARY(bf16, bf16_t, const void *, void *)

#undef PHIP_EXPORT_UNARY

}  // extern "C"
