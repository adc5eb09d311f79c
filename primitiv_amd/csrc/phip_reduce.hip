// Reductions along one dimension of a tensor seen as [outer][n][base]:
// sum, logsumexp, max, min, the gradient of max / min, and argmax / argmin.
//
// Two launch shapes.  "Column": one thread per output element walks the n
// inputs in order; neighbouring threads read neighbouring addresses when
// base > 1, and a thread reads a contiguous run when base == 1.  "Block":
// one 256-thread workgroup per output element, for long reductions with few
// outputs; the threads' partial results are combined through LDS by a tree of
// fixed shape.  Either way a result does not depend on scheduling.
#include <vector>

#include "phip_pointwise.h"

namespace phip {
namespace {

using namespace pointwise;

constexpr float kInf = __builtin_huge_valf();

// ---- combiners ----------------------------------------------------------------
// State of a partial reduction, how one input enters it, how two states merge,
// and the final value.

struct SumOp {
  struct State { float s; };
  __device__ static State init() { return {0.f}; }
  __device__ static void push(State &a, float v, uint32_t) { a.s += v; }
  __device__ static void merge(State &a, const State &b) { a.s += b.s; }
  __device__ static float result(const State &a) { return a.s; }
};

// log(sum(exp(v))) kept as (m, s) with sum = s * exp(m), m the largest input so far.
struct LogSumExpOp {
  struct State { float m, s; };
  __device__ static State init() { return {-kInf, 0.f}; }
  __device__ static void push(State &a, float v, uint32_t) {
    if (v > a.m) {
      a.s = a.s * expf(a.m - v) + 1.f;
      a.m = v;
    } else {
      a.s += expf(v - a.m);
    }
  }
  __device__ static void merge(State &a, const State &b) {
    if (b.m > a.m) {
      a.s = a.s * expf(a.m - b.m) + b.s;
      a.m = b.m;
    } else if (b.m > -kInf) {
      a.s += b.s * expf(b.m - a.m);
    }
  }
  __device__ static float result(const State &a) { return a.m + logf(a.s); }
};

// Extremum with the first index that attains it.  SIGN = +1: max, -1: min.
template <int SIGN>
struct ExtremumOp {
  struct State { float v; uint32_t j; };
  __device__ static State init() { return {-kInf, 0xffffffffu}; }
  __device__ static void push(State &a, float v, uint32_t j) {
    const float w = SIGN > 0 ? v : -v;
    if (w > a.v || (w == a.v && j < a.j)) {
      a.v = w;
      a.j = j;
    }
  }
  __device__ static void merge(State &a, const State &b) { push_state(a, b); }
  __device__ static void push_state(State &a, const State &b) {
    if (b.v > a.v || (b.v == a.v && b.j < a.j)) a = b;
  }
  __device__ static float result(const State &a) { return SIGN > 0 ? a.v : -a.v; }
};

// What a launch writes per output element.
enum class Emit { Value, Index, Gradient };

template <typename T, typename OP, Emit EMIT>
__device__ inline void emit(const typename OP::State &st, T *y, uint32_t *index_out, const T *gy, T *gx,
                            size_t out, size_t first_in, uint32_t base, uint32_t n) {
  if constexpr (EMIT == Emit::Value) {
    y[out] = from_f32<T>(OP::result(st));
  } else if constexpr (EMIT == Emit::Index) {
    index_out[out] = st.j < n ? st.j : 0;   // no input compared (all NaN): index 0, as the reference
  } else {
    if (st.j < n) {                         // all NaN: nothing equals the extremum, nothing is added
      T *g = gx + first_in + (size_t)st.j * base;
      *g = from_f32<T>(to_f32(*g) + to_f32(gy[out]));
    }
  }
}

// One thread per output element q = o*base + i.
template <typename T, typename OP, Emit EMIT>
__global__ __launch_bounds__(kBlock) void reduce_column_kernel(const T *x, T *y, uint32_t *index_out, const T *gy,
                                                                T *gx, uint32_t base, uint32_t n, size_t outputs) {
  for (size_t q = (size_t)blockIdx.x * kBlock + threadIdx.x; q < outputs; q += (size_t)gridDim.x * kBlock) {
    const size_t o = q / base;
    const size_t first = o * n * base + (q - o * base);
    typename OP::State st = OP::init();
    const T *p = x + first;
    for (uint32_t j = 0; j < n; ++j) OP::push(st, to_f32(p[(size_t)j * base]), j);
    emit<T, OP, EMIT>(st, y, index_out, gy, gx, q, first, base, n);
  }
}

// One workgroup per output element; thread t takes j = t, t + 256, ...
template <typename T, typename OP, Emit EMIT>
__global__ __launch_bounds__(kBlock) void reduce_block_kernel(const T *x, T *y, uint32_t *index_out, const T *gy,
                                                               T *gx, uint32_t base, uint32_t n, size_t outputs) {
  __shared__ typename OP::State part[kBlock];
  for (size_t q = blockIdx.x; q < outputs; q += gridDim.x) {
    const size_t o = q / base;
    const size_t first = o * n * base + (q - o * base);
    typename OP::State st = OP::init();
    const T *p = x + first;
    for (uint32_t j = threadIdx.x; j < n; j += kBlock) OP::push(st, to_f32(p[(size_t)j * base]), j);
    part[threadIdx.x] = st;
    __syncthreads();
    for (int w = kBlock / 2; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) OP::merge(part[threadIdx.x], part[threadIdx.x + w]);
      __syncthreads();
    }
    if (threadIdx.x == 0) emit<T, OP, EMIT>(part[0], y, index_out, gy, gx, q, first, base, n);
    __syncthreads();
  }
}

template <typename T, typename OP, Emit EMIT>
int launch_reduce(phip_ctx *ctx, const T *x, T *y, uint32_t *index_out, const T *gy, T *gx, uint32_t base,
                  uint32_t n, uint32_t outer) {
  const size_t outputs = (size_t)base * outer;
  const size_t cus = (size_t)ctx->prop.multiProcessorCount;
  const bool by_block = n >= 64 && (base == 1 || outputs < 16 * cus) && outputs < 64 * cus;
  if (by_block) {
    hipLaunchKernelGGL((reduce_block_kernel<T, OP, EMIT>), dim3((unsigned)outputs), dim3(kBlock), 0, ctx->stream, x,
                       y, index_out, gy, gx, base, n, outputs);
  } else {
    hipLaunchKernelGGL((reduce_column_kernel<T, OP, EMIT>), dim3(blocks_for(outputs, ctx)), dim3(kBlock), 0,
                       ctx->stream, x, y, index_out, gy, gx, base, n, outputs);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
int reduce_fw(phip_ctx *ctx, int op, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(op >= PHIP_SUM && op <= PHIP_MIN, "unknown reduction %d", op);
  if (base == 0 || outer == 0) return PHIP_OK;
  PHIP_REQUIRE(n > 0, "cannot reduce over an empty dimension");
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  const T *px = static_cast<const T *>(x);
  T *py = static_cast<T *>(y);
  switch (op) {
    case PHIP_SUM: return launch_reduce<T, SumOp, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
    case PHIP_LOGSUMEXP:
      return launch_reduce<T, LogSumExpOp, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
    case PHIP_MAX:
      return launch_reduce<T, ExtremumOp<1>, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
    default:
      return launch_reduce<T, ExtremumOp<-1>, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
  }
}

// The position of the extremum is found again from x (the first j attaining
// it, which is also the first j whose value equals the forward result).
template <typename T>
int extremum_bw(phip_ctx *ctx, int op, const void *x, const void *gy, void *gx, uint32_t base, uint32_t n,
                uint32_t outer) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(op == PHIP_MAX || op == PHIP_MIN, "operation %d has no such gradient", op);
  if (base == 0 || outer == 0) return PHIP_OK;
  PHIP_REQUIRE(n > 0, "cannot reduce over an empty dimension");
  PHIP_REQUIRE(x != nullptr && gy != nullptr && gx != nullptr, "null pointer");
  const T *px = static_cast<const T *>(x);
  const T *pgy = static_cast<const T *>(gy);
  T *pgx = static_cast<T *>(gx);
  if (op == PHIP_MAX)
    return launch_reduce<T, ExtremumOp<1>, Emit::Gradient>(ctx, px, nullptr, nullptr, pgy, pgx, base, n, outer);
  return launch_reduce<T, ExtremumOp<-1>, Emit::Gradient>(ctx, px, nullptr, nullptr, pgy, pgx, base, n, outer);
}

template <typename T>
int arg_extremum(phip_ctx *ctx, int op, const void *x, uint32_t *host_out, uint32_t base, uint32_t n,
                 uint32_t outer) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(op == PHIP_MAX || op == PHIP_MIN, "operation %d has no index form", op);
  if (base == 0 || outer == 0) return PHIP_OK;
  PHIP_REQUIRE(n > 0, "cannot reduce over an empty dimension");
  PHIP_REQUIRE(x != nullptr && host_out != nullptr, "null pointer");
  const size_t bytes = sizeof(uint32_t) * (size_t)base * outer;
  void *block = nullptr;
  int rc = phip_pool_alloc(ctx, bytes, &block, nullptr);
  if (rc != PHIP_OK) return rc;
  const T *px = static_cast<const T *>(x);
  uint32_t *idx = static_cast<uint32_t *>(block);
  rc = op == PHIP_MAX
           ? launch_reduce<T, ExtremumOp<1>, Emit::Index>(ctx, px, nullptr, idx, nullptr, nullptr, base, n, outer)
           : launch_reduce<T, ExtremumOp<-1>, Emit::Index>(ctx, px, nullptr, idx, nullptr, nullptr, base, n, outer);
  if (rc == PHIP_OK) rc = phip_memcpy_d2h(ctx, host_out, block, bytes);
  phip_pool_free(ctx, block);
  return rc;
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_REDUCE(SUF, T, CPTR, PTR)                                                                  \
  int phip_reduce_fw_##SUF(phip_ctx *ctx, int op, CPTR x, PTR y, uint32_t base, uint32_t n, uint32_t outer) {  \
    return reduce_fw<T>(ctx, op, x, y, base, n, outer);                                                        \
  }                                                                                                            \
  int phip_extremum_bw_##SUF(phip_ctx *ctx, int op, CPTR x, CPTR y, CPTR gy, PTR gx, uint32_t base,            \
                             uint32_t n, uint32_t outer) {                                                     \
    (void)y;                                                                                                   \
    return extremum_bw<T>(ctx, op, x, gy, gx, base, n, outer);                                                 \
  }                                                                                                            \
  int phip_arg_extremum_##SUF(phip_ctx *ctx, int op, CPTR x, uint32_t *host_out, uint32_t base, uint32_t n,    \
                              uint32_t outer) {                                                                \
    return arg_extremum<T>(ctx, op, x, host_out, base, n, outer);                                              \
  }

PHIP_EXPORT_REDUCE(f32, float, const float *, float *)
PHIP_EXPORT_REDUCE(f16, f16_t, const void *, void *)
PHIP_EXPORT_REDUCE(bf16, bf16_t, const void *, void *)

#undef PHIP_EXPORT_REDUCE

}  // extern "C"
