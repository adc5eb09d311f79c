// Reductions along one dimension of a tensor seen as [outer][n][base]:
// sum, logsumexp, max, min, the gradient of max / min, and argmax / argmin.
//
// Four launch shapes, all built on one combiner interface (state, push, merge):
//  * "rows"   (base == 1, n >= 32): a wavefront per output; its lanes stride
//    along the contiguous n axis (256 bytes per load instruction), four
//    independent partial states per lane keep four loads in flight, then the
//    lanes combine by a butterfly of fixed shape.
//  * "tiles"  (base >= 16): a workgroup is TX lanes along base (contiguous) by
//    TY lanes that split n; four partial states per thread, then the TY
//    partials combine through LDS in order.
//  * "block"  (few outputs, long n): one 256-thread workgroup per output with
//    an LDS tree of fixed shape.
// When "tiles" or "block" would start too few workgroups to fill the chip, n is
// cut into ranges reduced independently into partial states, which a second
// small launch merges in order.
//  * "column" (everything else, i.e. short reductions): one thread per output.
// A result never depends on scheduling; no atomics are used.
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

// Extremum alone, for a launch that writes values: the same comparisons as
// ExtremumOp (a NaN never enters, the first of equal values stays) without the
// index, at a third of the instructions per element and half the state.  (Of a
// +0 and a -0, which compare equal, the one returned need not be the first.)
template <int SIGN>
struct ExtremumValueOp {
  struct State { float v; };
  __device__ static State init() { return {-kInf}; }
  __device__ static void push(State &a, float v, uint32_t) {
    const float w = SIGN > 0 ? v : -v;
    a.v = w > a.v ? w : a.v;
  }
  __device__ static void merge(State &a, const State &b) { a.v = b.v > a.v ? b.v : a.v; }
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

// U independent partial states over j = first, first + step, ... < end: the
// loads of U consecutive steps are in flight together; the partials merge in a
// fixed order.
template <typename T, typename OP, int U = 4>
__device__ inline typename OP::State walk(const T *p, size_t stride_elems, uint32_t first, uint32_t step,
                                          uint32_t end) {
  typename OP::State st[U];
#pragma unroll
  for (int u = 0; u < U; ++u) st[u] = OP::init();
  uint32_t j = first;
  for (; j < end && end - j > (U - 1) * step; j += U * step) {
    float v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = to_f32(p[(size_t)(j + u * step) * stride_elems]);
#pragma unroll
    for (int u = 0; u < U; ++u) OP::push(st[u], v[u], j + u * step);
  }
#pragma unroll
  for (int u = 0; u < U - 1; ++u) {
    if (j < end) OP::push(st[u], to_f32(p[(size_t)j * stride_elems]), j);
    j += step;
  }
#pragma unroll
  for (int w = 1; w < U; w *= 2) {
#pragma unroll
    for (int u = 0; u + w < U; u += 2 * w) OP::merge(st[u], st[u + w]);
  }
  return st[0];
}

// A contiguous run of n elements (n a multiple of V, p aligned to V elements)
// taken V elements per access: lane `first` of `step` takes packs first,
// first + step, ...; U packs are in flight together.
template <typename T, typename OP, int V, int U = 4>
__device__ inline typename OP::State walk_packs(const T *p, uint32_t first, uint32_t step, uint32_t n) {
  struct alignas(V * sizeof(T)) Pack {
    T c[V];
  };
  const Pack *q = reinterpret_cast<const Pack *>(p);
  const uint32_t end = n / V;
  typename OP::State st[U];
#pragma unroll
  for (int u = 0; u < U; ++u) st[u] = OP::init();
  uint32_t j = first;
  for (; j < end && end - j > (U - 1) * step; j += U * step) {
    Pack v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = q[j + u * step];
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < V; ++k) OP::push(st[u], to_f32(v[u].c[k]), (j + u * step) * V + k);
  }
#pragma unroll
  for (int u = 0; u < U - 1; ++u) {
    if (j < end) {
      const Pack v = q[j];
#pragma unroll
      for (int k = 0; k < V; ++k) OP::push(st[u], to_f32(v.c[k]), j * V + k);
    }
    j += step;
  }
#pragma unroll
  for (int w = 1; w < U; w *= 2) {
#pragma unroll
    for (int u = 0; u + w < U; u += 2 * w) OP::merge(st[u], st[u + w]);
  }
  return st[0];
}

// A long reduction may be cut into `splits` ranges of `chunk` positions, each
// reduced by its own workgroup into partial[(o*splits + sp)*base + i]. The
// workgroup that finishes last of a group's ranges (a counter per group tells)
// merges them in order and writes the results.  splits == 1 writes the result
// directly.
struct Split {
  uint32_t splits, chunk;
  uint32_t *tickets;   // splits > 1: one zeroed counter per group of outputs, left zeroed
};

// Partial states travel between workgroups, which may sit on different L2s:
// device-scope accesses, word by word, go past those caches.
template <typename State>
__device__ inline void store_state(State *p, const State &st) {
  uint32_t w[sizeof(State) / 4];
  __builtin_memcpy(w, &st, sizeof(State));
#pragma unroll
  for (unsigned k = 0; k < sizeof(State) / 4; ++k)
    __hip_atomic_store(reinterpret_cast<uint32_t *>(p) + k, w[k], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename State>
__device__ inline State load_state(const State *p) {
  uint32_t w[sizeof(State) / 4];
#pragma unroll
  for (unsigned k = 0; k < sizeof(State) / 4; ++k)
    w[k] = __hip_atomic_load(reinterpret_cast<const uint32_t *>(p) + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  State st;
  __builtin_memcpy(&st, w, sizeof(State));
  return st;
}

// Called by all threads of a workgroup after its partial states were stored:
// true in the workgroup that is the last of the group's `splits` to get here.
// Each lane waits until memory has acknowledged its own stores, the barrier puts
// all of them before thread 0's ticket, and the ticket is a device-scope atomic
// on one address, so the one who draws the last ticket does so after every other
// workgroup's stores arrived. The counter is left zeroed for the next launch.
__device__ inline bool last_of_group(uint32_t *ticket, uint32_t splits, uint32_t *flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t drawn = __hip_atomic_fetch_add(ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = drawn == splits - 1u;
    if (last) __hip_atomic_store(ticket, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  return *flag != 0;
}

// The ranges of one output merged in order.
template <typename T, typename OP, Emit EMIT>
__device__ inline void merge_ranges(const typename OP::State *partial, uint32_t splits, T *y, uint32_t *index_out,
                                    const T *gy, T *gx, size_t o, uint32_t i, uint32_t base, uint32_t n) {
  // eight loads in flight at a time: one after the other they would cost a trip to memory each
  typename OP::State st = OP::init();
  for (uint32_t r0 = 0; r0 < splits; r0 += 8) {
    typename OP::State v[8];
#pragma unroll
    for (uint32_t u = 0; u < 8; ++u)
      v[u] = load_state(partial + (o * splits + (r0 + u < splits ? r0 + u : splits - 1)) * base + i);
#pragma unroll
    for (uint32_t u = 0; u < 8; ++u)
      if (r0 + u < splits) {
        if (r0 + u == 0) st = v[0];
        else OP::merge(st, v[u]);
      }
  }
  emit<T, OP, EMIT>(st, y, index_out, gy, gx, o * base + i, o * n * base + i, base, n);
}

template <typename T, typename OP, Emit EMIT>
__device__ inline void finish(const typename OP::State &st, typename OP::State *partial, Split sp, uint32_t r,
                              T *y, uint32_t *index_out, const T *gy, T *gx, size_t o, uint32_t i, uint32_t base,
                              uint32_t n) {
  if (sp.splits > 1) {
    store_state(partial + (o * sp.splits + r) * base + i, st);
  } else {
    emit<T, OP, EMIT>(st, y, index_out, gy, gx, o * base + i, o * n * base + i, base, n);
  }
}

// One workgroup per (output element, range); thread t takes j = lo + t, lo + t + 256, ...
template <typename T, typename OP, Emit EMIT>
__global__ __launch_bounds__(kBlock) void reduce_block_kernel(const T *x, T *y, uint32_t *index_out, const T *gy,
                                                               T *gx, typename OP::State *partial, Split sp,
                                                               uint32_t base, uint32_t n, size_t outputs) {
  __shared__ typename OP::State part[kBlock];
  __shared__ uint32_t last;
  for (size_t b = blockIdx.x; b < outputs * sp.splits; b += gridDim.x) {
    const size_t q = b / sp.splits;
    const uint32_t r = (uint32_t)(b - q * sp.splits);
    const size_t o = q / base;
    const uint32_t i = (uint32_t)(q - o * base);
    const uint32_t lo = r * sp.chunk, hi = n - lo < sp.chunk ? n : lo + sp.chunk;
    part[threadIdx.x] = walk<T, OP, 8>(x + o * n * base + i, base, lo + threadIdx.x, kBlock, hi);
    __syncthreads();
    for (int w = kBlock / 2; w > 0; w >>= 1) {
      if ((int)threadIdx.x < w) OP::merge(part[threadIdx.x], part[threadIdx.x + w]);
      __syncthreads();
    }
    if (threadIdx.x == 0) finish<T, OP, EMIT>(part[0], partial, sp, r, y, index_out, gy, gx, o, i, base, n);
    if (sp.splits > 1) {
      if (last_of_group(sp.tickets + q, sp.splits, &last) && threadIdx.x == 0)
        merge_ranges<T, OP, EMIT>(partial, sp.splits, y, index_out, gy, gx, o, i, base, n);
    }
    __syncthreads();
  }
}

// base == 1: wavefront w of the grid owns outputs w, w + waves, ...; its lanes
// stride along the contiguous run.
// V > 1: n is a multiple of V and x is aligned to V elements; a lane then takes V
// neighbouring elements per access.
template <typename T, typename OP, Emit EMIT, int V>
__global__ __launch_bounds__(kBlock) void reduce_rows_kernel(const T *x, T *y, uint32_t *index_out, const T *gy,
                                                              T *gx, uint32_t n, size_t outputs) {
  const uint32_t lane = threadIdx.x & 63;
  const size_t waves = (size_t)gridDim.x * (kBlock / 64);
  for (size_t q = (size_t)blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6); q < outputs; q += waves) {
    const size_t first = q * n;
    typename OP::State st;
    if constexpr (V > 1) st = walk_packs<T, OP, V>(x + first, lane, 64, n);
    else st = walk<T, OP>(x + first, 1, lane, 64, n);
#pragma unroll
    for (int w = 32; w > 0; w >>= 1) {
      typename OP::State other;
      unsigned char *dst = reinterpret_cast<unsigned char *>(&other);
      const unsigned char *src = reinterpret_cast<const unsigned char *>(&st);
#pragma unroll
      for (unsigned k = 0; k < sizeof(st) / 4; ++k) {
        int word;
        __builtin_memcpy(&word, src + 4 * k, 4);
        word = __shfl_down(word, w, 64);
        __builtin_memcpy(dst + 4 * k, &word, 4);
      }
      if (lane < (uint32_t)w) OP::merge(st, other);
    }
    if (lane == 0) emit<T, OP, EMIT>(st, y, index_out, gy, gx, q, first, 1, n);
  }
}

// V adjacent columns per lane, fetched as one V*sizeof(T)-byte access: U
// independent partial states per column over j = first, first + step, ... < end.
template <typename T, typename OP, int V, int U = 4>
__device__ inline void walk_cols(const T *p, size_t stride_elems, uint32_t first, uint32_t step, uint32_t end,
                                 typename OP::State (&out)[V]) {
  struct alignas(V * sizeof(T)) Cols {
    T c[V];
  };
  typename OP::State st[U][V];
#pragma unroll
  for (int u = 0; u < U; ++u)
#pragma unroll
    for (int k = 0; k < V; ++k) st[u][k] = OP::init();
  uint32_t j = first;
  for (; j < end && end - j > (U - 1) * step; j += U * step) {
    Cols v[U];
#pragma unroll
    for (int u = 0; u < U; ++u) v[u] = *reinterpret_cast<const Cols *>(p + (size_t)(j + u * step) * stride_elems);
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int k = 0; k < V; ++k) OP::push(st[u][k], to_f32(v[u].c[k]), j + u * step);
  }
#pragma unroll
  for (int u = 0; u < U - 1; ++u) {
    if (j < end) {
      const Cols v = *reinterpret_cast<const Cols *>(p + (size_t)j * stride_elems);
#pragma unroll
      for (int k = 0; k < V; ++k) OP::push(st[u][k], to_f32(v.c[k]), j);
    }
    j += step;
  }
#pragma unroll
  for (int w = 1; w < U; w *= 2) {
#pragma unroll
    for (int u = 0; u + w < U; u += 2 * w)
#pragma unroll
      for (int k = 0; k < V; ++k) OP::merge(st[u][k], st[u + w][k]);
  }
#pragma unroll
  for (int k = 0; k < V; ++k) out[k] = st[0][k];
}

// base >= 16: threads (tx, ty); tx walks base (contiguous, V columns per
// lane), ty splits the range of n that the workgroup owns.  V > 1 needs base
// to be a multiple of V and x aligned to V elements.
template <typename T, typename OP, Emit EMIT, int TX, int V>
__global__ __launch_bounds__(kBlock) void reduce_tiles_kernel(const T *x, T *y, uint32_t *index_out, const T *gy,
                                                               T *gx, typename OP::State *partial, Split sp,
                                                               uint32_t base, uint32_t n, uint32_t outer) {
  constexpr int TY = kBlock / TX;
  __shared__ typename OP::State part[TY][TX][V];
  __shared__ uint32_t last;
  const uint32_t tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const uint32_t per_o = (base + TX * V - 1) / (TX * V);
  for (size_t b = blockIdx.x; b < (size_t)per_o * outer * sp.splits; b += gridDim.x) {
    const uint32_t r = (uint32_t)(b % sp.splits);
    const size_t t = b / sp.splits;
    const size_t o = t / per_o;
    const uint32_t i = ((uint32_t)(t - o * per_o) * TX + tx) * V;
    const uint32_t lo = r * sp.chunk, hi = n - lo < sp.chunk ? n : lo + sp.chunk;
    typename OP::State st[V];
#pragma unroll
    for (int k = 0; k < V; ++k) st[k] = OP::init();
    if (i < base) walk_cols<T, OP, V>(x + o * n * base + i, base, lo + ty, TY, hi, st);
#pragma unroll
    for (int k = 0; k < V; ++k) part[ty][tx][k] = st[k];
    __syncthreads();
    if (ty == 0 && i < base) {
#pragma unroll
      for (int k = 0; k < V; ++k) {
        for (int u = 1; u < TY; ++u) OP::merge(st[k], part[u][tx][k]);
        finish<T, OP, EMIT>(st[k], partial, sp, r, y, index_out, gy, gx, o, i + k, base, n);
      }
    }
    if (sp.splits > 1) {
      if (last_of_group(sp.tickets + t, sp.splits, &last)) {
        const uint32_t i0 = (uint32_t)(t - o * per_o) * TX * V;
        for (uint32_t e = threadIdx.x; e < TX * V && i0 + e < base; e += kBlock)
          merge_ranges<T, OP, EMIT>(partial, sp.splits, y, index_out, gy, gx, o, i0 + e, base, n);
      }
    }
    __syncthreads();
  }
}

// How many ranges to cut n into so that `groups` workgroups become about four
// per compute unit, each range at least `min_chunk` long.
inline Split choose_split(size_t groups, uint32_t n, uint32_t min_chunk, size_t cus) {
  Split sp = {1, n, nullptr};
  const size_t want = 4 * cus;
  if (groups >= want || n < 2 * min_chunk) return sp;
  size_t splits = (want + groups - 1) / groups;
  const size_t most = n / min_chunk;
  if (splits > most) splits = most;
  if (splits < 2) return sp;
  sp.chunk = (uint32_t)((n + splits - 1) / splits);
  sp.splits = (uint32_t)((n + sp.chunk - 1) / sp.chunk);
  return sp;
}

template <typename T, typename OP, Emit EMIT>
int launch_reduce(phip_ctx *ctx, const T *x, T *y, uint32_t *index_out, const T *gy, T *gx, uint32_t base,
                  uint32_t n, uint32_t outer) {
  typedef typename OP::State State;
  const size_t outputs = (size_t)base * outer;
  const size_t cus = (size_t)ctx->prop.multiProcessorCount;
  const size_t cap = cus * 16;
  const bool by_block = n >= 256 && outputs < 2 * cus;
  const bool by_rows = !by_block && base == 1 && n >= 32;
  const bool by_tiles = !by_block && !by_rows && base >= 16 && n >= 16;
  if (!by_block && !by_tiles) {
    if (by_rows) {
      const size_t blocks = (outputs + kBlock / 64 - 1) / (kBlock / 64);
      constexpr int kPack = 16 / sizeof(T);   // 16 bytes per lane and access
      const dim3 rows_grid((unsigned)(blocks < cap ? blocks : cap));
      if (n % kPack == 0 && n >= 64 * kPack && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
        hipLaunchKernelGGL((reduce_rows_kernel<T, OP, EMIT, kPack>), rows_grid, dim3(kBlock), 0, ctx->stream, x, y,
                           index_out, gy, gx, n, outputs);
      } else {
        hipLaunchKernelGGL((reduce_rows_kernel<T, OP, EMIT, 1>), rows_grid, dim3(kBlock), 0, ctx->stream, x, y,
                           index_out, gy, gx, n, outputs);
      }
    } else {
      hipLaunchKernelGGL((reduce_column_kernel<T, OP, EMIT>), dim3(blocks_for(outputs, ctx)), dim3(kBlock), 0,
                         ctx->stream, x, y, index_out, gy, gx, base, n, outputs);
    }
    PHIP_LAUNCH_CHECK();
    return PHIP_OK;
  }
  // 8 bytes per lane and access (two fp32 or four 16-bit columns) when base and the address allow,
  // else 4 bytes for 16-bit storage (two columns)
  constexpr int kCols = 8 / sizeof(T), kHalf = sizeof(T) == 2 ? 2 : 1;
  const bool wide = base >= 64 * kCols && base % kCols == 0 && reinterpret_cast<uintptr_t>(x) % 8 == 0;
  const bool wide2 = !wide && kHalf > 1 && base >= 64 * kHalf && base % kHalf == 0 && reinterpret_cast<uintptr_t>(x) % 4 == 0;
  const int tx = base >= 64 ? 64 : 16;
  const int cols = wide ? kCols : wide2 ? kHalf : 1;
  const size_t groups = by_block ? outputs : (size_t)((base + tx * cols - 1) / (tx * cols)) * outer;
  Split sp = choose_split(groups, n, by_block ? 1024 : 256, cus);
  if (groups > (size_t)kTicketSlots) sp = Split{1, n, nullptr};  // a counter per group, or no ranges
  void *block = nullptr;
  if (sp.splits > 1) {
    const int rc = scratch_alloc(ctx, sizeof(State) * outputs * sp.splits, &block);  // the context's private scratch pool
    if (rc != PHIP_OK) return rc;
    sp.tickets = ctx->tile_tickets;
  }
  State *partial = static_cast<State *>(block);
  const size_t blocks = groups * sp.splits;
  const dim3 grid((unsigned)(blocks < cap ? blocks : cap));
  if (by_block) {
    hipLaunchKernelGGL((reduce_block_kernel<T, OP, EMIT>), grid, dim3(kBlock), 0, ctx->stream, x, y, index_out, gy,
                       gx, partial, sp, base, n, outputs);
  } else if (wide) {
    hipLaunchKernelGGL((reduce_tiles_kernel<T, OP, EMIT, 64, kCols>), grid, dim3(kBlock), 0, ctx->stream, x, y,
                       index_out, gy, gx, partial, sp, base, n, outer);
  } else if (wide2) {
    hipLaunchKernelGGL((reduce_tiles_kernel<T, OP, EMIT, 64, kHalf>), grid, dim3(kBlock), 0, ctx->stream, x, y,
                       index_out, gy, gx, partial, sp, base, n, outer);
  } else if (tx == 64) {
    hipLaunchKernelGGL((reduce_tiles_kernel<T, OP, EMIT, 64, 1>), grid, dim3(kBlock), 0, ctx->stream, x, y, index_out,
                       gy, gx, partial, sp, base, n, outer);
  } else {
    hipLaunchKernelGGL((reduce_tiles_kernel<T, OP, EMIT, 16, 1>), grid, dim3(kBlock), 0, ctx->stream, x, y, index_out,
                       gy, gx, partial, sp, base, n, outer);
  }
  if (sp.splits > 1) {
    scratch_free(ctx, block);  // the stream is in order: the block may be handed out again behind this launch
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
      return launch_reduce<T, ExtremumValueOp<1>, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
    default:
      return launch_reduce<T, ExtremumValueOp<-1>, Emit::Value>(ctx, px, py, nullptr, nullptr, nullptr, base, n, outer);
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
