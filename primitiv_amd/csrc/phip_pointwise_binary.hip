// Two-operand elementwise families with minibatch broadcasting:
//   y = a op b,  y = x op k[sample],  ga += dy/da * gy,  gb += dy/db * gy.
// An operand whose batch is 1 is re-read for every sample; its gradient is the
// sum over the samples, accumulated in registers by the threads that own the
// element and combined through LDS in a fixed order (no atomics).  16-byte
// accesses per lane wherever alignment and the sample size allow; a backward
// kernel loads only those of a, b, y that its formula uses.
#include "phip_pointwise.h"

namespace phip {
namespace {

using namespace pointwise;

// ---- formulas ---------------------------------------------------------------
// fw(a, b) is the forward value; bw() yields the amounts added to ga and gb.
// kA / kB / kY say whether bw reads a / b / y.

struct Add {
  static constexpr bool kA = false, kB = false, kY = false;
  __device__ static float fw(float a, float b) { return a + b; }
  __device__ static void bw(float, float, float, float gy, float &da, float &db) {
    da = gy;
    db = gy;
  }
};
struct Subtract {
  static constexpr bool kA = false, kB = false, kY = false;
  __device__ static float fw(float a, float b) { return a - b; }
  __device__ static void bw(float, float, float, float gy, float &da, float &db) {
    da = gy;
    db = -gy;
  }
};
struct Multiply {
  static constexpr bool kA = true, kB = true, kY = false;
  __device__ static float fw(float a, float b) { return a * b; }
  __device__ static void bw(float a, float b, float, float gy, float &da, float &db) {
    da = gy * b;
    db = gy * a;
  }
};
struct Divide {
  static constexpr bool kA = false, kB = true, kY = true;
  __device__ static float fw(float a, float b) { return a / b; }
  __device__ static void bw(float, float b, float y, float gy, float &da, float &db) {
    const float k = gy / b;
    da = k;
    db = -k * y;
  }
};
struct Pow {
  static constexpr bool kA = true, kB = true, kY = true;
  __device__ static float fw(float a, float b) { return powf(a, b); }
  __device__ static void bw(float a, float b, float y, float gy, float &da, float &db) {
    const float k = gy * y;
    da = k * b / a;
    db = k * logf(a);
  }
};

// ---- forward ----------------------------------------------------------------

// y[s][i] = a[s * sa + i] op b[s * sb + i] for i < volume, s < bs; sa and sb are
// `volume` or 0.  With VEC, volume is a multiple of the pack size unless
// bs == 1 (then the remainder is handled element by element).
template <typename T, typename OP, bool VEC>
__global__ __launch_bounds__(kBlock) void binary_fw_kernel(const T *a, const T *b, T *y, size_t volume, uint32_t bs,
                                                            size_t sa, size_t sb) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  for (uint32_t s = blockIdx.y; s < bs; s += gridDim.y) {
    const T *pa = a + s * sa;
    const T *pb = b + s * sb;
    T *py = y + (size_t)s * volume;
    if constexpr (VEC) {
      constexpr int N = Pack<T>::N;
      const size_t packs = volume / N;
      for (size_t p = first; p < packs; p += stride) {
        const Pack<T> va = load_pack(pa + p * N), vb = load_pack(pb + p * N);
        Pack<T> out;
#pragma unroll
        for (int e = 0; e < N; ++e) out.v[e] = from_f32<T>(OP::fw(to_f32(va.v[e]), to_f32(vb.v[e])));
        store_pack(py + p * N, out);
      }
      const size_t t = packs * N + first;
      if (t < volume) py[t] = from_f32<T>(OP::fw(to_f32(pa[t]), to_f32(pb[t])));
    } else {
      for (size_t i = first; i < volume; i += stride) py[i] = from_f32<T>(OP::fw(to_f32(pa[i]), to_f32(pb[i])));
    }
  }
}

// y[s][i] = x[s * sx + i] op k[s * sk]  (or k op x when `left`); sk is 1 or 0.
template <typename T, typename OP, bool VEC>
__global__ __launch_bounds__(kBlock) void scalar_fw_kernel(const T *x, const T *k, T *y, size_t volume, uint32_t bs,
                                                            size_t sx, size_t sk, bool left) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  for (uint32_t s = blockIdx.y; s < bs; s += gridDim.y) {
    const T *px = x + s * sx;
    const float kv = to_f32(k[s * sk]);
    T *py = y + (size_t)s * volume;
    auto f = [&](float xv) { return left ? OP::fw(kv, xv) : OP::fw(xv, kv); };
    if constexpr (VEC) {
      constexpr int N = Pack<T>::N;
      const size_t packs = volume / N;
      for (size_t p = first; p < packs; p += stride) {
        const Pack<T> vx = load_pack(px + p * N);
        Pack<T> out;
#pragma unroll
        for (int e = 0; e < N; ++e) out.v[e] = from_f32<T>(f(to_f32(vx.v[e])));
        store_pack(py + p * N, out);
      }
      const size_t t = packs * N + first;
      if (t < volume) py[t] = from_f32<T>(f(to_f32(px[t])));
    } else {
      for (size_t i = first; i < volume; i += stride) py[i] = from_f32<T>(f(to_f32(px[i])));
    }
  }
}

// ---- backward, same batch on both sides ---------------------------------------

// ga[i] += da, gb[i] += db.  `same` is set when ga and gb are one array (both
// operands are the same tensor): then the array receives da + db.  acc_a / acc_b off: that
// gradient's old value counts as zero and is not read.
template <typename T, typename OP, bool VEC>
__global__ __launch_bounds__(kBlock) void binary_bw_flat_kernel(const T *a, const T *b, const T *y, const T *gy,
                                                                 T *ga, T *gb, size_t n, bool same, bool acc_a,
                                                                 bool acc_b) {
  const size_t stride = (size_t)gridDim.x * kBlock;
  const size_t first = (size_t)blockIdx.x * kBlock + threadIdx.x;
  auto one = [&](size_t i) {
    float da, db;
    OP::bw(OP::kA ? to_f32(a[i]) : 0.f, OP::kB ? to_f32(b[i]) : 0.f, OP::kY ? to_f32(y[i]) : 0.f, to_f32(gy[i]),
           da, db);
    if (same) {
      ga[i] = from_f32<T>(to_f32(from_f32<T>((acc_a ? to_f32(ga[i]) : 0.f) + da)) + db);
    } else {
      ga[i] = from_f32<T>((acc_a ? to_f32(ga[i]) : 0.f) + da);
      gb[i] = from_f32<T>((acc_b ? to_f32(gb[i]) : 0.f) + db);
    }
  };
  if constexpr (VEC) {
    constexpr int N = Pack<T>::N;
    const size_t packs = n / N;
    for (size_t p = first; p < packs; p += stride) {
      Pack<T> va, vb, vy;
      if constexpr (OP::kA) va = load_pack(a + p * N);
      if constexpr (OP::kB) vb = load_pack(b + p * N);
      if constexpr (OP::kY) vy = load_pack(y + p * N);
      const Pack<T> vg = load_pack(gy + p * N);
      Pack<T> oa, ob;
      if (acc_a) oa = load_pack(ga + p * N);
      if (!same && acc_b) ob = load_pack(gb + p * N);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        float av = 0.f, bv = 0.f, yv = 0.f, da, db;
        if constexpr (OP::kA) av = to_f32(va.v[e]);
        if constexpr (OP::kB) bv = to_f32(vb.v[e]);
        if constexpr (OP::kY) yv = to_f32(vy.v[e]);
        OP::bw(av, bv, yv, to_f32(vg.v[e]), da, db);
        if (same) {
          oa.v[e] = from_f32<T>(to_f32(from_f32<T>((acc_a ? to_f32(oa.v[e]) : 0.f) + da)) + db);
        } else {
          oa.v[e] = from_f32<T>((acc_a ? to_f32(oa.v[e]) : 0.f) + da);
          ob.v[e] = from_f32<T>((acc_b ? to_f32(ob.v[e]) : 0.f) + db);
        }
      }
      store_pack(ga + p * N, oa);
      if (!same) store_pack(gb + p * N, ob);
    }
    const size_t t = packs * N + first;
    if (t < n) one(t);
  } else {
    for (size_t i = first; i < n; i += stride) one(i);
  }
}

// ---- backward, one operand broadcast ----------------------------------------

// One operand (a when `a_bcast`, else b) has batch 1.  A block is TX items
// wide (an item is a pack with VEC, else one element) and TY deep: thread
// (tx, ty) walks samples ty, ty + TY, ...; it updates the batched operand's
// gradient in place and keeps the broadcast operand's in registers.  The TY
// partial sums of an item are then added in order of ty and the total added
// to the broadcast gradient once.  acc_full / acc_one off: the old value of the batched / the
// broadcast operand's gradient counts as zero and is not read.
template <typename T, typename OP, bool VEC, int TY>
__global__ __launch_bounds__(kBlock) void binary_bw_bcast_kernel(const T *a, const T *b, const T *y, const T *gy,
                                                                  T *ga, T *gb, size_t volume, uint32_t bs,
                                                                  bool a_bcast, bool acc_full, bool acc_one) {
  constexpr int N = VEC ? Pack<T>::N : 1;
  constexpr int TX = kBlock / TY;
  const int tx = threadIdx.x % TX, ty = threadIdx.x / TX;
  const size_t items = volume / N;
  const size_t item = (size_t)blockIdx.x * TX + tx;
  const bool live = item < items;
  const size_t off1 = item * N;  // offset inside a sample
  float acc[N];
#pragma unroll
  for (int e = 0; e < N; ++e) acc[e] = 0.f;

  if (live) {
    for (uint32_t s = ty; s < bs; s += TY) {
      const size_t offn = (size_t)s * volume + off1;
      const size_t oa = a_bcast ? off1 : offn, ob = a_bcast ? offn : off1;
      T *gfull = a_bcast ? gb + offn : ga + offn;  // gradient of the batched operand
      if constexpr (VEC) {
        Pack<T> va, vb, vy;
        if constexpr (OP::kA) va = load_pack(a + oa);
        if constexpr (OP::kB) vb = load_pack(b + ob);
        if constexpr (OP::kY) vy = load_pack(y + offn);
        const Pack<T> vg = load_pack(gy + offn);
        Pack<T> out;
        if (acc_full) out = load_pack(gfull);
#pragma unroll
        for (int e = 0; e < N; ++e) {
          float av = 0.f, bv = 0.f, yv = 0.f, da, db;
          if constexpr (OP::kA) av = to_f32(va.v[e]);
          if constexpr (OP::kB) bv = to_f32(vb.v[e]);
          if constexpr (OP::kY) yv = to_f32(vy.v[e]);
          OP::bw(av, bv, yv, to_f32(vg.v[e]), da, db);
          acc[e] += a_bcast ? da : db;
          out.v[e] = from_f32<T>((acc_full ? to_f32(out.v[e]) : 0.f) + (a_bcast ? db : da));
        }
        store_pack(gfull, out);
      } else {
        float da, db;
        OP::bw(OP::kA ? to_f32(a[oa]) : 0.f, OP::kB ? to_f32(b[ob]) : 0.f, OP::kY ? to_f32(y[offn]) : 0.f,
               to_f32(gy[offn]), da, db);
        acc[0] += a_bcast ? da : db;
        *gfull = from_f32<T>((acc_full ? to_f32(*gfull) : 0.f) + (a_bcast ? db : da));
      }
    }
  }

  if constexpr (TY > 1) {
    __shared__ float partial[TY][N][TX];
#pragma unroll
    for (int e = 0; e < N; ++e) partial[ty][e][tx] = acc[e];
    __syncthreads();
    if (ty == 0) {
#pragma unroll
      for (int e = 0; e < N; ++e)
        for (int t = 1; t < TY; ++t) acc[e] += partial[t][e][tx];
    }
  }
  if (ty == 0 && live) {
    T *g1 = (a_bcast ? ga : gb) + off1;
    if constexpr (VEC) {
      Pack<T> out;
      if (acc_one) out = load_pack(g1);
#pragma unroll
      for (int e = 0; e < N; ++e) out.v[e] = from_f32<T>((acc_one ? to_f32(out.v[e]) : 0.f) + acc[e]);
      store_pack(g1, out);
    } else {
      *g1 = from_f32<T>((acc_one ? to_f32(*g1) : 0.f) + acc[0]);
    }
  }
}

// ---- launchers --------------------------------------------------------------

inline int check_batches(uint32_t b0, uint32_t b1) {
  PHIP_REQUIRE(b0 >= 1 && b1 >= 1 && (b0 == b1 || b0 == 1 || b1 == 1), "incompatible batch sizes: %u, %u", b0, b1);
  return PHIP_OK;
}

// Grid for `bs` samples of `items` work items each.
inline dim3 sample_grid(size_t items, uint32_t bs, const phip_ctx *ctx) {
  const unsigned gx = blocks_for(items, ctx);
  const unsigned cap = (unsigned)ctx->prop.multiProcessorCount * 32;
  unsigned gy = gx >= cap ? 1 : cap / gx;
  if (gy > bs) gy = bs;
  if (gy > 65535u) gy = 65535u;
  return dim3(gx, gy < 1 ? 1 : gy);
}

template <typename T, typename OP>
int launch_binary_fw(phip_ctx *ctx, const void *a, const void *b, void *y, uint32_t volume, uint32_t ba,
                     uint32_t bb) {
  PHIP_ENTER(ctx);
  const int rc = check_batches(ba, bb);
  if (rc != PHIP_OK) return rc;
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(a != nullptr && b != nullptr && y != nullptr, "null pointer");
  constexpr int N = Pack<T>::N;
  size_t vol = volume;
  uint32_t bs = ba > bb ? ba : bb;
  size_t sa = ba > 1 ? vol : 0, sb = bb > 1 ? vol : 0;
  if (ba == bb) {  // nothing is broadcast: one long sample
    vol *= bs;
    bs = 1;
    sa = sb = 0;
  }
  const bool vec = aligned16(a) && aligned16(b) && aligned16(y) && (bs == 1 || vol % N == 0);
  const T *pa = static_cast<const T *>(a);
  const T *pb = static_cast<const T *>(b);
  T *py = static_cast<T *>(y);
  if (vec) {
    hipLaunchKernelGGL((binary_fw_kernel<T, OP, true>), sample_grid(vol / N + N, bs, ctx), dim3(kBlock), 0,
                       ctx->stream, pa, pb, py, vol, bs, sa, sb);
  } else {
    hipLaunchKernelGGL((binary_fw_kernel<T, OP, false>), sample_grid(vol, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       pa, pb, py, vol, bs, sa, sb);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T, typename OP>
int launch_scalar_fw(phip_ctx *ctx, int k_on_left, const void *x, const void *k, void *y, uint32_t volume,
                     uint32_t bx, uint32_t bk) {
  PHIP_ENTER(ctx);
  const int rc = check_batches(bx, bk);
  if (rc != PHIP_OK) return rc;
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && k != nullptr && y != nullptr, "null pointer");
  constexpr int N = Pack<T>::N;
  size_t vol = volume;
  uint32_t bs = bx > bk ? bx : bk;
  size_t sx = bx > 1 ? vol : 0;
  const size_t sk = bk > 1 ? 1 : 0;
  if (bk == 1 && bx == bs) {  // one scalar for everything: one long sample
    vol *= bs;
    bs = 1;
    sx = 0;
  }
  const bool vec = aligned16(x) && aligned16(y) && (bs == 1 || vol % N == 0);
  const T *px = static_cast<const T *>(x);
  const T *pk = static_cast<const T *>(k);
  T *py = static_cast<T *>(y);
  if (vec) {
    hipLaunchKernelGGL((scalar_fw_kernel<T, OP, true>), sample_grid(vol / N + N, bs, ctx), dim3(kBlock), 0,
                       ctx->stream, px, pk, py, vol, bs, sx, sk, k_on_left != 0);
  } else {
    hipLaunchKernelGGL((scalar_fw_kernel<T, OP, false>), sample_grid(vol, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       px, pk, py, vol, bs, sx, sk, k_on_left != 0);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T, typename OP>
int launch_binary_bw(phip_ctx *ctx, const void *a, const void *b, const void *y, const void *gy, void *ga, void *gb,
                     uint32_t volume, uint32_t ba, uint32_t bb) {
  PHIP_ENTER_KEEP_ZEROS(ctx);
  const int rc = check_batches(ba, bb);
  if (rc != PHIP_OK) return rc;
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(gy != nullptr && ga != nullptr && gb != nullptr, "null pointer");
  PHIP_REQUIRE(!OP::kA || a != nullptr, "this gradient needs a");
  PHIP_REQUIRE(!OP::kB || b != nullptr, "this gradient needs b");
  PHIP_REQUIRE(!OP::kY || y != nullptr, "this gradient needs y");
  PHIP_REQUIRE(ba == bb || ga != gb, "gradients of operands with different batch sizes cannot share memory");
  // a gradient noted as zero and not yet filled is written instead of added into
  const size_t na = (size_t)volume * ba * sizeof(T), nb = (size_t)volume * bb * sizeof(T);
  const size_t ny = na > nb ? na : nb;
  auto read_too = [&](const void *g, size_t bytes) {
    return shares_memory(g, bytes, gy, ny) || (OP::kA && shares_memory(g, bytes, a, na)) ||
           (OP::kB && shares_memory(g, bytes, b, nb)) || (OP::kY && shares_memory(g, bytes, y, ny));
  };
  const bool apart = ga == gb || !shares_memory(ga, na, gb, nb);
  const bool acc_a = !apart || read_too(ga, na) || !zeros_take(ctx, ga, na);
  const bool acc_b = ga == gb ? acc_a : (!apart || read_too(gb, nb) || !zeros_take(ctx, gb, nb));
  PHIP_FLUSH_ZEROS(ctx);
  constexpr int N = Pack<T>::N;
  const T *pa = static_cast<const T *>(a);
  const T *pb = static_cast<const T *>(b);
  const T *py = static_cast<const T *>(y);
  const T *pgy = static_cast<const T *>(gy);
  T *pga = static_cast<T *>(ga);
  T *pgb = static_cast<T *>(gb);
  const bool all_aligned = aligned16(gy) && aligned16(ga) && aligned16(gb) && (!OP::kA || aligned16(a)) &&
                           (!OP::kB || aligned16(b)) && (!OP::kY || aligned16(y));
  if (ba == bb) {
    const size_t n = (size_t)volume * ba;
    const bool same = ga == gb;
    if (all_aligned) {
      hipLaunchKernelGGL((binary_bw_flat_kernel<T, OP, true>), dim3(blocks_for(n / N + N, ctx)), dim3(kBlock), 0,
                         ctx->stream, pa, pb, py, pgy, pga, pgb, n, same, acc_a, acc_b);
    } else {
      hipLaunchKernelGGL((binary_bw_flat_kernel<T, OP, false>), dim3(blocks_for(n, ctx)), dim3(kBlock), 0,
                         ctx->stream, pa, pb, py, pgy, pga, pgb, n, same, acc_a, acc_b);
    }
  } else {
    const bool a_bcast = ba == 1;
    const uint32_t bs = a_bcast ? bb : ba;
    const bool vec = all_aligned && volume % N == 0;
    const size_t items = vec ? volume / N : volume;
    // few items: put 8 threads on each so that the walk over the batch is shared
    const bool deep = items < (size_t)ctx->prop.multiProcessorCount * kBlock * 2 && bs >= 8;
#define PHIP_BCAST(VEC, TY)                                                                                       \
  hipLaunchKernelGGL((binary_bw_bcast_kernel<T, OP, VEC, TY>),                                                    \
                     dim3((unsigned)((items + kBlock / TY - 1) / (kBlock / TY))), dim3(kBlock), 0, ctx->stream,   \
                     pa, pb, py, pgy, pga, pgb, (size_t)volume, bs, a_bcast, a_bcast ? acc_b : acc_a,                \
                     a_bcast ? acc_a : acc_b)
    if (vec && deep) PHIP_BCAST(true, 8);
    else if (vec) PHIP_BCAST(true, 1);
    else if (deep) PHIP_BCAST(false, 8);
    else PHIP_BCAST(false, 1);
#undef PHIP_BCAST
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// Calls `call(formula)` for the formula an operation code names.
template <typename Call>
int with_binary(int op, Call &&call) {
  switch (op) {
    case PHIP_ADD: return call(Add{});
    case PHIP_SUBTRACT: return call(Subtract{});
    case PHIP_MULTIPLY: return call(Multiply{});
    case PHIP_DIVIDE: return call(Divide{});
    case PHIP_POW: return call(Pow{});
    default: return fail(PHIP_ERR_INVALID_ARGUMENT, "unknown binary operation %d", op);
  }
}

template <typename T>
int binary_fw(phip_ctx *ctx, int op, const void *a, const void *b, void *y, uint32_t volume, uint32_t ba,
              uint32_t bb) {
  return with_binary(op, [&](auto f) { return launch_binary_fw<T, decltype(f)>(ctx, a, b, y, volume, ba, bb); });
}
template <typename T>
int binary_bw(phip_ctx *ctx, int op, const void *a, const void *b, const void *y, const void *gy, void *ga,
              void *gb, uint32_t volume, uint32_t ba, uint32_t bb) {
  return with_binary(
      op, [&](auto f) { return launch_binary_bw<T, decltype(f)>(ctx, a, b, y, gy, ga, gb, volume, ba, bb); });
}
template <typename T>
int scalar_fw(phip_ctx *ctx, int op, int k_on_left, const void *x, const void *k, void *y, uint32_t volume,
              uint32_t bx, uint32_t bk) {
  return with_binary(
      op, [&](auto f) { return launch_scalar_fw<T, decltype(f)>(ctx, k_on_left, x, k, y, volume, bx, bk); });
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_BINARY(SUF, T, CPTR, PTR)                                                                   \
  int phip_binary_fw_##SUF(phip_ctx *ctx, int op, CPTR a, CPTR b, PTR y, uint32_t volume, uint32_t ba,          \
                           uint32_t bb) {                                                                       \
    return binary_fw<T>(ctx, op, a, b, y, volume, ba, bb);                                                      \
  }                                                                                                             \
  int phip_binary_bw_##SUF(phip_ctx *ctx, int op, CPTR a, CPTR b, CPTR y, CPTR gy, PTR ga, PTR gb,              \
                           uint32_t volume, uint32_t ba, uint32_t bb) {                                         \
    return binary_bw<T>(ctx, op, a, b, y, gy, ga, gb, volume, ba, bb);                                          \
  }                                                                                                             \
  int phip_scalar_fw_##SUF(phip_ctx *ctx, int op, int k_on_left, CPTR x, CPTR k, PTR y, uint32_t volume,        \
                           uint32_t bx, uint32_t bk) {                                                          \
    return scalar_fw<T>(ctx, op, k_on_left, x, k, y, volume, bx, bk);                                           \
  }

PHIP_EXPORT_BINARY(f32, float, const float *, float *)
PHIP_EXPORT_BINARY(f16, f16_t, const void *, void *)
PHIP_EXPORT_BINARY(bf16, bf16_t, const void *, void *)

#undef PHIP_EXPORT_BINARY

}  // extern "C"
