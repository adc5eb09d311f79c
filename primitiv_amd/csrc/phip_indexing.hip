// Data-movement operations between the matmuls: strided row copies (slice,
// concat, batch_slice, batch_concat), pick / batch_pick, transpose,
// permute_dims, flip and broadcast.  All move each element once; gradients
// are accumulated into.  Where several sources fall on one destination (a
// gradient summed over the minibatch, repeated indices) one thread owns the
// destination and adds the sources in order, so results do not depend on
// scheduling and no atomics are used.
#include <type_traits>
#include <vector>

#include "phip_pointwise.h"

namespace phip {
namespace {

using namespace pointwise;

template <typename T, bool ACC>
__device__ inline void put(T *p, float v) {
  if constexpr (ACC) *p = from_f32<T>(to_f32(*p) + v);
  else *p = from_f32<T>(v);
}

// ---- strided row copy ---------------------------------------------------------

// dst[b*dbs + r*ds + i] (=|+=) src[b*sbs + r*ss + i]; grid.y walks the samples.
template <typename T, bool ACC>
__global__ __launch_bounds__(kBlock) void copy_rows_kernel(const T *src, T *dst, uint32_t span, uint32_t total,
                                                            size_t ss, size_t ds, uint32_t bs, size_t sbs,
                                                            size_t dbs) {
  for (uint32_t idx = blockIdx.x * kBlock + threadIdx.x; idx < total; idx += gridDim.x * kBlock) {
    const uint32_t r = idx / span, i = idx - r * span;
    for (uint32_t b = blockIdx.y; b < bs; b += gridDim.y)
      put<T, ACC>(dst + b * dbs + r * ds + i, to_f32(src[b * sbs + r * ss + i]));
  }
}

// The same copy in 16-byte packs: span, the strides and both addresses are
// multiples of a pack, and every argument counts packs.
template <typename T, bool ACC>
__global__ __launch_bounds__(kBlock) void copy_rows_pack_kernel(const T *src, T *dst, uint32_t span, uint32_t total,
                                                                 size_t ss, size_t ds, uint32_t bs, size_t sbs,
                                                                 size_t dbs) {
  constexpr int N = Pack<T>::N;
  for (uint32_t idx = blockIdx.x * kBlock + threadIdx.x; idx < total; idx += gridDim.x * kBlock) {
    const uint32_t r = idx / span, i = idx - r * span;
    for (uint32_t b = blockIdx.y; b < bs; b += gridDim.y) {
      Pack<T> v = load_pack(src + (b * sbs + r * ss + i) * N);
      T *d = dst + (b * dbs + r * ds + i) * N;
      if constexpr (ACC) {
        const Pack<T> old = load_pack(d);
#pragma unroll
        for (int k = 0; k < N; ++k) v.v[k] = from_f32<T>(to_f32(old.v[k]) + to_f32(v.v[k]));
      }
      store_pack(d, v);
    }
  }
}

// dst[r*ds + i] += sum over b of src[b*sbs + r*ss + i], added in order of b.
template <typename T>
__global__ __launch_bounds__(kBlock) void copy_rows_sum_kernel(const T *src, T *dst, uint32_t span, uint32_t total,
                                                                size_t ss, size_t ds, uint32_t bs, size_t sbs) {
  for (uint32_t idx = blockIdx.x * kBlock + threadIdx.x; idx < total; idx += gridDim.x * kBlock) {
    const uint32_t r = idx / span, i = idx - r * span;
    T *d = dst + r * ds + i;
    float acc = to_f32(*d);
    const T *s = src + r * ss + i;
    for (uint32_t b = 0; b < bs; ++b) acc = to_f32(from_f32<T>(acc + to_f32(s[b * sbs])));
    *d = from_f32<T>(acc);
  }
}

// ---- pick -----------------------------------------------------------------------

// Up to kInlineIds indices travel in the kernel arguments; longer lists are
// copied to device memory first.
constexpr uint32_t kInlineIds = 256;
struct IdList {
  const uint32_t *device;   // used when not null
  uint32_t inline_ids[kInlineIds];
  __device__ uint32_t operator[](uint32_t i) const { return device ? device[i] : inline_ids[i]; }
};

// y[b][t] = x[b*sx + ids[b*si]*base + (t / base)*base*n + t % base], t < base*outer
template <typename T>
__global__ __launch_bounds__(kBlock) void pick_fw_kernel(const T *x, const IdList ids, T *y, uint32_t base,
                                                          uint32_t n, uint32_t sy, size_t sx, uint32_t si) {
  const uint32_t b = blockIdx.y;
  const T *px = x + b * sx + (size_t)ids[b * si] * base;
  for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < sy; t += gridDim.x * kBlock) {
    const uint32_t o = t / base, i = t - o * base;
    y[(size_t)b * sy + t] = px[(size_t)o * base * n + i];
  }
}

// Longest index list for which a workgroup row per sample is started (each row
// scans the list once).
constexpr uint32_t kOwnerSamples = 1024;

// Samples that pick the same index add into the same place of a shared gx.
// The first sample b that picks an index owns it: it adds, in sample order, the
// gradient of every sample that picks the same index; the others leave.  The
// result is the sequential sum whatever the schedule, and distinct indices
// proceed in parallel.  `b` is uniform over the workgroup.
__device__ inline bool owns_index(const IdList &ids, uint32_t b, uint32_t si) {
  const uint32_t id = ids[b * si];
  for (uint32_t p = 0; p < b; ++p)
    if (ids[p * si] == id) return false;
  return true;
}

// gx[b*sx + ...] += gy[b][t].  sx != 0: every sample has its own gx.  sx == 0
// and OWNERS: workgroup row b handles the samples that share ids[b] (see
// owns_index).  sx == 0 otherwise (very long lists): the thread that owns t
// walks the samples in order.
template <typename T, bool OWNERS>
__global__ __launch_bounds__(kBlock) void pick_bw_kernel(const T *gy, const IdList ids, T *gx, uint32_t base,
                                                          uint32_t n, uint32_t sy, size_t sx, uint32_t si,
                                                          uint32_t bs) {
  const uint32_t b = blockIdx.y;
  if (OWNERS && sx == 0 && !owns_index(ids, b, si)) return;
  for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < sy; t += gridDim.x * kBlock) {
    const uint32_t o = t / base, i = t - o * base;
    const size_t within = (size_t)o * base * n + i;
    if (sx != 0) {
      put<T, true>(gx + b * sx + (size_t)ids[b * si] * base + within, to_f32(gy[(size_t)b * sy + t]));
    } else if (OWNERS) {
      const uint32_t id = ids[b * si];
      T *g = gx + (size_t)id * base + within;
      float acc = to_f32(*g);
      for (uint32_t p = b; p < bs; ++p)
        if (ids[p * si] == id) acc = to_f32(from_f32<T>(acc + to_f32(gy[(size_t)p * sy + t])));
      *g = from_f32<T>(acc);
    } else {
      for (uint32_t p = 0; p < bs; ++p)
        put<T, true>(gx + (size_t)ids[p * si] * base + within, to_f32(gy[(size_t)p * sy + t]));
    }
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void batch_pick_fw_kernel(const T *x, const IdList ids, T *y, uint32_t sy) {
  const uint32_t b = blockIdx.y;
  const T *px = x + (size_t)ids[b] * sy;
  for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < sy; t += gridDim.x * kBlock)
    y[(size_t)b * sy + t] = px[t];
}

// gx[ids[b]][t] += gy[b][t]: indices may repeat.  OWNERS: workgroup row b handles
// the samples that share ids[b] (see owns_index); otherwise the owner of t
// walks b in order.
template <typename T, bool OWNERS>
__global__ __launch_bounds__(kBlock) void batch_pick_bw_kernel(const T *gy, const IdList ids, T *gx, uint32_t sy,
                                                                uint32_t bs) {
  const uint32_t b = blockIdx.y;
  if (OWNERS && !owns_index(ids, b, 1)) return;
  for (uint32_t t = blockIdx.x * kBlock + threadIdx.x; t < sy; t += gridDim.x * kBlock) {
    if (OWNERS) {
      const uint32_t id = ids[b];
      T *g = gx + (size_t)id * sy + t;
      float acc = to_f32(*g);
      for (uint32_t p = b; p < bs; ++p)
        if (ids[p] == id) acc = to_f32(from_f32<T>(acc + to_f32(gy[(size_t)p * sy + t])));
      *g = from_f32<T>(acc);
    } else {
      for (uint32_t p = 0; p < bs; ++p) put<T, true>(gx + (size_t)ids[p] * sy + t, to_f32(gy[(size_t)p * sy + t]));
    }
  }
}

// ---- transpose ------------------------------------------------------------------

// 64 x 64 tiles through LDS: a wavefront reads 64 consecutive elements of a
// source column and writes 64 consecutive elements of a destination column; the
// 16 loads of a thread are all issued before the first LDS write.
// dst (cols x rows) (=|+=) transpose(src (rows x cols)).
constexpr uint32_t kTr = 64;

template <typename T, bool ACC>
__global__ __launch_bounds__(kBlock) void transpose_kernel(const T *src, T *dst, uint32_t rows, uint32_t cols) {
  __shared__ float tile[kTr][kTr + 1];
  const size_t ofs = (size_t)blockIdx.z * rows * cols;
  const uint32_t tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const uint32_t i0 = blockIdx.x * kTr, j0 = blockIdx.y * kTr;
  float v[kTr / 4];
#pragma unroll
  for (uint32_t u = 0; u < kTr / 4; ++u) {
    const uint32_t i = i0 + tx, j = j0 + ty + 4 * u;
    v[u] = i < rows && j < cols ? to_f32(src[ofs + i + (size_t)j * rows]) : 0.f;
  }
#pragma unroll
  for (uint32_t u = 0; u < kTr / 4; ++u) tile[ty + 4 * u][tx] = v[u];
  __syncthreads();
#pragma unroll
  for (uint32_t u = 0; u < kTr / 4; ++u) {
    const uint32_t ii = ty + 4 * u, i = i0 + ii, j = j0 + tx;
    if (i < rows && j < cols) put<T, ACC>(dst + ofs + j + (size_t)i * cols, tile[tx][ii]);
  }
}

// rows and cols even: the matrix is taken as 2 x 2 blocks. A lane reads one pair
// of vertically adjacent elements (one word: 4 bytes of 16-bit storage, 8 of fp32)
// from each of two neighbouring source columns (rows 2a, 2a+1 of columns 2b, 2b+1),
// regroups the four elements into the two destination words (columns 2b, 2b+1 of
// destination rows 2a and 2a+1), and the blocks of a tile then move through LDS as
// whole words, one plane per destination-row parity. A wavefront reads 64 words
// in a row; a tile is 64 blocks along the source rows by kTb along its columns
// (32 KiB of source either way), so a thread has 32 KiB / 256 in flight before
// the first LDS write, twice what the one-element form holds.
template <typename T, bool ACC>
__global__ __launch_bounds__(kBlock) void transpose_pairs_kernel(const T *src, T *dst, uint32_t rows, uint32_t cols) {
  typedef typename std::conditional<sizeof(T) == 2, uint32_t, uint64_t>::type Word;
  constexpr uint32_t kHalf = 8 * sizeof(T);             // bits per element
  constexpr Word kLow = (Word(1) << kHalf) - 1;
  constexpr uint32_t kTb = sizeof(T) == 2 ? 64 : 32;    // blocks of a tile along the source columns
  constexpr uint32_t kRw = 64 / kTb;                    // destination rows a wavefront writes per access
  __shared__ Word tile[2][kTb][kTr + 1];
  const size_t ofs = (size_t)blockIdx.z * rows * cols;
  const uint32_t tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const uint32_t a0 = blockIdx.x * kTr, b0 = blockIdx.y * kTb;  // in 2 x 2 blocks
  const uint32_t ra = rows / 2, cb = cols / 2;
  const Word *sw = reinterpret_cast<const Word *>(src + ofs);
  Word w0[kTb / 4], w1[kTb / 4];
#pragma unroll
  for (uint32_t u = 0; u < kTb / 4; ++u) {
    const uint32_t a = a0 + tx, b = b0 + ty + 4 * u;
    const bool in = a < ra && b < cb;
    w0[u] = in ? sw[a + (size_t)(2 * b) * ra] : Word(0);
    w1[u] = in ? sw[a + (size_t)(2 * b + 1) * ra] : Word(0);
  }
#pragma unroll
  for (uint32_t u = 0; u < kTb / 4; ++u) {
    tile[0][ty + 4 * u][tx] = (w0[u] & kLow) | (w1[u] << kHalf);
    tile[1][ty + 4 * u][tx] = (w0[u] >> kHalf) | (w1[u] & ~kLow);
  }
  __syncthreads();
  Word *dw = reinterpret_cast<Word *>(dst + ofs);
  const uint32_t bl = tx % kTb, ah = tx / kTb;
#pragma unroll
  for (uint32_t u = 0; u < kTr / (4 * kRw); ++u) {
    const uint32_t aa = ty * kRw + ah + 4 * kRw * u, a = a0 + aa, b = b0 + bl;
    if (a < ra && b < cb) {
#pragma unroll
      for (uint32_t par = 0; par < 2; ++par) {
        Word *q = dw + b + (size_t)(2 * a + par) * cb;
        Word w = tile[par][bl][aa];
        if constexpr (ACC) {
          struct Two {
            T e[2];
          };
          const Two old = __builtin_bit_cast(Two, *q), add = __builtin_bit_cast(Two, w);
          Two r;
          r.e[0] = from_f32<T>(to_f32(old.e[0]) + to_f32(add.e[0]));
          r.e[1] = from_f32<T>(to_f32(old.e[1]) + to_f32(add.e[1]));
          w = __builtin_bit_cast(Word, r);
        }
        *q = w;
      }
    }
  }
}

// ---- permute_dims ---------------------------------------------------------------

struct PermuteArgs {
  uint32_t ndims;
  uint32_t x_dims[8];     // extents of x, dimension 0 first
  uint32_t y_strides[8];  // stride in y of x's dimension d
};

// FORWARD: y[j] = x[i]; otherwise gx[i] += gy[j], where j is i's position after the permutation.
template <typename T, bool FORWARD>
__global__ __launch_bounds__(kBlock) void permute_kernel(const T *src, T *dst, const PermuteArgs a, uint32_t volume) {
  const size_t ofs = (size_t)blockIdx.y * volume;
  for (uint32_t i = blockIdx.x * kBlock + threadIdx.x; i < volume; i += gridDim.x * kBlock) {
    uint32_t rest = i, j = 0;
    for (uint32_t d = 0; d < a.ndims; ++d) {
      const uint32_t c = rest % a.x_dims[d];
      rest /= a.x_dims[d];
      j += c * a.y_strides[d];
    }
    if constexpr (FORWARD) dst[ofs + j] = src[ofs + i];
    else put<T, true>(dst + ofs + i, to_f32(src[ofs + j]));
  }
}

// ---- flip and broadcast -----------------------------------------------------------

// dst[o][j][i] (=|+=) src[o][n-1-j][i]
template <typename T, bool ACC>
__global__ __launch_bounds__(kBlock) void flip_kernel(const T *src, T *dst, uint32_t base, uint32_t n, size_t total) {
  for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
    const size_t q = idx / base;
    const uint32_t i = (uint32_t)(idx - q * base);
    const size_t o = q / n;
    const uint32_t j = (uint32_t)(q - o * n);
    put<T, ACC>(dst + idx, to_f32(src[(o * n + (n - 1 - j)) * base + i]));
  }
}

// y[o][j][i] = x[o][i], j < size
template <typename T>
__global__ __launch_bounds__(kBlock) void broadcast_kernel(const T *x, T *y, uint32_t base, uint32_t size,
                                                            size_t total) {
  for (size_t idx = (size_t)blockIdx.x * kBlock + threadIdx.x; idx < total; idx += (size_t)gridDim.x * kBlock) {
    const size_t q = idx / base;
    const uint32_t i = (uint32_t)(idx - q * base);
    y[idx] = x[(q / size) * base + i];
  }
}

// ---- host side --------------------------------------------------------------------

inline dim3 grid2(size_t items, uint32_t ny, const phip_ctx *ctx) {
  unsigned gy = ny < 1 ? 1 : (ny > 65535u ? 65535u : ny);
  return dim3(blocks_for(items, ctx), gy);
}

template <typename T>
int copy_rows(phip_ctx *ctx, const void *src, void *dst, uint32_t span, uint32_t rows, uint64_t ss, uint64_t ds,
              uint32_t bs, uint64_t sbs, uint64_t dbs, int accumulate) {
  PHIP_ENTER(ctx);
  if (span == 0 || rows == 0 || bs == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  PHIP_REQUIRE((uint64_t)span * rows < (1ull << 32), "too many elements per sample: %u x %u", span, rows);
  PHIP_REQUIRE(dbs != 0 || bs == 1 || accumulate, "samples would overwrite each other (destination batch stride 0)");
  const uint32_t total = span * rows;
  const T *s = static_cast<const T *>(src);
  T *d = static_cast<T *>(dst);
  constexpr uint32_t N = Pack<T>::N;
  const bool packs = aligned16(src) && aligned16(dst) && span % N == 0 && ss % N == 0 && ds % N == 0 &&
                     sbs % N == 0 && dbs % N == 0;
  if (dbs == 0 && bs > 1) {
    hipLaunchKernelGGL(copy_rows_sum_kernel<T>, dim3(blocks_for(total, ctx)), dim3(kBlock), 0, ctx->stream, s, d,
                       span, total, (size_t)ss, (size_t)ds, bs, (size_t)sbs);
  } else if (packs) {
    if (accumulate) {
      hipLaunchKernelGGL((copy_rows_pack_kernel<T, true>), grid2(total / N, bs, ctx), dim3(kBlock), 0, ctx->stream, s,
                         d, span / N, total / N, (size_t)(ss / N), (size_t)(ds / N), bs, (size_t)(sbs / N),
                         (size_t)(dbs / N));
    } else {
      hipLaunchKernelGGL((copy_rows_pack_kernel<T, false>), grid2(total / N, bs, ctx), dim3(kBlock), 0, ctx->stream, s,
                         d, span / N, total / N, (size_t)(ss / N), (size_t)(ds / N), bs, (size_t)(sbs / N),
                         (size_t)(dbs / N));
    }
  } else if (accumulate) {
    hipLaunchKernelGGL((copy_rows_kernel<T, true>), grid2(total, bs, ctx), dim3(kBlock), 0, ctx->stream, s, d, span,
                       total, (size_t)ss, (size_t)ds, bs, (size_t)sbs, (size_t)dbs);
  } else {
    hipLaunchKernelGGL((copy_rows_kernel<T, false>), grid2(total, bs, ctx), dim3(kBlock), 0, ctx->stream, s, d, span,
                       total, (size_t)ss, (size_t)ds, bs, (size_t)sbs, (size_t)dbs);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// Index list of a launch; owns the device copy of a long list until released.
struct Ids {
  IdList list;
  void *device_block = nullptr;
};

// Checks every index against `limit` and makes the list reachable from a
// kernel.  A long list goes through a pool block and a blocking copy (the
// caller's array may disappear as soon as the call returns).
int prepare_ids(phip_ctx *ctx, const uint32_t *ids, uint32_t n_ids, uint32_t limit, Ids *out) {
  PHIP_REQUIRE(ids != nullptr && n_ids > 0, "no indices");
  for (uint32_t i = 0; i < n_ids; ++i)
    PHIP_REQUIRE(ids[i] < limit, "index %u (position %u) is out of range [0, %u)", ids[i], i, limit);
  out->list.device = nullptr;
  if (n_ids <= kInlineIds) {
    for (uint32_t i = 0; i < n_ids; ++i) out->list.inline_ids[i] = ids[i];
    return PHIP_OK;
  }
  int rc = phip_pool_alloc(ctx, sizeof(uint32_t) * (size_t)n_ids, &out->device_block, nullptr);
  if (rc != PHIP_OK) return rc;
  rc = phip_memcpy_h2d(ctx, out->device_block, ids, sizeof(uint32_t) * (size_t)n_ids);
  if (rc != PHIP_OK) {
    phip_pool_free(ctx, out->device_block);
    return rc;
  }
  out->list.device = static_cast<const uint32_t *>(out->device_block);
  return PHIP_OK;
}

// The stream is in order, so the block can go back to the pool as soon as
// the kernel that reads it has been enqueued.
void release_ids(phip_ctx *ctx, Ids *ids) {
  if (ids->device_block) phip_pool_free(ctx, ids->device_block);
  ids->device_block = nullptr;
}

template <typename T>
int pick(phip_ctx *ctx, bool forward, const void *src, const uint32_t *ids, uint32_t n_ids, void *dst, uint32_t base,
         uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(bx >= 1 && bs >= 1 && (bx == 1 || bx == bs) && (n_ids == 1 || n_ids == bs) &&
                   (bs == bx || bs == n_ids),
               "incompatible batch sizes: x %u, ids %u, y %u", bx, n_ids, bs);
  PHIP_REQUIRE(bs <= 65535u, "minibatch of %u exceeds the 65535 samples one launch covers", bs);
  if (base == 0 || n == 0 || outer == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  PHIP_REQUIRE((uint64_t)base * outer < (1ull << 32), "too many elements per sample");
  Ids list;
  const int rc = prepare_ids(ctx, ids, n_ids, n, &list);
  if (rc != PHIP_OK) return rc;
  const uint32_t sy = base * outer;
  const size_t sx = bx > 1 ? (size_t)sy * n : 0;
  const uint32_t si = n_ids > 1 ? 1 : 0;
  if (forward) {
    hipLaunchKernelGGL(pick_fw_kernel<T>, grid2(sy, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), base, n, sy, sx, si);
  } else if (sx != 0 || bs <= kOwnerSamples) {
    hipLaunchKernelGGL((pick_bw_kernel<T, true>), grid2(sy, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), base, n, sy, sx, si, bs);
  } else {
    hipLaunchKernelGGL((pick_bw_kernel<T, false>), grid2(sy, 1, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), base, n, sy, sx, si, bs);
  }
  release_ids(ctx, &list);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
int batch_pick(phip_ctx *ctx, bool forward, const void *src, const uint32_t *ids, uint32_t n_ids, void *dst,
               uint32_t volume, uint32_t bx) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(n_ids <= 65535u, "minibatch of %u exceeds the 65535 samples one launch covers", n_ids);
  if (volume == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  Ids list;
  const int rc = prepare_ids(ctx, ids, n_ids, bx, &list);
  if (rc != PHIP_OK) return rc;
  if (forward) {
    hipLaunchKernelGGL(batch_pick_fw_kernel<T>, grid2(volume, n_ids, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), volume);
  } else if (n_ids <= kOwnerSamples) {
    hipLaunchKernelGGL((batch_pick_bw_kernel<T, true>), grid2(volume, n_ids, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), volume, n_ids);
  } else {
    hipLaunchKernelGGL((batch_pick_bw_kernel<T, false>), grid2(volume, 1, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), list.list, static_cast<T *>(dst), volume, n_ids);
  }
  release_ids(ctx, &list);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

// dst (cols x rows) (=|+=) transpose of src (rows x cols), per sample
template <typename T>
int transpose(phip_ctx *ctx, bool accumulate, const void *src, void *dst, uint32_t rows, uint32_t cols, uint32_t bs) {
  PHIP_ENTER(ctx);
  if (rows == 0 || cols == 0 || bs == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  PHIP_REQUIRE(bs <= 65535u && (cols + kTr - 1) / kTr <= 65535u, "shape exceeds what one launch covers");
  {
    constexpr uint32_t kTb = sizeof(T) == 2 ? 64 : 32;
    if (rows % 2 == 0 && cols % 2 == 0 && reinterpret_cast<uintptr_t>(src) % (2 * sizeof(T)) == 0 &&
        reinterpret_cast<uintptr_t>(dst) % (2 * sizeof(T)) == 0 && (cols / 2 + kTb - 1) / kTb <= 65535u) {
      const dim3 pairs((rows / 2 + kTr - 1) / kTr, (cols / 2 + kTb - 1) / kTb, bs);
      if (accumulate) {
        hipLaunchKernelGGL((transpose_pairs_kernel<T, true>), pairs, dim3(kBlock), 0, ctx->stream,
                           static_cast<const T *>(src), static_cast<T *>(dst), rows, cols);
      } else {
        hipLaunchKernelGGL((transpose_pairs_kernel<T, false>), pairs, dim3(kBlock), 0, ctx->stream,
                           static_cast<const T *>(src), static_cast<T *>(dst), rows, cols);
      }
      PHIP_LAUNCH_CHECK();
      return PHIP_OK;
    }
  }
  const dim3 grid((rows + kTr - 1) / kTr, (cols + kTr - 1) / kTr, bs);
  if (accumulate) {
    hipLaunchKernelGGL((transpose_kernel<T, true>), grid, dim3(kBlock), 0, ctx->stream, static_cast<const T *>(src),
                       static_cast<T *>(dst), rows, cols);
  } else {
    hipLaunchKernelGGL((transpose_kernel<T, false>), grid, dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), static_cast<T *>(dst), rows, cols);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
int permute(phip_ctx *ctx, bool forward, const void *src, void *dst, uint32_t ndims, const uint32_t *dims,
            const uint32_t *perm, uint32_t bs) {
  PHIP_ENTER(ctx);
  PHIP_REQUIRE(ndims <= 8, "at most 8 dimensions, got %u", ndims);
  PHIP_REQUIRE(ndims == 0 || (dims != nullptr && perm != nullptr), "null pointer");
  PHIP_REQUIRE(bs <= 65535u, "minibatch of %u exceeds the 65535 samples one launch covers", bs);
  PermuteArgs a;
  a.ndims = ndims;
  uint64_t volume = 1;
  bool seen[8] = {false, false, false, false, false, false, false, false};
  uint32_t stride = 1;
  for (uint32_t i = 0; i < ndims; ++i) {  // y's dimension i is x's dimension perm[i]
    PHIP_REQUIRE(perm[i] < ndims && !seen[perm[i]], "not a permutation");
    seen[perm[i]] = true;
    a.y_strides[perm[i]] = stride;
    stride *= dims[perm[i]];
    a.x_dims[i] = dims[i];
    volume *= dims[i];
  }
  for (uint32_t i = ndims; i < 8; ++i) a.x_dims[i] = 1, a.y_strides[i] = 0;
  PHIP_REQUIRE(volume < (1ull << 32), "too many elements per sample");
  if (volume == 0 || bs == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  if (forward) {
    hipLaunchKernelGGL((permute_kernel<T, true>), grid2(volume, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), static_cast<T *>(dst), a, (uint32_t)volume);
  } else {
    hipLaunchKernelGGL((permute_kernel<T, false>), grid2(volume, bs, ctx), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), static_cast<T *>(dst), a, (uint32_t)volume);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
int flip(phip_ctx *ctx, bool accumulate, const void *src, void *dst, uint32_t base, uint32_t n, uint32_t outer) {
  PHIP_ENTER(ctx);
  const size_t total = (size_t)base * n * outer;
  if (total == 0) return PHIP_OK;
  PHIP_REQUIRE(src != nullptr && dst != nullptr, "null pointer");
  if (accumulate) {
    hipLaunchKernelGGL((flip_kernel<T, true>), dim3(blocks_for(total, ctx)), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), static_cast<T *>(dst), base, n, total);
  } else {
    hipLaunchKernelGGL((flip_kernel<T, false>), dim3(blocks_for(total, ctx)), dim3(kBlock), 0, ctx->stream,
                       static_cast<const T *>(src), static_cast<T *>(dst), base, n, total);
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <typename T>
int broadcast(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t size, uint32_t outer) {
  PHIP_ENTER(ctx);
  const size_t total = (size_t)base * size * outer;
  if (total == 0) return PHIP_OK;
  PHIP_REQUIRE(x != nullptr && y != nullptr, "null pointer");
  hipLaunchKernelGGL(broadcast_kernel<T>, dim3(blocks_for(total, ctx)), dim3(kBlock), 0, ctx->stream,
                     static_cast<const T *>(x), static_cast<T *>(y), base, size, total);
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace
}  // namespace phip

using namespace phip;

extern "C" {

#define PHIP_EXPORT_INDEXING(SUF, T, CPTR, PTR)                                                                    \
  int phip_copy_rows_##SUF(phip_ctx *ctx, CPTR src, PTR dst, uint32_t span, uint32_t rows, uint64_t src_stride,    \
                           uint64_t dst_stride, uint32_t bs, uint64_t src_bstride, uint64_t dst_bstride,           \
                           int accumulate) {                                                                       \
    return copy_rows<T>(ctx, src, dst, span, rows, src_stride, dst_stride, bs, src_bstride, dst_bstride,           \
                        accumulate);                                                                               \
  }                                                                                                                \
  int phip_pick_fw_##SUF(phip_ctx *ctx, CPTR x, const uint32_t *ids, uint32_t n_ids, PTR y, uint32_t base,         \
                         uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs) {                                   \
    return pick<T>(ctx, true, x, ids, n_ids, y, base, n, outer, bx, bs);                                           \
  }                                                                                                                \
  int phip_pick_bw_##SUF(phip_ctx *ctx, CPTR gy, const uint32_t *ids, uint32_t n_ids, PTR gx, uint32_t base,       \
                         uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs) {                                   \
    return pick<T>(ctx, false, gy, ids, n_ids, gx, base, n, outer, bx, bs);                                        \
  }                                                                                                                \
  int phip_batch_pick_fw_##SUF(phip_ctx *ctx, CPTR x, const uint32_t *ids, uint32_t n_ids, PTR y, uint32_t volume, \
                               uint32_t bx) {                                                                      \
    return batch_pick<T>(ctx, true, x, ids, n_ids, y, volume, bx);                                                 \
  }                                                                                                                \
  int phip_batch_pick_bw_##SUF(phip_ctx *ctx, CPTR gy, const uint32_t *ids, uint32_t n_ids, PTR gx,                \
                               uint32_t volume, uint32_t bx) {                                                     \
    return batch_pick<T>(ctx, false, gy, ids, n_ids, gx, volume, bx);                                              \
  }                                                                                                                \
  int phip_transpose_fw_##SUF(phip_ctx *ctx, CPTR x, PTR y, uint32_t rows, uint32_t cols, uint32_t bs) {           \
    return transpose<T>(ctx, false, x, y, rows, cols, bs);                                                         \
  }                                                                                                                \
  int phip_transpose_bw_##SUF(phip_ctx *ctx, CPTR gy, PTR gx, uint32_t rows, uint32_t cols, uint32_t bs) {         \
    /* gy is cols x rows; its transpose is added to the rows x cols gx */                                          \
    return transpose<T>(ctx, true, gy, gx, cols, rows, bs);                                                        \
  }                                                                                                                \
  int phip_permute_dims_fw_##SUF(phip_ctx *ctx, CPTR x, PTR y, uint32_t ndims, const uint32_t *dims,               \
                                 const uint32_t *perm, uint32_t bs) {                                              \
    return permute<T>(ctx, true, x, y, ndims, dims, perm, bs);                                                     \
  }                                                                                                                \
  int phip_permute_dims_bw_##SUF(phip_ctx *ctx, CPTR gy, PTR gx, uint32_t ndims, const uint32_t *dims,             \
                                 const uint32_t *perm, uint32_t bs) {                                              \
    return permute<T>(ctx, false, gy, gx, ndims, dims, perm, bs);                                                  \
  }                                                                                                                \
  int phip_flip_fw_##SUF(phip_ctx *ctx, CPTR x, PTR y, uint32_t base, uint32_t n, uint32_t outer) {                \
    return flip<T>(ctx, false, x, y, base, n, outer);                                                              \
  }                                                                                                                \
  int phip_flip_bw_##SUF(phip_ctx *ctx, CPTR gy, PTR gx, uint32_t base, uint32_t n, uint32_t outer) {              \
    return flip<T>(ctx, true, gy, gx, base, n, outer);                                                             \
  }                                                                                                                \
  int phip_broadcast_fw_##SUF(phip_ctx *ctx, CPTR x, PTR y, uint32_t base, uint32_t size, uint32_t outer) {        \
    return broadcast<T>(ctx, x, y, base, size, outer);                                                             \
  }

PHIP_EXPORT_INDEXING(f32, float, const float *, float *)
PHIP_EXPORT_INDEXING(f16, f16_t, const void *, void *)
PHIP_EXPORT_INDEXING(bf16, bf16_t, const void *, void *)

#undef PHIP_EXPORT_INDEXING

}  // extern "C"
