// GEMM for 16-bit storage (fp16 or bf16) with fp32 accumulation on the gfx950
// matrix cores (v_mfma_f32_32x32x16_f16 / _bf16).
//
// Same workgroup structure as the fp32 kernel, but the matrix instruction
// wants 8 consecutive k values per lane, so the common LDS layout is [m][k] /
// [n][k]: an operand that is contiguous along k in memory is copied with
// 16-byte accesses, one that is contiguous along m or n is transposed while it
// is written to LDS.  Results are rounded to the storage type once, after the
// whole K range has been accumulated in fp32; `C += ...` reads C, adds in fp32
// and rounds once.  When a long K meets few output tiles, the K range is cut
// between workgroups that leave fp32 partial tiles in scratch memory, and a
// second launch adds them in order, so the one rounding (and a result that
// does not depend on scheduling) is kept.
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int kPadH = 8;  // 16-bit elements appended to every LDS row

struct GemmArgsH {
  const uint16_t *A;
  const uint16_t *B;
  uint16_t *C;
  int M, N, K;
  long lda, ldb, ldc;
  long sA, sB, sC;
  long rA, rB;
  int tiles_m, tiles_n;
  int ktiles_per_r;
  int total_ktiles;
  int accumulate;
  int vec_c;        // C is 16-byte aligned with M and ldc multiples of 8: 16-byte C accesses
  int splits;       // workgroups that share one C tile, each taking a K range
  float *partial;   // splits > 1: fp32 tiles, element (m, n) of (sample z, range s) at ((z*splits + s)*N + n)*M + m
};

__device__ inline int xcd_remap(int bid, int total) {
  constexpr int kXcds = 8;
  const int xcd = bid % kXcds;
  const int idx = bid / kXcds;
  const int q = total / kXcds, rem = total % kXcds;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

union Pack8 {
  uint4v v;
  uint16_t h[8];
};

// Operand contiguous along k: element (x, k) at base[k + x*ld]; LDS rows are x.
template <int BX, int BK, int V>
struct LoaderKContigH {
  static constexpr int kVecPerX = BK / V;
  static constexpr int kTotal = BX * BK / V;
  static constexpr int kIters = (kTotal + kThreads - 1) / kThreads;
  Pack8 regs[kIters];

  __device__ inline void load(const uint16_t *base, long ld, int x0, int X, int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      const int x = x0 + v / kVecPerX;
      const int k = k0 + (v % kVecPerX) * V;
      const bool live = (kTotal % kThreads == 0 || v < kTotal) && x < X;
      if (V == 8 && live && k + 8 <= K) {
        regs[i].v = *reinterpret_cast<const uint4v *>(base + k + (long)x * ld);
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) regs[i].h[e] = (live && k + e < K) ? base[k + e + (long)x * ld] : (uint16_t)0;
      }
    }
  }

  __device__ inline void store(uint16_t *lds, int tid) const {
    constexpr int S = BK + kPadH;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      if (kTotal % kThreads != 0 && v >= kTotal) continue;
      uint16_t *p = lds + (v / kVecPerX) * S + (v % kVecPerX) * V;
      if (V == 8) {
        *reinterpret_cast<uint4v *>(p) = regs[i].v;
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) p[e] = regs[i].h[e];
      }
    }
  }
};

// Operand contiguous along x: element (x, k) at base[x + k*ld]; transposed on
// its way into LDS.
template <int BX, int BK, int V>
struct LoaderXContigH {
  static constexpr int kVecPerRow = BX / V;
  static constexpr int kTotal = BX * BK / V;
  static constexpr int kIters = (kTotal + kThreads - 1) / kThreads;
  Pack8 regs[kIters];

  __device__ inline void load(const uint16_t *base, long ld, int x0, int X, int k0, int K, int tid) {
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      const int k = k0 + v / kVecPerRow;
      const int x = x0 + (v % kVecPerRow) * V;
      const bool live = (kTotal % kThreads == 0 || v < kTotal) && k < K;
      if (V == 8 && live && x + 8 <= X) {
        regs[i].v = *reinterpret_cast<const uint4v *>(base + x + (long)k * ld);
      } else {
#pragma unroll
        for (int e = 0; e < V; ++e) regs[i].h[e] = (live && x + e < X) ? base[x + e + (long)k * ld] : (uint16_t)0;
      }
    }
  }

  __device__ inline void store(uint16_t *lds, int tid) const {
    constexpr int S = BK + kPadH;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      if (kTotal % kThreads != 0 && v >= kTotal) continue;
      uint16_t *p = lds + ((v % kVecPerRow) * V) * S + v / kVecPerRow;
#pragma unroll
      for (int e = 0; e < V; ++e) p[e * S] = regs[i].h[e];
    }
  }
};

template <bool KMAJOR, int BX, int BK, int V>
struct LoaderSelectH {
  typedef LoaderXContigH<BX, BK, V> type;
};
template <int BX, int BK, int V>
struct LoaderSelectH<true, BX, BK, V> {
  typedef LoaderKContigH<BX, BK, V> type;
};

template <bool BF16>
__device__ inline float16v mfma_32x32x16(uint4v a, uint4v b, float16v c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8v, a), __builtin_bit_cast(bf8v, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, a), __builtin_bit_cast(half8v, b), c, 0, 0, 0);
  }
}

template <bool BF16>
__device__ inline float load_c(const uint16_t *p) {
  if constexpr (BF16) {
    bf16_t t; t.bits = *p; return to_f32(t);
  } else {
    return to_f32(__builtin_bit_cast(f16_t, *p));
  }
}

template <bool BF16>
__device__ inline uint16_t round_c(float x) {
  if constexpr (BF16) {
    return from_f32<bf16_t>(x).bits;
  } else {
    return __builtin_bit_cast(uint16_t, from_f32<f16_t>(x));
  }
}

template <int BM, int BN, int BK, int WGM, int WGN, int WGK, bool A_KMAJOR, bool B_KMAJOR, int VA, int VB, bool BF16>
__global__ __launch_bounds__(kThreads) void gemm_h16_kernel(const GemmArgsH g) {
  static_assert(WGM * WGN * WGK == 4, "four wavefronts per workgroup");
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile is made of 32x32 blocks");
  static_assert((BK / 16) % WGK == 0, "k steps must divide among the k-split waves");
  constexpr int S = BK + kPadH;  // LDS row stride in 16-bit elements
  constexpr int kStageA = BM * S, kStageB = BN * S;
  constexpr int kTileBytes = 2 * (kStageA + kStageB) * 2;
  constexpr int kReduceBytes = WGK > 1 ? 4 * TM * TN * 16 * 64 * 4 : 0;
  // write-out through LDS: per wavefront one 32-column block of its tile in fp32, [column][row]
  constexpr int kColPitch = WTM + 8;  // floats; the pad staggers the columns over the banks
  constexpr int kEmitBytes = WGK == 1 ? 4 * 32 * kColPitch * 4 : 0;
  constexpr int kLdsMax1 = kTileBytes > kReduceBytes ? kTileBytes : kReduceBytes;
  constexpr int kLdsBytes = kLdsMax1 > kEmitBytes ? kLdsMax1 : kEmitBytes;
  __shared__ __attribute__((aligned(16))) unsigned char lds_raw[kLdsBytes];
  uint16_t *lds = reinterpret_cast<uint16_t *>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wk = wave % WGK;
  const int wm = (wave / WGK) % WGM;
  const int wn = (wave / WGK) / WGM;

  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;

  typename LoaderSelectH<A_KMAJOR, BM, BK, VA>::type la;
  typename LoaderSelectH<B_KMAJOR, BN, BK, VB>::type lb;

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  auto fetch = [&](int kt) {
    const int r = kt / g.ktiles_per_r;
    const int k0 = (kt - r * g.ktiles_per_r) * BK;
    la.load(Az + (long)r * g.rA, g.lda, m0, g.M, k0, g.K, tid);
    lb.load(Bz + (long)r * g.rB, g.ldb, n0, g.N, k0, g.K, tid);
  };

  // K tiles [kt_begin, kt_end) belong to this workgroup
  const int kt_begin = (int)((long)split * g.total_ktiles / g.splits);
  const int kt_end = (int)((long)(split + 1) * g.total_ktiles / g.splits);
  if (kt_end > kt_begin) {
    fetch(kt_begin);
    la.store(lds, tid);
    lb.store(lds + 2 * kStageA, tid);
  }
  __syncthreads();

  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int stage = (kt - kt_begin) & 1;
    const bool more = kt + 1 < kt_end;
    if (more) fetch(kt + 1);

    // lane l supplies row l%32 and the 8 k values starting at 8*(l/32)
    const uint16_t *as = lds + stage * kStageA + (wm * WTM + (lane & 31)) * S + 8 * (lane >> 5);
    const uint16_t *bs = lds + 2 * kStageA + stage * kStageB + (wn * WTN + (lane & 31)) * S + 8 * (lane >> 5);
#pragma unroll
    for (int s = 0; s < BK / 16 / WGK; ++s) {
      const int kk = (s * WGK + wk) * 16;
      uint4v af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = *reinterpret_cast<const uint4v *>(as + i * 32 * S + kk);
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[j] = *reinterpret_cast<const uint4v *>(bs + j * 32 * S + kk);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = mfma_32x32x16<BF16>(bf[j], af[i], acc[i][j]);
    }

    if (more) {
      la.store(lds + (stage ^ 1) * kStageA, tid);
      lb.store(lds + 2 * kStageA + (stage ^ 1) * kStageB, tid);
    }
    __syncthreads();
  }

  uint16_t *Cz = g.C + (long)z * g.sC;
  float *Pz = g.partial + ((long)z * g.splits + split) * g.M * g.N;
  const int cm = m0 + wm * WTM + (lane & 31);
  const int cn = n0 + wn * WTN + 4 * (lane >> 5);

  if (WGK > 1) {
    float *red = reinterpret_cast<float *>(lds_raw);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          red[(((wave * TM + i) * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
    __syncthreads();
    const int group = wave / WGK;
    constexpr int kPer = 16 / WGK;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
          const int v = wk * kPer + q;
          float s = 0.0f;
#pragma unroll
          for (int w = 0; w < WGK; ++w)
            s += red[((((group * WGK + w) * TM + i) * TN + j) * 16 + v) * 64 + lane];
          const int m = cm + i * 32;
          const int n = cn + j * 32 + 8 * (v / 4) + (v % 4);
          if (m < g.M && n < g.N) {
            if (g.splits > 1) {
              Pz[m + (long)n * g.M] = s;
            } else {
              uint16_t *p = Cz + m + (long)n * g.ldc;
              *p = round_c<BF16>(g.accumulate ? load_c<BF16>(p) + s : s);
            }
          }
        }
  } else if (g.vec_c && g.splits == 1) {
    // The matrix instruction leaves a lane with one row and 16 columns of each 32 x 32 block; C wants
    // 8 consecutive rows of a column per lane (16 bytes).  Each 32-column block of the wave's tile is
    // turned through an LDS area of the wave's own: written the way the accumulators lie, read back 8
    // rows at a time.  M is a multiple of 8: a lane's 8 rows are inside or outside together.
    float *area = reinterpret_cast<float *>(lds_raw) + wave * 32 * kColPitch;
    constexpr int kLanesPerCol = WTM / 8;           // 4 or 8 lanes cover a column of the tile
    constexpr int kColsPerPass = 64 / kLanesPerCol;
    const int r0 = 8 * (lane % kLanesPerCol), c_in_pass = lane / kLanesPerCol;
    const int m = m0 + wm * WTM + r0;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          area[(8 * (v / 4) + 4 * (lane >> 5) + (v % 4)) * kColPitch + 32 * i + (lane & 31)] = acc[i][j][v];
      // the area belongs to this wave alone: its own LDS accesses stay in order
#pragma unroll
      for (int pass = 0; pass < 32 / kColsPerPass; ++pass) {
        const int c = pass * kColsPerPass + c_in_pass;
        const int n = n0 + wn * WTN + j * 32 + c;
        const float4 lo = *reinterpret_cast<const float4 *>(area + c * kColPitch + r0);
        const float4 hi = *reinterpret_cast<const float4 *>(area + c * kColPitch + r0 + 4);
        if (m < g.M && n < g.N) {
          uint16_t *p = Cz + m + (long)n * g.ldc;
          float f[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
          Pack8 out;
          if (g.accumulate) {
            Pack8 old;
            old.v = *reinterpret_cast<const uint4v *>(p);
#pragma unroll
            for (int e = 0; e < 8; ++e) f[e] += load_c<BF16>(&old.h[e]);
          }
#pragma unroll
          for (int e = 0; e < 8; ++e) out.h[e] = round_c<BF16>(f[e]);
          *reinterpret_cast<uint4v *>(p) = out.v;
        }
      }
    }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = cm + i * 32;
          const int n = cn + j * 32 + 8 * (v / 4) + (v % 4);
          if (m < g.M && n < g.N) {
            const float s = acc[i][j][v];
            if (g.splits > 1) {
              Pz[m + (long)n * g.M] = s;
            } else {
              uint16_t *p = Cz + m + (long)n * g.ldc;
              *p = round_c<BF16>(g.accumulate ? load_c<BF16>(p) + s : s);
            }
          }
        }
  }
}

// C (=|+=) the sum, in order, of the `splits` fp32 partial tiles of every element; one rounding.
template <bool BF16>
__global__ __launch_bounds__(kThreads) void finish_split_h16_kernel(const float *partial, uint16_t *C, int M, int N,
                                                                    long ldc, long sC, int batch, int splits,
                                                                    int accumulate) {
  const long per = (long)M * N;
  const long total = per * batch;
  for (long idx = (long)blockIdx.x * kThreads + threadIdx.x; idx < total; idx += (long)gridDim.x * kThreads) {
    const long z = idx / per, e = idx - z * per;
    const float *p = partial + z * splits * per + e;
    float s = p[0];
    for (int r = 1; r < splits; ++r) s += p[r * per];
    uint16_t *c = C + z * sC + (e % M) + (e / M) * ldc;
    *c = round_c<BF16>(accumulate ? load_c<BF16>(c) + s : s);
  }
}

template <int BM, int BN, int BK, int WGM, int WGN, int WGK, bool BF16>
int launch_tile_h(phip_ctx *ctx, const Gemm &p, GemmArgsH a, bool vec_a, bool vec_b, bool may_split = false) {
  a.tiles_m = (p.M + BM - 1) / BM;
  a.tiles_n = (p.N + BN - 1) / BN;
  a.ktiles_per_r = (p.K + BK - 1) / BK;
  a.total_ktiles = a.ktiles_per_r * p.rbatch;
  const long tiles = (long)a.tiles_m * a.tiles_n * p.batch;
  // Few tiles over a long K (the second launch has to pay for itself: at least 32 K tiles): cut K so
  // that about two workgroups per compute unit run (never more workgroups than places, at least
  // eight K tiles each, at most 64 MiB of partial tiles).
  long splits = 1;
  if (may_split && tiles > 0 && a.total_ktiles >= 32) {
    splits = 2L * ctx->prop.multiProcessorCount / tiles;
    if (splits > a.total_ktiles / 8) splits = a.total_ktiles / 8;
    const long per_split = 4L * p.M * p.N * p.batch;
    if (per_split > 0 && splits > (64L << 20) / per_split) splits = (64L << 20) / per_split;
    if (splits < 1) splits = 1;
  }
  a.splits = (int)splits;
  a.partial = nullptr;
  void *block = nullptr;
  if (splits > 1) {
    const int rc = scratch_alloc(ctx, (size_t)(4L * p.M * p.N * p.batch * splits), &block);
    if (rc != PHIP_OK) return rc;
    a.partial = static_cast<float *>(block);
  }
  const long grid = tiles * splits;
  if (grid > 0x7fffffffL) {
    if (block) scratch_free(ctx, block);
    return fail(PHIP_ERR_INVALID_ARGUMENT, "matmul problem too large for one launch");
  }

#define PHIP_LAUNCH_V(AK, BKM, VVA, VVB)                                                                          \
  hipLaunchKernelGGL((gemm_h16_kernel<BM, BN, BK, WGM, WGN, WGK, AK, BKM, VVA, VVB, BF16>), dim3((unsigned)grid),  \
                     dim3(kThreads), 0, ctx->stream, a)
#define PHIP_LAUNCH(AK, BKM)                                                                                     \
  do {                                                                                                           \
    if (vec_a && vec_b) PHIP_LAUNCH_V(AK, BKM, 8, 8);                                                            \
    else if (vec_a) PHIP_LAUNCH_V(AK, BKM, 8, 1);                                                                \
    else if (vec_b) PHIP_LAUNCH_V(AK, BKM, 1, 8);                                                                \
    else PHIP_LAUNCH_V(AK, BKM, 1, 1);                                                                           \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) {
    PHIP_LAUNCH(false, true);
  } else if (!p.a_kmajor && !p.b_kmajor) {
    PHIP_LAUNCH(false, false);
  } else if (p.a_kmajor && p.b_kmajor) {
    PHIP_LAUNCH(true, true);
  } else {
    if (block) scratch_free(ctx, block);
    return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
  }
#undef PHIP_LAUNCH_V
#undef PHIP_LAUNCH
  if (splits > 1) {
    const long total = (long)p.M * p.N * p.batch;
    long blocks = (total + kThreads - 1) / kThreads;
    const long cap = 8L * ctx->prop.multiProcessorCount;
    if (blocks > cap) blocks = cap;
    hipLaunchKernelGGL((finish_split_h16_kernel<BF16>), dim3((unsigned)blocks), dim3(kThreads), 0, ctx->stream,
                       a.partial, a.C, p.M, p.N, p.ldc, p.sC, p.batch, (int)splits, a.accumulate);
    note_kernel(ctx, "h16_finish_split");
    scratch_free(ctx, block);  // the stream is in order: the block may be handed out again behind these launches
  }
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

template <bool BF16>
int gemm_h16_typed(phip_ctx *ctx, const Gemm &p) {
  GemmArgsH a;
  a.A = static_cast<const uint16_t *>(p.A);
  a.B = static_cast<const uint16_t *>(p.B);
  a.C = static_cast<uint16_t *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.accumulate = p.accumulate ? 1 : 0;
  a.vec_c = reinterpret_cast<uintptr_t>(p.C) % 16 == 0 && p.M % 8 == 0 && p.ldc % 8 == 0 && p.sC % 8 == 0;

  // 16-byte loads per operand: aligned rows (the loaders check the ragged edge per vector)
  const bool vec_a = rows_aligned16(p.A, 8, p.lda, p.sA, p.rA), vec_b = rows_aligned16(p.B, 8, p.ldb, p.sB, p.rB);

  const int cus = ctx->prop.multiProcessorCount;
  auto tiles = [&](int bm, int bn) {
    return (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batch;
  };
  if (tiles(128, 128) >= cus) {
    note_kernel(ctx, "h16_staged128");
    return launch_tile_h<128, 128, 32, 2, 2, 1, BF16>(ctx, p, a, vec_a, vec_b);
  }
  if (tiles(64, 64) >= cus) {
    note_kernel(ctx, "h16_staged64");
    return launch_tile_h<64, 64, 32, 2, 2, 1, BF16>(ctx, p, a, vec_a, vec_b);
  }
  note_kernel(ctx, "h16_staged32");
  return launch_tile_h<32, 32, 64, 1, 1, 4, BF16>(ctx, p, a, vec_a, vec_b, true);
}

}  // namespace

int gemm_h16(phip_ctx *ctx, const Gemm &p, Elem elem) {
  if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return PHIP_OK;
  bool handled = false;
  int rc = gemm_h16_skinny(ctx, p, elem, &handled);
  if (rc != PHIP_OK || handled) return rc;
  rc = gemm_h16_big(ctx, p, elem, &handled);
  if (rc != PHIP_OK || handled) return rc;
  return elem == Elem::BF16 ? gemm_h16_typed<true>(ctx, p) : gemm_h16_typed<false>(ctx, p);
}

}  // namespace phip
