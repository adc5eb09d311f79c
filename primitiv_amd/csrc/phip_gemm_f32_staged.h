// fp32 GEMM on the gfx950 matrix cores (v_mfma_f32_32x32x2_f32).
//
// One workgroup of 256 threads (4 wavefronts) owns a BM x BN tile of C and
// walks K in steps of BK.  Operand tiles are staged through LDS in a common
// [k][m] / [k][n] layout whatever their layout in memory: an operand that is
// contiguous along m (or n) is copied row by row with 16-byte accesses, one
// that is contiguous along k is transposed while it is written to LDS.  The
// three products of primitiv's matmul (a.b, gy.b^T, a^T.gy) are therefore the
// same inner loop behind different loaders, and no transposed copy of any
// operand is ever materialised.
//
// Two LDS stages: the loads of tile t+1 are issued before the matrix
// instructions of tile t and written to the other stage afterwards, with one
// barrier per tile.
#ifndef PHIP_GEMM_F32_STAGED_H_
#define PHIP_GEMM_F32_STAGED_H_

#include "phip_gemm_f32_common.h"

namespace phip {
namespace {

// The loaders below are branch-free so that the global loads of the next tile
// can stay in flight while the matrix instructions of the current one run: a
// vector that falls outside the matrix is read from the matrix origin instead
// (always a valid address) and replaced by zeros when it is written to LDS.
// With V == 4 the leading dimension is a multiple of 4, and so is the extent
// along the contiguous axis (dense column-major: it IS the leading dimension),
// so a vector is either entirely inside or entirely outside.

// Tile of an operand that is contiguous along x (m or n): element (x, k) at
// base[x + k*ld].  Rows of the LDS tile are k.
template <int BX, int BK, int V>
struct LoaderXContig {
  static constexpr int kVecPerRow = BX / V;
  static constexpr int kTotal = BX * BK / V;
  static constexpr int kIters = (kTotal + kThreads - 1) / kThreads;
  float regs[kIters][V];
  unsigned ok;

  __device__ inline void load(const float *base, long ld, int x0, int X, int k0, int K, int tid) {
    ok = 0;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      const int k = k0 + v / kVecPerRow;
      const int x = x0 + (v % kVecPerRow) * V;
      const bool in = (kTotal % kThreads == 0 || v < kTotal) && k < K && x < X;
      const float *p = in ? base + x + (long)k * ld : base;
      ok |= (in ? 1u : 0u) << i;
      if constexpr (V == 4) {
        const float4v t = *reinterpret_cast<const float4v *>(p);
        regs[i][0] = t.x; regs[i][1 % V] = t.y; regs[i][2 % V] = t.z; regs[i][3 % V] = t.w;
      } else {
        regs[i][0] = *p;
      }
    }
  }

  __device__ inline void store(float *lds, int tid) const {
    constexpr int S = BX + kPad;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      if (kTotal % kThreads != 0 && v >= kTotal) continue;
      const bool in = (ok >> i) & 1u;
      float *p = lds + (v / kVecPerRow) * S + (v % kVecPerRow) * V;
      if constexpr (V == 4) {
        float4v t = {in ? regs[i][0] : 0.0f, in ? regs[i][1 % V] : 0.0f, in ? regs[i][2 % V] : 0.0f,
                     in ? regs[i][3 % V] : 0.0f};
        *reinterpret_cast<float4v *>(p) = t;
      } else {
        p[0] = in ? regs[i][0] : 0.0f;
      }
    }
  }
};

// Tile of an operand that is contiguous along k: element (x, k) at
// base[k + x*ld].  Transposed on its way into LDS.
template <int BX, int BK, int V>
struct LoaderKContig {
  static constexpr int kVecPerX = BK / V;
  static constexpr int kTotal = BX * BK / V;
  static constexpr int kIters = (kTotal + kThreads - 1) / kThreads;
  float regs[kIters][V];
  unsigned ok;

  __device__ inline void load(const float *base, long ld, int x0, int X, int k0, int K, int tid) {
    ok = 0;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      const int x = x0 + v / kVecPerX;
      const int k = k0 + (v % kVecPerX) * V;
      const bool in = (kTotal % kThreads == 0 || v < kTotal) && x < X && k < K;
      const float *p = in ? base + k + (long)x * ld : base;
      ok |= (in ? 1u : 0u) << i;
      if constexpr (V == 4) {
        const float4v t = *reinterpret_cast<const float4v *>(p);
        regs[i][0] = t.x; regs[i][1 % V] = t.y; regs[i][2 % V] = t.z; regs[i][3 % V] = t.w;
      } else {
        regs[i][0] = *p;
      }
    }
  }

  __device__ inline void store(float *lds, int tid) const {
    constexpr int S = BX + kPad;
#pragma unroll
    for (int i = 0; i < kIters; ++i) {
      const int v = tid + i * kThreads;
      if (kTotal % kThreads != 0 && v >= kTotal) continue;
      const bool in = (ok >> i) & 1u;
      float *p = lds + ((v % kVecPerX) * V) * S + v / kVecPerX;
#pragma unroll
      for (int e = 0; e < V; ++e) p[e * S] = in ? regs[i][e] : 0.0f;
    }
  }
};

template <bool KMAJOR, int BX, int BK, int V>
struct LoaderSelect {
  typedef LoaderXContig<BX, BK, V> type;
};
template <int BX, int BK, int V>
struct LoaderSelect<true, BX, BK, V> {
  typedef LoaderKContig<BX, BK, V> type;
};

// LDS floats one workgroup needs: two stages of both operand tiles, reused for
// the sum of the k-split wavefronts' tiles.
template <int BM, int BN, int BK, int WGM, int WGN, int WGK>
constexpr int staged_lds_floats() {
  constexpr int tile = 2 * (BK * (BM + kPad) + BK * (BN + kPad));
  constexpr int reduce = WGK > 1 ? 4 * (BM / WGM / 32) * (BN / WGN / 32) * 16 * 64 : 0;
  return tile > reduce ? tile : reduce;
}

// WGM x WGN x WGK wavefronts: WGM*WGN of them tile the BM x BN block, WGK of
// them share each wave tile and split the k steps of every K tile between
// themselves (their partial tiles are summed through LDS at the end).
// One workgroup's work: workgroup `bid` of the `nblk` that share the problem
// `g`; `lds` holds staged_lds_floats<...>() floats, 16-byte aligned.
template <int BM, int BN, int BK, int WGM, int WGN, int WGK, bool A_KMAJOR, bool B_KMAJOR, int VA, int VB>
__device__ inline void staged_tile(const GemmArgs &g, float *lds, int bid, int nblk) {
  static_assert(WGM * WGN * WGK == 4, "four wavefronts per workgroup");
  constexpr int WTM = BM / WGM, WTN = BN / WGN;
  constexpr int TM = WTM / 32, TN = WTN / 32;
  static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile is made of 32x32 blocks");
  static_assert((BK / 2) % WGK == 0, "k steps must divide among the k-split waves");
  constexpr int SA = BM + kPad, SB = BN + kPad;
  constexpr int kStageA = BK * SA, kStageB = BK * SB;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wk = wave % WGK;
  const int wm = (wave / WGK) % WGM;
  const int wn = (wave / WGK) / WGM;

  int t = xcd_remap(bid, nblk);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const int kt_begin = (int)((long)split * g.total_ktiles / g.splits);
  const int kt_end = (int)((long)(split + 1) * g.total_ktiles / g.splits);

  const float *Az = g.A + (long)z * g.sA;
  const float *Bz = g.B + (long)z * g.sB;

  typename LoaderSelect<A_KMAJOR, BM, BK, VA>::type la;
  typename LoaderSelect<B_KMAJOR, BN, BK, VB>::type lb;

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

  if (kt_begin < kt_end) {
    fetch(kt_begin);
    la.store(lds, tid);
    lb.store(lds + 2 * kStageA, tid);
  }
  __syncthreads();

  for (int kt = kt_begin; kt < kt_end; ++kt) {
    const int stage = (kt - kt_begin) & 1;
    const bool more = kt + 1 < kt_end;
    if (more) fetch(kt + 1);

    const float *as = lds + stage * kStageA + wm * WTM + (lane & 31);
    const float *bs = lds + 2 * kStageA + stage * kStageB + wn * WTN + (lane & 31);
    const int khalf = lane >> 5;
#pragma unroll
    for (int s = 0; s < BK / 2 / WGK; ++s) {
      const int kk = (s * WGK + wk) * 2 + khalf;
      float af[TM], bf[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) af[i] = as[kk * SA + i * 32];
#pragma unroll
      for (int j = 0; j < TN; ++j) bf[j] = bs[kk * SB + j * 32];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          // rows of the instruction's result follow n, its columns follow m
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j], af[i], acc[i][j], 0, 0, 0);
    }

    if (more) {
      la.store(lds + (stage ^ 1) * kStageA, tid);
      lb.store(lds + 2 * kStageA + (stage ^ 1) * kStageB, tid);
    }
    __syncthreads();
  }

  // Lane l of result register v holds C(m, n) with m = l % 32 and
  // n = 8*(v/4) + 4*(l/32) + v%4 inside its 32x32 block.
  float *Cz = g.C + (long)z * g.sC;
  const int row0 = m0 + wm * WTM, col0 = n0 + wn * WTN;
  const bool interior = m0 + BM <= g.M && n0 + BN <= g.N;

  if (WGK > 1) {
    // Sum the k-split waves' tiles: every wave parks its registers in LDS,
    // then wave w reduces and writes registers [4w, 4w+4) of each block.
    float *red = lds;  // the tile stages are no longer read (barrier above)
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          red[(((wave * TM + i) * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
    __syncthreads();
    const int group = wave / WGK;  // waves of one group share a wave tile
    constexpr int kPer = 16 / WGK;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        float vals[kPer];
        int ns[kPer];
#pragma unroll
        for (int q = 0; q < kPer; ++q) {
          const int v = wk * kPer + q;
          float s = 0.0f;
#pragma unroll
          for (int w = 0; w < WGK; ++w)
            s += red[((((group * WGK + w) * TM + i) * TN + j) * 16 + v) * 64 + lane];
          vals[q] = s;
          ns[q] = 8 * (v / 4) + (v % 4);
        }
        emit_c<kPer>(Cz, g.ldc, row0 + i * 32, col0 + j * 32, lane, g.M, g.N, interior, ns, vals, g.atomic,
                     g.accumulate);
      }
  } else {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        float vals[16];
        int ns[16];
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          vals[v] = acc[i][j][v];
          ns[v] = 8 * (v / 4) + (v % 4);
        }
        emit_c<16>(Cz, g.ldc, row0 + i * 32, col0 + j * 32, lane, g.M, g.N, interior, ns, vals, g.atomic,
                   g.accumulate);
      }
  }
}

// Which tile shape runs a problem, and its launch geometry.
enum class StagedShape {
  k128x128x16,  // 2 x 2 wavefronts, four workgroups per CU
  k64x64x32,    // 2 x 2 wavefronts, two workgroups per CU
  k32x32x64,    // four wavefronts split the k steps of one 32 x 32 tile
};

struct StagedPlan {
  GemmArgs a;  // complete
  StagedShape shape;
  bool vec_a, vec_b;
  long grid;
};

inline void plan_staged(const phip_ctx *ctx, const Gemm &p, StagedPlan *plan) {
  GemmArgs &a = plan->a;
  a = problem_args(p);
  a.accumulate = p.accumulate ? 1 : 0;
  a.partial = nullptr;
  a.tickets = nullptr;

  // 16-byte loads need aligned rows and a contiguous-axis extent that is a
  // multiple of 4 (so that no vector straddles the matrix edge).
  plan->vec_a = rows_aligned16(p.A, 4, p.lda, p.sA, p.rA) && (p.a_kmajor ? p.K : p.M) % 4 == 0;
  plan->vec_b = rows_aligned16(p.B, 4, p.ldb, p.sB, p.rB) && (p.b_kmajor ? p.K : p.N) % 4 == 0;

  const int cus = ctx->prop.multiProcessorCount;
  auto tiles = [&](int bm, int bn) {
    return (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batch;
  };
  // 128x128x16 at four workgroups per CU (33 KiB of LDS and 128 VGPRs each)
  // measured fastest among BK 8/16/32 and 2..4 workgroups per CU.
  // A short contraction (K <= 128) is a rank-K update bound by the traffic of
  // C and by latency: 64x64 tiles put four times as many workgroups in flight.
  const long k_total = (long)p.K * p.rbatch;
  int bm, bk;
  if (tiles(128, 128) >= cus && k_total > 128) {
    plan->shape = StagedShape::k128x128x16; bm = 128; bk = 16;
  } else if (tiles(64, 64) >= cus) {
    plan->shape = StagedShape::k64x64x32; bm = 64; bk = 32;
  } else {
    plan->shape = StagedShape::k32x32x64; bm = 32; bk = 64;
  }
  a.tiles_m = (p.M + bm - 1) / bm;
  a.tiles_n = (p.N + bm - 1) / bm;
  a.ktiles_per_r = (p.K + bk - 1) / bk;
  a.total_ktiles = a.ktiles_per_r * p.rbatch;
  const long t = (long)a.tiles_m * a.tiles_n * p.batch;

  // Split K between workgroups when the C tiles alone cannot fill the chip.
  // (this kernel's split adds tiles with atomics: a context that wants the same bits on every run gets none)
  int splits = 1;
  if (t < 2 * cus && !ctx->deterministic) {
    const long want = (4L * cus + t - 1) / t;
    const int min_ktiles = bk >= 64 ? 2 : 4;  // K tiles per workgroup worth a launch
    long cap = a.total_ktiles / min_ktiles;
    if (cap < 1) cap = 1;
    splits = (int)(want < cap ? want : cap);
  }
  a.splits = splits;
  a.atomic = splits > 1;
  plan->grid = t * splits;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_STAGED_H_
