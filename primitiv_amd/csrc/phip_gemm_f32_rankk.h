// fp32 rank-K update of a large matrix, K <= 64: C (+)= A . B^T with both
// operands contiguous along the output's rows / columns.  This is the weight
// gradient of a per-timestep layer, gW += gy . x^T with a minibatch of 64: the
// cost is reading and writing C once.
//
// 128 x 128 output tiles.  A workgroup fetches the old C straight into the
// accumulators and the whole K extent of both operands into LDS (all in flight
// together), runs the matrix instructions, adds the old values and stores C: the
// old values have the longest way to come and are not waited for before the
// matrix instructions are done.  A workgroup that is given several tiles of
// one row block keeps A in LDS.
//
// Operands travel global -> LDS by buffer loads that write LDS directly, 16
// bytes per lane; such a load needs no more than 4-byte alignment, so rows of
// any length qualify (a chunk that straddles the end of a row carries elements
// of the next k row into columns past N, whose results are never stored).
// One workgroup = 4 wavefronts side by side, each all 128 rows by 32
// columns: 4 v_mfma_f32_32x32x2_f32 blocks whose rows interleave (block i
// holds rows 4r + i), so that a lane owns 4 consecutive rows of a column and C
// moves 16 bytes per lane, 512 contiguous bytes per half wavefront.  (Moved 4
// bytes per lane in the instruction's plain layout, the same read-then-write of
// C takes more than twice as long.)
#ifndef PHIP_GEMM_F32_RANKK_H_
#define PHIP_GEMM_F32_RANKK_H_

#include "phip_gemm_f32_lds.h"

namespace phip {
namespace {

constexpr int RBM = 128, RBN = 128;
constexpr int kKTiles = 2;                       // K <= 64: at most two tiles of 32 k
constexpr int kRegion = 16384;                   // bytes of one operand's 32-k tile
constexpr int kRankLdsBytes = 2 * kKTiles * kRegion;

// Element v of the lane's four interleaved blocks is rows row0 + 4*(lane%32) +
// 0..3 of column col0 + 4*(lane/32) + 8*(v/4) + v%4: one 16-byte access.  M is
// a multiple of 4, so the four rows are inside or outside together.
__device__ inline int column_of(int v) { return 8 * (v / 4) + (v % 4); }

// The lane's 16 addresses in a tile and whether they lie inside the matrix.
struct TileOfC {
  float *Cz;
  long ldc;
  int m, ncol, M, N;
  bool interior;
  __device__ inline bool ok(int v) const { return interior || (m < M && ncol + column_of(v) < N); }
  __device__ inline float4v *at(int v) const {
    return reinterpret_cast<float4v *>(ok(v) ? Cz + m + (long)(ncol + column_of(v)) * ldc : Cz);
  }
};

__device__ inline TileOfC tile_of_c(float *Cz, long ldc, int row0, int col0, int lane, int M, int N) {
  TileOfC t;
  t.Cz = Cz; t.ldc = ldc; t.M = M; t.N = N;
  t.m = row0 + 4 * (lane & 31);
  t.ncol = col0 + 4 * (lane >> 5);
  t.interior = row0 + RBM <= M && col0 + 32 <= N;
  return t;
}

// Issues the loads of the old values; nothing waits for them here.
__device__ inline void fetch_c(const TileOfC &t, float4v (&raw)[16]) {
#pragma unroll
  for (int v = 0; v < 16; ++v) raw[v] = *t.at(v);
}

// Adds the fetched values to the accumulators (elements outside the matrix are never stored).
__device__ inline void add_old(const TileOfC &t, const float4v (&raw)[16], float16v (&acc)[4]) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    acc[0][v] += raw[v].x;
    acc[1][v] += raw[v].y;
    acc[2][v] += raw[v].z;
    acc[3][v] += raw[v].w;
  }
  (void)t;
}

__device__ inline void store_c(const TileOfC &t, const float16v (&acc)[4]) {
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const float4v out = {acc[0][v], acc[1][v], acc[2][v], acc[3][v]};
    if (t.ok(v)) *t.at(v) = out;
  }
}

// One workgroup's work: the tiles (tile_m, tn_first .. tn_first + tn_count - 1) of
// sample z, one after the other.  `lds` holds kRankLdsBytes (1 KiB aligned).
__device__ inline void rankk_tiles(const LdsArgs &d, unsigned char *lds, int z, int tile_m, int tn_first, int tn_count) {
  const GemmArgs &g = d.g;
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int m0 = tile_m * RBM;

  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  const int n_kt = (g.K + LBK - 1) / LBK;
  float *Cz = g.C + (long)z * g.sC;

  const uint32_t a_base = (uint32_t)((4 * (lane >> 5)) * 512 + (lane & 31) * 16);
  const uint32_t b_base = (uint32_t)((4 * (lane >> 5)) * 512 + (wave * 32 + (lane & 31)) * 4);
  // Fragments of k group gk (8 k) for the lane's k slots 4*(lane/32) + e: A is
  // one 16-byte read per e (rows 4r..4r+3 = the four blocks), B one 4-byte read.
  auto read_a = [&](int group, int e, float4v (&fa)[4]) {
    fa[e] = *reinterpret_cast<const float4v *>(lds + (group >> 2) * kRegion + a_base + (8 * (group & 3) + e) * 512);
  };
  auto read_b = [&](int group, int e, float (&fb)[4]) {
    fb[e] = *reinterpret_cast<const float *>(lds + (kKTiles + (group >> 2)) * kRegion + b_base +
                                             (8 * (group & 3) + e) * 512);
  };
  const int groups = 4 * n_kt;

  // Operands first (they come from L2 and the matrix instructions wait for nothing else), the old C
  // behind them: its values are only needed when the tile's products are complete, and they travel
  // while the matrix instructions run.
  DmaLoader<false, RBM> la;
  la.init(g.lda, m0, g.M, wave, lane);
  const uint4v rsrc_a = make_rsrc_words(g.A + (long)z * g.sA, d.a_bytes);
#pragma unroll
  for (int kt = 0; kt < kKTiles; ++kt) {
#pragma unroll
    for (int q = 0; q < 4; ++q) la.issue(rsrc_a, lds_base + (uint32_t)kt * kRegion, wave, q, kt, g.K, kt < n_kt);
  }
  const uint4v rsrc_b = make_rsrc_words(g.B + (long)z * g.sB, d.b_bytes);
  auto load_b = [&](int n0) {
    DmaLoader<false, RBN> lb;
    lb.init(g.ldb, n0, g.N, wave, lane);
#pragma unroll
    for (int kt = 0; kt < kKTiles; ++kt) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        lb.issue(rsrc_b, lds_base + (uint32_t)(kKTiles + kt) * kRegion, wave, q, kt, g.K, kt < n_kt);
    }
  };
  load_b(tn_first * RBN);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  for (int j = 0; j < tn_count; ++j) {
    const int n0 = (tn_first + j) * RBN;
    const TileOfC tile = tile_of_c(Cz, g.ldc, m0, n0 + wave * 32, lane, g.M, g.N);
    float4v raw[16];
    if (g.accumulate) fetch_c(tile, raw);

    float16v acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;

    // a wavefront whose 32 columns lie outside the matrix has nothing to compute
    if (n0 + wave * 32 < g.N) {
      // Fragments are double-buffered in registers: group g+1 is read between the
      // matrix instructions of group g.
      float4v fa[2][4];
      float fb[2][4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        read_a(0, e, fa[0]);
        read_b(0, e, fb[0]);
      }
      for (int gg = 0; gg < groups; gg += 2) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int cu = h, nxt = h ^ 1;
          // the group after this one (past the end: group 0 again, read and not used)
          const int ng = gg + h + 1 < groups ? gg + h + 1 : 0;
#pragma unroll
          for (int q = 0; q < 16; ++q) {
            const int e = q >> 2, i = q & 3;
            // rows of the instruction's result follow n, its columns follow m
            acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cu][e], fa[cu][e][i], acc[i], 0, 0, 0);
            if (q < 4) read_a(ng, q, fa[nxt]);
            else if (q < 8) read_b(ng, q - 4, fb[nxt]);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
      }
    }
    const bool more = j + 1 < tn_count;
    if (more) {
      // every wave is done with B's image: the next tile's may come
      __syncthreads();
      load_b(n0 + RBN);
    }
    if (g.accumulate) add_old(tile, raw, acc);
    if (more) {
      // The next tile's operands have landed before this tile's stores go out: nothing then has to be
      // waited for while stores are outstanding (loads and stores do not complete in one order).
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
      __syncthreads();
    }
    store_c(tile, acc);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// How a problem is run by this kernel.
struct RankKPlan {
  LdsArgs d;
  long tiles;
};

// False when the problem is not a rank-K update for this kernel.
inline bool plan_rankk(const Gemm &p, RankKPlan *plan) {
  if (p.a_kmajor || p.b_kmajor || p.rbatch != 1 || p.K > kKTiles * LBK) return false;
  // C moves 16 bytes per lane
  if (!rows_aligned16(p.C, 4, p.ldc, p.sC)) return false;
  // the contiguous extent of a dense operand is its leading dimension
  if (p.M != p.lda || p.N != p.ldb) return false;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return false;
  LdsArgs &d = plan->d;
  GemmArgs &a = d.g;
  a = problem_args(p);
  a.tiles_m = (p.M + RBM - 1) / RBM;
  a.tiles_n = (p.N + RBN - 1) / RBN;
  a.splits = 1;
  a.ktiles_per_r = (p.K + LBK - 1) / LBK;
  a.total_ktiles = a.ktiles_per_r;
  a.atomic = 0;
  a.accumulate = p.accumulate ? 1 : 0;
  a.partial = nullptr;
  a.tickets = nullptr;
  d.a_bytes = (uint32_t)a_bytes;
  d.b_bytes = (uint32_t)b_bytes;
  d.whole_tiles = 0;
  plan->tiles = (long)a.tiles_m * a.tiles_n * p.batch;
  return true;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_RANKK_H_
