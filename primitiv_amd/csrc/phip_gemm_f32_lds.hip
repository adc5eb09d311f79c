// fp32 GEMM, 128 x 128 x 32 tiles, operands moved global -> LDS by buffer
// loads that write LDS directly (no staging registers, no LDS write
// instructions, ragged edges zero-filled by the buffer range check).
//
// One workgroup = 4 wavefronts in a 2 x 2 grid, each a 64 x 64 block of 2 x 2
// v_mfma_f32_32x32x2_f32 tiles.  Two 32 KiB LDS stages (A region then B region,
// 16 KiB each); two workgroups share a CU.
//
// MODE 1: a problem with too few output tiles for the chip cuts its K range
// between workgroups; an accumulating product adds its tiles into C with fp32
// atomics, an overwriting one meets through partial tiles and a per-tile
// ticket (see last_of_tile).  MODE 2: only the tiles of a partly filled last
// round are cut (see TileWork).  The unsplit instantiation (MODE 0) carries
// none of that.
//
// The LDS image of an operand tile is described with the loader that builds it.
#include "phip_gemm_f32_lds.h"

namespace phip {
namespace {

constexpr int LBM = 128, LBN = 128;
constexpr int kRegion = 16384;            // bytes per operand per stage
constexpr int kStage = 2 * kRegion;
constexpr int kLdsBytes = 2 * kStage;

// Which output tile and which K range a workgroup takes.
//  * unsplit: one tile each, the whole K range;
//  * split: every tile is shared by `splits` workgroups;
//  * mixed (whole_tiles > 0): the tiles do not fill a whole number of rounds on the chip.  The first
//    `whole_tiles` workgroups (a multiple of the CU count) take one tile each; the tiles that are left - too
//    few for a round of their own, so that a few CUs would carry one tile more than the others - are cut
//    into `splits` K ranges each, whose workgroups spread over all CUs behind the whole tiles.
struct TileWork {
  int tile_m, tile_n, z;
  int split;    // K range of a shared tile
  bool shared;  // the tile is shared: meet through atomics or partial tiles
  int tail;     // mixed: index of the shared tile among the shared ones
};

template <int MODE>
__device__ inline TileWork tile_work(const LdsArgs &d) {
  constexpr bool SPLIT = MODE != 0;
  const GemmArgs &g = d.g;
  TileWork w;
  w.split = 0;
  w.shared = SPLIT;
  w.tail = 0;
  int t;
  if constexpr (MODE == 2) {
    const int bid = blockIdx.x;
    if (bid < d.whole_tiles) {
      t = xcd_remap(bid, d.whole_tiles);
      w.shared = false;
    } else {
      const int rest = (int)gridDim.x - d.whole_tiles;
      const int tails = rest / g.splits;
      const int u = xcd_remap(bid - d.whole_tiles, rest);
      w.tail = u % tails;
      w.split = u / tails;
      t = d.whole_tiles + w.tail;
    }
    w.tile_m = t % g.tiles_m; t /= g.tiles_m;
    w.tile_n = t % g.tiles_n; t /= g.tiles_n;
    w.z = t;
    return w;
  } else {
  t = xcd_remap(blockIdx.x, gridDim.x);
  w.tile_m = t % g.tiles_m; t /= g.tiles_m;
  w.tile_n = t % g.tiles_n; t /= g.tiles_n;
  if (SPLIT) {
    w.split = t % g.splits;
    t /= g.splits;
  }
  w.z = t;
  return w;
  }
}

// Partial tiles of a mixed launch: SIDE x SIDE floats per shared tile and K range, tile-local coordinates
// (elements outside the matrix are zeros: their operands were zero-filled by the loads).  Same device-scope
// accesses and ticket as store_partial / sum_partials / last_of_tile.
template <int NV, int SIDE>
__device__ inline void store_tile_partial(float *P, int row0, int col0, int lane, const int (&nq)[NV], const float (&vals)[NV]) {
  const int m = row0 + (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
#pragma unroll
  for (int q = 0; q < NV; ++q)
    __hip_atomic_store(P + m + (ncol + nq[q]) * SIDE, vals[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <int NV, int SIDE>
__device__ inline void sum_tile_partials(const float *P, int splits, int row0, int col0, int lane, const int (&nq)[NV],
                                         float (&vals)[NV]) {
  const int m = row0 + (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
  constexpr int kPer = SIDE * SIDE;
#pragma unroll
  for (int q = 0; q < NV; ++q) vals[q] = 0.0f;
  for (int r0 = 0; r0 < splits; r0 += 4) {
    float part[4][NV];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < NV; ++q)
        part[u][q] = __hip_atomic_load(P + (r0 + u < splits ? r0 + u : r0) * kPer + m + (ncol + nq[q]) * SIDE,
                                       __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int q = 0; q < NV; ++q)
        if (r0 + u < splits) vals[q] += part[u][q];
  }
}

// MODE 0: unsplit, 1: every tile shared by K ranges, 2: mixed (see TileWork).
template <bool A_KMAJOR, bool B_KMAJOR, int MODE>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_lds_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  const TileWork tw = tile_work<MODE>(d);
  const int tile_m = tw.tile_m, tile_n = tw.tile_n, z = tw.z, split = tw.split;
  const int m0 = tile_m * LBM, n0 = tile_n * LBN;

  DmaLoader<A_KMAJOR> la;
  DmaLoader<B_KMAJOR> lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, n0, g.N, wave, lane);
  FragReaderF<A_KMAJOR> fra;
  FragReaderF<B_KMAJOR> frb;
  fra.init(wm * 64, lane);
  frb.init(wn * 64, lane);

  const float *Az = g.A + (long)z * g.sA;
  const float *Bz = g.B + (long)z * g.sB;

  float16v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // K tiles [kt_base, kt_base + kt_end) belong to this workgroup
  const int kt_base = tw.shared ? (int)((long)split * g.total_ktiles / g.splits) : 0;
  const int kt_end = tw.shared ? (int)((long)(split + 1) * g.total_ktiles / g.splits) - kt_base : g.total_ktiles;
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  auto issue_tile = [&](int kt, int q) {
    // instruction q of the 8 that move K tile kt (4 for A, then 4 for B)
    const bool live = kt < kt_end;
    const int ktc = live ? kt + kt_base : 0;
    const int r = ktc / g.ktiles_per_r;
    const int kt_in_r = ktc - r * g.ktiles_per_r;
    const uint32_t stage = lds_base + (uint32_t)(kt & 1) * kStage;
    if (q < 4) la.issue(make_rsrc_words(Az + (long)r * g.rA, d.a_bytes), stage, wave, q, kt_in_r, g.K, live);
    else lb.issue(make_rsrc_words(Bz + (long)r * g.rB, d.b_bytes), stage + kRegion, wave, q - 4, kt_in_r, g.K, live);
  };

#pragma unroll
  for (int q = 0; q < 8; ++q) issue_tile(0, q);
#pragma unroll
  for (int q = 0; q < 8; ++q) issue_tile(1, q);
  asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // tile 0 has landed
  __syncthreads();

  // Fragments are double-buffered in registers: group gk+1 is read between the
  // matrix instructions of group gk; the first group of the next tile is read
  // behind the barrier, under the last group of this one.
  float fa[2][2][4], fb[2][2][4];
  fra.read(lds, 0, fa[0]);
  frb.read(lds + kRegion, 0, fb[0]);

  constexpr int kReadsA = FragReaderF<A_KMAJOR>::kReads, kReadsB = FragReaderF<B_KMAJOR>::kReads;
  for (int kt = 0; kt < kt_end; ++kt) {
    const int stage = kt & 1;
#pragma unroll
    for (int gk = 0; gk < 4; ++gk) {
      const int cur = gk & 1, nxt = cur ^ 1;
      const unsigned char *src = lds + (gk < 3 ? stage : stage ^ 1) * kStage;
      const int ngk = gk < 3 ? gk + 1 : 0;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int e = q >> 2, i = (q >> 1) & 1, j = q & 1;
        // rows of the instruction's result follow n, its columns follow m
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][j][e], fa[cur][i][e], acc[i][j], 0, 0, 0);
        if (q < kReadsA) fra.read_one(src, ngk, q, fa[nxt]);
        else if (q < kReadsA + kReadsB) frb.read_one(src + kRegion, ngk, q - kReadsA, fb[nxt]);
        // K tile kt+2 refills this stage once everybody has left it
        if (gk == 3 && (q & 1)) issue_tile(kt + 2, q >> 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (gk == 2) {
        // own loads of tile kt+1 have landed and own reads of this stage are
        // done; behind the barrier that holds for every wave
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
      }
    }
  }
  // the loads issued for tiles past the end move nothing, but must have retired
  // before this workgroup's LDS can be handed to another one
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + LBM <= g.M && n0 + LBN <= g.N;
  int ns[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) ns[v] = 8 * (v / 4) + (v % 4);
  if constexpr (MODE == 2) {
    if (tw.shared && g.atomic == 2) {
      // mixed launch: tile-sized partial tiles of the shared tiles only
      __shared__ uint32_t last_flag_mixed;
      float *P = g.partial + (long)tw.tail * g.splits * (LBM * LBN);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float vals[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) vals[v] = acc[i][j][v];
          store_tile_partial<16, LBM>(P + split * (LBM * LBN), wm * 64 + i * 32, wn * 64 + j * 32, lane, ns, vals);
        }
      if (!last_of_tile(g, tw.tail, &last_flag_mixed)) return;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float vals[16];
          sum_tile_partials<16, LBM>(P, g.splits, wm * 64 + i * 32, wn * 64 + j * 32, lane, ns, vals);
          emit_c<16>(Cz, g.ldc, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, g.M, g.N, interior, ns, vals, 0,
                     g.accumulate);
        }
      return;
    }
  }
  if constexpr (MODE == 1) {
    if (g.atomic == 2) {
      // leave the partial tile; the last workgroup of the output tile adds the ranges in order
      __shared__ uint32_t last_flag;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float vals[16];
#pragma unroll
          for (int v = 0; v < 16; ++v) vals[v] = acc[i][j][v];
          store_partial<16>(g, z, split, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, ns, vals);
        }
      if (!last_of_tile(g, (z * g.tiles_n + tile_n) * g.tiles_m + tile_m, &last_flag)) return;
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          float vals[16];
          sum_partials<16>(g, z, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, ns, vals);
          emit_c<16>(Cz, g.ldc, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, g.M, g.N, interior, ns, vals, 0,
                     g.accumulate);
        }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float vals[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) vals[v] = acc[i][j][v];
      emit_c<16>(Cz, g.ldc, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, g.M, g.N, interior, ns, vals,
                 tw.shared ? g.atomic : 0, g.accumulate);
    }
}

// The same scheme with 64 x 64 x 32 tiles for problems with too few 128 x 128
// tiles: 2 x 2 wavefronts of one 32 x 32 block each (16 accumulator registers),
// two 16 KiB stages, four workgroups per CU, so that the matrix pipe of a SIMD
// has four wavefronts to draw from while any of them waits at a barrier.
constexpr int SBM = 64, SBN = 64;
constexpr int kRegion64 = 8192;
constexpr int kStage64 = 2 * kRegion64;
constexpr int kLds64Bytes = 2 * kStage64;

template <bool A_KMAJOR, bool B_KMAJOR, int MODE>
__global__ __launch_bounds__(kThreads, 4) void gemm_f32_lds64_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  const TileWork tw = tile_work<MODE>(d);
  const int tile_m = tw.tile_m, tile_n = tw.tile_n, z = tw.z, split = tw.split;
  const int m0 = tile_m * SBM, n0 = tile_n * SBN;

  DmaLoader<A_KMAJOR, SBM> la;
  DmaLoader<B_KMAJOR, SBN> lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, n0, g.N, wave, lane);
  FragReaderF<A_KMAJOR, SBM> fra;
  FragReaderF<B_KMAJOR, SBN> frb;
  fra.init(wm * 32, lane);
  frb.init(wn * 32, lane);

  const float *Az = g.A + (long)z * g.sA;
  const float *Bz = g.B + (long)z * g.sB;

  float16v acc;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc[v] = 0.0f;

  // K tiles [kt_base, kt_base + kt_end) belong to this workgroup
  const int kt_base = tw.shared ? (int)((long)split * g.total_ktiles / g.splits) : 0;
  const int kt_end = tw.shared ? (int)((long)(split + 1) * g.total_ktiles / g.splits) - kt_base : g.total_ktiles;
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  auto issue_tile = [&](int kt, int q) {
    // instruction q of the 4 that move K tile kt (2 for A, then 2 for B)
    const bool live = kt < kt_end;
    const int ktc = live ? kt + kt_base : 0;
    const int r = ktc / g.ktiles_per_r;
    const int kt_in_r = ktc - r * g.ktiles_per_r;
    const uint32_t stage = lds_base + (uint32_t)(kt & 1) * kStage64;
    if (q < 2) la.issue(make_rsrc_words(Az + (long)r * g.rA, d.a_bytes), stage, wave, q, kt_in_r, g.K, live);
    else lb.issue(make_rsrc_words(Bz + (long)r * g.rB, d.b_bytes), stage + kRegion64, wave, q - 2, kt_in_r, g.K, live);
  };

#pragma unroll
  for (int q = 0; q < 4; ++q) issue_tile(0, q);
#pragma unroll
  for (int q = 0; q < 4; ++q) issue_tile(1, q);
  asm volatile("s_waitcnt vmcnt(4)" ::: "memory");  // tile 0 has landed
  __syncthreads();

  // fragments of one group of 8 k (block 0 of the readers' two), double-buffered as above
  float fa[2][2][4], fb[2][2][4];
  constexpr int kReadsA = A_KMAJOR ? 1 : 4, kReadsB = B_KMAJOR ? 1 : 4;
#pragma unroll
  for (int q = 0; q < kReadsA; ++q) fra.read_one(lds, 0, q, fa[0]);
#pragma unroll
  for (int q = 0; q < kReadsB; ++q) frb.read_one(lds + kRegion64, 0, q, fb[0]);

  for (int kt = 0; kt < kt_end; ++kt) {
    const int stage = kt & 1;
#pragma unroll
    for (int gk = 0; gk < 4; ++gk) {
      const int cur = gk & 1, nxt = cur ^ 1;
      const unsigned char *src = lds + (gk < 3 ? stage : stage ^ 1) * kStage64;
      const int ngk = gk < 3 ? gk + 1 : 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // rows of the instruction's result follow n, its columns follow m
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][0][e], fa[cur][0][e], acc, 0, 0, 0);
        if (e < kReadsA) fra.read_one(src, ngk, e, fa[nxt]);
        if (e < kReadsB) frb.read_one(src + kRegion64, ngk, e, fb[nxt]);
        // K tile kt+2 refills this stage once everybody has left it
        if (gk == 3) issue_tile(kt + 2, e);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (gk == 2) {
        // own loads of tile kt+1 have landed and own reads of this stage are
        // done; behind the barrier that holds for every wave
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
      }
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");

  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + SBM <= g.M && n0 + SBN <= g.N;
  const int row0 = m0 + wm * 32, col0 = n0 + wn * 32;
  int ns[16];
  float vals[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    ns[v] = 8 * (v / 4) + (v % 4);
    vals[v] = acc[v];
  }
  if constexpr (MODE == 2) {
    if (tw.shared && g.atomic == 2) {
      __shared__ uint32_t last_flag_mixed;
      float *P = g.partial + (long)tw.tail * g.splits * (SBM * SBN);
      store_tile_partial<16, SBM>(P + split * (SBM * SBN), wm * 32, wn * 32, lane, ns, vals);
      if (!last_of_tile(g, tw.tail, &last_flag_mixed)) return;
      sum_tile_partials<16, SBM>(P, g.splits, wm * 32, wn * 32, lane, ns, vals);
      emit_c<16>(Cz, g.ldc, row0, col0, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
      return;
    }
  }
  if constexpr (MODE == 1) {
    if (g.atomic == 2) {
      __shared__ uint32_t last_flag;
      store_partial<16>(g, z, split, row0, col0, lane, ns, vals);
      if (!last_of_tile(g, (z * g.tiles_n + tile_n) * g.tiles_m + tile_m, &last_flag)) return;
      sum_partials<16>(g, z, row0, col0, lane, ns, vals);
      emit_c<16>(Cz, g.ldc, row0, col0, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
      return;
    }
  }
  emit_c<16>(Cz, g.ldc, row0, col0, lane, g.M, g.N, interior, ns, vals, tw.shared ? g.atomic : 0, g.accumulate);
}

// 64 x 64 tiles without a barrier in the K loop, for a launch that gives every CU at most one workgroup.
// With one workgroup on a CU nothing overlaps the wait at a barrier (timestamps in a variant of the kernel
// above with eight wavefronts: of the 1850 cycles that a K tile takes, 480 are the wait for loads plus the
// barrier, and the matrix pipe of a SIMD is busy 1024), so here no wavefront shares LDS with another: each
// of the eight wavefronts of a workgroup (two per SIMD) moves its own
// operands - the 32 rows of A and the 32 columns of B of its block, 32 k at a time, 8 KiB per stage, two
// stages - into its own 16 KiB of LDS and waits only for its own loads.  Wavefronts w and w + 4 share a
// block and take alternate K tiles; their tiles meet through LDS at the end.  Each wavefront alternates
// between two accumulators, so that a matrix instruction never waits for the result of the one before it.  An operand block is loaded by
// the two wavefront pairs that need it, twice the bytes from L2 (32 B / clk / CU), which the loads that
// write LDS directly deliver.
constexpr int kThreads64w = 512;
constexpr int kLds64wBytes = 8 * 16384;

template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kThreads64w, 2) void gemm_f32_lds64w_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int kh = wave >> 2;  // K tiles kh, kh + 2, ...
  const int wm = wave & 1, wn = (wave >> 1) & 1;

  const TileWork tw = tile_work<0>(d);
  const int tile_m = tw.tile_m, tile_n = tw.tile_n, z = tw.z;
  const int m0 = tile_m * SBM, n0 = tile_n * SBN;
  const int row0 = m0 + wm * 32, col0 = n0 + wn * 32;

  DmaLoader<A_KMAJOR, 32, 1> la;
  DmaLoader<B_KMAJOR, 32, 1> lb;
  la.init(g.lda, row0, g.M, 0, lane);
  lb.init(g.ldb, col0, g.N, 0, lane);
  FragReaderF<A_KMAJOR, 32> fra;
  FragReaderF<B_KMAJOR, 32> frb;
  fra.init(0, lane);
  frb.init(0, lane);

  const float *Az = g.A + (long)z * g.sA;
  const float *Bz = g.B + (long)z * g.sB;

  float16v acc0, acc1;
#pragma unroll
  for (int v = 0; v < 16; ++v) acc0[v] = acc1[v] = 0.0f;

  constexpr int kOwnRegion = 4096, kOwnStage = 2 * kOwnRegion;
  unsigned char *own = lds + wave * (2 * kOwnStage);
  const uint32_t own_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)own;
  const int own_tiles = (g.total_ktiles - kh + 1) / 2;
  auto issue_tile = [&](int t, int into, int q) {
    // instruction q of the 8 (4 for A, then 4 for B) that move this wavefront's K tile t into stage `into`
    const bool live = t < own_tiles;
    const int ktc = live ? 2 * t + kh : 0;
    const int r = ktc / g.ktiles_per_r;
    const int kt_in_r = ktc - r * g.ktiles_per_r;
    const uint32_t stage = own_base + (uint32_t)into * kOwnStage;
    if (q < 4) la.issue(make_rsrc_words(Az + (long)r * g.rA, d.a_bytes), stage, 0, q, kt_in_r, g.K, live);
    else lb.issue(make_rsrc_words(Bz + (long)r * g.rB, d.b_bytes), stage + kOwnRegion, 0, q - 4, kt_in_r, g.K, live);
  };

#pragma unroll
  for (int q = 0; q < 8; ++q) issue_tile(0, 0, q);
#pragma unroll
  for (int q = 0; q < 8; ++q) issue_tile(1, 1, q);
  asm volatile("s_waitcnt vmcnt(8)" ::: "memory");  // tile 0 has landed

  float fa[2][2][4], fb[2][2][4];
  constexpr int kReadsA = A_KMAJOR ? 1 : 4, kReadsB = B_KMAJOR ? 1 : 4;
#pragma unroll
  for (int q = 0; q < kReadsA; ++q) fra.read_one(own, 0, q, fa[0]);
#pragma unroll
  for (int q = 0; q < kReadsB; ++q) frb.read_one(own + kOwnRegion, 0, q, fb[0]);

  for (int t = 0; t < own_tiles; ++t) {
    const int stage = t & 1;
#pragma unroll
    for (int gk = 0; gk < 4; ++gk) {
      const int cur = gk & 1, nxt = cur ^ 1;
      const unsigned char *src = own + (gk < 3 ? stage : stage ^ 1) * kOwnStage;
      const int ngk = gk < 3 ? gk + 1 : 0;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        // rows of the instruction's result follow n, its columns follow m
        if (e & 1) acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][0][e], fa[cur][0][e], acc1, 0, 0, 0);
        else acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][0][e], fa[cur][0][e], acc0, 0, 0, 0);
        if (e < kReadsA) fra.read_one(src, ngk, e, fa[nxt]);
        if (e < kReadsB) frb.read_one(src + kOwnRegion, ngk, e, fb[nxt]);
        // tile t + 2 refills this stage: every read of it was waited for behind group 2
        if (gk == 3) {
          issue_tile(t + 2, stage, 2 * e);
          issue_tile(t + 2, stage, 2 * e + 1);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      // the loads of tile t + 1 have landed and the reads of this stage are done
      if (gk == 2) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
  }
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");

  // the upper four wavefronts hand their tiles to the lower four through their own LDS
  float16v acc = acc0 + acc1;
  if (kh == 1) {
    float *red = reinterpret_cast<float *>(own);
#pragma unroll
    for (int v = 0; v < 16; ++v) red[v * 64 + lane] = acc[v];
  }
  __syncthreads();
  if (kh == 1) return;

  const float *red = reinterpret_cast<const float *>(lds + (wave + 4) * (2 * kOwnStage));
  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + SBM <= g.M && n0 + SBN <= g.N;
  int ns[16];
  float vals[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    ns[v] = 8 * (v / 4) + (v % 4);
    vals[v] = acc[v] + red[v * 64 + lane];
  }
  emit_c<16>(Cz, g.ldc, row0, col0, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
}

// Fills the argument block shared by both tile sizes.
static void fill_args(const Gemm &p, int side, long splits, long total_ktiles, long a_bytes, long b_bytes,
                      phip_ctx *ctx, LdsArgs *d) {
  GemmArgs &a = d->g;
  a = problem_args(p);
  a.tiles_m = (p.M + side - 1) / side;
  a.tiles_n = (p.N + side - 1) / side;
  a.splits = (int)splits;
  a.ktiles_per_r = (p.K + LBK - 1) / LBK;
  a.total_ktiles = (int)total_ktiles;
  a.atomic = splits > 1;
  a.accumulate = p.accumulate ? 1 : 0;
  a.partial = nullptr;
  a.tickets = ctx->tile_tickets;
  d->a_bytes = (uint32_t)a_bytes;
  d->b_bytes = (uint32_t)b_bytes;
  d->whole_tiles = 0;
}

}  // namespace

// Large, 16-byte-aligned problems: at least one 128 x 128 tile per CU, or an
// eighth of that with a K long enough to be cut between workgroups; else
// 64 x 64 tiles when those fill the chip.  Sets *handled when it launched.
int gemm_f32_lds(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  if (!rows_aligned16(p.A, 4, p.lda, p.sA, p.rA) || !rows_aligned16(p.B, 4, p.ldb, p.sB, p.rB)) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return PHIP_OK;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  if ((long)p.K * p.rbatch <= 128) return PHIP_OK;
  if (p.a_kmajor && !p.b_kmajor) return PHIP_OK;
  const int cus = ctx->prop.multiProcessorCount;
  const long total_ktiles = (long)((p.K + LBK - 1) / LBK) * p.rbatch;
  auto tiles_of = [&](int side) { return (long)((p.M + side - 1) / side) * ((p.N + side - 1) / side) * p.batch; };

  // ---- 128 x 128 tiles
  int side = LBM;
  long tiles = tiles_of(LBM);
  long splits = 1;
  bool take = tiles >= cus && tiles <= 0x7fffffffL;
  if (!take && tiles < cus && total_ktiles >= 64 && tiles * 8 >= cus && tiles * 4 < cus * 3L) {
    // Fewer tiles than CUs: worth it for a long K (from 2048) cut into ranges of at least 8 K tiles, when the
    // tiles alone fill between an eighth and three quarters of the CUs (measured on M, N in 512 .. 4096).  The
    // number of ranges minimises a small cost model fitted to those measurements: a fixed cost per workgroup,
    // the time of a K tile when a workgroup has its CU to itself or shares it with a second one, and the
    // exchange of the partial results, which grows with the number of ranges.
    double best = 0.0;
    for (long s = 2; s <= 16 && s * 8 <= total_ktiles && tiles * s <= 2L * cus; ++s) {
      const double per_ktile = tiles * s <= cus ? 2.6 : 4.2;  // microseconds
      const double t = 8.0 + per_ktile * (double)total_ktiles / (double)s + 3.0 * (double)s;
      if (splits == 1 || t < best) {
        best = t;
        splits = s;
      }
    }
    take = splits >= 2;
  }
  // ---- 64 x 64 tiles
  if (!take) {
    // Measured on M, N in 256 .. 3072, K in 256 .. 1536 against the staged 64 x 64 tiles and the direct
    // kernel: an overwriting product gains (15 - 35 %) when it is not split and has at least half a tile per
    // CU (768^3: 32.4 -> 22.4 us; with a quarter, 512^3, the direct kernel is ahead, 13.0 against 15.1 us; the
    // exchange of partial tiles costs more than the idle CUs); an accumulating product gains
    // (10 - 25 %) from half a tile per CU on, its K cut into ranges of at least 8 tiles until the four
    // places of every CU are filled, the tiles added with atomics.
    side = SBM;
    tiles = tiles_of(SBM);
    const long least = cus / 2;
    if (tiles < least || tiles > 0x7fffffffL || 2L * p.M * p.N * p.batch < tiles * SBM * SBN) return PHIP_OK;
    splits = 1;
    if (p.accumulate && tiles < 4L * cus) {
      splits = 4L * cus / tiles;
      if (splits > total_ktiles / 8) splits = total_ktiles / 8;
      if (splits > 16) splits = 16;
      if (splits < 1) splits = 1;
    }
    take = true;
  }

  // ---- a last, partly filled round of tiles
  // Unsplit tiles that do not fill a whole number of rounds leave a few CUs with one tile more than the
  // rest, and those set the time: 576 tiles on 256 CUs take as long as 768 would.  When the tiles beyond
  // the last whole round are at most half a round, they are cut into K ranges (of at least 8 K tiles) that
  // spread over all CUs instead: 3072^3 forward 587 -> 478 us, both gradients 1146 -> 856 us.
  long whole = 0;
  Scratch partials(ctx);
  if (splits == 1 && !ctx->fixed_mode) {
    const long rounds = tiles / cus, rest = tiles - rounds * cus;
    if (rounds >= 1 && rounds <= 8 && rest > 0 && 2 * rest <= cus) {
      long s = cus / rest;
      if (s > 16) s = 16;
      if (s > total_ktiles / 8) s = total_ktiles / 8;
      bool ok = s >= 2;
      if (ok && wants_exchange(ctx, p)) {
        ok = rest <= kTicketSlots &&
             scratch_alloc(ctx, sizeof(float) * (size_t)rest * s * side * side, &partials.ptr) == PHIP_OK;
        if (!ok) partials.ptr = nullptr;
      }
      if (ok) {
        whole = rounds * cus;
        splits = s;
      }
    }
  }

  LdsArgs d;
  fill_args(p, side, splits, total_ktiles, a_bytes, b_bytes, ctx, &d);
  if (whole > 0) {
    d.whole_tiles = (int)whole;
    if (partials.ptr != nullptr) {
      d.g.atomic = 2;
      d.g.partial = static_cast<float *>(partials.ptr);
      d.g.tickets = tile_tickets(ctx);
    }
  } else if (splits > 1 && wants_exchange(ctx, p)) {
    const int rc0 = prepare_split_exchange(ctx, p, tiles, (size_t)(256L << 20), &d.g, &partials);
    if (rc0 != PHIP_OK) return rc0;
  }

  int rc = PHIP_OK;
  const unsigned grid = (unsigned)(whole > 0 ? whole + (tiles - whole) * splits : tiles * splits);
#define PHIP_LDS(SLOT, AK, BKM, MODE)                                                                        \
  do {                                                                                                       \
    auto kern = gemm_f32_lds_kernel<AK, BKM, MODE>;                                                          \
    rc = raise_lds_limit(ctx, SLOT + (MODE == 2 ? kSlotGemmF32LdsMixed - kSlotGemmF32Lds : MODE == 1 ? 3 : 0), \
                         reinterpret_cast<const void *>(kern), kLdsBytes);                                   \
    if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), kLdsBytes, ctx->stream, d);      \
  } while (0)
#define PHIP_LDS64(AK, BKM, MODE)                                                                            \
  hipLaunchKernelGGL((gemm_f32_lds64_kernel<AK, BKM, MODE>), dim3(grid), dim3(kThreads), kLds64Bytes, ctx->stream, d)
#define PHIP_LDS_LAYOUTS(MODE)                                                                               \
  do {                                                                                                       \
    if (side == LBM) {                                                                                       \
      if (!p.a_kmajor && p.b_kmajor) PHIP_LDS(kSlotGemmF32Lds + 0, false, true, MODE);                       \
      else if (!p.a_kmajor && !p.b_kmajor) PHIP_LDS(kSlotGemmF32Lds + 1, false, false, MODE);                \
      else PHIP_LDS(kSlotGemmF32Lds + 2, true, true, MODE);                                                  \
    } else {                                                                                                 \
      if (!p.a_kmajor && p.b_kmajor) PHIP_LDS64(false, true, MODE);                                          \
      else if (!p.a_kmajor && !p.b_kmajor) PHIP_LDS64(false, false, MODE);                                   \
      else PHIP_LDS64(true, true, MODE);                                                                     \
    }                                                                                                        \
  } while (0)
  // one workgroup per CU at most: the kernel whose wavefronts do not wait for each other
  const bool alone = side == SBM && splits == 1 && whole == 0 && tiles <= cus;
  if (alone) {
#define PHIP_LDS64W(SLOT, AK, BKM)                                                                           \
  do {                                                                                                       \
    auto kern = gemm_f32_lds64w_kernel<AK, BKM>;                                                             \
    rc = raise_lds_limit(ctx, kSlotGemmF32Lds64w + (SLOT), reinterpret_cast<const void *>(kern), kLds64wBytes); \
    if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads64w), kLds64wBytes, ctx->stream, d); \
  } while (0)
    if (!p.a_kmajor && p.b_kmajor) PHIP_LDS64W(0, false, true);
    else if (!p.a_kmajor && !p.b_kmajor) PHIP_LDS64W(1, false, false);
    else PHIP_LDS64W(2, true, true);
#undef PHIP_LDS64W
  } else if (whole > 0) PHIP_LDS_LAYOUTS(2);
  else if (splits > 1) PHIP_LDS_LAYOUTS(1);
  else PHIP_LDS_LAYOUTS(0);
#undef PHIP_LDS_LAYOUTS
#undef PHIP_LDS
#undef PHIP_LDS64
  if (rc != PHIP_OK) return rc;
  PHIP_LAUNCH_CHECK();
  if (alone) note_kernel(ctx, "f32_lds64w");
  else if (whole > 0) note_kernel(ctx, side == LBM ? "f32_lds128_mixed" : "f32_lds64_mixed");
  else note_kernel(ctx, side == LBM ? (splits > 1 ? "f32_lds128_split" : "f32_lds128") : (splits > 1 ? "f32_lds64_split" : "f32_lds64"));
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
