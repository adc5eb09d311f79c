// fp32 rank-K update of a large matrix, K <= 64: C (+)= A . B^T with both
// operands contiguous along the output's rows / columns.  This is the weight
// gradient of a per-timestep layer, gW += gy . x^T with a minibatch of 64: the
// cost is reading and writing C once.
//
// 128 x 128 output tiles chosen so that every workgroup is resident at once
// (two per compute unit): a launch is one round of: fetch the old C straight
// into the accumulators and the whole K extent of both operands into LDS (all
// in flight together), run the matrix instructions, store C.  Nothing waits
// for memory twice.
//
// Operands travel global -> LDS by buffer loads that write LDS directly, 16
// bytes per lane; a B whose rows are only 8-byte aligned goes through
// registers instead, 8 bytes per lane (4-byte loads into LDS would need four
// times as many instructions, and their issue alone then takes microseconds).
// One workgroup = 4 wavefronts side by side, each all 128 rows by 32
// columns: 4 v_mfma_f32_32x32x2_f32 blocks whose rows interleave (block i
// holds rows 4r + i), so that a lane owns 4 consecutive rows of a column and C
// moves 16 bytes per lane, 512 contiguous bytes per half wavefront.  (Moved 4
// bytes per lane in the instruction's plain layout, the same read-then-write of
// C takes more than twice as long.)
#include <type_traits>

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

template <bool STORE>
__device__ inline void move_c(float *Cz, long ldc, int row0, int col0, int lane, int M, int N, bool interior,
                              float16v (&acc)[4]) {
  const int m = row0 + 4 * (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int n = ncol + column_of(v);
    const bool ok = interior || (m < M && n < N);
    float4v *p = reinterpret_cast<float4v *>(ok ? Cz + m + (long)n * ldc : Cz);
    if constexpr (STORE) {
      const float4v out = {acc[0][v], acc[1][v], acc[2][v], acc[3][v]};
      if (ok) *p = out;
    } else {
      const float4v old = *p;
      acc[0][v] = ok ? old.x : 0.0f;
      acc[1][v] = ok ? old.y : 0.0f;
      acc[2][v] = ok ? old.z : 0.0f;
      acc[3][v] = ok ? old.w : 0.0f;
    }
  }
}

template <int VB>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_rankk_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int z = t;
  const int m0 = tile_m * RBM, n0 = tile_n * RBN;

  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  const int n_kt = (g.K + LBK - 1) / LBK;
  const float *Bz = g.B + (long)z * g.sB;

  // B through registers: wave w owns k rows 16w .. 16w+15, a lane two columns of each
  typedef float float2v __attribute__((ext_vector_type(2)));
  float2v breg[16];
  if constexpr (VB == 2) {
    const int n = n0 + 2 * lane;
#pragma unroll
    for (int q = 0; q < 16; ++q) {
      const int k = wave * 16 + q;
      const bool ok = k < g.K && n < g.N;
      const float2v got = *reinterpret_cast<const float2v *>(ok ? Bz + (long)k * g.ldb + n : Bz);
      breg[q] = ok ? got : float2v{0.0f, 0.0f};
    }
  }

  // the old C next: these loads have the longest way to go
  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + RBM <= g.M && n0 + RBN <= g.N;
  float16v acc[4];
  if (g.accumulate) {
    move_c<false>(Cz, g.ldc, m0, n0 + wave * 32, lane, g.M, g.N, interior, acc);
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][v] = 0.0f;
  }

  DmaLoader<false, RBM> la;
  la.init(g.lda, m0, g.M, wave, lane);
  const uint4v rsrc_a = make_rsrc_words(g.A + (long)z * g.sA, d.a_bytes);
#pragma unroll
  for (int kt = 0; kt < kKTiles; ++kt) {
    const bool live = kt < n_kt;
#pragma unroll
    for (int q = 0; q < 4; ++q) la.issue(rsrc_a, lds_base + (uint32_t)kt * kRegion, wave, q, kt, g.K, live);
  }
  if constexpr (VB == 4) {
    DmaLoader<false, RBN> lb;
    lb.init(g.ldb, n0, g.N, wave, lane);
    const uint4v rsrc_b = make_rsrc_words(Bz, d.b_bytes);
#pragma unroll
    for (int kt = 0; kt < kKTiles; ++kt) {
#pragma unroll
      for (int q = 0; q < 4; ++q)
        lb.issue(rsrc_b, lds_base + (uint32_t)(kKTiles + kt) * kRegion, wave, q, kt, g.K, kt < n_kt);
    }
  } else {
    // k row r of the B image sits at r * 512 bytes (two tiles of 32 rows back to back)
#pragma unroll
    for (int q = 0; q < 16; ++q)
      *reinterpret_cast<float2v *>(lds + kKTiles * kRegion + (wave * 16 + q) * 512 + lane * 8) = breg[q];
  }

  // Fragments of k group gk (8 k) for the lane's k slots 4*(lane/32) + e: A is
  // one 16-byte read per e (rows 4r..4r+3 = the four blocks), B one 4-byte read.
  const uint32_t a_base = (uint32_t)((4 * (lane >> 5)) * 512 + (lane & 31) * 16);
  const uint32_t b_base = (uint32_t)((4 * (lane >> 5)) * 512 + (wave * 32 + (lane & 31)) * 4);
  auto read_a = [&](int group, int e, float4v (&fa)[4]) {
    fa[e] = *reinterpret_cast<const float4v *>(lds + (group >> 2) * kRegion + a_base + (8 * (group & 3) + e) * 512);
  };
  auto read_b = [&](int group, int e, float (&fb)[4]) {
    fb[e] = *reinterpret_cast<const float *>(lds + (kKTiles + (group >> 2)) * kRegion + b_base +
                                             (8 * (group & 3) + e) * 512);
  };
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();

  // Fragments are double-buffered in registers: group g+1 is read between the
  // matrix instructions of group g.
  float4v fa[2][4];
  float fb[2][4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    read_a(0, e, fa[0]);
    read_b(0, e, fb[0]);
  }
  const int groups = 4 * n_kt;
  for (int gg = 0; gg < groups; gg += 2) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int cur = h, nxt = h ^ 1;
      // the group after this one (past the end: group 0 again, read and not used)
      const int ng = gg + h + 1 < groups ? gg + h + 1 : 0;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int e = q >> 2, i = q & 3;
        // rows of the instruction's result follow n, its columns follow m
        acc[i] = __builtin_amdgcn_mfma_f32_32x32x2f32(fb[cur][e], fa[cur][e][i], acc[i], 0, 0, 0);
        if (q < 4) read_a(ng, q, fa[nxt]);
        else if (q < 8) read_b(ng, q - 4, fb[nxt]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }

  // the old values are already in the accumulators
  move_c<true>(Cz, g.ldc, m0, n0 + wave * 32, lane, g.M, g.N, interior, acc);
}

}  // namespace

// Rank-K updates (K <= 64) of matrices large enough that C's traffic is the
// cost.  Sets *handled when it launched.
int gemm_f32_rankk(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  if (p.a_kmajor || p.b_kmajor || p.rbatch != 1 || p.K > kKTiles * LBK) return PHIP_OK;
  if (!rows_aligned16(p.A, 4, p.lda, p.sA) || !rows_aligned16(p.C, 4, p.ldc, p.sC)) return PHIP_OK;
  const bool vec_b = rows_aligned16(p.B, 4, p.ldb, p.sB);
  // rows of B that are 8-byte aligned can still move two columns per lane
  if (!vec_b && (reinterpret_cast<uintptr_t>(p.B) % 8 != 0 || p.ldb % 2 != 0 || p.sB % 2 != 0)) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if (p.M != p.lda || p.N != p.ldb) return PHIP_OK;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  // one round of resident workgroups (two per compute unit), most compute units busy
  const long tiles = (long)((p.M + RBM - 1) / RBM) * ((p.N + RBN - 1) / RBN) * p.batch;
  const int cus = ctx->prop.multiProcessorCount;
  if (tiles > 2L * cus || tiles * 2 < cus) return PHIP_OK;

  LdsArgs d;
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

#define PHIP_RANKK(SLOT, VB)                                                                          \
  do {                                                                                                \
    auto kern = gemm_f32_rankk_kernel<VB>;                                                            \
    const int rc = raise_lds_limit(ctx, SLOT, reinterpret_cast<const void *>(kern), kRankLdsBytes);   \
    if (rc != PHIP_OK) return rc;                                                                     \
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(kThreads), kRankLdsBytes, ctx->stream, d);   \
  } while (0)
  if (vec_b) PHIP_RANKK(kSlotGemmF32RankK + 0, 4);
  else PHIP_RANKK(kSlotGemmF32RankK + 1, 2);
#undef PHIP_RANKK
  PHIP_LAUNCH_CHECK();
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
