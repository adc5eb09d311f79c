// fp32 GEMM for skinny problems (few output tiles, long or short K): the
// per-timestep shapes of recurrent graphs, where a launch is bound by memory
// latency rather than by the matrix cores.
//
// No LDS staging and no barriers in the K loop: every wavefront loads its
// matrix-instruction operands straight from global memory, already in the
// instruction's register layout, and keeps many independent loads in flight.
// The WAVES (4 or 8) wavefronts of a workgroup share one (32*TM) x (32*TN)
// output tile and split its K range between them; their partial tiles are
// summed through LDS once, at the end.  More wavefronts shorten the chain of
// dependent load rounds of a long K without the zero fill and atomics that a
// split between workgroups costs an overwriting product.  K can also be split
// between workgroups, whose tiles are then added into C with fp32 atomics.
//
// K is walked in chunks of 8.  v_mfma_f32_32x32x2_f32 takes, per lane, one A
// and one B value for k slot (lane / 32); the four instructions of a chunk use
// k = k0 + 4*(lane/32) + e, e = 0..3, for both operands.  With that choice an
// operand that is contiguous along k is fetched as ONE 16-byte load per lane
// (4 consecutive k of the lane's row), and an operand that is contiguous along
// m or n as four 4-byte loads that are each 128 contiguous bytes per half wave.
#ifndef PHIP_GEMM_F32_DIRECT_H_
#define PHIP_GEMM_F32_DIRECT_H_

#include "phip_gemm_f32_common.h"

namespace phip {
namespace {

struct DirectArgs {
  GemmArgs g;
  int chunks_per_r;   // ceil(K / 8)
  int total_chunks;   // rbatch * chunks_per_r
};

// Raw values of one 32-row operand block for one chunk (v[e] belongs to k slot
// e) plus a 4-bit mask of the elements that lie inside the matrix.  An element
// outside reads the matrix origin instead; zero() replaces it afterwards.  The
// two steps are separate so that every load of an iteration can be issued
// before the first value is touched.
template <bool KMAJOR, int V>
__device__ inline unsigned load_block(const float *base, long ld, int x, int X, int k, int K, float (&v)[4]) {
  // x: this lane's row / column, k: first of its four k values (k0 + 4*(lane/32))
  unsigned mask = 0;
  if constexpr (KMAJOR && V == 4) {
    // K and ld are multiples of 4: the vector is inside or outside as a whole
    const bool in = x < X && k < K;
    const float4v t = *reinterpret_cast<const float4v *>(in ? base + k + (long)x * ld : base);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
    mask = in ? 15u : 0u;
  } else {
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const bool in = x < X && k + e < K;
      const long off = KMAJOR ? k + e + (long)x * ld : x + (long)(k + e) * ld;
      v[e] = *(in ? base + off : base);
      mask |= (in ? 1u : 0u) << e;
    }
  }
  return mask;
}

__device__ inline void zero_outside(float (&v)[4], unsigned mask) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = ((mask >> e) & 1u) ? v[e] : 0.0f;
}

template <int TM, int TN, int WAVES>
constexpr int kDirectRedFloats = WAVES * TM * TN * 16 * 64;

// One workgroup's work: workgroup `bid` of the `nblk` that share the problem `d`.
// `red` is LDS for kDirectRedFloats<TM, TN, WAVES> floats, `last_flag` one LDS word.

template <int TM, int TN, int U, bool A_KMAJOR, bool B_KMAJOR, int VA, int VB, int WAVES>
__device__ inline void direct_tile(const DirectArgs &d, float *red, uint32_t *last_flag, int bid, int nblk) {
  const GemmArgs &g = d.g;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;

  int t = xcd_remap(bid, nblk);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * 32 * TM, n0 = tile_n * 32 * TN;

  // chunks [cb, ce) belong to this workgroup; wave w takes cb + w, cb + w + WAVES, ...
  const int cb = (int)((long)split * d.total_chunks / g.splits);
  const int ce = (int)((long)(split + 1) * d.total_chunks / g.splits);

  const float *Az = g.A + (long)z * g.sA;
  const float *Bz = g.B + (long)z * g.sB;
  const int xl = lane & 31, kh = 4 * (lane >> 5);

  float16v acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  for (int c0 = cb + wave; c0 < ce; c0 += WAVES * U) {
    float av[U][TM][4], bv[U][TN][4];
    unsigned am[U][TM], bm[U][TN];
    // all loads of U chunks first ...
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + WAVES * u;
      const bool live = c < ce;
      const int cc = live ? c : cb;
      const int r = cc / d.chunks_per_r;
      // a chunk past the end gets k = K: every element reads as zero
      const int k = live ? (cc - r * d.chunks_per_r) * 8 + kh : g.K;
      const float *Ar = Az + (long)r * g.rA;
      const float *Br = Bz + (long)r * g.rB;
#pragma unroll
      for (int i = 0; i < TM; ++i)
        am[u][i] = load_block<A_KMAJOR, VA>(Ar, g.lda, m0 + i * 32 + xl, g.M, k, g.K, av[u][i]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bm[u][j] = load_block<B_KMAJOR, VB>(Br, g.ldb, n0 + j * 32 + xl, g.N, k, g.K, bv[u][j]);
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the loads above everything that consumes them
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int i = 0; i < TM; ++i) zero_outside(av[u][i], am[u][i]);
#pragma unroll
      for (int j = 0; j < TN; ++j) zero_outside(bv[u][j], bm[u][j]);
    }
    // ... then their matrix instructions
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int e = 0; e < 4; ++e)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            // rows of the instruction's result follow n, its columns follow m
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[u][j][e], av[u][i][e], acc[i][j], 0, 0, 0);
  }

  // Sum the waves' tiles: every wave parks its registers in LDS, then wave w
  // reduces and writes its share of the 16 registers of each 32x32 block.
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) red[(((wave * TM + i) * TN + j) * 16 + v) * 64 + lane] = acc[i][j][v];
  __syncthreads();

  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + 32 * TM <= g.M && n0 + 32 * TN <= g.N;
  constexpr int kShare = 16 / WAVES;  // registers of each block that this wave reduces
  // this wave's share of block (i, j), summed over the waves: values and their column offsets
  auto reduced = [&](int i, int j, float (&vals)[kShare], int (&ns)[kShare]) {
#pragma unroll
    for (int q = 0; q < kShare; ++q) {
      const int v = wave * kShare + q;
      float s = 0.0f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) s += red[(((w * TM + i) * TN + j) * 16 + v) * 64 + lane];
      vals[q] = s;
      ns[q] = 8 * (v / 4) + (v % 4);
    }
  };
  if (g.atomic == 2) {
    // K is split between workgroups: leave the partial tile; the last one of the tile adds them up
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        float vals[kShare];
        int ns[kShare];
        reduced(i, j, vals, ns);
        store_partial<kShare>(g, z, split, m0 + i * 32, n0 + j * 32, lane, ns, vals);
      }
    if (!last_of_tile(g, (z * g.tiles_n + tile_n) * g.tiles_m + tile_m, last_flag)) return;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        float vals[kShare];
        int ns[kShare];
#pragma unroll
        for (int q = 0; q < kShare; ++q) ns[q] = 8 * ((wave * kShare + q) / 4) + ((wave * kShare + q) % 4);
        sum_partials<kShare>(g, z, m0 + i * 32, n0 + j * 32, lane, ns, vals);
        emit_c<kShare>(Cz, g.ldc, m0 + i * 32, n0 + j * 32, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      float vals[kShare];
      int ns[kShare];
      reduced(i, j, vals, ns);
      emit_c<kShare>(Cz, g.ldc, m0 + i * 32, n0 + j * 32, lane, g.M, g.N, interior, ns, vals, g.atomic, g.accumulate);
    }
}

// How a problem is to be run by this kernel: tile shape (32 x 32 TN), chunks
// in flight per wavefront (U), wavefronts per workgroup, K ranges, and whether
// the k-contiguous operands can be read 16 bytes at a time.  `d` is complete
// except for the scratch memory of a split overwriting product.
struct DirectPlan {
  DirectArgs d;
  int tn, u, waves;
  bool vec_a, vec_b;
  long grid;
};

// False when the problem is not one for this kernel (its output alone fills the
// chip with staged tiles, or a k-contiguous operand is not 16-byte aligned).
inline bool plan_direct(const phip_ctx *ctx, const Gemm &p, DirectPlan *plan) {
  const int cus = ctx->prop.multiProcessorCount;
  auto tiles = [&](int bm, int bn) {
    return (long)((p.M + bm - 1) / bm) * ((p.N + bn - 1) / bn) * p.batch;
  };
  // Staged 64x64 tiles already give every CU a workgroup: not skinny.
  if (tiles(64, 64) >= cus) return false;

  DirectArgs &d = plan->d;
  GemmArgs &a = d.g;
  a = problem_args(p);
  a.accumulate = p.accumulate ? 1 : 0;
  a.ktiles_per_r = 0;
  a.total_ktiles = 0;
  a.partial = nullptr;
  a.tickets = ctx->tile_tickets;
  d.chunks_per_r = (p.K + 7) / 8;
  d.total_chunks = d.chunks_per_r * p.rbatch;

  plan->vec_a = p.a_kmajor && rows_aligned16(p.A, 4, p.lda, p.sA, p.rA) && p.K % 4 == 0;
  plan->vec_b = p.b_kmajor && rows_aligned16(p.B, 4, p.ldb, p.sB, p.rB) && p.K % 4 == 0;

  // A k-contiguous operand that cannot be read 16 bytes at a time would be
  // fetched as 4-byte loads scattered over 32 rows; the staged kernel reads
  // such an operand along k and does far better.
  if ((p.a_kmajor && !plan->vec_a) || (p.b_kmajor && !plan->vec_b)) return false;

  // Wide tiles (32 x 64) read the A operand once for 64 columns; use them
  // when they still leave enough workgroups, else 32 x 32.
  const bool wide = p.N > 32 && tiles(32, 64) * 2 >= cus;
  const long t = wide ? tiles(32, 64) : tiles(32, 32);
  // Split K between workgroups until about two workgroups per CU are busy,
  // keeping at least 4 chunks (32 k) per wavefront (measured best on the
  // recurrent-gate and output-projection gradients).  An overwriting product
  // is only split when it would otherwise leave most of the chip idle, or when
  // K is long (from 2048) and the tiles are fewer than the CUs: its ranges meet
  // through partial tiles in scratch memory.
  int splits = 1;
  const long want = (2L * cus + t - 1) / t;
  long cap = d.total_chunks / 16;
  if (cap < 1) cap = 1;
  if (p.accumulate || t * 8 <= cus || (d.total_chunks >= 256 && t < cus)) splits = (int)(want < cap ? want : cap);
  if (splits < 1) splits = 1;
  // An overwriting product whose K fits one round of loads of 8 wavefronts (at
  // most 8 chunks each) takes 8 wavefronts per workgroup.  (16 wavefronts for a
  // longer K measured slower than the split with its zero fill: a 1024-thread
  // workgroup leaves each lane 128 registers, too few for 8 chunks in flight.)
  plan->waves = 4;
  if (!p.accumulate && splits == 1 && d.total_chunks > 32 && d.total_chunks <= 64) plan->waves = 8;
  const long chunks_per_wave = d.total_chunks / ((long)plan->waves * splits);
  plan->u = (plan->waves == 8 || chunks_per_wave > 4) ? 8 : 4;
  plan->tn = wide ? 2 : 1;
  a.tiles_m = (p.M + 31) / 32;
  a.tiles_n = (p.N + 32 * plan->tn - 1) / (32 * plan->tn);
  a.splits = splits;
  a.atomic = splits > 1;
  plan->grid = (long)a.tiles_m * a.tiles_n * p.batch * splits;
  return true;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_DIRECT_H_
