// fp32 GEMM for products that stream one large operand against a narrow one
// (at most 64 columns of output): the per-timestep products of an output
// projection, y = W.x, gx = W^T.gy, whose cost is reading W once.
//
// 32 x 64 output tiles.  Operands move global -> LDS by buffer loads that write
// LDS directly, 16 bytes per lane, in stages of 32 k (A 4 KiB + B 8 KiB); four
// stages are in flight.  The four wavefronts of a workgroup split K: wavefront
// w takes k group w (8 k) of every stage, all 32 x 64 outputs (8 matrix
// instructions per stage), and the four partial tiles are summed through LDS at
// the end.  The fragments of stage l+1 are read, and the loads of stage l+4
// issued, between the matrix instructions of stage l.  When there are fewer
// output tiles than places for workgroups (two per compute unit), the K range
// is also cut between workgroups, whose tiles are added into C with fp32
// atomics; an overwriting product exchanges partial tiles instead.
//
// The 16-byte loads need no more than 4-byte alignment of their global address
// (measured: same results and the same time from rows that start 4 or 8 bytes
// off a 16-byte boundary), so the narrow operand's rows may have any length.  A
// k-contiguous row whose length is not a multiple of four ends inside a 16-byte
// chunk whose other elements belong to the next row: the lane that loaded such
// a chunk overwrites them with zeros in LDS before the stage is published.
#ifndef PHIP_GEMM_F32_SLAB_H_
#define PHIP_GEMM_F32_SLAB_H_

#include "phip_gemm_f32_lds.h"

namespace phip {
namespace {

constexpr int TBM = 32, TBN = 64;
constexpr int kSlots = 4;
constexpr int kSubA = TBM * 128, kSubB = TBN * 128;  // bytes of one stage per operand
constexpr int kSlabStage = kSubA + kSubB;
constexpr int kSlabLdsBytes = kSlots * kSlabStage;

template <int N>
__device__ inline void wait_vmcnt_lgkm0() {
  asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"(N) : "memory");
}

// Byte offsets, inside a stage's operand region, of the fragments of k group
// `group` for the lane: a k-contiguous operand is one 16-byte read (4
// consecutive k of the lane's row, chunk position swizzled as the loader wrote
// it), an m/n-contiguous operand four 4-byte reads one k row apart.
template <bool KMAJOR, int ROWS>
__device__ inline uint32_t frag_base(int group, int lane) {
  const int xl = lane & 31, half = lane >> 5;
  if constexpr (KMAJOR) return (uint32_t)(xl * 128 + (((2 * group + half) ^ ((xl >> 1) & 7)) * 16));
  else return (uint32_t)((8 * group + 4 * half) * (ROWS * 4) + xl * 4);
}

// LDS reads that fetch the fragments of one 32-row block.
template <bool KMAJOR>
constexpr int kFragReads = KMAJOR ? 1 : 4;

// Read r of them.
template <bool KMAJOR, int ROWS>
__device__ inline void frag_read(const unsigned char *region, uint32_t base, int block, int r, float (&v)[4]) {
  if constexpr (KMAJOR) {
    const float4v t = *reinterpret_cast<const float4v *>(region + base + block * 4096);
    v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
  } else {
    v[r] = *reinterpret_cast<const float *>(region + base + r * (ROWS * 4) + block * 128);
  }
}

// One workgroup's work: workgroup `bid` of the `nblk` that share the problem `d`.
// `lds` holds kSlabLdsBytes (1 KiB aligned), `last_flag` is one LDS word.
template <bool A_KMAJOR, bool B_KMAJOR>
__device__ inline void slab_tile(const LdsArgs &d, unsigned char *lds, uint32_t *last_flag, int bid, int nblk) {
  typedef DmaLoader<A_KMAJOR, TBM> LoaderA;
  typedef DmaLoader<B_KMAJOR, TBN> LoaderB;
  constexpr int kDmaB = LoaderB::kInstr;
  constexpr int kDma = 1 + kDmaB;  // load instructions per wavefront per stage
  const GemmArgs &g = d.g;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // tiles of one K range are neighbours: they read the same rows of B
  int t = xcd_remap(bid, nblk);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * TBM;

  // K tiles (32 k, one per stage) [kb, ke) belong to this workgroup
  const int kb = (int)((long)split * g.total_ktiles / g.splits);
  const int ke = (int)((long)(split + 1) * g.total_ktiles / g.splits);
  const int n_st = ke - kb;

  LoaderA la;
  LoaderB lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, 0, g.N, wave, lane);
  const uint32_t fa_base = frag_base<A_KMAJOR, TBM>(wave, lane);
  const uint32_t fb_base = frag_base<B_KMAJOR, TBN>(wave, lane);

  float16v acc[2];
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.0f;

  // The next stage to load: its K tile, the sample of the contraction it lies
  // in, and that sample's operands.
  int nx_kt = kb;
  int nx_r = kb / g.ktiles_per_r;
  int nx_in_r = kb - nx_r * g.ktiles_per_r;
  const float *nx_a = g.A + (long)z * g.sA + (long)nx_r * g.rA;
  const float *nx_b = g.B + (long)z * g.sB + (long)nx_r * g.rB;
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;

  // Instruction q (0: A, 1..: B) of the wave's loads of the next stage, into LDS slot `slot`.
  auto issue_one = [&](int slot, int q) {
    const bool live = nx_kt < ke;
    const uint32_t stage = lds_base + (uint32_t)slot * kSlabStage;
    if (q == 0) la.issue(make_rsrc_words(nx_a, d.a_bytes), stage, wave, 0, nx_in_r, g.K, live);
    else lb.issue(make_rsrc_words(nx_b, d.b_bytes), stage + kSubA, wave, q - 1, nx_in_r, g.K, live);
  };
  auto advance = [&]() {
    ++nx_kt;
    if (++nx_in_r == g.ktiles_per_r) {
      nx_in_r = 0;
      nx_a += g.rA;
      nx_b += g.rB;
    }
  };

  // A k-contiguous operand whose K is not a multiple of four: in the last K tile
  // of a sample the chunk that holds k = K-1 also holds elements of the next
  // row.  pub_in_r follows the stage that is published next.
  const bool ragged_k = (A_KMAJOR || B_KMAJOR) && (g.K & 3) != 0;
  int pub_in_r = nx_in_r;
  auto publish = [&](int slot) {
    if (ragged_k && pub_in_r == g.ktiles_per_r - 1) {
      unsigned char *stage = lds + slot * kSlabStage;
      if constexpr (A_KMAJOR) la.zero_tail(stage, wave, 0, lane, pub_in_r, g.K);
      if constexpr (B_KMAJOR) {
#pragma unroll
        for (int q = 0; q < kDmaB; ++q) lb.zero_tail(stage + kSubA, wave, q, lane, pub_in_r, g.K);
      }
    }
    if (++pub_in_r == g.ktiles_per_r) pub_in_r = 0;
  };

  // Fragments of one stage in registers.
  struct Frags {
    float a[4], b[2][4];
  };
  constexpr int kReadsA = kFragReads<A_KMAJOR>, kReadsB = 2 * kFragReads<B_KMAJOR>;
  auto read_one = [&](int slot, int r, Frags &f) {
    const unsigned char *st = lds + slot * kSlabStage;
    if (r < kReadsA) frag_read<A_KMAJOR, TBM>(st, fa_base, 0, r, f.a);
    else frag_read<B_KMAJOR, TBN>(st + kSubA, fb_base, (r - kReadsA) / kFragReads<B_KMAJOR>, (r - kReadsA) % kFragReads<B_KMAJOR>, f.b[(r - kReadsA) / kFragReads<B_KMAJOR>]);
  };

  // kSlots stages are in flight.  Stage l's fragments are read one iteration
  // early, so stages l and l+1 must both have landed behind the barrier that
  // ends iteration l-1.
#pragma unroll
  for (int l = 0; l < kSlots; ++l) {
#pragma unroll
    for (int q = 0; q < kDma; ++q) issue_one(l, q);
    advance();
  }
  wait_vmcnt_lgkm0<(kSlots - 2) * kDma>();  // stages 0 and 1 have landed
  publish(0);
  publish(1);
  __syncthreads();
  Frags f0, f1;
#pragma unroll
  for (int r = 0; r < kReadsA + kReadsB; ++r) read_one(0, r, f0);
  wait_vmcnt_lgkm0<(kSlots - 2) * kDma>();  // every wave has slot 0 in registers before it is refilled
  __syncthreads();

  // One stage: 8 matrix instructions; between them, the loads of stage
  // l+kSlots (into the slot this stage leaves) and the fragment reads of stage l+1.
  constexpr int kSide = kDma + kReadsA + kReadsB;
  auto step = [&](int slot, const Frags &cur, Frags &nxt) {
    const int nslot = slot == kSlots - 1 ? 0 : slot + 1;
#pragma unroll
    for (int q = 0; q < 8; ++q) {
      const int e = q >> 1, j = q & 1;
      // rows of the instruction's result follow n, its columns follow m
      acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.b[j][e], cur.a[e], acc[j], 0, 0, 0);
#pragma unroll
      for (int it = (q * kSide) / 8; it < ((q + 1) * kSide) / 8; ++it) {
        if (it < kDma) issue_one(slot, it);
        else read_one(nslot, it - kDma, nxt);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    advance();
    // own loads of stage l+2 have landed (later ones may still fly) and own
    // reads of stage l+1 are done; behind the barrier that holds for every wave
    wait_vmcnt_lgkm0<(kSlots - 2) * kDma>();
    publish(nslot == kSlots - 1 ? 0 : nslot + 1);
    __syncthreads();
  };
  int slot = 0;
  for (int l = 0; l < n_st; l += 2) {
    step(slot, f0, f1);
    slot = slot == kSlots - 1 ? 0 : slot + 1;
    if (l + 1 < n_st) {
      step(slot, f1, f0);
      slot = slot == kSlots - 1 ? 0 : slot + 1;
    }
  }
  // the loads issued for stages past the end move nothing, but must have
  // retired before LDS is reused below
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // Sum the four waves' tiles: every wave parks its registers in LDS, then
  // wave w reduces and writes registers [4w, 4w+4) of each 32x32 block.
  float *red = reinterpret_cast<float *>(lds);
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) red[((wave * 2 + j) * 16 + v) * 64 + lane] = acc[j][v];
  __syncthreads();

  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + TBM <= g.M && TBN <= g.N;
  // this wave's share of block j, summed over the waves: values and their column offsets
  auto reduced = [&](int j, float (&vals)[4], int (&ns)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int v = wave * 4 + q;
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < 4; ++w) sum += red[((w * 2 + j) * 16 + v) * 64 + lane];
      vals[q] = sum;
      ns[q] = 8 * (v / 4) + (v % 4);
    }
  };
  if (g.atomic == 2) {
    // K is split between workgroups: leave the partial tile; the last one of the tile adds them up
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float vals[4];
      int ns[4];
      reduced(j, vals, ns);
      store_partial<4>(g, z, split, m0, j * 32, lane, ns, vals);
    }
    if (!last_of_tile(g, z * g.tiles_m + tile_m, last_flag)) return;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float vals[4];
      int ns[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) ns[q] = 8 * ((wave * 4 + q) / 4) + ((wave * 4 + q) % 4);
      sum_partials<4>(g, z, m0, j * 32, lane, ns, vals);
      emit_c<4>(Cz, g.ldc, m0, j * 32, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    float vals[4];
    int ns[4];
    reduced(j, vals, ns);
    emit_c<4>(Cz, g.ldc, m0, j * 32, lane, g.M, g.N, interior, ns, vals, g.atomic, g.accumulate);
  }
}

// How a problem is run by this kernel; `d` is complete except for the scratch
// memory of a split overwriting product.
struct SlabPlan {
  LdsArgs d;
  long tiles;  // output tiles (rows of 32) times samples
  long grid;   // tiles times K ranges
};

// False when the problem is not one for this kernel.  `places` is the number of
// workgroups that may run at once (two per compute unit when the kernel has the
// chip to itself): the K range is cut so that they are filled at most once.
inline bool plan_slab(const Gemm &p, long places, SlabPlan *plan) {
  if (p.N > TBN) return false;
  if (p.a_kmajor && !p.b_kmajor) return false;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return false;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return false;
  // worth it when reading A is the cost: a large A and enough K tiles to pipeline
  const int ktiles_per_r = (p.K + LBK - 1) / LBK;
  const long total_ktiles = (long)ktiles_per_r * p.rbatch;
  const long tiles = (long)((p.M + TBM - 1) / TBM) * p.batch;
  if (a_bytes * p.rbatch * p.batch < kStreamedOperandBytes || total_ktiles > 0x7fffffffL || tiles > 0x3fffffffL) return false;
  // fill the places at most once (a workgroup that has to wait for a place doubles the launch's
  // duration), at least eight stages each
  long splits = places / tiles;
  if (splits > total_ktiles / 8) splits = total_ktiles / 8;
  if (splits < 1) splits = 1;

  LdsArgs &d = plan->d;
  GemmArgs &a = d.g;
  a = problem_args(p);
  a.tiles_m = (p.M + TBM - 1) / TBM;
  a.tiles_n = 1;
  a.splits = (int)splits;
  a.ktiles_per_r = ktiles_per_r;
  a.total_ktiles = (int)total_ktiles;
  a.atomic = splits > 1;
  a.accumulate = p.accumulate ? 1 : 0;
  a.partial = nullptr;
  a.tickets = nullptr;
  d.a_bytes = (uint32_t)a_bytes;
  d.b_bytes = (uint32_t)b_bytes;
  plan->tiles = tiles;
  plan->grid = tiles * splits;
  return true;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_SLAB_H_
