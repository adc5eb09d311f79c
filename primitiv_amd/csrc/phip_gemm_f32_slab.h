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

constexpr int TBN = 64;
constexpr int kSlots = 4;
constexpr int kSubB = TBN * 128;  // bytes of B in one stage
// MB blocks of 32 rows per tile, SA stages of A in flight: bytes of A in one stage, of the kernel's LDS
// (never less than the 32 KiB per block of 32 rows that the final sum over the wavefronts takes)
constexpr int slab_sub_a(int mb) { return mb * 32 * 128; }
constexpr int slab_lds_bytes(int mb, int sa) {
  return sa * slab_sub_a(mb) + kSlots * kSubB > mb * 32768 ? sa * slab_sub_a(mb) + kSlots * kSubB : mb * 32768;
}

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
// Tiles of 32 MB x 64 (MB = 1: the kernel on its own, two workgroups per compute
// unit; MB = 2: twice the bytes of A per stage, for a compute unit that holds
// only one such workgroup).  `lds` holds slab_lds_bytes(MB, SA) (1 KiB aligned),
// `last_flag` is one LDS word.
template <bool A_KMAJOR, bool B_KMAJOR, int MB, int SA>
__device__ inline void slab_tile(const LdsArgs &d, unsigned char *lds, uint32_t *last_flag, int bid, int nblk) {
  constexpr int TBM = 32 * MB;
  constexpr int kSubA = slab_sub_a(MB);
  typedef DmaLoader<A_KMAJOR, TBM> LoaderA;
  typedef DmaLoader<B_KMAJOR, TBN> LoaderB;
  constexpr int kDmaA = LoaderA::kInstr, kDmaB = LoaderB::kInstr;
  constexpr int kDma = kDmaA + kDmaB;  // load instructions per wavefront per stage
  const GemmArgs &g = d.g;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int tile_m, split, z, nsplits;
  if (d.whole_tiles > 0) {
    // Mixed launch (one sample): the first whole_tiles workgroups take a whole tile each, the others
    // one of g.splits K ranges of the remaining tiles.  whole_tiles is a multiple of 8, so both groups
    // meet the XCDs in the same order.
    z = 0;
    if (bid < d.whole_tiles) {
      tile_m = xcd_remap(bid, d.whole_tiles);
      split = 0;
      nsplits = 1;
    } else {
      const int u = xcd_remap(bid - d.whole_tiles, nblk - d.whole_tiles);
      tile_m = d.whole_tiles + u / g.splits;
      split = u % g.splits;
      nsplits = g.splits;
    }
  } else {
    // tiles of one K range are neighbours: they read the same rows of B
    int t = xcd_remap(bid, nblk);
    tile_m = t % g.tiles_m; t /= g.tiles_m;
    split = t % g.splits;
    z = t / g.splits;
    nsplits = g.splits;
  }
  const int m0 = tile_m * TBM;
  // how this workgroup's tile reaches C: 0 stored (or added) by this workgroup alone, 1 atomics, 2 exchange
  const int mode = nsplits > 1 ? g.atomic : 0;

  // K tiles (32 k, one per stage) [kb, ke) belong to this workgroup
  const int kb = (int)((long)split * g.total_ktiles / nsplits);
  const int ke = (int)((long)(split + 1) * g.total_ktiles / nsplits);
  const int n_st = ke - kb;

  LoaderA la;
  LoaderB lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, 0, g.N, wave, lane);
  const uint32_t fa_base = frag_base<A_KMAJOR, TBM>(wave, lane);
  const uint32_t fb_base = frag_base<B_KMAJOR, TBN>(wave, lane);

  float16v acc[MB][2];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  // Two rings of stages in LDS: SA stages of A and kSlots of B are in flight.  A comes from HBM and is
  // read once: what limits the kernel is how many of its bytes are in flight (a stage's loads take
  // about 2 us to land under load), so its ring is as deep as LDS allows; B is re-read by every tile
  // from L2 and needs no more than the four stages its latency asks for.
  // Cursor of the next stage to load, per operand: its K tile, the sample of the contraction it lies
  // in, and that sample's operand.
  struct Cursor {
    int kt, in_r;
    const float *base;
    long per_r;
  };
  const int r0 = kb / g.ktiles_per_r;
  Cursor ca = {kb, kb - r0 * g.ktiles_per_r, g.A + (long)z * g.sA + (long)r0 * g.rA, g.rA};
  Cursor cb = {kb, kb - r0 * g.ktiles_per_r, g.B + (long)z * g.sB + (long)r0 * g.rB, g.rB};
  auto advance = [&](Cursor &c) {
    ++c.kt;
    if (++c.in_r == g.ktiles_per_r) {
      c.in_r = 0;
      c.base += c.per_r;
    }
  };
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  constexpr int kRingB = SA * kSubA;  // B's ring starts behind A's

  // Instruction q of the wave's loads of A's / B's next stage, into that operand's ring slot `slot`.
  auto issue_a = [&](int slot, int q) {
    la.issue(make_rsrc_words(ca.base, d.a_bytes), lds_base + (uint32_t)slot * kSubA, wave, q, ca.in_r, g.K, ca.kt < ke);
  };
  auto issue_b = [&](int slot, int q) {
    lb.issue(make_rsrc_words(cb.base, d.b_bytes), lds_base + kRingB + (uint32_t)slot * kSubB, wave, q, cb.in_r, g.K,
             cb.kt < ke);
  };
  auto next = [](int slot, int ring) { return slot == ring - 1 ? 0 : slot + 1; };

  // A k-contiguous operand whose K is not a multiple of four: in the last K tile
  // of a sample the chunk that holds k = K-1 also holds elements of the next
  // row.  pub_in_r follows the stage that is published next.
  const bool ragged_k = (A_KMAJOR || B_KMAJOR) && (g.K & 3) != 0;
  int pub_in_r = ca.in_r;
  auto publish = [&](int slot_a, int slot_b) {
    if (ragged_k && pub_in_r == g.ktiles_per_r - 1) {
      if constexpr (A_KMAJOR) {
#pragma unroll
        for (int q = 0; q < kDmaA; ++q) la.zero_tail(lds + slot_a * kSubA, wave, q, lane, pub_in_r, g.K);
      }
      if constexpr (B_KMAJOR) {
#pragma unroll
        for (int q = 0; q < kDmaB; ++q) lb.zero_tail(lds + kRingB + slot_b * kSubB, wave, q, lane, pub_in_r, g.K);
      }
    }
    if (++pub_in_r == g.ktiles_per_r) pub_in_r = 0;
  };

  // Fragments of one stage in registers.
  struct Frags {
    float a[MB][4], b[2][4];
  };
  constexpr int kReadsA = MB * kFragReads<A_KMAJOR>, kReadsB = 2 * kFragReads<B_KMAJOR>;
  auto read_one = [&](int slot_a, int slot_b, int r, Frags &f) {
    if (r < kReadsA) frag_read<A_KMAJOR, TBM>(lds + slot_a * kSubA, fa_base, r / kFragReads<A_KMAJOR>, r % kFragReads<A_KMAJOR>, f.a[r / kFragReads<A_KMAJOR>]);
    else frag_read<B_KMAJOR, TBN>(lds + kRingB + slot_b * kSubB, fb_base, (r - kReadsA) / kFragReads<B_KMAJOR>, (r - kReadsA) % kFragReads<B_KMAJOR>, f.b[(r - kReadsA) / kFragReads<B_KMAJOR>]);
  };

  // Loads return in the order of their issue, so "at most N outstanding" names what has landed.
  // Order here: A(0 .. SA-2), B0, B1, B2, A(SA-1), B3; then step l issues A(l+SA), B(l+4).  Stage l's
  // fragments are read one step early, so stages l and l+1 must both have landed behind the barrier
  // that ends step l-1: behind B(l+2) there are then exactly two stages' worth of loads.
  static_assert(SA >= kSlots, "A's ring is at least as deep as B's");
#pragma unroll
  for (int l = 0; l < SA - 1; ++l) {
#pragma unroll
    for (int q = 0; q < kDmaA; ++q) issue_a(l, q);
    advance(ca);
  }
#pragma unroll
  for (int l = 0; l < kSlots; ++l) {
    if (l == kSlots - 1) {
#pragma unroll
      for (int q = 0; q < kDmaA; ++q) issue_a(SA - 1, q);
      advance(ca);
    }
#pragma unroll
    for (int q = 0; q < kDmaB; ++q) issue_b(l, q);
    advance(cb);
  }
  wait_vmcnt_lgkm0<kDmaA + 2 * kDmaB>();  // stages 0 and 1 have landed
  publish(0, 0);
  publish(1, 1);
  __syncthreads();
  Frags f0, f1;
#pragma unroll
  for (int r = 0; r < kReadsA + kReadsB; ++r) read_one(0, 0, r, f0);
  wait_vmcnt_lgkm0<kDmaA + 2 * kDmaB>();  // every wave has stage 0 in registers before its slots are refilled
  __syncthreads();

  // One stage: 8 MB matrix instructions; between them, the loads of A's stage l+SA and B's stage
  // l+kSlots (into the slots this stage leaves) and the fragment reads of stage l+1.
  constexpr int kSide = kDma + kReadsA + kReadsB;
  constexpr int kMfma = 8 * MB;
  int sa = 0, sb = 0;  // ring slots of the stage in progress
  auto step = [&](const Frags &cur, Frags &nxt) {
    const int na = next(sa, SA), nb = next(sb, kSlots);
    // the matrix instructions of a stage go ahead of the other workgroup's loads and bookkeeping on this
    // compute unit (measured on the output projection: 44.6 -> 43.7 us per timestep)
    __builtin_amdgcn_s_setprio(2);
#pragma unroll
    for (int q = 0; q < kMfma; ++q) {
      const int e = q / (2 * MB), i = (q / 2) % MB, j = q & 1;
      // rows of the instruction's result follow n, its columns follow m
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.b[j][e], cur.a[i][e], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int it = (q * kSide) / kMfma; it < ((q + 1) * kSide) / kMfma; ++it) {
        if (it < kDmaA) issue_a(sa, it);
        else if (it < kDma) issue_b(sb, it - kDmaA);
        else read_one(na, nb, it - kDma, nxt);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_setprio(0);
    advance(ca);
    advance(cb);
    // own loads of stage l+2 have landed (later ones may still fly) and own
    // reads of stage l+1 are done; behind the barrier that holds for every wave
    wait_vmcnt_lgkm0<2 * kDma>();
    publish(next(na, SA), next(nb, kSlots));
    __syncthreads();
    sa = na;
    sb = nb;
  };
  for (int l = 0; l < n_st; l += 2) {
    step(f0, f1);
    if (l + 1 < n_st) step(f1, f0);
  }
  // the loads issued for stages past the end move nothing, but must have
  // retired before LDS is reused below
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  // Sum the four waves' tiles: every wave parks its registers in LDS, then
  // wave w reduces and writes registers [4w, 4w+4) of each 32x32 block.
  float *red = reinterpret_cast<float *>(lds);
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) red[((wave * 2 * MB + 2 * i + j) * 16 + v) * 64 + lane] = acc[i][j][v];
  __syncthreads();

  float *Cz = g.C + (long)z * g.sC;
  const bool interior = m0 + TBM <= g.M && TBN <= g.N;
  // this wave's share of block b = 2 i + j, summed over the waves: values and their column offsets
  auto reduced = [&](int b, float (&vals)[4], int (&ns)[4]) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int v = wave * 4 + q;
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < 4; ++w) sum += red[((w * 2 * MB + b) * 16 + v) * 64 + lane];
      vals[q] = sum;
      ns[q] = 8 * (v / 4) + (v % 4);
    }
  };
  if (mode == 2) {
    // K is split between workgroups: leave the partial tile; the last one of the tile adds them up
#pragma unroll
    for (int b = 0; b < 2 * MB; ++b) {
      float vals[4];
      int ns[4];
      reduced(b, vals, ns);
      store_partial<4>(g, z, split, m0 + (b / 2) * 32, (b % 2) * 32, lane, ns, vals);
    }
    if (!last_of_tile(g, z * g.tiles_m + tile_m, last_flag)) return;
#pragma unroll
    for (int b = 0; b < 2 * MB; ++b) {
      float vals[4];
      int ns[4];
#pragma unroll
      for (int q = 0; q < 4; ++q) ns[q] = 8 * ((wave * 4 + q) / 4) + ((wave * 4 + q) % 4);
      sum_partials<4>(g, z, m0 + (b / 2) * 32, (b % 2) * 32, lane, ns, vals);
      emit_c<4>(Cz, g.ldc, m0 + (b / 2) * 32, (b % 2) * 32, lane, g.M, g.N, interior, ns, vals, 0, g.accumulate);
    }
    return;
  }
#pragma unroll
  for (int b = 0; b < 2 * MB; ++b) {
    float vals[4];
    int ns[4];
    reduced(b, vals, ns);
    emit_c<4>(Cz, g.ldc, m0 + (b / 2) * 32, (b % 2) * 32, lane, g.M, g.N, interior, ns, vals, mode, g.accumulate);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

// How a problem is run by this kernel; `d` is complete except for the scratch
// memory of a split overwriting product.
struct SlabPlan {
  LdsArgs d;
  long tiles;  // output tiles (rows of 32) times samples
  long grid;   // tiles times K ranges
};

// False when the problem is not one for this kernel.  `per_cu` workgroups may
// run on each of the `cus` compute units at once (two when the kernel has the
// chip to itself): the K range is cut so that those places are filled at most
// once.
inline bool plan_slab(const Gemm &p, int cus, int per_cu, SlabPlan *plan, int mb = 1) {
  const int TBM = 32 * mb;
  const long places = (long)cus * per_cu;
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
  d.whole_tiles = 0;
  plan->tiles = tiles;
  plan->grid = tiles * splits;
  // More tiles than compute units but fewer than places: unsplit, the compute units that hold two
  // tiles take twice as long as the others (313 tiles of the output projection's forward product on
  // 256 compute units: 57 of them).  Instead every compute unit gets one whole tile, and the tiles
  // that are left are cut into K ranges of at least four stages that fill the second places: the
  // matrix-instruction time per compute unit evens out (21 + 5 stages instead of 42), and the
  // exchange or the atomics of the short workgroups end while the long ones still run.
  const long rest = tiles - cus;
  if (p.batch == 1 && per_cu >= 2 && cus % 8 == 0 && rest > 0 && tiles < 2L * cus) {
    long s = cus / rest;
    if (s > total_ktiles / 4) s = total_ktiles / 4;
    if (s >= 2) {
      d.whole_tiles = cus;
      a.splits = (int)s;
      a.atomic = 1;
      plan->grid = cus + rest * s;
    }
  }
  return true;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_SLAB_H_
