// GEMM for 16-bit storage (fp16 / bf16, fp32 accumulation) when one side of the output is narrow:
// the per-timestep products of recurrent layers and output projections (a minibatch of at most a
// few hundred columns against a weight matrix), forward and both gradients.
//
// With 16-bit operands these products have next to no arithmetic (a 10000 x 650 weight matrix
// against 64 columns is 0.7 us of matrix instructions); what a launch costs is its latency.  So
// the kernel does one round of everything:
//  * 64 x 64 output tiles, four wavefronts of 32 x 32 (2 x 2 blocks of v_mfma_f32_16x16x32);
//  * a workgroup owns a range of at most kMaxStages K tiles of 64 and issues EVERY global -> LDS load
//    of that range before it waits for any (buffer loads that write LDS directly, 16 bytes per
//    lane, 16 KiB per K tile): one wait, one barrier, then the matrix instructions straight out of
//    LDS - no ring of stages, no bookkeeping inside a loop;
//  * an operand that is contiguous along k is read back with 16-byte LDS reads, one that is
//    contiguous along m or n is kept as it lies in memory and transposed by the LDS read
//    (ds_read_b64_tr_b16), as in the large-tile kernel;
//  * when K is longer than a workgroup's range (or the tiles alone leave the chip idle) the K
//    range is cut between workgroups: each leaves its fp32 tile in scratch memory and draws a
//    ticket, the one that draws a tile's last ticket adds the tiles in order, adds C's old value if
//    the product accumulates, and rounds once.  No atomics on C (there are none for 16-bit
//    values), the same bits on every run.
// Small outputs take a second shape of the same idea: 32 x 32 tiles whose four wavefronts split the K range
// between them (each holds the whole tile, 8 KiB per K tile, up to 18 K tiles resident) and add their tiles
// through LDS - four times the workgroups for the same output, and K ranges twice as long before anything
// has to go through memory.
// Rows may have any even length: the 16-byte loads need 4-byte alignment only, every load's whole
// offset is checked against the operand's size (what lies outside reads as zero), and a
// k-contiguous row that ends inside a 16-byte chunk has the rest of that chunk masked in
// registers.
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));
typedef short short4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int TM = 64, TN = 64, BK = 64;
constexpr int kRegion = 64 * BK * 2;   // bytes of one operand's K tile in LDS
constexpr int kStage = 2 * kRegion;    // A then B
constexpr int kMaxStages = 9;          // 144 KiB
constexpr uint32_t kOutOfRange = 0x80000000u;  // beyond any operand this kernel accepts

struct SkinnyArgs {
  const uint16_t *A;
  const uint16_t *B;
  uint16_t *C;
  int M, N, K;
  long lda, ldb, ldc;
  long sA, sB, sC;
  long rA, rB;
  int tiles_m, tiles_n;
  int splits;        // workgroups per output tile, each with its own K range
  int ktiles_per_r;  // ceil(K / BK)
  int total_ktiles;  // ktiles_per_r * rbatch
  int accumulate;
  int vec_c;         // C may be moved 8 bytes (4 rows of a column) at a time
  int small;         // 32 x 32 tiles with the wavefronts splitting K (skinny_tile_small) instead of 64 x 64
  uint32_t a_bytes, b_bytes;  // bytes of one sample of each operand
  float *partial;    // splits > 1: 64 x 64 fp32 tiles, ((z * tiles + tile) * splits + split) * 4096 floats each
  uint32_t *tickets; // splits > 1: one zeroed counter per output tile, left zeroed
};

template <class T>
__device__ inline __attribute__((address_space(3))) T *lds_ptr(uint32_t addr) {
  return (__attribute__((address_space(3))) T *)(size_t)addr;
}

__device__ inline int xcd_remap(int bid, int total) {
  constexpr int kXcds = 8;
  const int xcd = bid % kXcds;
  const int idx = bid / kXcds;
  const int q = total / kXcds, rem = total % kXcds;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

__device__ inline uint4v make_rsrc_words(const uint16_t *p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  uint4v r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
  return r;
}

// One 16-byte-per-lane buffer load whose destination is LDS: lane l's data lands at lds_addr + 16 l
// and comes from base + voffset; a voffset at or past the buffer's size yields zeros.
__device__ inline void lds_dma_b128(uint4v rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");  // m0 is scratch between instructions: nothing else in this kernel keeps a value in it
}

// A wavefront's two load instructions per operand and K tile (1 KiB of LDS each; the four wavefronts
// fill the 8 KiB region).  LDS image:
//  * k-contiguous operand: 64 rows (m or n) of 64 k = 128 bytes = 8 chunks; chunk c of row x sits at
//    position c ^ ((x >> 1) & 7);
//  * m/n-contiguous operand: 64 rows (k) of 64 elements = 8 chunks; chunk c of row k sits at
//    position c ^ ((k & 3) << 1), so the four k rows that the 16 lanes of a transposing read touch
//    lie in different banks.
// The swizzle is applied by choosing which global chunk a lane fetches.
template <bool KMAJOR>
struct Loader {
  uint32_t off[2];   // byte offset at K tile 0, or kOutOfRange where the row / column is outside the matrix
  int kpos[2];       // first k (inside a K tile) of the lane's chunk / the lane's k row
  uint32_t step;     // bytes per K tile

  __device__ inline void init(long ld, int x0, int X, int wave, int lane) {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      const int blk = wave * 2 + q;
      if constexpr (KMAJOR) {
        const int x = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((x >> 1) & 7);
        off[q] = x0 + x < X ? (uint32_t)(((long)(x0 + x) * ld + c * 8) * 2) : kOutOfRange;
        kpos[q] = c * 8;
      } else {
        const int k = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((k & 3) << 1);
        off[q] = x0 + c * 8 < X ? (uint32_t)(((long)k * ld + x0 + c * 8) * 2) : kOutOfRange;
        kpos[q] = k;
      }
    }
    step = KMAJOR ? (uint32_t)(BK * 2) : (uint32_t)(BK * ld * 2);
  }

  // Instruction q for K tile `kin` of a sample with K columns, into the operand's region at lds_region.
  __device__ inline void issue(uint4v rsrc, uint32_t lds_region, int wave, int q, int kin, int K) const {
    const bool inside = kin * BK + kpos[q] < K;
    const uint32_t v = inside ? off[q] + (uint32_t)kin * step : kOutOfRange;
    lds_dma_b128(rsrc, lds_region + (uint32_t)((wave * 2 + q) * 1024), v | (off[q] & kOutOfRange));
  }
};

// Fragment of the 16-row block that starts at row xb of the operand's tile, k step t (32 k) of the K
// tile in `region`: 8 consecutive k, from 8 (lane / 16) on, of row xb + lane % 16.
template <bool KMAJOR>
__device__ inline uint4v read_fragment(uint32_t region, int xb, int t, int lane) {
  if constexpr (KMAJOR) {
    const int x = xb + (lane & 15);
    return *lds_ptr<const uint4v>(region + (uint32_t)(x * 128 + (((4 * t + (lane >> 4)) ^ ((x >> 1) & 7)) * 16)));
  } else {
    // lane = 16 g + 4 cc + a supplies k row 8 g + cc (and the one 4 further on), columns 4 a .. + 3 of the block
    const int g = lane >> 4, cc = (lane & 15) >> 2, a = lane & 3;
    const uint32_t p = region + (uint32_t)((32 * t + 8 * g + cc) * 128 + (((xb / 8 + (a >> 1)) ^ (2 * cc)) * 16) + (a & 1) * 8);
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p + 4 * 128));
    uint4v r;
    r.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
    r.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
    r.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
    r.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
    return r;
  }
}

// Keeps the first `valid` (0 .. 8) of a fragment's 8 values, zeros the rest.
__device__ inline uint4v keep_first(uint4v f, int valid) {
  uint4v r;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    const int n = valid - 2 * w;
    r[w] = n >= 2 ? f[w] : (n == 1 ? (f[w] & 0xffffu) : 0u);
  }
  return r;
}

// 16 bytes to / from memory at device scope (past the per-XCD L2s), as the partial tiles of a split
// product travel.  The loads are not tracked by the compiler: the caller waits (wait_loads) before it
// reads what they return.
// (A store of more than 8 bytes reads its data registers a little after it has issued; the compiler keeps
// the next write of those registers away from stores it knows, the wait states here do it for this one.)
__device__ inline void store_device_scope(float *p, float4v v) {
  asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 2" : : "v"(p), "v"(v) : "memory");
}
// The four 16-byte pieces (1 KiB apart) of each of four partial tiles, all sixteen loads in flight at
// once, and the wait for them, in one statement: the compiler sees values that are there.
__device__ inline void load_four_tiles_device_scope(float4v (&v)[4][4], const float *q0, const float *q1,
                                                    const float *q2, const float *q3) {
  asm volatile(
      "global_load_dwordx4 %0, %16, off sc1\n\t"
      "global_load_dwordx4 %1, %16, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %2, %16, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %3, %16, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %4, %17, off sc1\n\t"
      "global_load_dwordx4 %5, %17, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %6, %17, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %7, %17, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %8, %18, off sc1\n\t"
      "global_load_dwordx4 %9, %18, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %10, %18, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %11, %18, off offset:3072 sc1\n\t"
      "global_load_dwordx4 %12, %19, off sc1\n\t"
      "global_load_dwordx4 %13, %19, off offset:1024 sc1\n\t"
      "global_load_dwordx4 %14, %19, off offset:2048 sc1\n\t"
      "global_load_dwordx4 %15, %19, off offset:3072 sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(v[0][0]), "=&v"(v[0][1]), "=&v"(v[0][2]), "=&v"(v[0][3]), "=&v"(v[1][0]), "=&v"(v[1][1]), "=&v"(v[1][2]),
        "=&v"(v[1][3]), "=&v"(v[2][0]), "=&v"(v[2][1]), "=&v"(v[2][2]), "=&v"(v[2][3]), "=&v"(v[3][0]), "=&v"(v[3][1]),
        "=&v"(v[3][2]), "=&v"(v[3][3])
      : "v"(q0), "v"(q1), "v"(q2), "v"(q3)
      : "memory");
}

template <bool BF16>
__device__ inline float4v mfma(uint4v a, uint4v b, float4v c) {
  if constexpr (BF16) return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf8v, a), __builtin_bit_cast(bf8v, b), c, 0, 0, 0);
  else return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8v, a), __builtin_bit_cast(half8v, b), c, 0, 0, 0);
}

template <bool BF16>
__device__ inline float widen(uint32_t bits16) {
  if constexpr (BF16) return __builtin_bit_cast(float, bits16 << 16);
  else return to_f32(__builtin_bit_cast(f16_t, (uint16_t)bits16));
}

// One value rounded to nearest even, as 16 bits.
template <bool BF16>
__device__ inline uint32_t narrow(float x) {
  if constexpr (BF16) return from_f32<bf16_t>(x).bits;
  else return __builtin_bit_cast(uint16_t, from_f32<f16_t>(x));
}

// One workgroup's work: workgroup `bid` of the `nblk` that share the problem.  `lds` holds
// (stages of the longest K range) x kStage bytes, 1 KiB aligned; `flag` is one LDS word.
template <bool A_KMAJOR, bool B_KMAJOR, bool BF16>
__device__ inline void skinny_tile(const SkinnyArgs &g, unsigned char *lds, uint32_t *flag, int bid, int nblk) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  int t = xcd_remap(bid, nblk);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * TM, n0 = tile_n * TN;

  const int kb = (int)((long)split * g.total_ktiles / g.splits);
  const int ke = (int)((long)(split + 1) * g.total_ktiles / g.splits);
  const int n_st = ke - kb;

  Loader<A_KMAJOR> la;
  Loader<B_KMAJOR> lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, n0, g.N, wave, lane);
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;

  // every load of the workgroup's K range, then one wait
  {
    int r = kb / g.ktiles_per_r, kin = kb - r * g.ktiles_per_r;
    for (int s = 0; s < n_st; ++s) {
      const uint4v ra = make_rsrc_words(Az + (long)r * g.rA, g.a_bytes);
      const uint4v rb = make_rsrc_words(Bz + (long)r * g.rB, g.b_bytes);
      const uint32_t stage = lds_base + (uint32_t)s * kStage;
#pragma unroll
      for (int q = 0; q < 2; ++q) la.issue(ra, stage, wave, q, kin, g.K);
#pragma unroll
      for (int q = 0; q < 2; ++q) lb.issue(rb, stage + kRegion, wave, q, kin, g.K);
      if (++kin == g.ktiles_per_r) {
        kin = 0;
        ++r;
      }
    }
  }
  // C's old values (an accumulating product) have the longest way to come of everything the epilogue
  // needs: fetched now, behind the operands' loads, they arrive under the same wait.  (Only the workgroup
  // that writes a tile touches that part of C in this launch, so the values stay current.)
  uint16_t *Cz = g.C + (long)z * g.sC;
  const int g4 = lane >> 4, nl = lane & 15;
  uint2v old[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = m0 + wm * 32 + 16 * i + 4 * g4;
      const int n = n0 + wn * 32 + 16 * j + nl;
      old[i][j] = uint2v{0u, 0u};
      if (g.accumulate && g.vec_c && n < g.N && m + 4 <= g.M) old[i][j] = *reinterpret_cast<const uint2v *>(Cz + m + (long)n * g.ldc);
    }
  float4v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();

  {
    const bool ragged = (A_KMAJOR || B_KMAJOR) && (g.K & 7) != 0;
    int kin = kb % g.ktiles_per_r;
    for (int s = 0; s < n_st; ++s) {
      const uint32_t stage = lds_base + (uint32_t)s * kStage;
      const bool tail = ragged && kin == g.ktiles_per_r - 1;  // the same for the whole workgroup
#pragma unroll
      for (int tt = 0; tt < 2; ++tt) {
        uint4v fa[2], fb[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[i] = read_fragment<A_KMAJOR>(stage, wm * 32 + 16 * i, tt, lane);
#pragma unroll
        for (int j = 0; j < 2; ++j) fb[j] = read_fragment<B_KMAJOR>(stage + kRegion, wn * 32 + 16 * j, tt, lane);
        if (tail) {
          // a k-contiguous row ends inside this chunk: what follows belongs to the next row
          int valid = g.K - (kin * BK + 32 * tt + 8 * (lane >> 4));
          valid = valid < 0 ? 0 : (valid > 8 ? 8 : valid);
          if constexpr (A_KMAJOR) {
#pragma unroll
            for (int i = 0; i < 2; ++i) fa[i] = keep_first(fa[i], valid);
          }
          if constexpr (B_KMAJOR) {
#pragma unroll
            for (int j = 0; j < 2; ++j) fb[j] = keep_first(fb[j], valid);
          }
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = mfma<BF16>(fa[i], fb[j], acc[i][j]);
      }
      if (++kin == g.ktiles_per_r) kin = 0;
    }
  }

  // K cut between workgroups: leave the fp32 tile as the registers hold it; whoever draws the tile's last
  // ticket adds the tiles of all ranges in order.  Device-scope accesses: the workgroups of a tile run on
  // XCDs with separate L2s, and publishing with fences would write back a whole L2 per workgroup.
  if (g.splits > 1) {
    const long tile_id = ((long)z * g.tiles_n + tile_n) * g.tiles_m + tile_m;
    float *P = g.partial + (tile_id * g.splits + split) * (long)(TM * TN) + wave * 1024 + lane * 4;
    // the stores below are assembly that the compiler does not look into: it would not keep the distance
    // that a matrix instruction's result needs before a memory instruction reads it
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) store_device_scope(P + (i * 2 + j) * 256, acc[i][j]);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own stores acknowledged before the ticket
    __syncthreads();
    if (tid == 0) {
      const uint32_t ticket = __hip_atomic_fetch_add(g.tickets + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = ticket == (uint32_t)g.splits - 1u;
      if (last) __hip_atomic_store(g.tickets + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*flag == 0) return;
    const float *Q = g.partial + tile_id * g.splits * (long)(TM * TN) + wave * 1024 + lane * 4;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};
    // four ranges at a time: sixteen 16-byte loads in flight per lane, added in the order of the ranges
    for (int r0 = 0; r0 < g.splits; r0 += 4) {
      float4v part[4][4];
      const float *q[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) q[u] = Q + (long)(r0 + u < g.splits ? r0 + u : r0) * (TM * TN);
      load_four_tiles_device_scope(part, q[0], q[1], q[2], q[3]);
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (r0 + u < g.splits) {
#pragma unroll
          for (int e = 0; e < 4; ++e) acc[e >> 1][e & 1] += part[u][e];
        }
    }
  }

  // C: block (i, j) holds rows 16 i + 4 (lane / 16) .. + 3 of column 16 j + lane % 16 of the wavefront's 32 x 32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int m = m0 + wm * 32 + 16 * i + 4 * g4;
      const int n = n0 + wn * 32 + 16 * j + nl;
      if (n >= g.N || m >= g.M) continue;
      uint16_t *p = Cz + m + (long)n * g.ldc;
      if (g.vec_c && m + 4 <= g.M) {
        uint2v out;
#pragma unroll
        for (int w = 0; w < 2; ++w) {
          float x0 = acc[i][j][2 * w], x1 = acc[i][j][2 * w + 1];
          if (g.accumulate) {
            x0 += widen<BF16>(old[i][j][w] & 0xffffu);
            x1 += widen<BF16>(old[i][j][w] >> 16);
          }
          out[w] = narrow<BF16>(x0) | (narrow<BF16>(x1) << 16);
        }
        *reinterpret_cast<uint2v *>(p) = out;
      } else {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          if (m + v < g.M) {
            float x = acc[i][j][v];
            if (g.accumulate) x += widen<BF16>(p[v]);
            p[v] = (uint16_t)narrow<BF16>(x);
          }
        }
      }
    }
}

// ---- 32 x 32 tiles, the wavefronts split K ---------------------------------------------------------------

constexpr int SM = 32, SN = 32;
constexpr int kRegionS = 32 * BK * 2;  // bytes of one operand's K tile: 32 rows (m or n) x 64 k
constexpr int kStageS = 2 * kRegionS;
constexpr int kMaxStagesS = 18;        // 144 KiB
constexpr int kRoundS = 9;             // a longer K range is walked in rounds of this many K tiles, two rounds resident
constexpr int kMaxRoundsS = 5;
constexpr int kReduceBytesS = 16384;   // the four wavefronts' tiles, when they are added up

// One piece (16 bytes per lane) of each of eight partial tiles, all in flight at once, and the wait.
__device__ inline void load_eight_device_scope(float4v (&v)[8], const float *const (&q)[8]) {
  asm volatile(
      "global_load_dwordx4 %0, %8, off sc1\n\t"
      "global_load_dwordx4 %1, %9, off sc1\n\t"
      "global_load_dwordx4 %2, %10, off sc1\n\t"
      "global_load_dwordx4 %3, %11, off sc1\n\t"
      "global_load_dwordx4 %4, %12, off sc1\n\t"
      "global_load_dwordx4 %5, %13, off sc1\n\t"
      "global_load_dwordx4 %6, %14, off sc1\n\t"
      "global_load_dwordx4 %7, %15, off sc1\n\t"
      "s_waitcnt vmcnt(0)"
      : "=&v"(v[0]), "=&v"(v[1]), "=&v"(v[2]), "=&v"(v[3]), "=&v"(v[4]), "=&v"(v[5]), "=&v"(v[6]), "=&v"(v[7])
      : "v"(q[0]), "v"(q[1]), "v"(q[2]), "v"(q[3]), "v"(q[4]), "v"(q[5]), "v"(q[6]), "v"(q[7])
      : "memory");
}

// A wavefront's one load instruction per operand and K tile (the four wavefronts fill the 4 KiB region).
//  * k-contiguous operand: 32 rows of 128 bytes, chunk c of row x at position c ^ ((x >> 1) & 7);
//  * m/n-contiguous operand: 64 rows (k) of 32 elements = 4 chunks; chunk c of row k at position
//    c ^ (((k >> 1) & 1) << 1): the four k rows of a transposing read land in different banks.
template <bool KMAJOR>
struct LoaderS {
  uint32_t off;
  int kpos;
  uint32_t step;

  __device__ inline void init(long ld, int x0, int X, int wave, int lane) {
    if constexpr (KMAJOR) {
      const int x = wave * 8 + (lane >> 3);
      const int c = (lane & 7) ^ ((x >> 1) & 7);
      off = x0 + x < X ? (uint32_t)(((long)(x0 + x) * ld + c * 8) * 2) : kOutOfRange;
      kpos = c * 8;
    } else {
      const int k = wave * 16 + (lane >> 2);
      const int c = (lane & 3) ^ (((k >> 1) & 1) << 1);
      off = x0 + c * 8 < X ? (uint32_t)(((long)k * ld + x0 + c * 8) * 2) : kOutOfRange;
      kpos = k;
    }
    step = KMAJOR ? (uint32_t)(BK * 2) : (uint32_t)(BK * ld * 2);
  }

  __device__ inline void issue(uint4v rsrc, uint32_t lds_region, int wave, int kin, int K) const {
    const bool inside = kin * BK + kpos < K;
    const uint32_t v = inside ? off + (uint32_t)kin * step : kOutOfRange;
    lds_dma_b128(rsrc, lds_region + (uint32_t)(wave * 1024), v | (off & kOutOfRange));
  }
};

template <bool KMAJOR>
__device__ inline uint4v read_fragment_small(uint32_t region, int xb, int t, int lane) {
  if constexpr (KMAJOR) {
    return read_fragment<true>(region, xb, t, lane);  // the same image: rows of 128 bytes
  } else {
    const int g = lane >> 4, cc = (lane & 15) >> 2, a = lane & 3;
    const uint32_t p = region + (uint32_t)((32 * t + 8 * g + cc) * 64 + (((xb / 8 + (a >> 1)) ^ (((cc >> 1) & 1) << 1)) * 16) + (a & 1) * 8);
    const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p));
    const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p + 4 * 64));
    uint4v r;
    r.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
    r.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
    r.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
    r.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
    return r;
  }
}

// One workgroup's work on a 32 x 32 tile.  `lds` holds max(stages x kStageS, kReduceBytesS) bytes.
template <bool A_KMAJOR, bool B_KMAJOR, bool BF16>
__device__ inline void skinny_tile_small(const SkinnyArgs &g, unsigned char *lds, uint32_t *flag, int bid, int nblk) {
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  int t = xcd_remap(bid, nblk);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * SM, n0 = tile_n * SN;

  const int kb = (int)((long)split * g.total_ktiles / g.splits);
  const int ke = (int)((long)(split + 1) * g.total_ktiles / g.splits);
  const int n_st = ke - kb;

  LoaderS<A_KMAJOR> la;
  LoaderS<B_KMAJOR> lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, n0, g.N, wave, lane);
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;
  // after the sum over the wavefronts, wavefront w owns the 16 x 16 block (w / 2, w % 2) of the tile
  uint16_t *Cz = g.C + (long)z * g.sC;
  const int g4 = lane >> 4, nl = lane & 15;
  const int m = m0 + 16 * (wave >> 1) + 4 * g4;
  const int n = n0 + 16 * (wave & 1) + nl;
  // C's old values first: they have the longest way to come, and as the oldest load they are covered by
  // every wait for operands below
  uint2v old = {0u, 0u};
  if (g.accumulate && g.vec_c && n < g.N && m + 4 <= g.M) old = *reinterpret_cast<const uint2v *>(Cz + m + (long)n * g.ldc);

  // K tiles [first, first + count) of the workgroup's range into LDS from `slot` on: two loads per wavefront
  // and K tile
  auto issue_stages = [&](int first, int count, int slot) {
    const int kt = kb + first;
    int r = kt / g.ktiles_per_r, kin = kt - r * g.ktiles_per_r;
    for (int s = 0; s < count; ++s) {
      const uint4v ra = make_rsrc_words(Az + (long)r * g.rA, g.a_bytes);
      const uint4v rb = make_rsrc_words(Bz + (long)r * g.rB, g.b_bytes);
      const uint32_t stage = lds_base + (uint32_t)(slot + s) * kStageS;
      la.issue(ra, stage, wave, kin, g.K);
      lb.issue(rb, stage + kRegionS, wave, kin, g.K);
      if (++kin == g.ktiles_per_r) {
        kin = 0;
        ++r;
      }
    }
  };
  // A range of at most kMaxStagesS K tiles is resident at once: one round of loads, one wait.  A longer one
  // is walked in rounds of kRoundS K tiles through two halves of LDS, the loads of round r + 1 in flight
  // under the matrix instructions of round r.
  const bool one_round = n_st <= kMaxStagesS;
  const int per_round = one_round ? n_st : kRoundS;
  const int rounds = one_round ? 1 : (n_st + kRoundS - 1) / kRoundS;
  issue_stages(0, per_round, 0);
  if (rounds > 1) issue_stages(kRoundS, n_st - kRoundS < kRoundS ? n_st - kRoundS : kRoundS, kRoundS);

  float4v acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = float4v{0.f, 0.f, 0.f, 0.f};

  const bool ragged = (A_KMAJOR || B_KMAJOR) && (g.K & 7) != 0;
  const int kin0 = kb % g.ktiles_per_r;
  for (int rd = 0; rd < rounds; ++rd) {
    const int done = rd * per_round;                       // K tiles of the rounds before
    const int count = n_st - done < per_round ? n_st - done : per_round;
    // loads return in order: with a whole round (2 kRoundS loads per wavefront) behind it, round rd has landed
    // when that many are still on their way
    if (rd + 1 < rounds && n_st - done - per_round >= kRoundS) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(2 * kRoundS) : "memory");
    else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    const uint32_t half = lds_base + (uint32_t)((rd & 1) * kRoundS) * kStageS;
    // k steps of 32: wavefront w takes steps w, w + 4, ... of the workgroup's range
    for (int ks = (wave - 2 * done) & 3; ks < 2 * count; ks += 4) {
      const int s = ks >> 1, tt = ks & 1;
      const uint32_t stage = half + (uint32_t)s * kStageS;
      const int kin = (kin0 + done + s) % g.ktiles_per_r;
      uint4v fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = read_fragment_small<A_KMAJOR>(stage, 16 * i, tt, lane);
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = read_fragment_small<B_KMAJOR>(stage + kRegionS, 16 * j, tt, lane);
      if (ragged && kin == g.ktiles_per_r - 1) {
        int valid = g.K - (kin * BK + 32 * tt + 8 * (lane >> 4));
        valid = valid < 0 ? 0 : (valid > 8 ? 8 : valid);
        if constexpr (A_KMAJOR) {
#pragma unroll
          for (int i = 0; i < 2; ++i) fa[i] = keep_first(fa[i], valid);
        }
        if constexpr (B_KMAJOR) {
#pragma unroll
          for (int j = 0; j < 2; ++j) fb[j] = keep_first(fb[j], valid);
        }
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = mfma<BF16>(fa[i], fb[j], acc[i][j]);
    }
    if (rd + 2 < rounds) {
      // round rd + 2 takes this round's half once every wavefront has read what it needed from it
      __syncthreads();
      const int next = (rd + 2) * kRoundS;
      issue_stages(next, n_st - next < kRoundS ? n_st - next : kRoundS, (rd & 1) * kRoundS);
    }
  }
  // the four wavefronts' tiles, added in the order of the wavefronts: wavefront w sums block w
  __syncthreads();  // every wavefront is done with the operands in LDS
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) *lds_ptr<float4v>(lds_base + (uint32_t)(((wave * 4 + 2 * i + j) * 64 + lane) * 16)) = acc[i][j];
  __syncthreads();
  float4v blk = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int w = 0; w < 4; ++w) blk += *lds_ptr<const float4v>(lds_base + (uint32_t)(((w * 4 + wave) * 64 + lane) * 16));

  if (g.splits > 1) {
    const long tile_id = ((long)z * g.tiles_n + tile_n) * g.tiles_m + tile_m;
    float *P = g.partial + (tile_id * g.splits + split) * (long)(SM * SN) + wave * 256 + lane * 4;
    store_device_scope(P, blk);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    if (tid == 0) {
      const uint32_t ticket = __hip_atomic_fetch_add(g.tickets + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      const bool last = ticket == (uint32_t)g.splits - 1u;
      if (last) __hip_atomic_store(g.tickets + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      *flag = last ? 1u : 0u;
    }
    __syncthreads();
    if (*flag == 0) return;
    const float *Q = g.partial + tile_id * g.splits * (long)(SM * SN) + wave * 256 + lane * 4;
    blk = float4v{0.f, 0.f, 0.f, 0.f};
    for (int r0 = 0; r0 < g.splits; r0 += 8) {
      float4v part[8];
      const float *q[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) q[u] = Q + (long)(r0 + u < g.splits ? r0 + u : r0) * (SM * SN);
      load_eight_device_scope(part, q);
#pragma unroll
      for (int u = 0; u < 8; ++u)
        if (r0 + u < g.splits) blk += part[u];
    }
  }

  if (n >= g.N || m >= g.M) return;
  uint16_t *p = Cz + m + (long)n * g.ldc;
  if (g.vec_c && m + 4 <= g.M) {
    uint2v out;
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      float x0 = blk[2 * w], x1 = blk[2 * w + 1];
      if (g.accumulate) {
        x0 += widen<BF16>(old[w] & 0xffffu);
        x1 += widen<BF16>(old[w] >> 16);
      }
      out[w] = narrow<BF16>(x0) | (narrow<BF16>(x1) << 16);
    }
    *reinterpret_cast<uint2v *>(p) = out;
  } else {
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      if (m + v < g.M) {
        float x = blk[v];
        if (g.accumulate) x += widen<BF16>(p[v]);
        p[v] = (uint16_t)narrow<BF16>(x);
      }
    }
  }
}

template <bool A_KMAJOR, bool B_KMAJOR, bool BF16>
__global__ __launch_bounds__(kThreads, 4) void gemm_h16_skinny_kernel(const SkinnyArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_skinny[];
  __shared__ uint32_t flag;
  if (g.small) skinny_tile_small<A_KMAJOR, B_KMAJOR, BF16>(g, lds_skinny, &flag, blockIdx.x, gridDim.x);
  else skinny_tile<A_KMAJOR, B_KMAJOR, BF16>(g, lds_skinny, &flag, blockIdx.x, gridDim.x);
}

// Both gradient products of one matmul_bw call in one grid: workgroups below `first` run ga += gy . b^T
// (operands contiguous along m and n), the others gb += a^T . gy (both contiguous along k).  Per-timestep
// launches are mostly fixed latency; the two products share it.
// The second problem's workgroups start at `second_at`, a multiple of 8, so that both problems meet the XCDs
// in the order their tile numbering expects; workgroups between the two do nothing.
template <bool BF16>
__global__ __launch_bounds__(kThreads, 4) void gemm_h16_skinny_pair_kernel(const SkinnyArgs g1, const SkinnyArgs g2, int first,
                                                                         int second_at) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds_skinny[];
  __shared__ uint32_t flag;
  const int bid = blockIdx.x;
  if (bid < first) {
    if (g1.small) skinny_tile_small<false, false, BF16>(g1, lds_skinny, &flag, bid, first);
    else skinny_tile<false, false, BF16>(g1, lds_skinny, &flag, bid, first);
  } else if (bid >= second_at) {
    if (g2.small) skinny_tile_small<true, true, BF16>(g2, lds_skinny, &flag, bid - second_at, (int)gridDim.x - second_at);
    else skinny_tile<true, true, BF16>(g2, lds_skinny, &flag, bid - second_at, (int)gridDim.x - second_at);
  }
}

struct SkinnyPlan {
  SkinnyArgs a;
  long tiles;   // output tiles times samples
  long grid;    // tiles times K ranges
  int stages;   // K tiles of the longest range
  int lds;      // bytes of LDS a workgroup needs
  int tile_floats;  // elements of one output tile (one partial tile of a split product)
};

// False when the problem is not one for this kernel.  `places_per_cu` caps how many workgroups may share a
// compute unit (0: as many as LDS allows).
bool plan_skinny(const phip_ctx *ctx, const Gemm &p, SkinnyPlan *plan, int places_per_cu = 0) {
  if (p.a_kmajor && !p.b_kmajor) return false;
  if (p.M < 1 || p.N < 1 || p.K < 16) return false;
  // the narrow side: at most 128 columns or rows of output, or a short K (a rank-K update)
  // ... or an output of at most half a million elements: such a product is a launch of a few microseconds whatever its K, and one
  // round of loads beats the staged loop (512^3: forward 6.8 -> 4.5 us, both gradients in one launch 13.7 -> 5.6;
  // 800 x 784 by 200 columns 9.8 -> 5.4 and 18.2 -> 10.1); from 768^3 on the 128 x 128 tiles are ahead (8.8
  // against 9.7 us)
  const bool narrow = p.N <= 128 || p.M <= 128 || p.K <= 128 || (long)p.M * p.N * p.batch <= 512L * 1024L;
  if (!narrow) return false;
  // 16-byte loads from 4-byte aligned addresses: even leading dimensions and strides, aligned bases
  if (reinterpret_cast<uintptr_t>(p.A) % 16 != 0 || reinterpret_cast<uintptr_t>(p.B) % 16 != 0) return false;
  if (p.lda % 2 != 0 || p.ldb % 2 != 0 || p.sA % 2 != 0 || p.sB % 2 != 0 || p.rA % 2 != 0 || p.rB % 2 != 0) return false;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return false;
  const long a_bytes = 2L * p.M * p.K, b_bytes = 2L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return false;
  const int cus = ctx->prop.multiProcessorCount;
  const int ktiles_per_r = (p.K + BK - 1) / BK;
  const long total_ktiles = (long)ktiles_per_r * p.rbatch;
  if (total_ktiles > 100000) return false;

  // Tile shape and stages per workgroup: the choice that a small cost model likes best (microseconds): the
  // loads of the workgroups that share a compute unit (about 0.4 per 16 KiB), the exchange of partial tiles
  // when K is cut (store, ticket: 2; then 2 per round trip through memory, one per four - small tiles: eight -
  // ranges: `gx = W^T gy` of the output projection, 20 ranges in five round trips, measured 16.4 us), the sum
  // over the wavefronts of a small tile, 1 for every further round of a range that LDS does not hold at once,
  // and a second round of workgroups if the grid does not fit the chip at once.  Ties go to the large tiles,
  // which load each operand fewer times.
  int best_s = 0, best_small = 0;
  long best_tiles = 0;
  double best = 0.0;
  for (int small = 0; small < 2; ++small) {
    // (a small tile's range may exceed what LDS holds: it is then walked in rounds of kRoundS K tiles)
    const int side = small ? SM : TM, stage_bytes = small ? kStageS : kStage;
    const int max_s = small ? kRoundS * kMaxRoundsS : kMaxStages;
    const long tiles = (long)((p.M + side - 1) / side) * ((p.N + side - 1) / side) * p.batch;
    if (tiles > kTicketSlots) continue;
    for (int s = 1; s <= max_s; ++s) {
      const long splits = (total_ktiles + s - 1) / s;
      const int s_eff = (int)((total_ktiles + splits - 1) / splits);
      if (s_eff != s && s != max_s) continue;  // the same cut as a smaller s
      const int rounds_of = small && s_eff > kMaxStagesS ? (s_eff + kRoundS - 1) / kRoundS : 1;
      int lds = (rounds_of > 1 ? kMaxStagesS : s_eff) * stage_bytes;
      if (small && lds < kReduceBytesS) lds = kReduceBytesS;
      int occ = (160 * 1024) / lds;
      if (occ > 4) occ = 4;  // registers: four wavefronts per SIMD
      if (places_per_cu > 0 && occ > places_per_cu) occ = places_per_cu;
      if (occ < 1) continue;
      const long grid = tiles * splits;
      if (grid > 0x7fffffffL) continue;
      if (splits > 1 && (size_t)grid * side * side * 4 > ((size_t)64 << 20)) continue;
      const long places = (long)cus * occ;
      const long rounds = (grid + places - 1) / places;
      long per_cu = (grid + cus - 1) / cus;
      if (per_cu > occ) per_cu = occ;
      const double loads = 0.4 * s_eff * per_cu * stage_bytes / kStage;
      const double exchange = splits > 1 ? 2.0 + 2.0 * ((splits + (small ? 7 : 3)) / (small ? 8 : 4)) : 0.0;
      const double cost = rounds * (1.0 + (small ? 0.3 : 0.0) + loads + 1.0 * (rounds_of - 1)) + exchange;
      if (best_s == 0 || cost < best - 1e-9) {
        best = cost;
        best_s = s_eff;
        best_small = small;
        best_tiles = tiles;
      }
    }
  }
  if (best_s == 0) return false;
  const long splits = (total_ktiles + best_s - 1) / best_s;
  const int side = best_small ? SM : TM;
  const long tiles = best_tiles;

  SkinnyArgs &a = plan->a;
  a.A = static_cast<const uint16_t *>(p.A);
  a.B = static_cast<const uint16_t *>(p.B);
  a.C = static_cast<uint16_t *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.tiles_m = (p.M + side - 1) / side;
  a.tiles_n = (p.N + side - 1) / side;
  a.splits = (int)splits;
  a.ktiles_per_r = ktiles_per_r;
  a.total_ktiles = (int)total_ktiles;
  a.accumulate = p.accumulate ? 1 : 0;
  a.vec_c = reinterpret_cast<uintptr_t>(p.C) % 8 == 0 && p.ldc % 4 == 0 && p.sC % 4 == 0;
  a.small = best_small;
  a.a_bytes = (uint32_t)a_bytes;
  a.b_bytes = (uint32_t)b_bytes;
  a.partial = nullptr;
  a.tickets = nullptr;
  plan->tiles = tiles;
  plan->grid = tiles * splits;
  plan->stages = (int)((total_ktiles + splits - 1) / splits);
  plan->lds = (best_small && plan->stages > kMaxStagesS ? kMaxStagesS : plan->stages) * (best_small ? kStageS : kStage);
  if (best_small && plan->lds < kReduceBytesS) plan->lds = kReduceBytesS;
  plan->tile_floats = side * side;
  return true;
}

// Scratch for the partial tiles of a plan whose K is cut; `block` goes back to the scratch pool once the
// launch has been enqueued.
int prepare_exchange(phip_ctx *ctx, SkinnyPlan *plan, void **block) {
  *block = nullptr;
  if (plan->a.splits <= 1) return PHIP_OK;
  const int rc = scratch_alloc(ctx, (size_t)plan->grid * plan->tile_floats * sizeof(float), block);
  if (rc != PHIP_OK) return rc;
  plan->a.partial = static_cast<float *>(*block);
  plan->a.tickets = tile_tickets(ctx);
  return PHIP_OK;
}

template <typename Kernel>
int raise_lds(phip_ctx *ctx, int slot, Kernel kern, int bytes) {
  // always the largest size the kernel is ever launched with: set once per context and kernel
  (void)bytes;
  return raise_lds_limit(ctx, slot, reinterpret_cast<const void *>(kern), kMaxStages * kStage);
}

}  // namespace

int gemm_h16_skinny(phip_ctx *ctx, const Gemm &p, Elem elem, bool *handled) {
  *handled = false;
  SkinnyPlan plan;
  if (!plan_skinny(ctx, p, &plan)) return PHIP_OK;
  void *block = nullptr;
  int rc = prepare_exchange(ctx, &plan, &block);
  if (rc != PHIP_OK) return rc;
  const int lds = plan.lds;
  const bool bf = elem == Elem::BF16;
#define PHIP_SKINNY(SLOT, AK, BKM)                                                                                 \
  do {                                                                                                             \
    if (bf) {                                                                                                      \
      auto kern = gemm_h16_skinny_kernel<AK, BKM, true>;                                                           \
      rc = raise_lds(ctx, kSlotGemmH16Skinny + (SLOT) + 3, kern, lds);                                             \
      if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3((unsigned)plan.grid), dim3(kThreads), lds, ctx->stream, plan.a); \
    } else {                                                                                                       \
      auto kern = gemm_h16_skinny_kernel<AK, BKM, false>;                                                          \
      rc = raise_lds(ctx, kSlotGemmH16Skinny + (SLOT), kern, lds);                                                 \
      if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3((unsigned)plan.grid), dim3(kThreads), lds, ctx->stream, plan.a); \
    }                                                                                                              \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) PHIP_SKINNY(0, false, true);
  else if (!p.a_kmajor && !p.b_kmajor) PHIP_SKINNY(1, false, false);
  else PHIP_SKINNY(2, true, true);
#undef PHIP_SKINNY
  if (block) scratch_free(ctx, block);  // the stream is in order: reusable behind this launch
  if (rc != PHIP_OK) return rc;
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, plan.a.small ? "h16_skinny32" : "h16_skinny");
  *handled = true;
  return PHIP_OK;
}

// ga += gy . b^T and gb += a^T . gy of one matmul_bw call in one launch (both accumulate, outputs apart).
int gemm_h16_skinny_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, Elem elem, bool *handled) {
  *handled = false;
  if (first.a_kmajor || first.b_kmajor || !second.a_kmajor || !second.b_kmajor) return PHIP_OK;
  if (first.batch != 1 || second.batch != 1) return PHIP_OK;
  SkinnyPlan p1, p2;
  // both grids resident at once: each problem is planned for half of the places
  if (!plan_skinny(ctx, first, &p1, 4) || !plan_skinny(ctx, second, &p2, 4)) return PHIP_OK;
  const int lds = p1.lds > p2.lds ? p1.lds : p2.lds;
  const int cus = ctx->prop.multiProcessorCount;
  int occ = (160 * 1024) / lds;
  if (occ > 4) occ = 4;  // registers: four wavefronts per SIMD
  const long second_at = (p1.grid + 7) / 8 * 8;
  if (second_at + p2.grid > (long)cus * occ) return PHIP_OK;  // would take a second round: two launches do as well
  void *b1 = nullptr, *b2 = nullptr;
  int rc = prepare_exchange(ctx, &p1, &b1);
  if (rc == PHIP_OK) rc = prepare_exchange(ctx, &p2, &b2);
  if (rc == PHIP_OK && p1.a.splits > 1 && p2.a.splits > 1) {
    // the two problems' tiles draw tickets from different counters
    if (p1.tiles + p2.tiles > kTicketSlots) rc = fail(PHIP_ERR_INVALID_ARGUMENT, "too many output tiles");
    else p2.a.tickets = tile_tickets(ctx) + p1.tiles;
  }
  if (rc == PHIP_OK) {
    const unsigned grid = (unsigned)(second_at + p2.grid);
    if (elem == Elem::BF16) {
      auto kern = gemm_h16_skinny_pair_kernel<true>;
      rc = raise_lds(ctx, kSlotGemmH16Skinny + 7, kern, lds);
      if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, ctx->stream, p1.a, p2.a, (int)p1.grid, (int)second_at);
    } else {
      auto kern = gemm_h16_skinny_pair_kernel<false>;
      rc = raise_lds(ctx, kSlotGemmH16Skinny + 6, kern, lds);
      if (rc == PHIP_OK) hipLaunchKernelGGL(kern, dim3(grid), dim3(kThreads), lds, ctx->stream, p1.a, p2.a, (int)p1.grid, (int)second_at);
    }
  }
  if (b1) scratch_free(ctx, b1);
  if (b2) scratch_free(ctx, b2);
  if (rc != PHIP_OK) return rc;
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "h16_skinny_pair");
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
