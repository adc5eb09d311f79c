// fp32 GEMM, 128 x 128 x 32 tiles, operands moved global -> LDS by buffer
// loads that write LDS directly (no staging registers, no LDS write
// instructions, ragged edges zero-filled by the buffer range check).
//
// One workgroup = 4 wavefronts in a 2 x 2 grid, each a 64 x 64 block of 2 x 2
// v_mfma_f32_32x32x2_f32 tiles.  Two 32 KiB LDS stages (A region then B region,
// 16 KiB each); two workgroups share a CU.
//
// LDS image of one operand:
//  * contiguous along m or n: 32 rows (k) of 128 floats, exactly as in memory.
//    A fragment is one 4-byte read per lane (32 consecutive floats per half
//    wave).
//  * contiguous along k: 128 rows (m or n) of 32 k = 128 bytes = 8 chunks of 16
//    bytes; chunk c of row x sits at position c ^ ((x >> 1) & 7), so that the
//    16-byte reads of 16 consecutive rows hit 16 different bank groups.  A
//    fragment is one 16-byte read per lane: 4 consecutive k of the lane's row.
// K is walked in groups of 8: the four matrix instructions of a group use
// k = k0 + 4*(lane/32) + e, e = 0..3, for both operands, which is what makes the
// 16-byte form possible.
#include "phip_gemm_f32_common.h"

namespace phip {
namespace {

typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int LBM = 128, LBN = 128, LBK = 32;
constexpr int kRegion = 16384;            // bytes per operand per stage
constexpr int kStage = 2 * kRegion;
constexpr int kLdsBytes = 2 * kStage;
constexpr uint32_t kOutOfRange = 0x80000000u;

struct LdsArgs {
  GemmArgs g;
  uint32_t a_bytes, b_bytes;  // size of one sample of each operand
};

__device__ inline uint4v make_rsrc_words(const float *p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  uint4v r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
  return r;
}

// One 16-byte-per-lane buffer load whose destination is LDS: lane l's data
// lands at lds_addr + 16*l.  Inline assembly keeps the compiler from putting a
// wait for it in front of every later LDS read; the kernel waits for these
// loads itself (s_waitcnt vmcnt) before the barrier that publishes the tile.
// m0 is scratch between instructions: nothing else here keeps a value in it.
__device__ inline void lds_dma_b128(uint4v rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}

// The wave's 4 load instructions (1 KiB of LDS each) for one operand tile.
template <bool KMAJOR>
struct DmaLoader {
  uint32_t off[4];     // byte offset of this lane's chunk per instruction, at K tile 0
  uint32_t step;       // bytes per K tile
  uint32_t live_mask;  // (m/n-contiguous) bit q: the chunk's columns exist
  int kc[4];           // (k-contiguous) first k of the chunk inside the tile

  __device__ inline void init(long ld, int x0, int X, int wave, int lane) {
    live_mask = 0;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int blk = wave * 4 + q;  // which 1 KiB block of the region
      if constexpr (KMAJOR) {
        const int x = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((x >> 1) & 7);
        off[q] = (uint32_t)(((long)(x0 + x) * ld + c * 4) * 4);  // a row past X is past the end
        kc[q] = c * 4;
      } else {
        const int k = blk * 2 + (lane >> 5);
        const int c = lane & 31;
        off[q] = (uint32_t)(((long)k * ld + x0 + c * 4) * 4);    // a row past K is past the end
        kc[q] = 0;
        if (x0 + c * 4 < X) live_mask |= 1u << q;
      }
    }
    step = KMAJOR ? (uint32_t)(LBK * 4) : (uint32_t)(LBK * ld * 4);
  }

  __device__ inline void issue(uint4v rsrc, uint32_t region_addr, int wave, int q, int kt_in_r, int K,
                               bool live) const {
    bool in = live;
    if constexpr (KMAJOR) in = in && kt_in_r * LBK + kc[q] < K;
    else in = in && ((live_mask >> q) & 1u);
    const uint32_t o = in ? off[q] + (uint32_t)kt_in_r * step : kOutOfRange;
    lds_dma_b128(rsrc, region_addr + (uint32_t)(wave * 4 + q) * 1024u, o);
  }
};

// Fragments of one operand for one group of 8 k: v[block][e].
template <bool KMAJOR>
struct FragReaderF {
  uint32_t base[4];  // byte offsets inside the region

  __device__ inline void init(int xw, int lane) {
    if constexpr (KMAJOR) {
      // row x = xw + 32 i + lane%32; group gk reads chunk (2 gk + lane/32) ^ swizzle: base[gk]
      const int sw = ((lane & 31) >> 1) & 7;
#pragma unroll
      for (int gk = 0; gk < 4; ++gk)
        base[gk] = (uint32_t)((xw + (lane & 31)) * 128 + (((2 * gk + (lane >> 5)) ^ sw) * 16));
    } else {
      // row k = 8 gk + 4 (lane/32) + e, column xw + 32 i + lane%32
      base[0] = (uint32_t)((4 * (lane >> 5)) * 512 + (xw + (lane & 31)) * 4);
      base[1] = base[2] = base[3] = 0;
    }
  }

  __device__ inline void read(const unsigned char *region, int gk, float (&v)[2][4]) const {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      if constexpr (KMAJOR) {
        const float4v t = *reinterpret_cast<const float4v *>(region + base[gk] + i * 4096);
        v[i][0] = t.x; v[i][1] = t.y; v[i][2] = t.z; v[i][3] = t.w;
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          v[i][e] = *reinterpret_cast<const float *>(region + base[0] + (8 * gk + e) * 512 + i * 128);
      }
    }
  }

  // the q-th of the reads above (8 for m/n-contiguous, 2 for k-contiguous)
  static constexpr int kReads = KMAJOR ? 2 : 8;
  __device__ inline void read_one(const unsigned char *region, int gk, int q, float (&v)[2][4]) const {
    if constexpr (KMAJOR) {
      const float4v t = *reinterpret_cast<const float4v *>(region + base[gk] + q * 4096);
      v[q][0] = t.x; v[q][1] = t.y; v[q][2] = t.z; v[q][3] = t.w;
    } else {
      const int i = q >> 2, e = q & 3;
      v[i][e] = *reinterpret_cast<const float *>(region + base[0] + (8 * gk + e) * 512 + i * 128);
    }
  }
};

template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_lds_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  const int z = t;
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

  const int kt_end = g.total_ktiles;
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds;
  auto issue_tile = [&](int kt, int q) {
    // instruction q of the 8 that move K tile kt (4 for A, then 4 for B)
    const bool live = kt < kt_end;
    const int ktc = live ? kt : 0;
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
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float vals[16];
      int ns[16];
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        vals[v] = acc[i][j][v];
        ns[v] = 8 * (v / 4) + (v % 4);
      }
      emit_c<16>(Cz, g.ldc, m0 + wm * 64 + i * 32, n0 + wn * 64 + j * 32, lane, g.M, g.N, interior, ns, vals, 0,
                 g.accumulate);
    }
}

}  // namespace

// Large, 16-byte-aligned problems.  Sets *handled when it launched.
int gemm_f32_lds(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  auto aligned = [](const void *ptr, long ld, long s, long r) {
    return (reinterpret_cast<uintptr_t>(ptr) % 16 == 0) && ld % 4 == 0 && s % 4 == 0 && r % 4 == 0;
  };
  if (!aligned(p.A, p.lda, p.sA, p.rA) || !aligned(p.B, p.ldb, p.sB, p.rB)) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return PHIP_OK;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  const long tiles = (long)((p.M + LBM - 1) / LBM) * ((p.N + LBN - 1) / LBN) * p.batch;
  const int cus = ctx->prop.multiProcessorCount;
  if (tiles < cus || (long)p.K * p.rbatch <= 128 || tiles > 0x7fffffffL) return PHIP_OK;
  if (p.a_kmajor && !p.b_kmajor) return PHIP_OK;

  LdsArgs d;
  GemmArgs &a = d.g;
  a.A = static_cast<const float *>(p.A);
  a.B = static_cast<const float *>(p.B);
  a.C = static_cast<float *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.tiles_m = (p.M + LBM - 1) / LBM;
  a.tiles_n = (p.N + LBN - 1) / LBN;
  a.splits = 1;
  a.ktiles_per_r = (p.K + LBK - 1) / LBK;
  a.total_ktiles = a.ktiles_per_r * p.rbatch;
  a.atomic = 0;
  a.accumulate = p.accumulate ? 1 : 0;
  d.a_bytes = (uint32_t)a_bytes;
  d.b_bytes = (uint32_t)b_bytes;

#define PHIP_LDS(SLOT, AK, BKM)                                                                 \
  do {                                                                                          \
    auto kern = gemm_f32_lds_kernel<AK, BKM>;                                                   \
    const int rc = raise_lds_limit(ctx, SLOT, reinterpret_cast<const void *>(kern), kLdsBytes); \
    if (rc != PHIP_OK) return rc;                                                               \
    hipLaunchKernelGGL(kern, dim3((unsigned)tiles), dim3(kThreads), kLdsBytes, ctx->stream, d); \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) PHIP_LDS(0, false, true);
  else if (!p.a_kmajor && !p.b_kmajor) PHIP_LDS(1, false, false);
  else PHIP_LDS(2, true, true);
#undef PHIP_LDS
  PHIP_LAUNCH_CHECK();
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
