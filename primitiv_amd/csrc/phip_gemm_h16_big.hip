// Large-tile GEMM for 16-bit storage (fp16 / bf16, fp32 accumulation):
// 256 x 256 x 64 tiles, one workgroup (4 wavefronts, each a 128 x 128 block of
// 8 x 8 v_mfma_f32_16x16x32 tiles, 256 accumulator registers per lane) per CU,
// two 64 KiB LDS stages.  Problems with too few such tiles for the chip take
// 128 x 128 x 64 tiles instead (wavefronts of 4 x 4 blocks, two 32 KiB stages,
// two workgroups per CU): the same code with half the extents.
//
// The 16 x 16 x 32 instruction, not the 32 x 32 x 16 one: these kernels run at
// the power limit, where the clock follows what the instructions draw, and a
// register-only loop of the smaller shape settles a fifth higher (1.97 against
// 1.63 GHz with fp16 operands).  Its price is a pipe that is busy for only 16
// cycles per instruction while a wavefront issues one instruction every 4, so
// the K loop is laid out with at most three other instructions between two of
// them.
//
// Nothing is staged through registers and nothing is transposed by ALU work:
//  * both operands are moved global -> LDS by buffer loads that write LDS
//    directly; everything past the end of a matrix reads as zero (buffer range
//    check), which covers ragged edges without branches;
//  * an operand that is contiguous along k is read back with 16-byte LDS reads
//    (8 consecutive k per lane is what the matrix instruction takes);
//  * an operand that is contiguous along m or n is kept in LDS as it is in
//    memory and transposed by the LDS read instruction (ds_read_b64_tr_b16).
// LDS rows are not padded (a load instruction fills 1 KiB of consecutive LDS);
// bank conflicts are avoided by XOR-swizzling which 16-byte chunk of a row
// each lane fetches.
#include <type_traits>

#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

// LDS pointer from an LDS byte address (a register plus an immediate, for the compiler)
template <class T>
__device__ inline __attribute__((address_space(3))) T *lds_ptr(uint32_t addr) {
  return (__attribute__((address_space(3))) T *)(size_t)addr;
}

constexpr int kThreads = 256;
constexpr int BK = 64;
// WB = 32 rows (two blocks of 16) per wavefront and direction: 4 -> 256 x 256 tiles (one workgroup per
// CU), 2 -> 128 x 128 tiles (two workgroups per CU) for problems with too few large tiles
template <int WB> constexpr int kTile = 64 * WB;                  // rows = columns of a workgroup's tile
template <int WB> constexpr int kRegion = kTile<WB> * BK * 2;     // bytes of one operand tile
template <int WB> constexpr int kStage = 2 * kRegion<WB>;
template <int WB> constexpr int kLds = 2 * kStage<WB>;
constexpr uint32_t kOutOfRange = 0x80000000u;   // beyond any buffer this kernel accepts

struct BigArgs {
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
  uint32_t a_bytes, b_bytes;  // size of one sample of each operand
};

__device__ inline int xcd_remap(int bid, int total) {
  constexpr int kXcds = 8;
  const int xcd = bid % kXcds;
  const int idx = bid / kXcds;
  const int q = total / kXcds, rem = total % kXcds;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

// D = A . B for a 16 x 16 block over 32 k: lane l supplies row l % 16 of A (and
// column l % 16 of B), k = 8 (l / 16) .. + 7, and receives rows 4 (l / 16) .. + 3
// of column l % 16.
//
// Written as inline assembly with the accumulator tied to an AGPR tuple: left to
// the register allocator, most of the 64 accumulators of a wavefront were
// copied to a spare tuple before every instruction (the form whose result
// must not overlap its addend).  The compiler therefore does not know these
// are matrix instructions; the kernel keeps its own distance between the last
// of them and the first ordinary read of an accumulator.
template <bool BF16>
__device__ inline void mfma(float4v &c, uint4v a, uint4v b) {
  if constexpr (BF16) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
  else asm volatile("v_mfma_f32_16x16x32_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b));
}

// More wait states than any matrix-instruction hazard asks for.
__device__ inline void settle_matrix_pipe() { asm volatile("s_nop 15\n\ts_nop 15" ::: "memory"); }

template <bool BF16>
__device__ inline float widen(uint32_t bits16) {
  if constexpr (BF16) return __builtin_bit_cast(float, bits16 << 16);
  else return to_f32(__builtin_bit_cast(f16_t, (uint16_t)bits16));
}

// Two results rounded to nearest even (the mode these conversions run in by
// default) and packed, x0 in the low half: one instruction per pair.
template <bool BF16>
__device__ inline uint32_t round_pair(float x0, float x1) {
  uint32_t r;
  if constexpr (BF16) asm("v_cvt_pk_bf16_f32 %0, %1, %2" : "=v"(r) : "v"(x0), "v"(x1));
  else asm("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(r) : "v"(x0), "v"(x1));
  return r;
}

// Writes the R x R block of results one wavefront holds (NBK x NBK blocks of
// 16 x 16, R = 16 NBK) into the 16-bit C, 16 bytes (8 consecutive rows of one
// column) per lane and store instruction, R / 8 lanes side by side on a column.
// The matrix instruction leaves a lane with 4 consecutive rows of one column
// per block and a wavefront with 16 columns per instruction; stored that way, a
// store instruction would scatter 32-byte pieces over 16 columns (with a
// power-of-two leading dimension: 16 requests to one memory channel; measured
// at twice the time).  So the block is turned through an LDS area that belongs
// to this wavefront alone, 64 columns (R x 64 floats) at a time: written as
// fp32, 16 bytes per lane, the way the accumulators lie; read back 8
// consecutive rows at a time.  For an accumulating write the old values are
// fetched (also 16 bytes per lane) before the LDS pass, added in fp32 and
// rounded once.  M is a multiple of 8 and C is 16-byte aligned (checked by the
// dispatcher), so a lane's 8 rows are either all inside the matrix or all
// outside.
//
// The area holds column c as R floats = R / 4 groups of 16 bytes; group G of
// column c sits at position (G ^ (G >> 4)) ^ (c & 15).  The second term spreads
// the 16 columns one write instruction touches (and the neighbouring columns
// one read instruction touches) over all banks; the first swaps the two halves
// of a lane's 8 rows for rows 64 and up, so that the 16 lanes that read one
// column of 128 rows cover all banks with their first 16 bytes.  Both are
// constants of a lane's address up to an XOR with a compile-time value.
//
// FULL: the block lies inside the matrix, no access is masked.
template <bool BF16, bool ACC, bool FULL, int NBK>
__device__ inline void emit_blocks_via_lds(unsigned char *area, uint16_t *Cz, long ldc, int row0, int col0, int lane,
                                           int M, int N, const float4v (&acc)[NBK][NBK]) {
  constexpr int R = 16 * NBK;      // rows of the block = floats per column of the area
  constexpr int LPC = R / 8;       // lanes per column on the read side
  constexpr int CPI = 64 / LPC;    // columns per store instruction
  constexpr int NIT = 64 / CPI;    // store instructions per pass of 64 columns
  constexpr int PASSES = R / 64;
  constexpr int V = 16 / CPI;      // distinct values of (column & 15) / CPI
  const uint32_t area_addr = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)area;

  // write side: rows 16 i + 4 g .. + 3 of column 16 jl + nl
  const int g = lane >> 4, nl = lane & 15;
  uint32_t waddr[NBK];
#pragma unroll
  for (int i = 0; i < NBK; ++i) {
    const int gg = g ^ (i >> 2);  // halves of 8 rows swapped from row 64 on
    waddr[i] = area_addr + (uint32_t)(nl * R * 4 + 16 * (((4 * i) | gg) ^ nl));
  }
  // read side: column CPI it + cq, rows 8 mc .. 8 mc + 7
  const int mc = lane % LPC, cq = lane / LPC;
  const int m = row0 + 8 * mc;
  uint32_t raddr[V];
#pragma unroll
  for (int v = 0; v < V; ++v)
    raddr[v] = area_addr + (uint32_t)(cq * R * 4 + 16 * (((2 * mc) | (mc >> 3)) ^ ((cq + CPI * v) & 15)));

#pragma unroll
  for (int h = 0; h < PASSES; ++h) {
    uint16_t *p0 = Cz + m + (long)(col0 + 64 * h + cq) * ldc;
    uint32_t ok = ~0u;
    if constexpr (!FULL) {
      ok = 0;
#pragma unroll
      for (int it = 0; it < NIT; ++it) ok |= (m < M && col0 + 64 * h + CPI * it + cq < N ? 1u : 0u) << it;
    }
    auto live = [&](int it) { return FULL || ((ok >> it) & 1u); };
    uint4v old[NIT];
    if constexpr (ACC) {
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        old[it] = uint4v{0, 0, 0, 0};
        if (live(it)) old[it] = *reinterpret_cast<const uint4v *>(p0 + (long)(CPI * it) * ldc);
      }
    }
#pragma unroll
    for (int i = 0; i < NBK; ++i)
#pragma unroll
      for (int jl = 0; jl < 4; ++jl) {
        // read where the matrix instructions left them: given the choice, the register
        // allocator moves all accumulators to VGPRs at once and spills
        float4v x;
#pragma unroll
        for (int v = 0; v < 4; ++v) asm("v_accvgpr_read_b32 %0, %1" : "=v"(x[v]) : "a"(acc[i][4 * h + jl][v]));
        *lds_ptr<float4v>(waddr[i] + (uint32_t)(16 * jl * R * 4)) = x;
      }
    float4v lo[NIT], hi[NIT];
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      const uint32_t at = raddr[it % V] + (uint32_t)(CPI * it * R * 4);
      lo[it] = *lds_ptr<const float4v>(at);
      hi[it] = *lds_ptr<const float4v>(at ^ 16u);
    }
#pragma unroll
    for (int it = 0; it < NIT; ++it) {
      float f[8] = {lo[it][0], lo[it][1], lo[it][2], lo[it][3], hi[it][0], hi[it][1], hi[it][2], hi[it][3]};
      uint4v out;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        float x0 = f[2 * e], x1 = f[2 * e + 1];
        if constexpr (ACC) {
          x0 += widen<BF16>(old[it][e] & 0xffffu);
          x1 += widen<BF16>(old[it][e] >> 16);
        }
        out[e] = round_pair<BF16>(x0, x1);
      }
      if (live(it)) *reinterpret_cast<uint4v *>(p0 + (long)(CPI * it) * ldc) = out;
    }
  }
}

// ---------------------------------------------------------------------------
// Operands go from global memory straight into LDS (buffer loads with the LDS
// destination: no registers, no LDS write instructions) and an operand that
// is contiguous along m or n is transposed by the LDS read itself
// (ds_read_b64_tr_b16).
//
// LDS image of one stage (64 KiB for the 256 x 256 tiles described here; the 128 x 128 tiles have half
// the rows and half the row length): A region then B region, 32 KiB each.
//  * k-contiguous operand: 256 rows (m or n) of 64 k = 128 bytes = 8 chunks
//    of 16 bytes.  Chunk c of row x sits at position c ^ ((x >> 1) & 7): the
//    16 lanes of a 16-byte fragment read (consecutive rows, same c) then hit
//    16 different 16-byte bank groups.
//  * m/n-contiguous operand: 64 rows (k) of 256 elements = 512 bytes = 32
//    chunks.  Chunk c of row k sits at position c ^ ((k & 3) << 2) ^ ((k & 8) >> 2):
//    the k rows that the lanes of one transposing read touch (four consecutive
//    ones, and the four 8 further on) land in different bank groups.
// A load instruction moves 64 x 16 bytes to 1 KiB of consecutive LDS (lane l
// to byte 16*l), so the swizzle is applied by choosing which global chunk each
// lane fetches.

typedef short short4v __attribute__((ext_vector_type(4)));

// Buffer descriptor spelled out as four dwords (base, base high + stride 0,
// size in bytes, format word), for use as an inline-assembly operand.
__device__ inline uint4v make_rsrc_words(const uint16_t *p, uint32_t bytes) {
  const uint64_t a = reinterpret_cast<uint64_t>(p);
  uint4v r = {(uint32_t)a, (uint32_t)(a >> 32) & 0xffffu, bytes, 0x00020000u};
  return r;
}

// One 16-byte-per-lane buffer load whose destination is LDS: lane l's data
// lands at lds_addr + 16*l and comes from base + voffset + soffset; lds_addr
// then moves on by the 1 KiB the load fills.  Only voffset is checked against
// the buffer's size, so whatever must read as zero has a voffset past it.
// Issued as inline assembly so that the compiler does not put a wait for it in
// front of every later LDS read; the kernel waits for these loads itself
// (s_waitcnt vmcnt) before the barrier that publishes the tile.  The
// instruction set asks for a wait state between the write of m0 and the load:
// the addition sits there.
__device__ inline void lds_dma_b128(uint4v rsrc, uint32_t &lds_addr, uint32_t voffset, uint32_t soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_add_u32 %0, %0, 0x400\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               : "+s"(lds_addr)
               : "v"(voffset), "s"(rsrc), "s"(soffset)
               : "memory", "scc");  // m0 is scratch between instructions: nothing else in this kernel keeps a value in it
}

// The wave's load instructions for one operand: per instruction a lane's byte
// offset at K tile 0, or kOutOfRange where its row or column lies outside the
// matrix, and a mask that sends it there in a last K tile that is only partly
// inside K.
template <bool KMAJOR, int WB>
struct LdsLoader {
  static constexpr int NI = 2 * WB;   // the wave's load instructions (1 KiB of LDS each) per operand tile
  static constexpr int CW = 8 * WB;   // (m/n-contiguous) 16-byte chunks per k row of the tile
  uint32_t off[NI];
  uint32_t cut[NI];    // kOutOfRange where the chunk lies outside a partial last K tile, else 0
  uint32_t use[NI];    // what the loads take: off, or off | cut while a partial tile is being fetched
  uint32_t step;       // bytes per K tile

  // k_tail: K % BK
  __device__ inline void init(long ld, int x0, int X, int k_tail, int wave, int lane) {
#pragma unroll
    for (int q = 0; q < NI; ++q) {
      const int blk = wave * NI + q;  // which 1 KiB block of the region
      if constexpr (KMAJOR) {
        const int x = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((x >> 1) & 7);
        off[q] = x0 + x < X ? (uint32_t)(((long)(x0 + x) * ld + c * 8) * 2) : kOutOfRange;
        cut[q] = c * 8 < k_tail ? 0u : kOutOfRange;
      } else {
        const int k = blk * (64 / CW) + lane / CW;
        const int c = (lane % CW) ^ ((k & 3) << 2) ^ (((k >> 3) & 1) << 1);
        off[q] = x0 + c * 8 < X ? (uint32_t)(((long)k * ld + x0 + c * 8) * 2) : kOutOfRange;
        cut[q] = k < k_tail ? 0u : kOutOfRange;
      }
    }
    step = KMAJOR ? (uint32_t)(BK * 2) : (uint32_t)(BK * ld * 2);
    select(0u);
  }

  // tail: all ones before the loads of a partial last K tile, 0 before those of a whole one
  __device__ inline void select(uint32_t tail) {
#pragma unroll
    for (int q = 0; q < NI; ++q) use[q] = off[q] | (cut[q] & tail);
  }

  // Issues instruction q for the K tile that starts `soffset` bytes after tile 0
  // into the next 1 KiB at lds_addr.
  __device__ inline void issue(uint4v rsrc, uint32_t &lds_addr, int q, uint32_t soffset) const {
    lds_dma_b128(rsrc, lds_addr, use[q], soffset);
  }
};

// The LDS addresses of one operand's fragment reads: per-lane values that point
// into the stage to be read next (`flip` moves them to the other stage), so
// that every read is one of them plus an immediate.
template <bool KMAJOR, int WB>
struct FragReader {
  static constexpr int kPitch = 128 * WB;  // (m/n-contiguous) bytes per k row
  static constexpr int NBK = 2 * WB;       // 16-row blocks of a wavefront's side
  uint32_t cur[KMAJOR ? 2 : NBK];

  // region_addr: LDS address of the operand's region in stage 0; xw: first row of the wavefront's block
  __device__ inline void init(uint32_t region_addr, int xw, int lane) {
    if constexpr (KMAJOR) {
      // row x = xw + 16 i + lane%16, chunk (4 t + lane/16) ^ swizzle: cur[t]
      const int sw = ((lane & 15) >> 1) & 7;
#pragma unroll
      for (int t = 0; t < 2; ++t)
        cur[t] = region_addr + (uint32_t)((xw + (lane & 15)) * 128 + (((4 * t + (lane >> 4)) ^ sw) * 16));
    } else {
      // lane = 16 g + 4 cc + a supplies k row 8 g + cc (and the one 4 further on),
      // columns 4 a .. + 3 of the block: cur[i].  Chunk xw/8 + 2 i + a/2 of row k
      // sits at that index ^ (4 (k & 3)) ^ (2 (k / 8 & 1)) = ^ (4 cc) ^ (2 (g & 1)).
      const int g = lane >> 4, cc = (lane & 15) >> 2, a = lane & 3;
      const int sw = (4 * cc) ^ (2 * (g & 1));
#pragma unroll
      for (int i = 0; i < NBK; ++i)
        cur[i] = region_addr +
                 (uint32_t)((8 * g + cc) * kPitch + ((xw / 8 + 2 * i + (a >> 1)) ^ sw) * 16 + (a & 1) * 8);
    }
  }

  // Moves the addresses that block i's reads use to the other stage; called for
  // every block in turn, just before its first read from that stage.
  __device__ inline void flip(int i, uint32_t delta) {
    if constexpr (KMAJOR) {
      if (i == 0) {
        cur[0] += delta;
        cur[1] += delta;
      }
    } else {
      cur[i] += delta;
    }
  }

  // Fragment of 16-row block i for k step t (32 k): 8 consecutive k, from 8 (lane / 16) on, of row lane % 16.
  __device__ inline uint4v read(int i, int t) const {
    if constexpr (KMAJOR) {
      return *lds_ptr<const uint4v>(cur[t] + (uint32_t)(i * 2048));
    } else {
      const uint32_t p = cur[i] + (uint32_t)(t * 32 * kPitch);
      const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p));
      const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<short4v>(p + (uint32_t)(4 * kPitch)));
      uint4v r;
      r.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
      r.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
      r.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
      r.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
      return r;
    }
  }
};

// NS: LDS stages (K tiles resident or on their way).  Two is what two workgroups per CU (128 x 128 tiles) or one
// (256 x 256) leave room for; a launch of 128 x 128 tiles with at most one workgroup per CU takes four, so that
// three K tiles are in flight where the loop otherwise waits for its loads at every barrier.
template <bool A_KMAJOR, bool B_KMAJOR, bool BF16, int WB, int NS = 2>
__global__ __launch_bounds__(kThreads, WB == 4 ? 1 : 2) void gemm_h16_lds_kernel(const BigArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds2[];
  constexpr int BM = kTile<WB>, BN = kTile<WB>;
  constexpr int kRegionBytes = kRegion<WB>, kStage2Bytes = kStage<WB>;
  constexpr int WT = 32 * WB;       // rows = columns of a wavefront's block
  constexpr int NI = 2 * WB;        // load instructions per wavefront, operand and K tile
  constexpr int NBK = 2 * WB;       // 16 x 16 blocks per side of a wavefront's block
  constexpr int NB = NBK * NBK;     // matrix instructions per k step of 32

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave & 1, wn = wave >> 1;

  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int per_z = g.tiles_m * g.tiles_n;
  const int z = t / per_z;
  t -= z * per_z;
  constexpr int GM = 8;
  const int group = t / (GM * g.tiles_n);
  const int first_m = group * GM;
  const int gm = g.tiles_m - first_m < GM ? g.tiles_m - first_m : GM;
  const int in_group = t - group * GM * g.tiles_n;
  const int tile_m = first_m + in_group % gm;
  const int tile_n = in_group / gm;
  const int m0 = tile_m * BM, n0 = tile_n * BN;

  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds2;
  const int k_tail = g.K % BK;
  LdsLoader<A_KMAJOR, WB> la;
  LdsLoader<B_KMAJOR, WB> lb;
  la.init(g.lda, m0, g.M, k_tail, wave, lane);
  lb.init(g.ldb, n0, g.N, k_tail, wave, lane);
  FragReader<A_KMAJOR, WB> fra;
  FragReader<B_KMAJOR, WB> frb;
  fra.init(lds_base, wm * WT, lane);
  frb.init(lds_base + kRegionBytes, wn * WT, lane);

  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;

  float4v acc[NBK][NBK];
#pragma unroll
  for (int i = 0; i < NBK; ++i)
#pragma unroll
    for (int j = 0; j < NBK; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[i][j][v] = 0.0f;

  const int kt_end = g.total_ktiles;
  // Every workgroup starts its walk over K at a different tile (and wraps
  // around): with power-of-two leading dimensions, workgroups marching through
  // K in lockstep would all pull from the same memory channels at once.
  //
  // State of the K tile to be loaded next, all scalar: which K range (r) and
  // which tile inside it, advanced by one tile at a time.
  int ld_ktc = (tile_m + tile_n + z) % kt_end;
  int ld_r = ld_ktc / g.ktiles_per_r;
  int ld_kin = ld_ktc - ld_r * g.ktiles_per_r;
  uint4v rs_a, rs_b;        // buffer descriptors of the K range
  uint32_t so_a, so_b;      // byte offset of the tile inside it
  uint32_t ld_tail;         // all ones: the tile is only partly inside K
  uint32_t sel_tail = 0;    // what the loaders' offsets are selected for
  uint32_t lds_run = 0;     // LDS address of the next load
  auto describe_range = [&]() {
    rs_a = make_rsrc_words(Az + (long)ld_r * g.rA, g.a_bytes);
    rs_b = make_rsrc_words(Bz + (long)ld_r * g.rB, g.b_bytes);
  };
  auto describe_tile = [&]() {
    so_a = (uint32_t)ld_kin * la.step;
    so_b = (uint32_t)ld_kin * lb.step;
    ld_tail = (uint32_t)__builtin_amdgcn_readfirstlane(k_tail != 0 && ld_kin == g.ktiles_per_r - 1 ? -1 : 0);
  };
  auto next_tile = [&]() {
    ++ld_ktc;
    ++ld_kin;
    if (ld_kin == g.ktiles_per_r) {
      ld_kin = 0;
      ++ld_r;
    }
    if (ld_ktc == kt_end) ld_ktc = ld_r = ld_kin = 0;
  };
  // a partial tile comes up, or is over (twice per K range at most)
  auto select_offsets = [&]() {
    if (ld_tail != sel_tail) {
      la.select(ld_tail);
      lb.select(ld_tail);
      sel_tail = ld_tail;
    }
  };
  // instruction q of the 2 NI that move the described tile into `stage` (NI for A, then NI for B):
  // the wave's share of each region is NI consecutive KiB
  auto issue = [&](int q, int stage) {
    if (q == 0) lds_run = lds_base + (uint32_t)stage * kStage2Bytes + (uint32_t)(wave * NI) * 1024u;
    if (q == NI) lds_run += (uint32_t)(kRegionBytes - NI * 1024);
    if (q < NI) la.issue(rs_a, lds_run, q, so_a);
    else lb.issue(rs_b, lds_run, q - NI, so_b);
  };

  // Loads return in the order of issue: a tile has landed once at most the loads of the tiles issued after it
  // (2 NI per tile and wavefront) are outstanding.
  auto wait_for_tile = [&](int later_tiles) {
    static_assert(NS <= 4 && (NS - 1) * 2 * NI <= 48, "wait counts are spelled out up to three tiles");
    if (later_tiles <= 0) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    else if (later_tiles == 1 && NI == 4) asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
    else if (later_tiles == 1) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
    else if (later_tiles == 2 && NI == 4) asm volatile("s_waitcnt vmcnt(16) lgkmcnt(0)" ::: "memory");
    else if (later_tiles == 2) asm volatile("s_waitcnt vmcnt(32) lgkmcnt(0)" ::: "memory");
    else if (NI == 4) asm volatile("s_waitcnt vmcnt(24) lgkmcnt(0)" ::: "memory");
    else asm volatile("s_waitcnt vmcnt(48) lgkmcnt(0)" ::: "memory");
  };
  describe_range();
  describe_tile();
  select_offsets();
#pragma unroll
  for (int q = 0; q < 2 * NI; ++q) issue(q, 0);
#pragma unroll
  for (int st = 1; st < NS; ++st) {
    if (kt_end > st) {
      next_tile();
      describe_range();
      describe_tile();
      select_offsets();
#pragma unroll
      for (int q = 0; q < 2 * NI; ++q) issue(q, st);
    }
  }
  wait_for_tile((kt_end < NS ? kt_end : NS) - 1);
  __syncthreads();

  // The fragments of the two k steps of a tile live in two register buffers and
  // are read one step (NB matrix instructions) ahead: step 1 of this tile
  // during step 0, then - behind the barrier - step 0 of the next tile during
  // step 1.  The barrier therefore sits in the middle of a tile, and the
  // global-to-LDS loads that refill the stage (K tile kt+2) are spread over
  // the instruction slots of step 1, with a whole tile time to land.
  //
  // A matrix instruction keeps its pipe busy for 16 cycles and the wavefront
  // issues one instruction every 4: whatever sits between two of them must be
  // at most three instructions, or the pipe idles.  Hence the scalar
  // bookkeeping of the next load is dealt out over the free slots of step 0
  // (pinned there by empty asm statements), a load costs three instructions
  // (m0, the next LDS address, the load), and every LDS address is a register
  // plus an immediate.
  uint4v fa[2][NBK], fb[2][NBK];
  auto read_frag = [&](int buf, int q, int t) {
    if (q < NBK) fa[buf][q] = fra.read(q, t);
    else fb[buf][q - NBK] = frb.read(q - NBK, t);
  };
#pragma unroll
  for (int q = 0; q < 2 * NBK; ++q) read_frag(0, q, 0);

  static_assert(WB == 2 || NB >= 3 * 2 * NBK, "every third slot holds a read");
  uint32_t flip_by = (uint32_t)kStage2Bytes;  // on to the next stage, or from the last back to the first
  int stage = 0;                              // the stage that holds the tile being multiplied
  settle_matrix_pipe();  // the zeroed accumulators
  // one K tile; LOADS: K tile kt + NS exists and is fetched into the stage this tile leaves
  auto tile = [&](auto loads_tag, int kt) {
    constexpr bool loads = decltype(loads_tag)::value;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int i = q / NBK, j = q % NBK;
        mfma<BF16>(acc[i][j], fa[t][i], fb[t][j]);
        // Slot plan.  Large tiles: the 4 waves' reads of a step are 64 KiB, 512 cycles
        // of LDS time, so one read per slot (16 cycles) asks for twice what LDS
        // delivers and the reads queue up in front of the matrix instructions;
        // one every third slot does not.  The loads take the slots after them,
        // the bookkeeping the third kind.  Small tiles: reads, then the rest.
        constexpr int kSpread = WB == 4 ? 3 : 1;
        const int rq = q / kSpread;  // which read / load / piece of bookkeeping
        const int kind = WB == 4 ? q % kSpread : (q < 2 * NBK ? 0 : 2);
        if (kind == 0 && rq < 2 * NBK) {
          if (t == 1) {
            // behind the barrier: on to the other stage
            if (rq < NBK) fra.flip(rq, flip_by);
            else frb.flip(rq - NBK, flip_by);
          }
          read_frag(t ^ 1, rq, t ^ 1);
        }
        if constexpr (loads) {
          if (t == 0) {
            // the tile after the one in flight: described piece by piece
            const int piece = WB == 4 ? (kind == 2 ? rq : -1) : q - 2 * NBK;
            if (piece == 0) {
              ++ld_ktc;
              ++ld_kin;
              if (ld_kin == g.ktiles_per_r) {
                ld_kin = 0;
                ++ld_r;
              }
              asm volatile("" : "+s"(ld_ktc), "+s"(ld_r), "+s"(ld_kin));
            } else if (piece == 2) {
              if (ld_ktc == kt_end) ld_ktc = ld_r = ld_kin = 0;
              asm volatile("" : "+s"(ld_ktc), "+s"(ld_r), "+s"(ld_kin));
            } else if (piece == 4) {
              if (g.ktiles_per_r != kt_end) describe_range();
              asm volatile("" : "+s"(rs_a), "+s"(rs_b));
            } else if (piece == 6) {
              describe_tile();
              asm volatile("" : "+s"(so_a), "+s"(so_b), "+s"(ld_tail));
            } else if (piece == 7) {
              select_offsets();
            }
          } else if constexpr (WB == 4) {
            if (kind == 1 && rq < 2 * NI) issue(rq, stage);
          } else {
            // few matrix instructions per tile: the loop waits for these loads, so out they go at once
            if (q < 2 * NI) issue(q, stage);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (t == 0) {
        // own loads of tile kt+1 have landed (the tiles behind it may still be on their way), own
        // reads of this stage are done; behind the barrier that holds for every wave
        if constexpr (NS == 2) {
          wait_for_tile(0);
        } else if constexpr (loads) {
          wait_for_tile(NS - 2);
        } else {
          const int later = kt_end - kt - 2;
          wait_for_tile(later < NS - 2 ? later : NS - 2);
        }
        __syncthreads();
      } else {
        stage = stage + 1 == NS ? 0 : stage + 1;
        flip_by = stage == NS - 1 ? 0u - (uint32_t)((NS - 1) * kStage2Bytes) : (uint32_t)kStage2Bytes;
      }
    }
  };
  int kt = 0;
  for (; kt + NS < kt_end; ++kt) tile(std::true_type{}, kt);
  for (; kt < kt_end; ++kt) tile(std::false_type{}, kt);
  // every wave must be done with the stages before LDS is reused below
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();
  settle_matrix_pipe();

  uint16_t *Cz = g.C + (long)z * g.sC;
  const int row0 = m0 + wm * WT, col0 = n0 + wn * WT;
  const bool full = row0 + WT <= g.M && col0 + WT <= g.N;  // the same for every lane of the wavefront
  // the stage buffers are free by now: a quarter of them per wavefront
  unsigned char *area = lds2 + wave * (kLds<WB> / 4);
  if (g.accumulate) {
    if (full) emit_blocks_via_lds<BF16, true, true, NBK>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    else emit_blocks_via_lds<BF16, true, false, NBK>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
  } else {
    if (full) emit_blocks_via_lds<BF16, false, true, NBK>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    else emit_blocks_via_lds<BF16, false, false, NBK>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
  }
}

template <bool BF16, int WB, int NS = 2>
int launch_big(phip_ctx *ctx, const Gemm &p, const BigArgs &a) {
  const long grid = (long)a.tiles_m * a.tiles_n * p.batch;
  constexpr int kFirstSlot = NS > 2 ? kSlotGemmH16MidDeep : WB == 4 ? kSlotGemmH16Big : kSlotGemmH16Mid;
  constexpr int kBytes = NS * kStage<WB>;
#define PHIP_LDS(SLOT, AK, BKM)                                                                   \
  do {                                                                                            \
    auto kern = gemm_h16_lds_kernel<AK, BKM, BF16, WB, NS>;                                       \
    const int rc = raise_lds_limit(ctx, kFirstSlot + (SLOT) + (BF16 ? 3 : 0),                     \
                                   reinterpret_cast<const void *>(kern), kBytes);                 \
    if (rc != PHIP_OK) return rc;                                                                 \
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), kBytes, ctx->stream, a);       \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) PHIP_LDS(0, false, true);
  else if (!p.a_kmajor && !p.b_kmajor) PHIP_LDS(1, false, false);
  else if (p.a_kmajor && p.b_kmajor) PHIP_LDS(2, true, true);
  else return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
#undef PHIP_LDS
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace

// Returns PHIP_OK and sets *handled when the problem suits the large-tile
// kernel (aligned, big enough, each operand sample under 2 GiB).
int gemm_h16_big(phip_ctx *ctx, const Gemm &p, Elem elem, bool *handled) {
  *handled = false;
  if (!rows_aligned16(p.A, 8, p.lda, p.sA, p.rA) || !rows_aligned16(p.B, 8, p.ldb, p.sB, p.rB)) return PHIP_OK;
  if ((p.a_kmajor ? p.K : p.M) % 8 != 0 || (p.b_kmajor ? p.K : p.N) % 8 != 0) return PHIP_OK;
  // C is written 8 rows (16 bytes) at a time
  if (!rows_aligned16(p.C, 8, p.ldc, p.sC, 0) || p.M % 8 != 0) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return PHIP_OK;
  const long a_bytes = 2L * p.M * p.K, b_bytes = 2L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  const int cus = ctx->prop.multiProcessorCount;
  auto tiles_of = [&](int side) { return (long)((p.M + side - 1) / side) * ((p.N + side - 1) / side) * p.batch; };
  if (p.K < 2 * BK) return PHIP_OK;
  // 256 x 256 tiles when they give at least half the CUs a workgroup; else 128 x 128 tiles (two workgroups
  // per CU) from an eighth of the CUs on, if at least half of what the tiles cover is matrix (measured on
  // M, N, K in 512 .. 4096 against the register-staged kernel: 1.3 to 3 times faster from 32 tiles on,
  // slower only where a narrow matrix leaves most of each tile empty).
  int side = kTile<4>;
  long tiles = tiles_of(side);
  if (tiles < cus / 2) {
    side = kTile<2>;
    tiles = tiles_of(side);
    if (tiles * 8 < cus || 2L * p.M * p.N * p.batch < tiles * side * side) return PHIP_OK;
  }
  if (tiles > 0x7fffffffL) return PHIP_OK;

  BigArgs a;
  a.A = static_cast<const uint16_t *>(p.A);
  a.B = static_cast<const uint16_t *>(p.B);
  a.C = static_cast<uint16_t *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.tiles_m = (p.M + side - 1) / side;
  a.tiles_n = (p.N + side - 1) / side;
  a.ktiles_per_r = (p.K + BK - 1) / BK;
  a.total_ktiles = a.ktiles_per_r * p.rbatch;
  a.accumulate = p.accumulate ? 1 : 0;
  a.a_bytes = (uint32_t)a_bytes;
  a.b_bytes = (uint32_t)b_bytes;
  // 128 x 128 tiles, at most one per CU: four stages (128 KiB), three K tiles in flight
  const bool deep = side == kTile<2> && tiles <= cus && a.total_ktiles >= 4;
  note_kernel(ctx, side == kTile<4> ? "h16_lds256" : deep ? "h16_lds128_deep" : "h16_lds128");
  *handled = true;
  if (side == kTile<4>) return elem == Elem::BF16 ? launch_big<true, 4>(ctx, p, a) : launch_big<false, 4>(ctx, p, a);
  if (deep) return elem == Elem::BF16 ? launch_big<true, 2, 4>(ctx, p, a) : launch_big<false, 2, 4>(ctx, p, a);
  return elem == Elem::BF16 ? launch_big<true, 2>(ctx, p, a) : launch_big<false, 2>(ctx, p, a);
}

}  // namespace phip
