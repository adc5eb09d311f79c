// Large-tile GEMM for 16-bit storage (fp16 / bf16, fp32 accumulation):
// 256 x 256 x 64 tiles, one workgroup (4 wavefronts, each a 128 x 128 block of
// 4 x 4 v_mfma_f32_32x32x16 tiles, 256 accumulator registers per lane) per CU,
// two 64 KiB LDS stages.  Problems with too few such tiles for the chip take
// 128 x 128 x 64 tiles instead (wavefronts of 2 x 2 blocks, two 32 KiB stages,
// two workgroups per CU): the same code with half the extents.
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
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int BK = 64;
// WB = 32 x 32 blocks per wavefront and direction: 4 -> 256 x 256 tiles (one workgroup per CU),
// 2 -> 128 x 128 tiles (two workgroups per CU) for problems with too few large tiles
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

template <bool BF16>
__device__ inline float16v mfma(uint4v a, uint4v b, float16v c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8v, a), __builtin_bit_cast(bf8v, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, a), __builtin_bit_cast(half8v, b), c, 0, 0, 0);
  }
}

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

// Writes the 128 x 128 block of results one wavefront holds into the 16-bit C,
// 16 bytes (8 consecutive rows of one column) per lane and store instruction.
// The matrix instruction leaves a lane with one row and 16 columns of each
// 32 x 32 block, so the block is turned through a 32 KiB LDS area that belongs
// to this wavefront alone: written as fp32 the way the accumulators lie,
// read back 8 consecutive rows at a time, in two halves of 64 columns.  For an
// accumulating write the old values are fetched (also 16 bytes per lane)
// before the LDS pass, added in fp32 and rounded once.  M is a multiple of 8
// and C is 16-byte aligned (checked by the dispatcher), so a lane's 8 rows are
// either all inside the matrix or all outside.
//
// The area holds column c as 128 floats; row r of column c sits at position
//   r ^ (4 * bit 6 of r) ^ (32 * bit 2 of c).
// The first term makes the two 16-byte halves of rows 64..127 change places,
// so that the 16 lanes of one read instruction (8 rows = 32 bytes apart) cover
// all banks; the second moves the columns the upper half wave writes (4 further
// on) to the other half of the banks.  Both are constants of a lane's address.
//
// FULL: the block lies inside the matrix, no lane is masked and the addresses
// step by a constant; otherwise every access is checked on its own.
template <bool BF16, bool ACC, bool FULL>
__device__ inline void emit_block_via_lds(float *area, uint16_t *Cz, long ldc, int row0, int col0, int lane, int M,
                                          int N, const float16v (&acc)[4][4]) {
  const int mc = lane & 15, cq = lane >> 4;
  const int m = row0 + 8 * mc;
  const int flip = mc >> 3;  // rows 64..127: halves swapped
  // write side: rows 32 i + lane % 32 of columns 32 jl + 8 (v / 4) + 4 (lane / 32) + v % 4
  float *wbase[4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
    wbase[i] = area + (4 * (lane >> 5)) * 128 + ((32 * i + (lane & 31)) ^ (4 * (i >> 1)) ^ (32 * (lane >> 5)));
  // read side: column 4 it + cq, rows 8 mc .. 8 mc + 7
  const float *reven = area + cq * 128 + 8 * mc;               // even it
  const float *rodd = area + cq * 128 + 8 * (mc ^ 4);          // odd it
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    uint16_t *p0 = Cz + m + (long)(col0 + 64 * h + cq) * ldc;
    uint32_t ok = 0xffffu;
    if constexpr (!FULL) {
      ok = 0;
#pragma unroll
      for (int it = 0; it < 16; ++it)
        ok |= (m < M && col0 + 64 * h + 4 * it + cq < N ? 1u : 0u) << it;
    }
    auto live = [&](int it) { return FULL || ((ok >> it) & 1u); };
    uint4v old[16];
    if constexpr (ACC) {
#pragma unroll
      for (int it = 0; it < 16; ++it) {
        old[it] = uint4v{0, 0, 0, 0};
        if (live(it)) old[it] = *reinterpret_cast<const uint4v *>(p0 + (long)(4 * it) * ldc);
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int jl = 0; jl < 2; ++jl)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          wbase[i][(32 * jl + 8 * (v / 4) + (v % 4)) * 128] = acc[i][2 * h + jl][v];
    float4 lo[16], hi[16];
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      const float4 *src = reinterpret_cast<const float4 *>(((it & 1) ? rodd : reven) + 4 * it * 128);
      lo[it] = src[flip];
      hi[it] = src[flip ^ 1];
    }
#pragma unroll
    for (int it = 0; it < 16; ++it) {
      float f[8] = {lo[it].x, lo[it].y, lo[it].z, lo[it].w, hi[it].x, hi[it].y, hi[it].z, hi[it].w};
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
      if (live(it)) *reinterpret_cast<uint4v *>(p0 + (long)(4 * it) * ldc) = out;
    }
  }
}

// The same for the 64 x 64 block of a wavefront of the 128 x 128 tiles: one pass
// through a 16 KiB area of 64 columns x 64 rows.  Row r of column c sits at
//   r ^ (4 * bit 0 of c) ^ (32 * bit 2 of c):
// a read instruction covers 8 columns (8 lanes of 8 rows each), and two
// neighbouring columns, 256 bytes apart, would meet in the same banks without
// the first term; the second separates the two half waves' writes as above.
template <bool BF16, bool ACC, bool FULL>
__device__ inline void emit_block64_via_lds(float *area, uint16_t *Cz, long ldc, int row0, int col0, int lane, int M,
                                            int N, const float16v (&acc)[2][2]) {
  const int mc = lane & 7, cq = lane >> 3;
  const int m = row0 + 8 * mc;
  const int flip = cq & 1;
  const int u = lane >> 5, l5 = lane & 31;
  // write side: rows 32 i + lane % 32 of columns 32 j + 8 (v / 4) + 4 (lane / 32) + v % 4
  float *wbase[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int par = 0; par < 2; ++par) wbase[i][par] = area + (4 * u) * 64 + 32 * (i ^ u) + (l5 ^ (4 * par));
  // read side: column 8 it + cq, rows 8 mc .. 8 mc + 7
  const float *rbase = area + cq * 64 + 8 * (mc ^ (4 * ((cq >> 2) & 1)));
  uint16_t *p0 = Cz + m + (long)(col0 + cq) * ldc;
  uint32_t ok = 0xffu;
  if constexpr (!FULL) {
    ok = 0;
#pragma unroll
    for (int it = 0; it < 8; ++it) ok |= (m < M && col0 + 8 * it + cq < N ? 1u : 0u) << it;
  }
  auto live = [&](int it) { return FULL || ((ok >> it) & 1u); };
  uint4v old[8];
  if constexpr (ACC) {
#pragma unroll
    for (int it = 0; it < 8; ++it) {
      old[it] = uint4v{0, 0, 0, 0};
      if (live(it)) old[it] = *reinterpret_cast<const uint4v *>(p0 + (long)(8 * it) * ldc);
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) wbase[i][v & 1][(32 * j + 8 * (v / 4) + (v % 4)) * 64] = acc[i][j][v];
  float4 lo[8], hi[8];
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const float4 *src = reinterpret_cast<const float4 *>(rbase + 8 * it * 64);
    lo[it] = src[flip];
    hi[it] = src[flip ^ 1];
  }
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    float f[8] = {lo[it].x, lo[it].y, lo[it].z, lo[it].w, hi[it].x, hi[it].y, hi[it].z, hi[it].w};
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
    if (live(it)) *reinterpret_cast<uint4v *>(p0 + (long)(8 * it) * ldc) = out;
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
//    chunks.  Chunk c of row k sits at position c ^ ((k & 3) << 2): the four k
//    rows one transposing read touches land in different bank groups.
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
// lands at lds_addr + 16*l.  Issued as inline assembly so that the compiler
// does not put a wait for it in front of every later LDS read; the kernel
// waits for these loads itself (s_waitcnt vmcnt) before the barrier that
// publishes the tile.
__device__ inline void lds_dma_b128(uint4v rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");  // m0 is scratch between instructions: nothing else in this kernel keeps a value in it
}

template <bool KMAJOR, int WB>
struct LdsLoader {
  static constexpr int NI = 2 * WB;   // the wave's load instructions (1 KiB of LDS each) per operand tile
  static constexpr int CW = 8 * WB;   // (m/n-contiguous) 16-byte chunks per k row of the tile
  uint32_t off[NI];    // byte offset of this lane's chunk for each of the wave's instructions, at K tile 0
  uint32_t step;       // bytes per K tile
  uint32_t live_mask;  // bit q: instruction q's chunk exists (along the axis that needs a predicate)
  int kc[NI];          // (k-contiguous only) first k of the chunk inside the tile, per instruction

  __device__ inline void init(long ld, int x0, int X, int wave, int lane) {
    live_mask = 0;
#pragma unroll
    for (int q = 0; q < NI; ++q) {
      const int blk = wave * NI + q;  // which 1 KiB block of the region
      if constexpr (KMAJOR) {
        const int x = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((x >> 1) & 7);
        off[q] = (uint32_t)(((long)(x0 + x) * ld + c * 8) * 2);  // a row past X is past the end
        kc[q] = c * 8;
      } else {
        const int k = blk * (64 / CW) + lane / CW;
        const int c = (lane % CW) ^ ((k & 3) << 2);
        off[q] = (uint32_t)(((long)k * ld + x0 + c * 8) * 2);    // a row past K is past the end
        kc[q] = 0;
        if (x0 + c * 8 < X) live_mask |= 1u << q;
      }
    }
    step = KMAJOR ? (uint32_t)(BK * 2) : (uint32_t)(BK * ld * 2);
  }

  // Issues instruction q of K tile `kt_in_r`; `live` false makes it a no-op read.
  __device__ inline void issue(uint4v rsrc, uint32_t region_addr, int wave, int q, int kt_in_r, int K,
                               bool live) const {
    bool in = live;
    if constexpr (KMAJOR) in = in && kt_in_r * BK + kc[q] < K;
    else in = in && ((live_mask >> q) & 1u);
    const uint32_t o = in ? off[q] + (uint32_t)kt_in_r * step : kOutOfRange;
    lds_dma_b128(rsrc, region_addr + (uint32_t)(wave * NI + q) * 1024u, o);
  }
};

// Per-lane constants of the fragment reads of one operand.
template <bool KMAJOR, int WB>
struct FragReader {
  static constexpr int kPitch = 128 * WB;  // (m/n-contiguous) bytes per k row
  uint32_t base[4];  // byte offsets inside the region

  __device__ inline void init(int xw, int lane) {
    if constexpr (KMAJOR) {
      // row x = xw + 32 i + lane%32, chunk (2 s + lane/32) ^ swizzle: base[s]
      const int sw = ((lane & 31) >> 1) & 7;
#pragma unroll
      for (int s = 0; s < 4; ++s)
        base[s] = (uint32_t)((xw + (lane & 31)) * 128 + (((2 * s + (lane >> 5)) ^ sw) * 16));
    } else {
      // lane = 16 g + 4 cc + a: supplies k row cc, columns 16 (g%2) + 4 a .. +3: base[i];
      // chunk xw/8 + 4 i + cl of row k sits at that index ^ (4 (k & 3))
      const int h = lane >> 5, cc = (lane & 15) >> 2, a = lane & 3;
      const int cl = (16 * ((lane >> 4) & 1) + 4 * a) >> 3;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        base[i] = (uint32_t)((8 * h + cc) * kPitch + ((xw / 8 + 4 * i + cl) ^ (4 * cc)) * 16 + (a & 1) * 8);
    }
  }

  // Fragment of 32x32 block i for k step s: 8 consecutive k of row lane%32.
  __device__ inline uint4v read(const unsigned char *region, int i, int s) const {
    if constexpr (KMAJOR) {
      return *reinterpret_cast<const uint4v *>(region + base[s] + i * 4096);
    } else {
      const unsigned char *p = region + base[i] + s * 16 * kPitch;
      const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) short4v *)(p));
      const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
          (__attribute__((address_space(3))) short4v *)(p + 4 * kPitch));
      uint4v r;
      r.x = (uint32_t)(uint16_t)lo[0] | ((uint32_t)(uint16_t)lo[1] << 16);
      r.y = (uint32_t)(uint16_t)lo[2] | ((uint32_t)(uint16_t)lo[3] << 16);
      r.z = (uint32_t)(uint16_t)hi[0] | ((uint32_t)(uint16_t)hi[1] << 16);
      r.w = (uint32_t)(uint16_t)hi[2] | ((uint32_t)(uint16_t)hi[3] << 16);
      return r;
    }
  }
};

template <bool A_KMAJOR, bool B_KMAJOR, bool BF16, int WB>
__global__ __launch_bounds__(kThreads, WB == 4 ? 1 : 2) void gemm_h16_lds_kernel(const BigArgs g) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds2[];
  constexpr int BM = kTile<WB>, BN = kTile<WB>;
  constexpr int kRegionBytes = kRegion<WB>, kStage2Bytes = kStage<WB>;
  constexpr int WT = 32 * WB;       // rows = columns of a wavefront's block
  constexpr int NI = 2 * WB;        // load instructions per wavefront, operand and K tile
  constexpr int NB = WB * WB;       // matrix instructions per k step

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

  LdsLoader<A_KMAJOR, WB> la;
  LdsLoader<B_KMAJOR, WB> lb;
  la.init(g.lda, m0, g.M, wave, lane);
  lb.init(g.ldb, n0, g.N, wave, lane);
  FragReader<A_KMAJOR, WB> fra;
  FragReader<B_KMAJOR, WB> frb;
  fra.init(wm * WT, lane);
  frb.init(wn * WT, lane);

  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;

  float16v acc[WB][WB];
#pragma unroll
  for (int i = 0; i < WB; ++i)
#pragma unroll
    for (int j = 0; j < WB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int kt_end = g.total_ktiles;
  // Every workgroup starts its walk over K at a different tile (and wraps
  // around): with power-of-two leading dimensions, workgroups marching through
  // K in lockstep would all pull from the same memory channels at once.
  const int kt_rot = (tile_m + tile_n + z) % kt_end;
  const uint32_t lds_base = (uint32_t)(size_t)(__attribute__((address_space(3))) unsigned char *)lds2;
  auto issue_tile = [&](int kt, int q_first, int q_count) {
    // instructions [q_first, q_first + q_count) of the 2 NI that move K tile kt (NI for A, then NI for B)
    const bool live = kt < kt_end;
    int ktc = live ? kt + kt_rot : 0;
    ktc = ktc >= kt_end ? ktc - kt_end : ktc;
    const int r = ktc / g.ktiles_per_r;
    const int kt_in_r = ktc - r * g.ktiles_per_r;
    const uint32_t stage = lds_base + (uint32_t)(kt & 1) * kStage2Bytes;
#pragma unroll
    for (int q = q_first; q < q_first + q_count; ++q) {
      if (q < NI) la.issue(make_rsrc_words(Az + (long)r * g.rA, g.a_bytes), stage, wave, q, kt_in_r, g.K, live);
      else lb.issue(make_rsrc_words(Bz + (long)r * g.rB, g.b_bytes), stage + kRegionBytes, wave, q - NI, kt_in_r,
                    g.K, live);
    }
  };

  issue_tile(0, 0, 2 * NI);
  issue_tile(1, 0, 2 * NI);
  // tile 0 has landed once all but the newest 2 NI loads are done
  if constexpr (WB == 4) asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
  else asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
  __syncthreads();

  // Fragments of the four k steps of a tile live in four register buffers and
  // are read two steps ahead: steps 2 and 3 of this tile during steps 0 and 1,
  // then - behind the barrier - steps 0 and 1 of the next tile during steps 2
  // and 3.  The barrier therefore sits in the middle of a tile, and the
  // global-to-LDS loads that refill the stage (K tile kt+2) are spread over
  // the instruction slots of steps 2 and 3, with a whole tile time to land.
  uint4v fa[4][WB], fb[4][WB];
  auto read_frag = [&](int buf, int q, int stage, int s) {
    const unsigned char *st = lds2 + stage * kStage2Bytes;
    if (q < WB) fa[buf][q] = fra.read(st, q, s);
    else fb[buf][q - WB] = frb.read(st + kRegionBytes, q - WB, s);
  };
#pragma unroll
  for (int q = 0; q < 2 * WB; ++q) read_frag(0, q, 0, 0);
#pragma unroll
  for (int q = 0; q < 2 * WB; ++q) read_frag(1, q, 0, 1);

  // the 2 NI loads of a K tile go out in steps 2 and 3: NI per step, one every NB / NI matrix instructions
  constexpr int kEvery = NB / NI;
  for (int kt = 0; kt < kt_end; ++kt) {
    const int stage = kt & 1;
#pragma unroll
    for (int s = 0; s < 4; ++s) {
#pragma unroll
      for (int q = 0; q < NB; ++q) {
        const int i = q / WB, j = q % WB;
        acc[i][j] = mfma<BF16>(fb[s][j], fa[s][i], acc[i][j]);
        if (q < 2 * WB) {
          if (s < 2) read_frag(s + 2, q, stage, s + 2);
          else read_frag(s - 2, q, stage ^ 1, s - 2);
        }
        if (s >= 2 && q % kEvery == kEvery - 1) issue_tile(kt + 2, (s - 2) * NI + q / kEvery, 1);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (s == 1) {
        // own loads of tile kt+1 have landed, own reads of this stage are done;
        // behind the barrier that holds for every wave
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        __syncthreads();
      }
    }
  }
  // The loads issued for tiles past the end move nothing, but must have retired,
  // and every wave must be done with the stages, before LDS is reused below.
  asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
  __syncthreads();

  uint16_t *Cz = g.C + (long)z * g.sC;
  const int row0 = m0 + wm * WT, col0 = n0 + wn * WT;
  const bool full = row0 + WT <= g.M && col0 + WT <= g.N;  // the same for every lane of the wavefront
  if constexpr (WB == 4) {
    float *area = reinterpret_cast<float *>(lds2 + wave * kRegionBytes);
    if (g.accumulate) {
      if (full) emit_block_via_lds<BF16, true, true>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
      else emit_block_via_lds<BF16, true, false>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    } else {
      if (full) emit_block_via_lds<BF16, false, true>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
      else emit_block_via_lds<BF16, false, false>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    }
  } else {
    float *area = reinterpret_cast<float *>(lds2 + wave * (kLds<WB> / 4));
    if (g.accumulate) {
      if (full) emit_block64_via_lds<BF16, true, true>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
      else emit_block64_via_lds<BF16, true, false>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    } else {
      if (full) emit_block64_via_lds<BF16, false, true>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
      else emit_block64_via_lds<BF16, false, false>(area, Cz, g.ldc, row0, col0, lane, g.M, g.N, acc);
    }
  }
}

template <bool BF16, int WB>
int launch_big(phip_ctx *ctx, const Gemm &p, const BigArgs &a) {
  const long grid = (long)a.tiles_m * a.tiles_n * p.batch;
  constexpr int kFirstSlot = WB == 4 ? kSlotGemmH16Big : kSlotGemmH16Mid;
#define PHIP_LDS(SLOT, AK, BKM)                                                                   \
  do {                                                                                            \
    auto kern = gemm_h16_lds_kernel<AK, BKM, BF16, WB>;                                           \
    const int rc = raise_lds_limit(ctx, kFirstSlot + (SLOT) + (BF16 ? 3 : 0),                     \
                                   reinterpret_cast<const void *>(kern), kLds<WB>);               \
    if (rc != PHIP_OK) return rc;                                                                 \
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), kLds<WB>, ctx->stream, a);     \
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
  *handled = true;
  if (side == kTile<4>) return elem == Elem::BF16 ? launch_big<true, 4>(ctx, p, a) : launch_big<false, 4>(ctx, p, a);
  return elem == Elem::BF16 ? launch_big<true, 2>(ctx, p, a) : launch_big<false, 2>(ctx, p, a);
}

}  // namespace phip
