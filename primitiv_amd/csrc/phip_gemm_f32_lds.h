// Pieces shared by the fp32 GEMM kernels whose operands travel global -> LDS by
// buffer loads that write LDS directly: the load instruction, the per-wave
// loader of one operand tile and the reader of matrix-instruction fragments.
//
// LDS image of one operand tile (ROWS rows or columns by 32 k):
//  * contiguous along m or n: 32 rows (k) of ROWS floats, exactly as in memory.
//    A fragment is one 4-byte read per lane (32 consecutive floats per half
//    wave).
//  * contiguous along k: ROWS rows (m or n) of 32 k = 128 bytes = 8 chunks of 16
//    bytes; chunk c of row x sits at position c ^ ((x >> 1) & 7), so that the
//    16-byte reads of 16 consecutive rows hit 16 different bank groups.  A
//    fragment is one 16-byte read per lane: 4 consecutive k of the lane's row.
// K is walked in groups of 8: the four matrix instructions of a group use
// k = k0 + 4*(lane/32) + e, e = 0..3, for both operands, which is what makes the
// 16-byte form possible.
#ifndef PHIP_GEMM_F32_LDS_H_
#define PHIP_GEMM_F32_LDS_H_

#include "phip_gemm_f32_common.h"

namespace phip {
namespace {

typedef uint32_t uint4v __attribute__((ext_vector_type(4)));


constexpr int LBK = 32;
constexpr uint32_t kOutOfRange = 0x80000000u;

struct LdsArgs {
  GemmArgs g;
  uint32_t a_bytes, b_bytes;  // size of one sample of each operand
  int whole_tiles;            // streamed-operand kernel: leading workgroups that take an unsplit tile each
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
// m0 is scratch between instructions: nothing else here keeps a value in it;
// the wait state between its write and the load is the one the instruction set
// asks for.
__device__ inline void lds_dma_b128(uint4v rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}

// The 4-byte form: lane l's data lands at lds_addr + 4*l.
__device__ inline void lds_dma_b32(uint4v rsrc, uint32_t lds_addr, uint32_t voffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dword %1, %2, 0 offen lds"
               :
               : "s"(lds_addr), "v"(voffset), "s"(rsrc)
               : "memory");
}

// The wave's load instructions (1 KiB of LDS each) for one operand tile of
// ROWS rows or columns by 32 k: ROWS / 32 per wavefront of a workgroup of four
// (ROWS / 8 between the WAVES wavefronts of the workgroup).
template <bool KMAJOR, int ROWS = 128, int WAVES = 4>
struct DmaLoader {
  static constexpr int kInstr = ROWS / 8 / WAVES;
  static constexpr int kLanesPerRow = ROWS / 4;  // (m/n-contiguous) lanes that cover one k row
  uint32_t off[kInstr];  // byte offset of this lane's chunk per instruction, at K tile 0
  uint32_t step;         // bytes per K tile
  uint32_t live_mask;    // (m/n-contiguous) bit q: the chunk's columns exist
  int kc[kInstr];        // (k-contiguous) first k of the chunk inside the tile

  __device__ inline void init(long ld, int x0, int X, int wave, int lane) {
    live_mask = 0;
#pragma unroll
    for (int q = 0; q < kInstr; ++q) {
      const int blk = wave * kInstr + q;  // which 1 KiB block of the region
      if constexpr (KMAJOR) {
        const int x = blk * 8 + (lane >> 3);
        const int c = (lane & 7) ^ ((x >> 1) & 7);
        off[q] = x0 + x < X ? (uint32_t)(((long)(x0 + x) * ld + c * 4) * 4) : kOutOfRange;
        kc[q] = c * 4;
      } else {
        const int k = blk * (64 / kLanesPerRow) + lane / kLanesPerRow;
        const int c = lane % kLanesPerRow;
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
    lds_dma_b128(rsrc, region_addr + (uint32_t)(wave * kInstr + q) * 1024u, o);
  }

  // (k-contiguous, K not a multiple of four) After instruction q of K tile kt_in_r has landed in
  // `region`: if this lane's chunk holds k = K-1, its elements from k = K on came from the next row
  // of the operand; they become zeros, so that they meet the other operand's zeros as zeros.
  __device__ inline void zero_tail(unsigned char *region, int wave, int q, int lane, int kt_in_r, int K) const {
    if constexpr (KMAJOR) {
      const int k0 = kt_in_r * LBK + kc[q];
      if (k0 < K && K < k0 + 4) {
        float *chunk = reinterpret_cast<float *>(region + (wave * kInstr + q) * 1024 + lane * 16);
#pragma unroll
        for (int e = 1; e < 4; ++e)
          if (k0 + e >= K) chunk[e] = 0.0f;
      }
    }
  }
};

// Fragments of one operand for one group of 8 k: v[block][e].
template <bool KMAJOR, int ROWS = 128>
struct FragReaderF {
  static constexpr int kPitch = ROWS * 4;  // (m/n-contiguous) bytes per k row
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
      base[0] = (uint32_t)((4 * (lane >> 5)) * kPitch + (xw + (lane & 31)) * 4);
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
          v[i][e] = *reinterpret_cast<const float *>(region + base[0] + (8 * gk + e) * kPitch + i * 128);
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
      v[i][e] = *reinterpret_cast<const float *>(region + base[0] + (8 * gk + e) * kPitch + i * 128);
    }
  }
};

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_LDS_H_
