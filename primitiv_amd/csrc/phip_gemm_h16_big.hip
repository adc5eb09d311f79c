// Large-tile GEMM for 16-bit storage (fp16 / bf16, fp32 accumulation):
// 256 x 256 x 64 tiles, one workgroup (4 wavefronts, each a 128 x 128 block of
// 4 x 4 v_mfma_f32_32x32x16 tiles) per CU, two 72 KiB LDS stages.
//
// LDS holds both operands as rows of 64 consecutive k (+8 elements of padding):
// the matrix instruction takes 8 consecutive k per lane, so every fragment is
// one 16-byte LDS read, conflict-free with the 144-byte row stride.
//  * An operand that is contiguous along k in memory is copied: 8 lanes read
//    one 128-byte line of a row and write it to the LDS row.
//  * An operand that is contiguous along m or n is transposed in registers:
//    a thread loads an 8 (k) x 8 (m) block as eight 16-byte rows, transposes
//    it with 32 byte-permutes and writes eight 16-byte LDS rows; 8 lanes
//    again cover 128 contiguous bytes on both sides.
// Global loads are raw buffer loads: everything past the end of the matrix
// reads as zero, which covers the ragged last K tile (or the last rows) without
// branches; the other edge is a per-lane offset select.
#include "phip_internal.h"
#include "phip_types.h"

namespace phip {
namespace {

typedef float float16v __attribute__((ext_vector_type(16)));
typedef _Float16 half8v __attribute__((ext_vector_type(8)));
typedef __bf16 bf8v __attribute__((ext_vector_type(8)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

constexpr int kThreads = 256;
constexpr int BM = 256, BN = 256, BK = 64;
constexpr int S = BK + 8;                       // LDS row stride in elements
constexpr int kStageA = BM * S, kStageB = BN * S;
constexpr int kLdsBytes = 2 * (kStageA + kStageB) * 2;
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

__device__ inline __amdgpu_buffer_rsrc_t make_rsrc(const uint16_t *p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<uint16_t *>(p), 0, (int)bytes, 0x00020000);
}

// One operand's 256 x 64 tile.  KMAJOR: element (x, k) at k + x*ld.
// Otherwise: element (x, k) at x + k*ld.
template <bool KMAJOR>
struct TileLoader {
  uint4v regs[8];
  uint32_t off[8];   // byte offsets of this thread's eight vectors at k0 = 0
  uint32_t step;     // bytes to advance per K tile
  int kg;            // which 8-wide k group of the tile this thread serves
  bool x_in;         // (x-contiguous only) the thread's 8 columns exist
  uint32_t lds_off;  // element offset of this thread's first LDS row segment

  __device__ inline void init(long ld, int x0, int X, int tid) {
    kg = tid & 7;
    const int xr = tid >> 3;
    if constexpr (KMAJOR) {
      // rows x = x0 + xr + 32 i; a row past X starts past the end of the matrix
#pragma unroll
      for (int i = 0; i < 8; ++i) off[i] = (uint32_t)(((long)(x0 + xr + 32 * i) * ld + kg * 8) * 2);
      step = BK * 2;
      x_in = true;
      lds_off = xr * S + kg * 8;
    } else {
      // an 8 x 8 block: k rows kg*8 + i, columns x0 + xr*8 .. +7
#pragma unroll
      for (int i = 0; i < 8; ++i) off[i] = (uint32_t)(((long)(kg * 8 + i) * ld + x0 + xr * 8) * 2);
      step = (uint32_t)(BK * ld * 2);
      x_in = x0 + xr * 8 < X;
      lds_off = (xr * 8) * S + kg * 8;
    }
  }

  // Prepares tile `kt_in_r` of the current sample; `live` false turns every
  // load of the tile into an out-of-range one (reads zeros, touches nothing).
  uint32_t adv;
  bool in;
  __device__ inline void begin(int kt_in_r, int K, bool live) {
    adv = (uint32_t)kt_in_r * step;
    if constexpr (KMAJOR) in = live && kt_in_r * BK + kg * 8 < K;  // the next column starts right after K
    else in = live && x_in;                                         // rows past K are past the end
  }
  __device__ inline void load_one(__amdgpu_buffer_rsrc_t rsrc, int i) {
    const uint32_t o = in ? off[i] + adv : kOutOfRange;
    regs[i] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, (int)o, 0, 0);
  }
  __device__ inline void load(__amdgpu_buffer_rsrc_t rsrc, int kt_in_r, int K) {
    begin(kt_in_r, K, true);
#pragma unroll
    for (int i = 0; i < 8; ++i) load_one(rsrc, i);
  }

  // Writes the j-th of this thread's eight 16-byte LDS row segments.
  __device__ inline void store_one(uint16_t *lds, int j) const {
    uint16_t *p = lds + lds_off;
    if constexpr (KMAJOR) {
      *reinterpret_cast<uint4v *>(p + 32 * j * S) = regs[j];
    } else {
      // regs[i] = 8 columns of k row i.  Output row j = column j across the 8
      // k rows: dword d of it packs (row 2d, row 2d+1) of element j.
      const uint32_t sel = (j & 1) ? 0x07060302u : 0x05040100u;
      uint4v o;
      o.x = __builtin_amdgcn_perm(regs[1][j >> 1], regs[0][j >> 1], sel);
      o.y = __builtin_amdgcn_perm(regs[3][j >> 1], regs[2][j >> 1], sel);
      o.z = __builtin_amdgcn_perm(regs[5][j >> 1], regs[4][j >> 1], sel);
      o.w = __builtin_amdgcn_perm(regs[7][j >> 1], regs[6][j >> 1], sel);
      *reinterpret_cast<uint4v *>(p + j * S) = o;
    }
  }
  __device__ inline void store(uint16_t *lds) const {
#pragma unroll
    for (int j = 0; j < 8; ++j) store_one(lds, j);
  }
};

template <bool BF16>
__device__ inline float16v mfma(uint4v a, uint4v b, float16v c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf8v, a), __builtin_bit_cast(bf8v, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8v, a), __builtin_bit_cast(half8v, b), c, 0, 0, 0);
  }
}

template <bool BF16>
__device__ inline float load_c(const uint16_t *p) {
  if constexpr (BF16) {
    bf16_t t; t.bits = *p; return to_f32(t);
  } else {
    return to_f32(__builtin_bit_cast(f16_t, *p));
  }
}

template <bool BF16>
__device__ inline uint16_t round_c(float x) {
  if constexpr (BF16) return from_f32<bf16_t>(x).bits;
  else return __builtin_bit_cast(uint16_t, from_f32<f16_t>(x));
}

template <bool A_KMAJOR, bool B_KMAJOR, bool BF16>
__global__ __launch_bounds__(kThreads, 1) void gemm_h16_big_kernel(const BigArgs g) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint16_t *lds = reinterpret_cast<uint16_t *>(lds_raw);

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;

  // Tile order: z slowest; inside one sample, groups of 8 tile rows are walked
  // column by column so that the ~32 tiles an XCD runs together share panels.
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

  TileLoader<A_KMAJOR> la;
  TileLoader<B_KMAJOR> lb;
  la.init(g.lda, m0, g.M, tid);
  lb.init(g.ldb, n0, g.N, tid);

  const uint16_t *Az = g.A + (long)z * g.sA;
  const uint16_t *Bz = g.B + (long)z * g.sB;

  float16v acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int kt_end = g.total_ktiles;
  {
    la.load(make_rsrc(Az, g.a_bytes), 0, g.K);
    lb.load(make_rsrc(Bz, g.b_bytes), 0, g.K);
    la.store(lds);
    lb.store(lds + 2 * kStageA);
  }
  __syncthreads();

  // Lane l supplies row l%32 and the 8 k values starting at 8*(l/32).
  const int frag_off = (lane & 31) * S + 8 * (lane >> 5);
  const uint16_t *a_frag = lds + wm * 128 * S + frag_off;
  const uint16_t *b_frag = lds + 2 * kStageA + wn * 128 * S + frag_off;

  // Fragments are double-buffered in registers: the reads of k step s+1 are
  // issued between the matrix instructions of step s, and the first step of
  // the next tile is read behind the barrier, under the last step of this one.
  uint4v fa[2][4], fb[2][4];
  auto read_frag = [&](int buf, int q, int stage, int s) {
    if (q < 4) fa[buf][q] = *reinterpret_cast<const uint4v *>(a_frag + stage * kStageA + q * 32 * S + s * 16);
    else fb[buf][q - 4] = *reinterpret_cast<const uint4v *>(b_frag + stage * kStageB + (q - 4) * 32 * S + s * 16);
  };
#pragma unroll
  for (int q = 0; q < 8; ++q) read_frag(0, q, 0, 0);

  for (int kt = 0; kt < kt_end; ++kt) {
    const int stage = kt & 1;
    // Next tile (loads degenerate to out-of-range reads after the last one).
    const bool more = kt + 1 < kt_end;
    const int nkt = more ? kt + 1 : kt;
    const int r = nkt / g.ktiles_per_r;
    const int kt_in_r = nkt - r * g.ktiles_per_r;
    const __amdgpu_buffer_rsrc_t ra = make_rsrc(Az + (long)r * g.rA, g.a_bytes);
    const __amdgpu_buffer_rsrc_t rb = make_rsrc(Bz + (long)r * g.rB, g.b_bytes);
    la.begin(kt_in_r, g.K, more);
    lb.begin(kt_in_r, g.K, more);
    uint16_t *next_a = lds + (stage ^ 1) * kStageA;
    uint16_t *next_b = lds + 2 * kStageA + (stage ^ 1) * kStageB;

#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int cur = s & 1, nxt = cur ^ 1;
#pragma unroll
      for (int q = 0; q < 16; ++q) {
        const int i = q >> 2, j = q & 3;
        acc[i][j] = mfma<BF16>(fb[cur][j], fa[cur][i], acc[i][j]);
        // work slotted in behind this matrix instruction
        if (s == 0) {
          if (q < 8) la.load_one(ra, q); else lb.load_one(rb, q - 8);
        }
        if (q < 8) {
          if (s < 3) read_frag(nxt, q, stage, s + 1);
          else read_frag(nxt, q, stage ^ 1, 0);
        }
        if (s == 2) {
          if (q < 8) la.store_one(next_a, q); else lb.store_one(next_b, q - 8);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (s == 2) __syncthreads();
    }
  }

  // Lane l of result register v holds C(m, n) with m = l % 32 and
  // n = 8*(v/4) + 4*(l/32) + v%4 inside its 32x32 block.
  uint16_t *Cz = g.C + (long)z * g.sC;
  const int cm = m0 + wm * 128 + (lane & 31);
  const int cn = n0 + wn * 128 + 4 * (lane >> 5);
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = cm + i * 32;
    if (m >= g.M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int n = cn + j * 32 + 8 * (v / 4) + (v % 4);
        if (n < g.N) {
          uint16_t *p = Cz + m + (long)n * g.ldc;
          const float s = acc[i][j][v];
          *p = round_c<BF16>(g.accumulate ? load_c<BF16>(p) + s : s);
        }
      }
  }
}

template <bool BF16>
int launch_big(phip_ctx *ctx, const Gemm &p, const BigArgs &a) {
  const long grid = (long)a.tiles_m * a.tiles_n * p.batch;
#define PHIP_BIG(AK, BKM)                                                                        \
  do {                                                                                           \
    auto kern = gemm_h16_big_kernel<AK, BKM, BF16>;                                              \
    static bool configured = false;                                                              \
    if (!configured) {                                                                           \
      PHIP_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(kern),                         \
                                   hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes));      \
      configured = true;                                                                         \
    }                                                                                            \
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), kLdsBytes, ctx->stream, a);   \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) PHIP_BIG(false, true);
  else if (!p.a_kmajor && !p.b_kmajor) PHIP_BIG(false, false);
  else if (p.a_kmajor && p.b_kmajor) PHIP_BIG(true, true);
  else return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
#undef PHIP_BIG
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace

// Returns PHIP_OK and sets *handled when the problem suits the large-tile
// kernel (aligned, big enough, each operand sample under 2 GiB).
int gemm_h16_big(phip_ctx *ctx, const Gemm &p, Elem elem, bool *handled) {
  *handled = false;
  auto aligned = [](const void *ptr, long ld, long s, long r) {
    return (reinterpret_cast<uintptr_t>(ptr) % 16 == 0) && ld % 8 == 0 && s % 8 == 0 && r % 8 == 0;
  };
  if (!aligned(p.A, p.lda, p.sA, p.rA) || !aligned(p.B, p.ldb, p.sB, p.rB)) return PHIP_OK;
  if ((p.a_kmajor ? p.K : p.M) % 8 != 0 || (p.b_kmajor ? p.K : p.N) % 8 != 0) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return PHIP_OK;
  const long a_bytes = 2L * p.M * p.K, b_bytes = 2L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  const long tiles = (long)((p.M + BM - 1) / BM) * ((p.N + BN - 1) / BN) * p.batch;
  const int cus = ctx->prop.multiProcessorCount;
  if (tiles < cus / 2 || p.K < 2 * BK) return PHIP_OK;
  if (tiles > 0x7fffffffL) return PHIP_OK;

  BigArgs a;
  a.A = static_cast<const uint16_t *>(p.A);
  a.B = static_cast<const uint16_t *>(p.B);
  a.C = static_cast<uint16_t *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.tiles_m = (p.M + BM - 1) / BM;
  a.tiles_n = (p.N + BN - 1) / BN;
  a.ktiles_per_r = (p.K + BK - 1) / BK;
  a.total_ktiles = a.ktiles_per_r * p.rbatch;
  a.accumulate = p.accumulate ? 1 : 0;
  a.a_bytes = (uint32_t)a_bytes;
  a.b_bytes = (uint32_t)b_bytes;
  *handled = true;
  return elem == Elem::BF16 ? launch_big<true>(ctx, p, a) : launch_big<false>(ctx, p, a);
}

}  // namespace phip
