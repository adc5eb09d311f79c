// fp32 GEMM for products that stream one large operand against a narrow one
// (at most 64 columns of output): the per-timestep products of an output
// projection, y = W.x, gx = W^T.gy, whose cost is reading W once.
//
// 32 x 64 output tiles.  Operands move global -> LDS by buffer loads that write
// LDS directly, in stages of 32 k (A 4 KiB + B 8 KiB); four stages are in
// flight.  The four wavefronts of a workgroup split K: wavefront w takes k
// group w (8 k) of every stage, all 32 x 64 outputs (8 matrix instructions per
// stage), and the four partial tiles are summed through LDS at the end.  The
// fragments of stage l+1 are read, and the loads of stage l+4 issued, between
// the matrix instructions of stage l.  When there are fewer output tiles than
// places for workgroups (two per compute unit), the K range is also cut
// between workgroups, whose tiles are added into C with fp32 atomics; an
// overwriting product zero-fills C first.
#include <type_traits>

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

template <bool A_KMAJOR, bool B_KMAJOR, int VB>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_slab_kernel(const LdsArgs d) {
  static_assert(VB == 4 || B_KMAJOR, "only a k-contiguous operand has the 4-byte loader");
  typedef typename std::conditional<VB == 4, DmaLoader<B_KMAJOR, TBN>, DmaLoaderDword<TBN>>::type LoaderB;
  constexpr int kDmaB = LoaderB::kInstr;
  constexpr int kDma = 1 + kDmaB;  // load instructions per wavefront per stage
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);

  // tiles of one K range are neighbours: they read the same rows of B
  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int split = t % g.splits;
  const int z = t / g.splits;
  const int m0 = tile_m * TBM;

  // K tiles (32 k, one per stage) [kb, ke) belong to this workgroup
  const int kb = (int)((long)split * g.total_ktiles / g.splits);
  const int ke = (int)((long)(split + 1) * g.total_ktiles / g.splits);
  const int n_st = ke - kb;

  DmaLoader<A_KMAJOR, TBM> la;
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
    __shared__ uint32_t last_flag;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      float vals[4];
      int ns[4];
      reduced(j, vals, ns);
      store_partial<4>(g, z, split, m0, j * 32, lane, ns, vals);
    }
    if (!last_of_tile(g, z * g.tiles_m + tile_m, &last_flag)) return;
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

// dst (rows of `kp` floats, 16-byte aligned) = the `n` rows of `k` floats of src (leading dimension ld),
// each followed by zeros
__global__ __launch_bounds__(kThreads) void pad_rows_kernel(const float *src, long ld, float *dst, int kp, int n, int k) {
  const int total = n * kp;
  for (int i = blockIdx.x * kThreads + threadIdx.x; i < total; i += gridDim.x * kThreads) {
    const int row = i / kp, col = i - row * kp;
    dst[i] = col < k ? src[row * ld + col] : 0.0f;
  }
}

}  // namespace

// Narrow outputs over a large streamed operand.  Sets *handled when it launched.
int gemm_f32_slab(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  if (p.N > TBN) return PHIP_OK;
  if (!rows_aligned16(p.A, 4, p.lda, p.sA, p.rA)) return PHIP_OK;
  // a k-contiguous B may have rows that are only 4-byte aligned: it is then moved by 4-byte loads
  const bool vec_b = rows_aligned16(p.B, 4, p.ldb, p.sB, p.rB);
  if (!vec_b && !p.b_kmajor) return PHIP_OK;
  // the contiguous extent of a dense operand is its leading dimension
  if ((p.a_kmajor ? p.K : p.M) != p.lda || (p.b_kmajor ? p.K : p.N) != p.ldb) return PHIP_OK;
  if (p.a_kmajor && !p.b_kmajor) return PHIP_OK;
  const long a_bytes = 4L * p.M * p.K, b_bytes = 4L * p.N * p.K;
  if (a_bytes >= (1L << 31) || b_bytes >= (1L << 31)) return PHIP_OK;
  // worth it when reading A is the cost: a large A and enough K tiles to pipeline
  const int ktiles_per_r = (p.K + LBK - 1) / LBK;
  const long total_ktiles = (long)ktiles_per_r * p.rbatch;
  const long tiles = (long)((p.M + TBM - 1) / TBM) * p.batch;
  const int cus = ctx->prop.multiProcessorCount;
  if (a_bytes * p.rbatch * p.batch < kStreamedOperandBytes || total_ktiles > 0x7fffffffL || tiles > 0x3fffffffL) return PHIP_OK;
  // two workgroups fit a compute unit: fill those places at most once (a workgroup that has to wait for
  // a place doubles the launch's duration), at least eight stages each
  long splits = 2L * cus / tiles;
  if (splits > total_ktiles / 8) splits = total_ktiles / 8;
  if (splits < 1) splits = 1;

  // A small k-contiguous B whose rows are only 4-byte aligned (a minibatch of 650-element vectors) is first
  // copied into rows padded to a multiple of four: 16-byte loads then move it, a quarter of the load
  // instructions per stage (19 against 24 us on a 10000 x 650 operand, the copy included 21).  The padding
  // is zeros and meets A rows past K, which read as zeros too.
  const float *b_ptr = static_cast<const float *>(p.B);
  long b_ld = p.ldb, b_size = b_bytes;
  bool b_vec = vec_b;
  Scratch padded(ctx);
  const int kp = (p.K + 3) / 4 * 4;
  if (!vec_b && p.batch == 1 && p.rbatch == 1 && (long)p.N * kp * 4 <= (1L << 20) &&
      scratch_alloc(ctx, sizeof(float) * (size_t)p.N * kp, &padded.ptr) == PHIP_OK) {
    const int total = p.N * kp;
    hipLaunchKernelGGL(pad_rows_kernel, dim3((unsigned)((total + kThreads - 1) / kThreads)), dim3(kThreads), 0,
                       ctx->stream, b_ptr, p.ldb, static_cast<float *>(padded.ptr), kp, p.N, p.K);
    b_ptr = static_cast<const float *>(padded.ptr);
    b_ld = kp;
    b_size = 4L * p.N * kp;
    b_vec = true;
  }

  LdsArgs d;
  GemmArgs &a = d.g;
  a = problem_args(p);
  a.B = b_ptr;
  a.ldb = b_ld;
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
  d.b_bytes = (uint32_t)b_size;

  Scratch partials(ctx);
  if (a.atomic && !p.accumulate) {
    const int rc = prepare_split_overwrite(ctx, p, tiles, (size_t)(64L << 20), &a, &partials);
    if (rc != PHIP_OK) return rc;
  }
  const long grid = tiles * splits;
#define PHIP_SLAB_G(SLOT, AK, BKM, VB)                                                              \
  do {                                                                                              \
    auto kern = gemm_f32_slab_kernel<AK, BKM, VB>;                                                  \
    const int rc = raise_lds_limit(ctx, SLOT, reinterpret_cast<const void *>(kern), kSlabLdsBytes); \
    if (rc != PHIP_OK) return rc;                                                                   \
    hipLaunchKernelGGL(kern, dim3((unsigned)grid), dim3(kThreads), kSlabLdsBytes, ctx->stream, d);  \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) {
    if (b_vec) PHIP_SLAB_G(kSlotGemmF32Slab + 0, false, true, 4);
    else PHIP_SLAB_G(kSlotGemmF32Slab + 1, false, true, 1);
  } else if (!p.a_kmajor && !p.b_kmajor) {
    PHIP_SLAB_G(kSlotGemmF32Slab + 2, false, false, 4);
  } else {
    if (b_vec) PHIP_SLAB_G(kSlotGemmF32Slab + 3, true, true, 4);
    else PHIP_SLAB_G(kSlotGemmF32Slab + 4, true, true, 1);
  }
#undef PHIP_SLAB_G
  PHIP_LAUNCH_CHECK();
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
