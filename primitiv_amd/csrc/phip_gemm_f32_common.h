// Pieces shared by the fp32 GEMM kernels: argument block, workgroup
// renumbering, the C write-out and the zero fill that precedes a split-K
// overwrite.
#ifndef PHIP_GEMM_F32_COMMON_H_
#define PHIP_GEMM_F32_COMMON_H_

#include "phip_internal.h"

namespace phip {
namespace {

typedef float float4v __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int kPad = 4;  // floats appended to every LDS row

struct GemmArgs {
  const float *A;
  const float *B;
  float *C;
  int M, N, K;
  long lda, ldb, ldc;
  long sA, sB, sC;
  long rA, rB;
  int tiles_m, tiles_n;
  int splits;        // workgroups that share one C tile, each taking a K range
  int ktiles_per_r;  // ceil(K / BK)
  int total_ktiles;  // rbatch * ktiles_per_r
  int atomic;        // split K: 1: add the tile into C with atomics; 2: leave an fp32 partial tile, the
                     // last workgroup of the output tile to finish sums the partial tiles in order
  int accumulate;    // 1: C += tile, 0: C = tile (ignored when atomic == 1)
  float *partial;    // atomic == 2: element (m, n) of (sample z, range s) at ((z*splits + s)*N + n)*M + m
  uint32_t *tickets; // atomic == 2: one zeroed counter per output tile, left zeroed
};

// The fields of the argument block that restate the problem; tile counts, K
// ranges and the split's exchange are the caller's.
inline GemmArgs problem_args(const Gemm &p) {
  GemmArgs a = {};
  a.A = static_cast<const float *>(p.A);
  a.B = static_cast<const float *>(p.B);
  a.C = static_cast<float *>(p.C);
  a.M = p.M; a.N = p.N; a.K = p.K;
  a.lda = p.lda; a.ldb = p.ldb; a.ldc = p.ldc;
  a.sA = p.sA; a.sB = p.sB; a.sC = p.sC;
  a.rA = p.rA; a.rB = p.rB;
  a.splits = 1;
  a.accumulate = p.accumulate ? 1 : 0;
  return a;
}

// Workgroups are dealt round-robin to the 8 XCDs, each with its own L2.
// Renumber them so that one XCD receives a contiguous run of tiles.
__device__ inline int xcd_remap(int bid, int total) {
  constexpr int kXcds = 8;
  const int xcd = bid % kXcds;
  const int idx = bid / kXcds;
  const int q = total / kXcds, rem = total % kXcds;
  return xcd * q + (xcd < rem ? xcd : rem) + idx;
}

// Writes NV results of one lane into C.  Result q belongs to row m and column
// ncol + nq[q], where (m, ncol) = (row0 + lane%32, col0 + 4*(lane/32)) and nq[]
// is the same for all lanes.  The old values of an accumulating write are
// fetched first, all NV loads in flight together.
//  * Interior tiles: every address is a wave-uniform base (row0, col0 + nq[q])
//    plus one per-lane 32-bit offset, no predicates.
//  * Edge tiles: per-element predicates; an element outside the matrix reads
//    the matrix origin instead and is not stored.
template <int NV>
__device__ inline void emit_c(float *Cz, long ldc, int row0, int col0, int lane, int M, int N, bool interior,
                              const int (&nq)[NV], const float (&vals)[NV], int atomic, int accumulate) {
  if (interior) {
    const unsigned voff = (unsigned)((lane & 31) + 4L * (lane >> 5) * ldc);
    float *base[NV];
#pragma unroll
    for (int q = 0; q < NV; ++q) base[q] = Cz + row0 + (long)(col0 + nq[q]) * ldc;  // uniform
    if (atomic) {
#pragma unroll
      for (int q = 0; q < NV; ++q) unsafeAtomicAdd(base[q] + voff, vals[q]);
    } else if (accumulate) {
      float old[NV];
#pragma unroll
      for (int q = 0; q < NV; ++q) old[q] = base[q][voff];
#pragma unroll
      for (int q = 0; q < NV; ++q) base[q][voff] = old[q] + vals[q];
    } else {
#pragma unroll
      for (int q = 0; q < NV; ++q) base[q][voff] = vals[q];
    }
    return;
  }
  const int m = row0 + (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
  constexpr int kChunk = NV < 4 ? NV : 4;  // few live addresses: this path is rare
#pragma unroll
  for (int c = 0; c < NV; c += kChunk) {
    bool ok[kChunk];
    float *p[kChunk];
    float old[kChunk];
#pragma unroll
    for (int q = 0; q < kChunk; ++q) {
      ok[q] = m < M && ncol + nq[c + q] < N;
      p[q] = ok[q] ? Cz + m + (long)(ncol + nq[c + q]) * ldc : Cz;
    }
    if (atomic) {
#pragma unroll
      for (int q = 0; q < kChunk; ++q)
        if (ok[q]) unsafeAtomicAdd(p[q], vals[c + q]);
    } else {
      if (accumulate) {
#pragma unroll
        for (int q = 0; q < kChunk; ++q) old[q] = *p[q];
      }
#pragma unroll
      for (int q = 0; q < kChunk; ++q)
        if (ok[q]) *p[q] = accumulate ? old[q] + vals[c + q] : vals[c + q];
    }
  }
}

// Split K without atomics on C and without a zero fill (GemmArgs::atomic == 2).
// Every workgroup of an output tile stores its NV results per lane (positions
// as for emit_c) into its range's partial tile and takes a ticket; the one
// that draws the last ticket adds the ranges in order, for the same positions,
// into `vals` and returns true: it then writes C.  Workgroups of one tile run
// on different XCDs, each with an L2 of its own, so the partial tiles are
// written and read with device-scope accesses (past the L2s) instead of being
// published by fences, which would write back a whole L2 per workgroup (38 us
// instead of 8 on a 256 x 128 product).  A workgroup's own stores have been
// acknowledged (s_waitcnt) before it takes its ticket, and the ticket is a
// device-scope atomic, so whoever draws the last one finds every partial tile.
template <int NV>
__device__ inline void store_partial(const GemmArgs &g, int z, int split, int row0, int col0, int lane,
                                     const int (&nq)[NV], const float (&vals)[NV]) {
  float *P = g.partial + ((long)z * g.splits + split) * g.M * g.N;
  const int m = row0 + (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
#pragma unroll
  for (int q = 0; q < NV; ++q) {
    const int n = ncol + nq[q];
    if (m < g.M && n < g.N)
      __hip_atomic_store(P + m + (long)n * g.M, vals[q], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
}

template <int NV>
__device__ inline void sum_partials(const GemmArgs &g, int z, int row0, int col0, int lane, const int (&nq)[NV],
                                    float (&vals)[NV]) {
  const float *P = g.partial + (long)z * g.splits * g.M * g.N;
  const long per = (long)g.M * g.N;
  const int m = row0 + (lane & 31);
  const int ncol = col0 + 4 * (lane >> 5);
  const float *p[NV];
  bool ok[NV];
#pragma unroll
  for (int q = 0; q < NV; ++q) {
    const int n = ncol + nq[q];
    ok[q] = m < g.M && n < g.N;
    p[q] = ok[q] ? P + m + (long)n * g.M : P;
    vals[q] = 0.0f;
  }
  // eight ranges at a time: the loads of a batch are all in flight before the first is added
  for (int r0 = 0; r0 < g.splits; r0 += 8) {
    float part[8][NV];
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int q = 0; q < NV; ++q)
        part[u][q] = __hip_atomic_load(p[q] + (r0 + u < g.splits ? r0 + u : r0) * per, __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
#pragma unroll
    for (int u = 0; u < 8; ++u)
#pragma unroll
      for (int q = 0; q < NV; ++q)
        if (r0 + u < g.splits) vals[q] += part[u][q];
  }
#pragma unroll
  for (int q = 0; q < NV; ++q) vals[q] = ok[q] ? vals[q] : 0.0f;
}

// Called by all threads of the workgroup after their store_partial calls.
// Ordering, spelled out (the exchange deliberately uses no agent-scope release /
// acquire fences, which on this part write back and invalidate a whole L2):
//  * the partial tiles are written and read by agent-scope atomic accesses, which
//    bypass the per-XCD L2s, so no cache can hold a stale copy of them;
//  * s_waitcnt vmcnt(0) holds every lane until its own such stores are acknowledged
//    by memory, and its "memory" clobber keeps the compiler from moving them below;
//  * __syncthreads() (a workgroup-scope release / acquire fence and a barrier) puts
//    all lanes' acknowledged stores before thread 0's ticket, and, after the second
//    barrier, keeps the loads of sum_partials from being moved above the ticket;
//  * the ticket is an agent-scope atomic on one address: whoever draws the last one
//    does so after every other workgroup's stores were acknowledged.
__device__ inline bool last_of_tile(const GemmArgs &g, int tile_id, uint32_t *flag) {
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own partial results have arrived, before the ticket
  __syncthreads();
  if (threadIdx.x == 0) {
    const uint32_t ticket = __hip_atomic_fetch_add(g.tickets + tile_id, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const bool last = ticket == (uint32_t)g.splits - 1u;
    // nobody else touches this counter any more in this launch: leave it zeroed for the next one
    if (last) __hip_atomic_store(g.tickets + tile_id, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *flag = last ? 1u : 0u;
  }
  __syncthreads();
  return *flag != 0;
}

__attribute__((unused)) __global__ __launch_bounds__(kThreads) void zero_c_kernel(float *C, int M, int N, long ldc, long sC, int batch) {
  const long per = (long)M * N;
  const long total = per * batch;
  for (long i = (long)blockIdx.x * kThreads + threadIdx.x; i < total; i += (long)gridDim.x * kThreads) {
    const long z = i / per, e = i - z * per;
    C[z * sC + (e % M) + (e / M) * ldc] = 0.0f;
  }
}

// Pool memory that goes back when the launches that use it have been enqueued
// (the stream is in order, so the block may be handed out again behind them).
struct Scratch {
  phip_ctx *ctx;
  void *ptr = nullptr;
  explicit Scratch(phip_ctx *c) : ctx(c) {}
  ~Scratch() {
    if (ptr) scratch_free(ctx, ptr);
  }
  Scratch(const Scratch &) = delete;
  Scratch &operator=(const Scratch &) = delete;
};

inline int zero_c(phip_ctx *ctx, const Gemm &p) {
  const int cus = ctx->prop.multiProcessorCount;
  const long total = (long)p.M * p.N * p.batch;
  long blocks = (total + kThreads * 4 - 1) / (kThreads * 4);
  if (blocks > cus * 8L) blocks = cus * 8L;
  hipLaunchKernelGGL(zero_c_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, ctx->stream, static_cast<float *>(p.C),
                     p.M, p.N, p.ldc, p.sC, p.batch);
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "zero_c");
  return PHIP_OK;
}

// True when a product whose K is split between workgroups has to meet through partial tiles: an
// overwriting one always (no zero fill, no atomics on C), an accumulating one when the context asks
// for results that are the same bits on every run.
inline bool wants_exchange(const phip_ctx *ctx, const Gemm &p) { return !p.accumulate || ctx->deterministic; }

// A product whose K is split between `a->splits` workgroups per tile (a->atomic == 1 on entry): fp32
// partial tiles in scratch memory, summed in order by the last workgroup of each tile, which then
// writes (or adds to) C once (a->atomic = 2: one launch, the same bits on every run).  Without room
// for them, or with more tiles than tickets: atomics on C, behind a zero fill for an overwriting
// product.  An allocation-free call keeps the exchange or fails.
inline int prepare_split_exchange(phip_ctx *ctx, const Gemm &p, long tiles, size_t max_bytes, GemmArgs *a,
                                  Scratch *partials) {
  const size_t bytes = sizeof(float) * (size_t)p.M * p.N * p.batch * a->splits;
  if (ctx->fixed_mode) {
    if (tiles > kTicketSlots) return fail(PHIP_ERR_INVALID_ARGUMENT, "%ld output tiles exceed the %d tile counters of an allocation-free call", tiles, kTicketSlots);
    const int rc = scratch_alloc(ctx, bytes, &partials->ptr);
    if (rc != PHIP_OK) return rc;
  } else if (!(tiles <= kTicketSlots && bytes <= max_bytes && scratch_alloc(ctx, bytes, &partials->ptr) == PHIP_OK)) {
    partials->ptr = nullptr;
    return p.accumulate ? PHIP_OK : zero_c(ctx, p);
  }
  a->atomic = 2;
  a->partial = static_cast<float *>(partials->ptr);
  a->tickets = tile_tickets(ctx);
  return PHIP_OK;
}

}  // namespace
}  // namespace phip

#endif  // PHIP_GEMM_F32_COMMON_H_
