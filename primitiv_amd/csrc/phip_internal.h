// Internal declarations shared by the translation units of libphip.
#ifndef PHIP_INTERNAL_H_
#define PHIP_INTERNAL_H_

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "../../include/phip.h"

namespace phip {

// Records the calling thread's error message and returns `code`.
int fail(int code, const char *fmt, ...) __attribute__((format(printf, 2, 3)));

// Power-of-two bucketed device memory pool (one per context).
struct Pool {
  std::vector<std::vector<void *>> reserved{64};
  std::unordered_map<void *, unsigned> supplied;
  static constexpr size_t kMinimumSize = 2 * sizeof(float);
};

// Two lanes for matrix products (phip_lanes.hip).  In a long enough run of matmul calls, calls that
// do not touch each other's operands run on two streams at once: the context's own (the main lane,
// which also carries every other operation) and that of a second, private context (the side lane,
// with its own scratch pool and tile counters, so that launches on the two lanes share nothing).
// What the caller observes is the order of its calls.
struct MemRange {
  uintptr_t lo, hi;
  bool write;
};
// A zero fill that has been asked for and not launched (phip_elementwise.hip): primitiv's backward
// pass gives every gradient a zero-filled tensor and then lets an operator add into it, which for
// the small per-timestep tensors of a recurrent network is two launches where one that writes
// instead of adding does the same.  A zero fill is only noted; the next entry point either takes
// the note for an output that it would add into (and overwrites instead: same bits, 0 + v), or
// launches the fill first.  Notes never outlive the next entry point that enqueues work.
struct PendingZero {
  uintptr_t lo;
  size_t bytes;
  int elem;  // 0: float, 1: f16, 2: bf16 (which fill kernel to launch)
};

struct Lanes {
  phip_ctx *side = nullptr;
  bool enabled = true;
  hipEvent_t main_tail = nullptr, side_tail = nullptr;
  // operands of the products enqueued on a lane and not yet ordered before the other lane
  std::vector<MemRange> main_ops, side_ops;
  bool engaged = false;    // the side lane is in use
  int streak = 0;          // matmul calls since the last operation of another kind
  int since_engaged = 0;   // of which since the lanes were engaged
  int engage_after = 0;    // length of the run that engages the lanes (grows when engaging did not pay)
  int engage_after_base = 0;
  bool back_off = true;
  int last_lane = 0;       // lane of the latest product
};

}  // namespace phip

struct phip_ctx {
  int device = -1;
  uint64_t id = 0;
  hipStream_t stream = nullptr;
  hipDeviceProp_t prop;
  phip::Pool pool;
  // Scratch of the matrix products (partial tiles of a split product, a transposed operand): blocks
  // that no caller ever sees.  A block freed when its launches have been enqueued may be handed out
  // again at once only to a launch on the same stream; a caller's tensor from `pool` can be written
  // by a product on the other lane, so the two kinds of block never trade places.
  phip::Pool scratch_pool;
  std::mutex mutex;  // guards `pool` and `scratch_pool`
  // Kernels whose dynamic-LDS limit has been raised on this context's device
  // (one bit per kernel, see phip::raise_lds_limit).
  uint64_t lds_limit_raised = 0;
  // One counter per output tile of a launch whose workgroups share tiles (see
  // phip::kTicketSlots); all zero between launches.
  uint32_t *tile_tickets = nullptr;
  // Allocation-free calls (phip_matmul_fw_f32_noalloc): this device's copy of the
  // library's fixed scratch array, how much of it the running call has handed out,
  // and whether such a call is running (scratch then comes from there, see
  // phip::scratch_alloc).
  // Products whose K range is split between workgroups add their tiles to an accumulated output
  // with fp32 atomics (any order) unless this is set (phip_set_deterministic).
  bool deterministic = false;
  unsigned char *fixed_scratch = nullptr;
  size_t fixed_used = 0;
  bool fixed_mode = false;
  // The second lane for matrix products; null in the side lane's own context.
  phip::Lanes *lanes = nullptr;
  // Names of the matrix-product kernels launched on this context since the last phip_gemm_trace call,
  // kept only while tracing is switched on (benchmarks and tests ask which kernel a shape went to).
  bool trace_on = false;
  std::string trace;
  // Zero fills noted and not yet launched (see phip::PendingZero); `defer_zero_fills` off: every fill launches.
  // Guarded by `mutex` (a handle deleter on another thread drops the notes of the block it returns);
  // zeros_count mirrors zeros.size() so that entry points can skip the lock when there is nothing.
  std::vector<phip::PendingZero> zeros;
  std::atomic<int> zeros_count{0};
  bool defer_zero_fills = true;
};

struct phip_event {
  hipEvent_t ev = nullptr;
  int device = -1;
};

#define PHIP_HIP(expr)                                                        \
  do {                                                                        \
    hipError_t phip_err__ = (expr);                                           \
    if (phip_err__ != hipSuccess) {                                           \
      return phip::fail(phip_err__ == hipErrorOutOfMemory                     \
                            ? PHIP_ERR_OUT_OF_MEMORY                          \
                            : PHIP_ERR_RUNTIME,                               \
                        "%s failed: %s (%s:%d)", #expr,                       \
                        hipGetErrorString(phip_err__), __FILE__, __LINE__);   \
    }                                                                         \
  } while (0)

#define PHIP_REQUIRE(cond, ...)                                               \
  do {                                                                        \
    if (!(cond)) return phip::fail(PHIP_ERR_INVALID_ARGUMENT, __VA_ARGS__);   \
  } while (0)

// Makes the context's device current and checks the context pointer: for entry points that enqueue
// nothing (memory pool, queries) and for the matrix products, which place themselves on a lane.
#define PHIP_ENTER_HOST(ctx)                                                  \
  PHIP_REQUIRE((ctx) != nullptr, "null context");                             \
  PHIP_HIP(hipSetDevice((ctx)->device))

// Launches the zero fills that were noted and not taken (no-op when there are none).
#define PHIP_FLUSH_ZEROS(ctx)                                                 \
  do {                                                                        \
    if ((ctx)->zeros_count.load(std::memory_order_relaxed) != 0) {            \
      const int phip_zero_rc__ = phip::zeros_flush(ctx);                      \
      if (phip_zero_rc__ != PHIP_OK) return phip_zero_rc__;                   \
    }                                                                         \
  } while (0)

// For the entry points that may take a noted zero fill for an output they add into: as PHIP_ENTER
// but the notes stay; the entry point calls zeros_take for such outputs and then PHIP_FLUSH_ZEROS.
#define PHIP_ENTER_KEEP_ZEROS(ctx)                                            \
  PHIP_ENTER_HOST(ctx);                                                       \
  do {                                                                        \
    if ((ctx)->lanes != nullptr) {                                            \
      const int phip_join_rc__ = phip::lanes_join(ctx);                       \
      if (phip_join_rc__ != PHIP_OK) return phip_join_rc__;                   \
    }                                                                         \
  } while (0)

// The same for every entry point that enqueues work on the context's stream or waits for it: noted
// zero fills are launched, then the stream waits for the matrix products that run on the side lane.
#define PHIP_ENTER(ctx)                                                       \
  PHIP_ENTER_HOST(ctx);                                                       \
  PHIP_FLUSH_ZEROS(ctx);                                                      \
  do {                                                                        \
    if ((ctx)->lanes != nullptr) {                                            \
      const int phip_join_rc__ = phip::lanes_join(ctx);                       \
      if (phip_join_rc__ != PHIP_OK) return phip_join_rc__;                   \
    }                                                                         \
  } while (0)

// For entry points that end with the host waiting for the context's stream (phip_sync, copies from
// and to host memory): the host waits for the side lane as well, which costs no wait of one stream
// for the other and leaves the lanes as they are.
#define PHIP_ENTER_BLOCKING(ctx)                                              \
  PHIP_ENTER_HOST(ctx);                                                       \
  PHIP_FLUSH_ZEROS(ctx);                                                      \
  do {                                                                        \
    if ((ctx)->lanes != nullptr) {                                            \
      const int phip_join_rc__ = phip::lanes_wait_host(ctx);                  \
      if (phip_join_rc__ != PHIP_OK) return phip_join_rc__;                   \
    }                                                                         \
  } while (0)

// Checks the status of the launch that was just enqueued.
#define PHIP_LAUNCH_CHECK() PHIP_HIP(hipGetLastError())

namespace phip {

// Noted zero fills (phip_elementwise.hip).  zeros_flush launches them all, in the order they were
// asked for.  zeros_take: true when exactly [p, p + bytes) is noted as zero; the note is removed and
// the caller writes the range instead of adding into it.  zeros_drop forgets the notes inside a range
// whose contents no longer matter (a block handed back to the pool).
int zeros_flush(phip_ctx *ctx);
bool zeros_take(phip_ctx *ctx, const void *p, size_t bytes);
// True when [p, p + bytes) and [q, q + qbytes) share memory (q may be null).  An output that is also
// read as an operand must see its fill before the operation, so its note is not taken.
inline bool shares_memory(const void *p, size_t bytes, const void *q, size_t qbytes) {
  const uintptr_t a = reinterpret_cast<uintptr_t>(p), b = reinterpret_cast<uintptr_t>(q);
  return q != nullptr && a < b + qbytes && b < a + bytes;
}
void zeros_drop(phip_ctx *ctx, const void *p, size_t bytes);

// phip_lanes.hip.  lanes_join: the main lane waits for everything on the side lane (no-op when
// nothing is in flight there).  lanes_place: picks the lane of a matrix product with the given
// operand ranges, enqueues the waits it needs and returns the context to launch it on.
// A context with (what phip_ctx_create gives) or without a side lane of its own (phip_runtime.hip).
int ctx_create(int device_id, bool with_lanes, phip_ctx **out);
int lanes_create(phip_ctx *ctx);
int lanes_destroy(phip_ctx *ctx);
int lanes_join(phip_ctx *ctx);
// The host waits for the products in flight on both lanes; the lanes stay engaged.
int lanes_wait_host(phip_ctx *ctx);
// What is enqueued on the main lane next comes after the side lane's work, and touches no tensor (an event).
int lanes_order_main_after_side(phip_ctx *ctx);
int lanes_place(phip_ctx *ctx, const MemRange *ranges, int n, bool may_overlap, phip_ctx **run_on);

// Notes that a matrix product went to the kernel `name` (phip_gemm_trace).
inline void note_kernel(phip_ctx *ctx, const char *name) {
  if (!ctx->trace_on || ctx->trace.size() > 4000) return;
  if (!ctx->trace.empty()) ctx->trace += ' ';
  ctx->trace += name;
}

// Entries of phip_ctx::tile_tickets.
constexpr int kTicketSlots = 65536;

// Scratch memory of a matrix product (partial tiles of a split product, a transposed
// operand): a block of the context's private scratch pool, or, during an
// allocation-free call, a piece of the device's fixed scratch array (no allocation;
// fails with a message when the call needs more than kFixedScratchBytes in total).
// scratch_free returns a block to the scratch pool; the stream is in order, so the
// block may be reused behind the launches that read it.  tile_tickets gives the
// zeroed per-tile counters that go with it.
constexpr size_t kFixedScratchBytes = 16u << 20;
int scratch_alloc(phip_ctx *ctx, size_t bytes, void **out);
void scratch_free(phip_ctx *ctx, void *ptr);
uint32_t *tile_tickets(phip_ctx *ctx);

// Bits of phip_ctx::lds_limit_raised: first slot of each kernel family that
// asks for a dynamic LDS size (one slot per instantiation, counted from here).
enum LdsSlot {
  kSlotGemmF32Lds = 0,    // 6 instantiations
  kSlotGemmH16Big = 8,    // 6
  kSlotGemmF32Slab = 16,  // 3
  kSlotGemmF32RankK = 21, // 1
  kSlotGemmF32StreamPair = 22,  // 1
  kSlotGemmH16Mid = 23,   // 6
  kSlotGemmH16Skinny = 29,  // 8
  kSlotGemmF32LdsMixed = 37,  // 3
  kSlotGemmF32Lds64w = 40,    // 3
  kSlotGemmH16MidDeep = 43,   // 6
};

// Allows `kernel` to use `bytes` of dynamic LDS (above the 64 KiB default) on
// the context's device; done once per context and kernel (`slot` < 64).
inline int raise_lds_limit(phip_ctx *ctx, int slot, const void *kernel, int bytes) {
  if (ctx->lds_limit_raised & (1ull << slot)) return PHIP_OK;
  PHIP_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes));
  ctx->lds_limit_raised |= 1ull << slot;
  return PHIP_OK;
}

// ---- GEMM layer (phip_gemm_*.hip) ------------------------------------------
//
// One problem:  C[z] (M x N, column-major, ldc)  (=|+=)
//                 sum_{r < rbatch} opA[z][r] (M x K) . opB[z][r] (K x N)
// for z < batch.  Operand element (m, k) of opA lives at
//   A + z*sA + r*rA + (a_kmajor ? k + m*lda : m + k*lda)
// and element (k, n) of opB at
//   B + z*sB + r*rB + (b_kmajor ? k + n*ldb : n + k*ldb).
// Strides are in elements and may be 0.
struct Gemm {
  int M = 0, N = 0, K = 0;
  const void *A = nullptr;
  const void *B = nullptr;
  void *C = nullptr;
  long lda = 0, ldb = 0, ldc = 0;
  long sA = 0, sB = 0, sC = 0;  // per-z strides
  long rA = 0, rB = 0;          // per-r strides (reduction over samples)
  int batch = 1;
  int rbatch = 1;
  bool a_kmajor = false;  // false: M-contiguous, true: K-contiguous
  bool b_kmajor = true;   // true: K-contiguous, false: N-contiguous
  bool accumulate = false;
};

enum class Elem { F32, F16, BF16 };

// True when an operand can be moved 16 bytes at a time: its base is 16-byte
// aligned and its leading dimension and strides are multiples of `per16`
// elements (4 for fp32, 8 for 16-bit storage).
inline bool rows_aligned16(const void *ptr, int per16, long ld, long s = 0, long r = 0) {
  return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && ld % per16 == 0 && s % per16 == 0 && r % per16 == 0;
}

int gemm_f32(phip_ctx *ctx, const Gemm &g);
int gemm_f32_direct(phip_ctx *ctx, const Gemm &g, bool *handled);
int gemm_f32_tile16(phip_ctx *ctx, const Gemm &g, bool *handled);
int gemm_f32_lds(phip_ctx *ctx, const Gemm &g, bool *handled);
int gemm_f32_slab(phip_ctx *ctx, const Gemm &g, bool *handled);
int gemm_f32_rankk(phip_ctx *ctx, const Gemm &g, bool *handled);
// Two independent accumulating products (outputs do not overlap) in one launch,
// for problems so small that a launch is mostly its fixed latency.  Sets
// *handled when it launched both; otherwise nothing has been done.
int gemm_f32_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, bool *handled);
// The same for a rank-K update of a large matrix beside a product that streams a large operand
// (the gradients of an output projection): one grid, all of it resident at once.
int gemm_f32_stream_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, bool *handled);
// An operand of at least this many bytes, read once against few output columns,
// is worth the streaming kernel (gemm_f32_slab).
constexpr long kStreamedOperandBytes = 8L << 20;
int gemm_h16(phip_ctx *ctx, const Gemm &g, Elem elem);
int gemm_h16_big(phip_ctx *ctx, const Gemm &g, Elem elem, bool *handled);
// 16-bit products with a narrow side or a short K (per-timestep shapes); the pair: both gradient products
// of one matmul_bw call in one launch.
int gemm_h16_skinny(phip_ctx *ctx, const Gemm &g, Elem elem, bool *handled);
int gemm_h16_skinny_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, Elem elem, bool *handled);

}  // namespace phip

#endif  // PHIP_INTERNAL_H_
