// primitiv's matmul forward / backward expressed as GEMM problems.
//
// a: [di x dj] x ba, b: [dj x dk] x bb, y: [di x dk] x max(ba, bb), all dense
// column-major with the minibatch outermost.  Four batch cases:
//
//   ba == 1 (b shared or not): the minibatch of b is folded into its columns,
//       so forward, gA and gB are ONE product each with n or k = dk*bb.  For
//       gA the contraction index runs over (column, sample): the reduction of
//       the shared operand's gradient over the minibatch is the K loop.
//   ba == bb > 1: one product per sample (grid z).
//   ba > 1, bb == 1: per-sample products with b's stride 0; gB has a single
//       [dj x dk] output whose K loop walks (sample, row), so the reduction
//       over the minibatch again happens inside the kernel.
#include "phip_internal.h"

namespace phip {

static int check_matmul_args(const void *a, const void *b, const void *c, uint32_t di, uint32_t dj,
                             uint32_t dk, uint32_t ba, uint32_t bb) {
  PHIP_REQUIRE(a != nullptr && b != nullptr && c != nullptr, "null tensor pointer");
  PHIP_REQUIRE(di >= 1 && dj >= 1 && dk >= 1, "matrix dimensions must be positive");
  PHIP_REQUIRE(ba >= 1 && bb >= 1 && (ba == bb || ba == 1 || bb == 1),
               "Invalid shapes to calculate the matrix product: batch sizes %u and %u", ba, bb);
  const uint64_t bs = ba > bb ? ba : bb;
  const uint64_t lim = 0x7fffffffull;
  PHIP_REQUIRE((uint64_t)dk * bs <= lim && (uint64_t)di <= lim && (uint64_t)dj <= lim,
               "matrix dimension exceeds 2^31-1");
  return PHIP_OK;
}

typedef int (*gemm_fn)(phip_ctx *, const Gemm &, Elem);

static int gemm_dispatch(phip_ctx *ctx, const Gemm &g, Elem elem) {
  return elem == Elem::F32 ? gemm_f32(ctx, g) : gemm_h16(ctx, g, elem);
}

// Products of up to this many floating-point operations may run beside another product on the
// context's second lane (phip_lanes.hip); a larger one occupies every compute unit for several
// rounds of workgroups and gains nothing from company.
constexpr double kMaxOverlapFlop = 4e9;

static MemRange range_of(const void *p, uint64_t elements, Elem elem, bool write) {
  const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
  return MemRange{lo, lo + (uintptr_t)(elements * (elem == Elem::F32 ? 4 : 2)), write};
}

// The context (lane) this call's launches go to.
static int place(phip_ctx *ctx, Elem elem, const MemRange *ranges, int n, uint32_t di, uint32_t dj, uint32_t dk,
                 uint32_t ba, uint32_t bb, phip_ctx **run_on) {
  const double flop = 2.0 * di * dj * dk * (ba > bb ? ba : bb);
  (void)elem;
  const bool may_overlap = !ctx->fixed_mode && flop <= kMaxOverlapFlop;
  return lanes_place(ctx, ranges, n, may_overlap, run_on);
}

static int matmul_fw(phip_ctx *ctx, Elem elem, const void *a, const void *b, void *y, uint32_t di,
                     uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  PHIP_ENTER_HOST(ctx);
  PHIP_FLUSH_ZEROS(ctx);
  int rc = check_matmul_args(a, b, y, di, dj, dk, ba, bb);
  if (rc != PHIP_OK) return rc;
  {
    const uint64_t bs = ba > bb ? ba : bb;
    const MemRange ranges[3] = {range_of(a, (uint64_t)di * dj * ba, elem, false), range_of(b, (uint64_t)dj * dk * bb, elem, false),
                                range_of(y, (uint64_t)di * dk * bs, elem, true)};
    rc = place(ctx, elem, ranges, 3, di, dj, dk, ba, bb, &ctx);
    if (rc != PHIP_OK) return rc;
  }
  Gemm g;
  g.A = a; g.B = b; g.C = y;
  g.lda = di; g.ldb = dj; g.ldc = di;
  g.a_kmajor = false;  // a(m, k) at m + k*di
  g.b_kmajor = true;   // b(k, n) at k + n*dj
  g.accumulate = false;
  g.M = di; g.K = dj;
  if (ba > 1) {
    g.N = dk;
    g.batch = ba;
    g.sA = (long)di * dj;
    g.sB = bb > 1 ? (long)dj * dk : 0;
    g.sC = (long)di * dk;
  } else {
    g.N = (int)(dk * bb);
    g.batch = 1;
  }
  // 16-bit storage, one large a against many columns: the large-tile kernel runs
  // at the power limit there, and its K loop settles at a clock a sixth higher
  // when both operands are contiguous along k (16-byte LDS reads) than when a
  // is transposed by the LDS reads (1.49 against 1.28 GHz, fp16, counted in the
  // kernel).  A transposed copy of a costs one pass over it; from 16 Ki columns
  // on that is less than what the product gains.
  if (elem != Elem::F32 && ba == 1 && di >= 1024 && dj >= 1024 && di % 8 == 0 && dj % 8 == 0 &&
      (long)dk * bb >= 16384 && (long)di * dj * 2 < (1L << 31)) {
    struct Block {  // back to the scratch pool on every way out; the stream orders its reuse
      phip_ctx *ctx;
      void *ptr;
      ~Block() {
        if (ptr) scratch_free(ctx, ptr);
      }
    } at{ctx, nullptr};
    rc = scratch_alloc(ctx, (size_t)di * dj * 2, &at.ptr);
    if (rc != PHIP_OK) return rc;
    rc = elem == Elem::F16 ? phip_transpose_fw_f16(ctx, a, at.ptr, di, dj, 1)
                           : phip_transpose_fw_bf16(ctx, a, at.ptr, di, dj, 1);
    if (rc != PHIP_OK) return rc;
    note_kernel(ctx, "transposed_copy");
    g.A = at.ptr;      // a^T: element (m, k) at k + m*dj
    g.lda = dj;
    g.a_kmajor = true;
    return gemm_dispatch(ctx, g, elem);
  }
  return gemm_dispatch(ctx, g, elem);
}

static int matmul_bw(phip_ctx *ctx, Elem elem, const void *a, const void *b, const void *gy, void *ga,
                     void *gb, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  PHIP_ENTER_HOST(ctx);
  PHIP_FLUSH_ZEROS(ctx);
  int rc = check_matmul_args(a, b, gy, di, dj, dk, ba, bb);
  if (rc != PHIP_OK) return rc;
  PHIP_REQUIRE(ga != nullptr && gb != nullptr, "null gradient pointer");
  {
    const uint64_t bs = ba > bb ? ba : bb;
    const MemRange ranges[5] = {range_of(a, (uint64_t)di * dj * ba, elem, false), range_of(b, (uint64_t)dj * dk * bb, elem, false),
                                range_of(gy, (uint64_t)di * dk * bs, elem, false), range_of(ga, (uint64_t)di * dj * ba, elem, true),
                                range_of(gb, (uint64_t)dj * dk * bb, elem, true)};
    rc = place(ctx, elem, ranges, 5, di, dj, dk, ba, bb, &ctx);
    if (rc != PHIP_OK) return rc;
  }

  // ga[di x dj] += gy[di x dk] . b^T : A = gy (m-contiguous), B = b^T with
  // element (k, n) at n + k*dj (n-contiguous).
  Gemm p;
  p.A = gy; p.B = b; p.C = ga;
  p.lda = di; p.ldb = dj; p.ldc = di;
  p.a_kmajor = false;
  p.b_kmajor = false;
  p.accumulate = true;
  p.M = di; p.N = dj;
  if (ba > 1) {
    p.K = dk;
    p.batch = ba;
    p.sA = (long)di * dk;
    p.sB = bb > 1 ? (long)dj * dk : 0;
    p.sC = (long)di * dj;
  } else {
    p.K = (int)(dk * bb);  // contraction over (column, sample)
    p.batch = 1;
  }

  // gb[dj x dk] += a^T . gy : A = a^T with element (m, k) at k + m*di, B = gy
  // with element (k, n) at k + n*di (both k-contiguous).
  Gemm q;
  q.A = a; q.B = gy; q.C = gb;
  q.lda = di; q.ldb = di; q.ldc = dj;
  q.a_kmajor = true;
  q.b_kmajor = true;
  q.accumulate = true;
  q.M = dj; q.K = di;
  if (ba > 1 && bb > 1) {
    q.N = dk;
    q.batch = ba;
    q.sA = (long)di * dj;
    q.sB = (long)di * dk;
    q.sC = (long)dj * dk;
  } else if (ba > 1) {
    // b is shared: one output, contraction over (sample, row).
    q.N = dk;
    q.batch = 1;
    q.rbatch = ba;
    q.rA = (long)di * dj;
    q.rB = (long)di * dk;
  } else {
    q.N = (int)(dk * bb);
    q.batch = 1;
  }

  // Small products whose outputs do not overlap share one launch.
  if (elem == Elem::F32) {
    const char *ga0 = static_cast<const char *>(ga), *gb0 = static_cast<const char *>(gb);
    const size_t ga_bytes = sizeof(float) * (size_t)di * dj * ba, gb_bytes = sizeof(float) * (size_t)dj * dk * bb;
    if (ga0 + ga_bytes <= gb0 || gb0 + gb_bytes <= ga0) {
      bool handled = false;
      rc = gemm_f32_pair(ctx, p, q, &handled);
      if (rc != PHIP_OK || handled) return rc;
      rc = gemm_f32_stream_pair(ctx, p, q, &handled);
      if (rc != PHIP_OK || handled) return rc;
    }
  }
  if (elem != Elem::F32) {
    const char *ga0 = static_cast<const char *>(ga), *gb0 = static_cast<const char *>(gb);
    const size_t ga_bytes = 2 * (size_t)di * dj * ba, gb_bytes = 2 * (size_t)dj * dk * bb;
    if (ga0 + ga_bytes <= gb0 || gb0 + gb_bytes <= ga0) {
      bool handled = false;
      rc = gemm_h16_skinny_pair(ctx, p, q, elem, &handled);
      if (rc != PHIP_OK || handled) return rc;
    }
  }
  rc = gemm_dispatch(ctx, p, elem);
  if (rc != PHIP_OK) return rc;
  return gemm_dispatch(ctx, q, elem);
}

}  // namespace phip

using namespace phip;

extern "C" {

int phip_matmul_fw_f32(phip_ctx *ctx, const float *a, const float *b, float *y, uint32_t di, uint32_t dj,
                       uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_fw(ctx, Elem::F32, a, b, y, di, dj, dk, ba, bb);
}
int phip_matmul_fw_f16(phip_ctx *ctx, const void *a, const void *b, void *y, uint32_t di, uint32_t dj,
                       uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_fw(ctx, Elem::F16, a, b, y, di, dj, dk, ba, bb);
}
int phip_matmul_fw_bf16(phip_ctx *ctx, const void *a, const void *b, void *y, uint32_t di, uint32_t dj,
                        uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_fw(ctx, Elem::BF16, a, b, y, di, dj, dk, ba, bb);
}

int phip_matmul_fw_f32_noalloc(phip_ctx *ctx, const float *a, const float *b, float *y, uint32_t di,
                               uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  PHIP_REQUIRE(ctx->fixed_scratch != nullptr, "device %d has no fixed scratch array", ctx->device);
  // every piece of scratch memory that the launchers ask for now comes out of the fixed array
  struct Mode {
    phip_ctx *ctx;
    explicit Mode(phip_ctx *c) : ctx(c) { ctx->fixed_mode = true; ctx->fixed_used = 0; }
    ~Mode() { ctx->fixed_mode = false; }
  } mode(ctx);
  return matmul_fw(ctx, Elem::F32, a, b, y, di, dj, dk, ba, bb);
}

int phip_gemm_trace(phip_ctx *ctx, int on, char *buf, size_t buf_size) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  phip_ctx *side = ctx->lanes != nullptr ? ctx->lanes->side : nullptr;
  if (buf != nullptr && buf_size > 0) {
    std::string all = ctx->trace;
    if (side != nullptr && !side->trace.empty()) all += (all.empty() ? "" : " ") + side->trace;
    std::snprintf(buf, buf_size, "%s", all.c_str());
  }
  ctx->trace.clear();
  ctx->trace_on = on != 0;
  if (side != nullptr) {
    side->trace.clear();
    side->trace_on = on != 0;
  }
  return PHIP_OK;
}

int phip_matmul_bw_f32(phip_ctx *ctx, const float *a, const float *b, const float *gy, float *ga,
                       float *gb, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_bw(ctx, Elem::F32, a, b, gy, ga, gb, di, dj, dk, ba, bb);
}
int phip_matmul_bw_f16(phip_ctx *ctx, const void *a, const void *b, const void *gy, void *ga, void *gb,
                       uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_bw(ctx, Elem::F16, a, b, gy, ga, gb, di, dj, dk, ba, bb);
}
int phip_matmul_bw_bf16(phip_ctx *ctx, const void *a, const void *b, const void *gy, void *ga, void *gb,
                        uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_bw(ctx, Elem::BF16, a, b, gy, ga, gb, di, dj, dk, ba, bb);
}

}  // extern "C"
