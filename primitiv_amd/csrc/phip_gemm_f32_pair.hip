// The two gradient products of a small matmul in ONE launch.
//
// ga += gy.b^T and gb += a^T.gy are independent when their outputs do not
// overlap, and on the per-timestep shapes of recurrent graphs each of them is a
// launch of a few microseconds that is mostly fixed latency (dispatch, the
// first round of loads, the write-out).  One grid carries both: workgroups
// below `first_blocks` work on the first problem, the others on the second,
// each running the code of the kernel that a launch of its own would have used:
//  * first (both operands contiguous along m / n): the direct-from-global
//    kernel, or - a rank-K update of a matrix of at least one 64 x 64 tile per
//    CU - the LDS-staged kernel with 64 x 64 x 32 tiles;
//  * second (both operands contiguous along k): the direct-from-global kernel.
#include "phip_gemm_f32_direct.h"
#include "phip_gemm_f32_staged.h"

namespace phip {
namespace {

// FIRST: 4 or 8 = chunks in flight of the direct kernel, or the staged 64 x 64 tiles with B moved 16 or
// (rows not 16-byte aligned: a hidden size such as 650) 4 bytes at a time
constexpr int kStaged = 64, kStagedB1 = 65;

template <int FIRST>
constexpr int pair_lds_floats() {
  constexpr int direct = kDirectRedFloats<1, 1, 4>;
  constexpr int staged = FIRST >= kStaged ? staged_lds_floats<64, 64, 32, 2, 2, 1>() : 0;
  return direct > staged ? direct : staged;
}

template <int FIRST, int U2>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_pair_kernel(const DirectArgs first, const DirectArgs second,
                                                                     int first_blocks, int first_padded) {
  __shared__ __attribute__((aligned(16))) float lds[pair_lds_floats<FIRST>()];
  __shared__ uint32_t last_flag;
  const int bid = blockIdx.x;
  if (bid < first_blocks) {
    if constexpr (FIRST == kStaged) staged_tile<64, 64, 32, 2, 2, 1, false, false, 4, 4>(first.g, lds, bid, first_blocks);
    else if constexpr (FIRST == kStagedB1) staged_tile<64, 64, 32, 2, 2, 1, false, false, 4, 1>(first.g, lds, bid, first_blocks);
    else direct_tile<1, 1, FIRST, false, false, 1, 1, 4>(first, lds, &last_flag, bid, first_blocks);
  } else if (bid >= first_padded) {
    // the second problem starts at a multiple of 8 so that its workgroups meet the XCDs in the same order
    direct_tile<1, 1, U2, true, true, 4, 4, 4>(second, lds, &last_flag, bid - first_padded,
                                               (int)gridDim.x - first_padded);
  }
}

}  // namespace

int gemm_f32_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, bool *handled) {
  *handled = false;
  if (!first.accumulate || !second.accumulate) return PHIP_OK;
  // the shared launch adds the tiles of a split product with atomics
  if (ctx->deterministic) return PHIP_OK;
  if (first.a_kmajor || first.b_kmajor || !second.a_kmajor || !second.b_kmajor) return PHIP_OK;
  if (first.M <= 0 || first.N <= 0 || first.batch <= 0 || second.M <= 0 || second.N <= 0 || second.batch <= 0)
    return PHIP_OK;
  // a large operand goes to the streaming kernel
  auto streamed = [](const Gemm &p) { return 4L * p.M * p.K * p.rbatch * p.batch >= kStreamedOperandBytes; };
  if (streamed(first) || streamed(second)) return PHIP_OK;

  DirectPlan p2;
  if (!plan_direct(ctx, second, &p2)) return PHIP_OK;
  if (p2.tn != 1 || p2.waves != 4 || !p2.vec_a || !p2.vec_b) return PHIP_OK;

  DirectPlan p1;
  int kind = 0;
  if (plan_direct(ctx, first, &p1)) {
    if (p1.tn != 1 || p1.waves != 4) return PHIP_OK;
    kind = p1.u;
  } else {
    // the staged kernel's rank-K case, below the sizes that the 128 x 128 rank-K kernel takes
    const int cus = ctx->prop.multiProcessorCount;
    const long tiles128 = (long)((first.M + 127) / 128) * ((first.N + 127) / 128) * first.batch;
    if ((long)first.K * first.rbatch > 128 || tiles128 * 2 >= cus) return PHIP_OK;
    StagedPlan sp;
    plan_staged(ctx, first, &sp);
    if (sp.shape != StagedShape::k64x64x32 || !sp.vec_a) return PHIP_OK;
    p1.d.g = sp.a;
    p1.d.chunks_per_r = 0;
    p1.d.total_chunks = 0;
    p1.grid = sp.grid;
    kind = sp.vec_b ? kStaged : kStagedB1;
  }
  const long padded = (p1.grid + 7) / 8 * 8;
  if (padded + p2.grid > 0x7fffffffL) return PHIP_OK;
  note_kernel(ctx, "f32_pair");
  *handled = true;
#define PHIP_PAIR(FIRST, U2)                                                                                  \
  hipLaunchKernelGGL((gemm_f32_pair_kernel<FIRST, U2>), dim3((unsigned)(padded + p2.grid)), dim3(kThreads), 0, \
                     ctx->stream, p1.d, p2.d, (int)p1.grid, (int)padded)
  if (p2.u == 8) {
    if (kind == kStaged) PHIP_PAIR(kStaged, 8);
    else if (kind == kStagedB1) PHIP_PAIR(kStagedB1, 8);
    else if (kind == 8) PHIP_PAIR(8, 8);
    else PHIP_PAIR(4, 8);
  } else {
    if (kind == kStaged) PHIP_PAIR(kStaged, 4);
    else if (kind == kStagedB1) PHIP_PAIR(kStagedB1, 4);
    else if (kind == 8) PHIP_PAIR(8, 4);
    else PHIP_PAIR(4, 4);
  }
#undef PHIP_PAIR
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace phip
