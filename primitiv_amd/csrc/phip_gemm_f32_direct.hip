// Launches of the direct-from-global fp32 GEMM for skinny problems: the kernel
// around one workgroup's work and the choice of its shape.
#include "phip_gemm_f32_direct.h"

namespace phip {
namespace {

template <int TM, int TN, int U, bool A_KMAJOR, bool B_KMAJOR, int VA, int VB, int WAVES>
__global__ __launch_bounds__(64 * WAVES) void gemm_f32_direct_kernel(const DirectArgs d) {
  __shared__ float red[kDirectRedFloats<TM, TN, WAVES>];
  __shared__ uint32_t last_flag;
  direct_tile<TM, TN, U, A_KMAJOR, B_KMAJOR, VA, VB, WAVES>(d, red, &last_flag, blockIdx.x, gridDim.x);
}

template <int TM, int TN, int U, int WAVES>
int launch_direct(phip_ctx *ctx, const Gemm &p, const DirectPlan &plan) {
  DirectArgs d = plan.d;
  GemmArgs &a = d.g;
  const long grid = plan.grid;
  if (grid > 0x7fffffffL) return fail(PHIP_ERR_INVALID_ARGUMENT, "matmul problem too large for one launch");
  Scratch partials(ctx);
  if (a.atomic && wants_exchange(ctx, p)) {
    const int rc = prepare_split_exchange(ctx, p, (long)a.tiles_m * a.tiles_n * p.batch, (size_t)(64L << 20), &a,
                                           &partials);
    if (rc != PHIP_OK) return rc;
  }
  const bool vec_a = plan.vec_a, vec_b = plan.vec_b;
#define PHIP_DIRECT_V(AK, BKM, VVA, VVB)                                                                 \
  hipLaunchKernelGGL((gemm_f32_direct_kernel<TM, TN, U, AK, BKM, VVA, VVB, WAVES>), dim3((unsigned)grid), \
                     dim3(64 * WAVES), 0, ctx->stream, d)
  // only a k-contiguous operand has a 16-byte form
  if (!p.a_kmajor && p.b_kmajor) {
    if (vec_b) PHIP_DIRECT_V(false, true, 1, 4); else PHIP_DIRECT_V(false, true, 1, 1);
  } else if (!p.a_kmajor && !p.b_kmajor) {
    PHIP_DIRECT_V(false, false, 1, 1);
  } else if (p.a_kmajor && p.b_kmajor) {
    if (vec_a && vec_b) PHIP_DIRECT_V(true, true, 4, 4);
    else if (vec_a) PHIP_DIRECT_V(true, true, 4, 1);
    else if (vec_b) PHIP_DIRECT_V(true, true, 1, 4);
    else PHIP_DIRECT_V(true, true, 1, 1);
  } else {
    return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
  }
#undef PHIP_DIRECT_V
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace

// Handles problems whose output is too small to fill the chip with staged
// tiles.  Sets *handled when it launched.
int gemm_f32_direct(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  DirectPlan plan;
  if (!plan_direct(ctx, p, &plan)) return PHIP_OK;
  note_kernel(ctx, "f32_direct");
  *handled = true;
  if (plan.waves == 8) {
    if (plan.tn == 2) return launch_direct<1, 2, 8, 8>(ctx, p, plan);
    return launch_direct<1, 1, 8, 8>(ctx, p, plan);
  }
  if (plan.tn == 2) {
    if (plan.u == 8) return launch_direct<1, 2, 8, 4>(ctx, p, plan);
    return launch_direct<1, 2, 4, 4>(ctx, p, plan);
  }
  if (plan.u == 8) return launch_direct<1, 1, 8, 4>(ctx, p, plan);
  return launch_direct<1, 1, 4, 4>(ctx, p, plan);
}

}  // namespace phip
