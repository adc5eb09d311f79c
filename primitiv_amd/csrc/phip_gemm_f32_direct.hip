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
  // An overwriting product that is split leaves fp32 partial tiles in scratch memory and lets the last
  // workgroup of each tile add them (no zero fill of C, no atomics on it, one launch); the atomics
  // remain for an accumulating product and as the fallback.
  void *block = nullptr;
  if (a.atomic && !p.accumulate) {
    const long tiles = (long)a.tiles_m * a.tiles_n * p.batch;
    const size_t bytes = sizeof(float) * (size_t)p.M * p.N * p.batch * a.splits;
    if (tiles <= kTicketSlots && bytes <= (size_t)(64L << 20) && phip_pool_alloc(ctx, bytes, &block, nullptr) == PHIP_OK) {
      a.atomic = 2;
      a.partial = static_cast<float *>(block);
    } else {
      const int cus = ctx->prop.multiProcessorCount;
      const long total = (long)p.M * p.N * p.batch;
      long blocks = (total + kThreads * 4 - 1) / (kThreads * 4);
      if (blocks > cus * 8L) blocks = cus * 8L;
      hipLaunchKernelGGL(zero_c_kernel, dim3((unsigned)blocks), dim3(kThreads), 0, ctx->stream, a.C, p.M, p.N,
                         p.ldc, p.sC, p.batch);
      PHIP_LAUNCH_CHECK();
    }
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
    if (block) phip_pool_free(ctx, block);
    return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
  }
#undef PHIP_DIRECT_V
  if (block) phip_pool_free(ctx, block);  // the stream is in order: reusable behind this launch
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
