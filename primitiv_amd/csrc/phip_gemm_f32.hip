// Launches of the LDS-staged fp32 GEMM and the choice among the fp32 kernels.
#include "phip_gemm_f32_staged.h"

namespace phip {
namespace {

template <int BM, int BN, int BK, int WGM, int WGN, int WGK, int OCC, bool A_KMAJOR, bool B_KMAJOR, int VA, int VB>
__global__ __launch_bounds__(kThreads, OCC) void gemm_f32_kernel(const GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float lds[staged_lds_floats<BM, BN, BK, WGM, WGN, WGK>()];
  staged_tile<BM, BN, BK, WGM, WGN, WGK, A_KMAJOR, B_KMAJOR, VA, VB>(g, lds, blockIdx.x, gridDim.x);
}

template <int BM, int BN, int BK, int WGM, int WGN, int WGK, int OCC>
int launch_tile(phip_ctx *ctx, const Gemm &p, const StagedPlan &plan) {
  const GemmArgs &a = plan.a;
  const long grid = plan.grid;
  if (grid > 0x7fffffffL) return fail(PHIP_ERR_INVALID_ARGUMENT, "matmul problem too large for one launch");

  if (a.atomic && !p.accumulate) {
    const int rc = zero_c(ctx, p);
    if (rc != PHIP_OK) return rc;
  }

  const bool vec_a = plan.vec_a, vec_b = plan.vec_b;
#define PHIP_LAUNCH_V(AK, BKM, VVA, VVB)                                                            \
  hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, BK, WGM, WGN, WGK, OCC, AK, BKM, VVA, VVB>),            \
                     dim3((unsigned)grid), dim3(kThreads), 0, ctx->stream, a)
#define PHIP_LAUNCH(AK, BKM)                                                                        \
  do {                                                                                              \
    if (vec_a && vec_b) PHIP_LAUNCH_V(AK, BKM, 4, 4);                                               \
    else if (vec_a) PHIP_LAUNCH_V(AK, BKM, 4, 1);                                                   \
    else if (vec_b) PHIP_LAUNCH_V(AK, BKM, 1, 4);                                                   \
    else PHIP_LAUNCH_V(AK, BKM, 1, 1);                                                              \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) {
    PHIP_LAUNCH(false, true);
  } else if (!p.a_kmajor && !p.b_kmajor) {
    PHIP_LAUNCH(false, false);
  } else if (p.a_kmajor && p.b_kmajor) {
    PHIP_LAUNCH(true, true);
  } else {
    return fail(PHIP_ERR_INVALID_ARGUMENT, "operand layout combination not used by matmul");
  }
#undef PHIP_LAUNCH_V
#undef PHIP_LAUNCH
  PHIP_LAUNCH_CHECK();
  return PHIP_OK;
}

}  // namespace

int gemm_f32(phip_ctx *ctx, const Gemm &p) {
  if (p.M <= 0 || p.N <= 0 || p.batch <= 0) return PHIP_OK;
  bool handled = false;
  int rc = gemm_f32_slab(ctx, p, &handled);
  if (rc != PHIP_OK || handled) return rc;
  rc = gemm_f32_rankk(ctx, p, &handled);
  if (rc != PHIP_OK || handled) return rc;
  rc = gemm_f32_lds(ctx, p, &handled);
  if (rc != PHIP_OK || handled) return rc;
  rc = gemm_f32_tile16(ctx, p, &handled);
  if (rc != PHIP_OK || handled) return rc;
  rc = gemm_f32_direct(ctx, p, &handled);
  if (rc != PHIP_OK || handled) return rc;
  StagedPlan plan;
  plan_staged(ctx, p, &plan);
  switch (plan.shape) {
    case StagedShape::k128x128x16:
      note_kernel(ctx, "f32_staged128");
      return launch_tile<128, 128, 16, 2, 2, 1, 4>(ctx, p, plan);
    case StagedShape::k64x64x32:
      note_kernel(ctx, "f32_staged64");
      return launch_tile<64, 64, 32, 2, 2, 1, 2>(ctx, p, plan);
    default:
      note_kernel(ctx, "f32_staged32");
      return launch_tile<32, 32, 64, 1, 1, 4, 2>(ctx, p, plan);
  }
}

}  // namespace phip
