// Launches of the fp32 rank-K update (phip_gemm_f32_rankk.h).
#include "phip_gemm_f32_rankk.h"

namespace phip {
namespace {

__global__ __launch_bounds__(kThreads, 2) void gemm_f32_rankk_kernel(const LdsArgs d) {
  const GemmArgs &g = d.g;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  int t = xcd_remap(blockIdx.x, gridDim.x);
  const int tile_m = t % g.tiles_m; t /= g.tiles_m;
  const int tile_n = t % g.tiles_n; t /= g.tiles_n;
  rankk_tiles(d, lds, t, tile_m, tile_n, 1);
}

}  // namespace

// Rank-K updates (K <= 64) of matrices large enough that C's traffic is the
// cost.  Sets *handled when it launched.
int gemm_f32_rankk(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  RankKPlan plan;
  if (!plan_rankk(p, &plan)) return PHIP_OK;
  // one round of resident workgroups (two per compute unit), most compute units busy
  const int cus = ctx->prop.multiProcessorCount;
  if (plan.tiles > 2L * cus || plan.tiles * 2 < cus) return PHIP_OK;
  auto kern = gemm_f32_rankk_kernel;
  const int rc = raise_lds_limit(ctx, kSlotGemmF32RankK, reinterpret_cast<const void *>(kern), kRankLdsBytes);
  if (rc != PHIP_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)plan.tiles), dim3(kThreads), kRankLdsBytes, ctx->stream, plan.d);
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "f32_rankk");
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
