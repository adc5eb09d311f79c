// Launches of the streamed-operand fp32 GEMM (phip_gemm_f32_slab.h).
#include "phip_gemm_f32_slab.h"

namespace phip {
namespace {

// Stages of A in flight: as many as of B.  Deeper rings (6 and 11 stages, 56 and 76 KiB of LDS, still two
// workgroups per compute unit) measured slower on the output projection's forward product: 16.3, 16.6 and
// 17.1 us; how far ahead A is fetched is not what its K loop waits for.
constexpr int kSlabRingA = 4;

template <bool A_KMAJOR, bool B_KMAJOR>
__global__ __launch_bounds__(kThreads, 2) void gemm_f32_slab_kernel(const LdsArgs d) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  __shared__ uint32_t last_flag;
  slab_tile<A_KMAJOR, B_KMAJOR, 1, kSlabRingA>(d, lds, &last_flag, blockIdx.x, gridDim.x);
}

}  // namespace

// Narrow outputs over a large streamed operand.  Sets *handled when it launched.
int gemm_f32_slab(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  SlabPlan plan;
  // two workgroups fit a compute unit
  if (!plan_slab(p, ctx->prop.multiProcessorCount, 2, &plan)) return PHIP_OK;
  LdsArgs &d = plan.d;
  Scratch partials(ctx);
  if (d.g.atomic && wants_exchange(ctx, p)) {
    const int rc = prepare_split_exchange(ctx, p, plan.tiles, (size_t)(64L << 20), &d.g, &partials);
    if (rc != PHIP_OK) return rc;
  }
#define PHIP_SLAB_G(SLOT, AK, BKM)                                                                           \
  do {                                                                                                       \
    auto kern = gemm_f32_slab_kernel<AK, BKM>;                                                               \
    const int lds_bytes = slab_lds_bytes(1, kSlabRingA);                                                     \
    const int rc = raise_lds_limit(ctx, SLOT, reinterpret_cast<const void *>(kern), lds_bytes);              \
    if (rc != PHIP_OK) return rc;                                                                            \
    hipLaunchKernelGGL(kern, dim3((unsigned)plan.grid), dim3(kThreads), lds_bytes, ctx->stream, d);          \
  } while (0)
  if (!p.a_kmajor && p.b_kmajor) PHIP_SLAB_G(kSlotGemmF32Slab + 0, false, true);
  else if (!p.a_kmajor && !p.b_kmajor) PHIP_SLAB_G(kSlotGemmF32Slab + 1, false, false);
  else PHIP_SLAB_G(kSlotGemmF32Slab + 2, true, true);
#undef PHIP_SLAB_G
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "f32_slab");
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip

