// The two gradient products of a large per-timestep layer in ONE launch:
//   ga += gy . b^T   a rank-K update of a large matrix (K = minibatch <= 64): bound by reading and
//                    writing ga, its matrix instructions are a small part of its time;
//   gb += a^T . gy   a large operand streamed against <= 64 columns: reads a once and keeps the
//                    matrix cores busy most of the time.
// Run one after the other, each leaves half of the chip's resources idle (the first the matrix
// cores, the second the memory system) and each pays the launch latency and the ramps at its ends.
// Here one grid carries both, sized so that every workgroup is resident at once (two per compute
// unit by LDS): workgroups below `first_blocks` take the rank-K update - each a strip of up to
// four 128 x 128 tiles of one row block, the next tile's old values fetched under the current
// tile's matrix instructions - the others one 32 x 64 tile of the streamed product over a K range.
// A compute unit then holds one of each and overlaps their phases.  The code of a workgroup is
// that of the stand-alone kernels (phip_gemm_f32_rankk.h, phip_gemm_f32_slab.h).
#include "phip_gemm_f32_rankk.h"
#include "phip_gemm_f32_slab.h"

namespace phip {
namespace {

// The streamed product's workgroups as on their own: 32 x 64 tiles, four stages in flight.  64 x 64 tiles
// with five stages of A in flight, and 32 x 64 tiles with 8 or 11, measured 1 - 3 % slower on the output
// projection: the mix of the two products is not bound by how much of the streamed operand is in flight.
constexpr int kPairMB = 1, kPairRingA = 4;
constexpr int kStreamPairLdsBytes =
    kRankLdsBytes > slab_lds_bytes(kPairMB, kPairRingA) ? kRankLdsBytes : slab_lds_bytes(kPairMB, kPairRingA);

struct StripArgs {
  int blocks;         // workgroups of the rank-K update
  int padded;         // the streamed product starts here (a multiple of 8: same XCD order as on its own)
  int tiles_per_wg;   // 128-column tiles per strip
};

__global__ __launch_bounds__(kThreads, 2) void gemm_f32_stream_pair_kernel(const LdsArgs first, const LdsArgs second,
                                                                            const StripArgs s) {
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  __shared__ uint32_t last_flag;
  const int bid = blockIdx.x;
  if (bid < s.blocks) {
    // strips of one column group are neighbours: they share B's rows
    int t = xcd_remap(bid, s.blocks);
    const int tile_m = t % first.g.tiles_m;
    const int group = t / first.g.tiles_m;
    const int tn0 = group * s.tiles_per_wg;
    const int left = first.g.tiles_n - tn0;
    rankk_tiles(first, lds, 0, tile_m, tn0, left < s.tiles_per_wg ? left : s.tiles_per_wg);
  } else if (bid >= s.padded) {
    slab_tile<true, true, kPairMB, kPairRingA>(second, lds, &last_flag, bid - s.padded, (int)gridDim.x - s.padded);
  }
}

}  // namespace

int gemm_f32_stream_pair(phip_ctx *ctx, const Gemm &first, const Gemm &second, bool *handled) {
  *handled = false;
  if (!first.accumulate || !second.accumulate) return PHIP_OK;
  // the shared launch adds the tiles of a split product with atomics
  if (ctx->deterministic) return PHIP_OK;
  if (first.batch != 1 || second.batch != 1 || first.rbatch != 1) return PHIP_OK;
  if (!second.a_kmajor || !second.b_kmajor) return PHIP_OK;
  const int cus = ctx->prop.multiProcessorCount;
  RankKPlan rp;
  if (!plan_rankk(first, &rp)) return PHIP_OK;
  // one place per compute unit for each product
  SlabPlan sp;
  if (!plan_slab(second, cus, 1, &sp, kPairMB) || sp.grid > cus) return PHIP_OK;
  // worth it when the update alone would occupy the chip (as for the stand-alone kernel)
  if (rp.tiles * 2 < cus) return PHIP_OK;
  const int per = (int)((rp.tiles + cus - 1) / cus);
  if (per > 4) return PHIP_OK;
  const int groups = (rp.d.g.tiles_n + per - 1) / per;
  StripArgs s;
  s.blocks = rp.d.g.tiles_m * groups;
  if (s.blocks > cus) return PHIP_OK;
  s.padded = (s.blocks + 7) / 8 * 8;
  s.tiles_per_wg = per;
  auto kern = gemm_f32_stream_pair_kernel;
  const int rc = raise_lds_limit(ctx, kSlotGemmF32StreamPair, reinterpret_cast<const void *>(kern), kStreamPairLdsBytes);
  if (rc != PHIP_OK) return rc;
  hipLaunchKernelGGL(kern, dim3((unsigned)(s.padded + sp.grid)), dim3(kThreads), kStreamPairLdsBytes, ctx->stream,
                     rp.d, sp.d, s);
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "f32_stream_pair");
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip

