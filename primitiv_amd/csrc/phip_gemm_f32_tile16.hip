// fp32 GEMM for an overwriting product with very few outputs and a long K: the forward product of
// a small dense layer, y[256 x 128] = W[256 x 784] . x[784 x 128].
//
// Such a product has 32 output tiles of 32 x 32: too few for 256 compute units, so the direct
// kernel cuts K between workgroups, and an overwriting product then pays for the exchange of
// partial tiles - three dependent trips through memory behind a K loop of 2 us.  Here the tiles
// are 16 x 16 (v_mfma_f32_16x16x4_f32): four times as many workgroups, none of which shares its
// tile.  The 8 wavefronts of a workgroup split K; each issues every load of its range at once
// (at most 8 chunks of 16 k: K <= 1024), runs its matrix instructions and the 8 tiles are summed
// through LDS.  One round of loads, one barrier, one store.
//
// Per lane the instruction takes A[row = lane % 16][k slot = lane / 16] and
// B[k slot = lane / 16][column = lane % 16]; the four instructions of a chunk use
// k = k0 + 4 * (lane / 16) + s, s = 0..3, for both operands, so that the operand that is contiguous
// along k (b) is one 16-byte load per lane and chunk, and the one contiguous along m (a) four
// 4-byte loads that are 64 contiguous bytes per 16 lanes.
#include "phip_gemm_f32_common.h"

namespace phip {
namespace {

constexpr int kT16Waves = 8;
constexpr int kT16Threads = kT16Waves * 64;
constexpr int kT16MaxChunks = 8;  // chunks of 16 k that a wavefront keeps in flight: its whole K range

struct Tile16Args {
  GemmArgs g;
  int chunks_per_wave;
};

typedef float float4a __attribute__((ext_vector_type(4)));

// VB4: rows of B may be fetched 16 bytes at a time (K and ldb multiples of four).
template <bool VB4>
__global__ __launch_bounds__(kT16Threads) void gemm_f32_tile16_kernel(const Tile16Args d) {
  const GemmArgs &g = d.g;
  __shared__ float red[kT16Waves][4][64];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int t = xcd_remap(blockIdx.x, gridDim.x);
  const int m0 = (t % g.tiles_m) * 16, n0 = (t / g.tiles_m) * 16;
  const int r = lane & 15, grp = lane >> 4;
  const bool row_in = m0 + r < g.M, col_in = n0 + r < g.N;
  const float *pa = g.A + (row_in ? m0 + r : 0);                   // a(m, k) at m + k * lda
  const float *pb = g.B + (col_in ? (long)(n0 + r) * g.ldb : 0);   // b(k, n) at k + n * ldb
  const int k_first = wave * d.chunks_per_wave * 16 + 4 * grp;

  float a[kT16MaxChunks][4];
  float b[kT16MaxChunks][4];
#pragma unroll
  for (int c = 0; c < kT16MaxChunks; ++c) {
    const int k = k_first + c * 16;
    const bool live = c < d.chunks_per_wave;
    if (VB4) {
      const bool in = live && col_in && k < g.K;
      const float4a v = *reinterpret_cast<const float4a *>(in ? pb + k : g.B);
      b[c][0] = in ? v.x : 0.0f; b[c][1] = in ? v.y : 0.0f; b[c][2] = in ? v.z : 0.0f; b[c][3] = in ? v.w : 0.0f;
    } else {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const bool in = live && col_in && k + s < g.K;
        const float v = *(in ? pb + k + s : g.B);
        b[c][s] = in ? v : 0.0f;
      }
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const bool in = live && row_in && k + s < g.K;
      const float v = *(in ? pa + (long)(k + s) * g.lda : g.A);
      a[c][s] = in ? v : 0.0f;
    }
  }

  float4a acc = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
  for (int c = 0; c < kT16MaxChunks; ++c) {
    if (c < d.chunks_per_wave) {
#pragma unroll
      for (int s = 0; s < 4; ++s) acc = __builtin_amdgcn_mfma_f32_16x16x4f32(a[c][s], b[c][s], acc, 0, 0, 0);
    }
  }
  // the lane holds rows 4 * (lane / 16) + v, v = 0..3, of column lane % 16
#pragma unroll
  for (int v = 0; v < 4; ++v) red[wave][v][lane] = acc[v];
  __syncthreads();
  if (tid < 256) {
    const int m = tid & 15, n = tid >> 4;  // 16 consecutive threads: 64 contiguous bytes of a column
    float sum = 0.0f;
#pragma unroll
    for (int w = 0; w < kT16Waves; ++w) sum += red[w][m & 3][(m >> 2) * 16 + n];
    if (m0 + m < g.M && n0 + n < g.N) g.C[(m0 + m) + (long)(n0 + n) * g.ldc] = sum;
  }
}

}  // namespace

// Sets *handled when it launched.
int gemm_f32_tile16(phip_ctx *ctx, const Gemm &p, bool *handled) {
  *handled = false;
  if (p.accumulate || p.batch != 1 || p.rbatch != 1 || p.a_kmajor || !p.b_kmajor) return PHIP_OK;
  if (p.K < 256 || p.K > kT16Waves * kT16MaxChunks * 16) return PHIP_OK;
  const int cus = ctx->prop.multiProcessorCount;
  const long tiles32 = (long)((p.M + 31) / 32) * ((p.N + 31) / 32);
  const long tiles16 = (long)((p.M + 15) / 16) * ((p.N + 15) / 16);
  // worth it where 32 x 32 tiles would have to share their K range between workgroups, and where
  // the smaller tiles still fit the chip at once.  (A recurrent gate's forward product, 2048 x 64
  // outputs with K = 512, already runs unsplit on 128 tiles of 32 x 32 with one round of loads;
  // on 512 tiles of 16 x 16 the doubled operand traffic costs what the extra workgroups gain:
  // 15.0 against 15.4 us per timestep in order, 9.8 against 9.2 with two products in flight.)
  if (tiles32 * 2 >= cus || tiles16 > 2L * cus) return PHIP_OK;
  Tile16Args d;
  d.g = problem_args(p);
  d.g.tiles_m = (p.M + 15) / 16;
  d.g.tiles_n = (p.N + 15) / 16;
  d.chunks_per_wave = (p.K + kT16Waves * 16 - 1) / (kT16Waves * 16);
  const bool vb4 = p.K % 4 == 0 && p.ldb % 4 == 0 && (reinterpret_cast<uintptr_t>(p.B) & 15) == 0;
  if (vb4) {
    hipLaunchKernelGGL(gemm_f32_tile16_kernel<true>, dim3((unsigned)tiles16), dim3(kT16Threads), 0, ctx->stream, d);
  } else {
    hipLaunchKernelGGL(gemm_f32_tile16_kernel<false>, dim3((unsigned)tiles16), dim3(kT16Threads), 0, ctx->stream, d);
  }
  PHIP_LAUNCH_CHECK();
  note_kernel(ctx, "f32_tile16");
  *handled = true;
  return PHIP_OK;
}

}  // namespace phip
