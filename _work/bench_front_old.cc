// Native timing loops for bench.py (host code only; links against libphip).
//
// The per-timestep workloads are bound by dispatch, so what the caller does
// around the two entry points is part of their cost.  phip_bench_front_loop
// does per timestep what primitiv's Device front does around matmul_fw /
// matmul_bw (primitiv/core/device.cc:20-24,268-301; functions::zeros ->
// reset_tensor): take y from the pool (uninitialised), run the forward product,
// take the gradient of the per-timestep operand from the pool and fill it with
// zeros, run the backward products, hand both blocks back.  phip_bench_raw_loop
// calls the two entry points on preallocated outputs, as bench.py's Python loop
// does.  Both bracket the timed region with events on the context's stream and
// also report the host clock.
#include <chrono>
#include <cstddef>
#include <cstdint>

#include "../include/phip.h"

extern "C" {

struct phip_bench_dims {
  uint32_t di, dj, dk, ba, bb;
};

static int timed(phip_ctx *ctx, int reps, int warmup, int (*pass)(void *), void *state, float *event_ms,
                 double *host_ms) {
  phip_event *e0 = nullptr, *e1 = nullptr;
  int rc = phip_event_create(ctx, &e0);
  if (rc == PHIP_OK) rc = phip_event_create(ctx, &e1);
  for (int i = 0; i < warmup && rc == PHIP_OK; ++i) rc = pass(state);
  if (rc == PHIP_OK) rc = phip_sync(ctx);
  const auto t0 = std::chrono::steady_clock::now();
  if (rc == PHIP_OK) rc = phip_event_record(ctx, e0);
  for (int i = 0; i < reps && rc == PHIP_OK; ++i) rc = pass(state);
  if (rc == PHIP_OK) rc = phip_event_record(ctx, e1);
  if (rc == PHIP_OK) rc = phip_sync(ctx);
  *host_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (rc == PHIP_OK) rc = phip_event_elapsed_ms(e0, e1, event_ms);
  phip_event_destroy(e0);
  phip_event_destroy(e1);
  return rc;
}

struct Loop {
  phip_ctx *ctx;
  const float *a;
  float *ga;
  const float *const *b;
  const float *const *gy;
  float *const *y;
  float *const *gb;
  phip_bench_dims d;
  int timesteps;
};

static int raw_pass(void *p) {
  const Loop &l = *static_cast<Loop *>(p);
  const phip_bench_dims &d = l.d;
  for (int t = 0; t < l.timesteps; ++t) {
    int rc = phip_matmul_fw_f32(l.ctx, l.a, l.b[t], l.y[t], d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc != PHIP_OK) return rc;
    rc = phip_matmul_bw_f32(l.ctx, l.a, l.b[t], l.gy[t], l.ga, l.gb[t], d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc != PHIP_OK) return rc;
  }
  return PHIP_OK;
}

static int front_pass(void *p) {
  const Loop &l = *static_cast<Loop *>(p);
  const phip_bench_dims &d = l.d;
  const uint32_t bs = d.ba > d.bb ? d.ba : d.bb;
  const size_t ny = (size_t)d.di * d.dk * bs, nb = (size_t)d.dj * d.dk * d.bb;
  for (int t = 0; t < l.timesteps; ++t) {
    void *y = nullptr, *gb = nullptr;
    int rc = phip_pool_alloc(l.ctx, ny * sizeof(float), &y, nullptr);
    if (rc != PHIP_OK) return rc;
    rc = phip_matmul_fw_f32(l.ctx, l.a, l.b[t], static_cast<float *>(y), d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc == PHIP_OK) rc = phip_pool_alloc(l.ctx, nb * sizeof(float), &gb, nullptr);
    if (rc == PHIP_OK) rc = phip_fill_f32(l.ctx, static_cast<float *>(gb), 0.0f, nb);
    if (rc == PHIP_OK)
      rc = phip_matmul_bw_f32(l.ctx, l.a, l.b[t], l.gy[t], l.ga, static_cast<float *>(gb), d.di, d.dj, d.dk, d.ba,
                              d.bb);
    // the stream is in order: the blocks may go back while the kernels that use them are still queued
    phip_pool_free(l.ctx, y);
    if (gb) phip_pool_free(l.ctx, gb);
    if (rc != PHIP_OK) return rc;
  }
  return PHIP_OK;
}

int phip_bench_raw_loop(phip_ctx *ctx, const float *a, float *ga, const float *const *b, const float *const *gy,
                        float *const *y, float *const *gb, const phip_bench_dims *d, int timesteps, int reps,
                        int warmup, float *event_ms, double *host_ms) {
  Loop l = {ctx, a, ga, b, gy, y, gb, *d, timesteps};
  return timed(ctx, reps, warmup, raw_pass, &l, event_ms, host_ms);
}

int phip_bench_front_loop(phip_ctx *ctx, const float *a, float *ga, const float *const *b, const float *const *gy,
                          const phip_bench_dims *d, int timesteps, int reps, int warmup, float *event_ms,
                          double *host_ms) {
  Loop l = {ctx, a, ga, b, gy, nullptr, nullptr, *d, timesteps};
  return timed(ctx, reps, warmup, front_pass, &l, event_ms, host_ms);
}

}  // extern "C"
