// Native timing loops for bench.py (host code only; links against libphip).
//
// The per-timestep workloads are bound by dispatch, so what the caller does
// around the entry points is part of their cost, and primitiv's callers are
// C++.  Every loop brackets its timed region with events on the context's
// stream and also reports the host clock.
//
//  * phip_bench_raw_loop: matmul_fw + matmul_bw on preallocated outputs.
//  * phip_bench_front_loop: per timestep what primitiv's Device front does
//    around matmul_fw / matmul_bw (primitiv/core/device.cc:20-24,268-301;
//    functions::zeros -> reset_tensor): y from the pool (uninitialised), the
//    forward product, the per-timestep operand's gradient from the pool and
//    zero-filled, the backward products, both blocks handed back.
//  * phip_bench_lstm_loop: one LSTM layer unrolled over its timesteps, forward
//    then backward, device call by device call as primitiv's Graph issues them
//    for the layer of examples/ptb/ptb_rnnlm_lstm.cc:101-109.
#include <chrono>
#include <cstddef>
#include <cstdint>
#include <vector>

#include "include/phip.h"

namespace {

// The entry points of one storage type behind one signature each.
struct Api {
  size_t item;
  int (*fill)(phip_ctx *, void *, float, size_t);
  int (*inplace_add)(phip_ctx *, const void *, void *, uint32_t, uint32_t, uint32_t);
  int (*matmul_fw)(phip_ctx *, const void *, const void *, void *, uint32_t, uint32_t, uint32_t, uint32_t, uint32_t);
  int (*matmul_bw)(phip_ctx *, const void *, const void *, const void *, void *, void *, uint32_t, uint32_t, uint32_t,
                   uint32_t, uint32_t);
  int (*unary_fw)(phip_ctx *, int, const void *, void *, size_t);
  int (*unary_bw)(phip_ctx *, int, const void *, const void *, const void *, void *, size_t);
  int (*binary_fw)(phip_ctx *, int, const void *, const void *, void *, uint32_t, uint32_t, uint32_t);
  int (*binary_bw)(phip_ctx *, int, const void *, const void *, const void *, const void *, void *, void *, uint32_t,
                   uint32_t, uint32_t);
  int (*copy_rows)(phip_ctx *, const void *, void *, uint32_t, uint32_t, uint64_t, uint64_t, uint32_t, uint64_t,
                   uint64_t, int);
};

#define F(p) static_cast<float *>(p)
#define CF(p) static_cast<const float *>(p)
const Api kF32 = {
    4,
    [](phip_ctx *c, void *p, float v, size_t n) { return phip_fill_f32(c, F(p), v, n); },
    [](phip_ctx *c, const void *x, void *y, uint32_t v, uint32_t bx, uint32_t by) {
      return phip_inplace_add_f32(c, CF(x), F(y), v, bx, by);
    },
    [](phip_ctx *c, const void *a, const void *b, void *y, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba,
       uint32_t bb) { return phip_matmul_fw_f32(c, CF(a), CF(b), F(y), di, dj, dk, ba, bb); },
    [](phip_ctx *c, const void *a, const void *b, const void *gy, void *ga, void *gb, uint32_t di, uint32_t dj,
       uint32_t dk, uint32_t ba, uint32_t bb) {
      return phip_matmul_bw_f32(c, CF(a), CF(b), CF(gy), F(ga), F(gb), di, dj, dk, ba, bb);
    },
    [](phip_ctx *c, int op, const void *x, void *y, size_t n) { return phip_unary_fw_f32(c, op, CF(x), F(y), n); },
    [](phip_ctx *c, int op, const void *x, const void *y, const void *gy, void *gx, size_t n) {
      return phip_unary_bw_f32(c, op, CF(x), CF(y), CF(gy), F(gx), n);
    },
    [](phip_ctx *c, int op, const void *a, const void *b, void *y, uint32_t v, uint32_t ba, uint32_t bb) {
      return phip_binary_fw_f32(c, op, CF(a), CF(b), F(y), v, ba, bb);
    },
    [](phip_ctx *c, int op, const void *a, const void *b, const void *y, const void *gy, void *ga, void *gb,
       uint32_t v, uint32_t ba, uint32_t bb) {
      return phip_binary_bw_f32(c, op, CF(a), CF(b), CF(y), CF(gy), F(ga), F(gb), v, ba, bb);
    },
    [](phip_ctx *c, const void *s, void *d, uint32_t span, uint32_t rows, uint64_t ss, uint64_t ds, uint32_t bs,
       uint64_t sbs, uint64_t dbs, int acc) {
      return phip_copy_rows_f32(c, CF(s), F(d), span, rows, ss, ds, bs, sbs, dbs, acc);
    },
};
#undef F
#undef CF
const Api kF16 = {2,
                  phip_fill_f16,
                  phip_inplace_add_f16,
                  phip_matmul_fw_f16,
                  phip_matmul_bw_f16,
                  phip_unary_fw_f16,
                  phip_unary_bw_f16,
                  phip_binary_fw_f16,
                  phip_binary_bw_f16,
                  phip_copy_rows_f16};
const Api kBF16 = {2,
                   phip_fill_bf16,
                   phip_inplace_add_bf16,
                   phip_matmul_fw_bf16,
                   phip_matmul_bw_bf16,
                   phip_unary_fw_bf16,
                   phip_unary_bw_bf16,
                   phip_binary_fw_bf16,
                   phip_binary_bw_bf16,
                   phip_copy_rows_bf16};

const Api *api_of(int storage) { return storage == 0 ? &kF32 : storage == 1 ? &kF16 : storage == 2 ? &kBF16 : nullptr; }

// Host time of the latest timed region up to the point where every call had returned (before the
// host waited for the device): close to the whole region's time when the host is the slower party.
double g_enqueue_ms = 0.0;

int timed(phip_ctx *ctx, int reps, int warmup, int (*pass)(void *), void *state, float *event_ms, double *host_ms) {
  phip_event *e0 = nullptr, *e1 = nullptr;
  int rc = phip_event_create(ctx, &e0);
  if (rc == PHIP_OK) rc = phip_event_create(ctx, &e1);
  for (int i = 0; i < warmup && rc == PHIP_OK; ++i) rc = pass(state);
  if (rc == PHIP_OK) rc = phip_sync(ctx);
  const auto t0 = std::chrono::steady_clock::now();
  if (rc == PHIP_OK) rc = phip_event_record(ctx, e0);
  for (int i = 0; i < reps && rc == PHIP_OK; ++i) rc = pass(state);
  if (rc == PHIP_OK) rc = phip_event_record(ctx, e1);
  g_enqueue_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (rc == PHIP_OK) rc = phip_sync(ctx);
  *host_ms = std::chrono::duration<double, std::milli>(std::chrono::steady_clock::now() - t0).count();
  if (rc == PHIP_OK) rc = phip_event_elapsed_ms(e0, e1, event_ms);
  phip_event_destroy(e0);
  phip_event_destroy(e1);
  return rc;
}

}  // namespace

extern "C" {

struct phip_bench_dims {
  uint32_t di, dj, dk, ba, bb;
};

}  // extern "C"

namespace {

struct Loop {
  phip_ctx *ctx;
  const Api *api;
  const void *a;
  void *ga;
  const void *const *b;
  const void *const *gy;
  void *const *y;
  void *const *gb;
  phip_bench_dims d;
  int timesteps;
  int which;  // 0: forward and backward, 1: forward only, 2: backward only
};

int raw_pass(void *p) {
  const Loop &l = *static_cast<Loop *>(p);
  const phip_bench_dims &d = l.d;
  for (int t = 0; t < l.timesteps; ++t) {
    int rc = PHIP_OK;
    if (l.which != 2) rc = l.api->matmul_fw(l.ctx, l.a, l.b[t], l.y[t], d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc != PHIP_OK) return rc;
    if (l.which != 1) rc = l.api->matmul_bw(l.ctx, l.a, l.b[t], l.gy[t], l.ga, l.gb[t], d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc != PHIP_OK) return rc;
  }
  return PHIP_OK;
}

int front_pass(void *p) {
  const Loop &l = *static_cast<Loop *>(p);
  const phip_bench_dims &d = l.d;
  const uint32_t bs = d.ba > d.bb ? d.ba : d.bb;
  const size_t ny = (size_t)d.di * d.dk * bs, nb = (size_t)d.dj * d.dk * d.bb;
  for (int t = 0; t < l.timesteps; ++t) {
    void *y = nullptr, *gb = nullptr;
    int rc = phip_pool_alloc(l.ctx, ny * l.api->item, &y, nullptr);
    if (rc != PHIP_OK) return rc;
    rc = l.api->matmul_fw(l.ctx, l.a, l.b[t], y, d.di, d.dj, d.dk, d.ba, d.bb);
    if (rc == PHIP_OK) rc = phip_pool_alloc(l.ctx, nb * l.api->item, &gb, nullptr);
    if (rc == PHIP_OK) rc = l.api->fill(l.ctx, gb, 0.0f, nb);
    if (rc == PHIP_OK) rc = l.api->matmul_bw(l.ctx, l.a, l.b[t], l.gy[t], l.ga, gb, d.di, d.dj, d.dk, d.ba, d.bb);
    // the stream is in order: the blocks may go back while the kernels that use them are still queued
    phip_pool_free(l.ctx, y);
    if (gb) phip_pool_free(l.ctx, gb);
    if (rc != PHIP_OK) return rc;
  }
  return PHIP_OK;
}

}  // namespace

extern "C" {

double phip_bench_last_enqueue_ms(void) { return g_enqueue_ms; }

// storage: 0 = f32, 1 = f16, 2 = bf16 (pointers are device addresses of that storage type);
// which: 0 = forward and backward calls, 1 = forward only, 2 = backward only.
int phip_bench_raw_loop(phip_ctx *ctx, int storage, int which, const void *a, void *ga, const void *const *b,
                        const void *const *gy, void *const *y, void *const *gb, const phip_bench_dims *d, int timesteps,
                        int reps, int warmup, float *event_ms, double *host_ms) {
  if (api_of(storage) == nullptr) return PHIP_ERR_INVALID_ARGUMENT;
  Loop l = {ctx, api_of(storage), a, ga, b, gy, y, gb, *d, timesteps, which};
  return timed(ctx, reps, warmup, raw_pass, &l, event_ms, host_ms);
}

int phip_bench_front_loop(phip_ctx *ctx, int storage, const void *a, void *ga, const void *const *b,
                          const void *const *gy, const phip_bench_dims *d, int timesteps, int reps, int warmup,
                          float *event_ms, double *host_ms) {
  if (api_of(storage) == nullptr) return PHIP_ERR_INVALID_ARGUMENT;
  Loop l = {ctx, api_of(storage), a, ga, b, gy, nullptr, nullptr, *d, timesteps, 0};
  return timed(ctx, reps, warmup, front_pass, &l, event_ms, host_ms);
}

// ---- one LSTM layer, forward and backward through time -------------------------------------------
//
//   u = W . concat(x[t], h[t-1]) + b;  (i, f, o, j) = split(u, 4)
//   c[t] = sigmoid(i) * tanh(j) + sigmoid(f) * c[t-1];  h[t] = sigmoid(o) * tanh(c[t])
// (examples/ptb/ptb_rnnlm_lstm.cc:101-109), W {4*hidden, in + hidden}, minibatch `batch`.  The
// device calls and their order are those of primitiv's operators (core/operator_impl.cc) under
// Graph::forward / Graph::backward (core/graph.cc:116-223): every node value is a pool block that
// lives until the graph is cleared; backward walks the operators in reverse order of creation,
// gives every argument without a gradient a zero-filled tensor first and lets the operator add
// into it; h[t] also receives gy[t], the gradient that the layer above sends down.  W's and b's
// gradients accumulate over the timesteps (and over repetitions) in gW, gb.
struct phip_bench_lstm {
  uint32_t in_size, hidden, batch, timesteps;
};

}  // extern "C"

namespace {

struct Lstm {
  phip_ctx *ctx;
  const Api *api;
  phip_bench_lstm d;
  const void *W, *b;
  void *gW, *gb;
  const void *const *x;
  const void *const *gy;
  void *h_last, *gx_first;  // optional copies out
  bool forward_only;
  std::vector<void *> blocks;
  int rc;

  void *raw(size_t elements) {
    void *p = nullptr;
    if (rc == PHIP_OK) rc = phip_pool_alloc(ctx, elements * api->item, &p, nullptr);
    if (p) blocks.push_back(p);
    return p;
  }
  void *zeros(size_t elements) {
    void *p = raw(elements);
    if (rc == PHIP_OK) rc = api->fill(ctx, p, 0.0f, elements);
    return p;
  }
  void release_all() {
    for (void *p : blocks) phip_pool_free(ctx, p);
    blocks.clear();
  }
  void *at(void *p, size_t elements) const { return static_cast<char *>(p) + elements * api->item; }
  const void *at(const void *p, size_t elements) const { return static_cast<const char *>(p) + elements * api->item; }
#define LSTM_DO(call) \
  do {                \
    if (rc == PHIP_OK) rc = (call); \
  } while (0)

  struct Step {
    void *xh, *u0, *u, *v[4], *g[4], *ij, *fc, *c, *tc, *h;
  };

  int pass() {
    const uint32_t H = d.hidden, I = d.in_size, B = d.batch, T = d.timesteps;
    const size_t nh = (size_t)H * B, nu = 4 * nh, nxh = (size_t)(I + H) * B;
    std::vector<Step> s(T);
    // forward; h[-1] = c[-1] = zeros({hidden}) without a minibatch, as LSTM::init makes them
    void *h0 = zeros(H), *c0 = zeros(H);
    for (uint32_t t = 0; t < T && rc == PHIP_OK; ++t) {
      Step &k = s[t];
      const void *hp = t ? s[t - 1].h : h0, *cp = t ? s[t - 1].c : c0;
      const uint32_t hb = t ? B : 1;
      k.xh = raw(nxh);  // concat({x, h}, 0): one strided copy per argument (a stride of 0 repeats h[-1] per sample)
      LSTM_DO(api->copy_rows(ctx, x[t], k.xh, I, 1, I, I + H, B, I, I + H, 0));
      LSTM_DO(api->copy_rows(ctx, hp, at(k.xh, I), H, 1, H, I + H, B, t ? H : 0, I + H, 0));
      k.u0 = raw(nu);
      LSTM_DO(api->matmul_fw(ctx, W, k.xh, k.u0, 4 * H, I + H, 1, 1, B));
      k.u = raw(nu);
      LSTM_DO(api->binary_fw(ctx, PHIP_ADD, k.u0, b, k.u, 4 * H, B, 1));
      for (int q = 0; q < 4; ++q) {  // split(u, 0, 4) = four slices
        k.v[q] = raw(nh);
        LSTM_DO(api->copy_rows(ctx, at(k.u, (size_t)q * H), k.v[q], H, B, 4 * H, H, 1, 0, 0, 0));
      }
      for (int q = 0; q < 4; ++q) {  // i, f, o = sigmoid; j = tanh
        k.g[q] = raw(nh);
        LSTM_DO(api->unary_fw(ctx, q < 3 ? PHIP_SIGMOID : PHIP_TANH, k.v[q], k.g[q], nh));
      }
      k.ij = raw(nh);
      LSTM_DO(api->binary_fw(ctx, PHIP_MULTIPLY, k.g[0], k.g[3], k.ij, H, B, B));
      k.fc = raw(nh);
      LSTM_DO(api->binary_fw(ctx, PHIP_MULTIPLY, k.g[1], cp, k.fc, H, B, hb));
      k.c = raw(nh);
      LSTM_DO(api->binary_fw(ctx, PHIP_ADD, k.ij, k.fc, k.c, H, B, B));
      k.tc = raw(nh);
      LSTM_DO(api->unary_fw(ctx, PHIP_TANH, k.c, k.tc, nh));
      k.h = raw(nh);
      LSTM_DO(api->binary_fw(ctx, PHIP_MULTIPLY, k.g[2], k.tc, k.h, H, B, B));
    }
    if (h_last && rc == PHIP_OK) rc = phip_memcpy_d2d(ctx, h_last, s[T - 1].h, nh * api->item);
    if (forward_only || rc != PHIP_OK) return rc;

    // backward, last timestep first.  gh / gc: gradients of h[t], c[t] as they stand when timestep t is reached.
    void *gh = zeros(nh), *gc = nullptr;
    LSTM_DO(api->inplace_add(ctx, gy[T - 1], gh, H, B, B));
    for (int t = (int)T - 1; t >= 0 && rc == PHIP_OK; --t) {
      Step &k = s[t];
      const void *cp = t ? s[t - 1].c : c0;
      const uint32_t hb = t ? B : 1;
      const size_t nhp = (size_t)H * hb;
      // h = o * tanh(c)
      void *go = zeros(nh), *gtc = zeros(nh);
      LSTM_DO(api->binary_bw(ctx, PHIP_MULTIPLY, k.g[2], k.tc, k.h, gh, go, gtc, H, B, B));
      if (gc == nullptr) gc = zeros(nh);
      LSTM_DO(api->unary_bw(ctx, PHIP_TANH, k.c, k.tc, gtc, gc, nh));
      // c = i*j + f*c[t-1]
      void *gij = zeros(nh), *gfc = zeros(nh);
      LSTM_DO(api->binary_bw(ctx, PHIP_ADD, k.ij, k.fc, k.c, gc, gij, gfc, H, B, B));
      void *gg[4];
      gg[1] = zeros(nh);
      void *gcp = zeros(nhp);
      LSTM_DO(api->binary_bw(ctx, PHIP_MULTIPLY, k.g[1], cp, k.fc, gfc, gg[1], gcp, H, B, hb));
      gg[0] = zeros(nh);
      gg[3] = zeros(nh);
      LSTM_DO(api->binary_bw(ctx, PHIP_MULTIPLY, k.g[0], k.g[3], k.ij, gij, gg[0], gg[3], H, B, B));
      // the four activations, last created first (j, o, f, i)
      void *gv[4];
      gg[2] = go;
      for (int q = 3; q >= 0; --q) {
        gv[q] = zeros(nh);
        LSTM_DO(api->unary_bw(ctx, q < 3 ? PHIP_SIGMOID : PHIP_TANH, k.v[q], k.g[q], gg[q], gv[q], nh));
      }
      // split: four slices added into the gradient of u
      void *gu = zeros(nu);
      for (int q = 0; q < 4; ++q) {
        LSTM_DO(api->copy_rows(ctx, gv[q], at(gu, (size_t)q * H), H, 1, H, 4 * H, B, H, 4 * H, 1));
      }
      // u = u0 + b
      void *gu0 = zeros(nu);
      LSTM_DO(api->binary_bw(ctx, PHIP_ADD, k.u0, b, k.u, gu, gu0, gb, 4 * H, B, 1));
      // u0 = W . xh
      void *gxh = zeros(nxh);
      LSTM_DO(api->matmul_bw(ctx, W, k.xh, gu0, gW, gxh, 4 * H, I + H, 1, 1, B));
      // concat: gx += slice(gxh, 0, in), gh[t-1] += slice(gxh, in, in + hidden)
      void *gx = zeros((size_t)I * B), *part = raw((size_t)I * B);
      LSTM_DO(api->copy_rows(ctx, gxh, part, I, B, I + H, I, 1, 0, 0, 0));
      LSTM_DO(api->inplace_add(ctx, part, gx, I, B, B));
      void *ghp = zeros(nhp), *part2 = raw(nh);
      LSTM_DO(api->copy_rows(ctx, at(gxh, I), part2, H, B, I + H, H, 1, 0, 0, 0));
      LSTM_DO(api->inplace_add(ctx, part2, ghp, H, B, hb));
      if (t == 0 && gx_first && rc == PHIP_OK) rc = phip_memcpy_d2d(ctx, gx_first, gx, (size_t)I * B * api->item);
      // the layer above adds its gradient of h[t-1]
      if (t > 0) LSTM_DO(api->inplace_add(ctx, gy[t - 1], ghp, H, B, B));
      gh = ghp;
      gc = gcp;
    }
    return rc;
  }
#undef LSTM_DO
};

int lstm_pass(void *p) {
  Lstm &l = *static_cast<Lstm *>(p);
  l.rc = PHIP_OK;
  const int rc = l.pass();
  l.release_all();  // the graph is cleared: every node value and gradient goes back to the pool
  return rc;
}

}  // namespace

extern "C" {

int phip_bench_lstm_loop(phip_ctx *ctx, int storage, const phip_bench_lstm *d, const void *W, const void *b, void *gW,
                         void *gb, const void *const *x, const void *const *gy, void *h_last, void *gx_first,
                         int forward_only, int reps, int warmup, float *event_ms, double *host_ms) {
  if (api_of(storage) == nullptr || d == nullptr || d->timesteps == 0) return PHIP_ERR_INVALID_ARGUMENT;
  Lstm l{ctx, api_of(storage), *d, W, b, gW, gb, x, gy, h_last, gx_first, forward_only != 0, {}, PHIP_OK};
  return timed(ctx, reps, warmup, lstm_pass, &l, event_ms, host_ms);
}

}  // extern "C"
