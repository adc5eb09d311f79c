// Two lanes for matrix products: which stream a matmul call runs on, and the waits that keep the
// order of the caller's calls observable.
//
// The per-timestep products of a recurrent network are launches of 6 - 30 us of which several us
// are dispatch, the first loads and the last stores; each leaves most of the chip idle most of
// that time.  Two such launches that do not depend on each other overlap well: measured on the
// three per-timestep workloads, a forward product on one stream beside the gradient products of
// the previous call on another takes 8.6 instead of 13.3 us (dense layer), 9.3 instead of 15.6
// (recurrent gate), 36.5 instead of 44 (output projection) per pair of calls.  What does not come
// cheap is a wait of one stream for the other: an event recorded on one and waited for on the
// other costs about 10 us on the GPU's timeline, whatever the event's flags (measured: a loop that
// needs three such pairs per iteration took 38 us per iteration instead of 15).  So the lanes are
// for runs of matmul calls, not for graphs that put other work between them:
//
//  * Only matrix products move; every other operation is enqueued on the main lane (PHIP_ENTER ->
//    lanes_join).
//  * The side lane is engaged by the kEngageAfter-th matmul call in a row (one wait: the side lane
//    starts behind what the main lane holds so far) and released by the first operation of another
//    kind that enqueues work (one wait: the main lane continues behind the side lane).  Calls that
//    make the host wait (phip_sync, copies from and to host memory) wait for both lanes on the host
//    and leave them engaged; phip_event_record orders the main lane behind the side lane and
//    leaves them engaged.  If that happens before
//    kWorthwhile products ran on the engaged lanes, the next run has to be twice as long to engage
//    them (up to kEngageAfterMax): a caller that never issues long runs pays for one attempt.
//  * While engaged, a product goes to the lane that holds the earlier products it overlaps in
//    memory (stream order then does the waiting); when both lanes hold such products it waits for
//    the tail of the other lane; when none does it takes the lane the previous product did not
//    take.
//  * Large products (more than the caller's limit) fill the chip by themselves and stay on the
//    main lane, as do the products of an allocation-free call.
// The side lane is a context of its own: scratch blocks and tile counters of launches on
// different lanes are never shared.
//
// Environment, read when a context is created: PHIP_OVERLAP=0 no side lane is ever engaged;
// PHIP_OVERLAP_AFTER=n the run length that engages it (tests use 1); PHIP_OVERLAP_BACKOFF=0 that
// length never grows.
#include <cstdlib>

#include "phip_internal.h"

namespace phip {

namespace {

constexpr int kEngageAfter = 6;
constexpr int kEngageAfterMax = 384;
constexpr int kWorthwhile = 8;
constexpr size_t kMaxTrackedRanges = 160;

bool overlaps(const MemRange *ranges, int n, const std::vector<MemRange> &ops) {
  for (const MemRange &o : ops) {
    for (int i = 0; i < n; ++i) {
      const MemRange &r = ranges[i];
      if ((r.write || o.write) && r.lo < o.hi && o.lo < r.hi) return true;
    }
  }
  return false;
}

// Adds the ranges to a lane's list; a range that is there already (the shared operand of every
// call of a run) is not added again.
void track(std::vector<MemRange> &ops, const MemRange *ranges, int n) {
  for (int i = 0; i < n; ++i) {
    bool known = false;
    for (MemRange &o : ops) {
      if (o.lo == ranges[i].lo && o.hi == ranges[i].hi) {
        o.write = o.write || ranges[i].write;
        known = true;
        break;
      }
    }
    if (!known) ops.push_back(ranges[i]);
  }
}

// Everything enqueued on `from` so far comes before whatever is enqueued on `to` from now on.
int order_after(hipStream_t to, hipStream_t from, hipEvent_t ev) {
  PHIP_HIP(hipEventRecord(ev, from));
  PHIP_HIP(hipStreamWaitEvent(to, ev, 0));
  return PHIP_OK;
}

int env_int(const char *name, int otherwise) {
  const char *v = std::getenv(name);
  return v != nullptr && v[0] != '\0' ? std::atoi(v) : otherwise;
}

}  // namespace

int lanes_create(phip_ctx *ctx) {
  Lanes *l = new Lanes();
  l->enabled = env_int("PHIP_OVERLAP", 1) != 0;
  l->engage_after_base = env_int("PHIP_OVERLAP_AFTER", kEngageAfter);
  if (l->engage_after_base < 1) l->engage_after_base = 1;
  l->engage_after = l->engage_after_base;
  l->back_off = env_int("PHIP_OVERLAP_BACKOFF", 1) != 0;
  hipError_t e = hipEventCreateWithFlags(&l->main_tail, hipEventDisableTiming);
  if (e == hipSuccess) e = hipEventCreateWithFlags(&l->side_tail, hipEventDisableTiming);
  int rc = e == hipSuccess ? PHIP_OK : fail(PHIP_ERR_RUNTIME, "hipEventCreate failed: %s", hipGetErrorString(e));
  if (rc == PHIP_OK) rc = ctx_create(ctx->device, false, &l->side);
  if (rc != PHIP_OK) {
    if (l->main_tail) (void)hipEventDestroy(l->main_tail);
    if (l->side_tail) (void)hipEventDestroy(l->side_tail);
    delete l;
    return rc;
  }
  // the lists never grow past this: no allocation once the context exists
  l->main_ops.reserve(kMaxTrackedRanges + 8);
  l->side_ops.reserve(kMaxTrackedRanges + 8);
  ctx->lanes = l;
  return PHIP_OK;
}

int lanes_destroy(phip_ctx *ctx) {
  Lanes *l = ctx->lanes;
  if (l == nullptr) return PHIP_OK;
  ctx->lanes = nullptr;
  int rc = PHIP_OK;
  if (l->side != nullptr) rc = phip_ctx_destroy(l->side);  // waits for its stream
  if (l->main_tail) (void)hipEventDestroy(l->main_tail);
  if (l->side_tail) (void)hipEventDestroy(l->side_tail);
  delete l;
  return rc;
}

// An operation of another kind follows on the main lane: it comes after everything on both.
int lanes_join(phip_ctx *ctx) {
  Lanes *l = ctx->lanes;
  l->streak = 0;
  if (!l->engaged) return PHIP_OK;
  if (!l->side_ops.empty()) {
    const int rc = order_after(ctx->stream, l->side->stream, l->side_tail);
    if (rc != PHIP_OK) return rc;
  }
  l->side_ops.clear();
  l->main_ops.clear();
  l->engaged = false;
  if (l->back_off && l->since_engaged < kWorthwhile) {
    l->engage_after = l->engage_after * 2 < kEngageAfterMax ? l->engage_after * 2 : kEngageAfterMax;
  } else {
    l->engage_after = l->engage_after_base;
  }
  return PHIP_OK;
}

int lanes_wait_host(phip_ctx *ctx) {
  Lanes *l = ctx->lanes;
  if (!l->engaged) return PHIP_OK;
  if (!l->side_ops.empty()) PHIP_HIP(hipStreamSynchronize(l->side->stream));
  if (!l->main_ops.empty()) PHIP_HIP(hipStreamSynchronize(ctx->stream));
  // nothing that the lists name is in flight any more
  l->side_ops.clear();
  l->main_ops.clear();
  return PHIP_OK;
}

int lanes_order_main_after_side(phip_ctx *ctx) {
  Lanes *l = ctx->lanes;
  if (!l->engaged || l->side_ops.empty()) return PHIP_OK;
  const int rc = order_after(ctx->stream, l->side->stream, l->side_tail);
  if (rc != PHIP_OK) return rc;
  l->side_ops.clear();
  return PHIP_OK;
}

int lanes_place(phip_ctx *ctx, const MemRange *ranges, int n, bool may_overlap, phip_ctx **run_on) {
  *run_on = ctx;
  Lanes *l = ctx->lanes;
  if (l == nullptr || !l->enabled) return PHIP_OK;
  ++l->streak;
  if (!l->engaged) {
    if (!may_overlap || l->streak < l->engage_after) return PHIP_OK;
    // the side lane starts behind everything the main lane holds
    const int rc = order_after(l->side->stream, ctx->stream, l->main_tail);
    if (rc != PHIP_OK) return rc;
    l->engaged = true;
    l->since_engaged = 0;
    l->last_lane = 0;
  }
  ++l->since_engaged;
  const bool on_main = overlaps(ranges, n, l->main_ops), on_side = overlaps(ranges, n, l->side_ops);
  int lane;
  if (!may_overlap) lane = 0;
  else if (on_main != on_side) lane = on_side ? 1 : 0;
  else if (on_main) lane = l->last_lane;
  else lane = 1 - l->last_lane;

  phip_ctx *side = l->side;
  if (lane == 0) {
    if (on_side) {
      const int rc = order_after(ctx->stream, side->stream, l->side_tail);
      if (rc != PHIP_OK) return rc;
      l->side_ops.clear();
    }
    if (l->main_ops.size() + n > kMaxTrackedRanges) {
      // the list is full: the side lane waits for what the main lane holds so far
      const int rc = order_after(side->stream, ctx->stream, l->main_tail);
      if (rc != PHIP_OK) return rc;
      l->main_ops.clear();
    }
    track(l->main_ops, ranges, n);
  } else {
    if (on_main) {
      const int rc = order_after(side->stream, ctx->stream, l->main_tail);
      if (rc != PHIP_OK) return rc;
      l->main_ops.clear();
    }
    if (l->side_ops.size() + n > kMaxTrackedRanges) {
      const int rc = order_after(ctx->stream, side->stream, l->side_tail);
      if (rc != PHIP_OK) return rc;
      l->side_ops.clear();
    }
    track(l->side_ops, ranges, n);
    side->deterministic = ctx->deterministic;
    *run_on = side;
  }
  l->last_lane = lane;
  return PHIP_OK;
}

}  // namespace phip

extern "C" int phip_set_overlap(phip_ctx *ctx, int on) {
  PHIP_ENTER(ctx);  // releases the side lane
  if (ctx->lanes != nullptr) ctx->lanes->enabled = on != 0;
  return PHIP_OK;
}
