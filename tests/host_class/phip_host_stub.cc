// Host stand-in for libphip, TEST INFRASTRUCTURE ONLY.
//
// Implements every entry point of include/phip.h in plain loops on host memory
// ("device pointers" are malloc'ed host blocks), so that the C++ class
// primitiv::devices::HIP can be linked against the real primitiv core and run
// in a container without a GPU.  It exists to execute the class's forwarding
// code (argument order, shapes, handles, copy-on-write, pool behaviour); it is
// never part of the product and never measured.  Arithmetic comes from the CPU
// oracle (oracle/ref_*.c) where the oracle has the operation, otherwise from
// the contract written next to each declaration in phip.h.
//
// Extra, stub-only controls (not in phip.h) let a test put a cap on "device"
// memory and read counters: phip_stub_*.
#include <algorithm>
#include <cmath>
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <random>
#include <vector>

#include <phip.h>

extern "C" {
// oracle/ref_primitiv.c
void ref_matmul_fw(const float *a, const float *b, float *y, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba,
                   uint32_t bb, int threads);
void ref_matmul_bw(const float *a, const float *b, const float *gy, float *ga, float *gb, uint32_t di, uint32_t dj,
                   uint32_t dk, uint32_t ba, uint32_t bb, int threads);
void ref_inplace_add(const float *x, float *y, uint32_t volume, uint32_t bx, uint32_t by);
void ref_batch_sum(const float *x, float *y, uint32_t volume, uint32_t bs);
// oracle/ref_pointwise.c
int ref_unary_fw(int op, const float *src, float *dest, size_t size);
int ref_unary_bw(int op, const float *px, const float *py, const float *pgy, float *pgx, size_t size);
int ref_const_fw(int op, const float *src, float k, float *dest, size_t size);
int ref_const_bw(int op, const float *px, const float *py, const float *pgy, float k, float *pgx, size_t size);
void ref_pown_fw(const float *src, int32_t k, float *dest, size_t size);
void ref_pown_bw(const float *px, const float *py, const float *pgy, int32_t k, float *pgx, size_t size);
int ref_scalar_fw(int op, int k_on_left, const float *src_x, const float *src_k, float *dest, uint32_t size,
                  uint32_t bx, uint32_t bk);
int ref_binary_fw(int op, const float *src_a, const float *src_b, float *dest, uint32_t size, uint32_t ba,
                  uint32_t bb);
int ref_binary_bw(int op, const float *pa, const float *pb, const float *py, const float *pgy, float *pga,
                  float *pgb, uint32_t size, uint32_t ba, uint32_t bb);
void ref_inplace_subtract(const float *src, float *dest, uint32_t size, uint32_t bx, uint32_t by);
// oracle/ref_indexing.c
int ref_reduce_fw(int op, const float *src, const uint32_t *dims, uint32_t depth, uint32_t batch, uint32_t dim,
                  float *dest);
void ref_extremum_bw(const float *px, const float *py, const float *pgy, const uint32_t *dims, uint32_t depth,
                     uint32_t batch, uint32_t dim, float *pgx);
void ref_arg_extremum(int want_max, const float *src, const uint32_t *dims, uint32_t depth, uint32_t batch,
                      uint32_t dim, uint32_t *ret);
// oracle/ref_random.c
int ref_random(int kind, uint64_t seed, uint64_t offset, float p0, float p1, float *y, size_t n);
// oracle/ref_conv_pool.c
void ref_conv2d_fw(const float *x, const float *w, float *y, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0,
                   uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0,
                   uint32_t str1, uint32_t dil0, uint32_t dil1);
void ref_conv2d_bw(const float *x, const float *w, const float *gy, float *gx, float *gw, uint32_t x0, uint32_t x1,
                   uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0,
                   uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1);
void ref_max_pool2d_fw(const float *x, float *y, uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0,
                       uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1);
void ref_max_pool2d_bw(const float *x, const float *y, const float *gy, float *gx, uint32_t x0, uint32_t x1,
                       uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,
                       uint32_t str1);
}

struct phip_ctx {
  int device;
  uint64_t id;
};
struct phip_event {
  int unused;
};
struct phip_randomizer {
  std::mt19937 rng;
};

namespace {

thread_local char g_error[512] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// "device" memory: host blocks with their sizes, a cap and counters
std::mutex g_mutex;
std::map<void *, size_t> g_blocks;
size_t g_live_bytes = 0, g_limit_bytes = ~size_t(0);
uint64_t g_malloc_calls = 0, g_failed_mallocs = 0, g_release_calls = 0, g_next_ctx = 1;
int g_live_contexts = 0;
constexpr int kDevices = 1;

int device_alloc(size_t bytes, void **out) {
  std::lock_guard<std::mutex> lock(g_mutex);
  ++g_malloc_calls;
  *out = nullptr;
  if (bytes > g_limit_bytes || g_live_bytes > g_limit_bytes - bytes) {
    ++g_failed_mallocs;
    return fail(PHIP_ERR_OUT_OF_MEMORY, "stub device memory exhausted: %zu live + %zu asked > %zu", g_live_bytes,
                bytes, g_limit_bytes);
  }
  void *p = std::malloc(bytes ? bytes : 1);
  if (!p) return fail(PHIP_ERR_OUT_OF_MEMORY, "host malloc(%zu) failed", bytes);
  std::memset(p, 0xcd, bytes);  // never hand out zeros by accident
  g_blocks[p] = bytes;
  g_live_bytes += bytes;
  *out = p;
  return PHIP_OK;
}

int device_free(void *p) {
  std::lock_guard<std::mutex> lock(g_mutex);
  auto it = g_blocks.find(p);
  if (it == g_blocks.end()) return fail(PHIP_ERR_INVALID_ARGUMENT, "Detected to dispose unknown handle: %p", p);
  g_live_bytes -= it->second;
  g_blocks.erase(it);
  std::free(p);
  return PHIP_OK;
}

// ---- storage types ------------------------------------------------------------
struct F16 { uint16_t bits; };
struct BF16 { uint16_t bits; };

float widen(float v) { return v; }
float widen(F16 h) {
  const uint32_t s = (h.bits >> 15) & 1u, e = (h.bits >> 10) & 31u, m = h.bits & 1023u;
  float v;
  if (e == 0) v = std::ldexp((float)m, -24);
  else if (e == 31) v = m ? NAN : INFINITY;
  else v = std::ldexp((float)(m | 1024u), (int)e - 25);
  return s ? -v : v;
}
float widen(BF16 h) {
  const uint32_t u = (uint32_t)h.bits << 16;
  float v;
  std::memcpy(&v, &u, 4);
  return v;
}
void narrow(float v, float *out) { *out = v; }
void narrow(float v, F16 *out) {  // round to nearest even
  uint32_t u;
  std::memcpy(&u, &v, 4);
  const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
  const float a = std::fabs(v);
  if (std::isnan(v)) { out->bits = sign | 0x7e00u; return; }
  if (a >= 65520.0f) { out->bits = sign | 0x7c00u; return; }
  if (a < 6.103515625e-05f) {  // subnormal half: multiples of 2^-24
    out->bits = sign | (uint16_t)std::nearbyint(std::ldexp(a, 24));
    return;
  }
  int e;
  const float f = std::frexp(a, &e);  // a = f * 2^e, f in [0.5, 1)
  uint32_t m = (uint32_t)std::nearbyint(std::ldexp(f, 11));  // 1024..2048
  int eh = e + 14;
  if (m == 2048u) { m = 1024u; ++eh; }
  out->bits = sign | (uint16_t)((eh << 10) | (m & 1023u));
}
void narrow(float v, BF16 *out) {
  uint32_t u;
  std::memcpy(&u, &v, 4);
  if (std::isnan(v)) { out->bits = (uint16_t)((u >> 16) | 0x40u); return; }
  u += 0x7fffu + ((u >> 16) & 1u);
  out->bits = (uint16_t)(u >> 16);
}

template <class T>
std::vector<float> load(const void *p, size_t n) {
  std::vector<float> v(n);
  if (p == nullptr) return v;  // an operand the formula does not use
  const T *q = static_cast<const T *>(p);
  for (size_t i = 0; i < n; ++i) v[i] = widen(q[i]);
  return v;
}
template <class T>
void store(const std::vector<float> &v, void *p) {
  T *q = static_cast<T *>(p);
  for (size_t i = 0; i < v.size(); ++i) narrow(v[i], q + i);
}

int check(phip_ctx *ctx) {
  if (ctx == nullptr) return fail(PHIP_ERR_INVALID_ARGUMENT, "null context");
  return PHIP_OK;
}
#define ENTER(ctx) do { int rc__ = check(ctx); if (rc__ != PHIP_OK) return rc__; } while (0)
#define REQUIRE(cond, ...) do { if (!(cond)) return fail(PHIP_ERR_INVALID_ARGUMENT, __VA_ARGS__); } while (0)

// ---- typed bodies ---------------------------------------------------------------

template <class T>
int fill(phip_ctx *ctx, void *p, float value, size_t n) {
  ENTER(ctx);
  T *q = static_cast<T *>(p);
  for (size_t i = 0; i < n; ++i) narrow(value, q + i);
  return PHIP_OK;
}

template <class S, class D>
int cvt(phip_ctx *ctx, const void *src, void *dst, size_t n) {
  ENTER(ctx);
  const S *s = static_cast<const S *>(src);
  D *d = static_cast<D *>(dst);
  for (size_t i = 0; i < n; ++i) narrow(widen(s[i]), d + i);
  return PHIP_OK;
}

template <class T>
int inplace_add(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  ENTER(ctx);
  REQUIRE(bx == by || bx == 1 || by == 1, "batch sizes %u and %u", bx, by);
  auto vx = load<T>(x, (size_t)volume * bx), vy = load<T>(y, (size_t)volume * by);
  ref_inplace_add(vx.data(), vy.data(), volume, bx, by);
  store<T>(vy, y);
  return PHIP_OK;
}

template <class T>
int inplace_subtract(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bx, uint32_t by) {
  ENTER(ctx);
  REQUIRE(bx == by || bx == 1 || by == 1, "batch sizes %u and %u", bx, by);
  auto vx = load<T>(x, (size_t)volume * bx), vy = load<T>(y, (size_t)volume * by);
  ref_inplace_subtract(vx.data(), vy.data(), volume, bx, by);
  store<T>(vy, y);
  return PHIP_OK;
}

template <class T>
int batch_sum(phip_ctx *ctx, const void *x, void *y, uint32_t volume, uint32_t bs) {
  ENTER(ctx);
  auto vx = load<T>(x, (size_t)volume * bs);
  std::vector<float> vy(volume);
  ref_batch_sum(vx.data(), vy.data(), volume, bs);
  store<T>(vy, y);
  return PHIP_OK;
}

int check_matmul(const void *a, const void *b, const void *c, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba,
                 uint32_t bb) {
  REQUIRE(a && b && c, "null tensor pointer");
  REQUIRE(di >= 1 && dj >= 1 && dk >= 1, "matrix dimensions must be positive");
  REQUIRE(ba >= 1 && bb >= 1 && (ba == bb || ba == 1 || bb == 1), "batch sizes %u and %u", ba, bb);
  return PHIP_OK;
}

template <class T>
int matmul_fw(phip_ctx *ctx, const void *a, const void *b, void *y, uint32_t di, uint32_t dj, uint32_t dk,
              uint32_t ba, uint32_t bb) {
  ENTER(ctx);
  int rc = check_matmul(a, b, y, di, dj, dk, ba, bb);
  if (rc != PHIP_OK) return rc;
  const uint32_t bs = std::max(ba, bb);
  auto va = load<T>(a, (size_t)di * dj * ba), vb = load<T>(b, (size_t)dj * dk * bb);
  std::vector<float> vy((size_t)di * dk * bs);
  ref_matmul_fw(va.data(), vb.data(), vy.data(), di, dj, dk, ba, bb, 1);
  store<T>(vy, y);
  return PHIP_OK;
}

template <class T>
int matmul_bw(phip_ctx *ctx, const void *a, const void *b, const void *gy, void *ga, void *gb, uint32_t di,
              uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb) {
  ENTER(ctx);
  int rc = check_matmul(a, b, gy, di, dj, dk, ba, bb);
  if (rc != PHIP_OK) return rc;
  REQUIRE(ga && gb, "null gradient pointer");
  const uint32_t bs = std::max(ba, bb);
  auto va = load<T>(a, (size_t)di * dj * ba), vb = load<T>(b, (size_t)dj * dk * bb);
  auto vgy = load<T>(gy, (size_t)di * dk * bs);
  if (ga == gb) {  // the gradient of a . a: one array takes both contributions
    auto vg = load<T>(ga, (size_t)di * dj * ba);
    std::vector<float> z(vg.size(), 0.0f);
    ref_matmul_bw(va.data(), vb.data(), vgy.data(), vg.data(), z.data(), di, dj, dk, ba, bb, 1);
    for (size_t i = 0; i < vg.size(); ++i) vg[i] += z[i];
    store<T>(vg, ga);
    return PHIP_OK;
  }
  auto vga = load<T>(ga, (size_t)di * dj * ba), vgb = load<T>(gb, (size_t)dj * dk * bb);
  ref_matmul_bw(va.data(), vb.data(), vgy.data(), vga.data(), vgb.data(), di, dj, dk, ba, bb, 1);
  store<T>(vga, ga);
  store<T>(vgb, gb);
  return PHIP_OK;
}

template <class T>
int unary_fw(phip_ctx *ctx, int op, const void *x, void *y, size_t n) {
  ENTER(ctx);
  auto vx = load<T>(x, n);
  std::vector<float> vy(n);
  REQUIRE(ref_unary_fw(op, vx.data(), vy.data(), n) == 0, "unknown unary operation %d", op);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int unary_bw(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx, size_t n) {
  ENTER(ctx);
  REQUIRE(op != PHIP_NEGATE, "negate has no backward operation");
  auto vx = load<T>(x, n), vy = load<T>(y, n), vgy = load<T>(gy, n), vgx = load<T>(gx, n);
  REQUIRE(ref_unary_bw(op, vx.data(), vy.data(), vgy.data(), vgx.data(), n) == 0, "unknown unary operation %d", op);
  store<T>(vgx, gx);
  return PHIP_OK;
}
template <class T>
int const_fw(phip_ctx *ctx, int op, const void *x, float k, void *y, size_t n) {
  ENTER(ctx);
  auto vx = load<T>(x, n);
  std::vector<float> vy(n);
  REQUIRE(ref_const_fw(op, vx.data(), k, vy.data(), n) == 0, "unknown constant operation %d", op);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int const_bw(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, float k, void *gx, size_t n) {
  ENTER(ctx);
  auto vx = load<T>(x, n), vy = load<T>(y, n), vgy = load<T>(gy, n), vgx = load<T>(gx, n);
  REQUIRE(ref_const_bw(op, vx.data(), vy.data(), vgy.data(), k, vgx.data(), n) == 0, "unknown constant operation %d", op);
  store<T>(vgx, gx);
  return PHIP_OK;
}
template <class T>
int pown_fw(phip_ctx *ctx, const void *x, int32_t k, void *y, size_t n) {
  ENTER(ctx);
  auto vx = load<T>(x, n);
  std::vector<float> vy(n);
  ref_pown_fw(vx.data(), k, vy.data(), n);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int pown_bw(phip_ctx *ctx, const void *x, const void *y, const void *gy, int32_t k, void *gx, size_t n) {
  ENTER(ctx);
  auto vx = load<T>(x, n), vy = load<T>(y, n), vgy = load<T>(gy, n), vgx = load<T>(gx, n);
  ref_pown_bw(vx.data(), vy.data(), vgy.data(), k, vgx.data(), n);
  store<T>(vgx, gx);
  return PHIP_OK;
}
template <class T>
int binary_fw(phip_ctx *ctx, int op, const void *a, const void *b, void *y, uint32_t volume, uint32_t ba,
              uint32_t bb) {
  ENTER(ctx);
  REQUIRE(ba == bb || ba == 1 || bb == 1, "batch sizes %u and %u", ba, bb);
  auto va = load<T>(a, (size_t)volume * ba), vb = load<T>(b, (size_t)volume * bb);
  std::vector<float> vy((size_t)volume * std::max(ba, bb));
  REQUIRE(ref_binary_fw(op, va.data(), vb.data(), vy.data(), volume, ba, bb) == 0, "unknown binary operation %d", op);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int binary_bw(phip_ctx *ctx, int op, const void *a, const void *b, const void *y, const void *gy, void *ga, void *gb,
              uint32_t volume, uint32_t ba, uint32_t bb) {
  ENTER(ctx);
  REQUIRE(ba == bb || ba == 1 || bb == 1, "batch sizes %u and %u", ba, bb);
  const size_t ny = (size_t)volume * std::max(ba, bb);
  auto va = load<T>(a, (size_t)volume * ba), vb = load<T>(b, (size_t)volume * bb), vy = load<T>(y, ny),
       vgy = load<T>(gy, ny);
  if (ga == gb) {
    auto vg = load<T>(ga, (size_t)volume * ba);
    std::vector<float> z(vg.size(), 0.0f);
    REQUIRE(ref_binary_bw(op, va.data(), vb.data(), vy.data(), vgy.data(), vg.data(), z.data(), volume, ba, bb) == 0,
            "unknown binary operation %d", op);
    for (size_t i = 0; i < vg.size(); ++i) vg[i] += z[i];
    store<T>(vg, ga);
    return PHIP_OK;
  }
  auto vga = load<T>(ga, (size_t)volume * ba), vgb = load<T>(gb, (size_t)volume * bb);
  REQUIRE(ref_binary_bw(op, va.data(), vb.data(), vy.data(), vgy.data(), vga.data(), vgb.data(), volume, ba, bb) == 0,
          "unknown binary operation %d", op);
  store<T>(vga, ga);
  store<T>(vgb, gb);
  return PHIP_OK;
}
template <class T>
int scalar_fw(phip_ctx *ctx, int op, int k_on_left, const void *x, const void *k, void *y, uint32_t volume,
              uint32_t bx, uint32_t bk) {
  ENTER(ctx);
  REQUIRE(bx == bk || bx == 1 || bk == 1, "batch sizes %u and %u", bx, bk);
  auto vx = load<T>(x, (size_t)volume * bx), vk = load<T>(k, bk);
  std::vector<float> vy((size_t)volume * std::max(bx, bk));
  REQUIRE(ref_scalar_fw(op, k_on_left, vx.data(), vk.data(), vy.data(), volume, bx, bk) == 0,
          "unknown binary operation %d", op);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int inplace_multiply_const(phip_ctx *ctx, float k, void *x, size_t n) {
  ENTER(ctx);
  T *q = static_cast<T *>(x);
  for (size_t i = 0; i < n; ++i) narrow(widen(q[i]) * k, q + i);
  return PHIP_OK;
}
template <class T>
int identity(phip_ctx *ctx, void *y, uint32_t rows) {
  ENTER(ctx);
  T *q = static_cast<T *>(y);
  for (uint32_t c = 0; c < rows; ++c)
    for (uint32_t r = 0; r < rows; ++r) narrow(r == c ? 1.0f : 0.0f, q + (size_t)c * rows + r);
  return PHIP_OK;
}

// dst[b][r][i] (= or +=) src[b][r][i]; a batch stride of 0 broadcasts the source or sums into the destination
template <class T>
int copy_rows(phip_ctx *ctx, const void *src, void *dst, uint32_t span, uint32_t rows, uint64_t ss, uint64_t ds,
              uint32_t bs, uint64_t sbs, uint64_t dbs, int accumulate) {
  ENTER(ctx);
  REQUIRE(accumulate || dbs != 0 || bs == 1, "an overwriting copy cannot fold the minibatch");
  const T *s = static_cast<const T *>(src);
  T *d = static_cast<T *>(dst);
  for (uint32_t b = 0; b < bs; ++b)
    for (uint32_t r = 0; r < rows; ++r)
      for (uint32_t i = 0; i < span; ++i) {
        const float v = widen(s[b * sbs + r * ss + i]);
        T *out = d + b * dbs + r * ds + i;
        narrow(accumulate ? widen(*out) + v : v, out);
      }
  return PHIP_OK;
}

template <class T>
int pick(phip_ctx *ctx, bool backward, const void *from, const uint32_t *ids, uint32_t n_ids, void *to, uint32_t base,
         uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs) {
  ENTER(ctx);
  REQUIRE(ids != nullptr && (n_ids == bs || n_ids == 1) && (bx == bs || bx == 1), "pick: %u ids, %u and %u samples",
          n_ids, bx, bs);
  for (uint32_t b = 0; b < n_ids; ++b) REQUIRE(ids[b] < n, "pick index %u out of range %u", ids[b], n);
  const size_t xs = (size_t)outer * n * base, ys = (size_t)outer * base;
  for (uint32_t b = 0; b < bs; ++b) {
    const uint32_t id = ids[n_ids == 1 ? 0 : b];
    const size_t xo = (bx == 1 ? 0 : b) * xs, yo = b * ys;
    for (uint32_t o = 0; o < outer; ++o)
      for (uint32_t i = 0; i < base; ++i) {
        const size_t xi = xo + ((size_t)o * n + id) * base + i, yi = yo + (size_t)o * base + i;
        if (!backward) {
          narrow(widen(static_cast<const T *>(from)[xi]), static_cast<T *>(to) + yi);
        } else {
          T *g = static_cast<T *>(to) + xi;
          narrow(widen(*g) + widen(static_cast<const T *>(from)[yi]), g);
        }
      }
  }
  return PHIP_OK;
}

template <class T>
int batch_pick(phip_ctx *ctx, bool backward, const void *from, const uint32_t *ids, uint32_t n_ids, void *to,
               uint32_t volume, uint32_t bx) {
  ENTER(ctx);
  for (uint32_t b = 0; b < n_ids; ++b) REQUIRE(ids[b] < bx, "batch_pick index %u out of range %u", ids[b], bx);
  for (uint32_t b = 0; b < n_ids; ++b)
    for (uint32_t i = 0; i < volume; ++i) {
      const size_t xi = (size_t)ids[b] * volume + i, yi = (size_t)b * volume + i;
      if (!backward) {
        narrow(widen(static_cast<const T *>(from)[xi]), static_cast<T *>(to) + yi);
      } else {
        T *g = static_cast<T *>(to) + xi;
        narrow(widen(*g) + widen(static_cast<const T *>(from)[yi]), g);
      }
    }
  return PHIP_OK;
}

// forward: y (cols x rows) = x^T with x rows x cols; backward: gx (rows x cols) += gy^T with gy cols x rows
template <class T>
int transpose(phip_ctx *ctx, bool backward, const void *from, void *to, uint32_t rows, uint32_t cols, uint32_t bs) {
  ENTER(ctx);
  const size_t per = (size_t)rows * cols;
  for (uint32_t b = 0; b < bs; ++b)
    for (uint32_t c = 0; c < cols; ++c)
      for (uint32_t r = 0; r < rows; ++r) {
        const size_t xi = b * per + (size_t)c * rows + r, yi = b * per + (size_t)r * cols + c;
        if (!backward) {
          narrow(widen(static_cast<const T *>(from)[xi]), static_cast<T *>(to) + yi);
        } else {
          T *g = static_cast<T *>(to) + xi;
          narrow(widen(*g) + widen(static_cast<const T *>(from)[yi]), g);
        }
      }
  return PHIP_OK;
}

// y's dimension i is x's dimension perm[i]
template <class T>
int permute_dims(phip_ctx *ctx, bool backward, const void *from, void *to, uint32_t ndims, const uint32_t *dims,
                 const uint32_t *perm, uint32_t bs) {
  ENTER(ctx);
  REQUIRE(ndims <= 8, "at most 8 dimensions");
  size_t xstride[8], volume = 1;
  for (uint32_t i = 0; i < ndims; ++i) { xstride[i] = volume; volume *= dims[i]; }
  for (uint32_t b = 0; b < bs; ++b)
    for (size_t yi = 0; yi < volume; ++yi) {
      size_t rest = yi, xi = 0;
      for (uint32_t i = 0; i < ndims; ++i) {
        const uint32_t extent = dims[perm[i]];
        xi += (rest % extent) * xstride[perm[i]];
        rest /= extent;
      }
      const size_t X = b * volume + xi, Y = b * volume + yi;
      if (!backward) {
        narrow(widen(static_cast<const T *>(from)[X]), static_cast<T *>(to) + Y);
      } else {
        T *g = static_cast<T *>(to) + X;
        narrow(widen(*g) + widen(static_cast<const T *>(from)[Y]), g);
      }
    }
  return PHIP_OK;
}

template <class T>
int flip(phip_ctx *ctx, bool backward, const void *from, void *to, uint32_t base, uint32_t n, uint32_t outer) {
  ENTER(ctx);
  for (uint32_t o = 0; o < outer; ++o)
    for (uint32_t j = 0; j < n; ++j)
      for (uint32_t i = 0; i < base; ++i) {
        const size_t a = ((size_t)o * n + j) * base + i, r = ((size_t)o * n + (n - 1 - j)) * base + i;
        T *out = static_cast<T *>(to) + a;
        const float v = widen(static_cast<const T *>(from)[r]);
        narrow(backward ? widen(*out) + v : v, out);
      }
  return PHIP_OK;
}

template <class T>
int broadcast_fw(phip_ctx *ctx, const void *x, void *y, uint32_t base, uint32_t size, uint32_t outer) {
  ENTER(ctx);
  for (uint32_t o = 0; o < outer; ++o)
    for (uint32_t j = 0; j < size; ++j)
      for (uint32_t i = 0; i < base; ++i)
        narrow(widen(static_cast<const T *>(x)[(size_t)o * base + i]), static_cast<T *>(y) + ((size_t)o * size + j) * base + i);
  return PHIP_OK;
}

template <class T>
int reduce_fw(phip_ctx *ctx, int op, const void *x, void *y, uint32_t base, uint32_t n, uint32_t outer) {
  ENTER(ctx);
  const uint32_t dims[3] = {base, n, outer};
  auto vx = load<T>(x, (size_t)base * n * outer);
  std::vector<float> vy((size_t)base * outer);
  REQUIRE(ref_reduce_fw(op, vx.data(), dims, 3, 1, 1, vy.data()) == 0, "unknown reduction %d", op);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int extremum_bw(phip_ctx *ctx, int op, const void *x, const void *y, const void *gy, void *gx, uint32_t base,
                uint32_t n, uint32_t outer) {
  ENTER(ctx);
  REQUIRE(op == PHIP_MAX || op == PHIP_MIN, "not an extremum: %d", op);
  const uint32_t dims[3] = {base, n, outer};
  const size_t nx = (size_t)base * n * outer, ny = (size_t)base * outer;
  auto vx = load<T>(x, nx), vy = load<T>(y, ny), vgy = load<T>(gy, ny), vgx = load<T>(gx, nx);
  ref_extremum_bw(vx.data(), vy.data(), vgy.data(), dims, 3, 1, 1, vgx.data());
  store<T>(vgx, gx);
  return PHIP_OK;
}
template <class T>
int arg_extremum(phip_ctx *ctx, int op, const void *x, uint32_t *host_out, uint32_t base, uint32_t n, uint32_t outer) {
  ENTER(ctx);
  REQUIRE(op == PHIP_MAX || op == PHIP_MIN, "not an extremum: %d", op);
  const uint32_t dims[3] = {base, n, outer};
  auto vx = load<T>(x, (size_t)base * n * outer);
  ref_arg_extremum(op == PHIP_MAX, vx.data(), dims, 3, 1, 1, host_out);
  return PHIP_OK;
}

template <class T>
int random_fill(phip_ctx *ctx, int kind, uint64_t seed, uint64_t offset, float p0, float p1, void *y, size_t n) {
  ENTER(ctx);
  std::vector<float> v(n);
  REQUIRE(ref_random(kind, seed, offset, p0, p1, v.data(), n) == 0, "unknown distribution %d", kind);
  store<T>(v, y);
  return PHIP_OK;
}

uint32_t conv_extent(uint32_t x, uint32_t w, uint32_t pad, uint32_t str, uint32_t dil) {
  return (x + 2 * pad - ((w - 1) * dil + 1)) / str + 1;
}

template <class T>
int conv2d_fw(phip_ctx *ctx, const void *x, const void *w, void *y, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0,
              uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0,
              uint32_t str1, uint32_t dil0, uint32_t dil1) {
  ENTER(ctx);
  const size_t ny = (size_t)conv_extent(x0, w0, pad0, str0, dil0) * conv_extent(x1, w1, pad1, str1, dil1) * oc *
                    std::max(bx, bw);
  auto vx = load<T>(x, (size_t)x0 * x1 * c * bx), vw = load<T>(w, (size_t)w0 * w1 * c * oc * bw);
  std::vector<float> vy(ny);
  ref_conv2d_fw(vx.data(), vw.data(), vy.data(), x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int conv2d_bw(phip_ctx *ctx, const void *x, const void *w, const void *gy, void *gx, void *gw, uint32_t x0,
              uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0,
              uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1) {
  ENTER(ctx);
  const size_t nx = (size_t)x0 * x1 * c * bx, nw = (size_t)w0 * w1 * c * oc * bw;
  const size_t ny = (size_t)conv_extent(x0, w0, pad0, str0, dil0) * conv_extent(x1, w1, pad1, str1, dil1) * oc *
                    std::max(bx, bw);
  auto vx = load<T>(x, nx), vw = load<T>(w, nw), vgy = load<T>(gy, ny), vgx = load<T>(gx, nx), vgw = load<T>(gw, nw);
  ref_conv2d_bw(vx.data(), vw.data(), vgy.data(), vgx.data(), vgw.data(), x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1,
                str0, str1, dil0, dil1);
  store<T>(vgx, gx);
  store<T>(vgw, gw);
  return PHIP_OK;
}
template <class T>
int max_pool2d_fw(phip_ctx *ctx, const void *x, void *y, uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0,
                  uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1) {
  ENTER(ctx);
  const size_t ny = (size_t)conv_extent(x0, win0, pad0, str0, 1) * conv_extent(x1, win1, pad1, str1, 1) * repeat;
  auto vx = load<T>(x, (size_t)x0 * x1 * repeat);
  std::vector<float> vy(ny);
  ref_max_pool2d_fw(vx.data(), vy.data(), x0, x1, repeat, win0, win1, pad0, pad1, str0, str1);
  store<T>(vy, y);
  return PHIP_OK;
}
template <class T>
int max_pool2d_bw(phip_ctx *ctx, const void *x, const void *y, const void *gy, void *gx, uint32_t x0, uint32_t x1,
                  uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, uint32_t pad1, uint32_t str0,
                  uint32_t str1) {
  ENTER(ctx);
  const size_t nx = (size_t)x0 * x1 * repeat;
  const size_t ny = (size_t)conv_extent(x0, win0, pad0, str0, 1) * conv_extent(x1, win1, pad1, str1, 1) * repeat;
  auto vx = load<T>(x, nx), vy = load<T>(y, ny), vgy = load<T>(gy, ny), vgx = load<T>(gx, nx);
  ref_max_pool2d_bw(vx.data(), vy.data(), vgy.data(), vgx.data(), x0, x1, repeat, win0, win1, pad0, pad1, str0, str1);
  store<T>(vgx, gx);
  return PHIP_OK;
}

}  // namespace

extern "C" {

// ---- stub-only controls ----------------------------------------------------------
void phip_stub_set_memory_limit(uint64_t bytes) {
  std::lock_guard<std::mutex> lock(g_mutex);
  g_limit_bytes = bytes == 0 ? ~size_t(0) : (size_t)bytes;
}
void phip_stub_stats(uint64_t *live_bytes, uint64_t *live_blocks, uint64_t *malloc_calls, uint64_t *failed_mallocs,
                     uint64_t *release_calls, int *live_contexts) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (live_bytes) *live_bytes = g_live_bytes;
  if (live_blocks) *live_blocks = g_blocks.size();
  if (malloc_calls) *malloc_calls = g_malloc_calls;
  if (failed_mallocs) *failed_mallocs = g_failed_mallocs;
  if (release_calls) *release_calls = g_release_calls;
  if (live_contexts) *live_contexts = g_live_contexts;
}

// ---- runtime ------------------------------------------------------------------------
const char *phip_last_error(void) { return g_error; }

int phip_device_count(int *count) {
  REQUIRE(count != nullptr, "null count");
  *count = kDevices;
  return PHIP_OK;
}
int phip_check_support(int device_id) {
  REQUIRE(device_id >= 0 && device_id < kDevices, "Invalid device ID: %d", device_id);
  return PHIP_OK;
}
int phip_ctx_create(int device_id, phip_ctx **out) {
  REQUIRE(out != nullptr, "null output pointer");
  *out = nullptr;
  int rc = phip_check_support(device_id);
  if (rc != PHIP_OK) return rc;
  std::lock_guard<std::mutex> lock(g_mutex);
  *out = new phip_ctx{device_id, g_next_ctx++};
  ++g_live_contexts;
  return PHIP_OK;
}
int phip_ctx_destroy(phip_ctx *ctx) {
  ENTER(ctx);
  std::lock_guard<std::mutex> lock(g_mutex);
  --g_live_contexts;
  delete ctx;
  return PHIP_OK;
}
uint64_t phip_ctx_id(const phip_ctx *ctx) { return ctx ? ctx->id : 0; }
int phip_device_info_get(phip_ctx *ctx, phip_device_info *out) {
  ENTER(ctx);
  REQUIRE(out != nullptr, "null argument");
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->name, sizeof(out->name), "host stand-in for libphip");
  std::snprintf(out->arch, sizeof(out->arch), "host");
  out->wavefront_size = 64;
  return PHIP_OK;
}
int phip_describe(phip_ctx *ctx, char *buf, size_t buf_size) {
  ENTER(ctx);
  REQUIRE(buf != nullptr && buf_size > 0, "null argument");
  std::snprintf(buf, buf_size, "Device %p\n  Type: HIP (host stand-in)\n", static_cast<void *>(ctx));
  return PHIP_OK;
}
int phip_sync(phip_ctx *ctx) {
  ENTER(ctx);
  return PHIP_OK;
}
int phip_set_deterministic(phip_ctx *ctx, int) {
  ENTER(ctx);  // the stand-in adds in one fixed order anyway
  return PHIP_OK;
}
int phip_set_overlap(phip_ctx *ctx, int) {
  ENTER(ctx);  // the stand-in runs every call at once, in order
  return PHIP_OK;
}

int phip_malloc(phip_ctx *ctx, size_t bytes, void **out) {
  ENTER(ctx);
  REQUIRE(out != nullptr, "null output pointer");
  *out = nullptr;
  if (bytes == 0) return PHIP_OK;
  return device_alloc(bytes, out);
}
int phip_free(phip_ctx *ctx, void *ptr) {
  ENTER(ctx);
  if (ptr == nullptr) return PHIP_OK;
  return device_free(ptr);
}
int phip_pool_alloc(phip_ctx *ctx, size_t bytes, void **out, size_t *allocated) {
  ENTER(ctx);
  REQUIRE(out != nullptr, "null output pointer");
  *out = nullptr;
  if (allocated) *allocated = 0;
  if (bytes == 0) return PHIP_OK;
  size_t block = 8;
  while (block < bytes) block <<= 1;
  int rc = device_alloc(block, out);
  if (rc == PHIP_OK && allocated) *allocated = block;
  return rc;
}
int phip_pool_free(phip_ctx *ctx, void *ptr) {
  ENTER(ctx);
  if (ptr == nullptr) return PHIP_OK;
  return device_free(ptr);
}
int phip_pool_free_by_id(uint64_t, void *ptr) {
  if (ptr == nullptr) return PHIP_OK;
  return device_free(ptr);
}
int phip_pool_release_reserved(phip_ctx *ctx) {
  ENTER(ctx);
  std::lock_guard<std::mutex> lock(g_mutex);
  ++g_release_calls;  // the stand-in keeps no idle blocks
  return PHIP_OK;
}
int phip_pool_stats(phip_ctx *ctx, uint64_t *supplied_bytes, uint64_t *reserved_bytes) {
  ENTER(ctx);
  std::lock_guard<std::mutex> lock(g_mutex);
  if (supplied_bytes) *supplied_bytes = g_live_bytes;
  if (reserved_bytes) *reserved_bytes = 0;
  return PHIP_OK;
}

int phip_memcpy_h2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  ENTER(ctx);
  if (bytes == 0) return PHIP_OK;
  REQUIRE(dst && src, "null pointer in h2d copy");
  std::memcpy(dst, src, bytes);
  return PHIP_OK;
}
int phip_memcpy_d2h(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  ENTER(ctx);
  if (bytes == 0) return PHIP_OK;
  REQUIRE(dst && src, "null pointer in d2h copy");
  std::memcpy(dst, src, bytes);
  return PHIP_OK;
}
int phip_memcpy_d2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  ENTER(ctx);
  if (bytes == 0) return PHIP_OK;
  REQUIRE(dst && src, "null pointer in d2d copy");
  std::memmove(dst, src, bytes);
  return PHIP_OK;
}

int phip_event_create(phip_ctx *ctx, phip_event **out) {
  ENTER(ctx);
  REQUIRE(out != nullptr, "null output pointer");
  *out = new phip_event{0};
  return PHIP_OK;
}
int phip_event_destroy(phip_event *ev) {
  delete ev;
  return PHIP_OK;
}
int phip_event_record(phip_ctx *ctx, phip_event *ev) {
  ENTER(ctx);
  REQUIRE(ev != nullptr, "null event");
  return PHIP_OK;
}
int phip_event_elapsed_ms(phip_event *start, phip_event *stop, float *ms) {
  REQUIRE(start && stop && ms, "null argument");
  *ms = 0.0f;
  return PHIP_OK;
}

int phip_randomizer_create(uint32_t seed, phip_randomizer **out) {
  REQUIRE(out != nullptr, "null output pointer");
  *out = new phip_randomizer{std::mt19937(seed)};
  return PHIP_OK;
}
int phip_randomizer_destroy(phip_randomizer *r) {
  delete r;
  return PHIP_OK;
}
int phip_randomizer_fill_uniform(phip_randomizer *r, float lower, float upper, size_t n, float *host_out) {
  REQUIRE(r != nullptr && (host_out != nullptr || n == 0) && lower < upper, "bad argument");
  std::uniform_real_distribution<float> dist(lower, upper);
  const float lower_eps = std::nextafter(lower, upper);
  for (size_t i = 0; i < n; ++i) {
    const float x = dist(r->rng);
    host_out[i] = x < lower_eps ? upper : x;
  }
  return PHIP_OK;
}
int phip_randomizer_fill_normal(phip_randomizer *r, float mean, float sd, size_t n, float *host_out) {
  REQUIRE(r != nullptr && (host_out != nullptr || n == 0) && sd > 0.0f, "bad argument");
  std::normal_distribution<float> dist(mean, sd);
  for (size_t i = 0; i < n; ++i) host_out[i] = dist(r->rng);
  return PHIP_OK;
}

// ---- fill and storage conversion ------------------------------------------------------
int phip_fill_f32(phip_ctx *c, float *p, float v, size_t n) { return fill<float>(c, p, v, n); }
int phip_fill_f16(phip_ctx *c, void *p, float v, size_t n) { return fill<F16>(c, p, v, n); }
int phip_fill_bf16(phip_ctx *c, void *p, float v, size_t n) { return fill<BF16>(c, p, v, n); }
int phip_cvt_f32_to_f16(phip_ctx *c, const float *s, void *d, size_t n) { return cvt<float, F16>(c, s, d, n); }
int phip_cvt_f16_to_f32(phip_ctx *c, const void *s, float *d, size_t n) { return cvt<F16, float>(c, s, d, n); }
int phip_cvt_f32_to_bf16(phip_ctx *c, const float *s, void *d, size_t n) { return cvt<float, BF16>(c, s, d, n); }
int phip_cvt_bf16_to_f32(phip_ctx *c, const void *s, float *d, size_t n) { return cvt<BF16, float>(c, s, d, n); }

// One entry per storage type: NAME_f32 takes float pointers, the 16-bit ones void pointers.
// CP / MP: const / mutable pointer type of the variant; the lists spell the parameters and how
// they are forwarded to the typed body.
#define PHIP_STUB3(NAME, BODY, PARAMS, ARGS)                                            \
  int NAME##_f32 PARAMS(const float *, float *) { return BODY<float> ARGS; }            \
  int NAME##_f16 PARAMS(const void *, void *) { return BODY<F16> ARGS; }                \
  int NAME##_bf16 PARAMS(const void *, void *) { return BODY<BF16> ARGS; }

#define P_INPLACE(CP, MP) (phip_ctx *c, CP x, MP y, uint32_t volume, uint32_t bx, uint32_t by)
PHIP_STUB3(phip_inplace_add, inplace_add, P_INPLACE, (c, x, y, volume, bx, by))
PHIP_STUB3(phip_inplace_subtract, inplace_subtract, P_INPLACE, (c, x, y, volume, bx, by))
#define P_BATCH_SUM(CP, MP) (phip_ctx *c, CP x, MP y, uint32_t volume, uint32_t bs)
PHIP_STUB3(phip_batch_sum, batch_sum, P_BATCH_SUM, (c, x, y, volume, bs))
#define P_MM_FW(CP, MP) (phip_ctx *c, CP a, CP b, MP y, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb)
PHIP_STUB3(phip_matmul_fw, matmul_fw, P_MM_FW, (c, a, b, y, di, dj, dk, ba, bb))
#define P_MM_BW(CP, MP) \
  (phip_ctx *c, CP a, CP b, CP gy, MP ga, MP gb, uint32_t di, uint32_t dj, uint32_t dk, uint32_t ba, uint32_t bb)
PHIP_STUB3(phip_matmul_bw, matmul_bw, P_MM_BW, (c, a, b, gy, ga, gb, di, dj, dk, ba, bb))

#define P_UNARY_FW(CP, MP) (phip_ctx *c, int op, CP x, MP y, size_t n)
PHIP_STUB3(phip_unary_fw, unary_fw, P_UNARY_FW, (c, op, x, y, n))
#define P_UNARY_BW(CP, MP) (phip_ctx *c, int op, CP x, CP y, CP gy, MP gx, size_t n)
PHIP_STUB3(phip_unary_bw, unary_bw, P_UNARY_BW, (c, op, x, y, gy, gx, n))
#define P_CONST_FW(CP, MP) (phip_ctx *c, int op, CP x, float k, MP y, size_t n)
PHIP_STUB3(phip_const_fw, const_fw, P_CONST_FW, (c, op, x, k, y, n))
#define P_CONST_BW(CP, MP) (phip_ctx *c, int op, CP x, CP y, CP gy, float k, MP gx, size_t n)
PHIP_STUB3(phip_const_bw, const_bw, P_CONST_BW, (c, op, x, y, gy, k, gx, n))
#define P_POWN_FW(CP, MP) (phip_ctx *c, CP x, int32_t k, MP y, size_t n)
PHIP_STUB3(phip_pown_fw, pown_fw, P_POWN_FW, (c, x, k, y, n))
#define P_POWN_BW(CP, MP) (phip_ctx *c, CP x, CP y, CP gy, int32_t k, MP gx, size_t n)
PHIP_STUB3(phip_pown_bw, pown_bw, P_POWN_BW, (c, x, y, gy, k, gx, n))
#define P_BINARY_FW(CP, MP) (phip_ctx *c, int op, CP a, CP b, MP y, uint32_t volume, uint32_t ba, uint32_t bb)
PHIP_STUB3(phip_binary_fw, binary_fw, P_BINARY_FW, (c, op, a, b, y, volume, ba, bb))
#define P_BINARY_BW(CP, MP) \
  (phip_ctx *c, int op, CP a, CP b, CP y, CP gy, MP ga, MP gb, uint32_t volume, uint32_t ba, uint32_t bb)
PHIP_STUB3(phip_binary_bw, binary_bw, P_BINARY_BW, (c, op, a, b, y, gy, ga, gb, volume, ba, bb))
#define P_SCALAR_FW(CP, MP) \
  (phip_ctx *c, int op, int k_on_left, CP x, CP k, MP y, uint32_t volume, uint32_t bx, uint32_t bk)
PHIP_STUB3(phip_scalar_fw, scalar_fw, P_SCALAR_FW, (c, op, k_on_left, x, k, y, volume, bx, bk))
#define P_MUL_CONST(CP, MP) (phip_ctx *c, float k, MP x, size_t n)
PHIP_STUB3(phip_inplace_multiply_const, inplace_multiply_const, P_MUL_CONST, (c, k, x, n))
#define P_IDENTITY(CP, MP) (phip_ctx *c, MP y, uint32_t rows)
PHIP_STUB3(phip_identity, identity, P_IDENTITY, (c, y, rows))

#define P_COPY_ROWS(CP, MP)                                                                                  \
  (phip_ctx *c, CP src, MP dst, uint32_t span, uint32_t rows, uint64_t ss, uint64_t ds, uint32_t bs, uint64_t sbs, \
   uint64_t dbs, int accumulate)
PHIP_STUB3(phip_copy_rows, copy_rows, P_COPY_ROWS, (c, src, dst, span, rows, ss, ds, bs, sbs, dbs, accumulate))
#define P_PICK(CP, MP) \
  (phip_ctx *c, CP from, const uint32_t *ids, uint32_t n_ids, MP to, uint32_t base, uint32_t n, uint32_t outer, uint32_t bx, uint32_t bs)
PHIP_STUB3(phip_pick_fw, pick, P_PICK, (c, false, from, ids, n_ids, to, base, n, outer, bx, bs))
PHIP_STUB3(phip_pick_bw, pick, P_PICK, (c, true, from, ids, n_ids, to, base, n, outer, bx, bs))
#define P_BATCH_PICK(CP, MP) (phip_ctx *c, CP from, const uint32_t *ids, uint32_t n_ids, MP to, uint32_t volume, uint32_t bx)
PHIP_STUB3(phip_batch_pick_fw, batch_pick, P_BATCH_PICK, (c, false, from, ids, n_ids, to, volume, bx))
PHIP_STUB3(phip_batch_pick_bw, batch_pick, P_BATCH_PICK, (c, true, from, ids, n_ids, to, volume, bx))
#define P_TRANSPOSE(CP, MP) (phip_ctx *c, CP from, MP to, uint32_t rows, uint32_t cols, uint32_t bs)
PHIP_STUB3(phip_transpose_fw, transpose, P_TRANSPOSE, (c, false, from, to, rows, cols, bs))
PHIP_STUB3(phip_transpose_bw, transpose, P_TRANSPOSE, (c, true, from, to, rows, cols, bs))
#define P_PERMUTE(CP, MP) (phip_ctx *c, CP from, MP to, uint32_t ndims, const uint32_t *dims, const uint32_t *perm, uint32_t bs)
PHIP_STUB3(phip_permute_dims_fw, permute_dims, P_PERMUTE, (c, false, from, to, ndims, dims, perm, bs))
PHIP_STUB3(phip_permute_dims_bw, permute_dims, P_PERMUTE, (c, true, from, to, ndims, dims, perm, bs))
#define P_FLIP(CP, MP) (phip_ctx *c, CP from, MP to, uint32_t base, uint32_t n, uint32_t outer)
PHIP_STUB3(phip_flip_fw, flip, P_FLIP, (c, false, from, to, base, n, outer))
PHIP_STUB3(phip_flip_bw, flip, P_FLIP, (c, true, from, to, base, n, outer))
#define P_BROADCAST(CP, MP) (phip_ctx *c, CP x, MP y, uint32_t base, uint32_t size, uint32_t outer)
PHIP_STUB3(phip_broadcast_fw, broadcast_fw, P_BROADCAST, (c, x, y, base, size, outer))
#define P_REDUCE(CP, MP) (phip_ctx *c, int op, CP x, MP y, uint32_t base, uint32_t n, uint32_t outer)
PHIP_STUB3(phip_reduce_fw, reduce_fw, P_REDUCE, (c, op, x, y, base, n, outer))
#define P_EXTREMUM_BW(CP, MP) (phip_ctx *c, int op, CP x, CP y, CP gy, MP gx, uint32_t base, uint32_t n, uint32_t outer)
PHIP_STUB3(phip_extremum_bw, extremum_bw, P_EXTREMUM_BW, (c, op, x, y, gy, gx, base, n, outer))
#define P_ARG(CP, MP) (phip_ctx *c, int op, CP x, uint32_t *host_out, uint32_t base, uint32_t n, uint32_t outer)
PHIP_STUB3(phip_arg_extremum, arg_extremum, P_ARG, (c, op, x, host_out, base, n, outer))

// distribution codes of oracle/ref_random.c: uniform 0, Bernoulli 1, normal 2, log-normal 3
#define P_RANDOM2(CP, MP) (phip_ctx *c, uint64_t seed, uint64_t offset, float p0, float p1, MP y, size_t n)
PHIP_STUB3(phip_random_uniform, random_fill, P_RANDOM2, (c, 0, seed, offset, p0, p1, y, n))
PHIP_STUB3(phip_random_normal, random_fill, P_RANDOM2, (c, 2, seed, offset, p0, p1, y, n))
PHIP_STUB3(phip_random_log_normal, random_fill, P_RANDOM2, (c, 3, seed, offset, p0, p1, y, n))
#define P_RANDOM1(CP, MP) (phip_ctx *c, uint64_t seed, uint64_t offset, float p, MP y, size_t n)
PHIP_STUB3(phip_random_bernoulli, random_fill, P_RANDOM1, (c, 1, seed, offset, p, 0.0f, y, n))

#define P_CONV_FW(CP, MP)                                                                                          \
  (phip_ctx *ctx, CP x, CP w, MP y, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, uint32_t oc,   \
   uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, uint32_t dil1)
PHIP_STUB3(phip_conv2d_fw, conv2d_fw, P_CONV_FW,
           (ctx, x, w, y, x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1))
#define P_CONV_BW(CP, MP)                                                                                        \
  (phip_ctx *ctx, CP x, CP w, CP gy, MP gx, MP gw, uint32_t x0, uint32_t x1, uint32_t c, uint32_t w0, uint32_t w1, \
   uint32_t oc, uint32_t bx, uint32_t bw, uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1, uint32_t dil0, \
   uint32_t dil1)
PHIP_STUB3(phip_conv2d_bw, conv2d_bw, P_CONV_BW,
           (ctx, x, w, gy, gx, gw, x0, x1, c, w0, w1, oc, bx, bw, pad0, pad1, str0, str1, dil0, dil1))
#define P_POOL_FW(CP, MP)                                                                                     \
  (phip_ctx *ctx, CP x, MP y, uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0, uint32_t win1, uint32_t pad0, \
   uint32_t pad1, uint32_t str0, uint32_t str1)
PHIP_STUB3(phip_max_pool2d_fw, max_pool2d_fw, P_POOL_FW, (ctx, x, y, x0, x1, repeat, win0, win1, pad0, pad1, str0, str1))
#define P_POOL_BW(CP, MP)                                                                                       \
  (phip_ctx *ctx, CP x, CP y, CP gy, MP gx, uint32_t x0, uint32_t x1, uint32_t repeat, uint32_t win0, uint32_t win1, \
   uint32_t pad0, uint32_t pad1, uint32_t str0, uint32_t str1)
PHIP_STUB3(phip_max_pool2d_bw, max_pool2d_bw, P_POOL_BW,
           (ctx, x, y, gy, gx, x0, x1, repeat, win0, win1, pad0, pad1, str0, str1))

int phip_set_deferred_zero_fill(phip_ctx *, int) { return PHIP_OK; }  // every fill runs at once here

int phip_gemm_trace(phip_ctx *, int, char *buf, size_t buf_size) {
  if (buf != nullptr && buf_size > 0) buf[0] = '\0';  // no kernels here
  return PHIP_OK;
}

int phip_matmul_fw_f32_noalloc(phip_ctx *c, const float *a, const float *b, float *y, uint32_t di, uint32_t dj,
                               uint32_t dk, uint32_t ba, uint32_t bb) {
  return matmul_fw<float>(c, a, b, y, di, dj, dk, ba, bb);
}

}  // extern "C"
