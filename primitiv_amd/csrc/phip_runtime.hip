// Contexts, the device memory pool, copies, events and the host randomizer.
#include <atomic>
#include <cstdlib>
#include <cstring>
#include <random>
#include <cmath>
#include <string>

#include "phip_internal.h"

namespace phip {

static thread_local char g_error[1024] = "";

int fail(int code, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return code;
}

// Registry of live contexts, so that a handle deleter can ask whether the
// pool it came from still exists.
static std::mutex g_registry_mutex;
static std::unordered_map<uint64_t, phip_ctx *> g_registry;
static std::atomic<uint64_t> g_next_id{1};

// Scratch of the allocation-free entry points: tile counters, then kFixedScratchBytes
// for partial tiles and operand copies.  Every GPU holds its own copy of the array
// at its own address until the process ends; `scratch` itself is only the host-side
// name of the symbol, g_fixed_scratch[device] the device address.  Device arrays
// start zeroed, and every launch leaves the counters it used zeroed again.
constexpr size_t kFixedTicketBytes = sizeof(uint32_t) * kTicketSlots;
static __device__ __align__(256) unsigned char scratch[kFixedTicketBytes + kFixedScratchBytes];
constexpr int kMaxDevices = 64;
static std::mutex g_fixed_scratch_mutex;
static unsigned char *g_fixed_scratch[kMaxDevices] = {};

// Device address of this device's copy of `scratch`; looked up once per device, with that device current.
static int fixed_scratch_of(int device, unsigned char **out) {
  *out = nullptr;
  if (device < 0 || device >= kMaxDevices) return PHIP_OK;  // no allocation-free calls on such a device
  std::lock_guard<std::mutex> lock(g_fixed_scratch_mutex);
  if (g_fixed_scratch[device] == nullptr) {
    PHIP_HIP(hipSetDevice(device));
    void *ptr = nullptr;
    PHIP_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    g_fixed_scratch[device] = static_cast<unsigned char *>(ptr);
  }
  *out = g_fixed_scratch[device];
  return PHIP_OK;
}

static int pool_alloc_from(phip_ctx *ctx, Pool &pool, size_t bytes, void **out, size_t *allocated);
static int pool_free_locked(phip_ctx *ctx, Pool &pool, void *ptr);

int scratch_alloc(phip_ctx *ctx, size_t bytes, void **out) {
  if (!ctx->fixed_mode) return pool_alloc_from(ctx, ctx->scratch_pool, bytes, out, nullptr);
  *out = nullptr;
  const size_t start = (ctx->fixed_used + 255) / 256 * 256;
  if (bytes > kFixedScratchBytes || start > kFixedScratchBytes - bytes) {
    return fail(PHIP_ERR_INVALID_ARGUMENT,
                "this product needs %zu bytes of scratch memory on top of %zu; an allocation-free call has %zu",
                bytes, start, kFixedScratchBytes);
  }
  *out = ctx->fixed_scratch + kFixedTicketBytes + start;
  ctx->fixed_used = start + bytes;
  return PHIP_OK;
}

void scratch_free(phip_ctx *ctx, void *ptr) {
  if (ptr == nullptr) return;
  const unsigned char *p = static_cast<const unsigned char *>(ptr);
  if (ctx->fixed_scratch && p >= ctx->fixed_scratch && p < ctx->fixed_scratch + kFixedTicketBytes + kFixedScratchBytes) return;
  std::lock_guard<std::mutex> lock(ctx->mutex);
  (void)pool_free_locked(ctx, ctx->scratch_pool, ptr);
}

uint32_t *tile_tickets(phip_ctx *ctx) {
  return ctx->fixed_mode ? reinterpret_cast<uint32_t *>(ctx->fixed_scratch) : ctx->tile_tickets;
}

static unsigned ceil_log2(uint64_t x) {
  unsigned s = 0;
  while ((1ull << s) < x) ++s;
  return s;
}

static int release_reserved_locked(phip_ctx *ctx) {
  int rc = PHIP_OK;
  for (Pool *pool : {&ctx->pool, &ctx->scratch_pool}) {
    for (auto &list : pool->reserved) {
      while (!list.empty()) {
        if (hipFree(list.back()) != hipSuccess) {
          rc = fail(PHIP_ERR_RUNTIME, "hipFree failed while releasing pool blocks");
        }
        list.pop_back();
      }
    }
  }
  return rc;
}

// Drains and empties the free lists of every live context on `device`.  Takes the
// registry's lock, then each context's: the caller holds neither.
static void release_reserved_on_device(int device) {
  std::lock_guard<std::mutex> reg(g_registry_mutex);
  for (auto &kv : g_registry) {
    phip_ctx *c = kv.second;
    if (c->device != device) continue;
    // idle blocks may still be read by kernels enqueued before they were freed
    (void)hipStreamSynchronize(c->stream);
    std::lock_guard<std::mutex> lock(c->mutex);
    (void)release_reserved_locked(c);
  }
}

static void zeros_drop_locked(phip_ctx *ctx, const void *p, size_t bytes) {
  if (ctx->zeros.empty()) return;
  const uintptr_t lo = reinterpret_cast<uintptr_t>(p), hi = lo + bytes;
  size_t kept = 0;
  for (const PendingZero &z : ctx->zeros) {
    if (!(z.lo >= lo && z.lo + z.bytes <= hi)) ctx->zeros[kept++] = z;
  }
  ctx->zeros.resize(kept);
  ctx->zeros_count.store((int)kept, std::memory_order_relaxed);
}

void zeros_drop(phip_ctx *ctx, const void *p, size_t bytes) {
  std::lock_guard<std::mutex> lock(ctx->mutex);
  zeros_drop_locked(ctx, p, bytes);
}

bool zeros_take(phip_ctx *ctx, const void *p, size_t bytes) {
  if (ctx->zeros_count.load(std::memory_order_relaxed) == 0) return false;
  std::lock_guard<std::mutex> lock(ctx->mutex);
  const uintptr_t lo = reinterpret_cast<uintptr_t>(p);
  for (size_t i = 0; i < ctx->zeros.size(); ++i) {
    if (ctx->zeros[i].lo == lo && ctx->zeros[i].bytes == bytes) {
      ctx->zeros.erase(ctx->zeros.begin() + (long)i);
      ctx->zeros_count.store((int)ctx->zeros.size(), std::memory_order_relaxed);
      return true;
    }
  }
  return false;
}

static int pool_free_locked(phip_ctx *ctx, Pool &pool, void *ptr) {
  auto it = pool.supplied.find(ptr);
  if (it == pool.supplied.end()) {
    return fail(PHIP_ERR_INVALID_ARGUMENT, "Detected to dispose unknown handle: %p", ptr);
  }
  // whatever the block was to be filled with no longer matters
  zeros_drop_locked(ctx, ptr, (size_t)1 << it->second);
  pool.reserved[it->second].push_back(ptr);
  pool.supplied.erase(it);
  return PHIP_OK;
}

// A block of at least `bytes` (rounded up to a power of two) from `pool`'s free lists or from hipMalloc.
static int pool_alloc_from(phip_ctx *ctx, Pool &pool, size_t bytes, void **out, size_t *allocated) {
  *out = nullptr;
  if (allocated) *allocated = 0;
  if (bytes == 0) return PHIP_OK;
  if (bytes < Pool::kMinimumSize) bytes = Pool::kMinimumSize;
  if (bytes > (1ull << 62)) {
    return fail(PHIP_ERR_INVALID_ARGUMENT, "Invalid memory size: %zu", bytes);
  }
  const unsigned shift = ceil_log2(bytes);
  const size_t block = 1ull << shift;
  void *ptr = nullptr;
  {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    auto &list = pool.reserved[shift];
    if (!list.empty()) {
      ptr = list.back();
      list.pop_back();
    }
  }
  if (ptr == nullptr) {
    hipError_t e = hipMalloc(&ptr, block);
    if (e != hipSuccess) {
      // Most likely out of memory: give back every idle block of every context on this GPU (a fp32 and a
      // 16-bit device object on one GPU each have a pool) and try again.
      (void)hipGetLastError();
      release_reserved_on_device(ctx->device);
      e = hipMalloc(&ptr, block);
    }
    if (e != hipSuccess) {
      (void)hipGetLastError();
      return fail(e == hipErrorOutOfMemory ? PHIP_ERR_OUT_OF_MEMORY : PHIP_ERR_RUNTIME,
                  "Memory allocation failed. Requested size: %zu (%s)", block,
                  hipGetErrorString(e));
    }
  }
  {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    pool.supplied.emplace(ptr, shift);
  }
  *out = ptr;
  if (allocated) *allocated = block;
  return PHIP_OK;
}

int ctx_create(int device_id, bool with_lanes, phip_ctx **out) {
  PHIP_REQUIRE(out != nullptr, "null output pointer");
  *out = nullptr;
  int rc = phip_check_support(device_id);
  if (rc != PHIP_OK) return rc;
  PHIP_HIP(hipSetDevice(device_id));
  phip_ctx *ctx = new phip_ctx();
  ctx->device = device_id;
  rc = phip::fixed_scratch_of(device_id, &ctx->fixed_scratch);
  if (rc != PHIP_OK) {
    delete ctx;
    return rc;
  }
  hipError_t e = hipGetDeviceProperties(&ctx->prop, device_id);
  if (e == hipSuccess) e = hipStreamCreateWithFlags(&ctx->stream, hipStreamNonBlocking);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&ctx->tile_tickets), sizeof(uint32_t) * phip::kTicketSlots);
  if (e == hipSuccess) e = hipMemset(ctx->tile_tickets, 0, sizeof(uint32_t) * phip::kTicketSlots);
  if (e != hipSuccess) {
    if (ctx->tile_tickets) (void)hipFree(ctx->tile_tickets);
    if (ctx->stream) (void)hipStreamDestroy(ctx->stream);
    delete ctx;
    return fail(PHIP_ERR_RUNTIME, "context creation failed: %s", hipGetErrorString(e));
  }
  {
    const char *v = std::getenv("PHIP_DEFER_ZERO_FILLS");
    ctx->defer_zero_fills = !(v != nullptr && v[0] == '0');
    ctx->zeros.reserve(16);
  }
  ctx->id = phip::g_next_id.fetch_add(1);
  {
    std::lock_guard<std::mutex> lock(phip::g_registry_mutex);
    phip::g_registry.emplace(ctx->id, ctx);
  }
  if (with_lanes) {
    rc = phip::lanes_create(ctx);
    if (rc != PHIP_OK) {
      (void)phip_ctx_destroy(ctx);
      return rc;
    }
  }
  *out = ctx;
  return PHIP_OK;
}

}  // namespace phip

using phip::fail;

extern "C" {

const char *phip_last_error(void) { return phip::g_error; }

int phip_device_count(int *count) {
  PHIP_REQUIRE(count != nullptr, "null count");
  *count = 0;
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e == hipErrorNoDevice) {
    (void)hipGetLastError();
    return PHIP_OK;
  }
  PHIP_HIP(e);
  *count = n;
  return PHIP_OK;
}

int phip_check_support(int device_id) {
  int n = 0;
  int rc = phip_device_count(&n);
  if (rc != PHIP_OK) return rc;
  PHIP_REQUIRE(device_id >= 0 && device_id < n, "Invalid device ID: %d", device_id);
  hipDeviceProp_t prop;
  PHIP_HIP(hipGetDeviceProperties(&prop, device_id));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
    return fail(PHIP_ERR_UNSUPPORTED,
                "HIP device %d is %s; this backend contains gfx950 (MI355X) code only",
                device_id, prop.gcnArchName);
  }
  if (prop.totalGlobalMem < (1ull << 30)) {
    return fail(PHIP_ERR_UNSUPPORTED, "HIP device %d has less than 1 GiB of memory", device_id);
  }
  if (prop.warpSize != 64) {
    return fail(PHIP_ERR_UNSUPPORTED, "HIP device %d does not run 64-wide wavefronts", device_id);
  }
  return PHIP_OK;
}

int phip_ctx_create(int device_id, phip_ctx **out) { return phip::ctx_create(device_id, true, out); }

int phip_ctx_destroy(phip_ctx *ctx) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  const int lanes_rc = phip::lanes_destroy(ctx);  // waits for the side lane
  {
    std::lock_guard<std::mutex> lock(phip::g_registry_mutex);
    phip::g_registry.erase(ctx->id);
  }
  int rc = lanes_rc;
  {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    ctx->zeros.clear();  // fills nobody will read
    ctx->zeros_count.store(0, std::memory_order_relaxed);
  }
  if (hipSetDevice(ctx->device) != hipSuccess ||
      hipStreamSynchronize(ctx->stream) != hipSuccess) {
    rc = fail(PHIP_ERR_RUNTIME, "synchronisation failed while destroying the context");
  }
  {
    std::lock_guard<std::mutex> lock(ctx->mutex);
    // Blocks still handed out are freed too: handles may outlive the device.
    for (phip::Pool *pool : {&ctx->pool, &ctx->scratch_pool}) {
      for (auto &kv : pool->supplied) {
        if (hipFree(kv.first) != hipSuccess) rc = fail(PHIP_ERR_RUNTIME, "hipFree failed");
      }
      pool->supplied.clear();
    }
    int r2 = phip::release_reserved_locked(ctx);
    if (r2 != PHIP_OK) rc = r2;
  }
  if (ctx->tile_tickets && hipFree(ctx->tile_tickets) != hipSuccess) rc = fail(PHIP_ERR_RUNTIME, "hipFree failed");
  if (hipStreamDestroy(ctx->stream) != hipSuccess) {
    rc = fail(PHIP_ERR_RUNTIME, "hipStreamDestroy failed");
  }
  delete ctx;
  return rc;
}

uint64_t phip_ctx_id(const phip_ctx *ctx) { return ctx ? ctx->id : 0; }

int phip_device_info_get(phip_ctx *ctx, phip_device_info *out) {
  PHIP_REQUIRE(ctx != nullptr && out != nullptr, "null argument");
  std::memset(out, 0, sizeof(*out));
  const hipDeviceProp_t &p = ctx->prop;
  std::snprintf(out->name, sizeof(out->name), "%s", p.name);
  std::snprintf(out->arch, sizeof(out->arch), "%s", p.gcnArchName);
  out->device_id = ctx->device;
  out->compute_units = p.multiProcessorCount;
  out->clock_mhz = p.clockRate / 1000;
  out->memory_clock_mhz = p.memoryClockRate / 1000;
  out->memory_bus_bits = p.memoryBusWidth;
  out->wavefront_size = p.warpSize;
  out->lds_bytes_per_workgroup = static_cast<int32_t>(p.sharedMemPerBlock);
  out->l2_bytes = p.l2CacheSize;
  out->global_memory_bytes = p.totalGlobalMem;
  return PHIP_OK;
}

int phip_describe(phip_ctx *ctx, char *buf, size_t buf_size) {
  PHIP_REQUIRE(ctx != nullptr && buf != nullptr && buf_size > 0, "null argument");
  const hipDeviceProp_t &p = ctx->prop;
  std::snprintf(
      buf, buf_size,
      "Device %p\n"
      "  Type: HIP\n"
      "  Device ID: %d\n"
      "    Name ................. %s\n"
      "    Architecture ......... %s\n"
      "    Global memory ........ %llu\n"
      "    LDS per workgroup .... %zu\n"
      "    Compute units ........ %d\n"
      "    Wavefront size ....... %d\n"
      "    Engine clock (kHz) ... %d\n"
      "    Memory clock (kHz) ... %d\n"
      "    Memory bus (bits) .... %d\n"
      "    L2 cache ............. %d\n",
      static_cast<void *>(ctx), ctx->device, p.name, p.gcnArchName,
      static_cast<unsigned long long>(p.totalGlobalMem), p.sharedMemPerBlock,
      p.multiProcessorCount, p.warpSize, p.clockRate, p.memoryClockRate,
      p.memoryBusWidth, p.l2CacheSize);
  return PHIP_OK;
}

int phip_set_deterministic(phip_ctx *ctx, int on) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  ctx->deterministic = on != 0;
  return PHIP_OK;
}

int phip_set_deferred_zero_fill(phip_ctx *ctx, int on) {
  PHIP_ENTER(ctx);  // launches what is noted
  ctx->defer_zero_fills = on != 0;
  return PHIP_OK;
}

int phip_sync(phip_ctx *ctx) {
  PHIP_ENTER_BLOCKING(ctx);
  PHIP_HIP(hipStreamSynchronize(ctx->stream));
  return PHIP_OK;
}

// ---- raw memory ---------------------------------------------------------------

int phip_malloc(phip_ctx *ctx, size_t bytes, void **out) {
  PHIP_ENTER_HOST(ctx);
  PHIP_REQUIRE(out != nullptr, "null output pointer");
  *out = nullptr;
  if (bytes == 0) return PHIP_OK;
  hipError_t e = hipMalloc(out, bytes);
  if (e == hipErrorOutOfMemory) {
    // the scratch pools of this GPU's contexts may hold idle blocks (powers of two, up to GiBs)
    (void)hipGetLastError();
    phip::release_reserved_on_device(ctx->device);
    e = hipMalloc(out, bytes);
  }
  if (e != hipSuccess) {
    (void)hipGetLastError();
    *out = nullptr;
    return fail(e == hipErrorOutOfMemory ? PHIP_ERR_OUT_OF_MEMORY : PHIP_ERR_RUNTIME,
                "hipMalloc(%zu) failed: %s", bytes, hipGetErrorString(e));
  }
  return PHIP_OK;
}

int phip_free(phip_ctx *ctx, void *ptr) {
  PHIP_ENTER_HOST(ctx);
  if (ptr == nullptr) return PHIP_OK;
  PHIP_FLUSH_ZEROS(ctx);  // a noted fill of this memory must not be launched after it is gone
  PHIP_HIP(hipFree(ptr));
  return PHIP_OK;
}

// ---- pool ---------------------------------------------------------------------

int phip_pool_alloc(phip_ctx *ctx, size_t bytes, void **out, size_t *allocated) {
  PHIP_ENTER_HOST(ctx);
  PHIP_REQUIRE(out != nullptr, "null output pointer");
  return phip::pool_alloc_from(ctx, ctx->pool, bytes, out, allocated);
}

int phip_pool_free(phip_ctx *ctx, void *ptr) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  if (ptr == nullptr) return PHIP_OK;
  std::lock_guard<std::mutex> lock(ctx->mutex);
  return phip::pool_free_locked(ctx, ctx->pool, ptr);
}

int phip_pool_free_by_id(uint64_t ctx_id, void *ptr) {
  if (ptr == nullptr) return PHIP_OK;
  std::lock_guard<std::mutex> reg(phip::g_registry_mutex);
  auto it = phip::g_registry.find(ctx_id);
  if (it == phip::g_registry.end()) return PHIP_OK;  // pool already gone
  std::lock_guard<std::mutex> lock(it->second->mutex);
  return phip::pool_free_locked(it->second, it->second->pool, ptr);
}

int phip_pool_release_reserved(phip_ctx *ctx) {
  PHIP_ENTER(ctx);
  // Idle blocks may still be read by kernels enqueued before they were freed.
  PHIP_HIP(hipStreamSynchronize(ctx->stream));
  if (ctx->lanes != nullptr) {
    const int rc = phip_pool_release_reserved(ctx->lanes->side);  // the side lane's scratch blocks
    if (rc != PHIP_OK) return rc;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);
  return phip::release_reserved_locked(ctx);
}

int phip_pool_stats(phip_ctx *ctx, uint64_t *supplied_bytes, uint64_t *reserved_bytes) {
  PHIP_REQUIRE(ctx != nullptr, "null context");
  std::lock_guard<std::mutex> lock(ctx->mutex);
  uint64_t s = 0, r = 0;
  for (const phip::Pool *pool : {&ctx->pool, &ctx->scratch_pool}) {
    for (auto &kv : pool->supplied) s += 1ull << kv.second;
    for (size_t i = 0; i < pool->reserved.size(); ++i) {
      r += (1ull << i) * pool->reserved[i].size();
    }
  }
  if (supplied_bytes) *supplied_bytes = s;
  if (reserved_bytes) *reserved_bytes = r;
  return PHIP_OK;
}

// ---- copies -------------------------------------------------------------------

int phip_memcpy_h2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  PHIP_ENTER_BLOCKING(ctx);
  if (bytes == 0) return PHIP_OK;
  PHIP_REQUIRE(dst != nullptr && src != nullptr, "null pointer in h2d copy");
  PHIP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, ctx->stream));
  PHIP_HIP(hipStreamSynchronize(ctx->stream));
  return PHIP_OK;
}

int phip_memcpy_d2h(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  PHIP_ENTER_BLOCKING(ctx);
  if (bytes == 0) return PHIP_OK;
  PHIP_REQUIRE(dst != nullptr && src != nullptr, "null pointer in d2h copy");
  PHIP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, ctx->stream));
  PHIP_HIP(hipStreamSynchronize(ctx->stream));
  return PHIP_OK;
}

int phip_memcpy_d2d(phip_ctx *ctx, void *dst, const void *src, size_t bytes) {
  PHIP_ENTER(ctx);
  if (bytes == 0) return PHIP_OK;
  PHIP_REQUIRE(dst != nullptr && src != nullptr, "null pointer in d2d copy");
  PHIP_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, ctx->stream));
  return PHIP_OK;
}

// ---- events -------------------------------------------------------------------

int phip_event_create(phip_ctx *ctx, phip_event **out) {
  PHIP_ENTER_HOST(ctx);
  PHIP_REQUIRE(out != nullptr, "null output pointer");
  phip_event *ev = new phip_event();
  ev->device = ctx->device;
  hipError_t e = hipEventCreate(&ev->ev);
  if (e != hipSuccess) {
    delete ev;
    return fail(PHIP_ERR_RUNTIME, "hipEventCreate failed: %s", hipGetErrorString(e));
  }
  *out = ev;
  return PHIP_OK;
}

int phip_event_destroy(phip_event *ev) {
  if (ev == nullptr) return PHIP_OK;
  hipError_t e = hipEventDestroy(ev->ev);
  delete ev;
  if (e != hipSuccess) return fail(PHIP_ERR_RUNTIME, "hipEventDestroy failed");
  return PHIP_OK;
}

int phip_event_record(phip_ctx *ctx, phip_event *ev) {
  PHIP_ENTER_HOST(ctx);
  PHIP_FLUSH_ZEROS(ctx);
  PHIP_REQUIRE(ev != nullptr, "null event");
  if (ctx->lanes != nullptr) {
    const int rc = phip::lanes_order_main_after_side(ctx);
    if (rc != PHIP_OK) return rc;
  }
  PHIP_HIP(hipEventRecord(ev->ev, ctx->stream));
  return PHIP_OK;
}

int phip_event_elapsed_ms(phip_event *start, phip_event *stop, float *ms) {
  PHIP_REQUIRE(start && stop && ms, "null argument");
  PHIP_HIP(hipEventSynchronize(stop->ev));
  PHIP_HIP(hipEventElapsedTime(ms, start->ev, stop->ev));
  return PHIP_OK;
}

}  // extern "C"

// ---- host randomizer ------------------------------------------------------------

struct phip_randomizer {
  std::mt19937 rng;
  explicit phip_randomizer(uint32_t seed) : rng(seed) {}
};

extern "C" {

int phip_randomizer_create(uint32_t seed, phip_randomizer **out) {
  PHIP_REQUIRE(out != nullptr, "null output pointer");
  *out = new phip_randomizer(seed);
  return PHIP_OK;
}

int phip_randomizer_destroy(phip_randomizer *r) {
  delete r;
  return PHIP_OK;
}

int phip_randomizer_fill_uniform(phip_randomizer *r, float lower, float upper, size_t n,
                                 float *host_out) {
  PHIP_REQUIRE(r != nullptr && (host_out != nullptr || n == 0), "null argument");
  PHIP_REQUIRE(lower < upper, "uniform bounds must satisfy lower < upper");
  // One distribution object per fill; the open end is the lower one.
  std::uniform_real_distribution<float> dist(lower, upper);
  const float lower_eps = std::nextafter(lower, upper);
  for (size_t i = 0; i < n; ++i) {
    const float x = dist(r->rng);
    host_out[i] = x < lower_eps ? upper : x;
  }
  return PHIP_OK;
}

int phip_randomizer_fill_normal(phip_randomizer *r, float mean, float sd, size_t n,
                                float *host_out) {
  PHIP_REQUIRE(r != nullptr && (host_out != nullptr || n == 0), "null argument");
  PHIP_REQUIRE(sd > 0.0f, "standard deviation must be positive");
  std::normal_distribution<float> dist(mean, sd);
  for (size_t i = 0; i < n; ++i) host_out[i] = dist(r->rng);
  return PHIP_OK;
}

}  // extern "C"
