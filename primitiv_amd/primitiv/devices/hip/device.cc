// primitiv::devices::HIP: host side of the MI355X backend.  Built when
// PRIMITIV_USE_HIP is on; links against libphip (phip.h).

#include <primitiv/devices/hip/device.h>

#include <iostream>
#include <random>
#include <string>

#include <phip.h>

namespace {

// Turns a libphip status into primitiv::Error, as CUDA_CALL does for the
// CUDA runtime (primitiv/internal/cuda/utils.h:20-28).
#define PHIP_CALL(f) { \
  const int phip_status__ = (f); \
  if (phip_status__ != PHIP_OK) { \
    PRIMITIV_THROW_ERROR( \
        "libphip call failed. statement: " << #f \
        << ", status: " << phip_status__ << ": " << ::phip_last_error()); \
  } \
}

const char *suffix_name(primitiv::devices::HIP::Storage s) {
  switch (s) {
    case primitiv::devices::HIP::Storage::F16: return "fp16 storage, fp32 accumulation";
    case primitiv::devices::HIP::Storage::BF16: return "bf16 storage, fp32 accumulation";
    default: return "fp32";
  }
}

}  // namespace

namespace primitiv {
namespace devices {

std::uint32_t HIP::num_devices() {
  int n = 0;
  PHIP_CALL(::phip_device_count(&n));
  return static_cast<std::uint32_t>(n);
}

void HIP::assert_support(std::uint32_t device_id) {
  if (device_id >= num_devices()) {
    PRIMITIV_THROW_ERROR("Invalid device ID: " << device_id);
  }
  PHIP_CALL(::phip_check_support(static_cast<int>(device_id)));
}

bool HIP::check_support(std::uint32_t device_id) {
  try {
    assert_support(device_id);
  } catch (...) {
    return false;
  }
  return true;
}

HIP::HIP(std::uint32_t device_id, std::uint32_t rng_seed, Storage storage)
: dev_id_(device_id), rng_seed_(rng_seed), storage_(storage), ctx_(nullptr) {
  assert_support(dev_id_);
  PHIP_CALL(::phip_ctx_create(static_cast<int>(dev_id_), &ctx_));
  phip_ctx *ctx = ctx_;
  // The pool asks libphip for raw blocks; a failed allocation must throw so
  // that the pool releases its idle blocks and retries
  // (primitiv/core/memory_pool.cc:53-63).
  pool_.reset(new MemoryPool(
      [ctx](std::size_t size) -> void * {
        void *ptr = nullptr;
        PHIP_CALL(::phip_malloc(ctx, size, &ptr));
        return ptr;
      },
      [ctx](void *ptr) -> void {
        PHIP_CALL(::phip_free(ctx, ptr));
      },
      2 * sizeof(float)));
}

HIP::HIP(std::uint32_t device_id, std::uint32_t rng_seed)
: HIP(device_id, rng_seed, Storage::F32) {}

HIP::HIP(std::uint32_t device_id)
: HIP(device_id, std::random_device()(), Storage::F32) {}

HIP::~HIP() {
  // Blocks may still be in flight on the stream; drain it before the pool
  // hands them back, then drop the pool, then the context.
  if (ctx_) ::phip_sync(ctx_);
  pool_.reset();
  if (ctx_) ::phip_ctx_destroy(ctx_);
}

HIP16::HIP16(std::uint32_t device_id, std::uint32_t rng_seed)
: HIP(device_id, rng_seed, Storage::F16) {}

HIP16::HIP16(std::uint32_t device_id)
: HIP(device_id, std::random_device()(), Storage::F16) {}

void HIP::unsupported(const char *op) {
  PRIMITIV_THROW_NOT_IMPLEMENTED_WITH_MESSAGE(
      "devices::HIP implements the matmul path only; `" << op << "` is not available.");
}

void HIP::dump_description() const {
  char buf[2048];
  PHIP_CALL(::phip_describe(ctx_, buf, sizeof(buf)));
  std::cerr << buf << "  Storage: " << suffix_name(storage_) << std::endl;
}

std::size_t HIP::storage_bytes(std::size_t n) const {
  if (storage_ == Storage::F32) return sizeof(float) * n;
  return 2 * (n + (n & 1));
}

std::shared_ptr<void> HIP::new_handle(const Shape &shape, std::size_t *const allocated_size) {
  return pool_->allocate(storage_bytes(shape.size()), allocated_size);
}

std::vector<float> HIP::tensor_to_vector_impl(const Tensor &x) {
  const std::size_t n = x.shape().size();
  std::vector<float> ret(n);
  if (storage_ == Storage::F32) {
    PHIP_CALL(::phip_memcpy_d2h(ctx_, ret.data(), get_handle(x), sizeof(float) * n));
  } else {
    // widen on the device into a pooled fp32 block, then copy out
    std::shared_ptr<void> tmp = pool_->allocate(sizeof(float) * n);
    float *pt = static_cast<float *>(tmp.get());
    if (storage_ == Storage::F16) {
      PHIP_CALL(::phip_cvt_f16_to_f32(ctx_, get_handle(x), pt, n));
    } else {
      PHIP_CALL(::phip_cvt_bf16_to_f32(ctx_, get_handle(x), pt, n));
    }
    PHIP_CALL(::phip_memcpy_d2h(ctx_, ret.data(), pt, sizeof(float) * n));
  }
  return ret;
}

void HIP::reset_tensor_impl(float k, Tensor &x) {
  const std::size_t n = x.shape().size();
  void *px = get_mutable_handle(x);
  switch (storage_) {
    case Storage::F32: PHIP_CALL(::phip_fill_f32(ctx_, static_cast<float *>(px), k, n)); break;
    case Storage::F16: PHIP_CALL(::phip_fill_f16(ctx_, px, k, n)); break;
    case Storage::BF16: PHIP_CALL(::phip_fill_bf16(ctx_, px, k, n)); break;
  }
}

void HIP::reset_tensor_by_array_impl(const float values[], Tensor &x) {
  const std::size_t n = x.shape().size();
  void *px = get_mutable_handle(x);
  if (storage_ == Storage::F32) {
    PHIP_CALL(::phip_memcpy_h2d(ctx_, px, values, sizeof(float) * n));
  } else {
    std::shared_ptr<void> tmp = pool_->allocate(sizeof(float) * n);
    float *pt = static_cast<float *>(tmp.get());
    PHIP_CALL(::phip_memcpy_h2d(ctx_, pt, values, sizeof(float) * n));
    if (storage_ == Storage::F16) {
      PHIP_CALL(::phip_cvt_f32_to_f16(ctx_, pt, px, n));
    } else {
      PHIP_CALL(::phip_cvt_f32_to_bf16(ctx_, pt, px, n));
    }
  }
}

void HIP::copy_tensor_impl(const Tensor &x, Tensor &y) {
  const DeviceType src = x.device().type();
  if (src == DeviceType::NAIVE || src == DeviceType::EIGEN) {
    // host tensors hand over their buffer directly
    reset_tensor_by_array(static_cast<const float *>(get_handle(x)), y);
  } else if (src == type() && static_cast<const HIP &>(x.device()).storage_ == storage_) {
    PHIP_CALL(::phip_memcpy_d2d(
        ctx_, get_mutable_handle(y), get_handle(x), storage_bytes(x.shape().size())));
  } else {
    reset_tensor_by_vector(x.to_vector(), y);
  }
}

void HIP::identity_impl(Tensor &y) {
  // size x size identity assembled on the host; only used to build constants
  const std::uint32_t size = y.shape()[0];
  std::vector<float> host(static_cast<std::size_t>(size) * size, 0.0f);
  for (std::uint32_t i = 0; i < size; ++i) host[static_cast<std::size_t>(i) * (size + 1)] = 1.0f;
  reset_tensor_by_array_impl(host.data(), y);
}

void HIP::matmul_fw_impl(const Tensor &a, const Tensor &b, Tensor &y) {
  const Shape &sa = a.shape(), &sb = b.shape();
  const std::uint32_t di = sa[0], dj = sa[1], dk = sb[1];
  const void *pa = get_handle(a), *pb = get_handle(b);
  void *py = get_mutable_handle(y);
  switch (storage_) {
    case Storage::F32:
      PHIP_CALL(::phip_matmul_fw_f32(
          ctx_, static_cast<const float *>(pa), static_cast<const float *>(pb),
          static_cast<float *>(py), di, dj, dk, sa.batch(), sb.batch()));
      break;
    case Storage::F16:
      PHIP_CALL(::phip_matmul_fw_f16(ctx_, pa, pb, py, di, dj, dk, sa.batch(), sb.batch()));
      break;
    case Storage::BF16:
      PHIP_CALL(::phip_matmul_fw_bf16(ctx_, pa, pb, py, di, dj, dk, sa.batch(), sb.batch()));
      break;
  }
}

void HIP::matmul_bw_impl(
    const Tensor &a, const Tensor &b, const Tensor &, const Tensor &gy,
    Tensor &ga, Tensor &gb) {
  const Shape &sa = a.shape(), &sb = b.shape();
  const std::uint32_t di = sa[0], dj = sa[1], dk = sb[1];
  // Writable pointers first: taking one may replace a shared block by a
  // private copy (primitiv/core/tensor.cc:33-41), which enqueues a copy that
  // has to precede the accumulation.
  void *pga = get_mutable_handle(ga), *pgb = get_mutable_handle(gb);
  const void *pa = get_handle(a), *pb = get_handle(b), *pgy = get_handle(gy);
  switch (storage_) {
    case Storage::F32:
      PHIP_CALL(::phip_matmul_bw_f32(
          ctx_, static_cast<const float *>(pa), static_cast<const float *>(pb),
          static_cast<const float *>(pgy), static_cast<float *>(pga), static_cast<float *>(pgb),
          di, dj, dk, sa.batch(), sb.batch()));
      break;
    case Storage::F16:
      PHIP_CALL(::phip_matmul_bw_f16(ctx_, pa, pb, pgy, pga, pgb, di, dj, dk, sa.batch(), sb.batch()));
      break;
    case Storage::BF16:
      PHIP_CALL(::phip_matmul_bw_bf16(ctx_, pa, pb, pgy, pga, pgb, di, dj, dk, sa.batch(), sb.batch()));
      break;
  }
}

void HIP::batch_sum_fw_impl(const Tensor &x, Tensor &y) {
  const std::uint32_t volume = y.shape().volume(), bs = x.shape().batch();
  const void *px = get_handle(x);
  void *py = get_mutable_handle(y);
  switch (storage_) {
    case Storage::F32:
      PHIP_CALL(::phip_batch_sum_f32(ctx_, static_cast<const float *>(px), static_cast<float *>(py), volume, bs));
      break;
    case Storage::F16: PHIP_CALL(::phip_batch_sum_f16(ctx_, px, py, volume, bs)); break;
    case Storage::BF16: PHIP_CALL(::phip_batch_sum_bf16(ctx_, px, py, volume, bs)); break;
  }
}

void HIP::inplace_add_impl(const Tensor &x, Tensor &y) {
  const std::uint32_t volume = y.shape().volume();
  const std::uint32_t bx = x.shape().batch(), by = y.shape().batch();
  void *py = get_mutable_handle(y);
  const void *px = get_handle(x);
  switch (storage_) {
    case Storage::F32:
      PHIP_CALL(::phip_inplace_add_f32(ctx_, static_cast<const float *>(px), static_cast<float *>(py), volume, bx, by));
      break;
    case Storage::F16: PHIP_CALL(::phip_inplace_add_f16(ctx_, px, py, volume, bx, by)); break;
    case Storage::BF16: PHIP_CALL(::phip_inplace_add_bf16(ctx_, px, py, volume, bx, by)); break;
  }
}

}  // namespace devices
}  // namespace primitiv
