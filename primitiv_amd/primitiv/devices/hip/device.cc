// primitiv::devices::HIP: host side of the MI355X backend.  Built when
// PRIMITIV_USE_HIP is on; links against libphip (phip.h).

#include <primitiv/devices/hip/device.h>

#include <algorithm>
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

// libphip's elementwise entry points for one storage type, behind one
// signature (the fp32 variants take float pointers, the 16-bit ones void).
struct PointwiseAbi {
  int (*unary_fw)(phip_ctx *, int, const void *, void *, size_t);
  int (*unary_bw)(phip_ctx *, int, const void *, const void *, const void *, void *, size_t);
  int (*const_fw)(phip_ctx *, int, const void *, float, void *, size_t);
  int (*const_bw)(phip_ctx *, int, const void *, const void *, const void *, float, void *, size_t);
  int (*pown_fw)(phip_ctx *, const void *, std::int32_t, void *, size_t);
  int (*pown_bw)(phip_ctx *, const void *, const void *, const void *, std::int32_t, void *, size_t);
  int (*binary_fw)(phip_ctx *, int, const void *, const void *, void *, std::uint32_t, std::uint32_t, std::uint32_t);
  int (*binary_bw)(phip_ctx *, int, const void *, const void *, const void *, const void *, void *, void *,
                   std::uint32_t, std::uint32_t, std::uint32_t);
  int (*scalar_fw)(phip_ctx *, int, int, const void *, const void *, void *, std::uint32_t, std::uint32_t,
                   std::uint32_t);
  int (*inplace_subtract)(phip_ctx *, const void *, void *, std::uint32_t, std::uint32_t, std::uint32_t);
  int (*inplace_multiply_const)(phip_ctx *, float, void *, size_t);
  int (*identity)(phip_ctx *, void *, std::uint32_t);
};

typedef std::uint32_t U32;
typedef std::uint64_t U64;

// The same for the operations that move or reduce along one dimension.
struct IndexingAbi {
  int (*copy_rows)(phip_ctx *, const void *, void *, U32, U32, U64, U64, U32, U64, U64, int);
  int (*pick_fw)(phip_ctx *, const void *, const U32 *, U32, void *, U32, U32, U32, U32, U32);
  int (*pick_bw)(phip_ctx *, const void *, const U32 *, U32, void *, U32, U32, U32, U32, U32);
  int (*batch_pick_fw)(phip_ctx *, const void *, const U32 *, U32, void *, U32, U32);
  int (*batch_pick_bw)(phip_ctx *, const void *, const U32 *, U32, void *, U32, U32);
  int (*transpose_fw)(phip_ctx *, const void *, void *, U32, U32, U32);
  int (*transpose_bw)(phip_ctx *, const void *, void *, U32, U32, U32);
  int (*permute_dims_fw)(phip_ctx *, const void *, void *, U32, const U32 *, const U32 *, U32);
  int (*permute_dims_bw)(phip_ctx *, const void *, void *, U32, const U32 *, const U32 *, U32);
  int (*flip_fw)(phip_ctx *, const void *, void *, U32, U32, U32);
  int (*flip_bw)(phip_ctx *, const void *, void *, U32, U32, U32);
  int (*broadcast_fw)(phip_ctx *, const void *, void *, U32, U32, U32);
  int (*reduce_fw)(phip_ctx *, int, const void *, void *, U32, U32, U32);
  int (*extremum_bw)(phip_ctx *, int, const void *, const void *, const void *, void *, U32, U32, U32);
  int (*arg_extremum)(phip_ctx *, int, const void *, U32 *, U32, U32, U32);
};

typedef const float *CF;
typedef float *MF;

const PointwiseAbi &pointwise_abi(primitiv::devices::HIP::Storage s) {
  static const PointwiseAbi f32 = {
    [](phip_ctx *c, int op, const void *x, void *y, size_t n) {
      return ::phip_unary_fw_f32(c, op, CF(x), MF(y), n); },
    [](phip_ctx *c, int op, const void *x, const void *y, const void *gy, void *gx, size_t n) {
      return ::phip_unary_bw_f32(c, op, CF(x), CF(y), CF(gy), MF(gx), n); },
    [](phip_ctx *c, int op, const void *x, float k, void *y, size_t n) {
      return ::phip_const_fw_f32(c, op, CF(x), k, MF(y), n); },
    [](phip_ctx *c, int op, const void *x, const void *y, const void *gy, float k, void *gx, size_t n) {
      return ::phip_const_bw_f32(c, op, CF(x), CF(y), CF(gy), k, MF(gx), n); },
    [](phip_ctx *c, const void *x, std::int32_t k, void *y, size_t n) {
      return ::phip_pown_fw_f32(c, CF(x), k, MF(y), n); },
    [](phip_ctx *c, const void *x, const void *y, const void *gy, std::int32_t k, void *gx, size_t n) {
      return ::phip_pown_bw_f32(c, CF(x), CF(y), CF(gy), k, MF(gx), n); },
    [](phip_ctx *c, int op, const void *a, const void *b, void *y, std::uint32_t v, std::uint32_t ba,
       std::uint32_t bb) { return ::phip_binary_fw_f32(c, op, CF(a), CF(b), MF(y), v, ba, bb); },
    [](phip_ctx *c, int op, const void *a, const void *b, const void *y, const void *gy, void *ga, void *gb,
       std::uint32_t v, std::uint32_t ba, std::uint32_t bb) {
      return ::phip_binary_bw_f32(c, op, CF(a), CF(b), CF(y), CF(gy), MF(ga), MF(gb), v, ba, bb); },
    [](phip_ctx *c, int op, int left, const void *x, const void *k, void *y, std::uint32_t v, std::uint32_t bx,
       std::uint32_t bk) { return ::phip_scalar_fw_f32(c, op, left, CF(x), CF(k), MF(y), v, bx, bk); },
    [](phip_ctx *c, const void *x, void *y, std::uint32_t v, std::uint32_t bx, std::uint32_t by) {
      return ::phip_inplace_subtract_f32(c, CF(x), MF(y), v, bx, by); },
    [](phip_ctx *c, float k, void *x, size_t n) { return ::phip_inplace_multiply_const_f32(c, k, MF(x), n); },
    [](phip_ctx *c, void *y, std::uint32_t rows) { return ::phip_identity_f32(c, MF(y), rows); },
  };
  static const PointwiseAbi f16 = {
    ::phip_unary_fw_f16, ::phip_unary_bw_f16, ::phip_const_fw_f16, ::phip_const_bw_f16, ::phip_pown_fw_f16,
    ::phip_pown_bw_f16, ::phip_binary_fw_f16, ::phip_binary_bw_f16, ::phip_scalar_fw_f16,
    ::phip_inplace_subtract_f16, ::phip_inplace_multiply_const_f16, ::phip_identity_f16,
  };
  static const PointwiseAbi bf16 = {
    ::phip_unary_fw_bf16, ::phip_unary_bw_bf16, ::phip_const_fw_bf16, ::phip_const_bw_bf16, ::phip_pown_fw_bf16,
    ::phip_pown_bw_bf16, ::phip_binary_fw_bf16, ::phip_binary_bw_bf16, ::phip_scalar_fw_bf16,
    ::phip_inplace_subtract_bf16, ::phip_inplace_multiply_const_bf16, ::phip_identity_bf16,
  };
  switch (s) {
    case primitiv::devices::HIP::Storage::F16: return f16;
    case primitiv::devices::HIP::Storage::BF16: return bf16;
    default: return f32;
  }
}

const IndexingAbi &indexing_abi(primitiv::devices::HIP::Storage s) {
  static const IndexingAbi f32 = {
    [](phip_ctx *c, const void *src, void *dst, U32 span, U32 rows, U64 ss, U64 ds, U32 bs, U64 sbs, U64 dbs,
       int acc) { return ::phip_copy_rows_f32(c, CF(src), MF(dst), span, rows, ss, ds, bs, sbs, dbs, acc); },
    [](phip_ctx *c, const void *x, const U32 *ids, U32 n_ids, void *y, U32 base, U32 n, U32 outer, U32 bx,
       U32 bs) { return ::phip_pick_fw_f32(c, CF(x), ids, n_ids, MF(y), base, n, outer, bx, bs); },
    [](phip_ctx *c, const void *gy, const U32 *ids, U32 n_ids, void *gx, U32 base, U32 n, U32 outer, U32 bx,
       U32 bs) { return ::phip_pick_bw_f32(c, CF(gy), ids, n_ids, MF(gx), base, n, outer, bx, bs); },
    [](phip_ctx *c, const void *x, const U32 *ids, U32 n_ids, void *y, U32 volume, U32 bx) {
      return ::phip_batch_pick_fw_f32(c, CF(x), ids, n_ids, MF(y), volume, bx); },
    [](phip_ctx *c, const void *gy, const U32 *ids, U32 n_ids, void *gx, U32 volume, U32 bx) {
      return ::phip_batch_pick_bw_f32(c, CF(gy), ids, n_ids, MF(gx), volume, bx); },
    [](phip_ctx *c, const void *x, void *y, U32 rows, U32 cols, U32 bs) {
      return ::phip_transpose_fw_f32(c, CF(x), MF(y), rows, cols, bs); },
    [](phip_ctx *c, const void *gy, void *gx, U32 rows, U32 cols, U32 bs) {
      return ::phip_transpose_bw_f32(c, CF(gy), MF(gx), rows, cols, bs); },
    [](phip_ctx *c, const void *x, void *y, U32 nd, const U32 *dims, const U32 *perm, U32 bs) {
      return ::phip_permute_dims_fw_f32(c, CF(x), MF(y), nd, dims, perm, bs); },
    [](phip_ctx *c, const void *gy, void *gx, U32 nd, const U32 *dims, const U32 *perm, U32 bs) {
      return ::phip_permute_dims_bw_f32(c, CF(gy), MF(gx), nd, dims, perm, bs); },
    [](phip_ctx *c, const void *x, void *y, U32 base, U32 n, U32 outer) {
      return ::phip_flip_fw_f32(c, CF(x), MF(y), base, n, outer); },
    [](phip_ctx *c, const void *gy, void *gx, U32 base, U32 n, U32 outer) {
      return ::phip_flip_bw_f32(c, CF(gy), MF(gx), base, n, outer); },
    [](phip_ctx *c, const void *x, void *y, U32 base, U32 size, U32 outer) {
      return ::phip_broadcast_fw_f32(c, CF(x), MF(y), base, size, outer); },
    [](phip_ctx *c, int op, const void *x, void *y, U32 base, U32 n, U32 outer) {
      return ::phip_reduce_fw_f32(c, op, CF(x), MF(y), base, n, outer); },
    [](phip_ctx *c, int op, const void *x, const void *y, const void *gy, void *gx, U32 base, U32 n, U32 outer) {
      return ::phip_extremum_bw_f32(c, op, CF(x), CF(y), CF(gy), MF(gx), base, n, outer); },
    [](phip_ctx *c, int op, const void *x, U32 *out, U32 base, U32 n, U32 outer) {
      return ::phip_arg_extremum_f32(c, op, CF(x), out, base, n, outer); },
  };
  static const IndexingAbi f16 = {
    ::phip_copy_rows_f16, ::phip_pick_fw_f16, ::phip_pick_bw_f16, ::phip_batch_pick_fw_f16,
    ::phip_batch_pick_bw_f16, ::phip_transpose_fw_f16, ::phip_transpose_bw_f16, ::phip_permute_dims_fw_f16,
    ::phip_permute_dims_bw_f16, ::phip_flip_fw_f16, ::phip_flip_bw_f16, ::phip_broadcast_fw_f16,
    ::phip_reduce_fw_f16, ::phip_extremum_bw_f16, ::phip_arg_extremum_f16,
  };
  static const IndexingAbi bf16 = {
    ::phip_copy_rows_bf16, ::phip_pick_fw_bf16, ::phip_pick_bw_bf16, ::phip_batch_pick_fw_bf16,
    ::phip_batch_pick_bw_bf16, ::phip_transpose_fw_bf16, ::phip_transpose_bw_bf16, ::phip_permute_dims_fw_bf16,
    ::phip_permute_dims_bw_bf16, ::phip_flip_fw_bf16, ::phip_flip_bw_bf16, ::phip_broadcast_fw_bf16,
    ::phip_reduce_fw_bf16, ::phip_extremum_bw_bf16, ::phip_arg_extremum_bf16,
  };
  switch (s) {
    case primitiv::devices::HIP::Storage::F16: return f16;
    case primitiv::devices::HIP::Storage::BF16: return bf16;
    default: return f32;
  }
}

// Address `elements` elements past p for a storage type.
inline const void *advance(const void *p, std::size_t elements, primitiv::devices::HIP::Storage s) {
  return static_cast<const char *>(p) + elements * (s == primitiv::devices::HIP::Storage::F32 ? 4 : 2);
}
inline void *advance(void *p, std::size_t elements, primitiv::devices::HIP::Storage s) {
  return static_cast<char *>(p) + elements * (s == primitiv::devices::HIP::Storage::F32 ? 4 : 2);
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
: dev_id_(device_id), rng_seed_(rng_seed), rng_offset_(0), storage_(storage), ctx_(nullptr) {
  assert_support(dev_id_);
  PHIP_CALL(::phip_ctx_create(static_cast<int>(dev_id_), &ctx_));
  phip_ctx *ctx = ctx_;
  // The pool asks libphip for raw blocks; a failed allocation must throw so
  // that the pool releases its idle blocks and retries
  // (primitiv/core/memory_pool.cc:53-63).  libphip keeps a pool of its own
  // for the scratch memory of its kernels (power-of-two blocks, cached when
  // idle): when the device is full those blocks are given back first.
  pool_.reset(new MemoryPool(
      [ctx](std::size_t size) -> void * {
        void *ptr = nullptr;
        int status = ::phip_malloc(ctx, size, &ptr);
        if (status == PHIP_ERR_OUT_OF_MEMORY) {
          PHIP_CALL(::phip_pool_release_reserved(ctx));
          status = ::phip_malloc(ctx, size, &ptr);
        }
        if (status != PHIP_OK) {
          PRIMITIV_THROW_ERROR(
              "libphip call failed. statement: phip_malloc, status: " << status << ": " << ::phip_last_error());
        }
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

void HIP::set_deterministic(bool on) {
  PHIP_CALL(::phip_set_deterministic(ctx_, on ? 1 : 0));
}

void HIP::set_overlap(bool on) {
  PHIP_CALL(::phip_set_overlap(ctx_, on ? 1 : 0));
}

void HIP::set_deferred_zero_fill(bool on) {
  PHIP_CALL(::phip_set_deferred_zero_fill(ctx_, on ? 1 : 0));
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
  const std::size_t n = x.shape().size();
  if (src == DeviceType::NAIVE || src == DeviceType::EIGEN) {
    // host tensors hand over their buffer directly
    reset_tensor_by_array(static_cast<const float *>(get_handle(x)), y);
    return;
  }
  if (src == DEVICE_TYPE_HIP || src == DEVICE_TYPE_HIP16) {
    const HIP &from = static_cast<const HIP &>(x.device());
    if (&from == this) {
      // ordered by this device's stream
      PHIP_CALL(::phip_memcpy_d2d(ctx_, get_mutable_handle(y), get_handle(x), storage_bytes(n)));
      return;
    }
    const bool convertible = from.storage_ == storage_ || from.storage_ == Storage::F32 || storage_ == Storage::F32;
    if (from.dev_id_ == dev_id_ && convertible) {
      // Another device object on the same GPU has a stream of its own: drain
      // it, copy or convert on the GPU, then drain this stream so that the
      // source may be released as soon as the call returns.
      PHIP_CALL(::phip_sync(from.ctx_));
      void *py = get_mutable_handle(y);
      const void *px = get_handle(x);
      if (from.storage_ == storage_) {
        PHIP_CALL(::phip_memcpy_d2d(ctx_, py, px, storage_bytes(n)));
      } else if (from.storage_ == Storage::F16) {
        PHIP_CALL(::phip_cvt_f16_to_f32(ctx_, px, static_cast<float *>(py), n));
      } else if (from.storage_ == Storage::BF16) {
        PHIP_CALL(::phip_cvt_bf16_to_f32(ctx_, px, static_cast<float *>(py), n));
      } else if (storage_ == Storage::F16) {
        PHIP_CALL(::phip_cvt_f32_to_f16(ctx_, static_cast<const float *>(px), py, n));
      } else {
        PHIP_CALL(::phip_cvt_f32_to_bf16(ctx_, static_cast<const float *>(px), py, n));
      }
      PHIP_CALL(::phip_sync(ctx_));
      return;
    }
  }
  // other devices, other GPUs, f16 <-> bf16: through the host
  reset_tensor_by_vector(x.to_vector(), y);
}

void HIP::identity_impl(Tensor &y) {
  PHIP_CALL(pointwise_abi(storage_).identity(ctx_, get_mutable_handle(y), y.shape()[0]));
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

void HIP::inplace_subtract_impl(const Tensor &x, Tensor &y) {
  void *py = get_mutable_handle(y);
  PHIP_CALL(pointwise_abi(storage_).inplace_subtract(
      ctx_, get_handle(x), py, y.shape().volume(), x.shape().batch(), y.shape().batch()));
}

void HIP::inplace_multiply_const_impl(float k, Tensor &x) {
  PHIP_CALL(pointwise_abi(storage_).inplace_multiply_const(ctx_, k, get_mutable_handle(x), x.shape().size()));
}

// ---- random tensors ------------------------------------------------------------
// Element i of a call is word i%4 of Philox block rng_offset_ + i/4; the
// offset then moves past the blocks the call used.

#define PHIP_DEF_RANDOM(name, ...) \
  const std::size_t n = y.shape().size(); \
  void *py = get_mutable_handle(y); \
  switch (storage_) { \
    case Storage::F32: \
      PHIP_CALL(::phip_random_##name##_f32(ctx_, rng_seed_, rng_offset_, __VA_ARGS__, static_cast<float *>(py), n)); \
      break; \
    case Storage::F16: PHIP_CALL(::phip_random_##name##_f16(ctx_, rng_seed_, rng_offset_, __VA_ARGS__, py, n)); break; \
    case Storage::BF16: PHIP_CALL(::phip_random_##name##_bf16(ctx_, rng_seed_, rng_offset_, __VA_ARGS__, py, n)); break; \
  } \
  rng_offset_ += (n + 3) / 4;

void HIP::random_bernoulli_impl(float p, Tensor &y) { PHIP_DEF_RANDOM(bernoulli, p) }
void HIP::random_uniform_impl(float lower, float upper, Tensor &y) { PHIP_DEF_RANDOM(uniform, lower, upper) }
void HIP::random_normal_impl(float mean, float sd, Tensor &y) { PHIP_DEF_RANDOM(normal, mean, sd) }
void HIP::random_log_normal_impl(float mean, float sd, Tensor &y) { PHIP_DEF_RANDOM(log_normal, mean, sd) }

#undef PHIP_DEF_RANDOM

// ---- moving and reducing along one dimension -------------------------------------
// A tensor is seen around `dim` as [outer][n][base] (base = lower_volume(dim));
// the offsets handed to libphip are those of the reference's kernels
// (primitiv/devices/cuda/ops/{slice,concat,pick,batch_pick,batch_slice,
// batch_concat,transpose,permute_dims,flip,sum,logsumexp,max,min,argmax,
// argmin,broadcast}.cu).

void HIP::slice_fw_impl(const Tensor &x, std::uint32_t dim, std::uint32_t offset, Tensor &y) {
  const std::uint32_t base = y.shape().lower_volume(dim);
  const std::uint32_t span = base * y.shape()[dim];
  const std::uint32_t skip = base * x.shape()[dim];
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).copy_rows(
      ctx_, advance(get_handle(x), static_cast<std::size_t>(base) * offset, storage_), py,
      span, y.shape().size() / span, skip, span, 1, 0, 0, 0));
}

void HIP::slice_bw_impl(const Tensor &gy, std::uint32_t dim, std::uint32_t offset, Tensor &gx) {
  const Shape &sx = gx.shape();
  const Shape &sy = gy.shape();
  const std::uint32_t base = sx.lower_volume(dim);
  const std::uint32_t span = base * sy[dim];
  const std::uint32_t skip = base * sx[dim];
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).copy_rows(
      ctx_, get_handle(gy), advance(pgx, static_cast<std::size_t>(base) * offset, storage_),
      span, sx.volume() / skip, span, skip, std::max(sx.batch(), sy.batch()),
      sy.has_batch() ? sy.volume() : 0, sx.has_batch() ? sx.volume() : 0, 1));
}

void HIP::concat_fw_impl(const std::vector<const Tensor *> &xs, std::uint32_t dim, Tensor &y) {
  const Shape &sy = y.shape();
  const std::uint32_t base = sy.lower_volume(dim);
  const std::uint32_t skip = base * sy[dim];
  const std::uint32_t repeat = sy.volume() / skip;
  void *py = get_mutable_handle(y);
  std::size_t offset = 0;
  for (const Tensor *x : xs) {
    const std::uint32_t span = base * x->shape()[dim];
    PHIP_CALL(indexing_abi(storage_).copy_rows(
        ctx_, get_handle(*x), advance(py, offset, storage_), span, repeat, span, skip, sy.batch(),
        x->shape().has_batch() ? x->shape().volume() : 0, sy.volume(), 0));
    offset += span;
  }
}

void HIP::pick_fw_impl(
    const Tensor &x, const std::vector<std::uint32_t> &ids, std::uint32_t dim, Tensor &y) {
  const Shape &sx = x.shape();
  const std::uint32_t base = sx.lower_volume(dim);
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).pick_fw(
      ctx_, get_handle(x), ids.data(), ids.size(), py, base, sx[dim], sx.volume() / (base * sx[dim]),
      sx.batch(), y.shape().batch()));
}

void HIP::pick_bw_impl(
    const Tensor &gy, const std::vector<std::uint32_t> &ids, std::uint32_t dim, Tensor &gx) {
  const Shape &sx = gx.shape();
  const std::uint32_t base = sx.lower_volume(dim);
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).pick_bw(
      ctx_, get_handle(gy), ids.data(), ids.size(), pgx, base, sx[dim], sx.volume() / (base * sx[dim]),
      sx.batch(), gy.shape().batch()));
}

void HIP::batch_pick_fw_impl(const Tensor &x, const std::vector<std::uint32_t> &ids, Tensor &y) {
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).batch_pick_fw(
      ctx_, get_handle(x), ids.data(), ids.size(), py, x.shape().volume(), x.shape().batch()));
}

void HIP::batch_pick_bw_impl(const Tensor &gy, const std::vector<std::uint32_t> &ids, Tensor &gx) {
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).batch_pick_bw(
      ctx_, get_handle(gy), ids.data(), ids.size(), pgx, gx.shape().volume(), gx.shape().batch()));
}

void HIP::batch_slice_fw_impl(const Tensor &x, std::uint32_t offset, Tensor &y) {
  const std::uint32_t volume = y.shape().volume();
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).copy_rows(
      ctx_, advance(get_handle(x), static_cast<std::size_t>(volume) * offset, storage_), py,
      volume, y.shape().batch(), volume, volume, 1, 0, 0, 0));
}

void HIP::batch_slice_bw_impl(const Tensor &gy, std::uint32_t offset, Tensor &gx) {
  const std::uint32_t volume = gy.shape().volume();
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).copy_rows(
      ctx_, get_handle(gy), advance(pgx, static_cast<std::size_t>(volume) * offset, storage_),
      volume, gy.shape().batch(), volume, volume, 1, 0, 0, 1));
}

void HIP::batch_concat_fw_impl(const std::vector<const Tensor *> &xs, Tensor &y) {
  const std::uint32_t volume = y.shape().volume();
  void *py = get_mutable_handle(y);
  std::size_t offset = 0;
  for (const Tensor *x : xs) {
    PHIP_CALL(indexing_abi(storage_).copy_rows(
        ctx_, get_handle(*x), advance(py, offset, storage_), volume, x->shape().batch(), volume, volume,
        1, 0, 0, 0));
    offset += x->shape().size();
  }
}

void HIP::transpose_fw_impl(const Tensor &x, Tensor &y) {
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).transpose_fw(
      ctx_, get_handle(x), py, x.shape()[0], x.shape()[1], x.shape().batch()));
}

void HIP::transpose_bw_impl(const Tensor &, const Tensor &, const Tensor &gy, Tensor &gx) {
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).transpose_bw(
      ctx_, get_handle(gy), pgx, gx.shape()[0], gx.shape()[1], gx.shape().batch()));
}

void HIP::permute_dims_fw_impl(const Tensor &x, const std::vector<std::uint32_t> &perm, Tensor &y) {
  std::vector<std::uint32_t> dims(perm.size());
  for (std::size_t i = 0; i < perm.size(); ++i) dims[i] = x.shape()[i];
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).permute_dims_fw(
      ctx_, get_handle(x), py, perm.size(), dims.data(), perm.data(), x.shape().batch()));
}

void HIP::permute_dims_bw_impl(
    const Tensor &, const Tensor &, const Tensor &gy, const std::vector<std::uint32_t> &perm, Tensor &gx) {
  std::vector<std::uint32_t> dims(perm.size());
  for (std::size_t i = 0; i < perm.size(); ++i) dims[i] = gx.shape()[i];
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).permute_dims_bw(
      ctx_, get_handle(gy), pgx, perm.size(), dims.data(), perm.data(), gx.shape().batch()));
}

void HIP::flip_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) {
  const Shape &s = x.shape();
  const std::uint32_t base = s.lower_volume(dim), n = s[dim];
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).flip_fw(ctx_, get_handle(x), py, base, n, s.size() / (base * n)));
}

void HIP::flip_bw_impl(const Tensor &gy, std::uint32_t dim, Tensor &gx) {
  const Shape &s = gx.shape();
  const std::uint32_t base = s.lower_volume(dim), n = s[dim];
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(indexing_abi(storage_).flip_bw(ctx_, get_handle(gy), pgx, base, n, s.size() / (base * n)));
}

void HIP::broadcast_fw_impl(const Tensor &x, std::uint32_t dim, std::uint32_t size, Tensor &y) {
  const std::uint32_t base = y.shape().lower_volume(dim);
  void *py = get_mutable_handle(y);
  PHIP_CALL(indexing_abi(storage_).broadcast_fw(ctx_, get_handle(x), py, base, size, x.shape().size() / base));
}

#define PHIP_DEF_REDUCE(name, code) \
void HIP::name##_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) { \
  const Shape &s = x.shape(); \
  const std::uint32_t base = s.lower_volume(dim), n = s[dim]; \
  void *py = get_mutable_handle(y); \
  PHIP_CALL(indexing_abi(storage_).reduce_fw(ctx_, code, get_handle(x), py, base, n, s.size() / (base * n))); \
}

#define PHIP_DEF_EXTREMUM(name, code) \
void HIP::name##_bw_impl( \
    const Tensor &x, const Tensor &y, const Tensor &gy, std::uint32_t dim, Tensor &gx) { \
  const Shape &s = x.shape(); \
  const std::uint32_t base = s.lower_volume(dim), n = s[dim]; \
  void *pgx = get_mutable_handle(gx); \
  PHIP_CALL(indexing_abi(storage_).extremum_bw( \
      ctx_, code, get_handle(x), get_handle(y), get_handle(gy), pgx, base, n, s.size() / (base * n))); \
} \
std::vector<std::uint32_t> HIP::arg##name##_impl(const Tensor &x, std::uint32_t dim) { \
  const Shape &s = x.shape(); \
  const std::uint32_t base = s.lower_volume(dim), n = s[dim]; \
  std::vector<std::uint32_t> ret(s.size() / n); \
  PHIP_CALL(indexing_abi(storage_).arg_extremum( \
      ctx_, code, get_handle(x), ret.data(), base, n, s.size() / (base * n))); \
  return ret; \
}

PHIP_DEF_REDUCE(sum, PHIP_SUM)
PHIP_DEF_REDUCE(logsumexp, PHIP_LOGSUMEXP)
PHIP_DEF_REDUCE(max, PHIP_MAX)
PHIP_DEF_REDUCE(min, PHIP_MIN)
PHIP_DEF_EXTREMUM(max, PHIP_MAX)
PHIP_DEF_EXTREMUM(min, PHIP_MIN)

#undef PHIP_DEF_REDUCE
#undef PHIP_DEF_EXTREMUM

// ---- elementwise families ------------------------------------------------------
// One definition per Device virtual; the libphip operation code names the
// member (the reference instantiates one kernel per member through
// CUDADEV_FW_X, CUDADEV_BW_X, ... in primitiv/devices/cuda/ops/common.h:77-151).
// Writable handles are taken first: taking one may clone a shared block.

void HIP::negate_fw_impl(const Tensor &x, Tensor &y) {
  void *py = get_mutable_handle(y);
  PHIP_CALL(pointwise_abi(storage_).unary_fw(ctx_, PHIP_NEGATE, get_handle(x), py, x.shape().size()));
}

#define PHIP_DEF_X(name, code) \
void HIP::name##_fw_impl(const Tensor &x, Tensor &y) { \
  void *py = get_mutable_handle(y); \
  PHIP_CALL(pointwise_abi(storage_).unary_fw(ctx_, code, get_handle(x), py, x.shape().size())); \
} \
void HIP::name##_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, Tensor &gx) { \
  void *pgx = get_mutable_handle(gx); \
  PHIP_CALL(pointwise_abi(storage_).unary_bw( \
      ctx_, code, get_handle(x), get_handle(y), get_handle(gy), pgx, x.shape().size())); \
}

#define PHIP_DEF_CONST(name, code) \
void HIP::name##_fw_impl(const Tensor &x, float k, Tensor &y) { \
  void *py = get_mutable_handle(y); \
  PHIP_CALL(pointwise_abi(storage_).const_fw(ctx_, code, get_handle(x), k, py, x.shape().size())); \
} \
void HIP::name##_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, float k, Tensor &gx) { \
  void *pgx = get_mutable_handle(gx); \
  PHIP_CALL(pointwise_abi(storage_).const_bw( \
      ctx_, code, get_handle(x), get_handle(y), get_handle(gy), k, pgx, x.shape().size())); \
}

#define PHIP_DEF_SCALAR(name, code, left) \
void HIP::name##_fw_impl(const Tensor &x, const Tensor &k, Tensor &y) { \
  void *py = get_mutable_handle(y); \
  PHIP_CALL(pointwise_abi(storage_).scalar_fw( \
      ctx_, code, left, get_handle(x), get_handle(k), py, y.shape().volume(), \
      x.shape().batch(), k.shape().batch())); \
}

#define PHIP_DEF_AB(name, code) \
void HIP::name##_fw_impl(const Tensor &a, const Tensor &b, Tensor &y) { \
  void *py = get_mutable_handle(y); \
  PHIP_CALL(pointwise_abi(storage_).binary_fw( \
      ctx_, code, get_handle(a), get_handle(b), py, y.shape().volume(), \
      a.shape().batch(), b.shape().batch())); \
} \
void HIP::name##_bw_impl( \
    const Tensor &a, const Tensor &b, const Tensor &y, const Tensor &gy, Tensor &ga, Tensor &gb) { \
  void *pga = get_mutable_handle(ga); \
  void *pgb = get_mutable_handle(gb); \
  PHIP_CALL(pointwise_abi(storage_).binary_bw( \
      ctx_, code, get_handle(a), get_handle(b), get_handle(y), get_handle(gy), pga, pgb, \
      y.shape().volume(), a.shape().batch(), b.shape().batch())); \
}

PHIP_DEF_X(abs, PHIP_ABS)
PHIP_DEF_X(sqrt, PHIP_SQRT)
PHIP_DEF_X(exp, PHIP_EXP)
PHIP_DEF_X(log, PHIP_LOG)
PHIP_DEF_X(tanh, PHIP_TANH)
PHIP_DEF_X(sigmoid, PHIP_SIGMOID)
PHIP_DEF_X(softplus, PHIP_SOFTPLUS)
PHIP_DEF_X(sin, PHIP_SIN)
PHIP_DEF_X(cos, PHIP_COS)
PHIP_DEF_X(tan, PHIP_TAN)

PHIP_DEF_CONST(add_const, PHIP_ADD_CONST)
PHIP_DEF_CONST(subtract_const_r, PHIP_SUBTRACT_CONST_R)
PHIP_DEF_CONST(subtract_const_l, PHIP_SUBTRACT_CONST_L)
PHIP_DEF_CONST(multiply_const, PHIP_MULTIPLY_CONST)
PHIP_DEF_CONST(divide_const_r, PHIP_DIVIDE_CONST_R)
PHIP_DEF_CONST(divide_const_l, PHIP_DIVIDE_CONST_L)
PHIP_DEF_CONST(pow_const_r, PHIP_POW_CONST_R)
PHIP_DEF_CONST(pow_const_l, PHIP_POW_CONST_L)
PHIP_DEF_CONST(prelu, PHIP_PRELU)
PHIP_DEF_CONST(elu, PHIP_ELU)

void HIP::pown_fw_impl(const Tensor &x, std::int32_t k, Tensor &y) {
  void *py = get_mutable_handle(y);
  PHIP_CALL(pointwise_abi(storage_).pown_fw(ctx_, get_handle(x), k, py, x.shape().size()));
}

void HIP::pown_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, std::int32_t k, Tensor &gx) {
  void *pgx = get_mutable_handle(gx);
  PHIP_CALL(pointwise_abi(storage_).pown_bw(
      ctx_, get_handle(x), get_handle(y), get_handle(gy), k, pgx, x.shape().size()));
}

PHIP_DEF_SCALAR(add_scalar, PHIP_ADD, 0)
PHIP_DEF_SCALAR(subtract_scalar_r, PHIP_SUBTRACT, 0)
PHIP_DEF_SCALAR(subtract_scalar_l, PHIP_SUBTRACT, 1)
PHIP_DEF_SCALAR(multiply_scalar, PHIP_MULTIPLY, 0)
PHIP_DEF_SCALAR(divide_scalar_r, PHIP_DIVIDE, 0)
PHIP_DEF_SCALAR(divide_scalar_l, PHIP_DIVIDE, 1)
PHIP_DEF_SCALAR(pow_scalar_r, PHIP_POW, 0)
PHIP_DEF_SCALAR(pow_scalar_l, PHIP_POW, 1)

PHIP_DEF_AB(add, PHIP_ADD)
PHIP_DEF_AB(subtract, PHIP_SUBTRACT)
PHIP_DEF_AB(multiply, PHIP_MULTIPLY)
PHIP_DEF_AB(divide, PHIP_DIVIDE)
PHIP_DEF_AB(pow, PHIP_POW)

#undef PHIP_DEF_X
#undef PHIP_DEF_CONST
#undef PHIP_DEF_SCALAR
#undef PHIP_DEF_AB

// ---- convolution and pooling --------------------------------------------------

void HIP::conv2d_fw_impl(
    const Tensor &x, const Tensor &w, std::uint32_t padding0, std::uint32_t padding1, std::uint32_t stride0,
    std::uint32_t stride1, std::uint32_t dilation0, std::uint32_t dilation1, Tensor &y) {
  const Shape &sx = x.shape();
  const Shape &sw = w.shape();
  void *py = get_mutable_handle(y);
  const void *px = get_handle(x), *pw = get_handle(w);
#define PHIP_CONV_FW(SUF, CPTR, PTR)                                                                        \
  PHIP_CALL(::phip_conv2d_fw_##SUF(ctx_, static_cast<CPTR>(px), static_cast<CPTR>(pw), static_cast<PTR>(py), \
                                   sx[0], sx[1], sx[2], sw[0], sw[1], sw[3], sx.batch(), sw.batch(),         \
                                   padding0, padding1, stride0, stride1, dilation0, dilation1))
  switch (storage_) {
    case Storage::F32: PHIP_CONV_FW(f32, const float *, float *); break;
    case Storage::F16: PHIP_CONV_FW(f16, const void *, void *); break;
    default: PHIP_CONV_FW(bf16, const void *, void *); break;
  }
#undef PHIP_CONV_FW
}

void HIP::conv2d_bw_impl(
    const Tensor &x, const Tensor &w, const Tensor &, const Tensor &gy, std::uint32_t padding0,
    std::uint32_t padding1, std::uint32_t stride0, std::uint32_t stride1, std::uint32_t dilation0,
    std::uint32_t dilation1, Tensor &gx, Tensor &gw) {
  const Shape &sx = x.shape();
  const Shape &sw = w.shape();
  // writable pointers first: taking them may clone a shared block
  void *pgx = get_mutable_handle(gx);
  void *pgw = get_mutable_handle(gw);
  const void *px = get_handle(x), *pw = get_handle(w), *pgy = get_handle(gy);
#define PHIP_CONV_BW(SUF, CPTR, PTR)                                                                          \
  PHIP_CALL(::phip_conv2d_bw_##SUF(ctx_, static_cast<CPTR>(px), static_cast<CPTR>(pw), static_cast<CPTR>(pgy), \
                                   static_cast<PTR>(pgx), static_cast<PTR>(pgw), sx[0], sx[1], sx[2], sw[0],   \
                                   sw[1], sw[3], sx.batch(), sw.batch(), padding0, padding1, stride0, stride1, \
                                   dilation0, dilation1))
  switch (storage_) {
    case Storage::F32: PHIP_CONV_BW(f32, const float *, float *); break;
    case Storage::F16: PHIP_CONV_BW(f16, const void *, void *); break;
    default: PHIP_CONV_BW(bf16, const void *, void *); break;
  }
#undef PHIP_CONV_BW
}

void HIP::max_pool2d_fw_impl(
    const Tensor &x, std::uint32_t window0, std::uint32_t window1, std::uint32_t padding0, std::uint32_t padding1,
    std::uint32_t stride0, std::uint32_t stride1, Tensor &y) {
  const Shape &sx = x.shape();
  const std::uint32_t repeat = sx.size() / (sx[0] * sx[1]);  // channels and samples alike
  void *py = get_mutable_handle(y);
  const void *px = get_handle(x);
#define PHIP_POOL_FW(SUF, CPTR, PTR)                                                                       \
  PHIP_CALL(::phip_max_pool2d_fw_##SUF(ctx_, static_cast<CPTR>(px), static_cast<PTR>(py), sx[0], sx[1], repeat, \
                                       window0, window1, padding0, padding1, stride0, stride1))
  switch (storage_) {
    case Storage::F32: PHIP_POOL_FW(f32, const float *, float *); break;
    case Storage::F16: PHIP_POOL_FW(f16, const void *, void *); break;
    default: PHIP_POOL_FW(bf16, const void *, void *); break;
  }
#undef PHIP_POOL_FW
}

void HIP::max_pool2d_bw_impl(
    const Tensor &x, const Tensor &y, const Tensor &gy, std::uint32_t window0, std::uint32_t window1,
    std::uint32_t padding0, std::uint32_t padding1, std::uint32_t stride0, std::uint32_t stride1, Tensor &gx) {
  const Shape &sx = x.shape();
  const std::uint32_t repeat = sx.size() / (sx[0] * sx[1]);
  void *pgx = get_mutable_handle(gx);
  const void *px = get_handle(x), *py = get_handle(y), *pgy = get_handle(gy);
#define PHIP_POOL_BW(SUF, CPTR, PTR)                                                                         \
  PHIP_CALL(::phip_max_pool2d_bw_##SUF(ctx_, static_cast<CPTR>(px), static_cast<CPTR>(py), static_cast<CPTR>(pgy), \
                                       static_cast<PTR>(pgx), sx[0], sx[1], repeat, window0, window1, padding0, \
                                       padding1, stride0, stride1))
  switch (storage_) {
    case Storage::F32: PHIP_POOL_BW(f32, const float *, float *); break;
    case Storage::F16: PHIP_POOL_BW(f16, const void *, void *); break;
    default: PHIP_POOL_BW(bf16, const void *, void *); break;
  }
#undef PHIP_POOL_BW
}

}  // namespace devices
}  // namespace primitiv
