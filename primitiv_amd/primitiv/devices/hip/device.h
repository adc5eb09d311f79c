#ifndef PRIMITIV_DEVICES_HIP_DEVICE_H_
#define PRIMITIV_DEVICES_HIP_DEVICE_H_

// primitiv::devices::HIP -- AMD MI355X (gfx950) backend.
//
// Drop-in subclass of primitiv::Device (primitiv/core/device.h): the existing
// Graph / Node / Tensor / Parameter code talks to it through the same virtual
// interface as to the CUDA backend (primitiv/devices/cuda/device.h).  All GPU
// work goes through libphip's C ABI (phip.h); this class only owns the
// context and the memory pool and forwards each operation.
//
// Every operation of the Device interface is implemented: matmul
// forward/backward (the path this backend was built around), the helpers the
// graph needs around them (allocation, fill, copies, in-place add with
// minibatch broadcasting, minibatch sum), the elementwise families, indexing
// and reductions, random tensors, convolution and pooling.

#include <cstdint>
#include <memory>
#include <vector>

#include <primitiv/core/device.h>
#include <primitiv/core/error.h>
#include <primitiv/core/memory_pool.h>

struct phip_ctx;

namespace primitiv {
namespace devices {

// Values to be added to enum DeviceType (primitiv/core/device.h:17-35) as a
// fourth group; spelled as casts here so that this header also compiles
// against an unpatched primitiv.
constexpr DeviceType DEVICE_TYPE_GROUP_HIP = static_cast<DeviceType>(0x00030000u);
constexpr DeviceType DEVICE_TYPE_HIP = static_cast<DeviceType>(0x00030000u);
constexpr DeviceType DEVICE_TYPE_HIP16 = static_cast<DeviceType>(0x00030001u);

class HIP : public Device {
public:
  // Element type of tensors in device memory.  The public API is float in
  // every case; F16 / BF16 store 16-bit values and accumulate in fp32 (the
  // counterpart of devices::CUDA16, primitiv/devices/cuda16/device.h).
  enum class Storage : std::uint32_t { F32 = 0, F16 = 1, BF16 = 2 };

  // Number of HIP devices visible to this process.
  static std::uint32_t num_devices();

  // Throws primitiv::Error unless `device_id` exists and is a gfx950 device
  // with 64-wide wavefronts and at least 1 GiB of memory.
  static void assert_support(std::uint32_t device_id);

  // Same test as assert_support, reported as a boolean.
  static bool check_support(std::uint32_t device_id);

  explicit HIP(std::uint32_t device_id);
  HIP(std::uint32_t device_id, std::uint32_t rng_seed);
  HIP(std::uint32_t device_id, std::uint32_t rng_seed, Storage storage);
  ~HIP() override;

  void dump_description() const override;
  DeviceType type() const override {
    return storage_ == Storage::F32 ? DEVICE_TYPE_HIP : DEVICE_TYPE_HIP16;
  }
  Storage storage() const { return storage_; }

  // Gradient products whose contraction is cut between workgroups normally add
  // their tiles with atomics (right to rounding, bits depend on the order of
  // arrival).  With `on` they are added in a fixed order instead: the same bits
  // on every run, like the CPU devices, at some cost per backward call.
  void set_deterministic(bool on);

  // Matmul calls that follow one another and do not touch each other's
  // operands run on two streams at once (the default); what the caller observes
  // stays in the order of its calls.  Off: every launch on one stream.
  void set_overlap(bool on);

  // reset_tensor with the value 0 is only noted, and the gradient operation that
  // follows writes its result instead of adding it to the zeros (the default):
  // one launch per gradient of a backward pass instead of two, the same bits.
  // Off: every fill is launched when it is asked for.
  void set_deferred_zero_fill(bool on);

private:
  // ---- implemented -------------------------------------------------------
  std::shared_ptr<void> new_handle(const Shape &shape, std::size_t *const allocated_size) override;
  std::vector<float> tensor_to_vector_impl(const Tensor &x) override;
  void reset_tensor_impl(float k, Tensor &x) override;
  void reset_tensor_by_array_impl(const float values[], Tensor &x) override;
  void copy_tensor_impl(const Tensor &x, Tensor &y) override;
  void identity_impl(Tensor &y) override;
  void matmul_fw_impl(const Tensor &a, const Tensor &b, Tensor &y) override;
  void matmul_bw_impl(const Tensor &a, const Tensor &b, const Tensor &y, const Tensor &gy,
                      Tensor &ga, Tensor &gb) override;
  void batch_sum_fw_impl(const Tensor &x, Tensor &y) override;
  void inplace_add_impl(const Tensor &x, Tensor &y) override;
  void inplace_subtract_impl(const Tensor &x, Tensor &y) override;
  void inplace_multiply_const_impl(float k, Tensor &x) override;

  // random tensors: a Philox stream keyed by the seed; rng_offset_ is the position in it
  void random_bernoulli_impl(float p, Tensor &y) override;
  void random_uniform_impl(float lower, float upper, Tensor &y) override;
  void random_normal_impl(float mean, float sd, Tensor &y) override;
  void random_log_normal_impl(float mean, float sd, Tensor &y) override;

  // moving and reducing along one dimension
  std::vector<std::uint32_t> argmax_impl(const Tensor &x, std::uint32_t dim) override;
  std::vector<std::uint32_t> argmin_impl(const Tensor &x, std::uint32_t dim) override;
  void pick_fw_impl(const Tensor &x, const std::vector<std::uint32_t> &ids, std::uint32_t dim, Tensor &y) override;
  void slice_fw_impl(const Tensor &x, std::uint32_t dim, std::uint32_t offset, Tensor &y) override;
  void concat_fw_impl(const std::vector<const Tensor *> &xs, std::uint32_t dim, Tensor &y) override;
  void pick_bw_impl(const Tensor &gy, const std::vector<std::uint32_t> &ids, std::uint32_t dim, Tensor &gx) override;
  void slice_bw_impl(const Tensor &gy, std::uint32_t dim, std::uint32_t offset, Tensor &gx) override;
  void transpose_fw_impl(const Tensor &x, Tensor &y) override;
  void transpose_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, Tensor &gx) override;
  void permute_dims_fw_impl(const Tensor &x, const std::vector<std::uint32_t> &perm, Tensor &y) override;
  void permute_dims_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy,
                            const std::vector<std::uint32_t> &perm, Tensor &gx) override;
  void flip_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) override;
  void flip_bw_impl(const Tensor &gy, std::uint32_t dim, Tensor &gx) override;
  void max_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) override;
  void min_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) override;
  void sum_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) override;
  void logsumexp_fw_impl(const Tensor &x, std::uint32_t dim, Tensor &y) override;
  void max_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, std::uint32_t dim, Tensor &gx) override;
  void min_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, std::uint32_t dim, Tensor &gx) override;
  void broadcast_fw_impl(const Tensor &x, std::uint32_t dim, std::uint32_t size, Tensor &y) override;
  void batch_pick_fw_impl(const Tensor &x, const std::vector<std::uint32_t> &ids, Tensor &y) override;
  void batch_slice_fw_impl(const Tensor &x, std::uint32_t offset, Tensor &y) override;
  void batch_concat_fw_impl(const std::vector<const Tensor *> &xs, Tensor &y) override;
  void batch_pick_bw_impl(const Tensor &gy, const std::vector<std::uint32_t> &ids, Tensor &gx) override;
  void batch_slice_bw_impl(const Tensor &gy, std::uint32_t offset, Tensor &gx) override;

  // elementwise families (libphip operation codes select the member)
#define PHIP_DECL_X(name) \
  void name##_fw_impl(const Tensor &x, Tensor &y) override; \
  void name##_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, Tensor &gx) override;
#define PHIP_DECL_CONST(name, K) \
  void name##_fw_impl(const Tensor &x, K k, Tensor &y) override; \
  void name##_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, K k, Tensor &gx) override;
#define PHIP_DECL_SCALAR(name) \
  void name##_fw_impl(const Tensor &x, const Tensor &k, Tensor &y) override;
#define PHIP_DECL_AB(name) \
  void name##_fw_impl(const Tensor &a, const Tensor &b, Tensor &y) override; \
  void name##_bw_impl(const Tensor &a, const Tensor &b, const Tensor &y, const Tensor &gy, \
                      Tensor &ga, Tensor &gb) override;
  void negate_fw_impl(const Tensor &x, Tensor &y) override;
  PHIP_DECL_X(abs) PHIP_DECL_X(sqrt) PHIP_DECL_X(exp) PHIP_DECL_X(log) PHIP_DECL_X(tanh)
  PHIP_DECL_X(sigmoid) PHIP_DECL_X(softplus) PHIP_DECL_X(sin) PHIP_DECL_X(cos) PHIP_DECL_X(tan)
  PHIP_DECL_CONST(add_const, float) PHIP_DECL_CONST(subtract_const_r, float)
  PHIP_DECL_CONST(subtract_const_l, float) PHIP_DECL_CONST(multiply_const, float)
  PHIP_DECL_CONST(divide_const_r, float) PHIP_DECL_CONST(divide_const_l, float)
  PHIP_DECL_CONST(pow_const_r, float) PHIP_DECL_CONST(pow_const_l, float) PHIP_DECL_CONST(prelu, float)
  PHIP_DECL_CONST(elu, float) PHIP_DECL_CONST(pown, std::int32_t)
  PHIP_DECL_SCALAR(add_scalar) PHIP_DECL_SCALAR(subtract_scalar_r) PHIP_DECL_SCALAR(subtract_scalar_l)
  PHIP_DECL_SCALAR(multiply_scalar) PHIP_DECL_SCALAR(divide_scalar_r) PHIP_DECL_SCALAR(divide_scalar_l)
  PHIP_DECL_SCALAR(pow_scalar_r) PHIP_DECL_SCALAR(pow_scalar_l)
  PHIP_DECL_AB(add) PHIP_DECL_AB(subtract) PHIP_DECL_AB(multiply) PHIP_DECL_AB(divide) PHIP_DECL_AB(pow)
#undef PHIP_DECL_X
#undef PHIP_DECL_CONST
#undef PHIP_DECL_SCALAR
#undef PHIP_DECL_AB

  // ---- convolution and pooling ----------------------------------------------
  void conv2d_fw_impl(const Tensor &x, const Tensor &w, std::uint32_t padding0, std::uint32_t padding1,
                      std::uint32_t stride0, std::uint32_t stride1, std::uint32_t dilation0,
                      std::uint32_t dilation1, Tensor &y) override;
  void conv2d_bw_impl(const Tensor &x, const Tensor &w, const Tensor &y, const Tensor &gy,
                      std::uint32_t padding0, std::uint32_t padding1, std::uint32_t stride0,
                      std::uint32_t stride1, std::uint32_t dilation0, std::uint32_t dilation1,
                      Tensor &gx, Tensor &gw) override;
  void max_pool2d_fw_impl(const Tensor &x, std::uint32_t window0, std::uint32_t window1, std::uint32_t padding0,
                          std::uint32_t padding1, std::uint32_t stride0, std::uint32_t stride1,
                          Tensor &y) override;
  void max_pool2d_bw_impl(const Tensor &x, const Tensor &y, const Tensor &gy, std::uint32_t window0,
                          std::uint32_t window1, std::uint32_t padding0, std::uint32_t padding1,
                          std::uint32_t stride0, std::uint32_t stride1, Tensor &gx) override;

  // Bytes of device storage for `n` elements (16-bit storage rounds the
  // element count up to even, as devices::CUDA16 does).
  std::size_t storage_bytes(std::size_t n) const;

  std::uint32_t dev_id_;
  std::uint32_t rng_seed_;
  std::uint64_t rng_offset_;
  Storage storage_;
  // Declared before the pool so that it is destroyed after it: the pool's
  // deleter still needs the context while it frees its blocks.
  phip_ctx *ctx_;
  std::unique_ptr<MemoryPool> pool_;
};

// Half-storage device with the constructor shape of devices::CUDA16.
class HIP16 : public HIP {
public:
  explicit HIP16(std::uint32_t device_id);
  HIP16(std::uint32_t device_id, std::uint32_t rng_seed);
};

}  // namespace devices
}  // namespace primitiv

#endif  // PRIMITIV_DEVICES_HIP_DEVICE_H_
