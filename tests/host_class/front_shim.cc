// C entry points over primitiv's own C++ front (primitiv::Device, primitiv::Tensor),
// TEST INFRASTRUCTURE ONLY: they let a Python test drive the public, non-virtual
// methods of Device (primitiv/core/device.h:60-366) on a device object, so that the
// calls reach devices::HIP's virtuals exactly the way Graph / Tensor / Parameter
// code reaches them.  Handles are primitiv's own objects: a Device* created by
// the C API constructors (primitiv/c/devices/hip/device.h) is passed in as is
// (the C API's primitivDevice_t* is that pointer, primitiv/c/internal/internal.h),
// tensors are heap-allocated primitiv::Tensor.
//
// Every function returns 0, or 1 after recording the exception's message.
#include <algorithm>
#include <cstdint>
#include <cstring>
#include <map>
#include <string>
#include <vector>

#include <primitiv/core/device.h>
#include <primitiv/core/error.h>
#include <primitiv/core/functions.h>
#include <primitiv/core/graph.h>
#include <primitiv/core/optimizer_impl.h>
#include <primitiv/core/parameter.h>
#include <primitiv/core/shape.h>
#include <primitiv/core/tensor.h>
#include <primitiv/devices/naive/device.h>
#include <primitiv/devices/hip/device.h>

using primitiv::Device;
using primitiv::Shape;
using primitiv::Tensor;
typedef std::uint32_t U32;

namespace {

thread_local std::string g_message;

#define HC_TRY try {
#define HC_END                                 \
  return 0;                                    \
  }                                            \
  catch (const std::exception &e) {            \
    g_message = e.what();                      \
    return 1;                                  \
  }                                            \
  catch (...) {                                \
    g_message = "unknown exception";           \
    return 1;                                  \
  }

Shape make_shape(const U32 *dims, U32 ndims, U32 batch) {
  return Shape(std::vector<U32>(dims, dims + ndims), batch);
}

int unknown(const char *family, const char *name) {
  g_message = std::string("front_shim: no ") + family + " operation named " + name;
  return 1;
}

typedef Tensor (Device::*FwX)(const Tensor &);
typedef void (Device::*BwX)(const Tensor &, const Tensor &, const Tensor &, Tensor &);
typedef Tensor (Device::*FwXK)(const Tensor &, float);
typedef void (Device::*BwXK)(const Tensor &, const Tensor &, const Tensor &, float, Tensor &);
typedef Tensor (Device::*FwAB)(const Tensor &, const Tensor &);
typedef void (Device::*BwAB)(const Tensor &, const Tensor &, const Tensor &, const Tensor &, Tensor &, Tensor &);
typedef Tensor (Device::*FwXDim)(const Tensor &, U32);
typedef void (Device::*BwXDim)(const Tensor &, const Tensor &, const Tensor &, U32, Tensor &);

const std::map<std::string, FwX> kFwX = {
  {"negate", &Device::negate_fw}, {"abs", &Device::abs_fw}, {"sqrt", &Device::sqrt_fw}, {"exp", &Device::exp_fw},
  {"log", &Device::log_fw}, {"tanh", &Device::tanh_fw}, {"sigmoid", &Device::sigmoid_fw},
  {"softplus", &Device::softplus_fw}, {"sin", &Device::sin_fw}, {"cos", &Device::cos_fw}, {"tan", &Device::tan_fw},
  {"transpose", &Device::transpose_fw}, {"batch_sum", &Device::batch_sum_fw}, {"copy_tensor", &Device::copy_tensor},
};
const std::map<std::string, BwX> kBwX = {
  {"abs", &Device::abs_bw}, {"sqrt", &Device::sqrt_bw}, {"exp", &Device::exp_bw}, {"log", &Device::log_bw},
  {"tanh", &Device::tanh_bw}, {"sigmoid", &Device::sigmoid_bw}, {"softplus", &Device::softplus_bw},
  {"sin", &Device::sin_bw}, {"cos", &Device::cos_bw}, {"tan", &Device::tan_bw}, {"transpose", &Device::transpose_bw},
};
const std::map<std::string, FwXK> kFwXK = {
  {"add_const", &Device::add_const_fw}, {"subtract_const_r", &Device::subtract_const_r_fw},
  {"subtract_const_l", &Device::subtract_const_l_fw}, {"multiply_const", &Device::multiply_const_fw},
  {"divide_const_r", &Device::divide_const_r_fw}, {"divide_const_l", &Device::divide_const_l_fw},
  {"pow_const_r", &Device::pow_const_r_fw}, {"pow_const_l", &Device::pow_const_l_fw}, {"prelu", &Device::prelu_fw},
  {"elu", &Device::elu_fw},
};
const std::map<std::string, BwXK> kBwXK = {
  {"add_const", &Device::add_const_bw}, {"subtract_const_r", &Device::subtract_const_r_bw},
  {"subtract_const_l", &Device::subtract_const_l_bw}, {"multiply_const", &Device::multiply_const_bw},
  {"divide_const_r", &Device::divide_const_r_bw}, {"divide_const_l", &Device::divide_const_l_bw},
  {"pow_const_r", &Device::pow_const_r_bw}, {"pow_const_l", &Device::pow_const_l_bw}, {"prelu", &Device::prelu_bw},
  {"elu", &Device::elu_bw},
};
const std::map<std::string, FwAB> kFwAB = {
  {"add", &Device::add_fw}, {"subtract", &Device::subtract_fw}, {"multiply", &Device::multiply_fw},
  {"divide", &Device::divide_fw}, {"pow", &Device::pow_fw}, {"matmul", &Device::matmul_fw},
  {"add_scalar", &Device::add_scalar_fw}, {"subtract_scalar_r", &Device::subtract_scalar_r_fw},
  {"subtract_scalar_l", &Device::subtract_scalar_l_fw}, {"multiply_scalar", &Device::multiply_scalar_fw},
  {"divide_scalar_r", &Device::divide_scalar_r_fw}, {"divide_scalar_l", &Device::divide_scalar_l_fw},
  {"pow_scalar_r", &Device::pow_scalar_r_fw}, {"pow_scalar_l", &Device::pow_scalar_l_fw},
};
const std::map<std::string, BwAB> kBwAB = {
  {"add", &Device::add_bw}, {"subtract", &Device::subtract_bw}, {"multiply", &Device::multiply_bw},
  {"divide", &Device::divide_bw}, {"pow", &Device::pow_bw}, {"matmul", &Device::matmul_bw},
};
const std::map<std::string, FwXDim> kFwXDim = {
  {"max", &Device::max_fw}, {"min", &Device::min_fw}, {"sum", &Device::sum_fw}, {"logsumexp", &Device::logsumexp_fw},
  {"flip", &Device::flip_fw},
};
const std::map<std::string, BwXDim> kBwXDim = {
  {"max", &Device::max_bw}, {"min", &Device::min_bw},
};

std::vector<const Tensor *> tensor_list(Tensor *const *xs, U32 n) { return std::vector<const Tensor *>(xs, xs + n); }

}  // namespace

extern "C" {

const char *hc_last_error() { return g_message.c_str(); }

// ---- devices (the C++ constructors; the C API constructors are called from the test directly) ----
// storage: 0 fp32, 1 fp16, 2 bf16
int hc_device_new(U32 device_id, U32 seed, U32 storage, Device **out) {
  HC_TRY
  *out = new primitiv::devices::HIP(device_id, seed, static_cast<primitiv::devices::HIP::Storage>(storage));
  HC_END
}
// primitiv's own plain CPU device (primitiv/devices/naive/device.h:15-28), to check the oracle against
int hc_device_new_naive(U32 seed, Device **out) {
  HC_TRY
  *out = new primitiv::devices::Naive(seed);
  HC_END
}
int hc_device_new_hip16(U32 device_id, U32 seed, Device **out) {
  HC_TRY
  *out = new primitiv::devices::HIP16(device_id, seed);
  HC_END
}
int hc_device_delete(Device *dev) {
  HC_TRY
  delete dev;
  HC_END
}
int hc_device_type(Device *dev, U32 *out) {
  HC_TRY
  *out = static_cast<U32>(dev->type());
  HC_END
}
int hc_device_dump_description(Device *dev) {
  HC_TRY
  dev->dump_description();
  HC_END
}
int hc_device_set_deterministic(Device *dev, int on) {
  HC_TRY
  static_cast<primitiv::devices::HIP *>(dev)->set_deterministic(on != 0);
  HC_END
}
int hc_device_set_overlap(Device *dev, int on) {
  HC_TRY
  static_cast<primitiv::devices::HIP *>(dev)->set_overlap(on != 0);
  HC_END
}
int hc_device_set_deferred_zero_fill(Device *dev, int on) {
  HC_TRY
  static_cast<primitiv::devices::HIP *>(dev)->set_deferred_zero_fill(on != 0);
  HC_END
}
int hc_num_devices(U32 *out) {
  HC_TRY
  *out = primitiv::devices::HIP::num_devices();
  HC_END
}
int hc_check_support(U32 device_id, int *out) {
  HC_TRY
  *out = primitiv::devices::HIP::check_support(device_id) ? 1 : 0;
  HC_END
}
int hc_assert_support(U32 device_id) {
  HC_TRY
  primitiv::devices::HIP::assert_support(device_id);
  HC_END
}

// ---- tensors --------------------------------------------------------------------------------
int hc_tensor_by_array(Device *dev, const U32 *dims, U32 ndims, U32 batch, const float *values, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->new_tensor_by_array(make_shape(dims, ndims, batch), values));
  HC_END
}
int hc_tensor_by_vector(Device *dev, const U32 *dims, U32 ndims, U32 batch, const float *values, size_t n,
                        Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->new_tensor_by_vector(make_shape(dims, ndims, batch), std::vector<float>(values, values + n)));
  HC_END
}
int hc_tensor_by_constant(Device *dev, const U32 *dims, U32 ndims, U32 batch, float k, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->new_tensor_by_constant(make_shape(dims, ndims, batch), k));
  HC_END
}
int hc_tensor_invalid(Tensor **out) {
  HC_TRY
  *out = new Tensor();
  HC_END
}
// a second Tensor object on the same memory: the copy constructor shares the handle
int hc_tensor_share(const Tensor *x, Tensor **out) {
  HC_TRY
  *out = new Tensor(*x);
  HC_END
}
int hc_tensor_assign(Tensor *dst, const Tensor *src) {
  HC_TRY
  *dst = *src;
  HC_END
}
int hc_tensor_delete(Tensor *x) {
  HC_TRY
  delete x;
  HC_END
}
int hc_tensor_valid(const Tensor *x, int *out) {
  HC_TRY
  *out = x->valid() ? 1 : 0;
  HC_END
}
// dims must hold 8 entries
int hc_tensor_shape(const Tensor *x, U32 *dims, U32 *depth, U32 *batch, U32 *size) {
  HC_TRY
  const Shape s = x->shape();
  *depth = s.depth();
  for (U32 i = 0; i < 8; ++i) dims[i] = s[i];
  *batch = s.batch();
  *size = s.size();
  HC_END
}
int hc_tensor_to_vector(const Tensor *x, float *out) {
  HC_TRY
  const std::vector<float> v = x->to_vector();
  std::memcpy(out, v.data(), sizeof(float) * v.size());
  HC_END
}
int hc_tensor_to_float(const Tensor *x, float *out) {
  HC_TRY
  *out = x->to_float();
  HC_END
}
int hc_tensor_reset(Tensor *x, float k) {
  HC_TRY
  x->reset(k);
  HC_END
}
int hc_tensor_reset_by_array(Tensor *x, const float *values) {
  HC_TRY
  x->reset_by_array(values);
  HC_END
}
int hc_tensor_argmax(const Tensor *x, U32 dim, U32 *out) {
  HC_TRY
  const std::vector<U32> v = x->argmax(dim);
  std::memcpy(out, v.data(), sizeof(U32) * v.size());
  HC_END
}
int hc_tensor_argmin(const Tensor *x, U32 dim, U32 *out) {
  HC_TRY
  const std::vector<U32> v = x->argmin(dim);
  std::memcpy(out, v.data(), sizeof(U32) * v.size());
  HC_END
}
// Tensor's own in-place operators (primitiv/core/tensor.cc:61-89)
int hc_tensor_inplace_add(Tensor *y, const Tensor *x) {
  HC_TRY
  y->inplace_add(*x);
  HC_END
}
int hc_tensor_inplace_subtract(Tensor *y, const Tensor *x) {
  HC_TRY
  y->inplace_subtract(*x);
  HC_END
}
int hc_tensor_inplace_multiply_const(Tensor *x, float k) {
  HC_TRY
  x->inplace_multiply_const(k);
  HC_END
}

// ---- Device front, one entry per signature; `name` selects the member --------------------------
int hc_fw_x(Device *dev, const char *name, const Tensor *x, Tensor **out) {
  HC_TRY
  auto it = kFwX.find(name);
  if (it == kFwX.end()) return unknown("fw_x", name);
  *out = new Tensor((dev->*(it->second))(*x));
  HC_END
}
int hc_bw_x(Device *dev, const char *name, const Tensor *x, const Tensor *y, const Tensor *gy, Tensor *gx) {
  HC_TRY
  auto it = kBwX.find(name);
  if (it == kBwX.end()) return unknown("bw_x", name);
  (dev->*(it->second))(*x, *y, *gy, *gx);
  HC_END
}
int hc_fw_xk(Device *dev, const char *name, const Tensor *x, float k, Tensor **out) {
  HC_TRY
  auto it = kFwXK.find(name);
  if (it == kFwXK.end()) return unknown("fw_xk", name);
  *out = new Tensor((dev->*(it->second))(*x, k));
  HC_END
}
int hc_bw_xk(Device *dev, const char *name, const Tensor *x, const Tensor *y, const Tensor *gy, float k, Tensor *gx) {
  HC_TRY
  auto it = kBwXK.find(name);
  if (it == kBwXK.end()) return unknown("bw_xk", name);
  (dev->*(it->second))(*x, *y, *gy, k, *gx);
  HC_END
}
int hc_pown_fw(Device *dev, const Tensor *x, std::int32_t k, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->pown_fw(*x, k));
  HC_END
}
int hc_pown_bw(Device *dev, const Tensor *x, const Tensor *y, const Tensor *gy, std::int32_t k, Tensor *gx) {
  HC_TRY
  dev->pown_bw(*x, *y, *gy, k, *gx);
  HC_END
}
int hc_fw_ab(Device *dev, const char *name, const Tensor *a, const Tensor *b, Tensor **out) {
  HC_TRY
  auto it = kFwAB.find(name);
  if (it == kFwAB.end()) return unknown("fw_ab", name);
  *out = new Tensor((dev->*(it->second))(*a, *b));
  HC_END
}
int hc_bw_ab(Device *dev, const char *name, const Tensor *a, const Tensor *b, const Tensor *y, const Tensor *gy,
             Tensor *ga, Tensor *gb) {
  HC_TRY
  auto it = kBwAB.find(name);
  if (it == kBwAB.end()) return unknown("bw_ab", name);
  (dev->*(it->second))(*a, *b, *y, *gy, *ga, *gb);
  HC_END
}
int hc_fw_xdim(Device *dev, const char *name, const Tensor *x, U32 dim, Tensor **out) {
  HC_TRY
  auto it = kFwXDim.find(name);
  if (it == kFwXDim.end()) return unknown("fw_xdim", name);
  *out = new Tensor((dev->*(it->second))(*x, dim));
  HC_END
}
int hc_bw_xdim(Device *dev, const char *name, const Tensor *x, const Tensor *y, const Tensor *gy, U32 dim, Tensor *gx) {
  HC_TRY
  auto it = kBwXDim.find(name);
  if (it == kBwXDim.end()) return unknown("bw_xdim", name);
  (dev->*(it->second))(*x, *y, *gy, dim, *gx);
  HC_END
}
int hc_flip_bw(Device *dev, const Tensor *gy, U32 dim, Tensor *gx) {
  HC_TRY
  dev->flip_bw(*gy, dim, *gx);
  HC_END
}
int hc_identity(Device *dev, U32 size, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->identity(size));
  HC_END
}
int hc_inplace_add(Device *dev, const Tensor *x, Tensor *y) {
  HC_TRY
  dev->inplace_add(*x, *y);
  HC_END
}
int hc_inplace_subtract(Device *dev, const Tensor *x, Tensor *y) {
  HC_TRY
  dev->inplace_subtract(*x, *y);
  HC_END
}
int hc_inplace_multiply_const(Device *dev, float k, Tensor *x) {
  HC_TRY
  dev->inplace_multiply_const(k, *x);
  HC_END
}
int hc_pick_fw(Device *dev, const Tensor *x, const U32 *ids, U32 n_ids, U32 dim, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->pick_fw(*x, std::vector<U32>(ids, ids + n_ids), dim));
  HC_END
}
int hc_pick_bw(Device *dev, const Tensor *gy, const U32 *ids, U32 n_ids, U32 dim, Tensor *gx) {
  HC_TRY
  dev->pick_bw(*gy, std::vector<U32>(ids, ids + n_ids), dim, *gx);
  HC_END
}
int hc_slice_fw(Device *dev, const Tensor *x, U32 dim, U32 lower, U32 upper, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->slice_fw(*x, dim, lower, upper));
  HC_END
}
int hc_slice_bw(Device *dev, const Tensor *gy, U32 dim, U32 offset, Tensor *gx) {
  HC_TRY
  dev->slice_bw(*gy, dim, offset, *gx);
  HC_END
}
int hc_concat_fw(Device *dev, Tensor *const *xs, U32 n, U32 dim, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->concat_fw(tensor_list(xs, n), dim));
  HC_END
}
int hc_permute_dims_fw(Device *dev, const Tensor *x, const U32 *perm, U32 n, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->permute_dims_fw(*x, std::vector<U32>(perm, perm + n)));
  HC_END
}
int hc_permute_dims_bw(Device *dev, const Tensor *x, const Tensor *y, const Tensor *gy, const U32 *perm, U32 n,
                       Tensor *gx) {
  HC_TRY
  dev->permute_dims_bw(*x, *y, *gy, std::vector<U32>(perm, perm + n), *gx);
  HC_END
}
int hc_broadcast_fw(Device *dev, const Tensor *x, U32 dim, U32 size, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->broadcast_fw(*x, dim, size));
  HC_END
}
int hc_batch_pick_fw(Device *dev, const Tensor *x, const U32 *ids, U32 n_ids, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->batch_pick_fw(*x, std::vector<U32>(ids, ids + n_ids)));
  HC_END
}
int hc_batch_pick_bw(Device *dev, const Tensor *gy, const U32 *ids, U32 n_ids, Tensor *gx) {
  HC_TRY
  dev->batch_pick_bw(*gy, std::vector<U32>(ids, ids + n_ids), *gx);
  HC_END
}
int hc_batch_slice_fw(Device *dev, const Tensor *x, U32 lower, U32 upper, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->batch_slice_fw(*x, lower, upper));
  HC_END
}
int hc_batch_slice_bw(Device *dev, const Tensor *gy, U32 offset, Tensor *gx) {
  HC_TRY
  dev->batch_slice_bw(*gy, offset, *gx);
  HC_END
}
int hc_batch_concat_fw(Device *dev, Tensor *const *xs, U32 n, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->batch_concat_fw(tensor_list(xs, n)));
  HC_END
}
// kind: 0 uniform(p0, p1), 1 bernoulli(p0), 2 normal(p0, p1), 3 log_normal(p0, p1)
int hc_random(Device *dev, int kind, const U32 *dims, U32 ndims, U32 batch, float p0, float p1, Tensor **out) {
  HC_TRY
  const Shape s = make_shape(dims, ndims, batch);
  switch (kind) {
    case 0: *out = new Tensor(dev->random_uniform(s, p0, p1)); break;
    case 1: *out = new Tensor(dev->random_bernoulli(s, p0)); break;
    case 2: *out = new Tensor(dev->random_normal(s, p0, p1)); break;
    case 3: *out = new Tensor(dev->random_log_normal(s, p0, p1)); break;
    default: return unknown("random", "kind");
  }
  HC_END
}
// p = padding0, padding1, stride0, stride1, dilation0, dilation1
int hc_conv2d_fw(Device *dev, const Tensor *x, const Tensor *w, const U32 *p, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->conv2d_fw(*x, *w, p[0], p[1], p[2], p[3], p[4], p[5]));
  HC_END
}
int hc_conv2d_bw(Device *dev, const Tensor *x, const Tensor *w, const Tensor *y, const Tensor *gy, const U32 *p,
                 Tensor *gx, Tensor *gw) {
  HC_TRY
  dev->conv2d_bw(*x, *w, *y, *gy, p[0], p[1], p[2], p[3], p[4], p[5], *gx, *gw);
  HC_END
}
// p = window0, window1, padding0, padding1, stride0, stride1
int hc_max_pool2d_fw(Device *dev, const Tensor *x, const U32 *p, Tensor **out) {
  HC_TRY
  *out = new Tensor(dev->max_pool2d_fw(*x, p[0], p[1], p[2], p[3], p[4], p[5]));
  HC_END
}
int hc_max_pool2d_bw(Device *dev, const Tensor *x, const Tensor *y, const Tensor *gy, const U32 *p, Tensor *gx) {
  HC_TRY
  dev->max_pool2d_bw(*x, *y, *gy, p[0], p[1], p[2], p[3], p[4], p[5], *gx);
  HC_END
}

// The reference's "dangling tensor" scenario (test/cuda_device_test.cc:66-78): a tensor outlives
// the device object it came from and is destroyed afterwards.
int hc_scenario_tensor_outlives_device(U32 storage) {
  HC_TRY
  Tensor x1;
  {
    primitiv::devices::HIP dev(0, 1, static_cast<primitiv::devices::HIP::Storage>(storage));
    x1 = dev.new_tensor_by_constant(Shape(), 0);
  }
  HC_END
}

// A small training step with primitiv's own Graph / Node / Parameter / Optimizer on `dev`:
// the two-layer perceptron on the four XOR samples (the network of the reference's graph
// test, test/graph_test.cc:362-435), loss = sum over the minibatch of (y - t)^2.
//   values:  the 14 node values in order of creation, concatenated (62 floats)
//   grads:   gradients of w1 (4), b1 (2), w2 (2), b2 (1) after backward
//   updated: the same parameters after one SGD step with learning rate `eta`
int hc_scenario_xor_training_step(Device *dev, float eta, float *values, float *grads, float *updated) {
  HC_TRY
  namespace F = primitiv::functions;
  using primitiv::Node;
  using primitiv::Parameter;
  Device::set_default(*dev);
  Parameter w1({2, 2}, std::vector<float>{1, -1, 1, -1});
  Parameter b1({2}, std::vector<float>{-1, -1});
  Parameter w2({1, 2}, std::vector<float>{1, 1});
  Parameter b2({}, std::vector<float>{1});
  primitiv::optimizers::SGD opt(eta);
  opt.add(w1, b1, w2, b2);
  opt.reset_gradients();

  primitiv::Graph g;
  primitiv::Graph::set_default(g);
  std::vector<Node> n;
  n.push_back(F::input<Node>(Shape({2}, 4), {1, 1, 1, -1, -1, 1, -1, -1}));
  n.push_back(F::parameter<Node>(w1));
  n.push_back(F::parameter<Node>(b1));
  n.push_back(F::parameter<Node>(w2));
  n.push_back(F::parameter<Node>(b2));
  n.push_back(F::matmul(n[1], n[0]));
  n.push_back(n[5] + n[2]);
  n.push_back(F::tanh(n[6]));
  n.push_back(F::matmul(n[3], n[7]));
  n.push_back(n[8] + n[4]);
  n.push_back(F::input<Node>(Shape({}, 4), {1, -1, -1, 1}));
  n.push_back(n[9] - n[10]);
  n.push_back(n[11] * n[11]);
  n.push_back(F::batch::sum(n[12]));
  g.forward(n.back());
  for (const Node &node : n) {
    const std::vector<float> v = node.to_vector();
    values = std::copy(v.begin(), v.end(), values);
  }
  g.backward(n.back());
  for (Parameter *p : {&w1, &b1, &w2, &b2}) {
    const std::vector<float> v = p->gradient().to_vector();
    grads = std::copy(v.begin(), v.end(), grads);
  }
  opt.update();
  for (Parameter *p : {&w1, &b1, &w2, &b2}) {
    const std::vector<float> v = p->value().to_vector();
    updated = std::copy(v.begin(), v.end(), updated);
  }
  HC_END
}

// One LSTM step with primitiv's own Graph on `dev`, written as the reference's graph tests write it
// (test/graph_test.cc:437-551 CheckLSTM with eight weight matrices and four biases when `stacked`
// is 0, :553-646 CheckConcatLSTM with stacked weights and slices otherwise).  `params` holds the
// parameters' initial values in the order the test declares them (40 floats either way).
//   losses: the 4 values of the loss node;  sum_loss: batch::sum(sum(loss, 0));
//   num_operators: what the graph counts;  grads: the parameters' gradients, same order as `params`.
int hc_scenario_lstm_step(Device *dev, int stacked, const float *params, const float *x_values, const float *h_values,
                          float *losses, float *sum_loss, U32 *num_operators, float *grads) {
  HC_TRY
  namespace F = primitiv::functions;
  using primitiv::Node;
  using primitiv::Parameter;
  Device::set_default(*dev);
  std::vector<Parameter *> ps;
  auto make = [&](const Shape &shape) {
    const U32 n = shape.size();
    ps.push_back(new Parameter(shape, std::vector<float>(params, params + n)));
    params += n;
    return ps.back();
  };
  struct Cleanup {
    std::vector<Parameter *> &v;
    ~Cleanup() { for (Parameter *p : v) delete p; }
  } cleanup{ps};

  primitiv::Graph g;
  primitiv::Graph::set_default(g);
  Node loss_node, total;
  const std::vector<float> xv(x_values, x_values + 4), hv(h_values, h_values + 4);
  if (!stacked) {
    for (int k = 0; k < 8; ++k) make(Shape({2, 2}));
    for (int k = 0; k < 4; ++k) make(Shape({2}));
    for (Parameter *p : ps) p->reset_gradient();
    const Node x = F::input<Node>(Shape({2}, 2), xv);
    const Node h = F::input<Node>(Shape({2}, 2), hv);
    const Node c = F::zeros<Node>({2});
    std::vector<Node> n;
    for (Parameter *p : ps) n.push_back(F::parameter<Node>(*p));
    const Node i = F::sigmoid(F::matmul(n[0], x) + F::matmul(n[4], h) + n[8]);
    const Node f = F::sigmoid(F::matmul(n[1], x) + F::matmul(n[5], h) + n[9]);
    const Node o = F::sigmoid(F::matmul(n[2], x) + F::matmul(n[6], h) + n[10]);
    const Node j = F::tanh(F::matmul(n[3], x) + F::matmul(n[7], h) + n[11]);
    const Node cc = f * c + i * j;
    const Node hh = o * F::tanh(cc);
    const Node t = F::zeros<Node>({2});
    const Node diff = hh - t;
    loss_node = diff * diff;
    total = F::batch::sum(F::sum(loss_node, 0));
  } else {
    make(Shape({8, 2}));
    make(Shape({8, 2}));
    make(Shape({8}));
    for (Parameter *p : ps) p->reset_gradient();
    const Node x = F::input<Node>(Shape({2}, 2), xv);
    const Node h = F::input<Node>(Shape({2}, 2), hv);
    const Node c = F::zeros<Node>({2});
    const Node Wx = F::parameter<Node>(*ps[0]);
    const Node Wh = F::parameter<Node>(*ps[1]);
    const Node b = F::parameter<Node>(*ps[2]);
    const Node u = F::matmul(Wx, x) + F::matmul(Wh, h) + b;
    const Node i = F::sigmoid(F::slice(u, 0, 0, 2));
    const Node f = F::sigmoid(F::slice(u, 0, 2, 4));
    const Node o = F::sigmoid(F::slice(u, 0, 4, 6));
    const Node j = F::tanh(F::slice(u, 0, 6, 8));
    const Node cc = f * c + i * j;
    const Node hh = o * F::tanh(cc);
    const Node t = F::zeros<Node>({2});
    const Node diff = hh - t;
    loss_node = diff * diff;
    total = F::batch::sum(F::sum(loss_node, 0));
  }
  *num_operators = g.num_operators();
  const std::vector<float> lv = g.forward(loss_node).to_vector();
  std::copy(lv.begin(), lv.end(), losses);
  *sum_loss = g.forward(total).to_float();
  total.backward();
  for (Parameter *p : ps) {
    const std::vector<float> v = p->gradient().to_vector();
    grads = std::copy(v.begin(), v.end(), grads);
  }
  HC_END
}

// Copies between a host device of the reference and `dev`, both ways (test/tensor_forward_test.cc:67-84):
// out receives the values after naive -> dev -> naive.
int hc_scenario_copy_through_naive(Device *dev, const float *values, U32 n, float *out) {
  HC_TRY
  primitiv::devices::Naive naive(1);
  const Tensor x = naive.new_tensor_by_vector(Shape({n}), std::vector<float>(values, values + n));
  const Tensor on_dev = dev->copy_tensor(x);
  if (&on_dev.device() != dev) PRIMITIV_THROW_ERROR("the copy does not live on the destination device");
  const Tensor back = naive.copy_tensor(on_dev);
  const std::vector<float> v = back.to_vector();
  std::copy(v.begin(), v.end(), out);
  HC_END
}

}  // extern "C"
