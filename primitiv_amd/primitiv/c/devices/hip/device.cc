#include <primitiv/c/devices/hip/device.h>
#include <primitiv/c/internal/internal.h>
#include <primitiv/devices/hip/device.h>

using primitiv::devices::HIP;
using primitiv::c::internal::to_c_ptr;

PRIMITIV_C_STATUS primitivCreateHipDevice(
    uint32_t device_id, primitivDevice_t **newobj) try {
  PRIMITIV_C_CHECK_NOT_NULL(newobj);
  *newobj = to_c_ptr(new HIP(device_id));
  return PRIMITIV_C_OK;
} PRIMITIV_C_HANDLE_EXCEPTIONS

PRIMITIV_C_STATUS primitivCreateHipDeviceWithSeed(
    uint32_t device_id, uint32_t rng_seed, primitivDevice_t **newobj) try {
  PRIMITIV_C_CHECK_NOT_NULL(newobj);
  *newobj = to_c_ptr(new HIP(device_id, rng_seed));
  return PRIMITIV_C_OK;
} PRIMITIV_C_HANDLE_EXCEPTIONS

PRIMITIV_C_STATUS primitivCreateHip16DeviceWithSeed(
    uint32_t device_id, uint32_t rng_seed, uint32_t use_bf16,
    primitivDevice_t **newobj) try {
  PRIMITIV_C_CHECK_NOT_NULL(newobj);
  *newobj = to_c_ptr(new HIP(
      device_id, rng_seed, use_bf16 ? HIP::Storage::BF16 : HIP::Storage::F16));
  return PRIMITIV_C_OK;
} PRIMITIV_C_HANDLE_EXCEPTIONS

PRIMITIV_C_STATUS primitivGetNumHipDevices(uint32_t *retval) try {
  PRIMITIV_C_CHECK_NOT_NULL(retval);
  *retval = HIP::num_devices();
  return PRIMITIV_C_OK;
} PRIMITIV_C_HANDLE_EXCEPTIONS
