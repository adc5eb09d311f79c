#ifndef PRIMITIV_C_DEVICES_HIP_DEVICE_H_
#define PRIMITIV_C_DEVICES_HIP_DEVICE_H_

#include <primitiv/c/define.h>
#include <primitiv/c/device.h>

/**
 * Creates a new Device object on an AMD MI355X (gfx950) GPU.
 * @param device_id ID of the physical GPU.
 * @param newobj Pointer to receive a handler.
 * @return Status code.
 * @remarks The random number generator is initialized using
 *          `std::random_device`.
 */
PRIMITIV_C_API PRIMITIV_C_STATUS primitivCreateHipDevice(
    uint32_t device_id, primitivDevice_t **newobj);

/**
 * Creates a new Device object on an AMD MI355X (gfx950) GPU.
 * @param device_id ID of the physical GPU.
 * @param rng_seed The seed value of the random number generator.
 * @param newobj Pointer to receive a handler.
 * @return Status code.
 */
PRIMITIV_C_API PRIMITIV_C_STATUS primitivCreateHipDeviceWithSeed(
    uint32_t device_id, uint32_t rng_seed, primitivDevice_t **newobj);

/**
 * Creates a half-storage Device object (16-bit tensors, fp32 accumulation).
 * @param device_id ID of the physical GPU.
 * @param rng_seed The seed value of the random number generator.
 * @param use_bf16 0 for IEEE fp16 storage, non-zero for bfloat16 storage.
 * @param newobj Pointer to receive a handler.
 * @return Status code.
 */
PRIMITIV_C_API PRIMITIV_C_STATUS primitivCreateHip16DeviceWithSeed(
    uint32_t device_id, uint32_t rng_seed, uint32_t use_bf16,
    primitivDevice_t **newobj);

/**
 * Retrieves the number of HIP devices visible to this process.
 * @param retval Pointer to receive the number of devices.
 * @return Status code.
 */
PRIMITIV_C_API PRIMITIV_C_STATUS primitivGetNumHipDevices(uint32_t *retval);

#endif  // PRIMITIV_C_DEVICES_HIP_DEVICE_H_
