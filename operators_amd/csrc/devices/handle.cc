// infiniopCreateHandle / infiniopDestroyHandle for a library that carries the
// amd-gpu device only.  Argument checks and their order follow
// src/devices/handle.cc:16-46 of the reference; every other device number is
// answered the way the reference answers a device it was built without.
#include "amd/amd_handle.h"
#include "infiniop.h"

INFINIOP_C infiniopStatus_t infiniopCreateHandle(infiniopHandle_t *handle_ptr, Device device, int device_id) {
    if (handle_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (device_id < 0) {
        return STATUS_BAD_PARAM;
    }
    if (device == DevAmdGpu) {
        return createAmdHandle(reinterpret_cast<AmdHandle_t *>(handle_ptr), device_id);
    }
    return STATUS_BAD_DEVICE;
}

INFINIOP_C infiniopStatus_t infiniopDestroyHandle(infiniopHandle_t handle) {
    if (handle != nullptr && handle->device == DevAmdGpu) {
        return deleteAmdHandle(reinterpret_cast<AmdHandle_t>(handle));
    }
    return STATUS_BAD_DEVICE;
}
