// Creation and destruction of the amd-gpu handle.  Counterpart of
// src/devices/cuda/cuda_handle.cc:3-47 in the reference: check the ordinal
// against the device count, bind the device, record the properties kernels
// are sized from.
#include "amd_handle.h"
#include "common_amd.h"
#include <new>

infiniopStatus_t createAmdHandle(AmdHandle_t *handle_ptr, int device_id) {
    int count = 0;
    AMD_CHECK_HIP(hipGetDeviceCount(&count), STATUS_BAD_DEVICE);
    if (device_id >= count) {
        return STATUS_BAD_DEVICE;
    }
    AMD_CHECK_HIP(hipSetDevice(device_id), STATUS_BAD_DEVICE);

    hipDeviceProp_t prop;
    AMD_CHECK_HIP(hipGetDeviceProperties(&prop, device_id), STATUS_BAD_DEVICE);
    // The kernels in this library exist as gfx950 code objects only.
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) {
        std::fprintf(stderr, "infiniop[amd-gpu]: device %d is %s; this library is built for gfx950 only\n",
                     device_id, prop.gcnArchName);
        return STATUS_BAD_DEVICE;
    }

    auto *ctx = new (std::nothrow) AmdContext{
        DevAmdGpu,
        device_id,
        prop.multiProcessorCount,
        static_cast<int>(prop.sharedMemPerBlock),
        prop.maxGridSize[0],
        prop.warpSize,
    };
    if (ctx == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *handle_ptr = ctx;
    return STATUS_SUCCESS;
}

infiniopStatus_t deleteAmdHandle(AmdHandle_t handle) {
    delete handle;
    return STATUS_SUCCESS;
}
