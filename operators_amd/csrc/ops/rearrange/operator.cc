// Public entry points of Rearrange; same routing as
// src/ops/rearrange/operator.cc of the reference, one device.
#include "amd/rearrange_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateRearrangeDescriptor(infiniopHandle_t handle, infiniopRearrangeDescriptor_t *desc_ptr,
                                                              infiniopTensorDescriptor_t dst, infiniopTensorDescriptor_t src) {
    if (handle == nullptr || dst == nullptr || src == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateRearrangeDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                                reinterpret_cast<RearrangeAmdDescriptor_t *>(desc_ptr), dst, src);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopRearrange(infiniopRearrangeDescriptor_t desc, void *dst, void const *src, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdRearrange(reinterpret_cast<RearrangeAmdDescriptor_t>(desc), dst, src, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyRearrangeDescriptor(infiniopRearrangeDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyRearrangeDescriptor(reinterpret_cast<RearrangeAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
