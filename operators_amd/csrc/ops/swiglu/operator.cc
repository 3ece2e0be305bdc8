// Public entry points of SwiGLU; same routing as
// src/ops/swiglu/operator.cc:18-101 of the reference, one device.
#include "amd/swiglu_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateSwiGLUDescriptor(infiniopHandle_t handle, infiniopSwiGLUDescriptor_t *desc_ptr,
                                                           infiniopTensorDescriptor_t c_desc,
                                                           infiniopTensorDescriptor_t a_desc,
                                                           infiniopTensorDescriptor_t b_desc) {
    if (handle == nullptr || c_desc == nullptr || a_desc == nullptr || b_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateSwiGLUDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                             reinterpret_cast<SwiGLUAmdDescriptor_t *>(desc_ptr), c_desc, a_desc, b_desc);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopSwiGLU(infiniopSwiGLUDescriptor_t desc, void *c, void const *a, void const *b, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdSwiGLU(reinterpret_cast<SwiGLUAmdDescriptor_t>(desc), c, a, b, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroySwiGLUDescriptor(infiniopSwiGLUDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroySwiGLUDescriptor(reinterpret_cast<SwiGLUAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
