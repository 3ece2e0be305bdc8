// Public entry points of RMSNorm; same routing as
// src/ops/rms_norm/operator.cc:21-142 of the reference, one device.
#include "amd/rms_norm_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateRMSNormDescriptor(infiniopHandle_t handle, infiniopRMSNormDescriptor_t *desc_ptr,
                                                            infiniopTensorDescriptor_t y_desc,
                                                            infiniopTensorDescriptor_t x_desc,
                                                            infiniopTensorDescriptor_t w_desc, float epsilon) {
    if (handle == nullptr || y_desc == nullptr || x_desc == nullptr || w_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateRMSNormDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                              reinterpret_cast<RMSNormAmdDescriptor_t *>(desc_ptr), y_desc, x_desc,
                                              w_desc, epsilon);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetRMSNormWorkspaceSize(infiniopRMSNormDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetRMSNormWorkspaceSize(reinterpret_cast<RMSNormAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopRMSNorm(infiniopRMSNormDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                            void *y, void const *x, void const *w, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdRMSNorm(reinterpret_cast<RMSNormAmdDescriptor_t>(desc), workspace, workspace_size, y, x, w, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyRMSNormDescriptor(infiniopRMSNormDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyRMSNormDescriptor(reinterpret_cast<RMSNormAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
