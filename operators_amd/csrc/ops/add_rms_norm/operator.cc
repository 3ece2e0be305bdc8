// Public entry points of the fused Add + RMSNorm.  The reference has no such
// operator; the routing follows its dispatchers (for instance
// src/ops/rms_norm/operator.cc:21-142), one device.
#include "amd/add_rms_norm_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateAddRMSNormDescriptor(infiniopHandle_t handle, infiniopAddRMSNormDescriptor_t *desc_ptr,
                                                               infiniopTensorDescriptor_t y_desc,
                                                               infiniopTensorDescriptor_t c_desc,
                                                               infiniopTensorDescriptor_t a_desc,
                                                               infiniopTensorDescriptor_t b_desc,
                                                               infiniopTensorDescriptor_t w_desc, float epsilon) {
    if (handle == nullptr || y_desc == nullptr || c_desc == nullptr || a_desc == nullptr || b_desc == nullptr || w_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateAddRMSNormDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                              reinterpret_cast<AddRMSNormAmdDescriptor_t *>(desc_ptr), y_desc, c_desc,
                                                 a_desc, b_desc, w_desc, epsilon);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetAddRMSNormWorkspaceSize(infiniopAddRMSNormDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetAddRMSNormWorkspaceSize(reinterpret_cast<AddRMSNormAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopAddRMSNorm(infiniopAddRMSNormDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                               void *y, void *c, void const *a, void const *b, void const *w, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdAddRMSNorm(reinterpret_cast<AddRMSNormAmdDescriptor_t>(desc), workspace, workspace_size, y, c, a, b, w,
                                 stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyAddRMSNormDescriptor(infiniopAddRMSNormDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyAddRMSNormDescriptor(reinterpret_cast<AddRMSNormAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
