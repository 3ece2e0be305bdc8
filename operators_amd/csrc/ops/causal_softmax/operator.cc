// Public entry points of CausalSoftmax; same routing as
// src/ops/causal_softmax/operator.cc:21-130 of the reference, one device.
#include "amd/causal_softmax_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateCausalSoftmaxDescriptor(infiniopHandle_t handle,
                                                                  infiniopCausalSoftmaxDescriptor_t *desc_ptr,
                                                                  infiniopTensorDescriptor_t y_desc) {
    if (handle == nullptr || y_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateCausalSoftmaxDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                                    reinterpret_cast<CausalSoftmaxAmdDescriptor_t *>(desc_ptr), y_desc);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetCausalSoftmaxWorkspaceSize(infiniopCausalSoftmaxDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetCausalSoftmaxWorkspaceSize(reinterpret_cast<CausalSoftmaxAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopCausalSoftmax(infiniopCausalSoftmaxDescriptor_t desc, void *workspace,
                                                  uint64_t workspace_size, void *data, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdCausalSoftmax(reinterpret_cast<CausalSoftmaxAmdDescriptor_t>(desc), workspace, workspace_size, data, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyCausalSoftmaxDescriptor(infiniopCausalSoftmaxDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyCausalSoftmaxDescriptor(reinterpret_cast<CausalSoftmaxAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
