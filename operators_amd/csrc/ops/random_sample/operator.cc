// Public entry points of RandomSample; same routing as
// src/ops/random_sample/operator.cc of the reference, one device.
#include "amd/random_sample_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateRandomSampleDescriptor(infiniopHandle_t handle,
                                                                 infiniopRandomSampleDescriptor_t *desc_ptr,
                                                                 infiniopTensorDescriptor_t result,
                                                                 infiniopTensorDescriptor_t probs) {
    if (handle == nullptr || result == nullptr || probs == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateRandomSampleDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                                   reinterpret_cast<RandomSampleAmdDescriptor_t *>(desc_ptr), result, probs);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetRandomSampleWorkspaceSize(infiniopRandomSampleDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetRandomSampleWorkspaceSize(reinterpret_cast<RandomSampleAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopRandomSample(infiniopRandomSampleDescriptor_t desc, void *workspace,
                                                 uint64_t workspace_size, void *result, void const *probs,
                                                 float random_val, float topp, int topk, float temperature,
                                                 void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdRandomSample(reinterpret_cast<RandomSampleAmdDescriptor_t>(desc), workspace, workspace_size,
                                   result, probs, random_val, topp, topk, temperature, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopRandomSampleNoAlloc(infiniopRandomSampleDescriptor_t desc, void *result, void const *probs,
                                                        float random_val, float topp, int topk, float temperature,
                                                        void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdRandomSampleNoAlloc(reinterpret_cast<RandomSampleAmdDescriptor_t>(desc), result, probs, random_val,
                                          topp, topk, temperature, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyRandomSampleDescriptor(infiniopRandomSampleDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyRandomSampleDescriptor(reinterpret_cast<RandomSampleAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
