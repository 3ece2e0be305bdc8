// Public entry points of RoPE; same routing as
// src/ops/rotary_embedding/operator.cc:24-151 of the reference, one device.
// The public descriptor type is opaque; like every descriptor it starts with
// its Device.
#include "amd/rotary_embedding_amd.h"

struct RoPEDescriptor {
    Device device;
};

INFINIOP_C infiniopStatus_t infiniopCreateRoPEDescriptor(infiniopHandle_t handle, infiniopRoPEDescriptor_t *desc_ptr,
                                                         infiniopTensorDescriptor_t t, infiniopTensorDescriptor_t pos_ids,
                                                         infiniopTensorDescriptor_t sin_table,
                                                         infiniopTensorDescriptor_t cos_table) {
    if (handle == nullptr || t == nullptr || pos_ids == nullptr || sin_table == nullptr || cos_table == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateRoPEDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                           reinterpret_cast<RoPEAmdDescriptor_t *>(desc_ptr), t, pos_ids, sin_table,
                                           cos_table);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetRoPEWorkspaceSize(infiniopRoPEDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetRoPEWorkspaceSize(reinterpret_cast<RoPEAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopRoPE(infiniopRoPEDescriptor_t desc, void *workspace, uint64_t workspace_size, void *t,
                                         void const *pos_ids, void const *sin_table, void const *cos_table, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdRoPE(reinterpret_cast<RoPEAmdDescriptor_t>(desc), workspace, workspace_size, t, pos_ids,
                           sin_table, cos_table, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyRoPEDescriptor(infiniopRoPEDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyRoPEDescriptor(reinterpret_cast<RoPEAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
