// Public entry points of Matmul; same routing as src/ops/matmul/operator.cc of
// the reference, one device.
#include "amd/matmul_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateMatmulDescriptor(infiniopHandle_t handle, infiniopMatmulDescriptor_t *desc_ptr,
                                                           infiniopTensorDescriptor_t c_desc, float alpha,
                                                           infiniopTensorDescriptor_t a_desc,
                                                           infiniopTensorDescriptor_t b_desc, float beta) {
    if (handle == nullptr || c_desc == nullptr || a_desc == nullptr || b_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateMatmulDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                              reinterpret_cast<MatmulAmdDescriptor_t *>(desc_ptr), c_desc, alpha,
                                             a_desc, b_desc, beta);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopGetMatmulWorkspaceSize(infiniopMatmulDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdGetMatmulWorkspaceSize(reinterpret_cast<MatmulAmdDescriptor_t>(desc), size);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopMatmul(infiniopMatmulDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                           void *c, void const *a, void const *b, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdMatmul(reinterpret_cast<MatmulAmdDescriptor_t>(desc), workspace, workspace_size, c, a, b, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyMatmulDescriptor(infiniopMatmulDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyMatmulDescriptor(reinterpret_cast<MatmulAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
