// Create-time validation for CausalSoftmax on the amd-gpu device.  Rank and
// element-type checks and their order are the reference's
// (src/ops/causal_softmax/cpu/causal_softmax_cpu.cc:6-15); the unit innermost
// stride is what its GPU back end demands (cuda/causal_softmax.cc:22-24).  Two
// additions: BF16 is accepted, and a matrix with fewer columns than rows is
// refused - the reference's column bound total - seq + i wraps around for it
// and its CPU loops then run past the row.
#include "causal_softmax_amd.h"
#include <new>

infiniopStatus_t amdCreateCausalSoftmaxDescriptor(AmdHandle_t handle, CausalSoftmaxAmdDescriptor_t *desc_ptr,
                                                  infiniopTensorDescriptor_t y) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    const uint64_t ndim = y->ndim;
    if (ndim != 2 && ndim != 3) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const amd::Elem elem = amd::elem_of(y->dt);
    if (elem != amd::Elem::F16 && elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    const uint64_t total = y->shape[ndim - 1], seq = y->shape[ndim - 2];
    if (y->strides[ndim - 1] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    if (total < seq) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    auto *desc = new (std::nothrow) CausalSoftmaxAmdDescriptor{
        DevAmdGpu, handle->device_id, handle->cu_count, elem,
        ndim == 3 ? y->shape[0] : 1, seq, total,
        ndim == 3 ? y->strides[0] : 0, y->strides[ndim - 2]};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

// 0 for every shape but few long rows, whose parts exchange a maximum and a sum each (see causal_softmax_parts).
infiniopStatus_t amdGetCausalSoftmaxWorkspaceSize(CausalSoftmaxAmdDescriptor_t desc, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    *size = desc->batch * desc->seq * causal_softmax_parts(*desc) * sizeof(CausalSoftmaxPart);
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyCausalSoftmaxDescriptor(CausalSoftmaxAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
