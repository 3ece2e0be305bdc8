// Create-time validation for RoPE on the amd-gpu device: the checks, their
// order and their status codes are those of the reference's CPU back end
// (src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc:47-102), with BF16 t
// admitted as an extension.  Unlike the NVIDIA back end
// (cuda/rotary_embedding.cc:35-37) there is no upper bound on head_dim.
#include "rotary_embedding_amd.h"
#include <new>

infiniopStatus_t amdCreateRoPEDescriptor(AmdHandle_t handle, RoPEAmdDescriptor_t *desc_ptr,
                                         infiniopTensorDescriptor_t t, infiniopTensorDescriptor_t pos_ids,
                                         infiniopTensorDescriptor_t sin_table, infiniopTensorDescriptor_t cos_table) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (t->ndim != 3 || pos_ids->ndim != 1 || sin_table->ndim != 2 || cos_table->ndim != 2) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const uint64_t tokens = t->shape[0], heads = t->shape[1], head_dim = t->shape[2];
    if (head_dim % 2 != 0) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (pos_ids->shape[0] != tokens || sin_table->shape[1] != head_dim || cos_table->shape[1] != head_dim ||
        sin_table->shape[0] != cos_table->shape[0]) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (t->strides[2] != 1 || pos_ids->strides[0] != 1 || sin_table->strides[1] != 1 || cos_table->strides[1] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    const amd::Elem elem = amd::elem_of(t->dt);
    if (elem != amd::Elem::F16 && elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (!amd::same_dt(sin_table->dt, F32) || !amd::same_dt(cos_table->dt, F32)) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (!amd::same_dt(pos_ids->dt, U64)) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    auto *desc = new (std::nothrow) RoPEAmdDescriptor{
        DevAmdGpu, handle->device_id, handle->cu_count, elem, tokens, heads, head_dim,
        sin_table->shape[0], t->strides[0], t->strides[1]};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdGetRoPEWorkspaceSize(RoPEAmdDescriptor_t, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    *size = 0;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyRoPEDescriptor(RoPEAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
