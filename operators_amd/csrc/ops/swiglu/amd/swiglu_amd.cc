// Create-time validation for SwiGLU on the amd-gpu device: the checks, their
// order and their status codes are those of the reference's CPU back end
// (src/ops/swiglu/cpu/swiglu_cpu.cc:7-47), with BF16 admitted as an extension.
#include "swiglu_amd.h"
#include <new>

infiniopStatus_t amdCreateSwiGLUDescriptor(AmdHandle_t handle, SwiGLUAmdDescriptor_t *desc_ptr,
                                           infiniopTensorDescriptor_t c_desc, infiniopTensorDescriptor_t a_desc,
                                           infiniopTensorDescriptor_t b_desc) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (c_desc->ndim != 2 || a_desc->ndim != 2 || b_desc->ndim != 2) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const amd::Elem elem = amd::elem_of(c_desc->dt);
    if (elem != amd::Elem::F16 && elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (a_desc->strides[1] != 1 || b_desc->strides[1] != 1 || c_desc->strides[1] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    const uint64_t rows = c_desc->shape[0], di = c_desc->shape[1];
    // A mismatch between the operands and the result is a bad parameter in the
    // reference, not a bad shape or dtype.
    if (a_desc->shape[0] != rows || a_desc->shape[1] != di || !amd::same_dt(a_desc->dt, c_desc->dt) ||
        b_desc->shape[0] != rows || b_desc->shape[1] != di || !amd::same_dt(b_desc->dt, c_desc->dt)) {
        return STATUS_BAD_PARAM;
    }
    auto *desc = new (std::nothrow) SwiGLUAmdDescriptor{
        DevAmdGpu, handle->device_id, handle->cu_count, elem, rows, di,
        a_desc->strides[0], b_desc->strides[0], c_desc->strides[0]};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroySwiGLUDescriptor(SwiGLUAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
