// Create-time validation for the fused Add + RMSNorm on the amd-gpu device.
//
// The operator stands for Add followed by RMSNorm, so it applies RMSNorm's
// checks (reference src/ops/rms_norm/cpu/rms_norm_cpu.cc:6-17) to y, c and w
// and asks of a and b what Add asks of operands that are not broadcast
// (src/ops/add/cpu/add_cpu.cc:18-45): the shape of c and one element type for
// all of them.  Rows may be strided; elements within a row may not.  The type
// verdict is left to the compute call, as in RMSNorm.
#include "add_rms_norm_amd.h"
#include <new>

infiniopStatus_t amdCreateAddRMSNormDescriptor(AmdHandle_t handle, AddRMSNormAmdDescriptor_t *desc_ptr,
                                               infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t c_desc,
                                               infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc,
                                               infiniopTensorDescriptor_t w_desc, float epsilon) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (y_desc->ndim != 2 || c_desc->ndim != 2 || a_desc->ndim != 2 || b_desc->ndim != 2 || w_desc->ndim != 1) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const uint64_t n = y_desc->shape[0], d = y_desc->shape[1];
    for (infiniopTensorDescriptor_t t : {c_desc, a_desc, b_desc}) {
        if (t->shape[0] != n || t->shape[1] != d) {
            return STATUS_BAD_TENSOR_SHAPE;
        }
    }
    if (w_desc->shape[0] != d) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    for (infiniopTensorDescriptor_t t : {y_desc, c_desc, a_desc, b_desc}) {
        if (t->strides[1] != 1) {
            return STATUS_BAD_TENSOR_STRIDES;
        }
    }
    if (w_desc->strides[0] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    const bool one_type = amd::same_dt(y_desc->dt, c_desc->dt) && amd::same_dt(y_desc->dt, a_desc->dt) &&
                          amd::same_dt(y_desc->dt, b_desc->dt);
    const amd::Elem elem = one_type ? amd::elem_of(y_desc->dt) : amd::Elem::Other;
    auto *desc = new (std::nothrow) AddRMSNormAmdDescriptor{
        DevAmdGpu, handle->device_id, handle->cu_count, handle->lds_per_block,
        elem, amd::elem_of(w_desc->dt), n, d,
        y_desc->strides[0], c_desc->strides[0], a_desc->strides[0], b_desc->strides[0], epsilon};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdGetAddRMSNormWorkspaceSize(AddRMSNormAmdDescriptor_t, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    *size = 0;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyAddRMSNormDescriptor(AddRMSNormAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
