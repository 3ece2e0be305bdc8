// Create-time validation for RMSNorm on the amd-gpu device.
//
// Shape checks and codes are the reference's
// (src/ops/rms_norm/cpu/rms_norm_cpu.cc:6-17).  The reference then records the
// layouts without looking at them and fails at compute time for anything but
// F16 data (rms_norm_cpu.cc:88-98); this back end keeps that split - a
// descriptor with an unsupported element type is created and every call on it
// answers STATUS_BAD_TENSOR_DTYPE - so callers see the same statuses at the
// same stage.  Two deliberate differences: x's row stride is taken from x's
// own descriptor (the CPU back end reads y's, rms_norm_cpu.cc:20; the NVIDIA
// one reads x's, cuda/rms_norm.cc:21-22), and BF16 data is accepted.
#include "rms_norm_amd.h"
#include <new>

infiniopStatus_t amdCreateRMSNormDescriptor(AmdHandle_t handle, RMSNormAmdDescriptor_t *desc_ptr,
                                            infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t x_desc,
                                            infiniopTensorDescriptor_t w_desc, float epsilon) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (y_desc->ndim != 2 || x_desc->ndim != 2 || w_desc->ndim != 1) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const uint64_t n = y_desc->shape[0], d = y_desc->shape[1];
    if (x_desc->shape[0] != n || x_desc->shape[1] != d || w_desc->shape[0] != d) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    // The kernels walk rows with unit element stride; the reference assumes
    // the same without checking.  Refuse what it would silently misread.
    if (y_desc->strides[1] != 1 || x_desc->strides[1] != 1 || w_desc->strides[0] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    // x must have y's element type; if not, the descriptor is created and
    // every call on it reports the bad type, like any other unsupported type.
    const amd::Elem elem = amd::same_dt(y_desc->dt, x_desc->dt) ? amd::elem_of(y_desc->dt) : amd::Elem::Other;
    auto *desc = new (std::nothrow) RMSNormAmdDescriptor{
        DevAmdGpu, handle->device_id, handle->cu_count, handle->lds_per_block,
        elem, amd::elem_of(w_desc->dt), n, d,
        y_desc->strides[0], x_desc->strides[0], epsilon};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdGetRMSNormWorkspaceSize(RMSNormAmdDescriptor_t, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    *size = 0;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyRMSNormDescriptor(RMSNormAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
