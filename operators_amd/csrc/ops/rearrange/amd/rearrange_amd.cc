// Create-time validation and layout analysis for Rearrange on the amd-gpu
// device.  Checks, order and status codes are those of the reference's CPU
// back end (src/ops/rearrange/cpu/rearrange_cpu.cc:7-54) - which, unlike its
// NVIDIA back end (cuda/rearrange.cc:29-58), takes ranks above 3.
#include "rearrange_amd.h"
#include <new>

infiniopStatus_t amdCreateRearrangeDescriptor(AmdHandle_t handle, RearrangeAmdDescriptor_t *desc_ptr,
                                              infiniopTensorDescriptor_t dst, infiniopTensorDescriptor_t src) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (!amd::same_dt(dst->dt, src->dt)) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    const uint64_t ndim = dst->ndim;
    if (src->ndim != ndim || ndim == 0) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    for (uint64_t i = 0; i < ndim; ++i) {
        if (dst->shape[i] != src->shape[i]) {
            return STATUS_BAD_TENSOR_SHAPE;
        }
    }
    if (dst->strides[ndim - 1] != 1 || src->strides[ndim - 1] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    if (ndim >= 4) {
        for (uint64_t i = ndim - 3; i >= 1; --i) {
            if (static_cast<int64_t>(dst->shape[i]) * dst->strides[i] != dst->strides[i - 1] ||
                static_cast<int64_t>(src->shape[i]) * src->strides[i] != src->strides[i - 1]) {
                return STATUS_BAD_TENSOR_STRIDES;
            }
        }
    }

    const int64_t elem = dst->dt.size;
    auto *desc = new (std::nothrow) RearrangeAmdDescriptor{};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    desc->device = DevAmdGpu;
    desc->device_id = handle->device_id;
    desc->cu_count = handle->cu_count;
    // An extent of zero anywhere: nothing to copy (the reference's loops run
    // zero times).  Decided here, before any extent is divided by.
    for (uint64_t i = 0; i < ndim; ++i) {
        if (dst->shape[i] == 0) {
            desc->rows = 0;
            desc->row_bytes = 0;
            desc->ndim = 0;
            *desc_ptr = desc;
            return STATUS_SUCCESS;
        }
    }
    desc->row_bytes = dst->shape[ndim - 1] * static_cast<uint64_t>(elem);
    desc->rows = 1;

    // Outer dimensions, outermost first; extent-1 dimensions are dropped and a
    // dimension that nests exactly inside its predecessor in both tensors is
    // merged with it.  A row that follows its predecessor without a gap in
    // both tensors lengthens the row instead.
    uint64_t shp[16];
    int64_t sd[16], ss[16];
    int n = 0;
    for (uint64_t i = 0; i + 1 < ndim; ++i) {
        const uint64_t ext = dst->shape[i];
        desc->rows *= ext;
        if (ext == 1) continue;
        const int64_t d = dst->strides[i] * elem, s = src->strides[i] * elem;
        if (n > 0 && sd[n - 1] == static_cast<int64_t>(ext) * d && ss[n - 1] == static_cast<int64_t>(ext) * s) {
            shp[n - 1] *= ext;
            sd[n - 1] = d;
            ss[n - 1] = s;
            continue;
        }
        if (n == 16) {
            delete desc;
            return STATUS_BAD_TENSOR_SHAPE;
        }
        shp[n] = ext, sd[n] = d, ss[n] = s;
        ++n;
    }
    while (n > 0 && sd[n - 1] == static_cast<int64_t>(desc->row_bytes) && ss[n - 1] == static_cast<int64_t>(desc->row_bytes)) {
        desc->row_bytes *= shp[n - 1];
        desc->rows /= shp[n - 1];
        --n;
    }
    if (n > kRearrangeMaxDims) {
        delete desc;
        return STATUS_BAD_TENSOR_SHAPE;
    }
    desc->ndim = n;
    // The kernels number the rows with dimension 0 varying fastest; any
    // numbering copies the same bytes.  They are numbered in the tensors' own
    // dimension order.  Sorting the dimensions by destination stride (writes
    // in address order, the source gathered) or by source stride (the
    // reverse) was measured on MI355X with the head transpose of attention,
    // bf16 [8192, 64, 128] inside [8192, 80, 128] <-> dense [64, 8192, 128]:
    // into the dense tensor 43.4 us as is and 49.6 us by destination order;
    // back out of it 42.3 us as is and 58.6 us by source order.  In both the
    // tensors' own order walks the 64 heads of a token first - 16 KiB in one
    // piece on the wide side, 2 MiB steps on the dense side - and the sorted
    // order walks tokens first, 20 KiB steps on the wide side, which is what
    // costs.  No rule based on one tensor's strides alone gets both right, so
    // the order is left as the caller wrote it.
    for (int k = 0; k < n; ++k) {// innermost outer dimension first
        desc->shape[k] = shp[n - 1 - k];
        desc->dst_stride[k] = sd[n - 1 - k];
        desc->src_stride[k] = ss[n - 1 - k];
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyRearrangeDescriptor(RearrangeAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
