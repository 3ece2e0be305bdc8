// Create-time validation and layout analysis for Add on the amd-gpu device.
// Accepts and rejects exactly what the reference's CPU back end does
// (src/ops/add/cpu/add_cpu.cc:18-45, src/ops/utils.h:85-143,174-188), in the
// same order - shape, strides, dtype - plus BF16 as an extension.
#include "add_amd.h"
#include <new>

namespace {

// numpy-style broadcast of a and b, right aligned, must give exactly c.
bool broadcast_matches(infiniopTensorDescriptor_t a, infiniopTensorDescriptor_t b, infiniopTensorDescriptor_t c) {
    const uint64_t rank = a->ndim > b->ndim ? a->ndim : b->ndim;
    if (rank != c->ndim) return false;
    for (uint64_t i = 0; i < rank; ++i) {
        const uint64_t da = i < rank - a->ndim ? 1 : a->shape[i - (rank - a->ndim)];
        const uint64_t db = i < rank - b->ndim ? 1 : b->shape[i - (rank - b->ndim)];
        if (!(da == db || da == 1 || db == 1)) return false;
        if ((da > db ? da : db) != c->shape[i]) return false;
    }
    return true;
}

}// namespace

infiniopStatus_t amdCreateAddDescriptor(AmdHandle_t handle, AddAmdDescriptor_t *desc_ptr,
                                        infiniopTensorDescriptor_t c, infiniopTensorDescriptor_t a,
                                        infiniopTensorDescriptor_t b) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (!broadcast_matches(a, b, c)) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (!amd::ref_contiguous(a) || !amd::ref_contiguous(b) || !amd::ref_contiguous(c)) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    const amd::Elem elem = amd::elem_of(c->dt);
    if (elem == amd::Elem::Other) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (!amd::same_dt(c->dt, a->dt) || !amd::same_dt(c->dt, b->dt)) {
        return STATUS_BAD_TENSOR_DTYPE;
    }

    // Per-dimension view of the operands over c's index space: an operand
    // steps with its own stride where it has c's extent and stands still where
    // it is absent or broadcast (reference add_cpu.cc:40-45).  Extent-1
    // dimensions are dropped and neighbours along which both operands advance
    // like one longer dimension are merged, outermost to innermost.
    const uint64_t rank = c->ndim;
    uint64_t total = 1;
    uint64_t shp[kAddMaxDims];
    int64_t sa[kAddMaxDims], sb[kAddMaxDims];
    int n = 0;// merged dims so far, outermost first
    for (uint64_t i = 0; i < rank; ++i) {
        const uint64_t ext = c->shape[i];
        total *= ext;
        if (ext == 1) continue;
        const uint64_t lack_a = rank - a->ndim, lack_b = rank - b->ndim;
        const int64_t step_a = (i < lack_a || a->shape[i - lack_a] != ext) ? 0 : a->strides[i - lack_a];
        const int64_t step_b = (i < lack_b || b->shape[i - lack_b] != ext) ? 0 : b->strides[i - lack_b];
        if (n > 0 && sa[n - 1] == static_cast<int64_t>(ext) * step_a && sb[n - 1] == static_cast<int64_t>(ext) * step_b) {
            shp[n - 1] *= ext;
            sa[n - 1] = step_a;
            sb[n - 1] = step_b;
            continue;
        }
        if (n == kAddMaxDims) {
            return STATUS_BAD_TENSOR_SHAPE;
        }
        shp[n] = ext;
        sa[n] = step_a;
        sb[n] = step_b;
        ++n;
    }
    if (n == 0) {// a single element (rank 0 or all extents 1), or an empty tensor
        shp[0] = total == 0 ? 0 : 1;
        sa[0] = sb[0] = 1;
        n = 1;
    }

    auto *desc = new (std::nothrow) AddAmdDescriptor{};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    desc->device = DevAmdGpu;
    desc->device_id = handle->device_id;
    desc->cu_count = handle->cu_count;
    desc->elem = elem;
    desc->total = total;
    desc->ndim = n;
    desc->flat = (n == 1 && sa[0] == 1 && sb[0] == 1) || total <= 1;
    for (int i = 0; i < n; ++i) {// store innermost first
        desc->shape[i] = shp[n - 1 - i];
        desc->a_stride[i] = sa[n - 1 - i];
        desc->b_stride[i] = sb[n - 1 - i];
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyAddDescriptor(AddAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
