// Tensor descriptors: a deep copy of rank, extents, strides (in elements) and
// element type.  Same contract as src/tensor/tensor_descriptor.cc:4-26 of the
// reference: NULL strides mean contiguous row-major; rank 0 is allowed.
#include "infiniop.h"
#include <algorithm>
#include <new>

INFINIOP_C infiniopStatus_t infiniopCreateTensorDescriptor(infiniopTensorDescriptor_t *desc_ptr, uint64_t ndim,
                                                           uint64_t const *shape, int64_t const *strides,
                                                           DataLayout datatype) {
    if (desc_ptr == nullptr || (ndim != 0 && shape == nullptr)) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    auto *desc = new (std::nothrow) TensorDescriptor{datatype, ndim, nullptr, nullptr};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    desc->shape = new (std::nothrow) uint64_t[ndim ? ndim : 1];
    desc->strides = new (std::nothrow) int64_t[ndim ? ndim : 1];
    if (desc->shape == nullptr || desc->strides == nullptr) {
        delete[] desc->shape;
        delete[] desc->strides;
        delete desc;
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    std::copy(shape, shape + ndim, desc->shape);
    if (strides != nullptr) {
        std::copy(strides, strides + ndim, desc->strides);
    } else {
        int64_t run = 1;
        for (uint64_t i = ndim; i-- > 0;) {
            desc->strides[i] = run;
            run *= static_cast<int64_t>(shape[i]);
        }
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

INFINIOP_C infiniopStatus_t infiniopDestroyTensorDescriptor(infiniopTensorDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    delete[] desc->shape;
    delete[] desc->strides;
    delete desc;
    return STATUS_SUCCESS;
}
