// Public entry points of Add: route on the device recorded in the handle or
// descriptor, as src/ops/add/operator.cc:13-73 of the reference does.  This
// library carries one device; every other value answers STATUS_BAD_DEVICE.
#include "amd/add_amd.h"

INFINIOP_C infiniopStatus_t infiniopCreateAddDescriptor(infiniopHandle_t handle, infiniopAddDescriptor_t *desc_ptr,
                                                        infiniopTensorDescriptor_t c, infiniopTensorDescriptor_t a,
                                                        infiniopTensorDescriptor_t b) {
    if (handle == nullptr || c == nullptr || a == nullptr || b == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (handle->device) {
        case DevAmdGpu:
            return amdCreateAddDescriptor(reinterpret_cast<AmdHandle_t>(handle),
                                          reinterpret_cast<AddAmdDescriptor_t *>(desc_ptr), c, a, b);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopAdd(infiniopAddDescriptor_t desc, void *c, void const *a, void const *b, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdAdd(reinterpret_cast<AddAmdDescriptor_t>(desc), c, a, b, stream);
        default:
            return STATUS_BAD_DEVICE;
    }
}

INFINIOP_C infiniopStatus_t infiniopDestroyAddDescriptor(infiniopAddDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    switch (desc->device) {
        case DevAmdGpu:
            return amdDestroyAddDescriptor(reinterpret_cast<AddAmdDescriptor_t>(desc));
        default:
            return STATUS_BAD_DEVICE;
    }
}
