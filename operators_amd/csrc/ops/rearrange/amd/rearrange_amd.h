// amd-gpu back end of Rearrange.  Interface shape follows the per-device
// functions the reference's dispatcher calls (src/ops/rearrange/operator.cc).
#ifndef INFINIOP_AMD_REARRANGE_H
#define INFINIOP_AMD_REARRANGE_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

// Largest number of outer dimensions left after merging those that step together.
constexpr int kRearrangeMaxDims = 6;

struct RearrangeAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    uint64_t row_bytes;// bytes of one innermost row
    uint64_t rows;     // product of the outer extents
    int ndim;          // merged outer dimensions, innermost of them first
    uint64_t shape[kRearrangeMaxDims];
    int64_t dst_stride[kRearrangeMaxDims];// bytes
    int64_t src_stride[kRearrangeMaxDims];// bytes
};
typedef RearrangeAmdDescriptor *RearrangeAmdDescriptor_t;

infiniopStatus_t amdCreateRearrangeDescriptor(AmdHandle_t handle, RearrangeAmdDescriptor_t *desc_ptr,
                                              infiniopTensorDescriptor_t dst, infiniopTensorDescriptor_t src);
infiniopStatus_t amdRearrange(RearrangeAmdDescriptor_t desc, void *dst, void const *src, void *stream);
infiniopStatus_t amdDestroyRearrangeDescriptor(RearrangeAmdDescriptor_t desc);

#endif
