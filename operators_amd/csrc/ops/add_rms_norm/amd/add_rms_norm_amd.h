// amd-gpu back end of the fused residual form  c = a + b;  y = RMSNorm(c) * w.
// The reference has no such operator: its callers issue Add
// (src/ops/add/operator.cc:13-73) and then RMSNorm
// (src/ops/rms_norm/operator.cc:21-142) on the sum.  This one produces the
// results of that pair in a single pass over memory.
#ifndef INFINIOP_AMD_ADD_RMS_NORM_H
#define INFINIOP_AMD_ADD_RMS_NORM_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct AddRMSNormAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    int lds_per_block;
    amd::Elem elem;  // type of y, c, a and b
    amd::Elem w_elem;// type of w
    uint64_t n;      // rows
    uint64_t d;      // row length
    int64_t stride_y, stride_c, stride_a, stride_b;// row strides, elements
    float epsilon;
};
typedef AddRMSNormAmdDescriptor *AddRMSNormAmdDescriptor_t;

infiniopStatus_t amdCreateAddRMSNormDescriptor(AmdHandle_t handle, AddRMSNormAmdDescriptor_t *desc_ptr,
                                               infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t c_desc,
                                               infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc,
                                               infiniopTensorDescriptor_t w_desc, float epsilon);
infiniopStatus_t amdGetAddRMSNormWorkspaceSize(AddRMSNormAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdAddRMSNorm(AddRMSNormAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                               void *y, void *c, void const *a, void const *b, void const *w, void *stream);
infiniopStatus_t amdDestroyAddRMSNormDescriptor(AddRMSNormAmdDescriptor_t desc);

#endif
