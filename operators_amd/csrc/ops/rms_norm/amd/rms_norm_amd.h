// amd-gpu back end of RMSNorm.  Interface shape follows the per-device
// functions the reference's dispatcher calls
// (src/ops/rms_norm/operator.cc:21-142, src/ops/rms_norm/cuda/rms_norm.cuh:21-36).
#ifndef INFINIOP_AMD_RMS_NORM_H
#define INFINIOP_AMD_RMS_NORM_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct RMSNormAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    int lds_per_block;
    amd::Elem elem;  // type of x and y
    amd::Elem w_elem;// type of w
    uint64_t n;      // rows
    uint64_t d;      // row length
    int64_t stride_y, stride_x;// row strides, elements
    float epsilon;
};
typedef RMSNormAmdDescriptor *RMSNormAmdDescriptor_t;

infiniopStatus_t amdCreateRMSNormDescriptor(AmdHandle_t handle, RMSNormAmdDescriptor_t *desc_ptr,
                                            infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t x_desc,
                                            infiniopTensorDescriptor_t w_desc, float epsilon);
infiniopStatus_t amdGetRMSNormWorkspaceSize(RMSNormAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdRMSNorm(RMSNormAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                            void *y, void const *x, void const *w, void *stream);
infiniopStatus_t amdDestroyRMSNormDescriptor(RMSNormAmdDescriptor_t desc);

#endif
