// amd-gpu back end of CausalSoftmax.  Interface shape follows the per-device
// functions the reference's dispatcher calls
// (src/ops/causal_softmax/operator.cc:21-130).
#ifndef INFINIOP_AMD_CAUSAL_SOFTMAX_H
#define INFINIOP_AMD_CAUSAL_SOFTMAX_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct CausalSoftmaxAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    amd::Elem elem;
    uint64_t batch;// product of the leading dimensions
    uint64_t seq;  // rows per matrix
    uint64_t total;// columns
    int64_t stride_b, stride_i;// elements; the innermost stride is 1
};
typedef CausalSoftmaxAmdDescriptor *CausalSoftmaxAmdDescriptor_t;

infiniopStatus_t amdCreateCausalSoftmaxDescriptor(AmdHandle_t handle, CausalSoftmaxAmdDescriptor_t *desc_ptr,
                                                  infiniopTensorDescriptor_t y_desc);
infiniopStatus_t amdGetCausalSoftmaxWorkspaceSize(CausalSoftmaxAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdCausalSoftmax(CausalSoftmaxAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                  void *data, void *stream);
infiniopStatus_t amdDestroyCausalSoftmaxDescriptor(CausalSoftmaxAmdDescriptor_t desc);

#endif
