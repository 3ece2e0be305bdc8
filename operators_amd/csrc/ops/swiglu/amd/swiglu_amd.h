// amd-gpu back end of SwiGLU.  Interface shape follows the per-device
// functions the reference's dispatcher calls (src/ops/swiglu/operator.cc:18-101).
#ifndef INFINIOP_AMD_SWIGLU_H
#define INFINIOP_AMD_SWIGLU_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct SwiGLUAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    amd::Elem elem;
    uint64_t rows;// tokens
    uint64_t di;  // intermediate width
    int64_t stride_a, stride_b, stride_c;// row strides, elements
};
typedef SwiGLUAmdDescriptor *SwiGLUAmdDescriptor_t;

infiniopStatus_t amdCreateSwiGLUDescriptor(AmdHandle_t handle, SwiGLUAmdDescriptor_t *desc_ptr,
                                           infiniopTensorDescriptor_t c_desc, infiniopTensorDescriptor_t a_desc,
                                           infiniopTensorDescriptor_t b_desc);
infiniopStatus_t amdSwiGLU(SwiGLUAmdDescriptor_t desc, void *c, void const *a, void const *b, void *stream);
infiniopStatus_t amdDestroySwiGLUDescriptor(SwiGLUAmdDescriptor_t desc);

#endif
