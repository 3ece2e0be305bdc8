// amd-gpu back end of Add.  Interface shape follows the per-device functions
// the reference's dispatcher calls (src/ops/add/operator.cc:20-73,
// src/ops/add/cuda/add.cuh:10-36).
#ifndef INFINIOP_AMD_ADD_H
#define INFINIOP_AMD_ADD_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

// Largest rank left after adjacent dimensions that step together have been
// merged.  The reference has no limit; shapes that alternate broadcast and
// non-broadcast dimensions more than this many times are refused at create.
constexpr int kAddMaxDims = 8;

// Everything the launch needs, captured at create time; never modified later.
struct AddAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    amd::Elem elem;
    uint64_t total;// elements of c
    bool flat;     // a and b are both read at c's flat index
    int ndim;      // merged rank, innermost dimension first in the arrays below
    uint64_t shape[kAddMaxDims];
    int64_t a_stride[kAddMaxDims];// elements; 0 where a is broadcast
    int64_t b_stride[kAddMaxDims];
};
typedef AddAmdDescriptor *AddAmdDescriptor_t;

infiniopStatus_t amdCreateAddDescriptor(AmdHandle_t handle, AddAmdDescriptor_t *desc_ptr,
                                        infiniopTensorDescriptor_t c, infiniopTensorDescriptor_t a,
                                        infiniopTensorDescriptor_t b);
infiniopStatus_t amdAdd(AddAmdDescriptor_t desc, void *c, void const *a, void const *b, void *stream);
infiniopStatus_t amdDestroyAddDescriptor(AddAmdDescriptor_t desc);

#endif
