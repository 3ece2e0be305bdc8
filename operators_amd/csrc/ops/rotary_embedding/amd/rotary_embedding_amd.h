// amd-gpu back end of RoPE.  Interface shape follows the per-device functions
// the reference's dispatcher calls (src/ops/rotary_embedding/operator.cc:24-151).
#ifndef INFINIOP_AMD_ROTARY_EMBEDDING_H
#define INFINIOP_AMD_ROTARY_EMBEDDING_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct RoPEAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    amd::Elem elem;
    uint64_t tokens;    // t.shape[0]
    uint64_t heads;     // t.shape[1]
    uint64_t head_dim;  // t.shape[2], even
    uint64_t table_rows;// rows of the sin/cos tables
    int64_t stride_token, stride_head;// elements
};
typedef RoPEAmdDescriptor *RoPEAmdDescriptor_t;

infiniopStatus_t amdCreateRoPEDescriptor(AmdHandle_t handle, RoPEAmdDescriptor_t *desc_ptr,
                                         infiniopTensorDescriptor_t t, infiniopTensorDescriptor_t pos_ids,
                                         infiniopTensorDescriptor_t sin_table, infiniopTensorDescriptor_t cos_table);
infiniopStatus_t amdGetRoPEWorkspaceSize(RoPEAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdRoPE(RoPEAmdDescriptor_t desc, void *workspace, uint64_t workspace_size, void *t,
                         void const *pos_ids, void const *sin_table, void const *cos_table, void *stream);
infiniopStatus_t amdDestroyRoPEDescriptor(RoPEAmdDescriptor_t desc);

#endif
