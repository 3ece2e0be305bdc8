// amd-gpu back end of RandomSample.  Interface shape follows the per-device
// functions the reference's dispatcher calls (src/ops/random_sample/operator.cc).
#ifndef INFINIOP_AMD_RANDOM_SAMPLE_H
#define INFINIOP_AMD_RANDOM_SAMPLE_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

// Largest number of candidates (topk after clamping to the vocabulary size)
// the sampling form keeps; they live in the workgroup's LDS.
constexpr int kRandomSampleMaxTopk = 1024;

struct RandomSampleAmdDescriptor {
    Device device;
    int device_id;
    uint32_t voc;// number of logits
};
typedef RandomSampleAmdDescriptor *RandomSampleAmdDescriptor_t;

infiniopStatus_t amdCreateRandomSampleDescriptor(AmdHandle_t handle, RandomSampleAmdDescriptor_t *desc_ptr,
                                                 infiniopTensorDescriptor_t result, infiniopTensorDescriptor_t probs);
infiniopStatus_t amdGetRandomSampleWorkspaceSize(RandomSampleAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdRandomSample(RandomSampleAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                 void *result, void const *probs, float random_val, float topp, int topk,
                                 float temperature, void *stream);
infiniopStatus_t amdDestroyRandomSampleDescriptor(RandomSampleAmdDescriptor_t desc);

#endif
