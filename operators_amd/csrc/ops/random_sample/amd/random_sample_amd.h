// amd-gpu back end of RandomSample.  Interface shape follows the per-device
// functions the reference's dispatcher calls (src/ops/random_sample/operator.cc).
#ifndef INFINIOP_AMD_RANDOM_SAMPLE_H
#define INFINIOP_AMD_RANDOM_SAMPLE_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

// Largest number of candidates (topk after clamping to the vocabulary size)
// the sampling form keeps; they live in the workgroup's LDS.
constexpr int kRandomSampleMaxTopk = 1024;

// Geometry of the two-launch form: workgroups of 256 lanes, each over
// 2048 * vecs consecutive logits, each with room for 512 surviving candidates
// in the workspace; at most 48 of them.
constexpr int kRandomSamplePartLanes = 256;
constexpr int kRandomSamplePartCap = 512;
constexpr int kRandomSampleMaxGroups = 48;
// topk up to which the two-launch form is used (one candidate bound per lane)
constexpr int kRandomSamplePartTopk = 256;
// vocabularies below this are sampled by one workgroup in one launch
constexpr uint32_t kRandomSampleSplitVoc = 4096;
// keys of the histogram form: every 16-bit code has one
constexpr uint32_t kRandomSampleKeys = 1u << 16;
// largest vocabulary the entry point without workspace and allocation serves
constexpr uint32_t kRandomSampleNoAllocMaxVoc = 1u << 20;

// What one workgroup of the first launch leaves for the second.
struct RandomSamplePart {
    uint32_t count;  // candidates it found (more than the cap: the list is incomplete)
    uint32_t key_max;// key of its largest logit
    float sum;       // sum of expf((x - its largest) / temperature) over its logits
    uint32_t unused;
};

struct RandomSampleAmdDescriptor {
    Device device;
    int device_id;
    amd::Elem elem; // F16 or BF16
    uint32_t voc;   // number of logits
    uint32_t groups;// workgroups of the first launch of the two-launch form; 0: never used
    uint32_t vecs;  // 8-element vectors per lane in them
    void *scratch;  // this GPU's copy of the library's own lists (see amdRandomSampleScratch); null if it could not be found
};
typedef RandomSampleAmdDescriptor *RandomSampleAmdDescriptor_t;

infiniopStatus_t amdCreateRandomSampleDescriptor(AmdHandle_t handle, RandomSampleAmdDescriptor_t *desc_ptr,
                                                 infiniopTensorDescriptor_t result, infiniopTensorDescriptor_t probs);
// bytes of workspace the two forms that use one need: candidate lists (topk <= 256), a histogram of all 16-bit
// keys (more candidates); the descriptor asks for the larger
uint64_t amdRandomSampleListBytes(const RandomSampleAmdDescriptor &desc);
uint64_t amdRandomSampleHistogramBytes(const RandomSampleAmdDescriptor &desc);
uint64_t amdRandomSampleWorkspaceBytes(const RandomSampleAmdDescriptor &desc);
infiniopStatus_t amdGetRandomSampleWorkspaceSize(RandomSampleAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdRandomSample(RandomSampleAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                 void *result, void const *probs, float random_val, float topp, int topk,
                                 float temperature, void *stream);
// The address, on GPU `device_id`, of the array the library keeps for calls that bring no workspace.  Asked of the
// runtime once per GPU (with that GPU made current) and kept; descriptors take it at creation, so that the call
// itself neither queries nor locks anything.
infiniopStatus_t amdRandomSampleScratch(int device_id, void **address);
infiniopStatus_t amdRandomSampleNoAlloc(RandomSampleAmdDescriptor_t desc, void *result, void const *probs, float random_val,
                                        float topp, int topk, float temperature, void *stream);
infiniopStatus_t amdDestroyRandomSampleDescriptor(RandomSampleAmdDescriptor_t desc);

#endif
