// Create-time validation for RandomSample on the amd-gpu device.  Checks,
// their order and their status codes are the reference's
// (src/ops/random_sample/cpu/random_sample.cc:7-33): logits of rank 1, F16;
// result U64; a result that is neither of rank 1 nor has a first extent of 1
// is refused.  A result without dimensions (whose first extent the reference
// reads anyway) is taken as a scalar.  Additions: BF16 logits are accepted
// (probabilities then round to nearest even where fp16 ones are truncated as
// in the reference); a unit stride on the logits
// (the reference reads them as dense without looking), at least one logit,
// and fewer than 2^31 of them (the reference keeps the count in an int).
#include "random_sample_amd.h"
#include <new>

infiniopStatus_t amdCreateRandomSampleDescriptor(AmdHandle_t handle, RandomSampleAmdDescriptor_t *desc_ptr,
                                                 infiniopTensorDescriptor_t result, infiniopTensorDescriptor_t probs) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (probs->ndim != 1) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const amd::Elem elem = amd::elem_of(probs->dt);
    if (elem != amd::Elem::F16 && elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (!amd::same_dt(result->dt, U64)) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (result->ndim != 1 && result->ndim != 0 && result->shape[0] != 1) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (probs->shape[0] == 0 || probs->shape[0] >= (1ull << 31)) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (probs->shape[0] > 1 && probs->strides[0] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    const uint32_t voc = static_cast<uint32_t>(probs->shape[0]);
    uint32_t groups = 0, vecs = 0;
    if (voc >= kRandomSampleSplitVoc) {
        const uint64_t per_vec = kRandomSamplePartLanes * 8ull;
        vecs = static_cast<uint32_t>(amd::ceil_div(voc, per_vec * kRandomSampleMaxGroups));
        groups = static_cast<uint32_t>(amd::ceil_div(voc, per_vec * vecs));
    }
    void *scratch = nullptr;
    if (amdRandomSampleScratch(handle->device_id, &scratch) != STATUS_SUCCESS) {
        scratch = nullptr;// infiniopRandomSampleNoAlloc will say so; every other entry point works without it
    }
    auto *desc = new (std::nothrow) RandomSampleAmdDescriptor{DevAmdGpu, handle->device_id, elem, voc, groups, vecs, scratch};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

// The reference's back ends sort in a workspace of voc * 12 (CPU) or voc * 20
// bytes plus what their sorting library allocates per call (CUDA).  Here the
// workspace carries what a first launch spread over the chip leaves for the
// workgroup that draws: for up to 256 candidates one header and 512 candidates
// of 8 bytes per workgroup (under 200 KiB whatever the vocabulary); for more,
// the headers and a count for every 16-bit key (257 KiB).  Small vocabularies
// need none.  A call that comes without it is served by one workgroup.
uint64_t amdRandomSampleListBytes(const RandomSampleAmdDescriptor &d) {
    if (d.groups == 0) {
        return 0;
    }
    return kRandomSampleMaxGroups * sizeof(RandomSamplePart) + static_cast<uint64_t>(d.groups) * kRandomSamplePartCap * sizeof(uint64_t);
}

uint64_t amdRandomSampleHistogramBytes(const RandomSampleAmdDescriptor &d) {
    if (d.groups == 0) {
        return 0;
    }
    return kRandomSampleMaxGroups * sizeof(RandomSamplePart) + static_cast<uint64_t>(kRandomSampleKeys) * sizeof(uint32_t);
}

uint64_t amdRandomSampleWorkspaceBytes(const RandomSampleAmdDescriptor &d) {
    const uint64_t lists = amdRandomSampleListBytes(d), histogram = amdRandomSampleHistogramBytes(d);
    return lists > histogram ? lists : histogram;
}

infiniopStatus_t amdGetRandomSampleWorkspaceSize(RandomSampleAmdDescriptor_t desc, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    *size = amdRandomSampleWorkspaceBytes(*desc);
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyRandomSampleDescriptor(RandomSampleAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
