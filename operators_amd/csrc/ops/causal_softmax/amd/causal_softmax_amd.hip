// gfx950 CausalSoftmax: stage 4 and the bf16 kernels.
//
// The kernels live in causal_softmax_kernels.h.  The fp16 instantiations are
// compiled in causal_softmax_f16.hip: a code object is loaded whole at the
// first launch of any kernel in it, and two halves make that first call
// faster for a caller that uses one element type (15 ms in one piece).
#include "causal_softmax_amd.h"
#include "causal_softmax_kernels.h"

using namespace causal_softmax_kernels;

void causal_softmax_launch_f16(const CausalSoftmaxAmdDescriptor &desc, void *data, CausalSoftmaxPart *parts, hipStream_t stream);

// Stage 4 of CausalSoftmax.  The workspace serves the split form of few long rows only; a call that comes
// without it (or with less than amdGetCausalSoftmaxWorkspaceSize asks for) is served a workgroup per row.
infiniopStatus_t amdCausalSoftmax(CausalSoftmaxAmdDescriptor_t desc, void *workspace, uint64_t workspace_size, void *data, void *stream) {
    if (desc->batch == 0 || desc->seq == 0 || desc->total == 0) {
        return STATUS_SUCCESS;
    }
    if (data == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    CausalSoftmaxPart *parts = nullptr;
    const uint64_t parts_bytes = desc->batch * desc->seq * causal_softmax_parts(*desc) * sizeof(CausalSoftmaxPart);
    if (parts_bytes != 0 && workspace != nullptr && workspace_size >= parts_bytes && amd::aligned16(workspace) && amd::aligned16(data)) {
        parts = static_cast<CausalSoftmaxPart *>(workspace);
    }
    switch (desc->elem) {
        case amd::Elem::F16:
            causal_softmax_launch_f16(*desc, data, parts, s);// its kernels are a translation unit of their own
            break;
        case amd::Elem::BF16:
            launch_causal_softmax<amd::BF16Rne>(*desc, data, parts, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
