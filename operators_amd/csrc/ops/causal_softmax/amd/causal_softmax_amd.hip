// gfx950 CausalSoftmax: stage 4 and the bf16 kernels.
//
// The kernels live in causal_softmax_kernels.h.  The fp16 instantiations are
// compiled in causal_softmax_f16.hip: a code object is loaded whole at the
// first launch of any kernel in it, and two halves make that first call
// faster for a caller that uses one element type (15 ms in one piece).
#include "causal_softmax_amd.h"
#include "causal_softmax_kernels.h"

using namespace causal_softmax_kernels;

void causal_softmax_launch_f16(const CausalSoftmaxAmdDescriptor &desc, void *data, hipStream_t stream);

// Stage 4 of CausalSoftmax.  The workspace is unused (its size is 0).
infiniopStatus_t amdCausalSoftmax(CausalSoftmaxAmdDescriptor_t desc, void *, uint64_t, void *data, void *stream) {
    if (desc->batch == 0 || desc->seq == 0 || desc->total == 0) {
        return STATUS_SUCCESS;
    }
    if (data == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    switch (desc->elem) {
        case amd::Elem::F16:
            causal_softmax_launch_f16(*desc, data, s);// its kernels are a translation unit of their own
            break;
        case amd::Elem::BF16:
            launch_causal_softmax<amd::BF16Rne>(*desc, data, s);
            break;
        default:
            return STATUS_BAD_TENSOR_DTYPE;
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
