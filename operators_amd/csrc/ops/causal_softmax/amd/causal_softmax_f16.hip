// The fp16 instantiations of the CausalSoftmax kernels, in a translation unit
// (and so a code object) of their own; see causal_softmax_amd.hip.
#include "causal_softmax_amd.h"
#include "causal_softmax_kernels.h"

using namespace causal_softmax_kernels;

void causal_softmax_launch_f16(const CausalSoftmaxAmdDescriptor &desc, void *data, CausalSoftmaxPart *parts, hipStream_t stream) {
    launch_causal_softmax<amd::F16Ref>(desc, data, parts, stream);
}
