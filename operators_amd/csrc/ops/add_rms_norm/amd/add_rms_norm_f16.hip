// The fp16 instantiations of the fused Add + RMSNorm kernels, in a translation
// unit (and so a code object) of their own; see add_rms_norm_amd.hip.
#include "add_rms_norm_amd.h"
#include "../../rms_norm/amd/rms_norm_kernels.h"

using namespace rms_norm_kernels;

void add_rms_norm_launch_f16(const RowsShape &shape, void *y, const void *a, const void *w, int w_kind,
                             const Residual<true> &res, hipStream_t stream) {
    launch_rms_norm<amd::F16Ref, true>(shape, y, a, w, w_kind, res, stream);
}
