// The fp16 instantiations of the RMSNorm kernels, in a translation unit (and
// so a code object) of their own; see rms_norm_amd.hip.
#include "rms_norm_amd.h"
#include "rms_norm_kernels.h"

using namespace rms_norm_kernels;

void rms_norm_launch_f16(const RowsShape &shape, void *y, const void *x, const void *w, int w_kind, hipStream_t stream) {
    launch_rms_norm<amd::F16Ref, false>(shape, y, x, w, w_kind, Residual<false>{}, stream);
}
