// gfx950 kernels for RMSNorm and their launch.
//
// The kernels live in rms_norm_kernels.h, which the fused Add + RMSNorm
// operator shares.
#include "rms_norm_amd.h"
#include "rms_norm_kernels.h"

using namespace rms_norm_kernels;

// The fp16 kernels are compiled in rms_norm_f16.hip: a code object is loaded
// whole at the first launch of any kernel in it, and two halves make that
// first call faster for a caller that uses one element type.
void rms_norm_launch_f16(const RowsShape &shape, void *y, const void *x, const void *w, int w_kind, hipStream_t stream);

// Stage 4 of RMSNorm.  The workspace is unused (its size is 0).
infiniopStatus_t amdRMSNorm(RMSNormAmdDescriptor_t desc, void *, uint64_t, void *y, void const *x, void const *w, void *stream) {
    if (desc->elem != amd::Elem::F16 && desc->elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (desc->n == 0 || desc->d == 0) {
        return STATUS_SUCCESS;
    }
    if (y == nullptr || x == nullptr || w == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsShape shape{desc->cu_count, desc->lds_per_block, desc->n, desc->d, desc->stride_y, desc->stride_x, desc->epsilon};
    const Residual<false> none{};
    const int w_kind = weight_kind(desc->w_elem);
    if (w_kind < 0) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (desc->elem == amd::Elem::F16) {
        rms_norm_launch_f16(shape, y, x, w, w_kind, s);// its kernels are a translation unit of their own
    } else {
        launch_rms_norm<amd::BF16Rne, false>(shape, y, x, w, w_kind, none, s);
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
