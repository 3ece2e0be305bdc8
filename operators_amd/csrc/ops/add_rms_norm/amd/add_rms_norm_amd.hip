// Stage 4 of the fused Add + RMSNorm: RMSNorm's kernels in their residual form
// (rms_norm_kernels.h).  Each row of a and b is read once; the sum is rounded
// as Add rounds it, written to c, and normalised from registers, so the pair
// moves 4 bytes per byte of y instead of the 5 that Add followed by RMSNorm
// moves.  y and c are bit for bit what those two calls produce.
//
// c may be a or b (the residual stream updated in place); y must not overlap
// any of the others, and rows must not overlap each other.
#include "add_rms_norm_amd.h"
#include "../../rms_norm/amd/rms_norm_kernels.h"

using namespace rms_norm_kernels;

// The fp16 kernels are compiled in add_rms_norm_f16.hip: a code object is
// loaded whole at the first launch of any kernel in it, and two halves make
// that first call twice as fast for a caller that uses one element type.
void add_rms_norm_launch_f16(const RowsShape &shape, void *y, const void *a, const void *w, int w_kind,
                             const Residual<true> &res, hipStream_t stream);

infiniopStatus_t amdAddRMSNorm(AddRMSNormAmdDescriptor_t desc, void *, uint64_t, void *y, void *c, void const *a,
                               void const *b, void const *w, void *stream) {
    if (desc->elem != amd::Elem::F16 && desc->elem != amd::Elem::BF16) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (desc->n == 0 || desc->d == 0) {
        return STATUS_SUCCESS;
    }
    if (y == nullptr || c == nullptr || a == nullptr || b == nullptr || w == nullptr) {
        return STATUS_BAD_PARAM;
    }
    AMD_CHECK_HIP(hipSetDevice(desc->device_id), STATUS_BAD_DEVICE);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const RowsShape shape{desc->cu_count, desc->lds_per_block, desc->n, desc->d, desc->stride_y, desc->stride_a, desc->epsilon};
    const Residual<true> res{static_cast<uint16_t *>(c), static_cast<const uint16_t *>(b), desc->stride_c, desc->stride_b};
    const int w_kind = weight_kind(desc->w_elem);
    if (w_kind < 0) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (desc->elem == amd::Elem::F16) {
        add_rms_norm_launch_f16(shape, y, a, w, w_kind, res, s);// its kernels are a translation unit of their own
    } else {
        launch_rms_norm<amd::BF16Rne, true>(shape, y, a, w, w_kind, res, s);
    }
    AMD_CHECK_HIP(hipGetLastError(), STATUS_EXECUTION_FAILED);
    return STATUS_SUCCESS;
}
