// amd-gpu back end of CausalSoftmax.  Interface shape follows the per-device
// functions the reference's dispatcher calls
// (src/ops/causal_softmax/operator.cc:21-130).
#ifndef INFINIOP_AMD_CAUSAL_SOFTMAX_H
#define INFINIOP_AMD_CAUSAL_SOFTMAX_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

struct CausalSoftmaxAmdDescriptor {
    Device device;
    int device_id;
    int cu_count;
    amd::Elem elem;
    uint64_t batch;// product of the leading dimensions
    uint64_t seq;  // rows per matrix
    uint64_t total;// columns
    int64_t stride_b, stride_i;// elements; the innermost stride is 1
};
typedef CausalSoftmaxAmdDescriptor *CausalSoftmaxAmdDescriptor_t;

// Very few very long rows - decoding over a context of 128 Ki keys and more has one query row per head - leave
// most compute units idle at a workgroup per row.  Such a call splits every row into parts of 16 384 (or 4096)
// columns, a workgroup each, in two launches that exchange the parts' maxima and sums
// through the workspace (causal_softmax_split_stats, causal_softmax_split_apply).  That reads the rows twice and
// costs a second launch, so it pays only where the rows are few: measured on MI355X, bf16, a workgroup per row /
// split, us: [8, 1, 131072] 16.0 / 7.8, [32, 1, 131072] 18.0 / 12.9, [64, 1, 131072] 18.7 / 19.7,
// [128, 1, 131072] 21.1 / 34.2, [16, 1, 262144] 45.3 / 12.9, [64, 1, 262144] 47.3 / 34.3, [128, 1, 262144]
// 49.5 / 61.9; [64, 1, 65536] 12.2 / 12.9, [64, 1, 32768] 7.0 / 11.6.  Without the workspace the call is served a
// workgroup per row, as every other shape is.
struct CausalSoftmaxPart {
    float max, min, sum, unused;// of the part's kept columns; the sum is of exp(x - max)
};
// Lanes of the workgroup that takes a part, 4 vectors of 8 columns per lane: 512 (parts of 16 384 columns), or 128
// where even those would be 64 workgroups and fewer ([8, 1, 131072]: 7.8 us with 128 lanes, 10.9 with 512;
// [32, 1, 131072] 12.9 / 12.6, [16, 1, 262144] 13.0 / 12.6).
inline uint32_t causal_softmax_part_lanes(const CausalSoftmaxAmdDescriptor &d) {
    return d.total <= 262144 && d.batch * d.seq * ((d.total + 16383) / 16384) <= 64 ? 128 : 512;
}
// Parts per row when the descriptor's shape takes the split form, else 0.
inline uint32_t causal_softmax_parts(const CausalSoftmaxAmdDescriptor &d) {
    const uint64_t rows = d.batch * d.seq, units = static_cast<uint64_t>(d.cu_count);
    const uint64_t columns = causal_softmax_part_lanes(d) * 32ull;
    if (rows == 0 || d.total < 131072 || d.total >= (1ull << 31)) return 0;
    if (d.total % 8 != 0 || d.stride_i % 8 != 0 || d.stride_b % 8 != 0) return 0;// rows of whole 16-byte vectors
    const uint64_t parts = (d.total + columns - 1) / columns;
    if (parts > 64) return 0;// a wavefront puts a row's parts together, one per lane
    // up to a workgroup per compute unit; rows beyond 131 072 columns, which a workgroup on its own reads twice, up to a row per four units
    const bool few = rows * ((d.total + 16383) / 16384) <= units || (d.total > 131072 && rows * 4 <= units);
    return few ? static_cast<uint32_t>(parts) : 0;
}

infiniopStatus_t amdCreateCausalSoftmaxDescriptor(AmdHandle_t handle, CausalSoftmaxAmdDescriptor_t *desc_ptr,
                                                  infiniopTensorDescriptor_t y_desc);
infiniopStatus_t amdGetCausalSoftmaxWorkspaceSize(CausalSoftmaxAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdCausalSoftmax(CausalSoftmaxAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                                  void *data, void *stream);
infiniopStatus_t amdDestroyCausalSoftmaxDescriptor(CausalSoftmaxAmdDescriptor_t desc);

#endif
