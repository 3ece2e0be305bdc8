// amd-gpu back end of Matmul:  c = alpha * a @ b + beta * c, 2-D or batched 3-D.
// Interface shape follows the per-device functions the reference's dispatcher
// calls (src/ops/matmul/operator.cc, src/ops/matmul/cuda/matmul_cuda.h); the
// layout analysis follows src/ops/matmul/blas.h:9-113.  The product itself is
// a plain library GEMM (rocBLAS, MFMA kernels chosen by the library), as the
// reference's GPU back end uses cuBLAS (src/ops/matmul/cuda/matmul_cuda.cu).
#ifndef INFINIOP_AMD_MATMUL_H
#define INFINIOP_AMD_MATMUL_H

#include "../../../devices/amd/amd_handle.h"
#include "../../../devices/amd/common_amd.h"

namespace amd {

// One operand as a BLAS library sees it: `batch` matrices `stride` elements
// apart, each rows x cols with one of the two strides equal to 1.
struct GemmMatrix {
    int64_t batch;
    int64_t stride;
    int64_t rows, cols;
    int64_t row_stride, col_stride;

    void transpose() {
        int64_t t = rows;
        rows = cols;
        cols = t;
        t = row_stride;
        row_stride = col_stride;
        col_stride = t;
    }
    // leading dimension of the column-major view (or of its transpose)
    int64_t ld() const { return row_stride == 1 ? col_stride : row_stride; }
    // true when the matrix, as stored, is column-major
    bool column_major() const { return row_stride == 1; }
};

}// namespace amd

struct MatmulAmdDescriptor {
    Device device;
    int device_id;
    amd::Elem elem;
    // The problem after it has been turned into column-major form: when c is
    // stored row-major, c^T = b^T a^T is computed instead, and a and b (and
    // the data pointers at call time) change places.
    amd::GemmMatrix a, b, c;
    int64_t m, n, k, batch;
    bool operands_swapped;
    float alpha, beta;
};
typedef MatmulAmdDescriptor *MatmulAmdDescriptor_t;

infiniopStatus_t amdCreateMatmulDescriptor(AmdHandle_t handle, MatmulAmdDescriptor_t *desc_ptr,
                                           infiniopTensorDescriptor_t c_desc, float alpha,
                                           infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc, float beta);
infiniopStatus_t amdGetMatmulWorkspaceSize(MatmulAmdDescriptor_t desc, uint64_t *size);
infiniopStatus_t amdMatmul(MatmulAmdDescriptor_t desc, void *workspace, uint64_t workspace_size,
                           void *c, void const *a, void const *b, void *stream);
infiniopStatus_t amdDestroyMatmulDescriptor(MatmulAmdDescriptor_t desc);

// Few columns against very many rows of 32-512 contiguous elements (the scores of an attention while decoding):
// this library's own kernel, bound by reading a once (matmul_skinny.hip).  a, b, c as the descriptor's
// column-major problem has them; false when the call is not of that shape (nothing launched then).
bool amd_matmul_skinny(const MatmulAmdDescriptor &desc, void *c, const void *a, const void *b, hipStream_t stream);
// Few columns and up to 256 rows summed over very many k (the weighted values of an attention while decoding):
// k split over workgroups, their partial sums through the workspace (matmul_long_k.hip).  The first gives the
// bytes of workspace the descriptor's shape needs for it (0: not a shape for it); the second is false when the
// call is not of that shape or came without that workspace (nothing launched then).
uint64_t amd_matmul_long_k_workspace(const MatmulAmdDescriptor &desc);
bool amd_matmul_long_k(const MatmulAmdDescriptor &desc, void *workspace, uint64_t workspace_size, void *c, const void *a, const void *b,
                       hipStream_t stream);

#endif
