// Create-time validation and layout analysis for Matmul on the amd-gpu device.
//
// Rules and codes are the reference's (src/ops/matmul/blas.h:19-113,
// src/ops/matmul/cuda/matmul_cuda.cc:5-33): F16 or F32 by c's type (BF16 is
// this back end's extension); every operand 2-D or 3-D, else
// STATUS_BAD_TENSOR_SHAPE; one of its two matrix strides must be 1, else
// STATUS_BAD_TENSOR_STRIDES; a and b have c's batch count or 1, else
// STATUS_BAD_PARAM.  One deliberate difference: where the reference ends the
// process on mismatched extents (its ASSERT_EQ, blas.h:88-90), this back end
// answers STATUS_BAD_TENSOR_SHAPE.
#include "matmul_amd.h"
#include <new>

namespace {

infiniopStatus_t read_matrix(infiniopTensorDescriptor_t t, amd::GemmMatrix *out) {
    if (t->ndim == 2) {
        *out = amd::GemmMatrix{1, 0, static_cast<int64_t>(t->shape[0]), static_cast<int64_t>(t->shape[1]), t->strides[0], t->strides[1]};
    } else if (t->ndim == 3) {
        const int64_t batch = static_cast<int64_t>(t->shape[0]);
        *out = amd::GemmMatrix{batch, batch == 1 ? 0 : t->strides[0], static_cast<int64_t>(t->shape[1]),
                               static_cast<int64_t>(t->shape[2]), t->strides[1], t->strides[2]};
    } else {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (out->row_stride != 1 && out->col_stride != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    return STATUS_SUCCESS;
}

}// namespace

infiniopStatus_t amdCreateMatmulDescriptor(AmdHandle_t handle, MatmulAmdDescriptor_t *desc_ptr,
                                           infiniopTensorDescriptor_t c_desc, float alpha,
                                           infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc, float beta) {
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    const amd::Elem elem = amd::elem_of(c_desc->dt);
    if (elem == amd::Elem::Other) {
        return STATUS_BAD_TENSOR_DTYPE;
    }
    if (!amd::same_dt(c_desc->dt, a_desc->dt) || !amd::same_dt(c_desc->dt, b_desc->dt)) {
        return STATUS_BAD_TENSOR_DTYPE;// the reference reads a and b as c's type without looking
    }
    amd::GemmMatrix a, b, c;
    infiniopStatus_t st;
    if ((st = read_matrix(a_desc, &a)) != STATUS_SUCCESS) return st;
    if ((st = read_matrix(b_desc, &b)) != STATUS_SUCCESS) return st;
    if ((st = read_matrix(c_desc, &c)) != STATUS_SUCCESS) return st;
    if (c.rows != a.rows || c.cols != b.cols || a.cols != b.rows) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    const int64_t batch = c.batch;
    if ((a.batch != batch && a.batch != 1) || (b.batch != batch && b.batch != 1)) {
        return STATUS_BAD_PARAM;
    }
    // BLAS libraries produce a column-major c.  A row-major c is the
    // column-major c^T = b^T a^T: transpose all three and let a and b change
    // places (blas.h:100-106).
    bool swapped = false;
    if (c.col_stride == 1) {
        a.transpose();
        b.transpose();
        c.transpose();
        const amd::GemmMatrix t = a;
        a = b;
        b = t;
        swapped = true;
    }
    // what the library call needs to hold in 32-bit integers
    const int64_t lim = 0x7FFFFFFF;
    if (c.rows > lim || c.cols > lim || a.cols > lim || a.ld() > lim || b.ld() > lim || c.ld() > lim || batch > lim) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    auto *desc = new (std::nothrow) MatmulAmdDescriptor{DevAmdGpu, handle->device_id, elem, a, b, c, c.rows, c.cols, a.cols,
                                                        batch, swapped, alpha, beta};
    if (desc == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    *desc_ptr = desc;
    return STATUS_SUCCESS;
}

infiniopStatus_t amdGetMatmulWorkspaceSize(MatmulAmdDescriptor_t desc, uint64_t *size) {
    if (size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    // 0 as in the reference (matmul_cuda.cc:35-38; the BLAS library manages its own scratch), except for the one
    // shape this library splits along k itself; a call that comes without that workspace goes to the BLAS library
    *size = amd_matmul_long_k_workspace(*desc);
    return STATUS_SUCCESS;
}

infiniopStatus_t amdDestroyMatmulDescriptor(MatmulAmdDescriptor_t desc) {
    delete desc;
    return STATUS_SUCCESS;
}
