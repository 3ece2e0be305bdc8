// MLP:  y = alpha * (SwiGLU(x @ w12)) @ w3  (+ y when `residual` is set).
//
// A composite of this library's own public operators, as in the reference
// (src/ops/mlp/operator.cc:22-122): Matmul into a [tokens, 2*di] scratch
// tensor, SwiGLU on its two halves (gate = columns 0..di-1, up = columns
// di..2di-1 - the fused gate/up layout the SwiGLU kernels have a row-strided
// fast path for), Matmul into y.  The caller provides the scratch memory:
// workspace = [tokens, 2*di] followed by [tokens, di], in x's element type.
#include "../../devices/amd/common_amd.h"
#include <new>

namespace {

struct MlpDescriptor {
    Device device;
    infiniopMatmulDescriptor_t gate_up_proj;
    infiniopSwiGLUDescriptor_t activation;
    infiniopMatmulDescriptor_t down_proj;
    uint64_t gate_up_bytes; // [tokens, 2*di]
    uint64_t hidden_bytes;  // [tokens, di]
    uint64_t up_offset_bytes;// where the `up` half of a gate/up row starts
    uint64_t matmul_bytes;   // the larger of what the two Matmuls ask for (few tokens: their sums are split over workgroups), used by one after the other
};

uint64_t matmul_offset(const MlpDescriptor &d) { return (d.gate_up_bytes + d.hidden_bytes + 15) / 16 * 16; }
uint64_t workspace_bytes(const MlpDescriptor &d) {
    return d.matmul_bytes != 0 ? matmul_offset(d) + d.matmul_bytes : d.gate_up_bytes + d.hidden_bytes;
}

uint64_t elem_size(DataLayout dt) { return dt.size; }

void destroy_all(MlpDescriptor *d) {
    if (d->gate_up_proj) infiniopDestroyMatmulDescriptor(d->gate_up_proj);
    if (d->activation) infiniopDestroySwiGLUDescriptor(d->activation);
    if (d->down_proj) infiniopDestroyMatmulDescriptor(d->down_proj);
    delete d;
}

}// namespace

INFINIOP_C infiniopStatus_t infiniopCreateMLPDescriptor(infiniopHandle_t handle, infiniopMLPDescriptor_t *desc_ptr,
                                                        infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t x_desc,
                                                        infiniopTensorDescriptor_t w12_desc, infiniopTensorDescriptor_t w3_desc,
                                                        float alpha, char residual) {
    if (handle == nullptr || y_desc == nullptr || x_desc == nullptr || w12_desc == nullptr || w3_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (handle->device != DevAmdGpu) {
        return STATUS_BAD_DEVICE;
    }
    if (y_desc->ndim != 2 || x_desc->ndim != 2 || w12_desc->ndim != 2 || w3_desc->ndim != 2) {
        return STATUS_BAD_TENSOR_SHAPE;
    }
    if (x_desc->strides[1] != 1 || y_desc->strides[1] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    if (w12_desc->shape[1] % 2 != 0) {
        return STATUS_BAD_TENSOR_SHAPE;// the reference halves it without looking
    }
    const uint64_t tokens = x_desc->shape[0], two_di = w12_desc->shape[1], di = two_di / 2;
    auto *d = new (std::nothrow) MlpDescriptor{handle->device, nullptr, nullptr, nullptr, 0, 0, 0, 0};
    if (d == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    infiniopTensorDescriptor_t gate_up = nullptr, hidden = nullptr, half = nullptr;
    const uint64_t gate_up_shape[2] = {tokens, two_di}, hidden_shape[2] = {tokens, di};
    const int64_t half_strides[2] = {static_cast<int64_t>(two_di), 1};
    infiniopStatus_t st = infiniopCreateTensorDescriptor(&gate_up, 2, gate_up_shape, nullptr, x_desc->dt);
    if (st == STATUS_SUCCESS) st = infiniopCreateTensorDescriptor(&hidden, 2, hidden_shape, nullptr, x_desc->dt);
    if (st == STATUS_SUCCESS) st = infiniopCreateTensorDescriptor(&half, 2, hidden_shape, half_strides, x_desc->dt);
    if (st == STATUS_SUCCESS) st = infiniopCreateMatmulDescriptor(handle, &d->gate_up_proj, gate_up, 1.0f, x_desc, w12_desc, 0.0f);
    if (st == STATUS_SUCCESS) st = infiniopCreateSwiGLUDescriptor(handle, &d->activation, hidden, half, half);
    if (st == STATUS_SUCCESS) st = infiniopCreateMatmulDescriptor(handle, &d->down_proj, y_desc, alpha, hidden, w3_desc, residual ? 1.0f : 0.0f);
    if (gate_up) infiniopDestroyTensorDescriptor(gate_up);
    if (hidden) infiniopDestroyTensorDescriptor(hidden);
    if (half) infiniopDestroyTensorDescriptor(half);
    if (st != STATUS_SUCCESS) {
        destroy_all(d);
        return st;
    }
    d->gate_up_bytes = tokens * two_di * elem_size(x_desc->dt);
    d->hidden_bytes = tokens * di * elem_size(x_desc->dt);
    d->up_offset_bytes = di * elem_size(x_desc->dt);
    uint64_t first = 0, second = 0;
    infiniopGetMatmulWorkspaceSize(d->gate_up_proj, &first);
    infiniopGetMatmulWorkspaceSize(d->down_proj, &second);
    d->matmul_bytes = first > second ? first : second;
    *desc_ptr = reinterpret_cast<infiniopMLPDescriptor_t>(d);
    return STATUS_SUCCESS;
}

INFINIOP_C infiniopStatus_t infiniopGetMLPWorkspaceSize(infiniopMLPDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr || size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    auto *d = reinterpret_cast<MlpDescriptor *>(desc);
    *size = workspace_bytes(*d);
    return STATUS_SUCCESS;
}

INFINIOP_C infiniopStatus_t infiniopMLP(infiniopMLPDescriptor_t desc, void *workspace, uint64_t workspace_size, void *y,
                                        void const *x, void const *w12, void const *w3, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    auto *d = reinterpret_cast<MlpDescriptor *>(desc);
    if (workspace_size < workspace_bytes(*d) || (workspace == nullptr && workspace_bytes(*d) > 0)) {
        return STATUS_MEMORY_NOT_ALLOCATED;// the reference's answer to a short workspace (mlp/operator.cc:100-102)
    }
    char *gate_up = static_cast<char *>(workspace);
    char *hidden = gate_up + d->gate_up_bytes;
    char *for_matmul = d->matmul_bytes != 0 ? static_cast<char *>(workspace) + matmul_offset(*d) : nullptr;
    infiniopStatus_t st = infiniopMatmul(d->gate_up_proj, for_matmul, d->matmul_bytes, gate_up, x, w12, stream);
    if (st != STATUS_SUCCESS) return st;
    st = infiniopSwiGLU(d->activation, hidden, gate_up + d->up_offset_bytes, gate_up, stream);
    if (st != STATUS_SUCCESS) return st;
    return infiniopMatmul(d->down_proj, for_matmul, d->matmul_bytes, y, hidden, w3, stream);
}

INFINIOP_C infiniopStatus_t infiniopDestroyMLPDescriptor(infiniopMLPDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    destroy_all(reinterpret_cast<MlpDescriptor *>(desc));
    return STATUS_SUCCESS;
}
