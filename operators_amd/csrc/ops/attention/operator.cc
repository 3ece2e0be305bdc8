// Attention with a KV cache:
//     k, v -> their caches at position `pos`
//     out = softmax_causal(q @ K^T / sqrt(head_dim)) @ V        K, V = the caches up to pos + seq_len
// for q [n_q_head, seq, head_dim], k and v [n_kv_head, seq, head_dim], caches
// [n_kv_head, capacity, head_dim] (any strides with a unit innermost one), out
// [seq, n_q_head, head_dim] contiguous; n_q_head a multiple of n_kv_head (the
// query heads of a group share their K and V).
//
// A composite of this library's own public operators, as in the reference
// (src/ops/attention/operator.cc:31-320): Rearrange (cache writes, q made
// contiguous, the final head transpose), two batched Matmuls and CausalSoftmax
// in place on the scores.  Checks and status codes are the reference's.  The
// caller provides the scratch memory: q made contiguous (when it is not),
// the scores [n_q_head, seq, pos + seq] and the head-major result (unless seq or
// n_q_head is 1, when it is out itself), in q's type.
#include "../../devices/amd/common_amd.h"
#include <cmath>
#include <new>

namespace {

struct AttentionPlan {
    Device device;
    infiniopRearrangeDescriptor_t store_k, store_v, pack_q, unpack_out;
    infiniopMatmulDescriptor_t scores, weighted;
    infiniopCausalSoftmaxDescriptor_t softmax;
    uint64_t q_bytes;     // 0 when q is used where it lies
    uint64_t scores_bytes;// [n_q_head, seq, total]
    uint64_t result_bytes;// [n_q_head, seq, head_dim]
    uint64_t softmax_bytes;// what CausalSoftmax asks for (few long rows: decoding over a long context), behind the rest on a 16-byte boundary
    uint64_t weighted_bytes;// what the second Matmul asks for (decoding: its sum over the keys is split over workgroups), behind that
    uint64_t k_offset_bytes, v_offset_bytes;// position `pos` in the caches
};

uint64_t softmax_offset(const AttentionPlan &p) { return (p.q_bytes + p.scores_bytes + p.result_bytes + 15) / 16 * 16; }
uint64_t weighted_offset(const AttentionPlan &p) { return (softmax_offset(p) + p.softmax_bytes + 15) / 16 * 16; }
uint64_t workspace_bytes(const AttentionPlan &p) {
    if (p.weighted_bytes != 0) return weighted_offset(p) + p.weighted_bytes;
    return p.softmax_bytes != 0 ? softmax_offset(p) + p.softmax_bytes : p.q_bytes + p.scores_bytes + p.result_bytes;
}

void destroy_all(AttentionPlan *p) {
    if (p->store_k) infiniopDestroyRearrangeDescriptor(p->store_k);
    if (p->store_v) infiniopDestroyRearrangeDescriptor(p->store_v);
    if (p->pack_q) infiniopDestroyRearrangeDescriptor(p->pack_q);
    if (p->unpack_out) infiniopDestroyRearrangeDescriptor(p->unpack_out);
    if (p->scores) infiniopDestroyMatmulDescriptor(p->scores);
    if (p->weighted) infiniopDestroyMatmulDescriptor(p->weighted);
    if (p->softmax) infiniopDestroyCausalSoftmaxDescriptor(p->softmax);
    delete p;
}

// A scratch list of tensor descriptors that are all released together.
struct Descriptors {
    infiniopTensorDescriptor_t made[12];
    int count = 0;
    infiniopStatus_t status = STATUS_SUCCESS;

    infiniopTensorDescriptor_t make(DataLayout dt, uint64_t d0, uint64_t d1, uint64_t d2, int64_t s0, int64_t s1, int64_t s2) {
        const uint64_t shape[3] = {d0, d1, d2};
        const int64_t strides[3] = {s0, s1, s2};
        infiniopTensorDescriptor_t t = nullptr;
        const infiniopStatus_t st = infiniopCreateTensorDescriptor(&t, 3, shape, strides, dt);
        if (st != STATUS_SUCCESS) {
            status = st;
            return nullptr;
        }
        made[count++] = t;
        return t;
    }
    infiniopTensorDescriptor_t dense(DataLayout dt, uint64_t d0, uint64_t d1, uint64_t d2) {
        return make(dt, d0, d1, d2, static_cast<int64_t>(d1 * d2), static_cast<int64_t>(d2), 1);
    }
    ~Descriptors() {
        for (int i = 0; i < count; ++i) infiniopDestroyTensorDescriptor(made[i]);
    }
};

}// namespace

INFINIOP_C infiniopStatus_t infiniopCreateAttentionDescriptor(infiniopHandle_t handle, infiniopAttentionDescriptor_t *desc_ptr,
                                                              infiniopTensorDescriptor_t out_desc, infiniopTensorDescriptor_t q_desc,
                                                              infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,
                                                              infiniopTensorDescriptor_t k_cache_desc,
                                                              infiniopTensorDescriptor_t v_cache_desc, uint64_t pos) {
    if (handle == nullptr || out_desc == nullptr || q_desc == nullptr || k_desc == nullptr || v_desc == nullptr ||
        k_cache_desc == nullptr || v_cache_desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    if (desc_ptr == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    if (handle->device != DevAmdGpu) {
        return STATUS_BAD_DEVICE;
    }
    for (infiniopTensorDescriptor_t t : {out_desc, q_desc, k_desc, v_desc, k_cache_desc, v_cache_desc}) {
        if (t->ndim != 3) return STATUS_BAD_TENSOR_SHAPE;
    }
    if (!amd::ref_contiguous(out_desc) || out_desc->strides[2] != 1) {
        return STATUS_BAD_TENSOR_STRIDES;
    }
    for (infiniopTensorDescriptor_t t : {q_desc, k_desc, v_desc, k_cache_desc, v_cache_desc}) {
        if (t->strides[2] != 1) return STATUS_BAD_TENSOR_STRIDES;
    }
    const uint64_t heads = q_desc->shape[0], seq = q_desc->shape[1], hd = q_desc->shape[2];
    const uint64_t kv_heads = k_desc->shape[0], total = seq + pos;
    if (out_desc->shape[0] != seq || out_desc->shape[1] != heads || out_desc->shape[2] != hd) return STATUS_BAD_PARAM;
    if (k_desc->shape[1] != seq || k_desc->shape[2] != hd) return STATUS_BAD_PARAM;
    if (v_desc->shape[0] != kv_heads || v_desc->shape[1] != seq || v_desc->shape[2] != hd) return STATUS_BAD_PARAM;
    for (infiniopTensorDescriptor_t t : {k_cache_desc, v_cache_desc}) {
        if (t->shape[0] != kv_heads || t->shape[1] < total || t->shape[2] != hd) return STATUS_BAD_PARAM;
    }
    if (kv_heads == 0 || heads % kv_heads != 0) {
        return STATUS_BAD_PARAM;// the query heads must split evenly over the K/V heads
    }
    const uint64_t group = heads / kv_heads;
    const DataLayout dt = q_desc->dt;
    const uint64_t es = dt.size;

    auto *p = new (std::nothrow) AttentionPlan{handle->device, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0, 0, 0, 0, 0, 0};
    if (p == nullptr) {
        return STATUS_MEMORY_NOT_ALLOCATED;
    }
    Descriptors d;
    infiniopStatus_t st = STATUS_SUCCESS;
    auto ok = [&]() { return st == STATUS_SUCCESS && d.status == STATUS_SUCCESS; };

    // k and v into their caches, seq rows starting at row `pos`
    infiniopTensorDescriptor_t k_slot = d.make(k_cache_desc->dt, kv_heads, seq, hd, k_cache_desc->strides[0], k_cache_desc->strides[1], 1);
    infiniopTensorDescriptor_t v_slot = d.make(v_cache_desc->dt, kv_heads, seq, hd, v_cache_desc->strides[0], v_cache_desc->strides[1], 1);
    if (ok()) st = infiniopCreateRearrangeDescriptor(handle, &p->store_k, k_slot, k_desc);
    if (ok()) st = infiniopCreateRearrangeDescriptor(handle, &p->store_v, v_slot, v_desc);

    // q as a dense [heads, seq, hd]; copied there unless it already is
    // (the stride of a dimension of extent 1 says nothing: one decoded token's q is dense whatever buffer its heads are a view of)
    const bool q_dense = (seq == 1 || q_desc->strides[1] == static_cast<int64_t>(hd)) &&
                         (heads == 1 || q_desc->strides[0] == static_cast<int64_t>(seq * hd));
    infiniopTensorDescriptor_t q_packed = d.dense(dt, heads, seq, hd);
    if (!q_dense) {
        if (ok()) st = infiniopCreateRearrangeDescriptor(handle, &p->pack_q, q_packed, q_desc);
        p->q_bytes = heads * seq * hd * es;
    }

    // scores[kv, group*seq, total] = q[kv, group*seq, hd] @ K^T[kv, hd, total] / sqrt(hd)
    infiniopTensorDescriptor_t q_grouped = d.dense(dt, kv_heads, group * seq, hd);
    infiniopTensorDescriptor_t k_t = d.make(k_cache_desc->dt, kv_heads, hd, total, k_cache_desc->strides[0], 1, k_cache_desc->strides[1]);
    infiniopTensorDescriptor_t scores_grouped = d.dense(dt, kv_heads, group * seq, total);
    if (ok()) st = infiniopCreateMatmulDescriptor(handle, &p->scores, scores_grouped, 1 / sqrt(hd), q_grouped, k_t, 0.0f);
    p->scores_bytes = heads * seq * total * es;

    // causal softmax in place on scores seen as [heads, seq, total]
    infiniopTensorDescriptor_t scores_by_head = d.dense(dt, heads, seq, total);
    if (ok()) st = infiniopCreateCausalSoftmaxDescriptor(handle, &p->softmax, scores_by_head);
    if (ok()) st = infiniopGetCausalSoftmaxWorkspaceSize(p->softmax, &p->softmax_bytes);

    // result[kv, group*seq, hd] = scores[kv, group*seq, total] @ V[kv, total, hd]
    infiniopTensorDescriptor_t v_full = d.make(v_cache_desc->dt, kv_heads, total, hd, v_cache_desc->strides[0], v_cache_desc->strides[1], 1);
    infiniopTensorDescriptor_t result_grouped = d.dense(dt, kv_heads, group * seq, hd);
    if (ok()) st = infiniopCreateMatmulDescriptor(handle, &p->weighted, result_grouped, 1.0f, scores_grouped, v_full, 0.0f);
    if (ok()) st = infiniopGetMatmulWorkspaceSize(p->weighted, &p->weighted_bytes);
    // out[seq, heads, hd] = result[heads, seq, hd] with its first two dimensions exchanged - which moves nothing when
    // one of the two has extent 1 (one decoded token): the second Matmul then writes out itself
    if (seq != 1 && heads != 1) {
        p->result_bytes = heads * seq * hd * es;
        infiniopTensorDescriptor_t result_t = d.make(dt, seq, heads, hd, static_cast<int64_t>(hd), static_cast<int64_t>(seq * hd), 1);
        if (ok()) st = infiniopCreateRearrangeDescriptor(handle, &p->unpack_out, out_desc, result_t);
    }

    if (!ok()) {
        destroy_all(p);
        return st != STATUS_SUCCESS ? st : d.status;
    }
    p->k_offset_bytes = pos * static_cast<uint64_t>(k_cache_desc->strides[1]) * k_cache_desc->dt.size;
    p->v_offset_bytes = pos * static_cast<uint64_t>(v_cache_desc->strides[1]) * v_cache_desc->dt.size;
    *desc_ptr = reinterpret_cast<infiniopAttentionDescriptor_t>(p);
    return STATUS_SUCCESS;
}

INFINIOP_C infiniopStatus_t infiniopGetAttentionWorkspaceSize(infiniopAttentionDescriptor_t desc, uint64_t *size) {
    if (desc == nullptr || size == nullptr) {
        return STATUS_BAD_PARAM;
    }
    auto *p = reinterpret_cast<AttentionPlan *>(desc);
    *size = workspace_bytes(*p);
    return STATUS_SUCCESS;
}

INFINIOP_C infiniopStatus_t infiniopAttention(infiniopAttentionDescriptor_t desc, void *workspace, uint64_t workspace_size, void *out,
                                              void const *q, void const *k, void const *v, void *k_cache, void *v_cache, void *stream) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    auto *p = reinterpret_cast<AttentionPlan *>(desc);
    const uint64_t need = workspace_bytes(*p);
    if (workspace_size < need || (workspace == nullptr && need > 0)) {
        return STATUS_MEMORY_NOT_ALLOCATED;// the reference's answer to a short workspace (attention/operator.cc:264-266)
    }
    if (out == nullptr || q == nullptr || k == nullptr || v == nullptr || k_cache == nullptr || v_cache == nullptr) {
        return STATUS_BAD_PARAM;
    }
    char *q_packed = static_cast<char *>(workspace);
    char *scores = q_packed + p->q_bytes;
    char *result = p->unpack_out != nullptr ? scores + p->scores_bytes : static_cast<char *>(out);
    char *softmax_parts = p->softmax_bytes != 0 ? static_cast<char *>(workspace) + softmax_offset(*p) : nullptr;
    char *weighted_parts = p->weighted_bytes != 0 ? static_cast<char *>(workspace) + weighted_offset(*p) : nullptr;

    infiniopStatus_t st = infiniopRearrange(p->store_k, static_cast<char *>(k_cache) + p->k_offset_bytes, k, stream);
    if (st == STATUS_SUCCESS) st = infiniopRearrange(p->store_v, static_cast<char *>(v_cache) + p->v_offset_bytes, v, stream);
    if (st == STATUS_SUCCESS && p->pack_q != nullptr) {
        st = infiniopRearrange(p->pack_q, q_packed, q, stream);
        q = q_packed;
    }
    if (st == STATUS_SUCCESS) st = infiniopMatmul(p->scores, nullptr, 0, scores, q, k_cache, stream);
    if (st == STATUS_SUCCESS) st = infiniopCausalSoftmax(p->softmax, softmax_parts, p->softmax_bytes, scores, stream);
    if (st == STATUS_SUCCESS) st = infiniopMatmul(p->weighted, weighted_parts, p->weighted_bytes, result, scores, v_cache, stream);
    if (st == STATUS_SUCCESS && p->unpack_out != nullptr) st = infiniopRearrange(p->unpack_out, out, result, stream);
    return st;
}

INFINIOP_C infiniopStatus_t infiniopDestroyAttentionDescriptor(infiniopAttentionDescriptor_t desc) {
    if (desc == nullptr) {
        return STATUS_BAD_PARAM;
    }
    destroy_all(reinterpret_cast<AttentionPlan *>(desc));
    return STATUS_SUCCESS;
}
