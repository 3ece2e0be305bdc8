/*
 * infiniop.h - the C ABI exported by this build of libinfiniop.so.
 *
 * The library implements ONE device of the InfiniOperators operator library,
 * `DevAmdGpu` (AMD Instinct MI355X, gfx950), for the four memory-bound LLM-layer
 * operators Add, RMSNorm, RoPE and SwiGLU, plus CausalSoftmax, Rearrange,
 * Matmul, RandomSample, the MLP and Attention composites and a fused AddRMSNorm (the one operator here that
 * the reference does not have).
 * The entry points below have the
 * names, argument order, argument meaning and status codes of the reference
 * library, so that a caller written against the reference (its ctypes harness,
 * its composite operators, any C client) binds to this library unchanged and
 * only selects another device number.  Each declaration names the reference
 * declaration it stands in for (paths relative to the reference checkout).
 *
 * Calling convention ("3+1 stages"):
 *   1. infiniopCreateHandle(&handle, DevAmdGpu, device_id)
 *   2. infiniopCreate<Op>Descriptor(handle, &desc, tensor descriptors...)
 *        all shape/stride/dtype checking happens here, once
 *   3. infiniopGet<Op>WorkspaceSize(desc, &bytes)        (RMSNorm, RoPE, CausalSoftmax, Matmul, AddRMSNorm: always 0; RandomSample: candidate lists, optional; MLP, Attention: their intermediates)
 *   4. infiniop<Op>(desc, ..., data pointers..., stream)
 *        enqueues on `stream` (a hipStream_t, NULL = the null stream) and
 *        returns without synchronising
 *   +  infiniopDestroy<Op>Descriptor(desc), infiniopDestroyHandle(handle)
 *
 * All data pointers are device pointers on the handle's GPU.  Strides are in
 * elements.  Descriptors are immutable after creation: one descriptor may be
 * used from several host threads and streams at once.
 */
#ifndef INFINIOP_AMD_INFINIOP_H
#define INFINIOP_AMD_INFINIOP_H

#include <stdint.h>

#if defined(__GNUC__)
#define INFINIOP_EXPORT __attribute__((visibility("default")))
#else
#define INFINIOP_EXPORT
#endif

#ifdef __cplusplus
#define INFINIOP_C extern "C"
#else
#define INFINIOP_C
#endif

/* ---- status codes: replaces include/status.h:4-14 ---------------------- */
typedef enum {
    STATUS_SUCCESS = 0,
    STATUS_EXECUTION_FAILED = 1,
    STATUS_BAD_PARAM = 2,
    STATUS_BAD_TENSOR_DTYPE = 3,
    STATUS_BAD_TENSOR_SHAPE = 4,
    STATUS_BAD_TENSOR_STRIDES = 5,
    STATUS_MEMORY_NOT_ALLOCATED = 6,
    STATUS_INSUFFICIENT_WORKSPACE = 7,
    STATUS_BAD_DEVICE = 8,
} infiniopStatus_t;

/* ---- devices: replaces include/device.h:4-9 ----------------------------
 * Values 0..3 are the reference's and keep their meaning; this library answers
 * STATUS_BAD_DEVICE for them.  DevAmdGpu = 4 is the value a maintainer appends
 * to the reference enum. */
enum DeviceEnum {
    DevCpu = 0,
    DevNvGpu = 1,
    DevCambriconMlu = 2,
    DevAscendNpu = 3,
    DevAmdGpu = 4,
};
typedef enum DeviceEnum Device;

/* ---- element types: replaces include/data_type.h:4-46 ------------------
 * A 4-byte bitfield passed BY VALUE; two layouts are the same type when their
 * 32-bit images are equal. */
typedef struct DataLayout {
    unsigned short
        packed : 8,
        sign : 1,
        size : 7,
        mantissa : 8,
        exponent : 8;
} DataLayout;
typedef struct DataLayout DT;

#define INFINIOP_DT(p, s, z, m, e) {p, s, z, m, e}
static const DataLayout
    I8 = INFINIOP_DT(1, 1, 1, 7, 0),
    I16 = INFINIOP_DT(1, 1, 2, 15, 0),
    I32 = INFINIOP_DT(1, 1, 4, 31, 0),
    I64 = INFINIOP_DT(1, 1, 8, 63, 0),
    U8 = INFINIOP_DT(1, 0, 1, 8, 0),
    U16 = INFINIOP_DT(1, 0, 2, 16, 0),
    U32 = INFINIOP_DT(1, 0, 4, 32, 0),
    U64 = INFINIOP_DT(1, 0, 8, 64, 0),
    F16 = INFINIOP_DT(1, 1, 2, 10, 5),
    BF16 = INFINIOP_DT(1, 1, 2, 7, 8),
    F32 = INFINIOP_DT(1, 1, 4, 23, 8),
    F64 = INFINIOP_DT(1, 1, 8, 52, 11);

/* ---- tensor descriptor: replaces include/tensor.h:7-18 ----------------- */
struct TensorDescriptor {
    DT dt;            /* element type */
    uint64_t ndim;    /* number of dimensions, 0 allowed */
    uint64_t *shape;  /* ndim extents */
    int64_t *strides; /* ndim strides, in elements */
};
typedef struct TensorDescriptor *infiniopTensorDescriptor_t;

/* replaces include/tensor/tensor_descriptor.h:8 - deep-copies shape and strides;
 * strides == NULL means contiguous row-major. */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateTensorDescriptor(
    infiniopTensorDescriptor_t *desc_ptr, uint64_t ndim, uint64_t const *shape,
    int64_t const *strides, DataLayout datatype);
/* replaces include/tensor/tensor_descriptor.h:10 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyTensorDescriptor(infiniopTensorDescriptor_t desc);

/* ---- handle: replaces include/handle.h:6-10 ----------------------------
 * Every handle and every operator descriptor begins with its Device; callers
 * may read that field and nothing else. */
typedef struct HandleStruct {
    Device device;
} HandleStruct;
typedef HandleStruct *infiniopHandle_t;

/* replaces include/handle/handle_export.h:8.  NULL handle_ptr ->
 * STATUS_MEMORY_NOT_ALLOCATED; device_id < 0 -> STATUS_BAD_PARAM; any device
 * other than DevAmdGpu, no such GPU, or a GPU that is not gfx950 ->
 * STATUS_BAD_DEVICE. */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateHandle(infiniopHandle_t *handle_ptr, Device device, int device_id);
/* replaces include/handle/handle_export.h:10 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyHandle(infiniopHandle_t handle);

/* ======================================================================== *
 * Add:  c = a + b with numpy-style broadcasting of a and b onto c.
 * F16, F32 (reference) and BF16 (extension).  c, a, b must be "contiguous" in
 * the reference's sense; c is written in flat row-major order.  In-place on a
 * or b is allowed when no broadcasting is involved.
 * ======================================================================== */
typedef struct AddDescriptor {
    Device device;
} AddDescriptor;
typedef AddDescriptor *infiniopAddDescriptor_t;

/* replaces include/ops/add/add.h:13-17 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateAddDescriptor(
    infiniopHandle_t handle, infiniopAddDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t c, infiniopTensorDescriptor_t a, infiniopTensorDescriptor_t b);
/* replaces include/ops/add/add.h:19-23 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopAdd(
    infiniopAddDescriptor_t desc, void *c, void const *a, void const *b, void *stream);
/* replaces include/ops/add/add.h:25 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyAddDescriptor(infiniopAddDescriptor_t desc);

/* ======================================================================== *
 * RMSNorm:  y[i][j] = x[i][j] * w[j] / sqrt(mean_j(x[i][j]^2) + epsilon)
 * x, y: 2-D F16 (reference) or BF16 (extension) with unit inner stride and
 * independent row strides; w: 1-D F16, BF16 or F32.
 * ======================================================================== */
typedef struct RMSNormDescriptor {
    Device device;
} RMSNormDescriptor;
typedef RMSNormDescriptor *infiniopRMSNormDescriptor_t;

/* replaces include/ops/rms_norm/rms_norm.h:13-19 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateRMSNormDescriptor(
    infiniopHandle_t handle, infiniopRMSNormDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t x_desc,
    infiniopTensorDescriptor_t w_desc, float epsilon);
/* replaces include/ops/rms_norm/rms_norm.h:21 - always 0 bytes */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetRMSNormWorkspaceSize(infiniopRMSNormDescriptor_t desc, uint64_t *size);
/* replaces include/ops/rms_norm/rms_norm.h:23-24 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopRMSNorm(
    infiniopRMSNormDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *y, void const *x, void const *w, void *stream);
/* replaces include/ops/rms_norm/rms_norm.h:26 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyRMSNormDescriptor(infiniopRMSNormDescriptor_t desc);

/* ======================================================================== *
 * RoPE:  in-place rotation of adjacent pairs (2k, 2k+1) of t[token][head][:]
 * by the angle whose sin/cos are rows pos_ids[token] of two caller-supplied
 * F32 tables [rows, head_dim].  t: 3-D F16 (reference) or BF16 (extension)
 * with arbitrary token and head strides, unit inner stride; pos_ids: 1-D U64.
 * The tables are indexed with row stride head_dim, as the reference does.
 * ======================================================================== */
typedef struct RoPEDescriptor RoPEDescriptor; /* opaque, as in the reference */
typedef RoPEDescriptor *infiniopRoPEDescriptor_t;

/* replaces include/ops/rotary_embedding/rotary_embedding.h:10-16 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateRoPEDescriptor(
    infiniopHandle_t handle, infiniopRoPEDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t t, infiniopTensorDescriptor_t pos_ids,
    infiniopTensorDescriptor_t sin_table, infiniopTensorDescriptor_t cos_table);
/* replaces include/ops/rotary_embedding/rotary_embedding.h:18 - always 0 bytes */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetRoPEWorkspaceSize(infiniopRoPEDescriptor_t desc, uint64_t *size);
/* replaces include/ops/rotary_embedding/rotary_embedding.h:20-28 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopRoPE(
    infiniopRoPEDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *t, void const *pos_ids, void const *sin_table, void const *cos_table, void *stream);
/* replaces include/ops/rotary_embedding/rotary_embedding.h:30 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyRoPEDescriptor(infiniopRoPEDescriptor_t desc);

/* ======================================================================== *
 * SwiGLU:  c = a * b * sigmoid(b)   (b is the gated operand, a the linear one)
 * 2-D F16 (reference) or BF16 (extension), unit inner stride, one row stride
 * per tensor - so a and b may be the two halves of one fused gate/up buffer.
 * In-place on a or on b is allowed.
 * ======================================================================== */
typedef struct SwiGLUDescriptor {
    Device device;
} SwiGLUDescriptor;
typedef SwiGLUDescriptor *infiniopSwiGLUDescriptor_t;

/* replaces include/ops/swiglu/swiglu.h:13-17 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateSwiGLUDescriptor(
    infiniopHandle_t handle, infiniopSwiGLUDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t c_desc, infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc);
/* replaces include/ops/swiglu/swiglu.h:19-23 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopSwiGLU(
    infiniopSwiGLUDescriptor_t desc, void *c, void const *a, void const *b, void *stream);
/* replaces include/ops/swiglu/swiglu.h:25 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroySwiGLUDescriptor(infiniopSwiGLUDescriptor_t desc);

/* ======================================================================== *
 * CausalSoftmax (first operator beyond the four-operator path):  in place,
 * over the last dimension of a [seq, total] or [batch, seq, total] tensor,
 * row i keeps columns j <= total - seq + i, is soft-maxed over them in fp32
 * and gets exact zeros in the remaining columns.  F16 (reference) or BF16
 * (extension); unit innermost stride (as the reference's GPU back end
 * requires); total >= seq.
 * ======================================================================== */
typedef struct CausalSoftmaxDescriptor {
    Device device;
} CausalSoftmaxDescriptor;
typedef CausalSoftmaxDescriptor *infiniopCausalSoftmaxDescriptor_t;

/* replaces include/ops/causal_softmax/causal_softmax.h:13-15 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateCausalSoftmaxDescriptor(
    infiniopHandle_t handle, infiniopCausalSoftmaxDescriptor_t *desc_ptr, infiniopTensorDescriptor_t y_desc);
/* replaces include/ops/causal_softmax/causal_softmax.h:17 - 0 bytes, except for very few very long rows
 * (decoding over 131 072 keys and more with up to a few dozen heads): 16 bytes per 16 384 columns of every
 * row, through which the workgroups that share a row exchange its maximum and sum.  A call that comes
 * without that workspace is served all the same, a workgroup per row. */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetCausalSoftmaxWorkspaceSize(infiniopCausalSoftmaxDescriptor_t desc, uint64_t *size);
/* replaces include/ops/causal_softmax/causal_softmax.h:19-23 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCausalSoftmax(
    infiniopCausalSoftmaxDescriptor_t desc, void *workspace, uint64_t workspace_size, void *data, void *stream);
/* replaces include/ops/causal_softmax/causal_softmax.h:25 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyCausalSoftmaxDescriptor(infiniopCausalSoftmaxDescriptor_t desc);

/* ======================================================================== *
 * Rearrange (second operator beyond the four-operator path):  dst = src for
 * two tensors of equal shape and element type whose other strides are free
 * (KV-cache writes, head transposes).  Any element type; unit innermost
 * strides; for rank >= 4 the leading dimensions must nest as the reference
 * demands.
 * ======================================================================== */
typedef struct RearrangeDescriptor {
    Device device;
} RearrangeDescriptor;
typedef RearrangeDescriptor *infiniopRearrangeDescriptor_t;

/* replaces include/ops/rearrange/rearrange.h:12-15 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateRearrangeDescriptor(
    infiniopHandle_t handle, infiniopRearrangeDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t dst, infiniopTensorDescriptor_t src);
/* replaces include/ops/rearrange/rearrange.h:17 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopRearrange(
    infiniopRearrangeDescriptor_t desc, void *dst, void const *src, void *stream);
/* replaces include/ops/rearrange/rearrange.h:19 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyRearrangeDescriptor(infiniopRearrangeDescriptor_t desc);

/* ======================================================================== *
 * Matmul:  c = alpha * a @ b + beta * c; operands 2-D [rows, cols] or 3-D
 * [batch, rows, cols] with one of the two matrix strides equal to 1 (row- or
 * column-major), a and b with c's batch count or 1.  F16, F32 (reference) and
 * BF16 (extension), one type for all three; accumulation in fp32.  A plain
 * library GEMM (rocBLAS), as the reference's GPU back end uses cuBLAS.
 * ======================================================================== */
typedef struct MatmulDescriptor {
    Device device;
} MatmulDescriptor;
typedef MatmulDescriptor *infiniopMatmulDescriptor_t;

/* replaces include/ops/matmul/matmul.h:13-19 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateMatmulDescriptor(
    infiniopHandle_t handle, infiniopMatmulDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t c_desc, float alpha,
    infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc, float beta);
/* replaces include/ops/matmul/matmul.h:21 - 0 bytes, except where up to 8 rows of a (tokens, or the queries of
 * a decoding attention) meet 1024 and more of k: 32 bytes per column of c and chunk of 128 to 2048 of k, for the
 * partial sums of the workgroups that share the sum.  A call that comes without that workspace is served all
 * the same, by the BLAS library. */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetMatmulWorkspaceSize(infiniopMatmulDescriptor_t desc, uint64_t *size);
/* replaces include/ops/matmul/matmul.h:23-29 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopMatmul(
    infiniopMatmulDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *c, void const *a, void const *b, void *stream);
/* replaces include/ops/matmul/matmul.h:31 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyMatmulDescriptor(infiniopMatmulDescriptor_t desc);

/* ======================================================================== *
 * MLP:  y = alpha * SwiGLU(x @ w12) @ w3 (+ y when residual != 0), where
 * x @ w12 is [tokens, 2*di] with the gate in columns 0..di-1 and the up
 * projection in columns di..2*di-1.  x, y: 2-D with unit inner stride; w12
 * [d, 2*di], w3 [di, d].  The caller provides the workspace (the [tokens,
 * 2*di] and [tokens, di] intermediates).  A composite of Matmul and SwiGLU.
 * ======================================================================== */
typedef struct MLPDescriptor {
    Device device;
} MLPDescriptor;
typedef MLPDescriptor *infiniopMLPDescriptor_t;

/* replaces include/ops/mlp/mlp.h:15-22 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateMLPDescriptor(
    infiniopHandle_t handle, infiniopMLPDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t x_desc,
    infiniopTensorDescriptor_t w12_desc, infiniopTensorDescriptor_t w3_desc,
    float alpha, char residual);
/* replaces include/ops/mlp/mlp.h:24 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetMLPWorkspaceSize(infiniopMLPDescriptor_t desc, uint64_t *size);
/* replaces include/ops/mlp/mlp.h:26-33 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopMLP(
    infiniopMLPDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *y, void const *x, void const *w12, void const *w3, void *stream);
/* replaces include/ops/mlp/mlp.h:35 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyMLPDescriptor(infiniopMLPDescriptor_t desc);

/* ======================================================================== *
 * Attention with a KV cache: k and v are written into their caches at row
 * `pos`, then out = softmax_causal(q @ K^T / sqrt(head_dim)) @ V over the
 * caches up to row pos + seq.  q [n_q_head, seq, head_dim]; k, v [n_kv_head,
 * seq, head_dim]; caches [n_kv_head, capacity, head_dim]; unit innermost
 * strides, the others free; out [seq, n_q_head, head_dim] contiguous.  A
 * composite of Rearrange, Matmul and CausalSoftmax; the caller provides the
 * workspace.
 * ======================================================================== */
typedef struct AttentionDescriptor {
    Device device;
} AttentionDescriptor;
typedef AttentionDescriptor *infiniopAttentionDescriptor_t;

/* replaces include/ops/attention/attention.h:15-23 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateAttentionDescriptor(
    infiniopHandle_t handle, infiniopAttentionDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t out_desc, infiniopTensorDescriptor_t q_desc,
    infiniopTensorDescriptor_t k_desc, infiniopTensorDescriptor_t v_desc,
    infiniopTensorDescriptor_t k_cache_desc, infiniopTensorDescriptor_t v_cache_desc, uint64_t pos);
/* replaces include/ops/attention/attention.h:25 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetAttentionWorkspaceSize(infiniopAttentionDescriptor_t desc, uint64_t *size);
/* replaces include/ops/attention/attention.h:27-36 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopAttention(
    infiniopAttentionDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *out, void const *q, void const *k, void const *v, void *k_cache, void *v_cache, void *stream);
/* replaces include/ops/attention/attention.h:38 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyAttentionDescriptor(infiniopAttentionDescriptor_t desc);

/* ======================================================================== *
 * RandomSample: one token index drawn from a vector of fp16 logits.  With
 * topp > 0 and topk > 1: the topk largest logits in descending order, their
 * probabilities f16(expf((x - max) / temperature) / sum over all logits), the
 * shortest prefix whose running sum reaches topp (plus one entry), and the
 * first entry of it whose running sum exceeds random_val times the prefix sum.
 * Otherwise: the first index of the maximum.  probs: 1-D F16 (reference) or
 * BF16 (extension: probabilities round to nearest even), unit stride;
 * result: U64, one element written.  Equal logits are ordered by ascending
 * index.  Any topk is served (it is clamped to the vocabulary size, as in the
 * reference).  The workspace (262 912 bytes, 0 below 4096 logits) lets the
 * sampling form spread its passes over the logits over the chip; a call
 * without it, or with less, is served by one workgroup, with the same result.
 * ======================================================================== */
typedef struct RandomSampleDescriptor {
    Device device;
} RandomSampleDescriptor;
typedef RandomSampleDescriptor *infiniopRandomSampleDescriptor_t;

/* replaces include/ops/random_sample/random_sample.h:14 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateRandomSampleDescriptor(
    infiniopHandle_t handle, infiniopRandomSampleDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t result, infiniopTensorDescriptor_t probs);
/* replaces include/ops/random_sample/random_sample.h:16 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetRandomSampleWorkspaceSize(infiniopRandomSampleDescriptor_t desc, uint64_t *size);
/* replaces include/ops/random_sample/random_sample.h:18-27 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopRandomSample(
    infiniopRandomSampleDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *result, void const *probs, float random_val, float topp, int topk, float temperature, void *stream);
/* no counterpart in the reference.  For callers that cannot allocate device
 * memory or hand over a workspace (code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc): infiniopRandomSample with what its
 * first launches leave for the drawing workgroup (candidate lists, or a count
 * per 16-bit key) kept in an array of 262 912 bytes
 * that the library holds on every GPU it runs on until the process ends.  The
 * call allocates nothing.  Same results as infiniopRandomSample with a
 * workspace.  Descriptors of more than 1 048 576 logits answer
 * STATUS_BAD_PARAM (and a line on stderr).  All calls on one GPU share the
 * array: calls that overlap in time on one GPU, on whatever streams, race. */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopRandomSampleNoAlloc(
    infiniopRandomSampleDescriptor_t desc, void *result, void const *probs,
    float random_val, float topp, int topk, float temperature, void *stream);
/* replaces include/ops/random_sample/random_sample.h:29 */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyRandomSampleDescriptor(infiniopRandomSampleDescriptor_t desc);

/* ======================================================================== *
 * AddRMSNorm (fused residual form; no counterpart in the reference, whose
 * callers issue infiniopAdd and then infiniopRMSNorm on the sum):
 *     c[i][j] = a[i][j] + b[i][j]                       rounded as Add rounds
 *     y[i][j] = c[i][j] * w[j] / sqrt(mean_j(c[i][j]^2) + epsilon)
 * in one pass over memory.  y and c are bit for bit what infiniopAdd followed
 * by infiniopRMSNorm of this library produce.  y, c, a, b: 2-D [n, d], one
 * element type (F16 or BF16), unit inner strides, free row strides; w: 1-D
 * [d], F16, BF16 or F32.  c may be a or b; y must not overlap the others.
 * ======================================================================== */
typedef struct AddRMSNormDescriptor {
    Device device;
} AddRMSNormDescriptor;
typedef AddRMSNormDescriptor *infiniopAddRMSNormDescriptor_t;

/* no counterpart in the reference; argument order follows include/ops/rms_norm/rms_norm.h:13-19
 * with the Add operands (include/ops/add/add.h:13-17) between y and w */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopCreateAddRMSNormDescriptor(
    infiniopHandle_t handle, infiniopAddRMSNormDescriptor_t *desc_ptr,
    infiniopTensorDescriptor_t y_desc, infiniopTensorDescriptor_t c_desc,
    infiniopTensorDescriptor_t a_desc, infiniopTensorDescriptor_t b_desc,
    infiniopTensorDescriptor_t w_desc, float epsilon);
/* no counterpart in the reference (pattern of include/ops/rms_norm/rms_norm.h:21) - always 0 bytes */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopGetAddRMSNormWorkspaceSize(infiniopAddRMSNormDescriptor_t desc, uint64_t *size);
/* no counterpart in the reference (pattern of include/ops/rms_norm/rms_norm.h:23-24) */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopAddRMSNorm(
    infiniopAddRMSNormDescriptor_t desc, void *workspace, uint64_t workspace_size,
    void *y, void *c, void const *a, void const *b, void const *w, void *stream);
/* no counterpart in the reference (pattern of include/ops/rms_norm/rms_norm.h:26) */
INFINIOP_C INFINIOP_EXPORT infiniopStatus_t infiniopDestroyAddRMSNormDescriptor(infiniopAddRMSNormDescriptor_t desc);

#endif /* INFINIOP_AMD_INFINIOP_H */
