/* A C11 client written the way a user of the reference writes one: it includes
 * the reference's header paths (reference include/infini_operators.h:1-19,
 * include/operators.h, include/export.h, include/ops/<op>/<op>.h), follows the
 * calling sequence the reference documents (reference README.md:10-40: handle,
 * descriptor, workspace size, compute, destroy) and uses every type and entry
 * point of the hot path.
 *
 * tests/test_boundary.py compiles it with `gcc -std=c11 -fsyntax-only`;
 * the library's build also links it against libinfiniop.so and the HIP
 * runtime (tests/c_client/client), and tests/test_gpu_c_client.py runs that
 * program on the GPU:
 *
 *     client <in.bin> <out.bin>
 *
 * in.bin : eight uint64 (element type 0 = fp16 / 1 = bf16, tokens, hidden
 *          width, heads rotated, heads in the fused buffer, head width, SwiGLU
 *          width, rows of the sin/cos tables), then x [tokens, hidden],
 *          w fp32 [hidden], qkv [tokens, buffer heads, head width],
 *          pos uint64 [tokens], sin and cos fp32 [rows, head width],
 *          gate_up [tokens, 2 * SwiGLU width].
 * out.bin: y = RMSNorm(x) * w, qkv with its first heads rotated in place,
 *          act = SwiGLU(up, gate) of the two halves of gate_up,
 *          res = x + y.
 * The program allocates its own device buffers, makes one call of each of the
 * four operators on one stream and prints a checksum of out.bin. */
#include <stddef.h>
#include <stdio.h>
#include <stdlib.h>

#include "infini_operators.h"
#include "operators.h"
#include "export.h"
#include "device.h"
#include "status.h"
#include "data_type.h"
#include "tensor.h"
#include "handle.h"
#include "ops/add/add.h"
#include "ops/rms_norm/rms_norm.h"
#include "ops/rotary_embedding/rotary_embedding.h"
#include "ops/swiglu/swiglu.h"
#include "ops/causal_softmax/causal_softmax.h"
#include "ops/rearrange/rearrange.h"
#include "ops/matmul/matmul.h"
#include "ops/mlp/mlp.h"
#include "ops/attention/attention.h"
#include "ops/random_sample/random_sample.h"
#include "handle/handle_export.h"
#include "tensor/tensor_descriptor.h"

_Static_assert(sizeof(DataLayout) == 4, "DataLayout is passed by value as a 32-bit image");
_Static_assert(sizeof(struct TensorDescriptor) == 32, "dt, ndim, shape, strides");
_Static_assert(DevAmdGpu == 4, "the device number appended to the reference's enum");
_Static_assert(STATUS_BAD_DEVICE == 8, "status codes 0..8");

/* a declaration of the caller's own, spelled with the reference's two macros */
__C __export int chain(const uint64_t *dims, void *stream, void *x, void *y, void *w, void *qkv, void *pos, void *sin_t,
                       void *cos_t, void *gate_up, void *act, void *res);

enum { ELEM, TOKENS, HIDDEN, HEADS, BUF_HEADS, HEAD_DIM, FFN, TABLE_ROWS, NDIMS };

#define TRY(call)                                                            \
    do {                                                                     \
        infiniopStatus_t st_ = (call);                                       \
        if (st_ != STATUS_SUCCESS) {                                         \
            fprintf(stderr, "%s -> status %d\n", #call, (int) st_);          \
            return 10 + (int) st_;                                           \
        }                                                                    \
    } while (0)

/* One pass of RMSNorm -> RoPE -> SwiGLU -> Add, all pointers device pointers.
 * At dims = {1, 8192, 8192, 64, 80, 128, 28672, 8192} this is the bf16 prefill
 * chain on 8192 tokens (RoPE on the q heads). */
int chain(const uint64_t *dims, void *stream, void *x, void *y, void *w, void *qkv, void *pos, void *sin_t, void *cos_t,
          void *gate_up, void *act, void *res) {
    const DataLayout dt = dims[ELEM] == 0 ? F16 : BF16;
    infiniopHandle_t handle;
    TRY(infiniopCreateHandle(&handle, DevAmdGpu, 0));

    uint64_t xs[2] = {dims[TOKENS], dims[HIDDEN]}, ws[1] = {dims[HIDDEN]};
    infiniopTensorDescriptor_t xd, yd, wd;
    TRY(infiniopCreateTensorDescriptor(&xd, 2, xs, NULL, dt));
    TRY(infiniopCreateTensorDescriptor(&yd, 2, xs, NULL, dt));
    TRY(infiniopCreateTensorDescriptor(&wd, 1, ws, NULL, F32));
    infiniopRMSNormDescriptor_t rms;
    uint64_t bytes = 0;
    TRY(infiniopCreateRMSNormDescriptor(handle, &rms, yd, xd, wd, 1e-5f));
    TRY(infiniopGetRMSNormWorkspaceSize(rms, &bytes));
    TRY(infiniopRMSNorm(rms, NULL, bytes, y, x, w, stream));

    uint64_t ts[3] = {dims[TOKENS], dims[HEADS], dims[HEAD_DIM]}, ps[1] = {dims[TOKENS]}, tab[2] = {dims[TABLE_ROWS], dims[HEAD_DIM]};
    int64_t tstr[3] = {(int64_t) (dims[BUF_HEADS] * dims[HEAD_DIM]), (int64_t) dims[HEAD_DIM], 1};
    infiniopTensorDescriptor_t td, pd, sd, cd;
    TRY(infiniopCreateTensorDescriptor(&td, 3, ts, tstr, dt));
    TRY(infiniopCreateTensorDescriptor(&pd, 1, ps, NULL, U64));
    TRY(infiniopCreateTensorDescriptor(&sd, 2, tab, NULL, F32));
    TRY(infiniopCreateTensorDescriptor(&cd, 2, tab, NULL, F32));
    infiniopRoPEDescriptor_t rope;
    TRY(infiniopCreateRoPEDescriptor(handle, &rope, td, pd, sd, cd));
    TRY(infiniopGetRoPEWorkspaceSize(rope, &bytes));
    TRY(infiniopRoPE(rope, NULL, bytes, qkv, pos, sin_t, cos_t, stream));

    uint64_t as[2] = {dims[TOKENS], dims[FFN]};
    int64_t fused[2] = {(int64_t) (2 * dims[FFN]), 1};
    infiniopTensorDescriptor_t ad, bd, od;
    TRY(infiniopCreateTensorDescriptor(&ad, 2, as, fused, dt));
    TRY(infiniopCreateTensorDescriptor(&bd, 2, as, fused, dt));
    TRY(infiniopCreateTensorDescriptor(&od, 2, as, NULL, dt));
    infiniopSwiGLUDescriptor_t swiglu;
    TRY(infiniopCreateSwiGLUDescriptor(handle, &swiglu, od, ad, bd));
    /* gate = columns [0, FFN), up = columns [FFN, 2 FFN) of one row of gate_up: act = up * gate * sigmoid(gate) */
    TRY(infiniopSwiGLU(swiglu, act, (char *) gate_up + 2 * dims[FFN], gate_up, stream));

    infiniopAddDescriptor_t add;
    TRY(infiniopCreateAddDescriptor(handle, &add, yd, xd, yd));
    TRY(infiniopAdd(add, res, x, y, stream));

    /* a caller may read the device of a descriptor and nothing else */
    int dev = add->device == DevAmdGpu && rms->device == DevAmdGpu && swiglu->device == DevAmdGpu && handle->device == DevAmdGpu;

    TRY(infiniopDestroyAddDescriptor(add));
    TRY(infiniopDestroySwiGLUDescriptor(swiglu));
    TRY(infiniopDestroyRoPEDescriptor(rope));
    TRY(infiniopDestroyRMSNormDescriptor(rms));
    infiniopTensorDescriptor_t all[] = {xd, yd, wd, td, pd, sd, cd, ad, bd, od};
    for (unsigned i = 0; i < sizeof(all) / sizeof(all[0]); ++i) TRY(infiniopDestroyTensorDescriptor(all[i]));
    TRY(infiniopDestroyHandle(handle));
    return dev ? 0 : 2;
}

/* ---- the program: only when built against the HIP runtime ----------------- */
#ifdef CLIENT_WITH_HIP_RUNTIME
#include <hip/hip_runtime_api.h>

#define HIP_TRY(call)                                                                  \
    do {                                                                               \
        hipError_t e_ = (call);                                                        \
        if (e_ != hipSuccess) {                                                        \
            fprintf(stderr, "%s -> %s\n", #call, hipGetErrorString(e_));               \
            return 3;                                                                  \
        }                                                                              \
    } while (0)

static int upload(FILE *in, void **dev, size_t bytes) {
    void *host = malloc(bytes ? bytes : 1);
    if (host == NULL || fread(host, 1, bytes, in) != bytes) {
        fprintf(stderr, "short input file\n");
        return 4;
    }
    HIP_TRY(hipMalloc(dev, bytes ? bytes : 16));
    HIP_TRY(hipMemcpy(*dev, host, bytes, hipMemcpyHostToDevice));
    free(host);
    return 0;
}

static int download(FILE *out, const void *dev, size_t bytes, uint64_t *sum) {
    unsigned char *host = malloc(bytes ? bytes : 1);
    if (host == NULL) return 4;
    HIP_TRY(hipMemcpy(host, dev, bytes, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < bytes; ++i) *sum = (*sum ^ host[i]) * 1099511628211ull; /* FNV-1a */
    if (fwrite(host, 1, bytes, out) != bytes) return 4;
    free(host);
    return 0;
}

int main(int argc, char **argv) {
    if (argc != 3) {
        fprintf(stderr, "usage: %s <in.bin> <out.bin>\n", argv[0]);
        return 1;
    }
    FILE *in = fopen(argv[1], "rb"), *out = fopen(argv[2], "wb");
    uint64_t dims[NDIMS];
    if (in == NULL || out == NULL || fread(dims, sizeof(uint64_t), NDIMS, in) != NDIMS) {
        fprintf(stderr, "cannot open the files or read the header\n");
        return 1;
    }
    const size_t es = 2, n = dims[TOKENS];
    const size_t x_bytes = n * dims[HIDDEN] * es, qkv_bytes = n * dims[BUF_HEADS] * dims[HEAD_DIM] * es;
    const size_t table_bytes = dims[TABLE_ROWS] * dims[HEAD_DIM] * sizeof(float), act_bytes = n * dims[FFN] * es;
    void *x, *w, *qkv, *pos, *sin_t, *cos_t, *gate_up, *y, *act, *res;
    int rc;
    if ((rc = upload(in, &x, x_bytes)) || (rc = upload(in, &w, dims[HIDDEN] * sizeof(float))) || (rc = upload(in, &qkv, qkv_bytes)) ||
        (rc = upload(in, &pos, n * sizeof(uint64_t))) || (rc = upload(in, &sin_t, table_bytes)) || (rc = upload(in, &cos_t, table_bytes)) ||
        (rc = upload(in, &gate_up, 2 * act_bytes))) {
        return rc;
    }
    HIP_TRY(hipMalloc(&y, x_bytes ? x_bytes : 16));
    HIP_TRY(hipMalloc(&act, act_bytes ? act_bytes : 16));
    HIP_TRY(hipMalloc(&res, x_bytes ? x_bytes : 16));
    hipStream_t stream;
    HIP_TRY(hipStreamCreate(&stream));

    rc = chain(dims, stream, x, y, w, qkv, pos, sin_t, cos_t, gate_up, act, res);
    if (rc != 0) return rc;
    HIP_TRY(hipStreamSynchronize(stream));

    uint64_t sum = 14695981039346656037ull;
    if ((rc = download(out, y, x_bytes, &sum)) || (rc = download(out, qkv, qkv_bytes, &sum)) || (rc = download(out, act, act_bytes, &sum)) ||
        (rc = download(out, res, x_bytes, &sum))) {
        return rc;
    }
    fclose(in);
    if (fclose(out) != 0) return 4;
    HIP_TRY(hipStreamDestroy(stream));
    void *all[] = {x, w, qkv, pos, sin_t, cos_t, gate_up, y, act, res};
    for (unsigned i = 0; i < sizeof(all) / sizeof(all[0]); ++i) HIP_TRY(hipFree(all[i]));
    printf("checksum %016llx\n", (unsigned long long) sum);
    return 0;
}
#endif
