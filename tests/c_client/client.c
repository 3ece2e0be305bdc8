/* A C11 client written the way a user of the reference writes one: it includes
 * the reference's header paths (reference include/infini_operators.h:1-19,
 * include/operators.h, include/ops/<op>/<op>.h) and uses every type and entry
 * point of the hot path.  tests/test_boundary.py compiles it with
 * `gcc -std=c11 -fsyntax-only -I include`; it is never linked or run. */
#include <stddef.h>

#include "infini_operators.h"
#include "operators.h"
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

int chain(void *stream, void *x, void *y, void *w, void *qkv, void *pos, void *sin_t, void *cos_t,
          void *gate_up, void *act, void *res) {
    infiniopHandle_t handle;
    if (infiniopCreateHandle(&handle, DevAmdGpu, 0) != STATUS_SUCCESS) return 1;

    uint64_t xs[2] = {8192, 8192}, ws[1] = {8192};
    infiniopTensorDescriptor_t xd, yd, wd;
    infiniopCreateTensorDescriptor(&xd, 2, xs, NULL, BF16);
    infiniopCreateTensorDescriptor(&yd, 2, xs, NULL, BF16);
    infiniopCreateTensorDescriptor(&wd, 1, ws, NULL, F32);
    infiniopRMSNormDescriptor_t rms;
    uint64_t bytes = 0;
    infiniopCreateRMSNormDescriptor(handle, &rms, yd, xd, wd, 1e-5f);
    infiniopGetRMSNormWorkspaceSize(rms, &bytes);
    infiniopRMSNorm(rms, NULL, bytes, y, x, w, stream);

    uint64_t ts[3] = {8192, 64, 128}, ps[1] = {8192}, tab[2] = {8192, 128};
    int64_t tstr[3] = {80 * 128, 128, 1};
    infiniopTensorDescriptor_t td, pd, sd, cd;
    infiniopCreateTensorDescriptor(&td, 3, ts, tstr, BF16);
    infiniopCreateTensorDescriptor(&pd, 1, ps, NULL, U64);
    infiniopCreateTensorDescriptor(&sd, 2, tab, NULL, F32);
    infiniopCreateTensorDescriptor(&cd, 2, tab, NULL, F32);
    infiniopRoPEDescriptor_t rope;
    infiniopCreateRoPEDescriptor(handle, &rope, td, pd, sd, cd);
    infiniopGetRoPEWorkspaceSize(rope, &bytes);
    infiniopRoPE(rope, NULL, bytes, qkv, pos, sin_t, cos_t, stream);

    uint64_t as[2] = {8192, 28672};
    int64_t fused[2] = {57344, 1};
    infiniopTensorDescriptor_t ad, bd, od;
    infiniopCreateTensorDescriptor(&ad, 2, as, fused, BF16);
    infiniopCreateTensorDescriptor(&bd, 2, as, fused, BF16);
    infiniopCreateTensorDescriptor(&od, 2, as, NULL, BF16);
    infiniopSwiGLUDescriptor_t swiglu;
    infiniopCreateSwiGLUDescriptor(handle, &swiglu, od, ad, bd);
    infiniopSwiGLU(swiglu, act, (char *) gate_up + 2 * 28672, gate_up, stream);

    infiniopAddDescriptor_t add;
    infiniopCreateAddDescriptor(handle, &add, yd, xd, yd);
    infiniopAdd(add, res, x, y, stream);

    /* a caller may read the device of a descriptor and nothing else */
    int dev = add->device == DevAmdGpu && rms->device == DevAmdGpu && swiglu->device == DevAmdGpu && handle->device == DevAmdGpu;

    infiniopDestroyAddDescriptor(add);
    infiniopDestroySwiGLUDescriptor(swiglu);
    infiniopDestroyRoPEDescriptor(rope);
    infiniopDestroyRMSNormDescriptor(rms);
    infiniopTensorDescriptor_t all[] = {xd, yd, wd, td, pd, sd, cd, ad, bd, od};
    for (unsigned i = 0; i < sizeof(all) / sizeof(all[0]); ++i) infiniopDestroyTensorDescriptor(all[i]);
    infiniopDestroyHandle(handle);
    return dev ? 0 : 2;
}
