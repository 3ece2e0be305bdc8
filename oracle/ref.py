"""numpy front end of the COMPILED REFERENCE CPU back end
(oracle/_ref/libinfiniop_ref.so, built by `make -C oracle ref` from the
reference checkout).  TEST INFRASTRUCTURE ONLY.

The library exists only where the reference sources were present at build
time; `available()` says whether it does.  Everything goes through the
reference's public C API with device 0 (CPU); the function signatures mirror
those of the `oracle` package so that tests can call either.
"""
import ctypes
import os

import numpy as np

from operators_amd import data_layout as dl
from operators_amd.liboperators import (
    bind_prototypes,
    infiniopAddDescriptor_t,
    infiniopCausalSoftmaxDescriptor_t,
    infiniopRearrangeDescriptor_t,
    infiniopRandomSampleDescriptor_t,
    infiniopHandle_t,
    infiniopRMSNormDescriptor_t,
    infiniopRoPEDescriptor_t,
    infiniopSwiGLUDescriptor_t,
    infiniopTensorDescriptor_t,
)

_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_DIR, "_ref", "libinfiniop_ref.so")
LAYOUT = {"f16": dl.F16, "bf16": dl.BF16, "f32": dl.F32, "f64": dl.F64, "u64": dl.U64, "i64": dl.I64, "u8": dl.U8}

_lib = None
_handle = None


def available():
    return os.path.isfile(LIB_PATH)


def lib():
    global _lib, _handle
    if _lib is None:
        L = bind_prototypes(ctypes.CDLL(LIB_PATH), extensions=False)
        # the reference also exports its scalar conversions as C++ symbols
        L._Z10f16_to_f32t.argtypes, L._Z10f16_to_f32t.restype = [ctypes.c_uint16], ctypes.c_float
        L._Z10f32_to_f16f.argtypes, L._Z10f32_to_f16f.restype = [ctypes.c_float], ctypes.c_uint16
        h = infiniopHandle_t()
        assert L.infiniopCreateHandle(ctypes.byref(h), 0, 0) == 0
        _lib, _handle = L, h
    return _lib


def handle():
    lib()
    return _handle


def f16_to_f32_scalar(code):
    return lib()._Z10f16_to_f32t(int(code))


def f32_to_f16_scalar(value):
    return lib()._Z10f32_to_f16f(ctypes.c_float(value))


def descriptor(dtype, shape, strides=None):
    n = len(shape)
    c_shape = (ctypes.c_uint64 * max(n, 1))(*shape)
    c_strides = None if strides is None else (ctypes.c_int64 * max(n, 1))(*strides)
    d = infiniopTensorDescriptor_t()
    assert lib().infiniopCreateTensorDescriptor(ctypes.byref(d), n, c_shape, c_strides, LAYOUT[dtype]) == 0
    return d


def _desc_of(array, dtype):
    item = array.dtype.itemsize
    return descriptor(dtype, array.shape, [s // item for s in array.strides])


def _free(*descs):
    for d in descs:
        lib().infiniopDestroyTensorDescriptor(d)


def add_status(c, a, b):
    """Create-time status for (dtype, shape, strides) triples."""
    dc, da, db = (descriptor(*s) for s in (c, a, b))
    desc = infiniopAddDescriptor_t()
    st = lib().infiniopCreateAddDescriptor(handle(), ctypes.byref(desc), dc, da, db)
    if st == 0:
        lib().infiniopDestroyAddDescriptor(desc)
    _free(dc, da, db)
    return st


def add(a, b, c_shape, dtype, c=None):
    if c is None:
        c = np.empty(c_shape, a.dtype)
    dc, da, db = _desc_of(c, dtype), _desc_of(a, dtype), _desc_of(b, dtype)
    desc = infiniopAddDescriptor_t()
    st = lib().infiniopCreateAddDescriptor(handle(), ctypes.byref(desc), dc, da, db)
    assert st == 0, st
    st = lib().infiniopAdd(desc, c.ctypes.data, a.ctypes.data, b.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyAddDescriptor(desc)
    _free(dc, da, db)
    return c


def rms_norm_status(y, x, w, eps=1e-5, run=False):
    """Create-time status; with run=True and a successful create, the status
    of the compute call on small zero buffers instead (the reference defers
    its dtype check to that stage)."""
    dy, dx, dw = (descriptor(*s) for s in (y, x, w))
    desc = infiniopRMSNormDescriptor_t()
    st = lib().infiniopCreateRMSNormDescriptor(handle(), ctypes.byref(desc), dy, dx, dw, eps)
    if st == 0:
        if run:
            n, d = y[1]
            span = max(1, (n - 1) * (y[2][0] if y[2] else d) + d)
            buf_y, buf_x, buf_w = np.zeros(span * 8, np.uint8), np.zeros(span * 8, np.uint8), np.zeros(d * 8 + 8, np.uint8)
            st = lib().infiniopRMSNorm(desc, None, 0, buf_y.ctypes.data, buf_x.ctypes.data, buf_w.ctypes.data, None)
        lib().infiniopDestroyRMSNormDescriptor(desc)
    _free(dy, dx, dw)
    return st


def rms_norm(x, w, eps, dtype, w_dtype, y=None):
    n, d = x.shape
    if y is None:
        y = np.empty((n, d), np.uint16)
    w = np.ascontiguousarray(w)
    dy, dx, dw = _desc_of(y, dtype), _desc_of(x, dtype), _desc_of(w, w_dtype)
    desc = infiniopRMSNormDescriptor_t()
    st = lib().infiniopCreateRMSNormDescriptor(handle(), ctypes.byref(desc), dy, dx, dw, eps)
    assert st == 0, st
    size = ctypes.c_uint64(99)
    assert lib().infiniopGetRMSNormWorkspaceSize(desc, ctypes.byref(size)) == 0 and size.value == 0
    st = lib().infiniopRMSNorm(desc, None, 0, y.ctypes.data, x.ctypes.data, w.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyRMSNormDescriptor(desc)
    _free(dy, dx, dw)
    return y


def rope_status(t, pos, sin_t, cos_t):
    ds = [descriptor(*s) for s in (t, pos, sin_t, cos_t)]
    desc = infiniopRoPEDescriptor_t()
    st = lib().infiniopCreateRoPEDescriptor(handle(), ctypes.byref(desc), *ds)
    if st == 0:
        lib().infiniopDestroyRoPEDescriptor(desc)
    _free(*ds)
    return st


def rope(t, pos, sin_t, cos_t, dtype):
    pos = np.ascontiguousarray(pos, dtype=np.uint64)
    sin_t = np.ascontiguousarray(sin_t, dtype=np.float32)
    cos_t = np.ascontiguousarray(cos_t, dtype=np.float32)
    ds = [_desc_of(t, dtype), _desc_of(pos, "u64"), _desc_of(sin_t, "f32"), _desc_of(cos_t, "f32")]
    desc = infiniopRoPEDescriptor_t()
    st = lib().infiniopCreateRoPEDescriptor(handle(), ctypes.byref(desc), *ds)
    assert st == 0, st
    size = ctypes.c_uint64(99)
    assert lib().infiniopGetRoPEWorkspaceSize(desc, ctypes.byref(size)) == 0 and size.value == 0
    st = lib().infiniopRoPE(desc, None, 0, t.ctypes.data, pos.ctypes.data, sin_t.ctypes.data, cos_t.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyRoPEDescriptor(desc)
    _free(*ds)
    return t


def swiglu_status(c, a, b):
    dc, da, db = (descriptor(*s) for s in (c, a, b))
    desc = infiniopSwiGLUDescriptor_t()
    st = lib().infiniopCreateSwiGLUDescriptor(handle(), ctypes.byref(desc), dc, da, db)
    if st == 0:
        lib().infiniopDestroySwiGLUDescriptor(desc)
    _free(dc, da, db)
    return st


def swiglu(a, b, dtype, c=None):
    n, di = a.shape
    if c is None:
        c = np.empty((n, di), np.uint16)
    dc, da, db = _desc_of(c, dtype), _desc_of(a, dtype), _desc_of(b, dtype)
    desc = infiniopSwiGLUDescriptor_t()
    st = lib().infiniopCreateSwiGLUDescriptor(handle(), ctypes.byref(desc), dc, da, db)
    assert st == 0, st
    st = lib().infiniopSwiGLU(desc, c.ctypes.data, a.ctypes.data, b.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroySwiGLUDescriptor(desc)
    _free(dc, da, db)
    return c


def causal_softmax_status(y):
    d = descriptor(*y)
    desc = infiniopCausalSoftmaxDescriptor_t()
    st = lib().infiniopCreateCausalSoftmaxDescriptor(handle(), ctypes.byref(desc), d)
    if st == 0:
        lib().infiniopDestroyCausalSoftmaxDescriptor(desc)
    _free(d)
    return st


def causal_softmax(y, dtype):
    d = _desc_of(y, dtype)
    desc = infiniopCausalSoftmaxDescriptor_t()
    st = lib().infiniopCreateCausalSoftmaxDescriptor(handle(), ctypes.byref(desc), d)
    assert st == 0, st
    size = ctypes.c_uint64(99)
    assert lib().infiniopGetCausalSoftmaxWorkspaceSize(desc, ctypes.byref(size)) == 0 and size.value == 0
    st = lib().infiniopCausalSoftmax(desc, None, 0, y.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyCausalSoftmaxDescriptor(desc)
    _free(d)
    return y


def rearrange_status(dst, src):
    dd, ds = descriptor(*dst), descriptor(*src)
    desc = infiniopRearrangeDescriptor_t()
    st = lib().infiniopCreateRearrangeDescriptor(handle(), ctypes.byref(desc), dd, ds)
    if st == 0:
        lib().infiniopDestroyRearrangeDescriptor(desc)
    _free(dd, ds)
    return st


def rearrange(dst, src, dtype):
    dd, ds = _desc_of(dst, dtype), _desc_of(src, dtype)
    desc = infiniopRearrangeDescriptor_t()
    st = lib().infiniopCreateRearrangeDescriptor(handle(), ctypes.byref(desc), dd, ds)
    assert st == 0, st
    st = lib().infiniopRearrange(desc, dst.ctypes.data, src.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyRearrangeDescriptor(desc)
    _free(dd, ds)
    return dst


def matmul(c, a, b, alpha, beta, dtype):
    """In place on c, through the reference's own CPU back end."""
    from operators_amd.liboperators import infiniopMatmulDescriptor_t

    dc, da, db = _desc_of(c, dtype), _desc_of(a, dtype), _desc_of(b, dtype)
    desc = infiniopMatmulDescriptor_t()
    st = lib().infiniopCreateMatmulDescriptor(handle(), ctypes.byref(desc), dc, alpha, da, db, beta)
    assert st == 0, st
    st = lib().infiniopMatmul(desc, None, 0, c.ctypes.data, a.ctypes.data, b.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyMatmulDescriptor(desc)
    _free(dc, da, db)
    return c


def matmul_status(c, a, b):
    """Create-time status for (dtype, shape, strides) triples."""
    from operators_amd.liboperators import infiniopMatmulDescriptor_t

    dc, da, db = (descriptor(*s) for s in (c, a, b))
    desc = infiniopMatmulDescriptor_t()
    st = lib().infiniopCreateMatmulDescriptor(handle(), ctypes.byref(desc), dc, 1.0, da, db, 0.0)
    if st == 0:
        lib().infiniopDestroyMatmulDescriptor(desc)
    _free(dc, da, db)
    return st


def mlp(y, x, w12, w3, alpha, residual, dtype):
    """In place on y, through the reference's own composite and CPU back end."""
    from operators_amd.liboperators import infiniopMLPDescriptor_t

    ds = [_desc_of(t, dtype) for t in (y, x, w12, w3)]
    desc = infiniopMLPDescriptor_t()
    st = lib().infiniopCreateMLPDescriptor(handle(), ctypes.byref(desc), *ds, alpha, ctypes.c_char(b"\x01" if residual else b"\x00"))
    assert st == 0, st
    size = ctypes.c_uint64(0)
    assert lib().infiniopGetMLPWorkspaceSize(desc, ctypes.byref(size)) == 0
    ws = np.zeros(max(1, size.value), np.uint8)
    st = lib().infiniopMLP(desc, ws.ctypes.data, size.value, y.ctypes.data, x.ctypes.data, w12.ctypes.data, w3.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyMLPDescriptor(desc)
    _free(*ds)
    return y


def attention(out, q, k, v, k_cache, v_cache, pos, dtype):
    """In place on out and the caches, through the reference's own composite and CPU back end."""
    from operators_amd.liboperators import infiniopAttentionDescriptor_t

    ds = [_desc_of(t, dtype) for t in (out, q, k, v, k_cache, v_cache)]
    desc = infiniopAttentionDescriptor_t()
    st = lib().infiniopCreateAttentionDescriptor(handle(), ctypes.byref(desc), *ds, pos)
    assert st == 0, st
    size = ctypes.c_uint64(0)
    assert lib().infiniopGetAttentionWorkspaceSize(desc, ctypes.byref(size)) == 0
    ws = np.zeros(max(1, size.value), np.uint8)
    st = lib().infiniopAttention(desc, ws.ctypes.data, size.value, out.ctypes.data, q.ctypes.data, k.ctypes.data, v.ctypes.data,
                                 k_cache.ctypes.data, v_cache.ctypes.data, None)
    assert st == 0, st
    lib().infiniopDestroyAttentionDescriptor(desc)
    _free(*ds)
    return out


def random_sample_status(result, probs):
    dr, dp = descriptor(*result), descriptor(*probs)
    desc = infiniopRandomSampleDescriptor_t()
    st = lib().infiniopCreateRandomSampleDescriptor(handle(), ctypes.byref(desc), dr, dp)
    if st == 0:
        lib().infiniopDestroyRandomSampleDescriptor(desc)
    _free(dr, dp)
    return st


def random_sample(probs, random_val, topp, topk, temperature):
    """Chosen index through the reference's own CPU back end, or None when it
    leaves the result unwritten."""
    probs = np.ascontiguousarray(probs, dtype=np.uint16)
    result = np.full(1, 0xFFFFFFFFFFFFFFFF, dtype=np.uint64)
    dr, dp = _desc_of(result, "u64"), _desc_of(probs, "f16")
    desc = infiniopRandomSampleDescriptor_t()
    st = lib().infiniopCreateRandomSampleDescriptor(handle(), ctypes.byref(desc), dr, dp)
    assert st == 0, st
    size = ctypes.c_uint64(0)
    assert lib().infiniopGetRandomSampleWorkspaceSize(desc, ctypes.byref(size)) == 0
    work = np.empty(max(int(size.value), 1), dtype=np.uint8)
    st = lib().infiniopRandomSample(desc, work.ctypes.data, size.value, result.ctypes.data, probs.ctypes.data,
                                    random_val, topp, topk, temperature, None)
    assert st == 0, st
    lib().infiniopDestroyRandomSampleDescriptor(desc)
    _free(dr, dp)
    return None if int(result[0]) == 0xFFFFFFFFFFFFFFFF else int(result[0])
