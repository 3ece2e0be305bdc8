"""numpy front end of the CPU oracle (oracle.c -> liboracle.so).

TEST INFRASTRUCTURE ONLY.  Import this from tests/, from the smoke check and
from the benchmark's CPU-baseline leg - never from the operators_amd package.

16-bit floating point data travels as numpy uint16 arrays holding the raw
codes; `dtype` arguments are the strings "f16", "bf16", "f32".  Arrays may be
strided views: strides are passed to the C code in elements.
"""
import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_DIR, "liboracle.so")


def _dt_code(packed, sign, size, mant, exp):
    return packed | (sign << 8) | (size << 9) | (mant << 16) | (exp << 24)


DT = {
    "f16": _dt_code(1, 1, 2, 10, 5),
    "bf16": _dt_code(1, 1, 2, 7, 8),
    "f32": _dt_code(1, 1, 4, 23, 8),
    "f64": _dt_code(1, 1, 8, 52, 11),
    "u64": _dt_code(1, 0, 8, 64, 0),
    "i64": _dt_code(1, 1, 8, 63, 0),
    "u8": _dt_code(1, 0, 1, 8, 0),
}
NP_DTYPE = {"f16": np.uint16, "bf16": np.uint16, "f32": np.float32}


class _Tensor(ctypes.Structure):
    _fields_ = [
        ("dt", ctypes.c_uint32),
        ("ndim", ctypes.c_uint64),
        ("shape", ctypes.POINTER(ctypes.c_uint64)),
        ("strides", ctypes.POINTER(ctypes.c_int64)),
    ]


def build(force=False):
    """Compile liboracle.so with gcc (a second or two)."""
    if force or not os.path.isfile(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(os.path.join(_DIR, "oracle.c")):
        subprocess.run(["make", "-s", "-C", _DIR, "-B", "liboracle.so"], check=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_LIB_PATH)
        vp, u64, i64, u32, f32 = ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int64, ctypes.c_uint32, ctypes.c_float
        tp = ctypes.POINTER(_Tensor)
        L.oracle_f16_to_f32.argtypes, L.oracle_f16_to_f32.restype = [ctypes.c_uint16], f32
        L.oracle_f32_to_f16.argtypes, L.oracle_f32_to_f16.restype = [f32], ctypes.c_uint16
        L.oracle_bf16_to_f32.argtypes, L.oracle_bf16_to_f32.restype = [ctypes.c_uint16], f32
        L.oracle_f32_to_bf16.argtypes, L.oracle_f32_to_bf16.restype = [f32], ctypes.c_uint16
        for name in ("oracle_f16_to_f32_array", "oracle_f32_to_f16_array", "oracle_bf16_to_f32_array", "oracle_f32_to_bf16_array"):
            getattr(L, name).argtypes = [vp, vp, u64]
            getattr(L, name).restype = None
        L.oracle_add_check.argtypes, L.oracle_add_check.restype = [tp, tp, tp, ctypes.c_int], ctypes.c_int
        L.oracle_add.argtypes, L.oracle_add.restype = [tp, tp, tp, vp, vp, vp], ctypes.c_int
        L.oracle_rms_norm_check.argtypes, L.oracle_rms_norm_check.restype = [tp, tp, tp], ctypes.c_int
        L.oracle_rms_norm.argtypes = [u32, u32, u64, u64, i64, i64, f32, vp, vp, vp]
        L.oracle_rms_norm.restype = ctypes.c_int
        L.oracle_rope_check.argtypes, L.oracle_rope_check.restype = [tp, tp, tp, tp, ctypes.c_int], ctypes.c_int
        L.oracle_rope.argtypes = [u32, u64, u64, u64, i64, i64, vp, vp, vp, vp]
        L.oracle_rope.restype = ctypes.c_int
        L.oracle_swiglu_check.argtypes, L.oracle_swiglu_check.restype = [tp, tp, tp, ctypes.c_int], ctypes.c_int
        L.oracle_swiglu.argtypes = [u32, u64, u64, i64, i64, i64, vp, vp, vp]
        L.oracle_swiglu.restype = ctypes.c_int
        L.oracle_causal_softmax_check.argtypes, L.oracle_causal_softmax_check.restype = [tp, ctypes.c_int, ctypes.c_int], ctypes.c_int
        L.oracle_causal_softmax.argtypes = [u32, u64, u64, u64, i64, i64, i64, vp]
        L.oracle_causal_softmax.restype = ctypes.c_int
        L.oracle_rearrange_check.argtypes, L.oracle_rearrange_check.restype = [tp, tp], ctypes.c_int
        L.oracle_rearrange.argtypes = [u32, u64, vp, vp, vp, vp, vp]
        L.oracle_rearrange.restype = ctypes.c_int
        L.oracle_random_sample_check.argtypes, L.oracle_random_sample_check.restype = [tp, tp, ctypes.c_int], ctypes.c_int
        L.oracle_random_sample.argtypes = [u32, vp, vp, ctypes.c_int, f32, f32, ctypes.c_int, f32, vp, vp]
        L.oracle_random_sample.restype = ctypes.c_int
        _lib = L
    return _lib


class Spec:
    """Shape/strides/dtype of a tensor as the create-time checks see it."""

    def __init__(self, dtype, shape, strides=None):
        self.dtype = dtype
        self.shape = tuple(int(s) for s in shape)
        if strides is None:
            strides, run = [], 1
            for n in reversed(self.shape):
                strides.append(run)
                run *= n
            strides.reverse()
        self.strides = tuple(int(s) for s in strides)
        n = len(self.shape)
        self._shape = (ctypes.c_uint64 * max(n, 1))(*self.shape)
        self._strides = (ctypes.c_int64 * max(n, 1))(*self.strides)
        self.c = _Tensor(DT[dtype], n, self._shape, self._strides)

    @staticmethod
    def of(array, dtype):
        item = array.dtype.itemsize
        return Spec(dtype, array.shape, [s // item for s in array.strides])

    def ref(self):
        return ctypes.byref(self.c)


def _ptr(a):
    return a.ctypes.data


# ---- conversions ---------------------------------------------------------------
def f16_to_f32(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint16)
    out = np.empty(codes.shape, np.float32)
    lib().oracle_f16_to_f32_array(_ptr(out), _ptr(codes), codes.size)
    return out


def f32_to_f16(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, np.uint16)
    lib().oracle_f32_to_f16_array(_ptr(out), _ptr(values), values.size)
    return out


def bf16_to_f32(codes):
    codes = np.ascontiguousarray(codes, dtype=np.uint16)
    out = np.empty(codes.shape, np.float32)
    lib().oracle_bf16_to_f32_array(_ptr(out), _ptr(codes), codes.size)
    return out


def f32_to_bf16(values):
    values = np.ascontiguousarray(values, dtype=np.float32)
    out = np.empty(values.shape, np.uint16)
    lib().oracle_f32_to_bf16_array(_ptr(out), _ptr(values), values.size)
    return out


def encode(values, dtype):
    """fp32 values -> storage array of `dtype` using the oracle's own narrowing."""
    if dtype == "f32":
        return np.ascontiguousarray(values, dtype=np.float32)
    return f32_to_f16(values) if dtype == "f16" else f32_to_bf16(values)


def decode(codes, dtype):
    if dtype == "f32":
        return np.asarray(codes, dtype=np.float32)
    return f16_to_f32(codes) if dtype == "f16" else bf16_to_f32(codes)


# ---- operators -------------------------------------------------------------------
def add_check(c, a, b, allow_bf16=False):
    return lib().oracle_add_check(c.ref(), a.ref(), b.ref(), int(allow_bf16))


def add(a, b, c_shape, dtype):
    """c = a + b with broadcasting; a, b are numpy arrays of the storage type."""
    c = np.empty(c_shape, NP_DTYPE[dtype])
    sc, sa, sb = Spec.of(c, dtype), Spec.of(a, dtype), Spec.of(b, dtype)
    st = lib().oracle_add(sc.ref(), sa.ref(), sb.ref(), _ptr(c), _ptr(a), _ptr(b))
    if st != 0:
        raise RuntimeError(f"oracle_add status {st}")
    return c


def add_into(c, a, b, dtype):
    """As `add`, writing into an existing contiguous array (which may be a or b)."""
    sc, sa, sb = Spec.of(c, dtype), Spec.of(a, dtype), Spec.of(b, dtype)
    st = lib().oracle_add(sc.ref(), sa.ref(), sb.ref(), _ptr(c), _ptr(a), _ptr(b))
    if st != 0:
        raise RuntimeError(f"oracle_add status {st}")
    return c


def rms_norm_check(y, x, w):
    return lib().oracle_rms_norm_check(y.ref(), x.ref(), w.ref())


def rms_norm(x, w, eps, dtype, w_dtype, y=None):
    """x: [n, d] storage array (rows may be strided); returns y (contiguous unless given)."""
    n, d = x.shape
    if y is None:
        y = np.empty((n, d), np.uint16)
    assert x.strides[1] == x.itemsize and y.strides[1] == y.itemsize
    w = np.ascontiguousarray(w)
    st = lib().oracle_rms_norm(DT[dtype], DT[w_dtype], n, d, y.strides[0] // 2, x.strides[0] // 2,
                               ctypes.c_float(eps), _ptr(y), _ptr(x), _ptr(w))
    if st != 0:
        raise RuntimeError(f"oracle_rms_norm status {st}")
    return y


def add_rms_norm(a, b, w, eps, dtype, w_dtype):
    """The reference's two calls behind the fused operator: c = a + b
    (src/ops/add/cpu/add_cpu.cc:72-89), then y = RMSNorm(c) * w
    (src/ops/rms_norm/cpu/rms_norm_cpu.cc:46-86).  a, b: contiguous [n, d]
    storage arrays.  Returns (c, y)."""
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    c = add(a, b, a.shape, dtype)
    return c, rms_norm(c, w, eps, dtype, w_dtype)


def _matrix(x):
    """(batch, batch stride, row stride, col stride) of a 2-D or 3-D storage array, in elements."""
    st = [s // x.itemsize for s in x.strides]
    if x.ndim == 2:
        return 1, 0, st[0], st[1]
    assert x.ndim == 3
    return x.shape[0], (0 if x.shape[0] == 1 else st[0]), st[1], st[2]


def matmul(c, a, b, alpha, beta, dtype):
    """In place on c: c = alpha * a @ b + beta * c (src/ops/matmul/cpu/matmul_cpu.cc:47-82).
    2-D or batched 3-D storage arrays with any strides; a and b may have one
    matrix for all of c's batches."""
    cb, csb, crs, ccs = _matrix(c)
    ab, asb, ars, acs = _matrix(a)
    bb, bsb, brs, bcs = _matrix(b)
    m, n, k = c.shape[-2], c.shape[-1], a.shape[-1]
    assert a.shape[-2] == m and b.shape[-1] == n and b.shape[-2] == k and ab in (1, cb) and bb in (1, cb)
    f = lib().oracle_matmul
    f.argtypes = [ctypes.c_uint32] + [ctypes.c_uint64] * 4 + [ctypes.c_int64] * 9 + [ctypes.c_float] * 2 + [ctypes.c_void_p] * 3
    st = f(DT[dtype], cb, m, n, k, csb, crs, ccs, asb if ab > 1 else 0, ars, acs, bsb if bb > 1 else 0, brs, bcs,
           alpha, beta, _ptr(c), _ptr(a), _ptr(b))
    if st != 0:
        raise RuntimeError(f"oracle_matmul status {st}")
    return c


def mlp(y, x, w12, w3, alpha, residual, dtype):
    """In place on y: the reference's composite (src/ops/mlp/operator.cc:22-122) -
    gate_up = x @ w12 rounded to the storage type, hidden = swiglu(up = second
    half, gate = first half), y = alpha * hidden @ w3 (+ y when residual)."""
    n, two_di = x.shape[0], w12.shape[1]
    di = two_di // 2
    gate_up = np.zeros((n, two_di), NP_DTYPE[dtype])
    matmul(gate_up, x, w12, 1.0, 0.0, dtype)
    hidden = swiglu(gate_up[:, di:], gate_up[:, :di], dtype)
    return matmul(y, hidden, w3, alpha, 1.0 if residual else 0.0, dtype)


def attention(out, q, k, v, k_cache, v_cache, pos, dtype):
    """In place on out and on the caches: the reference's composite
    (src/ops/attention/operator.cc:31-320) - rearrange k, v into the caches at
    row pos; scores = q @ K^T / sqrt(head_dim) per K/V head over its group of
    query heads, rounded to the storage type; causal softmax in place; scores
    @ V, rounded; head-major result transposed into out [seq, heads, dim]."""
    heads, seq, hd = q.shape
    kv_heads, total = k.shape[0], pos + seq
    group = heads // kv_heads
    rearrange(k_cache[:, pos:total, :], k)
    rearrange(v_cache[:, pos:total, :], v)
    packed = np.zeros((heads, seq, hd), NP_DTYPE[dtype])
    rearrange(packed, q)
    scores = np.zeros((kv_heads, group * seq, total), NP_DTYPE[dtype])
    matmul(scores, packed.reshape(kv_heads, group * seq, hd), k_cache[:, :total, :].transpose(0, 2, 1), 1 / np.sqrt(hd), 0.0, dtype)
    causal_softmax(scores.reshape(heads, seq, total), dtype)
    result = np.zeros((kv_heads, group * seq, hd), NP_DTYPE[dtype])
    matmul(result, scores, v_cache[:, :total, :], 1.0, 0.0, dtype)
    rearrange(out, result.reshape(heads, seq, hd).transpose(1, 0, 2))
    return out


def rope_check(t, pos, sin_t, cos_t, allow_bf16=False):
    return lib().oracle_rope_check(t.ref(), pos.ref(), sin_t.ref(), cos_t.ref(), int(allow_bf16))


def rope(t, pos, sin_t, cos_t, dtype):
    """In-place on t: [tokens, heads, head_dim] storage array, any token/head strides."""
    nt, nh, dh = t.shape
    assert t.strides[2] == 2
    pos = np.ascontiguousarray(pos, dtype=np.uint64)
    sin_t = np.ascontiguousarray(sin_t, dtype=np.float32)
    cos_t = np.ascontiguousarray(cos_t, dtype=np.float32)
    st = lib().oracle_rope(DT[dtype], nt, nh, dh, t.strides[0] // 2, t.strides[1] // 2,
                           _ptr(t), _ptr(pos), _ptr(sin_t), _ptr(cos_t))
    if st != 0:
        raise RuntimeError(f"oracle_rope status {st}")
    return t


def swiglu_check(c, a, b, allow_bf16=False):
    return lib().oracle_swiglu_check(c.ref(), a.ref(), b.ref(), int(allow_bf16))


def swiglu(a, b, dtype, c=None):
    """c = a * b * sigmoid(b); a, b: [n, di] storage arrays, rows may be strided."""
    n, di = a.shape
    if c is None:
        c = np.empty((n, di), np.uint16)
    assert a.strides[1] == 2 and b.strides[1] == 2 and c.strides[1] == 2
    st = lib().oracle_swiglu(DT[dtype], n, di, c.strides[0] // 2, a.strides[0] // 2, b.strides[0] // 2,
                             _ptr(c), _ptr(a), _ptr(b))
    if st != 0:
        raise RuntimeError(f"oracle_swiglu status {st}")
    return c


def causal_softmax_check(y, allow_bf16=False, unit_inner=False):
    return lib().oracle_causal_softmax_check(y.ref(), int(allow_bf16), int(unit_inner))


def causal_softmax(y, dtype):
    """In place on y: [seq, total] or [batch, seq, total] storage array, any strides."""
    assert y.ndim in (2, 3)
    st = [s // 2 for s in y.strides]
    batch, sb = (y.shape[0], st[0]) if y.ndim == 3 else (1, 0)
    rc = lib().oracle_causal_softmax(DT[dtype], batch, y.shape[-2], y.shape[-1], sb, st[-2], st[-1], _ptr(y))
    if rc != 0:
        raise RuntimeError(f"oracle_causal_softmax status {rc}")
    return y


def rearrange_check(dst, src):
    return lib().oracle_rearrange_check(dst.ref(), src.ref())


def rearrange(dst, src):
    """dst[...] = src[...]: numpy arrays (views) of equal shape and dtype, unit innermost strides."""
    assert dst.shape == src.shape and dst.dtype == src.dtype
    n, item = dst.ndim, dst.dtype.itemsize
    shape = (ctypes.c_uint64 * n)(*dst.shape)
    sd = (ctypes.c_int64 * n)(*[s // item for s in dst.strides])
    ss = (ctypes.c_int64 * n)(*[s // item for s in src.strides])
    rc = lib().oracle_rearrange(item, n, shape, sd, ss, _ptr(dst), _ptr(src))
    if rc != 0:
        raise RuntimeError(f"oracle_rearrange status {rc}")
    return dst


def random_sample_check(result, probs, allow_bf16=False):
    return lib().oracle_random_sample_check(result.ref(), probs.ref(), int(allow_bf16))


def random_sample(probs, random_val, topp, topk, temperature, dtype="f16"):
    """probs: 1-D contiguous array of fp16 (or, as an extension, bf16) codes.  Returns the chosen index, or
    None when the reference's CPU path would leave the result unwritten."""
    probs = np.ascontiguousarray(probs, dtype=np.uint16)
    voc = probs.shape[0]
    result = np.full(1, 0xFFFFFFFFFFFFFFFF, dtype=np.uint64)
    logits = np.empty(voc, dtype=np.uint16)
    order = np.empty(voc, dtype=np.uint64)
    wrote = lib().oracle_random_sample(DT[dtype], _ptr(result), _ptr(probs), voc, random_val, topp, topk, temperature,
                                       _ptr(logits), _ptr(order))
    if wrote < 0:
        raise RuntimeError(f"oracle_random_sample status {-wrote}")
    return int(result[0]) if wrote else None
