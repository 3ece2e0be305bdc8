"""Write the golden fixtures in this directory from the COMPILED REFERENCE.

Run where a checkout of the reference is present:

    make -C oracle ref && python tests/golden/make_golden.py

Every expected output below is produced by the reference's own CPU back end
(oracle/_ref/libinfiniop_ref.so, compiled unmodified from the reference's
sources) through its public C API; inputs come from numpy's PCG64 generator
with fixed seeds.  The reference holds no fixtures of its own (its tests draw
unseeded random inputs), so these vectors are what pins the oracle and the GPU
kernels on machines that do not have the reference.  The files are data only:
inputs, expected outputs and expected status codes.
"""
import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import ref  # noqa: E402


def f16(values):
    """fp32 samples -> fp16 codes by numpy's round-to-nearest (input preparation only)."""
    return np.asarray(values, dtype=np.float32).astype(np.float16).view(np.uint16)


def conversions(rng):
    # fp32 -> fp16: hand-picked boundary values, then random bit patterns
    # spread over every exponent the conversion distinguishes.
    special = np.array([
        0.0, -0.0, 1.0, -1.0, 1.0 + 2.0 ** -11, 1.0 + 3 * 2.0 ** -11, 1.0 + 2.0 ** -10 - 2.0 ** -20,
        65504.0, 65519.996, 65520.0, 65535.996, 65536.0, 70000.0, 131008.0, 131072.0, 1e6, 1e10, 3.0e38,
        -65536.0, -131072.0, -1e10,
        2.0 ** -14, 2.0 ** -14 - 2.0 ** -30, 2.0 ** -15, 2.0 ** -24, 2.0 ** -24 - 2.0 ** -40, 2.0 ** -25, 1e-30,
        np.inf, -np.inf,
    ], dtype=np.float32)
    nan_bits = np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF, 0x7FA00000], dtype=np.uint32)
    expo = rng.integers(127 - 40, 127 + 40, size=40000, dtype=np.uint32)
    rand_bits = (rng.integers(0, 2, size=40000, dtype=np.uint32) << 31) | (expo << 23) | rng.integers(0, 1 << 23, size=40000, dtype=np.uint32)
    bits = np.concatenate([special.view(np.uint32), nan_bits, rand_bits]).astype(np.uint32)
    vals = bits.view(np.float32)
    out = np.array([ref.f32_to_f16_scalar(v) for v in vals], dtype=np.uint16)
    # fp16 -> fp32 for every code
    codes = np.arange(65536, dtype=np.uint16)
    wide = np.array([ref.f16_to_f32_scalar(int(c)) for c in codes], dtype=np.float32)
    return {"f32_bits": bits, "f16_codes": out, "all_f16_as_f32_bits": wide.view(np.uint32)}


ADD_CASES = [
    # (c_shape, a_shape, b_shape): the reference's own test table (operatorspy/tests/add.py:114-130),
    # the two huge shapes reduced, plus the leading-dimension broadcast of the residual-add use
    ((1, 3), (1, 3), (1, 3)),
    ((), (), ()),
    ((3, 3), (3, 3), (3, 3)),
    ((2, 20, 3), (2, 1, 3), (2, 20, 3)),
    ((8, 20, 512), (8, 20, 512), (8, 20, 512)),
    ((4, 8, 14, 14), (4, 8, 14, 1), (4, 8, 14, 14)),
    ((4, 8, 14, 16), (4, 8, 14, 16), (4, 8, 14, 16)),
    ((2, 4, 3), (2, 1, 3), (4, 3)),
    ((2, 3, 4, 5), (2, 3, 4, 5), (5,)),
    ((3, 2, 4, 5), (4, 5), (3, 2, 1, 1)),
    ((64, 256), (64, 256), (256,)),
    ((5, 16, 24), (5, 1, 24), (16, 1)),
]


def add_vectors(rng):
    out = {}
    for i, (cs, as_, bs) in enumerate(ADD_CASES):
        for dt in ("f16", "f32"):
            a = rng.standard_normal(as_).astype(np.float32)
            b = rng.standard_normal(bs).astype(np.float32)
            if dt == "f16":
                a, b = f16(a), f16(b)
            a, b = np.array(a).reshape(as_), np.array(b).reshape(bs)  # reshape keeps rank 0 (ascontiguousarray would not)
            c = ref.add(a, b, cs, dt)
            out[f"add{i}_{dt}_a"], out[f"add{i}_{dt}_b"], out[f"add{i}_{dt}_c"] = a, b, c
    # every fp16 code plus +0: the identity except for -0 and NaNs
    codes = np.arange(65536, dtype=np.uint16)
    out["add_all_codes_plus_zero"] = ref.add(codes, np.zeros(65536, np.uint16), (65536,), "f16")
    # a 256x256 block of the full fp16 x fp16 addition table, chosen to include
    # the largest finite values (overflow quirk), subnormals, infinities and NaNs
    rows = np.concatenate([np.arange(0x7B80, 0x7C40), np.arange(0x0000, 0x0040), np.arange(0xFBC0, 0xFC40), rng.integers(0, 65536, 64)]).astype(np.uint16)
    cols = np.concatenate([np.arange(0x7BC0, 0x7C40), np.arange(0x83E0, 0x8420), np.arange(0x3BE0, 0x3C20), rng.integers(0, 65536, 0)]).astype(np.uint16)
    table = ref.add(np.ascontiguousarray(rows.reshape(-1, 1)), cols, (rows.size, cols.size), "f16")
    out["add_table_rows"], out["add_table_cols"], out["add_table_c"] = rows, cols, table
    return out


def rms_norm_vectors(rng):
    out = {}
    # the benchmark's first configuration: x ~ N(0,1) [16, 2048], w ~ U(0.5, 1.5), eps 1e-5
    x = f16(rng.standard_normal((16, 2048)))
    w16 = f16(rng.uniform(0.5, 1.5, 2048))
    w32 = rng.uniform(0.5, 1.5, 2048).astype(np.float32)
    out["rms0_x"], out["rms0_w16"], out["rms0_w32"] = x, w16, w32
    out["rms0_y_w16"] = ref.rms_norm(x, w16, 1e-5, "f16", "f16")
    out["rms0_y_w32"] = ref.rms_norm(x, w32, 1e-5, "f16", "f32")
    # odd sizes, large and tiny magnitudes
    for i, (n, d, scale) in enumerate([(3, 7, 1.0), (5, 1000, 30.0), (4, 8200, 1e-3), (2, 64, 200.0)], start=1):
        x = f16(rng.standard_normal((n, d)) * scale)
        w = rng.uniform(-2, 2, d).astype(np.float32)
        out[f"rms{i}_x"], out[f"rms{i}_w32"] = x, w
        out[f"rms{i}_y_w32"] = ref.rms_norm(x, w, 1e-6, "f16", "f32")
    return out


def table(rows, dh, theta):
    pos = np.arange(rows, dtype=np.float32)
    freqs = (1.0 / (np.float32(theta) ** (np.arange(0, dh, 2, dtype=np.float32) / np.float32(dh)))).astype(np.float32)
    ang = np.outer(pos, np.repeat(freqs, 2)).astype(np.float32)
    return np.sin(ang).astype(np.float32), np.cos(ang).astype(np.float32)


ROPE_CASES = [
    # (shape, strides or None, table rows): shapes of operatorspy/tests/rotary_embedding.py:169-178
    ((1, 32, 128), None, 2), ((1, 32, 64), None, 2), ((4, 1, 32), None, 8),
    ((3, 32, 128), (8000, 200, 1), 6),
    ((7, 5, 6), None, 40), ((16, 8, 128), (3 * 8 * 128, 128, 1), 300),
]


def rope_vectors(rng):
    out = {}
    for i, (shape, strides, rows) in enumerate(ROPE_CASES):
        nt, nh, dh = shape
        vals = f16(rng.standard_normal(shape))
        if strides is None:
            t = vals.copy()
        else:
            span = 1 + sum((n - 1) * s for n, s in zip(shape, strides))
            buf = f16(rng.standard_normal(span))  # the gaps hold data that must survive
            t = np.lib.stride_tricks.as_strided(buf, shape, [s * 2 for s in strides])
            t[...] = vals
            out[f"rope{i}_buf_in"] = buf.copy()
        sin_t, cos_t = table(rows, dh, 1e4)
        if i >= 4:  # tables whose paired entries differ: all four reads per pair matter
            sin_t = rng.uniform(-1, 1, sin_t.shape).astype(np.float32)
            cos_t = rng.uniform(-1, 1, cos_t.shape).astype(np.float32)
        pos = (np.arange(nt) if i < 4 else rng.integers(0, rows, nt)).astype(np.uint64)
        out[f"rope{i}_t_in"] = np.array(t)  # a copy: the call below rotates t in place
        out[f"rope{i}_pos"], out[f"rope{i}_sin"], out[f"rope{i}_cos"] = pos, sin_t, cos_t
        ref.rope(t, pos, sin_t, cos_t, "f16")
        out[f"rope{i}_t_out"] = np.array(t)
        if strides is not None:
            out[f"rope{i}_buf_out"] = buf.copy()
    return out


SWIGLU_CASES = [
    # (shape, a_stride, b_stride, c_stride): operatorspy/tests/swiglu.py:240-246 plus a fused gate/up layout
    ((13, 4), None, None, None), ((13, 4), 10, 10, 10),
    ((16, 5632), None, None, None), ((16, 5632), 13312, 13312, 13312),
    ((6, 1000), 2000, 2000, 1000),
]


def swiglu_vectors(rng):
    out = {}
    for i, (shape, sa, sb, sc) in enumerate(SWIGLU_CASES):
        n, di = shape

        def strided(stride, values):
            if stride is None:
                return values.copy()
            buf = np.zeros((n - 1) * stride + di, np.uint16)
            v = np.lib.stride_tricks.as_strided(buf, shape, (stride * 2, 2))
            v[...] = values
            return v

        scale = 4.0 if i % 2 == 0 else 1.0
        a = strided(sa, f16(rng.standard_normal(shape) * scale))
        b = strided(sb, f16(rng.standard_normal(shape) * scale))
        if i == 4:  # gate = first half, up = second half of one fused row
            fused = f16(rng.standard_normal((n, 2 * di)))
            b, a = fused[:, :di], fused[:, di:]
        c = strided(sc, np.zeros(shape, np.uint16))
        ref.swiglu(a, b, "f16", c=c)
        out[f"swiglu{i}_a"], out[f"swiglu{i}_b"], out[f"swiglu{i}_c"] = (np.array(v) for v in (a, b, c))
    # saturation: large |b| and b = 0
    b = f16(np.array([[0.0, -0.0, 20.0, -20.0, 60.0, -60.0, 11.09, -17.3, 1e-4, -1e-4, 65504.0, -65504.0]]))
    a = f16(np.full(b.shape, 1.5))
    out["swiglu_sat_a"], out["swiglu_sat_b"], out["swiglu_sat_c"] = a, b, ref.swiglu(a, b, "f16")
    return out


CAUSAL_CASES = [
    # (shape, strides or None): the reference's test shape (operatorspy/tests/causal_softmax.py:111-115), smaller, plus odd ones
    ((4, 20, 512), None), ((4, 20, 512), (20480, 512, 1)), ((7, 13), None), ((5, 5), None), ((1, 40), None),
    ((3, 16, 16), None), ((2, 9, 1000), (9 * 1024, 1024, 1)),
]


def causal_softmax_vectors(rng):
    out = {}
    for i, (shape, strides) in enumerate(CAUSAL_CASES):
        vals = f16(rng.standard_normal(shape) * (3.0 if i % 2 else 1.0))
        if strides is None:
            y = vals.copy()
        else:
            span = 1 + sum((n - 1) * s for n, s in zip(shape, strides))
            buf = f16(rng.standard_normal(span))
            y = np.lib.stride_tricks.as_strided(buf, shape, [s * 2 for s in strides])
            y[...] = vals
        out[f"causal{i}_in"] = np.array(y)
        ref.causal_softmax(y, "f16")
        out[f"causal{i}_out"] = np.array(y)
    return out


REARRANGE_CASES = [
    # (dtype, shape, src_strides or None, dst_strides or None): operatorspy/tests/rearrange.py:108-116, then more ranks and element sizes
    ("f16", (2, 4, 32), None, (256, 64, 1)),
    ("f16", (32, 6, 64), (64, 2560, 1), None),
    ("f16", (4, 6, 64), (64, 2560, 1), (16384, 64, 1)),  # the reference uses 131072; shortened to keep the fixture small
    ("f16", (1, 32, 64), (2048, 64, 1), (2048, 64, 1)),
    ("f16", (32, 1, 64), (64, 2560, 1), (64, 64, 1)),
    ("f16", (4, 1, 64), (64, 2560, 1), (64, 11264, 1)),
    ("f16", (100,), None, None),
    ("f32", (7, 33), (40, 1), (35, 1)),
    ("u8", (5, 3, 13), (64, 16, 1), (45, 15, 1)),
    ("f16", (2, 3, 4, 8), (3 * 64, 64, 10, 1), (3 * 40, 40, 9, 1)),
    ("f64", (3, 2, 5), (40, 8, 1), None),
]
NP_OF = {"f16": np.uint16, "f32": np.float32, "u8": np.uint8, "f64": np.float64}


def contiguous_strides(shape):
    out, run = [], 1
    for n in reversed(shape):
        out.append(run)
        run *= n
    return tuple(reversed(out))


def rearrange_vectors(rng):
    out = {}
    for i, (dt, shape, ss, sd) in enumerate(REARRANGE_CASES):
        ss, sd = ss or contiguous_strides(shape), sd or contiguous_strides(shape)
        item = np.dtype(NP_OF[dt]).itemsize
        span = lambda st: 1 + sum((n - 1) * s for n, s in zip(shape, st))  # noqa: E731
        src_buf = rng.integers(0, 200, span(ss) * item, dtype=np.uint8).view(NP_OF[dt])
        dst_buf = rng.integers(0, 200, span(sd) * item, dtype=np.uint8).view(NP_OF[dt])
        out[f"rearrange{i}_src"], out[f"rearrange{i}_dst_before"] = src_buf.copy(), dst_buf.copy()
        src = np.lib.stride_tricks.as_strided(src_buf, shape, [s * item for s in ss])
        dst = np.lib.stride_tricks.as_strided(dst_buf, shape, [s * item for s in sd])
        ref.rearrange(dst, src, dt)
        out[f"rearrange{i}_dst_after"] = dst_buf.copy()
    return out


# (voc, random_val, topp, topk, temperature, kind of logits).  The first nine are the reference's own test
# cases (operatorspy/tests/random_sample.py:161-171, uniform [0, 1) logits as there); the rest vary the
# distribution, the tail length, the ties and the special values.
RANDOM_SAMPLE_CASES = [
    (512, 0.92, 0.8, 3, 0.5, "uniform"), (4096, 0.95, 0.9, 5, 1.0, "uniform"), (16384, 0.85, 0.85, 10, 2.0, "uniform"),
    (512, 0.92, 0.0, 3, 0.5, "uniform"), (4096, 0.95, 0.9, 1, 1.0, "uniform"), (16384, 0.85, 0.0, 1, 2.0, "uniform"),
    (16384, 0.85, 0.0, 1, 2.0, "uniform"), (32000, 0.8, 0.8, 50, 1.0, "uniform"), (32000, 0.8, 1.0, 25, 1.0, "uniform"),
    (32000, 0.31, 0.95, 40, 0.7, "normal"), (32000, 0.999, 1.0, 64, 1.5, "normal"), (32003, 0.5, 0.9, 20, 1.0, "normal"),
    (1001, 0.0, 0.5, 8, 1.0, "normal"), (1001, 0.77, 0.3, 8, 0.25, "normal"), (5, 0.6, 0.9, 9, 1.0, "normal"),
    (2, 0.99, 1.0, 2, 1.0, "normal"), (1, 0.5, 0.9, 4, 1.0, "normal"), (1, 0.5, 0.0, 1, 1.0, "normal"),
    (4096, 0.4, 0.9, 12, 1.0, "few_values"), (4096, 0.9, 1.0, 300, 1.0, "few_values"), (777, 0.2, 0.0, 5, 1.0, "few_values"),
    (8192, 0.66, 0.99, 1000, 3.0, "normal"), (50000, 0.45, 0.8, 30, 0.9, "normal"),
    (640, 1.0, 0.9, 6, 1.0, "normal"),            # random_val = 1: nothing is written
    (640, 0.3, 0.0, 1, 1.0, "nan_inside"), (640, 0.3, 0.0, 1, 1.0, "nan_first"), (640, 0.3, 0.9, 1, 1.0, "neg_zero_first"),
    (900, 0.5, 0.9, 7, 1.0, "with_inf"),
    # more candidates than any fixed-size list: the reference clamps topk to the vocabulary and nothing else
    (5000, 0.42, 0.9, 1025, 1.0, "normal"), (32000, 0.77, 0.95, 4096, 0.8, "normal"), (8192, 0.63, 1.0, 8192, 2.0, "normal"),
    (3000, 0.15, 0.99, 5000, 1.0, "uniform"), (16384, 0.9, 0.999, 16384, 1.0, "uniform"),
]


def random_sample_logits(rng, voc, kind):
    if kind == "uniform":
        return rng.random(voc, dtype=np.float32).astype(np.float16).view(np.uint16)
    if kind == "few_values":
        return rng.choice(np.array([-1.5, 0.0, 0.25, 2.0, 3.5], np.float16), voc).view(np.uint16)
    x = (rng.standard_normal(voc, dtype=np.float32) * 3).astype(np.float16).view(np.uint16)
    if kind == "nan_inside":
        x[voc // 2] = 0x7E01
    elif kind == "nan_first":
        x[0] = 0xFE00
    elif kind == "neg_zero_first":
        x[:] = np.where(x & 0x8000, x, 0x0000)  # nothing positive: the maximum is zero
        x[0], x[5] = 0x8000, 0x0000
    elif kind == "with_inf":
        x[3], x[17] = 0xFC00, 0xFC00
    return x


def random_sample_vectors():
    rng = np.random.default_rng(20241126)
    out, index = {}, []
    for i, (voc, rv, topp, topk, temp, kind) in enumerate(RANDOM_SAMPLE_CASES):
        x = random_sample_logits(rng, voc, kind)
        got = ref.random_sample(x, rv, topp, topk, temp)
        out[f"rs{i}_logits"] = x
        index.append(-1 if got is None else got)
    out["rs_index"] = np.array(index, np.int64)
    return out


def status_cases():
    """Create-time (and, for RMSNorm, compute-time) status codes of the reference."""
    cases = []

    def rec(op, tensors, **extra):
        specs = [(dt, list(shape), None if st is None else list(st)) for dt, shape, st in tensors]
        if op == "add":
            st = ref.add_status(*tensors)
        elif op == "swiglu":
            st = ref.swiglu_status(*tensors)
        elif op == "rope":
            st = ref.rope_status(*tensors)
        elif op == "rms_norm":
            st = ref.rms_norm_status(*tensors, run=extra.get("run", False))
        elif op == "causal_softmax":
            st = ref.causal_softmax_status(*tensors)
        elif op == "rearrange":
            st = ref.rearrange_status(*tensors)
        elif op == "random_sample":
            st = ref.random_sample_status(*tensors)
        cases.append({"op": op, "tensors": specs, "status": int(st), **extra})

    T = lambda dt, shape, st=None: (dt, tuple(shape), None if st is None else tuple(st))  # noqa: E731
    # Add (c, a, b)
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4)), T("f16", (8, 4))])
    rec("add", [T("f32", (8, 4)), T("f32", (8, 4)), T("f32", (4,))])
    rec("add", [T("f16", ()), T("f16", ()), T("f16", ())])
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4)), T("f16", (8, 4), (0, 1))])  # explicit stride-0 operand
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4), (8, 1)), T("f16", (8, 4))])  # padded rows
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4), (8, 2)), T("f16", (8, 4))])  # passes the reference's contiguity rule
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4)), T("f16", (8, 3))])
    rec("add", [T("f16", (8, 4)), T("f16", (4,)), T("f16", (4,))])
    rec("add", [T("f16", (1, 8, 4)), T("f16", (8, 4)), T("f16", (8, 4))])
    rec("add", [T("f16", (8, 4)), T("f16", (8, 4)), T("f32", (8, 4))])
    rec("add", [T("f64", (8, 4)), T("f64", (8, 4)), T("f64", (8, 4))])
    rec("add", [T("bf16", (8, 4)), T("bf16", (8, 4)), T("bf16", (8, 4))], bf16_extension=True)
    rec("add", [T("f16", (8, 3)), T("f16", (8, 4), (8, 1)), T("f16", (8, 4))])  # shape is reported before strides
    rec("add", [T("f64", (8, 4)), T("f64", (8, 4), (8, 1)), T("f64", (8, 4))])  # strides before dtype
    # SwiGLU (c, a, b)
    rec("swiglu", [T("f16", (4, 16)), T("f16", (4, 16)), T("f16", (4, 16))])
    rec("swiglu", [T("f16", (4, 16)), T("f16", (4, 16), (32, 1)), T("f16", (4, 16), (32, 1))])
    rec("swiglu", [T("f16", (4, 16)), T("f16", (4, 16)), T("f16", (4, 8))])  # -> BAD_PARAM
    rec("swiglu", [T("f16", (4, 16)), T("f32", (4, 16)), T("f16", (4, 16))])  # -> BAD_PARAM
    rec("swiglu", [T("f32", (4, 16)), T("f32", (4, 16)), T("f32", (4, 16))])
    rec("swiglu", [T("f16", (4, 16)), T("f16", (4, 16), (32, 2)), T("f16", (4, 16))])
    rec("swiglu", [T("f16", (4, 4, 4)), T("f16", (4, 16)), T("f16", (4, 16))])
    rec("swiglu", [T("f16", (64,)), T("f16", (64,)), T("f16", (64,))])
    rec("swiglu", [T("bf16", (4, 16)), T("bf16", (4, 16)), T("bf16", (4, 16))], bf16_extension=True)
    rec("swiglu", [T("f32", (4, 16), (16, 2)), T("f32", (4, 16)), T("f32", (4, 16))])  # dtype before strides
    # RoPE (t, pos, sin, cos)
    good = [T("f16", (4, 2, 8)), T("u64", (4,)), T("f32", (16, 8)), T("f32", (16, 8))]
    rec("rope", good)
    rec("rope", [T("f16", (4, 2, 8), (48, 24, 1))] + good[1:])
    rec("rope", [T("f16", (4, 2, 7))] + good[1:3] + [T("f32", (16, 8))])
    rec("rope", [T("f16", (4, 2, 7)), T("u64", (4,)), T("f32", (16, 7)), T("f32", (16, 7))])
    rec("rope", [good[0], T("u64", (5,)), good[2], good[3]])
    rec("rope", [good[0], good[1], T("f32", (16, 8)), T("f32", (17, 8))])
    rec("rope", [good[0], good[1], T("f32", (16, 4)), T("f32", (16, 4))])
    rec("rope", [T("f16", (4, 2, 8), (32, 16, 2))] + good[1:])
    rec("rope", [good[0], T("u64", (4,), (2,)), good[2], good[3]])
    rec("rope", [good[0], good[1], T("f32", (16, 8), (16, 2)), good[3]])
    rec("rope", [T("f32", (4, 2, 8))] + good[1:])
    rec("rope", [good[0], T("i64", (4,)), good[2], good[3]])
    rec("rope", [good[0], good[1], T("f16", (16, 8)), T("f16", (16, 8))])
    rec("rope", [T("f16", (4, 16))] + good[1:])
    rec("rope", [T("bf16", (4, 2, 8))] + good[1:], bf16_extension=True)
    # RMSNorm (y, x, w); run=True reports the compute-stage status after a successful create
    rec("rms_norm", [T("f16", (4, 32)), T("f16", (4, 32)), T("f16", (32,))], run=True)
    rec("rms_norm", [T("f16", (4, 32)), T("f16", (4, 32)), T("f32", (32,))], run=True)
    rec("rms_norm", [T("f16", (4, 32)), T("f16", (4, 32)), T("f16", (16,))])
    rec("rms_norm", [T("f16", (4, 32)), T("f16", (3, 32)), T("f16", (32,))])
    rec("rms_norm", [T("f16", (4, 32)), T("f16", (4, 32)), T("f16", (1, 32))])
    rec("rms_norm", [T("f16", (128,)), T("f16", (128,)), T("f16", (128,))])
    rec("rms_norm", [T("f32", (4, 32)), T("f32", (4, 32)), T("f32", (32,))], run=True)
    rec("rms_norm", [T("bf16", (4, 32)), T("bf16", (4, 32)), T("f32", (32,))], run=True, bf16_extension=True)
    # causal softmax (y)
    rec("causal_softmax", [T("f16", (4, 8, 16))])
    rec("causal_softmax", [T("f16", (8, 16))])
    rec("causal_softmax", [T("f16", (8, 16), (32, 1))])
    rec("causal_softmax", [T("f16", (16,))])
    rec("causal_softmax", [T("f16", (2, 2, 8, 16))])
    rec("causal_softmax", [T("f32", (8, 16))])
    rec("causal_softmax", [T("bf16", (8, 16))], bf16_extension=True)
    rec("causal_softmax", [T("f16", (8, 16), (32, 2))], cpu_only_layout=True)  # accepted by the CPU back end, refused by the GPU ones
    # rearrange (dst, src)
    rec("rearrange", [T("f16", (4, 6, 64)), T("f16", (4, 6, 64), (64, 2560, 1))])
    rec("rearrange", [T("f16", (64,)), T("f16", (64,))])
    rec("rearrange", [T("f16", (4, 64)), T("f32", (4, 64))])
    rec("rearrange", [T("f16", (4, 64)), T("f16", (4, 1, 64))])
    rec("rearrange", [T("f16", ()), T("f16", ())])
    rec("rearrange", [T("f16", (4, 64)), T("f16", (4, 32))])
    rec("rearrange", [T("f16", (4, 64), (128, 2)), T("f16", (4, 64))])
    rec("rearrange", [T("f16", (4, 64)), T("f16", (4, 64), (1, 4))])
    rec("rearrange", [T("f16", (2, 3, 4, 8)), T("f16", (2, 3, 4, 8), (192, 64, 10, 1))])
    rec("rearrange", [T("f16", (2, 3, 4, 8)), T("f16", (2, 3, 4, 8), (200, 64, 10, 1))])   # dim 1 does not nest in dim 0
    rec("rearrange", [T("f16", (2, 2, 3, 4, 8)), T("f16", (2, 2, 3, 4, 8), (400, 192, 64, 10, 1))])  # dim 1 does not nest in dim 0
    rec("rearrange", [T("bf16", (4, 64)), T("bf16", (4, 64))])
    rec("rearrange", [T("u8", (4, 64)), T("u8", (4, 64), (100, 1))])
    rec("rearrange", [T("f16", (0, 4)), T("f16", (0, 4))])                      # an extent of zero: accepted, nothing to copy
    rec("rearrange", [T("f16", (3, 0, 8)), T("f16", (3, 0, 8), (64, 8, 1))])
    rec("rearrange", [T("f16", (4, 0)), T("f16", (4, 0))])
    # RandomSample (result, probs)
    rec("random_sample", [T("u64", (1,)), T("f16", (512,))])
    rec("random_sample", [T("u64", (4,)), T("f16", (512,))])         # rank 1 of any length passes
    rec("random_sample", [T("u64", (1, 3)), T("f16", (512,))])       # first extent 1 passes
    rec("random_sample", [T("u64", (2, 3)), T("f16", (512,))])
    rec("random_sample", [T("u64", (1,)), T("f16", (2, 256))])
    rec("random_sample", [T("u64", (1,)), T("f32", (512,))])
    rec("random_sample", [T("i64", (1,)), T("f16", (512,))])
    rec("random_sample", [T("i64", (2, 3)), T("f16", (512,))])       # type is reported before shape
    rec("random_sample", [T("u64", (1,)), T("bf16", (512,))], bf16_extension=True)
    return cases


def main(only=None):
    """With `only` (a set of fixture names) the other .npz files are left as they are."""
    assert ref.available(), "build oracle/_ref first: make -C oracle ref"
    if only is not None:
        if "random_sample" in only:
            np.savez_compressed(os.path.join(HERE, "random_sample.npz"), **random_sample_vectors())
        write_json()
        return
    rng = np.random.default_rng(20241125)
    np.savez_compressed(os.path.join(HERE, "conversions.npz"), **conversions(rng))
    np.savez_compressed(os.path.join(HERE, "add.npz"), **add_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "rms_norm.npz"), **rms_norm_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "rope.npz"), **rope_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "swiglu.npz"), **swiglu_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "causal_softmax.npz"), **causal_softmax_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "rearrange.npz"), **rearrange_vectors(rng))
    np.savez_compressed(os.path.join(HERE, "random_sample.npz"), **random_sample_vectors())
    write_json()


def write_json():
    with open(os.path.join(HERE, "status_cases.json"), "w") as f:
        json.dump({"add_cases": [list(map(list, c)) for c in ADD_CASES],
                   "rope_cases": [[list(s), None if st is None else list(st), r] for s, st, r in ROPE_CASES],
                   "swiglu_cases": [[list(s), a, b, c] for s, a, b, c in SWIGLU_CASES],
                   "rearrange_cases": [[dt, list(sh), None if a is None else list(a), None if b is None else list(b)] for dt, sh, a, b in REARRANGE_CASES],
                   "causal_cases": [[list(s), None if st is None else list(st)] for s, st in CAUSAL_CASES],
                   "random_sample_cases": [list(c) for c in RANDOM_SAMPLE_CASES],
                   "status": status_cases()}, f, indent=1)
    for name in sorted(os.listdir(HERE)):
        print(f"{name:24s} {os.path.getsize(os.path.join(HERE, name)):>9d} bytes")


if __name__ == "__main__":
    main(set(sys.argv[1:]) or None)
