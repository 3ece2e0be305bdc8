"""Pins the oracle's four operators (oracle.c) on the CPU:
  * the golden vectors written by the compiled reference (always);
  * the compiled reference itself on fresh seeded inputs (where oracle/_ref
    was built, i.e. where the reference sources are present);
  * closed forms and invariants that a dropped term, a wrong sign or a
    swapped operand would break;
  * for the bf16 extension, torch's CPU bf16 arithmetic.
"""
import numpy as np
import pytest

import oracle
from helpers import assert_codes_close, assert_codes_equal, golden, golden_json
from oracle import ref

needs_ref = pytest.mark.skipif(not ref.available(), reason="oracle/_ref not built (no reference checkout on this machine)")


def same_bits(a, b):
    if a.dtype == np.float32:
        nan = np.isnan(b)
        return np.array_equal(np.isnan(a), nan) and np.array_equal(a.view(np.uint32)[~nan], b.view(np.uint32)[~nan])
    return np.array_equal(a, b)


# ---- Add --------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_add_golden(dt):
    g = golden("add")
    for i, (cs, as_, bs) in enumerate(golden_json()["add_cases"]):
        got = oracle.add(g[f"add{i}_{dt}_a"].reshape(as_), g[f"add{i}_{dt}_b"].reshape(bs), tuple(cs), dt)
        assert same_bits(got, g[f"add{i}_{dt}_c"].reshape(cs)), (i, cs, as_, bs)


def test_add_golden_special_values():
    g = golden("add")
    codes = np.arange(65536, dtype=np.uint16)
    got = oracle.add(codes, np.zeros(65536, np.uint16), (65536,), "f16")
    assert np.array_equal(got, g["add_all_codes_plus_zero"])
    # x + 0 is the identity except for -0 (-> +0) and NaNs (-> canonical)
    nan = ((codes & 0x7C00) == 0x7C00) & ((codes & 0x3FF) != 0)
    keep = ~nan & (codes != 0x8000)
    assert np.array_equal(got[keep], codes[keep]) and got[0x8000] == 0
    rows, cols = g["add_table_rows"], g["add_table_cols"]
    got = oracle.add(np.ascontiguousarray(rows.reshape(-1, 1)), cols, (rows.size, cols.size), "f16")
    assert_codes_equal(got, g["add_table_c"], "f16", nan_sign_free=False, what="addition table block")


def test_add_is_exact_sum_truncated():
    """Independent statement of fp16 add: the exact sum (fp16+fp16 is exact in
    fp64) rounded to nearest fp32 - that is what an fp32 add returns - and then
    truncated toward zero onto the fp16 grid."""
    rng = np.random.default_rng(11)
    a = rng.integers(0, 0x7800, 200_000, dtype=np.uint16) | (rng.integers(0, 2, 200_000, dtype=np.uint16) << 15)
    b = rng.integers(0, 0x7800, 200_000, dtype=np.uint16) | (rng.integers(0, 2, 200_000, dtype=np.uint16) << 15)
    got = oracle.add(a, b, a.shape, "f16")
    exact = (a.view(np.float16).astype(np.float64) + b.view(np.float16).astype(np.float64)).astype(np.float32).astype(np.float64)
    with np.errstate(over="ignore"):
        near = exact.astype(np.float16)
    away = np.abs(near.astype(np.float64)) > np.abs(exact)
    want = np.where(away, np.nextafter(near, np.float16(0)), near).view(np.uint16)
    ok = np.abs(exact) < 65504  # below the overflow quirk
    nz = ok & (exact != 0)
    assert np.array_equal(got[nz], want[nz])


@needs_ref
@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_add_vs_compiled_reference(dt):
    rng = np.random.default_rng(12)
    for cs, as_, bs in [((40, 33, 17), (40, 33, 17), (40, 33, 17)), ((40, 33, 17), (33, 1), (40, 1, 17)), ((6, 5, 4, 3, 2), (5, 1, 3, 1), (6, 1, 4, 1, 2))]:
        a = oracle.encode(rng.standard_normal(as_).astype(np.float32) * 100, dt)
        b = oracle.encode(rng.standard_normal(bs).astype(np.float32) * 100, dt)
        assert same_bits(oracle.add(a, b, cs, dt), ref.add(a, b, cs, dt))
    if dt == "f16":  # random codes incl. NaN/Inf/subnormal, sign of NaN included
        a = rng.integers(0, 65536, (300, 300), dtype=np.uint16)
        b = rng.integers(0, 65536, (300, 300), dtype=np.uint16)
        assert np.array_equal(oracle.add(a, b, a.shape, dt), ref.add(a, b, a.shape, dt))


def test_add_bf16_extension_is_torch_cpu():
    import torch

    rng = np.random.default_rng(13)
    a = oracle.encode(rng.standard_normal((64, 96)).astype(np.float32) * 50, "bf16")
    b = oracle.encode(rng.standard_normal((96,)).astype(np.float32) * 50, "bf16")
    ta = torch.from_numpy(a.view(np.int16)).view(torch.bfloat16)
    tb = torch.from_numpy(b.view(np.int16)).view(torch.bfloat16)
    want = (ta + tb).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(oracle.add(a, b, (64, 96), "bf16"), want)


# ---- RMSNorm ----------------------------------------------------------------------
def test_rms_norm_golden():
    g = golden("rms_norm")
    assert_codes_close(oracle.rms_norm(g["rms0_x"], g["rms0_w16"], 1e-5, "f16", "f16"), g["rms0_y_w16"], "f16", max_ulp=1, max_frac=1e-3, what="w f16")
    assert_codes_close(oracle.rms_norm(g["rms0_x"], g["rms0_w32"], 1e-5, "f16", "f32"), g["rms0_y_w32"], "f16", max_ulp=1, max_frac=1e-3, what="w f32")
    for i in range(1, 5):
        got = oracle.rms_norm(g[f"rms{i}_x"], g[f"rms{i}_w32"], 1e-6, "f16", "f32")
        # bit-exact where libm's pow agrees with the one that wrote the fixture; never more than an ulp
        assert_codes_close(got, g[f"rms{i}_y_w32"], "f16", max_ulp=1, max_frac=1e-3, what=f"case {i}")


@needs_ref
def test_rms_norm_vs_compiled_reference():
    rng = np.random.default_rng(14)
    for n, d in [(16, 2048), (7, 333), (3, 5000)]:
        x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32) * 5, "f16")
        for wdt in ("f16", "f32"):
            w = oracle.encode(rng.uniform(-2, 2, d).astype(np.float32), wdt)
            assert np.array_equal(oracle.rms_norm(x, w, 1e-5, "f16", wdt), ref.rms_norm(x, w, 1e-5, "f16", wdt))


def test_rms_norm_closed_forms():
    # constant row c, w = 1: c / sqrt(c^2 + eps), truncated
    for c in (0.5, -3.0, 100.0):
        x = oracle.encode(np.full((2, 256), c, np.float32), "f16")
        got = oracle.decode(oracle.rms_norm(x, np.ones(256, np.float32), 1e-5, "f16", "f32"), "f16")
        exact = c / np.sqrt(np.float64(c) ** 2 + 1e-5)
        assert np.all(np.abs(got - exact) <= 2.0 ** -10 * abs(exact))
        assert np.all(np.abs(got) <= abs(exact) * (1 + 1e-6))  # truncation never rounds away from zero
    # scaling w scales y; a unit-RMS row with w = 1 comes back (to truncation)
    rng = np.random.default_rng(15)
    v = rng.standard_normal((4, 512))
    v /= np.sqrt((v ** 2).mean(axis=1, keepdims=True))
    x = oracle.encode(v.astype(np.float32), "f16")
    y = oracle.decode(oracle.rms_norm(x, np.ones(512, np.float32), 0.0, "f16", "f32"), "f16")
    xv = oracle.decode(x, "f16")
    assert np.all(np.abs(y - xv) <= 2e-3 * np.abs(xv) + 1e-6)
    y2 = oracle.decode(oracle.rms_norm(x, np.full(512, 2.0, np.float32), 0.0, "f16", "f32"), "f16")
    assert np.all(np.abs(y2 - 2 * y) <= 2.0 ** -9 * np.abs(y2) + 1e-6)


def test_rms_norm_bf16_extension_matches_float64_formula():
    rng = np.random.default_rng(16)
    x = oracle.encode(rng.standard_normal((8, 1024)).astype(np.float32), "bf16")
    w = rng.uniform(0.5, 1.5, 1024).astype(np.float32)
    got = oracle.decode(oracle.rms_norm(x, w, 1e-5, "bf16", "f32"), "bf16").astype(np.float64)
    xv = oracle.decode(x, "bf16").astype(np.float64)
    want = xv / np.sqrt((xv ** 2).mean(axis=1, keepdims=True) + 1e-5) * w
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)  # half a bf16 ulp, with slack for fp32 steps


# ---- fused Add + RMSNorm: the reference's two calls in sequence ------------------------
@needs_ref
def test_add_rms_norm_is_the_reference_add_then_rms_norm():
    rng = np.random.default_rng(17)
    for n, d in [(16, 2048), (5, 333)]:
        a = oracle.encode(rng.standard_normal((n, d)).astype(np.float32) * 3, "f16")
        b = oracle.encode(rng.standard_normal((n, d)).astype(np.float32) * 3, "f16")
        w = oracle.encode(rng.uniform(0.5, 1.5, d).astype(np.float32), "f32")
        c, y = oracle.add_rms_norm(a, b, w, 1e-5, "f16", "f32")
        rc = ref.add(a, b, (n, d), "f16")
        assert np.array_equal(c, rc) and np.array_equal(y, ref.rms_norm(rc, w, 1e-5, "f16", "f32"))


def test_add_rms_norm_normalises_the_rounded_sum():
    """The norm is taken over the 16-bit sum, not over the exact one: a + b with
    a = 1, b = 2^-12 rounds to 1 in fp16, so y must equal RMSNorm of a row of ones."""
    a = oracle.encode(np.ones((1, 64), np.float32), "f16")
    b = oracle.encode(np.full((1, 64), 2.0 ** -12, np.float32), "f16")
    w = np.ones(64, np.float32)
    c, y = oracle.add_rms_norm(a, b, w, 0.0, "f16", "f32")
    assert np.all(c == a) and np.array_equal(y, oracle.rms_norm(a, w, 0.0, "f16", "f32"))


# ---- RoPE ---------------------------------------------------------------------------
def test_rope_golden():
    g = golden("rope")
    for i, (shape, strides, rows) in enumerate(golden_json()["rope_cases"]):
        t = g[f"rope{i}_t_in"].copy()
        oracle.rope(t, g[f"rope{i}_pos"], g[f"rope{i}_sin"], g[f"rope{i}_cos"], "f16")
        assert np.array_equal(t, g[f"rope{i}_t_out"]), (i, shape)
        if i >= 2:
            assert not np.array_equal(g[f"rope{i}_t_in"], g[f"rope{i}_t_out"])  # the fixture really rotates
        if strides is not None:  # same through the strided buffer, gaps untouched
            buf = g[f"rope{i}_buf_in"].copy()
            view = np.lib.stride_tricks.as_strided(buf, shape, [s * 2 for s in strides])
            oracle.rope(view, g[f"rope{i}_pos"], g[f"rope{i}_sin"], g[f"rope{i}_cos"], "f16")
            assert np.array_equal(buf, g[f"rope{i}_buf_out"])


@needs_ref
def test_rope_vs_compiled_reference():
    rng = np.random.default_rng(17)
    for shape in [(9, 4, 64), (5, 3, 10), (2, 1, 2)]:
        t = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 4, "f16")
        pos = rng.integers(0, 50, shape[0]).astype(np.uint64)
        s = rng.uniform(-1, 1, (50, shape[2])).astype(np.float32)
        c = rng.uniform(-1, 1, (50, shape[2])).astype(np.float32)
        assert np.array_equal(oracle.rope(t.copy(), pos, s, c, "f16"), ref.rope(t.copy(), pos, s, c, "f16"))


def test_rope_closed_forms():
    rng = np.random.default_rng(18)
    t = oracle.encode(rng.standard_normal((6, 2, 16)).astype(np.float32), "f16")
    ones, zeros = np.ones((4, 16), np.float32), np.zeros((4, 16), np.float32)
    pos = np.array([0, 1, 2, 3, 0, 1], np.uint64)
    # angle 0 is the identity
    assert np.array_equal(oracle.rope(t.copy(), pos, zeros, ones, "f16"), t)
    # a quarter turn maps (a, b) to (-b, a): catches a wrong sign or swapped sin/cos
    q = oracle.rope(t.copy(), pos, ones, zeros, "f16")
    assert np.array_equal(q[..., 0::2], t[..., 1::2] ^ 0x8000) and np.array_equal(q[..., 1::2], t[..., 0::2])
    # each output uses its own table column: sin differs between the two members of a pair
    s = np.zeros((4, 16), np.float32)
    s[:, 1::2] = 1.0  # sin[2k] = 0, sin[2k+1] = 1, cos = 0 -> t[2k] = 0*a - b*0 = 0 ; t[2k+1] = a*1 + b*0 = a
    r = oracle.rope(t.copy(), pos, s, zeros, "f16")
    assert np.array_equal(r[..., 1::2], t[..., 0::2]) and not (r[..., 0::2] & 0x7FFF).any()
    # the table row is pos*head_dim: token 1 (pos 1) must see row 1 only
    s2 = np.zeros((4, 16), np.float32)
    c2 = np.ones((4, 16), np.float32)
    s2[1], c2[1] = 1.0, 0.0
    r2 = oracle.rope(t.copy(), pos, s2, c2, "f16")
    assert np.array_equal(r2[0], t[0]) and np.array_equal(r2[2], t[2]) and np.array_equal(r2[1, :, 1::2], t[1, :, 0::2])


def test_rope_bf16_extension_matches_float64_rotation():
    rng = np.random.default_rng(19)
    t = oracle.encode(rng.standard_normal((5, 3, 32)).astype(np.float32), "bf16")
    ang = rng.uniform(0, 6.28, (7, 16))
    s, c = np.repeat(np.sin(ang), 2, axis=1).astype(np.float32), np.repeat(np.cos(ang), 2, axis=1).astype(np.float32)
    pos = rng.integers(0, 7, 5).astype(np.uint64)
    got = oracle.decode(oracle.rope(t.copy(), pos, s, c, "bf16"), "bf16").astype(np.float64)
    v = oracle.decode(t, "bf16").astype(np.float64)
    z = (v[..., 0::2] + 1j * v[..., 1::2]) * np.exp(1j * ang[pos.astype(int)])[:, None, :]
    want = np.stack([z.real, z.imag], -1).reshape(v.shape)
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-6)


# ---- SwiGLU -------------------------------------------------------------------------
def test_swiglu_golden():
    g = golden("swiglu")
    for i, (shape, sa, sb, sc) in enumerate(golden_json()["swiglu_cases"]):
        got = oracle.swiglu(g[f"swiglu{i}_a"], g[f"swiglu{i}_b"], "f16")
        assert_codes_close(got, g[f"swiglu{i}_c"], "f16", max_ulp=1, max_frac=1e-3, what=f"case {i}")
    assert_codes_close(oracle.swiglu(g["swiglu_sat_a"], g["swiglu_sat_b"], "f16"), g["swiglu_sat_c"], "f16", max_ulp=1, max_frac=0.1, what="saturation")


@needs_ref
def test_swiglu_vs_compiled_reference():
    rng = np.random.default_rng(20)
    buf = oracle.encode(rng.standard_normal((9, 2 * 120)).astype(np.float32) * 6, "f16")
    b, a = buf[:, :120], buf[:, 120:]  # fused gate/up halves: strided rows
    assert np.array_equal(oracle.swiglu(a, b, "f16"), ref.swiglu(a, b, "f16"))
    a2 = rng.integers(0, 65536, (100, 64), dtype=np.uint16)  # any codes, NaN/Inf included
    b2 = rng.integers(0, 65536, (100, 64), dtype=np.uint16)
    assert_codes_equal(oracle.swiglu(a2, b2, "f16"), ref.swiglu(a2, b2, "f16"), "f16", what="random codes")


def test_swiglu_closed_forms():
    f = lambda v: oracle.encode(np.array([v], np.float32), "f16")  # noqa: E731
    d = lambda c: oracle.decode(c, "f16")[0]  # noqa: E731
    a = f([1.5, -2.0, 3.0, 0.5, 2.0, 7.0])
    b = f([0.0, -0.0, 30.0, 40.0, -30.0, 1.0])
    got = d(oracle.swiglu(a, b, "f16"))
    assert got[0] == 0 and got[1] == 0            # b = 0 -> 0 whatever a is
    assert got[2] == 90.0 and got[3] == 20.0      # large b: gate is the identity, c = a*b
    assert abs(got[4]) < 1e-10                    # very negative b: c -> 0
    assert abs(got[5] - 7.0 / (1 + np.exp(-1.0))) <= 2.0 ** -9 * 6  # b is the gated operand, a the linear one
    # and against float64 on random data
    rng = np.random.default_rng(21)
    av = oracle.encode(rng.standard_normal((4, 300)).astype(np.float32) * 3, "f16")
    bv = oracle.encode(rng.standard_normal((4, 300)).astype(np.float32) * 3, "f16")
    x, y = oracle.decode(av, "f16").astype(np.float64), oracle.decode(bv, "f16").astype(np.float64)
    want = x * y / (1 + np.exp(-y))
    got = oracle.decode(oracle.swiglu(av, bv, "f16"), "f16")
    assert np.all(np.abs(got - want) <= 2.0 ** -10 * np.abs(want) + 2.0 ** -24)


def test_swiglu_bf16_extension_matches_float64_formula():
    rng = np.random.default_rng(22)
    av = oracle.encode(rng.standard_normal((4, 300)).astype(np.float32) * 3, "bf16")
    bv = oracle.encode(rng.standard_normal((4, 300)).astype(np.float32) * 3, "bf16")
    x, y = oracle.decode(av, "bf16").astype(np.float64), oracle.decode(bv, "bf16").astype(np.float64)
    want = x * y / (1 + np.exp(-y))
    got = oracle.decode(oracle.swiglu(av, bv, "bf16"), "bf16")
    assert np.all(np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-30)


# ---- causal softmax (first operator beyond the four-operator path) -------------------
def test_causal_softmax_golden():
    g = golden("causal_softmax")
    for i, (shape, strides) in enumerate(golden_json()["causal_cases"]):
        y = g[f"causal{i}_in"].copy()
        oracle.causal_softmax(y, "f16")
        assert_codes_close(y, g[f"causal{i}_out"], "f16", max_ulp=1, max_frac=1e-3, what=f"case {i} {shape}")


@needs_ref
def test_causal_softmax_vs_compiled_reference():
    rng = np.random.default_rng(23)
    for shape in [(3, 17, 64), (9, 9), (2, 5, 333)]:
        y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 4, "f16")
        assert np.array_equal(oracle.causal_softmax(y.copy(), "f16"), ref.causal_softmax(y.copy(), "f16"))


@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_causal_softmax_against_float64(dt):
    rng = np.random.default_rng(24)
    seq, total = 12, 40
    y = oracle.encode(rng.standard_normal((3, seq, total)).astype(np.float32), dt)
    x = oracle.decode(y, dt).astype(np.float64)
    got = oracle.decode(oracle.causal_softmax(y.copy(), dt), dt).astype(np.float64)
    j, i = np.arange(total)[None, :], np.arange(seq)[:, None]
    keep = j <= total - seq + i                      # row i keeps columns up to total - seq + i
    z = np.where(keep, x, -np.inf)
    want = np.exp(z - z.max(-1, keepdims=True))
    want /= want.sum(-1, keepdims=True)
    ulp = 2.0 ** -10 if dt == "f16" else 2.0 ** -7
    assert np.all(np.abs(got - want) <= ulp * want + 1e-7)
    assert np.all(got[:, ~keep] == 0) and np.all(got[:, keep] > 0)
    assert np.all(np.abs(got.sum(-1) - 1) < 40 * ulp)  # truncation loses up to one ulp per kept element
    assert got[:, 0, : total - seq + 1].min() > 0 and np.count_nonzero(got[:, 0]) == 3 * (total - seq + 1)


# ---- rearrange (second operator beyond the four-operator path) ------------------------
NP_OF = {"f16": np.uint16, "f32": np.float32, "u8": np.uint8, "f64": np.float64}


def _views(g, i, dt, shape, ss, sd):
    def contig(sh):
        out, run = [], 1
        for n in reversed(sh):
            out.append(run)
            run *= n
        return list(reversed(out))
    item = np.dtype(NP_OF[dt]).itemsize
    ss, sd = ss or contig(shape), sd or contig(shape)
    src_buf, dst_buf = g[f"rearrange{i}_src"].copy(), g[f"rearrange{i}_dst_before"].copy()
    src = np.lib.stride_tricks.as_strided(src_buf, shape, [s * item for s in ss])
    dst = np.lib.stride_tricks.as_strided(dst_buf, shape, [s * item for s in sd])
    return src, dst, dst_buf


def test_rearrange_golden_and_numpy():
    g = golden("rearrange")
    for i, (dt, shape, ss, sd) in enumerate(golden_json()["rearrange_cases"]):
        src, dst, dst_buf = _views(g, i, dt, shape, ss, sd)
        oracle.rearrange(dst, src)
        assert np.array_equal(dst_buf.view(np.uint8), g[f"rearrange{i}_dst_after"].view(np.uint8)), (i, dt, shape)
        # and numpy's own strided assignment says the same
        src2, dst2, dst_buf2 = _views(g, i, dt, shape, ss, sd)
        dst2[...] = src2
        assert np.array_equal(dst_buf2.view(np.uint8), dst_buf.view(np.uint8))


# ---- matmul and the MLP composite (third step beyond the four-operator path) ------------
MATMUL_CASES = [
    # alpha, beta, a, b, c shapes, a, b, c strides: the reference's own test list (operatorspy/tests/matmul.py:297-306) ...
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), None, None, None),
    (1.0, 0.0, (2, 4, 2048), (2, 2048, 2048), (2, 4, 2048), None, None, None),
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), (4096, 1), (4096, 1), (4096, 1)),
    (1.0, 1.0, (6, 2048), (2048, 2560), (6, 2560), (2048, 1), (1, 2048), (2560, 1)),
    (1.0 / 8.0, 0.0, (4, 8 * 6, 64), (4, 64, 6), (4, 8 * 6, 6), None, None, None),
    # ... and layouts it does not cover
    (0.5, -1.5, (33, 100), (100, 17), (33, 17), (1, 33), (1, 100), (1, 33)),
    (2.0, 1.0, (3, 16, 32), (32, 24), (3, 16, 24), None, None, None),
]


def _strided(x, strides):
    if strides is None:
        return x
    span = 1 + sum((n - 1) * s for n, s in zip(x.shape, strides))
    buf = np.zeros(span, x.dtype)
    view = np.lib.stride_tricks.as_strided(buf, x.shape, [s * x.itemsize for s in strides])
    view[...] = x
    return view


@needs_ref
@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("case", range(len(MATMUL_CASES)))
def test_matmul_vs_compiled_reference(dt, case):
    alpha, beta, a_shape, b_shape, c_shape, a_st, b_st, c_st = MATMUL_CASES[case]
    rng = np.random.default_rng(300 + case)
    mk = (lambda s: rng.standard_normal(s).astype(np.float32)) if dt == "f32" else (lambda s: oracle.encode(rng.standard_normal(s).astype(np.float32), dt))
    a, b, c = _strided(mk(a_shape), a_st), _strided(mk(b_shape), b_st), mk(c_shape)
    c1, c2 = _strided(c.copy(), c_st), _strided(c.copy(), c_st)
    oracle.matmul(c1, a, b, alpha, beta, dt)
    ref.matmul(c2, a, b, alpha, beta, dt)
    assert np.array_equal(c1.view(np.uint8) if c_st is None else np.ascontiguousarray(c1).view(np.uint8),
                          c2.view(np.uint8) if c_st is None else np.ascontiguousarray(c2).view(np.uint8))


def test_matmul_against_float64_and_exact_cases():
    rng = np.random.default_rng(41)
    a = oracle.encode(rng.standard_normal((20, 300)).astype(np.float32), "f16")
    b = oracle.encode(rng.standard_normal((300, 30)).astype(np.float32), "f16")
    c0 = oracle.encode(rng.standard_normal((20, 30)).astype(np.float32), "f16")
    fa, fb, fc = (oracle.decode(t, "f16").astype(np.float64) for t in (a, b, c0))
    got = oracle.decode(oracle.matmul(c0.copy(), a, b, 0.25, 2.0, "f16"), "f16").astype(np.float64)
    exact = 0.25 * fa @ fb + 2.0 * fc
    mag = 0.25 * np.abs(fa) @ np.abs(fb) + 2.0 * np.abs(fc)
    assert np.all(np.abs(got - exact) <= 2.0 ** -10 * np.abs(exact) + 300 * 2.0 ** -23 * mag)
    assert np.all(np.abs(got) <= np.abs(exact) + 300 * 2.0 ** -23 * mag)  # truncation never rounds away from zero
    # a transposed operand (column-major b) gives the same bits as its row-major copy
    bt = np.ascontiguousarray(b.T).T
    assert np.array_equal(oracle.matmul(c0.copy(), a, bt, 0.25, 2.0, "f16"), oracle.matmul(c0.copy(), a, b, 0.25, 2.0, "f16"))
    # identity and permutation matrices: exact
    eye = oracle.encode(np.eye(300, dtype=np.float32), "f16")
    out = oracle.matmul(np.zeros((20, 300), np.uint16), a, eye, 1.0, 0.0, "f16")
    assert np.array_equal(out, a)
    # beta == 0 never reads c: NaNs in c do not reach the result
    nan_c = np.full((20, 30), 0x7E00, np.uint16)
    assert np.array_equal(oracle.matmul(nan_c, a, b, 1.0, 0.0, "f16"), oracle.matmul(np.zeros((20, 30), np.uint16), a, b, 1.0, 0.0, "f16"))


@needs_ref
@pytest.mark.parametrize("residual", [False, True])
def test_mlp_vs_compiled_reference(residual):
    rng = np.random.default_rng(43)
    n, d, di = 9, 64, 96
    x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), "f16")
    w12 = oracle.encode(rng.standard_normal((d, 2 * di)).astype(np.float32) * 0.1, "f16")
    w3 = oracle.encode(rng.standard_normal((di, d)).astype(np.float32) * 0.1, "f16")
    y = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), "f16")
    assert np.array_equal(oracle.mlp(y.copy(), x, w12, w3, 0.7, residual, "f16"), ref.mlp(y.copy(), x, w12, w3, 0.7, residual, "f16"))


MATMUL_STATUS = [
    # (c, a, b) as (dtype, shape, strides) -> create status
    ((("f16", (4, 6), None), ("f16", (4, 5), None), ("f16", (5, 6), None)), 0),
    ((("f32", (2, 4, 6), None), ("f32", (2, 4, 5), None), ("f32", (5, 6), None)), 0),
    ((("f16", (2, 2, 4, 6), None), ("f16", (4, 5), None), ("f16", (5, 6), None)), 4),
    ((("f16", (4, 6), (12, 2)), ("f16", (4, 5), None), ("f16", (5, 6), None)), 5),
    ((("f16", (3, 4, 6), None), ("f16", (2, 4, 5), None), ("f16", (5, 6), None)), 2),
    ((("u8", (4, 6), None), ("u8", (4, 5), None), ("u8", (5, 6), None)), 3),
]


@needs_ref
@pytest.mark.parametrize("i", range(len(MATMUL_STATUS)))
def test_matmul_status_table_is_the_reference_s(i):
    tensors, want = MATMUL_STATUS[i]
    assert ref.matmul_status(*tensors) == want


ATTENTION_CASES = [
    # n_q_head, n_kv_head, seq, head_dim, pos, capacity, q/k/v strides, cache strides (operatorspy/tests/attention.py:310-358)
    (32, 4, 5, 64, 0, 2048, (64, 2560, 1), (64, 11264, 1)),
    (32, 4, 1, 64, 3, 2048, (64, 2560, 1), (64, 11264, 1)),
    (8, 4, 2, 16, 1, 8, None, None),
]


@needs_ref
@pytest.mark.parametrize("case", range(len(ATTENTION_CASES)))
def test_attention_vs_compiled_reference(case):
    """The oracle's composition of rearrange, matmul and causal softmax is the reference's infiniopAttention."""
    heads, kv_heads, seq, hd, pos, cap, qkv_st, cache_st = ATTENTION_CASES[case]
    rng = np.random.default_rng(600 + case)
    enc = lambda s: oracle.encode(rng.standard_normal(s).astype(np.float32), "f16")  # noqa: E731
    q, k, v = (_strided(enc(s), qkv_st) for s in ((heads, seq, hd), (kv_heads, seq, hd), (kv_heads, seq, hd)))
    kc, vc = enc((kv_heads, cap, hd)), enc((kv_heads, cap, hd))
    kc1, vc1, kc2, vc2 = (_strided(t.copy(), cache_st) for t in (kc, vc, kc, vc))
    o1 = oracle.attention(np.zeros((seq, heads, hd), np.uint16), q, k, v, kc1, vc1, pos, "f16")
    o2 = ref.attention(np.zeros((seq, heads, hd), np.uint16), q, k, v, kc2, vc2, pos, "f16")
    assert np.array_equal(o1, o2)
    assert np.array_equal(np.ascontiguousarray(kc1), np.ascontiguousarray(kc2)) and np.array_equal(np.ascontiguousarray(vc1), np.ascontiguousarray(vc2))

