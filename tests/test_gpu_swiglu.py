"""SwiGLU on the GPU through the C ABI, against the oracle and the reference's
golden vectors.  Bar (fp16): |gpu - ref| <= 1e-3 + 1e-3*|ref|, and in fact at
most one unit in the last place on a small fraction of elements (the only
source of difference is the last bit of expf).  bf16: 1e-2."""
import numpy as np
import pytest

import oracle
from helpers import (assert_allclose16, assert_codes_close, assert_codes_equal, golden, golden_json, strided_like,
                     to_codes, to_torch)

pytestmark = pytest.mark.gpu
TOL = {"f16": 1e-3, "bf16": 1e-2}


def check(got, want, dt, what):
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), TOL[dt], TOL[dt], what)
    return assert_codes_close(got, want, dt, max_ulp=1, max_frac=5e-3, what=what)


def test_golden_cases(ctx):
    import torch

    g = golden("swiglu")
    for i, (shape, sa, sb, sc) in enumerate(golden_json()["swiglu_cases"]):
        a, b, want = g[f"swiglu{i}_a"], g[f"swiglu{i}_b"], g[f"swiglu{i}_c"]
        n, di = shape
        ta = strided_like(a, shape, (sa, 1), "f16")[0] if sa else to_torch(a, "f16")
        tb = strided_like(b, shape, (sb, 1), "f16")[0] if sb else to_torch(b, "f16")
        if sc:
            tc, cbuf = strided_like(np.zeros(shape, np.uint16), shape, (sc, 1), "f16")
            before = to_codes(cbuf)
        else:
            tc = torch.empty(shape, dtype=torch.float16, device="cuda")
        ctx.swiglu(tc, ta, tb)
        torch.cuda.synchronize()
        check(to_codes(tc), want, "f16", f"golden swiglu case {i}")
        if sc:  # bytes between the rows of c are untouched
            after = to_codes(cbuf)
            mask = np.ones(after.size, bool)
            for r in range(n):
                mask[r * sc:r * sc + di] = False
            assert np.array_equal(after[mask], before[mask])


def test_golden_saturation(ctx):
    import torch

    g = golden("swiglu")
    ta, tb = to_torch(g["swiglu_sat_a"], "f16"), to_torch(g["swiglu_sat_b"], "f16")
    tc = torch.empty_like(ta)
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    check(to_codes(tc), g["swiglu_sat_c"], "f16", "saturation")


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("shape,fused", [((13, 4), False), ((16, 5632), False), ((33, 1000), True), ((64, 11008), True), ((5, 7), False),
                                         ((1, 5), False), ((3, 1001), False), ((257, 4099), False), ((7, 1001), True)])
def test_against_oracle(ctx, dt, shape, fused):
    import torch

    n, di = shape
    rng = np.random.default_rng(n * 1000 + di)
    if fused:  # gate = first half, up = second half of one [n, 2*di] buffer
        buf = oracle.encode(rng.standard_normal((n, 2 * di)).astype(np.float32) * 2, dt)
        b, a = buf[:, :di], buf[:, di:]
        tbuf = to_torch(buf, dt)
        tb, ta = tbuf[:, :di], tbuf[:, di:]
    else:
        a = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 2, dt)
        b = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 2, dt)
        ta, tb = to_torch(a, dt), to_torch(b, dt)
    want = oracle.swiglu(a, b, dt)
    tc = torch.empty(shape, dtype=ta.dtype, device="cuda")
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    check(to_codes(tc), want, dt, f"{shape} fused={fused} {dt}")


@pytest.mark.parametrize("which", ["a", "b"])
def test_in_place(ctx, which):
    import torch

    rng = np.random.default_rng(9)
    a = oracle.encode(rng.standard_normal((16, 5632)).astype(np.float32), "f16")
    b = oracle.encode(rng.standard_normal((16, 5632)).astype(np.float32), "f16")
    want = oracle.swiglu(a, b, "f16")
    ta, tb = to_torch(a, "f16"), to_torch(b, "f16")
    tc = ta if which == "a" else tb
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    check(to_codes(tc), want, "f16", f"in place on {which}")


def test_closed_forms(ctx):
    """b = 0 gives 0 for any a; for large b the gate is the identity (c = a*b);
    for very negative b the result vanishes."""
    import torch

    a = oracle.encode(np.array([[1.5, -2.0, 3.0, 0.5, 2.0, -1.0, 1.0, 1.0]], np.float32), "f16")
    b = oracle.encode(np.array([[0.0, -0.0, 30.0, 40.0, -30.0, -100.0, 0.0, 20.0]], np.float32), "f16")
    ta, tb = to_torch(a, "f16"), to_torch(b, "f16")
    tc = torch.empty_like(ta)
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    got = oracle.decode(to_codes(tc), "f16")[0]
    assert got[0] == 0 and got[1] == 0 and got[6] == 0
    assert got[2] == 90.0 and got[3] == 20.0 and got[7] == 20.0
    assert abs(got[4]) < 1e-10 and got[5] == 0


def test_every_fp16_gate_code(ctx):
    """All 65 536 gate codes (subnormals, huge magnitudes, infinities, NaNs)
    against four `up` values: exercises the range test that routes extreme
    gates to the library formula."""
    import torch

    gates = np.arange(65536, dtype=np.uint16)
    for up_value in (1.0, -2.5, 300.0, 6.1e-5):
        b = gates.reshape(64, 1024)
        a = oracle.encode(np.full((64, 1024), up_value, np.float32), "f16")
        tc = torch.empty((64, 1024), dtype=torch.float16, device="cuda")
        ctx.swiglu(tc, to_torch(a, "f16"), to_torch(b, "f16"))
        torch.cuda.synchronize()
        want = oracle.swiglu(a, b, "f16")
        frac, worst = assert_codes_close(to_codes(tc), want, "f16", max_ulp=1, max_frac=2e-3, what=f"all gate codes, up={up_value}")


def test_bf16_extreme_gates(ctx):
    """bf16 gates far outside the lean form's range, both signs, plus inf/NaN."""
    import torch

    gate_values = np.array([88.0, -88.0, 90.0, -90.0, 1e4, -1e4, 3e38, -3e38, np.inf, -np.inf, np.nan, 87.0, -87.0, 86.5, -86.5, 0.0], np.float32)
    b = oracle.encode(np.tile(gate_values, (8, 64)), "bf16")
    a = oracle.encode(np.full(b.shape, 1.25, np.float32), "bf16")
    tc = torch.empty(b.shape, dtype=torch.bfloat16, device="cuda")
    ctx.swiglu(tc, to_torch(a, "bf16"), to_torch(b, "bf16"))
    torch.cuda.synchronize()
    assert_codes_close(to_codes(tc), oracle.swiglu(a, b, "bf16"), "bf16", max_ulp=1, max_frac=0.2, what="bf16 extreme gates")


def test_status_codes_match_reference(ctx):
    import ctypes

    from operators_amd import infiniopSwiGLUDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    for case in golden_json()["status"]:
        if case["op"] != "swiglu":
            continue
        descs = [make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
        d = infiniopSwiGLUDescriptor_t()
        st = lib.infiniopCreateSwiGLUDescriptor(ctx.handle, ctypes.byref(d), *descs)
        want = 0 if case.get("bf16_extension") else case["status"]
        assert st == want, (case, st)
        if st == 0:
            assert lib.infiniopDestroySwiGLUDescriptor(d) == 0
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)
