"""RMSNorm on the GPU through the C ABI, against the oracle and the
reference's golden vectors.  Bar (fp16): |gpu - ref| <= 1e-3 + 1e-3*|ref|; the
sum of squares is a tree on the GPU and a running sum on the CPU, so a few
elements in 10^4 differ by one unit in the last place.  bf16: 1e-2."""
import numpy as np
import pytest

import oracle
from helpers import assert_allclose16, assert_codes_close, golden, golden_json, strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
TOL = {"f16": 1e-3, "bf16": 1e-2}


def run(ctx, x, w, eps, dt, wdt, x_stride=None, y_stride=None):
    import torch

    n, d = x.shape
    tx = strided_like(x, x.shape, (x_stride, 1), dt)[0] if x_stride else to_torch(x, dt)
    tw = to_torch(w, wdt)
    if y_stride:
        ty = strided_like(np.zeros(x.shape, np.uint16), x.shape, (y_stride, 1), dt)[0]
    else:
        ty = torch.empty((n, d), dtype=tx.dtype, device="cuda")
    ctx.rms_norm(ty, tx, tw, eps)
    torch.cuda.synchronize()
    return to_codes(ty)


def check(got, want, dt, what, max_frac=5e-3):
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), TOL[dt], TOL[dt], what)
    return assert_codes_close(got, want, dt, max_ulp=1, max_frac=max_frac, what=what)


def test_golden_first_config(ctx):
    g = golden("rms_norm")
    check(run(ctx, g["rms0_x"], g["rms0_w16"], 1e-5, "f16", "f16"), g["rms0_y_w16"], "f16", "[16,2048] w f16")
    check(run(ctx, g["rms0_x"], g["rms0_w32"], 1e-5, "f16", "f32"), g["rms0_y_w32"], "f16", "[16,2048] w f32")


def test_golden_odd_sizes(ctx):
    g = golden("rms_norm")
    for i in range(1, 5):
        x, w, want = g[f"rms{i}_x"], g[f"rms{i}_w32"], g[f"rms{i}_y_w32"]
        check(run(ctx, x, w, 1e-6, "f16", "f32"), want, "f16", f"golden rms case {i} {x.shape}", max_frac=2e-2)


@pytest.mark.parametrize("dt,wdt", [("f16", "f16"), ("f16", "f32"), ("bf16", "f32"), ("bf16", "bf16")])
@pytest.mark.parametrize("n,d", [(16, 2048), (3, 8), (700, 512), (9, 4096), (5, 8192), (1100, 8192), (3, 16384), (2, 32768), (2, 65536), (2, 70000), (4, 1023),
                                 # widths of common models, more rows than workgroups (the looping kernels with their exact launch shapes)
                                 (1100, 5120), (1030, 6144), (600, 7168), (520, 10240), (300, 12288), (290, 14336), (280, 16384),
                                 # other multiples of 512 (the kernel whose lane count is the launch's): 576 x 1, 576 x 2, 704 x 2, 832 x 1 lanes x vectors
                                 (1100, 4608), (300, 9216), (280, 11264), (290, 6656),
                                 # and two of them with an output large enough to be written through L2
                                 (5600, 6144), (4700, 7168),
                                 # rows whose fp32 weights take more than 64 KiB of LDS (up to 160 KiB per workgroup), and the first size beyond
                                 (300, 18432), (290, 20480), (280, 24576), (270, 32768), (265, 40704), (262, 40960),
                                 # the wide-row kernel, 5 to 8 vectors per lane: weights in LDS (33 000: 832 lanes), from memory in batches, few rows
                                 (270, 33000), (264, 36864), (300, 49152), (260, 57344), (258, 65536), (40, 49152),
                                 # short rows, several to a wavefront (per-head norms): full and ragged last wavefronts, rows that
                                 # do not fill their lanes, an output large enough to be written through L2
                                 (5001, 128), (4096, 128), (1003, 64), (777, 256), (333, 72), (101, 16), (50, 200), (270000, 128),
                                 # rows that leave a quarter and more of their lanes idle: two groups of rows per turn of a wavefront
                                 # (one, odd and large row counts; 320 and 384: two rows per one-wavefront workgroup)
                                 (1001, 80), (7, 96), (1, 160), (5, 192), (9, 24), (430000, 80), (1003, 320), (3, 384), (1, 320)])
def test_against_oracle(ctx, dt, wdt, n, d):
    rng = np.random.default_rng(n * 7 + d)
    x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    w = oracle.encode(rng.uniform(0.5, 1.5, d).astype(np.float32), wdt)
    want = oracle.rms_norm(x, w, 1e-5, dt, wdt)
    # The CPU adds d squares one after the other in fp32, so its sum carries an
    # error that grows with d; the GPU's tree sum does not.  The share of
    # outputs that land on the other side of a rounding boundary grows with it.
    check(run(ctx, x, w, 1e-5, dt, wdt), want, dt, f"[{n},{d}] {dt} w {wdt}", max_frac=5e-3 if d <= 16384 else 3e-2)


def test_row_strides_of_x_and_y_are_independent(ctx):
    """x rows 4096 apart, y rows 2304 apart: x's stride comes from x's descriptor."""
    rng = np.random.default_rng(21)
    x = oracle.encode(rng.standard_normal((12, 2048)).astype(np.float32), "f16")
    w = oracle.encode(rng.uniform(0.5, 1.5, 2048).astype(np.float32), "f32")
    want = oracle.rms_norm(x, w, 1e-5, "f16", "f32")
    check(run(ctx, x, w, 1e-5, "f16", "f32", x_stride=4096, y_stride=2304), want, "f16", "strided rows")
    check(run(ctx, x, w, 1e-5, "f16", "f32", x_stride=2049, y_stride=2051), want, "f16", "odd row strides")
    # short rows (several to a wavefront): one head of 128 out of every 640 elements, written 256 apart
    x = oracle.encode(rng.standard_normal((1001, 128)).astype(np.float32), "bf16")
    w = oracle.encode(rng.uniform(0.5, 1.5, 128).astype(np.float32), "f32")
    want = oracle.rms_norm(x, w, 1e-6, "bf16", "f32")
    check(run(ctx, x, w, 1e-6, "bf16", "f32", x_stride=640, y_stride=256), want, "bf16", "strided short rows")
    # and with two groups of rows per turn: heads of 80 out of every 400 elements, written 88 apart
    x = oracle.encode(rng.standard_normal((1003, 80)).astype(np.float32), "f16")
    w = oracle.encode(rng.uniform(0.5, 1.5, 80).astype(np.float32), "f16")
    want = oracle.rms_norm(x, w, 1e-6, "f16", "f16")
    check(run(ctx, x, w, 1e-6, "f16", "f16", x_stride=400, y_stride=88), want, "f16", "strided short rows, two groups per turn")


def test_in_place(ctx):
    import torch

    rng = np.random.default_rng(22)
    x = oracle.encode(rng.standard_normal((300, 4096)).astype(np.float32), "f16")
    w = oracle.encode(rng.uniform(0.5, 1.5, 4096).astype(np.float32), "f16")
    want = oracle.rms_norm(x, w, 1e-5, "f16", "f16")
    tx, tw = to_torch(x, "f16"), to_torch(w, "f16")
    ctx.rms_norm(tx, tx, tw, 1e-5)
    torch.cuda.synchronize()
    check(to_codes(tx), want, "f16", "in place")


def test_constant_rows_closed_form(ctx):
    """A row of constants c with w = 1 normalises to c / sqrt(c^2 + eps)."""
    for c in (0.5, -3.0, 100.0):
        x = oracle.encode(np.full((4, 1024), c, np.float32), "f16")
        w = np.ones(1024, np.float32)
        got = oracle.decode(run(ctx, x, w, 1e-5, "f16", "f32"), "f16")
        exact = c / np.sqrt(np.float64(c) ** 2 + 1e-5)
        assert np.all(np.abs(got - exact) <= 2.0 ** -10 * abs(exact)), (c, got[0, 0], exact)
    zeros = run(ctx, np.zeros((2, 64), np.uint16), np.ones(64, np.float32), 1e-5, "f16", "f32")
    assert not zeros.any()


def test_status_codes_match_reference(ctx):
    """Create-stage statuses recorded from the compiled reference; where the
    reference defers its dtype check to the compute call, so does this library."""
    import ctypes

    import torch

    from operators_amd import infiniopRMSNormDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    scratch = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    for case in golden_json()["status"]:
        if case["op"] != "rms_norm":
            continue
        descs = [make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
        d = infiniopRMSNormDescriptor_t()
        st = lib.infiniopCreateRMSNormDescriptor(ctx.handle, ctypes.byref(d), *descs, 1e-5)
        if st == 0:
            if case.get("run"):
                p = scratch.data_ptr()
                st = lib.infiniopRMSNorm(d, None, 0, p, p + (1 << 14), p + (1 << 15), None)
                torch.cuda.synchronize()
            assert lib.infiniopDestroyRMSNormDescriptor(d) == 0
        want = 0 if case.get("bf16_extension") else case["status"]
        assert st == want, (case, st)
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)
