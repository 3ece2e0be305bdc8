"""The fused Add + RMSNorm on the GPU through the C ABI.

The reference has no such operator: its callers run Add, then RMSNorm on the
sum.  Bars: c is bit-exact against the reference's Add (oracle and compiled
reference agree on it bit for bit); y meets RMSNorm's bar against the oracle's
Add -> RMSNorm (|gpu - ref| <= 1e-3 + 1e-3*|ref| for fp16, 1e-2 for bf16, and at
most one unit in the last place on a bounded share of elements); and both are
bit for bit what this library's own infiniopAdd followed by infiniopRMSNorm
produce."""
import numpy as np
import pytest

import oracle
from helpers import assert_allclose16, assert_codes_close, assert_codes_equal, strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
TOL = {"f16": 1e-3, "bf16": 1e-2}


def inputs(n, d, dt, wdt, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    a = oracle.encode(rng.standard_normal((n, d)).astype(np.float32) * scale, dt)
    b = oracle.encode(rng.standard_normal((n, d)).astype(np.float32) * scale, dt)
    w = oracle.encode(rng.uniform(0.5, 1.5, d).astype(np.float32), wdt)
    return a, b, w


def fused(ctx, a, b, w, eps, dt, wdt):
    import torch

    ta, tb, tw = to_torch(a, dt), to_torch(b, dt), to_torch(w, wdt)
    ty, tc = torch.empty_like(ta), torch.empty_like(ta)
    ctx.add_rms_norm(ty, tc, ta, tb, tw, eps)
    torch.cuda.synchronize()
    return to_codes(tc), to_codes(ty)


def separate(ctx, a, b, w, eps, dt, wdt):
    import torch

    ta, tb, tw = to_torch(a, dt), to_torch(b, dt), to_torch(w, wdt)
    ty, tc = torch.empty_like(ta), torch.empty_like(ta)
    ctx.add(tc, ta, tb)
    ctx.rms_norm(ty, tc, tw, eps)
    torch.cuda.synchronize()
    return to_codes(tc), to_codes(ty)


def check_y(got, want, dt, what, max_frac=5e-3):
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), TOL[dt], TOL[dt], what)
    return assert_codes_close(got, want, dt, max_ulp=1, max_frac=max_frac, what=what)


@pytest.mark.parametrize("dt,wdt", [("f16", "f16"), ("f16", "f32"), ("bf16", "f32"), ("bf16", "bf16")])
@pytest.mark.parametrize("n,d", [(16, 2048), (3, 8), (700, 512), (9, 4096), (1100, 8192), (3, 16384), (2, 65536), (2, 70000), (4, 1023),
                                 # short rows, several to a wavefront (per-head norms), with ragged last wavefronts
                                 (5001, 128), (1003, 64), (777, 256), (333, 72), (50, 200),
                                 # widths of common models on the looping kernels
                                 (600, 5120), (530, 7168), (300, 12288),
                                 # rows whose fp32 weights take more than 64 KiB of LDS, and the first size beyond what LDS holds
                                 (300, 18432), (270, 32768), (265, 40704), (262, 40960),
                                 # the wide-row kernel (from 10 240 elements): 2 to 8 vectors per lane, lane counts that are no power of
                                 # two (11 000: 704 lanes), weights in LDS and from memory, fewer rows than compute units
                                 (520, 10240), (300, 11000), (280, 14336), (290, 16384), (280, 20480), (270, 24576), (264, 36864), (300, 49152),
                                 (258, 65536), (40, 12288)])
def test_against_oracle_and_against_the_two_separate_calls(ctx, dt, wdt, n, d):
    a, b, w = inputs(n, d, dt, wdt, n * 11 + d)
    want_c, want_y = oracle.add_rms_norm(a, b, w, 1e-5, dt, wdt)
    got_c, got_y = fused(ctx, a, b, w, 1e-5, dt, wdt)
    assert_codes_equal(got_c, want_c, dt, what=f"c [{n},{d}] {dt}")
    check_y(got_y, want_y, dt, f"y [{n},{d}] {dt} w {wdt}", max_frac=5e-3 if d <= 16384 else 3e-2)
    sep_c, sep_y = separate(ctx, a, b, w, 1e-5, dt, wdt)
    assert np.array_equal(got_c, sep_c) and np.array_equal(got_y, sep_y), "fused and separate calls differ"


def test_fp16_sums_that_overflow_or_cancel(ctx):
    """Large addends: sums beyond the fp16 range follow the reference's
    conversion (its unguarded overflow pattern) in c; rows holding such values
    are compared in c only, the rest in y too."""
    a, b, w = inputs(64, 4096, "f16", "f32", 5, scale=20000.0)
    a[1::2], b[1::2], _ = inputs(32, 4096, "f16", "f32", 6)  # ordinary rows in between
    b[3] = a[3] ^ 0x8000  # a row that cancels exactly: c = 0, y = 0
    want_c, want_y = oracle.add_rms_norm(a, b, w, 1e-5, "f16", "f32")
    got_c, got_y = fused(ctx, a, b, w, 1e-5, "f16", "f32")
    assert_codes_equal(got_c, want_c, "f16", what="c with overflowing sums")
    check_y(got_y[1::2], want_y[1::2], "f16", "y of the ordinary rows")
    assert not got_y[3].astype(np.uint16).any() or set(np.unique(got_y[3])) <= {0, 0x8000}


def test_residual_updated_in_place_and_strided_rows(ctx):
    """c is a (the residual stream), rows of every tensor have their own stride."""
    import torch

    n, d = 200, 4096
    a, b, w = inputs(n, d, "bf16", "f32", 9)
    want_c, want_y = oracle.add_rms_norm(a, b, w, 1e-6, "bf16", "f32")
    ta = strided_like(a, (n, d), (d + 64, 1), "bf16")[0]
    tb = strided_like(b, (n, d), (2 * d, 1), "bf16")[0]
    ty = strided_like(np.zeros((n, d), np.uint16), (n, d), (d + 8, 1), "bf16")[0]
    tw = to_torch(w, "f32")
    ctx.add_rms_norm(ty, ta, ta, tb, tw, 1e-6)
    torch.cuda.synchronize()
    assert_codes_equal(to_codes(ta), want_c, "bf16", what="c written over a")
    check_y(to_codes(ty), want_y, "bf16", "y, strided")


def test_large_residual_stream(ctx):
    """[8192, 8192] bf16 with fp32 weights: the benchmark shape (write-through stores)."""
    import torch

    n, d = 8192, 8192
    gen = torch.Generator(device="cuda")
    gen.manual_seed(3)
    ta = torch.randn((n, d), device="cuda", dtype=torch.float32, generator=gen).to(torch.bfloat16)
    tb = torch.randn((n, d), device="cuda", dtype=torch.float32, generator=gen).to(torch.bfloat16)
    tw = torch.rand(d, device="cuda", dtype=torch.float32, generator=gen) + 0.5
    ty, tc = torch.empty_like(ta), torch.empty_like(ta)
    ctx.add_rms_norm(ty, tc, ta, tb, tw, 1e-5)
    ty2, tc2 = torch.empty_like(ta), torch.empty_like(ta)
    ctx.add(tc2, ta, tb)
    ctx.rms_norm(ty2, tc2, tw, 1e-5)
    torch.cuda.synchronize()
    assert torch.equal(tc.view(torch.int16), tc2.view(torch.int16)) and torch.equal(ty.view(torch.int16), ty2.view(torch.int16))
    rows = slice(4000, 4064)  # and a band of rows against the CPU oracle
    a, b, w = to_codes(ta[rows]), to_codes(tb[rows]), tw.cpu().numpy()
    want_c, want_y = oracle.add_rms_norm(a, b, w, 1e-5, "bf16", "f32")
    assert_codes_equal(to_codes(tc[rows]), want_c, "bf16", what="c band")
    check_y(to_codes(ty[rows]), want_y, "bf16", "y band")


def test_status_codes(ctx):
    """Create-time checks: shapes, inner strides, mixed element types."""
    import torch

    from operators_amd import InfiniopError
    from operators_amd.ops import AddRMSNormPlan

    f16 = torch.float16
    mk = lambda *shape, dtype=f16: torch.zeros(shape, dtype=dtype, device="cuda")  # noqa: E731
    y, c, a, b, w = mk(4, 64), mk(4, 64), mk(4, 64), mk(4, 64), mk(64)
    AddRMSNormPlan(ctx, y, c, a, b, w, 1e-5).close()
    for bad, code in [((y, c, a, mk(4, 32), w), 4), ((y, c, a, b, mk(32)), 4), ((y, c, mk(64), b, w), 4),
                      ((y, c, a, mk(4, 128)[:, ::2], w), 5)]:
        with pytest.raises(InfiniopError) as err:
            AddRMSNormPlan(ctx, *bad, 1e-5)
        assert err.value.status == code, (err.value.status, code)
    # mixed element types: created, refused at compute time like RMSNorm does
    plan = AddRMSNormPlan(ctx, y, c, a, mk(4, 64, dtype=torch.bfloat16), w, 1e-5)
    with pytest.raises(InfiniopError) as err:
        plan(y, c, a, mk(4, 64, dtype=torch.bfloat16), w)
    assert err.value.status == 3
    plan.close()
