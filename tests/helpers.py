"""Shared pieces of the test suite: fixtures on disk, code-level comparisons,
numpy <-> torch plumbing for 16-bit floating point storage."""
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def golden(name):
    return np.load(os.path.join(GOLDEN, name + ".npz"))


def golden_json():
    import json

    with open(os.path.join(GOLDEN, "status_cases.json")) as f:
        return json.load(f)


def ordered(codes):
    """Map 16-bit sign-magnitude float codes to integers that increase with the
    value, so that a difference of 1 is one unit in the last place."""
    c = codes.astype(np.int32)
    return np.where(c & 0x8000, -(c & 0x7FFF), c & 0x7FFF)


def is_nan16(codes, dtype):
    c = codes.astype(np.uint32) & 0x7FFF
    return c > (0x7C00 if dtype == "f16" else 0x7F80)


def ulp_report(got, want, dtype="f16"):
    """(fraction of differing elements, largest difference in ulps); NaN
    positions must coincide and are otherwise ignored."""
    got, want = np.asarray(got).ravel(), np.asarray(want).ravel()
    ng, nw = is_nan16(got, dtype), is_nan16(want, dtype)
    assert np.array_equal(ng, nw), "NaN positions differ"
    d = np.abs(ordered(got) - ordered(want))
    d[nw] = 0
    return float((d != 0).mean()) if d.size else 0.0, int(d.max()) if d.size else 0


def assert_codes_equal(got, want, dtype="f16", nan_sign_free=True, what=""):
    """Bit-exact comparison of 16-bit codes.  With nan_sign_free, a NaN result
    must be a NaN with the same payload but may differ in sign (the sign of a
    generated NaN is a property of the host FPU, not of the algorithm)."""
    got, want = np.asarray(got), np.asarray(want)
    assert got.shape == want.shape, (got.shape, want.shape)
    if nan_sign_free:
        nanmask = is_nan16(want, dtype)
        g = np.where(nanmask, got & 0x7FFF, got)
        w = np.where(nanmask, want & 0x7FFF, want)
    else:
        g, w = got, want
    bad = np.flatnonzero(g.ravel() != w.ravel())
    if bad.size:
        i = bad[0]
        raise AssertionError(f"{what}: {bad.size} of {g.size} codes differ; first at {i}: got 0x{int(got.ravel()[i]):04x} want 0x{int(want.ravel()[i]):04x}")


def assert_codes_close(got, want, dtype, max_ulp=1, max_frac=2e-3, what=""):
    """For results that depend on libm / summation order: every element within
    max_ulp units in the last place and at most max_frac of them different."""
    frac, worst = ulp_report(got, want, dtype)
    assert worst <= max_ulp and frac <= max_frac, f"{what}: {frac:.2e} of elements differ, worst {worst} ulp"
    return frac, worst


def assert_allclose16(got_f32, want_f32, atol, rtol, what=""):
    """The reference harness's criterion: |got - want| <= atol + rtol*|want|."""
    got_f32, want_f32 = np.asarray(got_f32, np.float64), np.asarray(want_f32, np.float64)
    finite = np.isfinite(want_f32)
    assert np.array_equal(np.isfinite(got_f32), finite), f"{what}: finiteness differs"
    err = np.abs(got_f32[finite] - want_f32[finite])
    lim = atol + rtol * np.abs(want_f32[finite])
    assert (err <= lim).all(), f"{what}: max excess {(err - lim).max():.3e}"


# ---- torch plumbing -----------------------------------------------------------
def torch_dtype(dtype):
    import torch

    return {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32}[dtype]


def to_torch(codes, dtype, device="cuda"):
    """numpy storage array (uint16 codes, or float32) -> torch tensor on device."""
    import torch

    arr = np.ascontiguousarray(codes)
    if dtype == "f32":
        return torch.from_numpy(arr.astype(np.float32)).to(device)
    return torch.from_numpy(arr.view(np.int16)).to(device).view(torch_dtype(dtype))


def to_codes(tensor):
    """torch tensor -> numpy storage array (uint16 codes for 16-bit types)."""
    import torch

    t = tensor.detach().contiguous().cpu()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.numpy().copy()


def strided_like(values_codes, shape, strides, dtype, device="cuda", fill_seed=1234):
    """A torch tensor of `shape`/`strides` (elements) on device holding the
    given codes, inside a buffer whose gaps hold random data.  Returns
    (view, whole buffer)."""
    import torch

    span = 1 + sum((n - 1) * s for n, s in zip(shape, strides))
    rng = np.random.default_rng(fill_seed)
    buf_np = rng.integers(0, 0x3C00, span, dtype=np.uint16)  # finite positive fp16/bf16 codes
    buf = to_torch(buf_np, dtype, device)
    view = torch.as_strided(buf, tuple(shape), tuple(strides))
    view.copy_(to_torch(values_codes, dtype, device).reshape(tuple(shape)))
    return view, buf
