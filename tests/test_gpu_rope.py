"""RoPE on the GPU through the C ABI, against the oracle and the reference's
golden vectors.  Only IEEE multiply/add and the reference's narrowing are
involved, so the bar is bit-exact for fp16 and for bf16."""
import numpy as np
import pytest

import oracle
from helpers import assert_codes_equal, golden, golden_json, strided_like, to_codes, to_torch
from operators_amd.ops import sin_cos_table

pytestmark = pytest.mark.gpu


def run(ctx, t_codes, shape, strides, pos, sin_t, cos_t, dt):
    """Returns (rotated values, whole buffer before, whole buffer after)."""
    import torch

    if strides is None:
        tt = to_torch(t_codes, dt).reshape(shape)
        buf = tt
    else:
        tt, buf = strided_like(t_codes, shape, strides, dt)
    before = to_codes(buf)
    tpos = torch.from_numpy(np.asarray(pos, np.uint64).view(np.int64).copy()).cuda().view(torch.uint64)
    ts, tc = torch.from_numpy(sin_t).cuda(), torch.from_numpy(cos_t).cuda()
    ctx.rope(tt, tpos, ts, tc)
    torch.cuda.synchronize()
    return to_codes(tt), before, to_codes(buf)


def test_golden_cases(ctx):
    g = golden("rope")
    for i, (shape, strides, rows) in enumerate(golden_json()["rope_cases"]):
        got, before, after = run(ctx, g[f"rope{i}_t_in"], shape, strides, g[f"rope{i}_pos"], g[f"rope{i}_sin"], g[f"rope{i}_cos"], "f16")
        assert_codes_equal(got, g[f"rope{i}_t_out"], "f16", what=f"golden rope case {i} {shape} {strides}")
        if strides is not None:  # everything outside the view is untouched
            mask = np.ones(before.size, bool)
            idx = np.add.outer(np.add.outer(np.arange(shape[0]) * strides[0], np.arange(shape[1]) * strides[1]), np.arange(shape[2]))
            mask[idx.ravel()] = False
            assert np.array_equal(before[mask], after[mask])


CASES = [
    # shape, strides, table rows
    ((1, 32, 128), None, 64), ((4, 1, 32), None, 64), ((3, 32, 128), (8000, 200, 1), 64),
    ((129, 32, 128), (96 * 128, 128, 1), 4096),  # q heads of a fused qkv buffer
    ((130, 8, 128), (80 * 128, 128, 1), 4096),   # 8 kv heads: several tokens per workgroup
    ((33, 3, 64), None, 100),                    # head count not a multiple of the per-lane head loop
    ((9, 5, 200), None, 50),                     # head_dim/8 not a power of two
    ((7, 5, 6), None, 40), ((5, 2, 2), None, 9), # head_dim not a multiple of 8: pair path
    ((6, 4, 64), (4 * 64 + 3, 65, 1), 30),       # odd strides: pair path
]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_against_oracle(ctx, dt, case):
    shape, strides, rows = CASES[case]
    rng = np.random.default_rng(300 + case)
    t = oracle.encode(rng.standard_normal(shape).astype(np.float32), dt)
    pos = rng.integers(0, rows, shape[0]).astype(np.uint64)
    # independent entries everywhere: the four table reads of a pair all matter
    sin_t = rng.uniform(-1, 1, (rows, shape[2])).astype(np.float32)
    cos_t = rng.uniform(-1, 1, (rows, shape[2])).astype(np.float32)
    want = oracle.rope(t.copy(), pos, sin_t, cos_t, dt)
    got, _, _ = run(ctx, t, shape, strides, pos, sin_t, cos_t, dt)
    assert_codes_equal(got, want, dt, what=f"{shape} {strides} {dt}")


def test_position_zero_is_identity_and_norm_is_preserved(ctx):
    rng = np.random.default_rng(31)
    shape = (64, 8, 128)
    t = oracle.encode(rng.standard_normal(shape).astype(np.float32), "f16")
    sin_t, cos_t = (x.numpy() for x in sin_cos_table(512, 128, 1e4))
    same, _, _ = run(ctx, t, shape, None, np.zeros(64, np.uint64), sin_t, cos_t, "f16")
    assert np.array_equal(same, t)  # sin 0 = 0, cos 0 = 1: exact
    pos = rng.integers(1, 512, 64).astype(np.uint64)
    rot, _, _ = run(ctx, t, shape, None, pos, sin_t, cos_t, "f16")
    a, b = oracle.decode(t, "f16").astype(np.float64), oracle.decode(rot, "f16").astype(np.float64)
    na = np.hypot(a[..., 0::2], a[..., 1::2])
    nb = np.hypot(b[..., 0::2], b[..., 1::2])
    assert np.all(np.abs(na - nb) <= 2.5e-3 * np.maximum(na, 1e-3) + 2e-7)  # two truncations to fp16


def test_matches_complex_rotation(ctx):
    """The reference harness's own criterion: multiply pairs, seen as complex
    numbers, by exp(i*pos*freq) (atol 1e-4, rtol 1e-2)."""
    rng = np.random.default_rng(32)
    shape, theta = (16, 4, 64), 1e4
    vals = rng.random(shape).astype(np.float32)
    t = oracle.encode(vals, "f16")
    pos = np.arange(16, dtype=np.uint64)
    sin_t, cos_t = (x.numpy() for x in sin_cos_table(32, 64, theta))
    got, _, _ = run(ctx, t, shape, None, pos, sin_t, cos_t, "f16")
    v = oracle.decode(t, "f16").astype(np.float64)
    freqs = 1.0 / theta ** (np.arange(0, 64, 2) / 64)
    z = (v[..., 0::2] + 1j * v[..., 1::2]) * np.exp(1j * np.outer(np.arange(16), freqs))[:, None, :]
    want = np.stack([z.real, z.imag], -1).reshape(shape)
    g = oracle.decode(got, "f16")
    assert np.all(np.abs(g - want) <= 1e-4 + 1e-2 * np.abs(want))


def test_null_pointers_are_bad_param(ctx):
    import ctypes

    import torch

    from operators_amd.ops import RoPEPlan

    t = torch.zeros((2, 2, 8), dtype=torch.float16, device="cuda")
    pos = torch.zeros(2, dtype=torch.int64, device="cuda").view(torch.uint64)
    s = torch.zeros((4, 8), dtype=torch.float32, device="cuda")
    with RoPEPlan(ctx, t, pos, s, s) as plan:
        for args in [(None, pos.data_ptr(), s.data_ptr(), s.data_ptr()), (t.data_ptr(), None, s.data_ptr(), s.data_ptr()),
                     (t.data_ptr(), pos.data_ptr(), None, s.data_ptr()), (t.data_ptr(), pos.data_ptr(), s.data_ptr(), None)]:
            assert ctx.lib.infiniopRoPE(plan.desc, None, 0, *args, None) == 2
    assert ctx.lib.infiniopCreateRoPEDescriptor(ctx.handle, None, *[None] * 4) == 2
    _ = ctypes


def test_status_codes_match_reference(ctx):
    import ctypes

    from operators_amd import infiniopRoPEDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    for case in golden_json()["status"]:
        if case["op"] != "rope":
            continue
        descs = [make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
        d = infiniopRoPEDescriptor_t()
        st = lib.infiniopCreateRoPEDescriptor(ctx.handle, ctypes.byref(d), *descs)
        want = 0 if case.get("bf16_extension") else case["status"]
        assert st == want, (case, st)
        if st == 0:
            assert lib.infiniopDestroyRoPEDescriptor(d) == 0
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)
