"""Add on the GPU through the C ABI, against the oracle and the reference's
golden vectors.  Bar: bit-exact (a generated NaN may differ in sign only)."""
import json

import numpy as np
import pytest

import oracle
from helpers import assert_codes_equal, golden, golden_json, to_codes, to_torch

pytestmark = pytest.mark.gpu


def run_add(ctx, a, b, c_shape, dtype):
    import torch

    ta, tb = to_torch(a, dtype).reshape(a.shape), to_torch(b, dtype).reshape(b.shape)
    tc = torch.empty(tuple(c_shape), dtype=ta.dtype, device="cuda")
    ctx.add(tc, ta, tb)
    torch.cuda.synchronize()
    return to_codes(tc).reshape(c_shape)


def check(got, want, dtype, what):
    if dtype == "f32":
        g, w = got.view(np.uint32), want.view(np.uint32)
        nan = np.isnan(want)
        assert np.array_equal(np.isnan(got), nan), what
        assert np.array_equal(g[~nan], w[~nan]), what
    else:
        assert_codes_equal(got, want, dtype, what=what)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_golden_cases(ctx, dt):
    g = golden("add")
    cases = golden_json()["add_cases"]
    for i, (cs, as_, bs) in enumerate(cases):
        a, b, want = g[f"add{i}_{dt}_a"], g[f"add{i}_{dt}_b"], g[f"add{i}_{dt}_c"]
        got = run_add(ctx, a.reshape(as_), b.reshape(bs), tuple(cs), dt)
        check(got, want.reshape(cs), dt, f"golden add case {i} {cs} = {as_} + {bs} {dt}")


def test_golden_all_codes_plus_zero(ctx):
    g = golden("add")
    codes = np.arange(65536, dtype=np.uint16)
    got = run_add(ctx, codes, np.zeros(65536, np.uint16), (65536,), "f16")
    assert_codes_equal(got, g["add_all_codes_plus_zero"], "f16", nan_sign_free=False, what="x + 0")


def test_golden_table_block(ctx):
    g = golden("add")
    rows, cols = g["add_table_rows"], g["add_table_cols"]
    got = run_add(ctx, rows.reshape(-1, 1), cols, (rows.size, cols.size), "f16")
    assert_codes_equal(got, g["add_table_c"], "f16", what="fp16 addition table block")


SHAPES = [
    # c, a, b
    ((1000003,), (1000003,), (1000003,)),           # flat, odd length: vector body + tail
    ((257, 4096), (257, 4096), (4096,)),            # residual-style leading broadcast
    ((6, 5, 40), (6, 1, 40), (1, 5, 1)),            # both operands broadcast, along different dims
    ((7, 33, 16), (7, 1, 16), (33, 1)),             # alternating broadcast, inner vectorisable
    ((7, 33, 15), (7, 1, 15), (33, 1)),             # same with an odd inner extent: element path
    ((5, 6, 7, 8), (5, 6, 7, 8), (1,)),             # scalar-like operand
    ((3, 64, 64), (64,), (3, 64, 1)),               # a broadcast along leading dims, b along inner
    ((2, 3, 4, 5, 6, 8), (2, 1, 4, 1, 6, 8), (3, 1, 5, 1, 8)),  # six merged dims
    # a whole tensor plus an operand broadcast along outer dimensions only, rows of whole wavefronts of vectors (the tiled form):
    ((3, 5, 512), (3, 5, 512), (3, 1, 512)),        # a bias per batch entry
    ((3, 5, 1024), (3, 1, 1024), (3, 5, 1024)),     # the same with the operands swapped, two tiles per row
    ((2, 3, 4, 512), (2, 3, 4, 512), (2, 1, 4, 512)),  # an attention mask: the inner two dimensions merge
    ((2, 3, 4, 512), (2, 3, 4, 512), (1, 3, 1, 512)),  # broadcast along two separate outer dimensions
    ((2, 3, 2, 2, 3, 512), (2, 3, 2, 2, 3, 512), (2, 1, 2, 1, 3, 512)),  # and along alternating ones
    ((70, 600, 512), (70, 600, 512), (70, 1, 512)), # large enough to be written through L2
]


@pytest.mark.parametrize("dt", ["f16", "f32", "bf16"])
@pytest.mark.parametrize("case", range(len(SHAPES)))
def test_against_oracle(ctx, dt, case):
    cs, as_, bs = SHAPES[case]
    spec = lambda s: oracle.Spec(dt, s)  # noqa: E731
    assert oracle.add_check(spec(cs), spec(as_), spec(bs), allow_bf16=True) == 0, "every triple of SHAPES is a valid broadcast"
    rng = np.random.default_rng(100 + case)
    a = oracle.encode(rng.standard_normal(as_).astype(np.float32) * 3, dt)
    b = oracle.encode(rng.standard_normal(bs).astype(np.float32) * 3, dt)
    want = oracle.add(a, b, cs, dt)
    got = run_add(ctx, a, b, cs, dt)
    check(got, want, dt, f"{cs} = {as_} + {bs} {dt}")


@pytest.mark.parametrize("which", ["a", "b"])
def test_in_place(ctx, which):
    import torch

    rng = np.random.default_rng(5)
    a = oracle.encode(rng.standard_normal((32, 20, 512)).astype(np.float32), "f16")
    b = oracle.encode(rng.standard_normal((32, 20, 512)).astype(np.float32), "f16")
    want = oracle.add(a, b, a.shape, "f16")
    ta, tb = to_torch(a, "f16"), to_torch(b, "f16")
    tc = ta if which == "a" else tb
    ctx.add(tc, ta, tb)
    torch.cuda.synchronize()
    assert_codes_equal(to_codes(tc), want, "f16", what=f"in place on {which}")


@pytest.mark.parametrize("n", [5, 5000, 5003, 1 << 20])
def test_misaligned_pointers(ctx, n):
    """Operands that start on different 2-byte boundaries: the same vectors as 16-byte accesses at those
    boundaries, the last few elements one by one; what lies in front of and behind c stays."""
    import torch

    rng = np.random.default_rng(6)
    a = oracle.encode(rng.standard_normal(n + 3).astype(np.float32), "f16")
    b = oracle.encode(rng.standard_normal(n + 5).astype(np.float32), "f16")
    ta, tb = to_torch(a, "f16")[3:], to_torch(b, "f16")[5:]  # 2-byte aligned only
    whole = torch.full((n + 2,), 7.0, dtype=torch.float16, device="cuda")
    tc = whole[1:n + 1]
    ctx.add(tc, ta, tb)
    torch.cuda.synchronize()
    assert_codes_equal(to_codes(tc), oracle.add(a[3:].copy(), b[5:].copy(), (n,), "f16"), "f16", what="misaligned")
    assert whole[0] == 7.0 and whole[n + 1] == 7.0


def test_more_than_2_to_31_elements_uses_64_bit_indexing(ctx):
    """c = [2, 2^14 + 1, 2^16] (just over 2^31 elements, 4 GiB of bf16) from
    a = [2, 1, 2^16] and b = [2^14 + 1, 1]: three merged dimensions, so the
    general broadcast kernel runs with 64-bit index arithmetic.  bf16 add is
    exactly torch's, so the check runs on the GPU."""
    import torch

    d0, d1, d2 = 2, (1 << 14) + 1, 1 << 16
    g = torch.Generator(device="cuda")
    g.manual_seed(7)
    a = torch.randn((d0, 1, d2), generator=g, device="cuda").to(torch.bfloat16)
    b = torch.randn((d1, 1), generator=g, device="cuda").to(torch.bfloat16)
    c = torch.empty((d0, d1, d2), dtype=torch.bfloat16, device="cuda")
    ctx.add(c, a, b)
    torch.cuda.synchronize()
    for i in range(d0):
        for r0 in range(0, d1, 4096):  # compare in slabs to bound memory
            want = a[i] + b[r0:r0 + 4096]
            assert torch.equal(c[i, r0:r0 + 4096].view(torch.int16), want.view(torch.int16)), (i, r0)
    del c
    # the flat kernel over the same count
    x = torch.randn((d0 * d1 * d2 // 4,), generator=g, device="cuda").to(torch.bfloat16).repeat(4)
    y = torch.empty_like(x)
    ctx.add(y, x, x)
    torch.cuda.synchronize()
    assert torch.equal(y.view(torch.int16), (x + x).view(torch.int16))


def test_empty_tensor_is_a_no_op(ctx):
    import torch

    t = torch.empty((0, 8), dtype=torch.float16, device="cuda")
    ctx.add(t, t, t)
    torch.cuda.synchronize()


def test_special_values_against_oracle(ctx):
    """Every finite/infinite/NaN class against every other, both signs."""
    specials = np.array([0x0000, 0x8000, 0x0001, 0x8001, 0x03FF, 0x0400, 0x3C00, 0xBC00, 0x7BFF, 0xFBFF,
                         0x7C00, 0xFC00, 0x7E00, 0xFE00, 0x7C01, 0x7BFE, 0x7800, 0xF800], dtype=np.uint16)
    a = np.repeat(specials, specials.size).reshape(specials.size, specials.size)
    b = np.ascontiguousarray(a.T)
    want = oracle.add(a, b, a.shape, "f16")
    got = run_add(ctx, a, b, a.shape, "f16")
    assert_codes_equal(got, want, "f16", what="special values")


def test_status_codes_match_reference(ctx):
    """Create-time statuses recorded from the compiled reference."""
    import ctypes

    from operators_amd import infiniopAddDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    for case in golden_json()["status"]:
        if case["op"] != "add":
            continue
        descs = [make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
        d = infiniopAddDescriptor_t()
        st = lib.infiniopCreateAddDescriptor(ctx.handle, ctypes.byref(d), *descs)
        want = 0 if case.get("bf16_extension") else case["status"]
        assert st == want, (case, st)
        if st == 0:
            assert lib.infiniopDestroyAddDescriptor(d) == 0
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)
