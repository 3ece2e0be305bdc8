"""The benchmark's configurations at their full sizes, through the C ABI, each
compared element for element with the CPU oracle on the same seeded inputs,
plus size-independent properties (identities, equivalence of layouts,
untouched neighbours).  fp16 bars: Add and RoPE bit-exact; RMSNorm and SwiGLU
|gpu - ref| <= 1e-3 + 1e-3*|ref| and at most one unit in the last place.
bf16 (this project's extension of the reference): Add and RoPE bit-exact
against the extended oracle, RMSNorm and SwiGLU within 1e-2."""
import numpy as np
import pytest

import oracle
from helpers import assert_allclose16, assert_codes_close, assert_codes_equal, to_codes
from operators_amd.ops import sin_cos_table

pytestmark = pytest.mark.gpu


def randn(shape, dtype, seed, scale=1.0):
    """Seeded N(0, scale^2) tensor on the GPU (the same bytes go to the oracle)."""
    import torch

    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return (torch.randn(shape, generator=g, device="cuda", dtype=torch.float32) * scale).to(dtype)


def close16(got, want, dt, what, max_frac):
    tol = 1e-3 if dt == "f16" else 1e-2
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), tol, tol, what)
    return assert_codes_close(got, want, dt, max_ulp=1, max_frac=max_frac, what=what)


def test_c1_rms_norm_f16_16x2048(ctx):
    import torch

    x = randn((16, 2048), torch.float16, 0)
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    for wdt, tdt in (("f16", torch.float16), ("f32", torch.float32)):
        w = (torch.rand(2048, generator=g, device="cuda") + 0.5).to(tdt)
        y = torch.empty_like(x)
        ctx.rms_norm(y, x, w, 1e-5)
        torch.cuda.synchronize()
        want = oracle.rms_norm(to_codes(x), to_codes(w), 1e-5, "f16", wdt)
        close16(to_codes(y), want, "f16", f"C1 w {wdt}", 2e-3)


def test_c2_swiglu_f16_4096x11008_contiguous_and_fused(ctx):
    import torch

    n, di = 4096, 11008
    gate_up = randn((n, 2 * di), torch.float16, 2)
    b, a = gate_up[:, :di], gate_up[:, di:]          # gate first, up second: the layout of the reference's MLP
    c_fused = torch.empty((n, di), dtype=torch.float16, device="cuda")
    ctx.swiglu(c_fused, a, b)
    ac, bc = a.contiguous(), b.contiguous()
    c_dense = torch.empty_like(c_fused)
    ctx.swiglu(c_dense, ac, bc)
    torch.cuda.synchronize()
    assert torch.equal(c_fused, c_dense), "fused gate/up halves and separate tensors must give identical bits"
    want = oracle.swiglu(to_codes(ac), to_codes(bc), "f16")
    frac, worst = close16(to_codes(c_dense), want, "f16", "C2", 1e-3)
    print(f"C2 swiglu: {frac:.2e} of elements differ by {worst} ulp")


def test_c3_rope_f16_4096x32x128_in_fused_qkv(ctx):
    import torch

    nt, nh_buf, nh, dh, rows = 4096, 96, 32, 128, 32768
    qkv = randn((nt, nh_buf, dh), torch.float16, 3)
    before = to_codes(qkv)
    rng = np.random.default_rng(3)
    pos = rng.integers(0, rows, nt).astype(np.uint64)
    sin_t, cos_t = sin_cos_table(rows, dh, 1e4, device="cuda")
    tpos = torch.from_numpy(pos.view(np.int64)).cuda().view(torch.uint64)
    t = qkv[:, :nh, :]
    assert t.stride() == (nh_buf * dh, dh, 1)
    ctx.rope(t, tpos, sin_t, cos_t)
    torch.cuda.synchronize()
    after = to_codes(qkv)
    want = before.copy()
    oracle.rope(want[:, :nh, :], pos, sin_t.cpu().numpy(), cos_t.cpu().numpy(), "f16")
    assert_codes_equal(after[:, :nh, :], want[:, :nh, :], "f16", what="C3 rotated heads")
    assert np.array_equal(after[:, nh:, :], before[:, nh:, :]), "heads outside the view were modified"


def test_c3_rope_position_zero_is_identity_at_full_size(ctx):
    import torch

    qkv = randn((4096, 96, 128), torch.float16, 4)
    before = qkv.clone()
    sin_t, cos_t = sin_cos_table(64, 128, 1e4, device="cuda")
    pos = torch.zeros(4096, dtype=torch.int64, device="cuda").view(torch.uint64)
    ctx.rope(qkv[:, :32, :], pos, sin_t, cos_t)
    torch.cuda.synchronize()
    assert torch.equal(qkv, before)


@pytest.mark.parametrize("broadcast", [False, True])
def test_c4_add_f16_8192x4096(ctx, broadcast):
    import torch

    a = randn((8192, 4096), torch.float16, 5)
    b = randn((4096,) if broadcast else (8192, 4096), torch.float16, 6)
    c = torch.empty_like(a)
    ctx.add(c, a, b)
    torch.cuda.synchronize()
    want = oracle.add(to_codes(a), to_codes(b), (8192, 4096), "f16")
    assert_codes_equal(to_codes(c), want, "f16", what=f"C4 broadcast={broadcast}")
    # a + b == b + a, bit for bit, and in-place on a gives the same bits
    c2 = torch.empty_like(a)
    ctx.add(c2, b, a)
    ctx.add(a, a, b)
    torch.cuda.synchronize()
    assert torch.equal(c2.view(torch.int16), c.view(torch.int16)) and torch.equal(a.view(torch.int16), c.view(torch.int16))


def test_c5_bf16_chain_8192_tokens(ctx):
    """RMSNorm -> RoPE(q), RoPE(k) -> SwiGLU -> Add at Llama-70B shapes."""
    import torch

    T, bf16 = 8192, torch.bfloat16
    # RMSNorm [T, 8192], fp32 weights
    x = randn((T, 8192), bf16, 10)
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    w = torch.rand(8192, generator=g, device="cuda") + 0.5
    y = torch.empty_like(x)
    ctx.rms_norm(y, x, w, 1e-5)
    torch.cuda.synchronize()
    want = oracle.rms_norm(to_codes(x), to_codes(w), 1e-5, "bf16", "f32")
    frac, worst = close16(to_codes(y), want, "bf16", "C5 rms_norm", 5e-3)
    print(f"C5 rms_norm: {frac:.2e} of elements differ by {worst} ulp")
    del x, y, want

    # RoPE on q [T, 64, 128] and k [T, 8, 128], views of qkv [T, 80, 128]; pos = 0..T-1, theta 5e5
    qkv = randn((T, 80, 128), bf16, 12)
    before = to_codes(qkv)
    sin_t, cos_t = sin_cos_table(T, 128, 5e5, device="cuda")
    pos = torch.arange(T, device="cuda", dtype=torch.int64).view(torch.uint64)
    ctx.rope(qkv[:, :64, :], pos, sin_t, cos_t)
    ctx.rope(qkv[:, 64:72, :], pos, sin_t, cos_t)
    torch.cuda.synchronize()
    after = to_codes(qkv)
    want = before.copy()
    npos, s, c = np.arange(T, dtype=np.uint64), sin_t.cpu().numpy(), cos_t.cpu().numpy()
    oracle.rope(want[:, :64, :], npos, s, c, "bf16")
    oracle.rope(want[:, 64:72, :], npos, s, c, "bf16")
    assert_codes_equal(after, want, "bf16", what="C5 rope q+k (v heads must be untouched)")
    del qkv, before, after, want

    # SwiGLU [T, 28672] from the fused gate/up buffer [T, 57344]
    gate_up = randn((T, 57344), bf16, 13)
    out = torch.empty((T, 28672), dtype=bf16, device="cuda")
    ctx.swiglu(out, gate_up[:, 28672:], gate_up[:, :28672])
    torch.cuda.synchronize()
    gu = to_codes(gate_up)
    want = oracle.swiglu(gu[:, 28672:], gu[:, :28672], "bf16")
    frac, worst = close16(to_codes(out), want, "bf16", "C5 swiglu", 1e-3)
    print(f"C5 swiglu: {frac:.2e} of elements differ by {worst} ulp")
    del gate_up, out, gu, want

    # residual Add [T, 8192]
    a, b = randn((T, 8192), bf16, 14), randn((T, 8192), bf16, 15)
    cc = torch.empty_like(a)
    ctx.add(cc, a, b)
    torch.cuda.synchronize()
    assert_codes_equal(to_codes(cc), oracle.add(to_codes(a), to_codes(b), (T, 8192), "bf16"), "bf16", what="C5 add")
    assert torch.equal((a + b).view(torch.int16), cc.view(torch.int16)), "bf16 add must also equal torch's"


def test_add_f16_all_2_to_32_pairs(ctx):
    """Every fp16 code plus every fp16 code: c[i, j] = a[i] + b[j] through the
    broadcasting path, 4096 rows at a time, against the oracle (a generated
    NaN may differ in sign only)."""
    import concurrent.futures

    import torch

    codes = np.arange(65536, dtype=np.uint16)
    tb = torch.from_numpy(codes.view(np.int16)).cuda().view(torch.float16)
    rows = 4096
    tc = torch.empty((rows, 65536), dtype=torch.float16, device="cuda")
    pool = concurrent.futures.ThreadPoolExecutor(16)
    bad_total = 0
    for r0 in range(0, 65536, rows):
        a = codes[r0:r0 + rows].reshape(rows, 1).copy()
        ta = torch.from_numpy(a.view(np.int16)).cuda().view(torch.float16)
        ctx.add(tc, ta, tb)
        parts = list(pool.map(lambda k: oracle.add(a[k:k + 256], codes, (256, 65536), "f16"), range(0, rows, 256)))
        want = np.concatenate(parts)
        torch.cuda.synchronize()
        got = tc.view(torch.int16).cpu().numpy().view(np.uint16)
        diff = got != want
        if diff.any():
            nan_want = ((want & 0x7C00) == 0x7C00) & ((want & 0x3FF) != 0)
            diff &= ~(nan_want & ((got ^ want) == 0x8000))
            bad_total += int(diff.sum())
            if bad_total:
                i, j = np.argwhere(diff)[0]
                raise AssertionError(f"0x{r0 + i:04x} + 0x{j:04x}: got 0x{got[i, j]:04x} want 0x{want[i, j]:04x} ({bad_total} so far)")
    assert bad_total == 0
