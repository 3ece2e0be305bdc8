"""Tensors of more than 2^31 elements (over 4 GiB of 16-bit data): every
offset a kernel forms must be 64-bit.  A GPU with 288 GB holds such tensors
as a matter of course (a residual stream of 2^19 tokens x 4096, an attention
score block of a long prompt).

The check is the library against itself: slabs of the large call (the first
rows, the rows either side of element 2^31, the last rows) must equal, bit for
bit, a small call on copies of those slabs.  The small shapes are the ones the
other test files hold against the oracle; a wrapped 32-bit offset in the large
call would read or write the wrong rows and cannot pass."""
import pytest

pytestmark = pytest.mark.gpu


def randn16(shape, seed, dtype):
    import torch

    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return torch.randn(shape, generator=g, device="cuda", dtype=dtype)


def same_bits(a, b):
    import torch

    return torch.equal(a.contiguous().view(torch.int16), b.contiguous().view(torch.int16))


def slabs(rows, rows_at_2_31, width=48):
    """Row ranges at the start, around the row that holds element 2^31, and at the end."""
    mid = min(max(rows_at_2_31 - width // 2, 0), rows - width)
    return [(0, width), (mid, mid + width), (rows - width, rows)]


def test_swiglu_flat_and_fused_buffer(ctx):
    import torch

    d = 4096  # the operator takes 2-D tensors (reference: src/ops/swiglu/cpu/swiglu_cpu.cc:12-14); dense ones are walked flat
    rows = (1 << 19) + 257
    a, b = randn16((rows, d), 1, torch.float16), randn16((rows, d), 2, torch.float16)
    c = torch.zeros_like(a)
    ctx.swiglu(c, a, b)
    torch.cuda.synchronize()
    for lo, hi in slabs(rows, (1 << 31) // d, width=256):
        want = torch.zeros((hi - lo, d), dtype=torch.float16, device="cuda")
        ctx.swiglu(want, a[lo:hi].clone(), b[lo:hi].clone())
        torch.cuda.synchronize()
        assert same_bits(c[lo:hi], want), (lo, hi)
    del a, b, c
    # gate and up halves of one [rows, 2 d] buffer: the operands' offsets pass 2^31, the output's do not
    rows, d = (1 << 18) + 3, 4096
    gate_up = randn16((rows, 2 * d), 3, torch.float16)
    h = torch.zeros((rows, d), dtype=torch.float16, device="cuda")
    ctx.swiglu(h, gate_up[:, d:], gate_up[:, :d])
    torch.cuda.synchronize()
    for lo, hi in slabs(rows, (1 << 31) // (2 * d)):
        part = gate_up[lo:hi].clone()
        want = torch.zeros((hi - lo, d), dtype=torch.float16, device="cuda")
        ctx.swiglu(want, part[:, d:], part[:, :d])
        torch.cuda.synchronize()
        assert same_bits(h[lo:hi], want), (lo, hi)


@pytest.mark.parametrize("rows,d", [((1 << 19) + 5, 4096), ((1 << 24) + 3, 128), ((1 << 17) + 1, 16384)])
def test_rms_norm_and_fused(ctx, rows, d):
    import torch

    x = randn16((rows, d), 4, torch.bfloat16)
    w = torch.rand(d, device="cuda") + 0.5
    y = torch.zeros_like(x)
    ctx.rms_norm(y, x, w, 1e-5)
    torch.cuda.synchronize()
    where = slabs(rows, (1 << 31) // d)
    for lo, hi in where:
        want = torch.zeros((hi - lo, d), dtype=torch.bfloat16, device="cuda")
        ctx.rms_norm(want, x[lo:hi].clone(), w, 1e-5)
        torch.cuda.synchronize()
        assert same_bits(y[lo:hi], want), (lo, hi)
    # fused with the residual add, the sum written over the first addend
    a, b = x, randn16((rows, d), 5, torch.bfloat16)
    y.zero_()
    keep = [(a[lo:hi].clone(), b[lo:hi].clone()) for lo, hi in where]
    ctx.add_rms_norm(y, a, a, b, w, 1e-5)
    torch.cuda.synchronize()
    for (lo, hi), (pa, pb) in zip(where, keep):
        py = torch.zeros_like(pa)
        ctx.add_rms_norm(py, pa, pa, pb, w, 1e-5)
        torch.cuda.synchronize()
        assert same_bits(a[lo:hi], pa) and same_bits(y[lo:hi], py), (lo, hi)


def test_rearrange_tokens_to_heads(ctx):
    import torch

    tokens, heads, dim = (1 << 17) + 1, 128, 128
    src = randn16((tokens, heads, dim), 6, torch.float16)
    dst = torch.zeros((heads, tokens, dim), dtype=torch.float16, device="cuda")
    ctx.rearrange(dst.permute(1, 0, 2), src)
    torch.cuda.synchronize()
    for h0 in range(0, heads, 16):  # a copy moves bits: torch's own permute is the check, in slabs to bound memory
        assert same_bits(dst[h0:h0 + 16], src[:, h0:h0 + 16].permute(1, 0, 2)), h0
    # and back, into a padded buffer (row stride of 160 heads)
    wide = torch.zeros((tokens, 160, dim), dtype=torch.float16, device="cuda")
    ctx.rearrange(wide[:, :heads], dst.permute(1, 0, 2))
    torch.cuda.synchronize()
    for t0 in range(0, tokens, 1 << 14):
        assert same_bits(wide[t0:t0 + (1 << 14), :heads], src[t0:t0 + (1 << 14)]), t0
    assert not wide[:, heads:].any()


def test_rearrange_more_than_2_to_31_units(ctx):
    """Rows of 33 bytes out of rows of 40: one-byte units, and more than 2^31 of
    them, so positions are split with 64-bit divisions."""
    import torch

    rows, width, pitch = (1 << 26) + 5, 33, 40
    g = torch.Generator(device="cuda")
    g.manual_seed(11)
    src = torch.randint(-128, 128, (rows, pitch), generator=g, device="cuda", dtype=torch.int8)
    dst = torch.zeros((rows, width), dtype=torch.int8, device="cuda")
    ctx.rearrange(dst, src[:, :width])
    torch.cuda.synchronize()
    for r0 in range(0, rows, 1 << 23):  # in slabs to bound memory
        assert torch.equal(dst[r0:r0 + (1 << 23)], src[r0:r0 + (1 << 23), :width]), r0


@pytest.mark.parametrize("heads", [128, 8])
def test_rope_in_place(ctx, heads):
    import torch

    from operators_amd.ops import sin_cos_table

    dim = 128
    tokens = ((1 << 31) // (heads * dim)) + 33
    t = randn16((tokens, heads, dim), 7, torch.float16)
    g = torch.Generator(device="cuda")
    g.manual_seed(8)
    pos = torch.randint(0, 4096, (tokens,), generator=g, device="cuda", dtype=torch.int64).view(torch.uint64)
    sin_t, cos_t = sin_cos_table(4096, dim, 1e4, device="cuda")
    where = slabs(tokens, (1 << 31) // (heads * dim), width=32)
    keep = [t[lo:hi].clone() for lo, hi in where]
    untouched = t[where[0][1]:where[0][1] + 8].clone()
    ctx.rope(t, pos, sin_t, cos_t)
    torch.cuda.synchronize()
    for (lo, hi), part in zip(where, keep):
        ctx.rope(part, pos.view(torch.int64)[lo:hi].clone().view(torch.uint64), sin_t, cos_t)
        torch.cuda.synchronize()
        assert same_bits(t[lo:hi], part), (lo, hi)
    assert not same_bits(t[where[0][1]:where[0][1] + 8], untouched)  # rows between the slabs were rotated too


def test_causal_softmax_in_place(ctx):
    import torch

    batch, seq = 9, 16384  # 9 * 2^28 elements
    y = randn16((batch, seq, seq), 9, torch.float16)
    first, last = y[0].clone(), y[batch - 1].clone()
    straddle = y[7].clone()  # element 2^31 is the first of batch 8; batch 7 ends just below it
    ctx.causal_softmax(y)
    torch.cuda.synchronize()
    for b, part in ((0, first), (7, straddle), (batch - 1, last)):
        ctx.causal_softmax(part.view(1, seq, seq))
        torch.cuda.synchronize()
        assert same_bits(y[b], part), b


def test_causal_softmax_ragged_rows_in_place(ctx):
    """Rows of 21 001 elements: no row starts where another does within its
    128-byte line, and element 2^31 lies in the last matrix.  The copy of a
    matrix is placed at the same distance from a 128-byte boundary, so that the
    lanes take the same vectors and the sums add in the same order."""
    import torch

    batch, seq, total = 6, 20001, 21001
    y = randn16((batch, seq, total), 12, torch.float16)
    parts = {}
    for b in (0, 3, batch - 1):
        start = (b * seq * total) % 64
        buf = torch.zeros(start + seq * total, dtype=torch.float16, device="cuda")
        parts[b] = buf[start:].view(1, seq, total)
        parts[b].copy_(y[b])
    ctx.causal_softmax(y)
    torch.cuda.synchronize()
    for b, part in parts.items():
        ctx.causal_softmax(part)
        torch.cuda.synchronize()
        assert same_bits(y[b], part[0]), b
