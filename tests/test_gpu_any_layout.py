"""The kernels that take what the 16-byte vector paths refuse (odd widths, odd
strides, views that start on odd 2-byte boundaries) move whole groups of 8
elements as 16-byte accesses at whatever boundary they lie on.  Here every
output sits inside a larger buffer of known content - one element in front,
gaps between the rows, some elements behind - and after the call the results
must agree with the oracle AND every element outside the output must still be
what it was: a 16-byte store that reached past a row's end would show here."""
import numpy as np
import pytest

import oracle
from helpers import assert_codes_close, assert_codes_equal, to_codes, to_torch
from operators_amd.ops import sin_cos_table

pytestmark = pytest.mark.gpu


def framed(values, shape, pitch, dt, lead, seed):
    """A view of `shape` with row pitch `pitch` that starts `lead` elements into a buffer of random finite codes.
    Returns (view, whole buffer as codes before the call, boolean mask of the view's elements in the buffer)."""
    import torch

    rows, width = int(np.prod(shape[:-1])), shape[-1]
    span = lead + rows * pitch + 11
    rng = np.random.default_rng(seed)
    before = rng.integers(0x3000, 0x3C00, span, dtype=np.uint16)
    idx = lead + (np.arange(rows) * pitch)[:, None] + np.arange(width)[None, :]
    if values is not None:
        before[idx.ravel()] = np.asarray(values, np.uint16).ravel()
    buf = to_torch(before, dt)
    view = torch.as_strided(buf, (rows, width), (pitch, 1), lead)
    mask = np.zeros(span, bool)
    mask[idx.ravel()] = True
    return view, buf, before, mask


def outside_untouched(buf, before, mask, what):
    after = to_codes(buf)
    assert np.array_equal(after[~mask], before[~mask]), what + ": elements outside the output were written"
    return after[mask]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("n,d,pad,lead", [(5, 1001, 3, 1), (3, 8191, 0, 0), (4, 4096, 5, 3), (7, 24, 1, 1), (2, 20003, 1, 5), (9, 520, 0, 7)])
def test_rms_norm_and_the_fused_form(ctx, dt, n, d, pad, lead):
    import torch

    rng = np.random.default_rng(n * 100003 + d)
    x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    b = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    w = rng.uniform(0.5, 1.5, d).astype(np.float32)
    tw = to_torch(w, "f32")
    tx, _, _, _ = framed(x, (n, d), d + pad, dt, lead, 1)
    ty, ybuf, ybefore, ymask = framed(None, (n, d), d + pad + 2, dt, lead + 1, 2)
    ctx.rms_norm(ty, tx, tw, 1e-5)
    torch.cuda.synchronize()
    got = outside_untouched(ybuf, ybefore, ymask, f"rms_norm [{n},{d}] {dt}").reshape(n, d)
    assert_codes_close(got, oracle.rms_norm(x, w, 1e-5, dt, "f32"), dt, max_ulp=1, max_frac=1e-2, what=f"rms_norm [{n},{d}] {dt}")

    tb, _, _, _ = framed(b, (n, d), d + 1, dt, 2, 3)
    tc, cbuf, cbefore, cmask = framed(None, (n, d), d + pad + 1, dt, lead, 4)
    ty2, ybuf2, ybefore2, ymask2 = framed(None, (n, d), d + pad, dt, lead + 2, 5)
    ctx.add_rms_norm(ty2, tc, tx, tb, tw, 1e-5)
    torch.cuda.synchronize()
    want_c, want_y = oracle.add_rms_norm(x, b, w, 1e-5, dt, "f32")
    assert_codes_equal(outside_untouched(cbuf, cbefore, cmask, "fused c").reshape(n, d), want_c, dt, what=f"fused c [{n},{d}] {dt}")
    assert_codes_close(outside_untouched(ybuf2, ybefore2, ymask2, "fused y").reshape(n, d), want_y, dt, max_ulp=1, max_frac=1e-2,
                       what=f"fused y [{n},{d}] {dt}")


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("n,di,lead", [(6, 1001, 1), (3, 11007, 0), (5, 16, 3), (4, 4096, 1), (2, 9, 1)])
def test_swiglu_on_the_halves_of_a_fused_buffer(ctx, dt, n, di, lead):
    import torch

    rng = np.random.default_rng(n * 7919 + di)
    both = oracle.encode(rng.standard_normal((n, 2 * di)).astype(np.float32) * 2, dt)
    tboth, _, _, _ = framed(both, (n, 2 * di), 2 * di + 1, dt, lead, 6)
    tb, ta = tboth[:, :di], tboth[:, di:]
    tc, cbuf, cbefore, cmask = framed(None, (n, di), di + 3, dt, lead + 1, 7)
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    got = outside_untouched(cbuf, cbefore, cmask, f"swiglu [{n},{di}] {dt}").reshape(n, di)
    assert_codes_close(got, oracle.swiglu(both[:, di:], both[:, :di], dt), dt, max_ulp=1, max_frac=1e-2, what=f"swiglu [{n},{di}] {dt}")


@pytest.mark.parametrize("n,d,lead", [(9, 4095, 1), (5, 1001, 0), (3, 17, 5), (6, 4096, 3)])
def test_add_of_a_tensor_and_a_row(ctx, n, d, lead):
    import torch

    rng = np.random.default_rng(n * 31 + d)
    a = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), "f16")
    b = oracle.encode(rng.standard_normal((1, d)).astype(np.float32), "f16")
    # c and a are dense (Add takes dense tensors, as in the reference) but start `lead` elements into their buffers
    ta, _, _, _ = framed(a, (n, d), d, "f16", lead, 8)
    tbrow, _, _, _ = framed(b, (1, d), d, "f16", lead + 1, 9)
    tc, cbuf, cbefore, cmask = framed(None, (n, d), d, "f16", lead + 2, 10)
    ctx.add(tc, ta, tbrow)
    torch.cuda.synchronize()
    got = outside_untouched(cbuf, cbefore, cmask, f"add [{n},{d}] + [1,{d}]").reshape(n, d)
    assert_codes_equal(got, oracle.add(a, b, (n, d), "f16"), "f16", what=f"add [{n},{d}] + [1,{d}]")


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("tokens,heads,buf_heads,head_dim,lead", [(7, 3, 5, 100, 0), (5, 2, 2, 98, 1), (9, 4, 6, 128, 1), (3, 2, 3, 36, 4), (4, 1, 1, 6, 1)])
def test_rope(ctx, dt, tokens, heads, buf_heads, head_dim, lead):
    import torch

    rng = np.random.default_rng(tokens * 131 + head_dim)
    rows = 64
    qkv = oracle.encode(rng.standard_normal((tokens, buf_heads, head_dim)).astype(np.float32), dt)
    pos = rng.integers(0, rows, tokens).astype(np.uint64)
    sin_t, cos_t = sin_cos_table(rows, head_dim, 1e4)
    flat, buf, before, _ = framed(qkv.reshape(tokens, buf_heads * head_dim), (tokens, buf_heads * head_dim), buf_heads * head_dim + 2, dt, lead, 11)
    t = torch.as_strided(buf, (tokens, heads, head_dim), (buf_heads * head_dim + 2, head_dim, 1), lead)
    ctx.rope(t, torch.from_numpy(pos.view(np.int64)).cuda().view(torch.uint64), sin_t.cuda(), cos_t.cuda())
    torch.cuda.synchronize()
    want = qkv.copy()
    oracle.rope(want[:, :heads, :], pos, sin_t.numpy(), cos_t.numpy(), dt)
    after = to_codes(buf)
    expect = before.copy()
    idx = lead + (np.arange(tokens) * (buf_heads * head_dim + 2))[:, None] + np.arange(buf_heads * head_dim)[None, :]
    expect[idx.ravel()] = want.reshape(tokens, -1).ravel()
    assert_codes_equal(after, expect, dt, what=f"rope [{tokens},{heads},{head_dim}] in [{tokens},{buf_heads},{head_dim}] {dt} (rotated heads bit for bit, everything else as it was)")
