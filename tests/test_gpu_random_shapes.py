"""Seeded random shapes and strides through every launch path of the row and
element operators, against the oracle.

The fixed-shape tests pick the sizes somebody thought of; the launch code
chooses among many kernels by row length, row count, alignment and stride
(RMSNorm alone: several short rows per wavefront, one-pass shapes of 64, 128
and 256 lanes, shapes compiled for common widths, the run-time lane count,
the general ladder, the element kernel).  Here the sizes come from a seeded
generator that is biased towards the boundaries between those paths, so every
run checks the same few hundred cases and a new path gets exercised without
anybody having to think of its edge."""
import numpy as np
import pytest

import oracle
from helpers import assert_allclose16, assert_codes_close, assert_codes_equal, strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
TOL = {"f16": 1e-3, "bf16": 1e-2}

# row lengths at and around the switches of the launch code
EDGES = [8, 16, 24, 64, 72, 128, 136, 248, 256, 264, 504, 512, 520, 768, 1016, 1024, 1032, 1536, 2040, 2048, 2056, 2560, 3584,
         4088, 4096, 4104, 4608, 5120, 5632, 6144, 6656, 7168, 8184, 8192, 8200, 9216, 10240, 11264, 12288, 14336, 16384, 16392,
         18432, 20480]


def pick_width(rng, multiple_of_8=True):
    r = rng.random()
    if r < 0.6:
        d = int(rng.choice(EDGES))
    elif r < 0.85:
        d = int(rng.integers(1, 1200)) * 8
    else:
        d = int(rng.integers(1, 9000))
    if multiple_of_8 and rng.random() < 0.9:
        d = max(8, d // 8 * 8)
    return d


def pick_rows(rng, d, budget=1 << 21):
    cap = max(1, budget // d)
    r = rng.random()
    if r < 0.3:
        return int(rng.integers(1, 9))
    if r < 0.6:
        return int(min(cap, rng.choice([255, 256, 257, 511, 512, 513, 600, 1000, 1030])))
    return int(rng.integers(1, cap + 1))


def close(got, want, dt, what, max_frac=5e-3):
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), TOL[dt], TOL[dt], what)
    assert_codes_close(got, want, dt, max_ulp=1, max_frac=max_frac, what=what)


@pytest.mark.parametrize("seed", range(60))
def test_rms_norm_and_fused(ctx, seed):
    import torch

    rng = np.random.default_rng(9000 + seed)
    dt = str(rng.choice(["f16", "bf16"]))
    wdt = str(rng.choice(["f32", dt]))
    d = pick_width(rng)
    n = pick_rows(rng, d)
    x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    b = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    w = oracle.encode(rng.uniform(0.5, 1.5, d).astype(np.float32), wdt)
    eps = float(rng.choice([1e-5, 1e-6]))
    # row strides: dense, padded to a multiple of 8, or odd (which sends the call to the element kernels)
    pad = int(rng.choice([0, 0, 8, 64, 3]))
    sx, sy = d + pad, d + int(rng.choice([0, pad, 16]))
    tx = strided_like(x, (n, d), (sx, 1), dt)[0] if sx != d else to_torch(x, dt)
    ty = strided_like(np.zeros((n, d), np.uint16), (n, d), (sy, 1), dt)[0] if sy != d else torch.empty((n, d), dtype=tx.dtype, device="cuda")
    tw = to_torch(w, wdt)
    what = f"seed {seed}: [{n},{d}] {dt} w {wdt} strides {sx},{sy}"
    frac = 5e-3 if d <= 16384 else 3e-2
    ctx.rms_norm(ty, tx, tw, eps)
    torch.cuda.synchronize()
    got_y = to_codes(ty)
    close(got_y, oracle.rms_norm(x, w, eps, dt, wdt), dt, "rms_norm " + what, frac)
    if seed % 3 == 0:  # in place: the same bits as out of place
        tx_copy = tx.clone() if sx == d else strided_like(x, (n, d), (sx, 1), dt)[0]
        ctx.rms_norm(tx_copy, tx_copy, tw, eps)
        torch.cuda.synchronize()
        assert np.array_equal(to_codes(tx_copy), got_y), "in place differs: " + what
    # the fused form on the same rows: c = x + b bit for bit Add's, y RMSNorm's of that sum
    tb = to_torch(b, dt)
    tc = torch.empty((n, d), dtype=tx.dtype, device="cuda")
    ty2 = torch.empty((n, d), dtype=tx.dtype, device="cuda")
    ctx.add_rms_norm(ty2, tc, tx, tb, tw, eps)
    torch.cuda.synchronize()
    want_c, want_y = oracle.add_rms_norm(x, b, w, eps, dt, wdt)
    assert_codes_equal(to_codes(tc), want_c, dt, what="fused c " + what)
    close(to_codes(ty2), want_y, dt, "fused y " + what, frac)
    # and it is what the two separate calls give, to the bit
    tc2 = torch.empty_like(tc)
    ty3 = torch.empty_like(tc)
    ctx.add(tc2, to_torch(x, dt), tb)  # Add takes dense operands only, as in the reference
    ctx.rms_norm(ty3, tc2, tw, eps)
    torch.cuda.synchronize()
    assert torch.equal(ty3.view(torch.int16), ty2.view(torch.int16)), "fused y differs from Add then RMSNorm: " + what


@pytest.mark.parametrize("seed", range(40))
def test_swiglu(ctx, seed):
    import torch

    rng = np.random.default_rng(9100 + seed)
    dt = str(rng.choice(["f16", "bf16"]))
    di = pick_width(rng)
    n = pick_rows(rng, di, 1 << 20)
    a = oracle.encode(rng.standard_normal((n, di)).astype(np.float32) * 2, dt)
    b = oracle.encode(rng.standard_normal((n, di)).astype(np.float32) * 3, dt)
    layout = int(rng.integers(0, 3))
    if layout == 0:  # dense
        ta, tb = to_torch(a, dt), to_torch(b, dt)
    elif layout == 1:  # the MLP's fused buffer: gate in the first half of every row, up in the second
        both = to_torch(np.concatenate([b, a], axis=1), dt)
        tb, ta = both[:, :di], both[:, di:]
    else:  # unrelated row strides
        ta = strided_like(a, (n, di), (di + 8 * int(rng.integers(0, 5)), 1), dt)[0]
        tb = strided_like(b, (n, di), (di + int(rng.choice([0, 8, 5])), 1), dt)[0]
    # the result into a tensor of its own, or in place over a or over b (the reference's tests do both)
    where = int(rng.integers(0, 3))
    tc = torch.empty((n, di), dtype=ta.dtype, device="cuda") if where == 0 else (ta if where == 1 else tb)
    ctx.swiglu(tc, ta, tb)
    torch.cuda.synchronize()
    close(to_codes(tc), oracle.swiglu(a, b, dt), dt, f"seed {seed}: swiglu [{n},{di}] {dt} layout {layout} result {where}")


@pytest.mark.parametrize("seed", range(40))
def test_add(ctx, seed):
    import torch

    rng = np.random.default_rng(9200 + seed)
    dt = str(rng.choice(["f16", "bf16", "f32"]))
    nd = int(rng.integers(1, 5))
    shape = [int(rng.choice([1, 2, 3, 5, 8, 16, 40, 64, 96, 128, 520])) for _ in range(nd)]
    while int(np.prod(shape)) > (1 << 21):
        shape[int(np.argmax(shape))] //= 2
    shape = [max(1, s) for s in shape]

    def operand():  # the full shape, or some dimensions of extent 1, or fewer leading dimensions
        s = list(shape)
        for i in range(nd):
            if rng.random() < 0.35:
                s[i] = 1
        cut = int(rng.integers(0, nd)) if rng.random() < 0.4 else 0
        return s[cut:]

    sa, sb = operand(), operand()
    if rng.random() < 0.5:
        sa = list(shape)  # one full operand at least half of the time
    want_shape = list(np.broadcast_shapes(tuple(sa), tuple(sb)))
    if dt == "f32":
        a = rng.standard_normal(sa).astype(np.float32)
        b = rng.standard_normal(sb).astype(np.float32)
    else:
        a = oracle.encode(rng.standard_normal(sa).astype(np.float32), dt)
        b = oracle.encode(rng.standard_normal(sb).astype(np.float32), dt)
    ta, tb = to_torch(a, dt), to_torch(b, dt)
    tc = torch.empty(want_shape, dtype=ta.dtype, device="cuda")
    if list(sa) == want_shape and rng.random() < 0.3:
        tc = ta  # in place over the operand that has the result's shape
    ctx.add(tc, ta, tb)
    torch.cuda.synchronize()
    want = oracle.add(a, b, tuple(want_shape), dt)
    got = to_codes(tc)
    what = f"seed {seed}: add {sa} + {sb} -> {want_shape} {dt}"
    if dt == "f32":
        assert np.array_equal(got.view(np.uint32), np.asarray(want, np.float32).view(np.uint32)), what
    else:
        assert_codes_equal(got, want, dt, what=what)


@pytest.mark.parametrize("seed", range(40))
def test_rope(ctx, seed):
    import torch

    from operators_amd.ops import sin_cos_table

    rng = np.random.default_rng(9300 + seed)
    dt = str(rng.choice(["f16", "bf16"]))
    head_dim = int(rng.choice([8, 16, 32, 64, 80, 96, 128, 256, 6, 34]))
    heads = int(rng.choice([1, 2, 3, 4, 7, 8, 12, 16, 28, 32, 40]))
    tokens = int(rng.choice([1, 2, 5, 31, 64, 100, 257, 600]))
    extra = int(rng.choice([0, 0, 2, 8]))  # heads of the buffer that the view leaves out
    first = int(rng.integers(0, extra + 1))
    rows = int(rng.choice([tokens, 2 * tokens + 3, 4096]))
    buf = oracle.encode(rng.standard_normal((tokens, heads + extra, head_dim)).astype(np.float32), dt)
    pos = rng.integers(0, rows, tokens).astype(np.uint64)
    sin_t, cos_t = sin_cos_table(rows, head_dim, 1e4, device="cuda")
    tbuf = to_torch(buf, dt)
    view = tbuf[:, first:first + heads, :]
    tpos = torch.from_numpy(pos.astype(np.int64)).cuda().view(torch.uint64)
    ctx.rope(view, tpos, sin_t, cos_t)
    torch.cuda.synchronize()
    want = buf.copy()
    want[:, first:first + heads, :] = oracle.rope(buf[:, first:first + heads, :], pos, sin_t.cpu().numpy(), cos_t.cpu().numpy(), dt)
    # bit-exact, and the heads outside the view are untouched
    assert_codes_equal(to_codes(tbuf), want, dt, what=f"seed {seed}: rope [{tokens},{heads},{head_dim}] of {heads + extra} heads from {first}, {dt}")


@pytest.mark.parametrize("seed", range(30))
def test_causal_softmax(ctx, seed):
    import torch

    rng = np.random.default_rng(9400 + seed)
    dt = str(rng.choice(["f16", "bf16"]))
    total = int(rng.choice([8, 64, 72, 256, 504, 512, 520, 1024, 2048, 2056, 4096, 4104, 8192, 9000, 16384, 1000, 77]))
    seq = int(min(total, rng.choice([1, 2, 7, 64, 100, 300, total])))
    batch = int(rng.choice([1, 1, 2, 5]))
    while batch * seq * total > (1 << 21):
        if seq > 8:
            seq //= 2
        else:
            batch = 1
            break
    y = oracle.encode(rng.standard_normal((batch, seq, total)).astype(np.float32) * 3, dt)
    ty = to_torch(y, dt)
    ctx.causal_softmax(ty)
    torch.cuda.synchronize()
    got, want = to_codes(ty), oracle.causal_softmax(y, dt)
    what = f"seed {seed}: causal_softmax [{batch},{seq},{total}] {dt}"
    close(got, want, dt, what, max_frac=5e-3 if total <= 4096 else 2e-2)
    # the masked part is exact zeros
    for i in range(seq):
        assert not got[:, i, total - seq + i + 1:].any(), what


@pytest.mark.parametrize("seed", range(40))
def test_rearrange(ctx, seed):
    import torch

    rng = np.random.default_rng(9500 + seed)
    nd = int(rng.integers(1, 4))
    shape = [int(rng.choice([1, 2, 3, 4, 8, 16, 31, 64, 128, 352])) for _ in range(nd)]
    while int(np.prod(shape)) > (1 << 20):
        shape[int(np.argmax(shape))] //= 2
    shape = [max(1, s) for s in shape]
    dtype = rng.choice([torch.uint8, torch.float16, torch.float32, torch.float64])

    def layout():  # a permuted, padded arrangement of the dimensions (the innermost stays innermost: the reference demands it)
        order = list(rng.permutation(nd - 1)) + [nd - 1] if nd > 1 else [0]
        strides, step = [0] * nd, 1
        for ax in reversed(order):
            strides[ax] = step
            step *= shape[ax]
            if rng.random() < 0.4:
                step += int(rng.choice([1, 8, 24]))
        return strides, step

    (ss, span_s), (sd, span_d) = layout(), layout()
    if nd == 3 and shape[0] % 2 == 0 and rng.random() < 0.5:
        # rank 4: the reference takes more than three dimensions when the leading ones nest exactly
        # (rearrange_cpu.cc:22-30), so the outermost dimension is split in two in both tensors
        shape = [2, shape[0] // 2] + shape[1:]
        ss = [ss[0] * shape[1], ss[0]] + ss[1:]
        sd = [sd[0] * shape[1], sd[0]] + sd[1:]
    src_buf = torch.from_numpy(rng.integers(0, 255, span_s * 8, dtype=np.uint8)).cuda().view(dtype)[:span_s]
    dst_buf = torch.from_numpy(rng.integers(0, 255, span_d * 8, dtype=np.uint8)).cuda().view(dtype)[:span_d]
    before = dst_buf.clone()
    src = torch.as_strided(src_buf, shape, ss)
    dst = torch.as_strided(dst_buf, shape, sd)
    ctx.rearrange(dst, src)
    torch.cuda.synchronize()
    what = f"seed {seed}: rearrange {shape} {dtype} strides {ss} -> {sd}"
    as_bytes = lambda t: t.contiguous().view(torch.uint8)  # noqa: E731
    assert torch.equal(as_bytes(dst), as_bytes(src)), what
    # bytes of the destination buffer outside the view are untouched
    touched = torch.zeros(span_d, dtype=torch.bool, device="cuda")
    torch.as_strided(touched, shape, sd).fill_(True)
    assert torch.equal(as_bytes(dst_buf[~touched]), as_bytes(before[~touched])), what
