"""CausalSoftmax on the GPU through the C ABI, against the oracle and the
reference's golden vectors.  Bar (fp16): |gpu - ref| <= 1e-3 + 1e-3*|ref| and
at most one unit in the last place (tree sum on the GPU, running sum on the
CPU; last bit of expf).  bf16: 1e-2.  Masked columns must be exact zeros."""
import numpy as np
import pytest

import oracle
from helpers import assert_allclose16, assert_codes_close, golden, golden_json, strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
TOL = {"f16": 1e-3, "bf16": 1e-2}


def run(ctx, codes, shape, strides, dt, use_workspace=True):
    import torch

    if strides is None:
        t = to_torch(codes, dt).reshape(shape)
        buf = t
    else:
        t, buf = strided_like(codes, shape, strides, dt)
    before = to_codes(buf)
    ctx.causal_softmax(t, use_workspace=use_workspace)
    torch.cuda.synchronize()
    return to_codes(t), before, to_codes(buf)


def check(got, want, dt, what, max_frac=5e-3):
    assert_allclose16(oracle.decode(got, dt), oracle.decode(want, dt), TOL[dt], TOL[dt], what)
    return assert_codes_close(got, want, dt, max_ulp=1, max_frac=max_frac, what=what)


def test_golden_cases(ctx):
    g = golden("causal_softmax")
    for i, (shape, strides) in enumerate(golden_json()["causal_cases"]):
        got, before, after = run(ctx, g[f"causal{i}_in"], shape, strides, "f16")
        check(got, g[f"causal{i}_out"], "f16", f"golden causal case {i} {shape} {strides}")
        if strides is not None:  # gaps between rows untouched
            idx = np.zeros(shape, np.int64)
            for ax, st in enumerate(strides):
                ix = np.arange(shape[ax]).reshape([-1 if a == ax else 1 for a in range(len(shape))])
                idx = idx + ix * st
            mask = np.ones(before.size, bool)
            mask[idx.ravel()] = False
            assert np.array_equal(before[mask], after[mask])


CASES = [
    ((32, 20, 512), None), ((32, 20, 512), (20480, 512, 1)),   # the reference's test
    ((7, 13), None), ((5, 5), None), ((1, 8), None), ((3, 16, 16), None),
    ((2, 300, 4096), None), ((2, 64, 8192), None), ((1, 9, 32768), None), ((1, 5, 40000), None),
    ((4, 33, 1000), None), ((2, 128, 136), (128 * 144, 144, 1)), ((3, 10, 64), (1000, 65, 1)),
    # rows of up to 256 elements, several to a wavefront: 8, 16 and 32 lanes per row, rows that do not fill their lanes, padded rows,
    # a row count that is no multiple of the rows per wavefront (one row per wavefront again), more groups of rows than wavefronts
    ((5, 64, 128), None), ((3, 100, 256), None), ((2, 30, 200), None), ((6, 24, 40), None), ((4, 16, 64), (16 * 80 + 8, 80, 1)),
    ((3, 13, 64), None), ((300000, 16, 16), None), ((9, 256, 256), None),
    # rows of 257-512 elements, two to a wavefront with two vectors per lane: square, wide, ragged, padded, an odd number of rows
    # lengths that are no multiple of 8 and rows that do not start on 16-byte boundaries (what attention over an arbitrary number
    # of keys produces): the aligned vectors that cover a row, its two edge vectors written element by element; every workgroup size
    ((32, 20, 333), None), ((3, 100, 1027), None), ((2, 50, 4099), None), ((2, 9, 33001), None), ((5, 60, 63), None), ((4, 7, 7), None),
    ((2, 130, 2050), None), ((3, 40, 2048), (40 * 2051, 2051, 1)), ((2, 5, 70003), None), ((6, 300, 301), None),
    # short rows in whole lines whose matrices do not fill wavefronts (decoding: one row per matrix), any consecutive rows per wavefront
    ((37, 1, 320), None), ((9, 3, 128), None), ((50, 7, 512), None), ((5, 1, 64), (64 * 3, 64, 1)), ((33, 1, 300), None), ((3, 127, 128), None),
    ((2, 40, 4100), None), ((2, 33, 2104), None), ((2, 33, 2105), None), ((3, 50, 1080), None), ((2, 1000, 1000), None), ((1, 600, 4088), None),
    # rows of 32 769-131 072 elements held in registers as raw words (512 lanes x 12 / 16 / 20 vectors, 1024 lanes x 12 / 14 / 16),
    # padded rows; beyond that, and ragged, two passes with 16-byte accesses
    ((2, 6, 65536), None), ((1, 4, 100000), None), ((2, 3, 40000), (3 * 40008, 40008, 1)), ((1, 7, 32776), None),
    ((1, 5, 81920), None), ((2, 3, 70000), None), ((1, 4, 90000), None), ((1, 3, 131072), None), ((1, 3, 120000), None), ((1, 3, 131080), None),
    ((1, 70, 32840), None), ((1, 40, 65544), (40 * 65600, 65600, 1)),
    # 16 385-32 768 elements: 512 lanes x 8 vectors, whole lines and ragged
    ((2, 5, 20480), None), ((1, 6, 32768), None), ((2, 4, 20001), None), ((1, 3, 32760), (3 * 32776, 32776, 1)),
    ((5, 512, 512), None), ((3, 40, 400), None), ((2, 300, 512), None), ((3, 64, 264), None), ((2, 16, 504), (16 * 520, 520, 1)), ((2, 33, 512), None),
]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_against_oracle(ctx, dt, case):
    shape, strides = CASES[case]
    rng = np.random.default_rng(500 + case)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 2, dt)
    want = oracle.causal_softmax(y.copy(), dt)
    got, _, _ = run(ctx, y, shape, strides, dt)
    seq, total = shape[-2], shape[-1]
    keep = np.arange(total)[None, :] <= total - seq + np.arange(seq)[:, None]
    assert not got[..., ~keep].any(), "masked columns must be exact zeros"
    check(got, want, dt, f"{shape} {strides} {dt}", max_frac=2e-2 if total > 4096 else 5e-3)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("start,shape,pitch", [(3, (4, 50, 333), 341), (1, (2, 30, 1000), 1001), (5, (3, 17, 2047), 2047), (7, (2, 9, 4101), 4110),
                                               (2, (2, 4, 33333), 33339), (0, (3, 21, 77), 77), (6, (40, 3, 5), 5), (4, (2, 6, 520), 523),
                                               # up to 56 elements behind a workgroup's vectors are taken one by one, also for rows in whole lines
                                               (0, (2, 10, 4152), 4160), (0, (3, 12, 2104), 2112), (3, (2, 12, 2105), 2111), (0, (2, 7, 32800), 32832),
                                               (5, (2, 9, 32830), 32831), (1, (3, 10, 16), 16), (0, (3, 10, 15), 15), (3, (2, 16, 17), 19), (0, (2, 70, 568), 576),
                                               # long rows at any boundary, held in registers: body vectors turned to line boundaries, ends one by one
                                               (3, (1, 3, 65537), 65541), (1, (1, 2, 100001), 100003), (7, (1, 3, 131073), 131075), (0, (1, 5, 40001), 40001),
                                               (4, (1, 3, 81913), 81920)])
def test_ragged_rows_leave_their_neighbours_alone(ctx, dt, start, shape, pitch):
    """Rows that start anywhere and end anywhere, inside a buffer of other data:
    `start` elements in front of the first row, `pitch - total` between rows.
    The kernels read the 16-byte vectors that cover a row and must write the
    row's own elements only."""
    import torch

    batch, seq, total = shape
    rng = np.random.default_rng(900 + start + total)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 2, dt)
    want = oracle.causal_softmax(y.copy(), dt)
    span = start + batch * seq * pitch + 11
    before = rng.integers(0, 0x3C00, span, dtype=np.uint16)
    buf = to_torch(before, dt)
    view = torch.as_strided(buf, shape, (seq * pitch, pitch, 1), storage_offset=start)
    view.copy_(to_torch(y, dt).reshape(shape))
    ctx.causal_softmax(view)
    torch.cuda.synchronize()
    got, after = to_codes(view), to_codes(buf)
    check(got, want, dt, f"{start} {shape} {pitch} {dt}", max_frac=2e-2 if total > 4096 else 5e-3)
    keep = np.arange(total)[None, :] <= total - seq + np.arange(seq)[:, None]
    assert not got[..., ~keep].any()
    own = np.zeros(span, bool)
    rows = start + (np.arange(batch * seq) * pitch)[:, None] + np.arange(total)[None, :]
    own[rows.ravel()] = True
    assert np.array_equal(before[~own], after[~own]), "elements outside the rows were written"


@pytest.mark.parametrize("seed", range(48))
def test_random_ragged_views(ctx, seed):
    """Any row length, any pitch, any distance of the first row from a 128-byte
    boundary, drawn at random: against the oracle, masked columns exact zeros,
    every element outside the rows untouched."""
    import torch

    rng = np.random.default_rng(7100 + seed)
    dt = str(rng.choice(["f16", "bf16"]))
    total = int(np.exp(rng.uniform(np.log(1), np.log(70000))))
    seq = int(min(total, rng.choice([1, 2, 3, 9, 40, 130, total])))
    batch = int(rng.choice([1, 2, 3]))
    while batch * seq * total > (1 << 21):
        if seq > 4:
            seq //= 2
        else:
            batch = 1
            break
    pitch = total + int(rng.choice([0, 0, 1, 3, 8, 11, 64]))
    start = int(rng.integers(0, 64))
    shape = (batch, seq, total)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 3, dt)
    want = oracle.causal_softmax(y.copy(), dt)
    span = start + batch * seq * pitch + 9
    before = rng.integers(0, 0x3C00, span, dtype=np.uint16)
    buf = to_torch(before, dt)
    view = torch.as_strided(buf, shape, (seq * pitch, pitch, 1), storage_offset=start)
    view.copy_(to_torch(y, dt).reshape(shape))
    ctx.causal_softmax(view)
    torch.cuda.synchronize()
    got, after = to_codes(view), to_codes(buf)
    what = f"seed {seed}: {shape} pitch {pitch} start {start} {dt}"
    check(got, want, dt, what, max_frac=2e-2 if total > 4096 else 5e-3)
    keep = np.arange(total)[None, :] <= total - seq + np.arange(seq)[:, None]
    assert not got[..., ~keep].any(), what
    own = np.zeros(span, bool)
    rows = start + (np.arange(batch * seq) * pitch)[:, None] + np.arange(total)[None, :]
    own[rows.ravel()] = True
    assert np.array_equal(before[~own], after[~own]), what + ": elements outside the rows were written"


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(2, 8, 4096), (2, 8, 20001), (2, 8, 65536), (1, 6, 100003)])
def test_where_gpu_and_cpu_path_differ_the_gpu_is_the_exact_one(ctx, dt, shape):
    """The CPU path adds a row's exponentials one after the other in fp32
    (causal_softmax_cpu.cc:71-75), which loses small addends on long rows; the
    GPU adds them in trees.  Where the two results differ (by one unit in the
    last place), the GPU's is the float64 quotient narrowed by the type's own
    rule in all but a few cases, and over all kept elements the GPU matches
    that exact result more often than the CPU path does."""
    rng = np.random.default_rng(31)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 3, dt)
    want = oracle.causal_softmax(y.copy(), dt).reshape(shape)
    got, _, _ = run(ctx, y, shape, None, dt)
    got = got.reshape(shape)
    seq, total = shape[1], shape[2]
    keep = np.broadcast_to(np.arange(total)[None, :] <= total - seq + np.arange(seq)[:, None], shape)
    x = np.where(keep, oracle.decode(y, dt).astype(np.float64).reshape(shape), -np.inf)
    e = np.exp(x - x.max(-1, keepdims=True))
    exact = oracle.encode((e / e.sum(-1, keepdims=True)).astype(np.float32).ravel(), dt).reshape(shape)
    differ = got != want
    n = int(differ.sum())
    gpu_right, cpu_right = int((got == exact)[differ].sum()), int((want == exact)[differ].sum())
    print(f"causal softmax {shape} {dt}: {n} of {differ.size} differ; of those the GPU has the exact result in {gpu_right}, the CPU path in {cpu_right}")
    assert gpu_right >= 0.8 * n and gpu_right >= cpu_right
    assert (got == exact)[keep].mean() >= (want == exact)[keep].mean()
    assert (got == exact)[keep].mean() > 0.9995


@pytest.mark.parametrize("use_workspace", [False, True])
@pytest.mark.parametrize("dt", ["f16", "bf16"])
def test_long_row_forms_against_the_float64_quotient(ctx, dt, use_workspace):
    """(With the workspace these few rows are split over several workgroups each; without it a workgroup takes a row.)
    Rows of 32 769 elements and more form their exponentials with the hardware exp2 of one fused multiply-add
    (relative error below 3e-6), the shorter ones with a corrected exponential: the same row is therefore not
    promised the same bits through both.  What is promised, and recorded here: every output of either form is
    within one unit in the last place of the float64 quotient narrowed by the type's rule, and the long-row form
    hits it exactly about as often as the register form does on a row of 32 768."""
    rng = np.random.default_rng(41)
    rates = {}
    for total in (32768, 40000, 40001, 65536, 65537, 100000, 131072, 200000):
        shape = (1, 4, total)
        y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 3, dt)
        got, _, _ = run(ctx, y, shape, None, dt, use_workspace)
        got = got.reshape(shape)
        keep = np.broadcast_to(np.arange(total)[None, :] <= total - 4 + np.arange(4)[:, None], shape)
        x = np.where(keep, oracle.decode(y, dt).astype(np.float64).reshape(shape), -np.inf)
        e = np.exp(x - x.max(-1, keepdims=True))
        exact = oracle.encode((e / e.sum(-1, keepdims=True)).astype(np.float32).ravel(), dt).reshape(shape)
        frac, worst = check(got, exact, dt, f"[1,4,{total}] {dt} against float64", max_frac=1e-2)
        rates[total] = 1.0 - frac
        assert worst <= 1
    print(f"causal softmax {dt}: share of outputs equal to the narrowed float64 quotient, by row length: " + ", ".join(f"{t}: {r:.5f}" for t, r in rates.items()))
    assert min(rates.values()) > 0.999 and rates[32768] - min(rates.values()) < 5e-4


def test_attention_scores_shape(ctx):
    """[heads, seq, total] = [8, 2048, 2048] fp16 with a scale typical of q.k/sqrt(d)."""
    rng = np.random.default_rng(77)
    shape = (8, 2048, 2048)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 1.5, "f16")
    want = oracle.causal_softmax(y.copy(), "f16")
    got, _, _ = run(ctx, y, shape, None, "f16")
    frac, worst = check(got, want, "f16", "attention scores")
    print(f"causal softmax [8,2048,2048]: {frac:.2e} of elements differ by {worst} ulp")
    rows = oracle.decode(got, "f16").astype(np.float64).sum(-1)
    assert np.all(np.abs(rows - 1) < 0.02)


def test_infinities_and_long_tails(ctx):
    """-inf entries inside the kept part (a second, caller-made mask) contribute
    zero; entries more than 126 below the row maximum take the library
    exponential; a row that is -inf throughout yields NaN, as on the CPU."""
    rng = np.random.default_rng(78)
    vals = rng.standard_normal((2, 24, 64)).astype(np.float32) * 2
    vals[0, :, 3] = -np.inf
    vals[0, 5, :] = -np.inf
    vals[1, :, 10] = -300.0
    vals[1, 7, 0] = 200.0
    vals[1, 9, :20] = -60000.0
    y = oracle.encode(vals, "f16")
    want = oracle.causal_softmax(y.copy(), "f16")
    got, _, _ = run(ctx, y, y.shape, None, "f16")
    check(got, want, "f16", "infinities and tails", max_frac=2e-2)
    assert np.isnan(oracle.decode(got, "f16")[0, 5, 0])


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("start,shape", [(3, (2, 24, 77)), (5, (2, 12, 333)), (1, (2, 6, 4095)), (0, (2, 6, 4100)), (7, (2, 4, 20001)), (2, (2, 3, 33000)), (0, (2, 5, 2048))])
def test_infinities_and_long_tails_in_ragged_rows(ctx, dt, start, shape):
    """The special values at the places a ragged row treats apart: its first
    and last elements (taken one per lane), the vector that straddles the mask,
    and the body; rows that lie `start` elements behind a 128-byte boundary."""
    import torch

    batch, seq, total = shape
    rng = np.random.default_rng(80 + total)
    vals = rng.standard_normal(shape).astype(np.float32) * 2
    vals[0, :, 0] = -np.inf                      # a first element
    vals[0, :, total - 1] = -np.inf              # a last element (kept only in the last row)
    vals[0, seq - 1, total - 3:] = -300.0        # a long tail at the end of the last row
    vals[0, 0, :] = -np.inf                      # a row that is -inf throughout: NaN, as on the CPU
    vals[1, :, 1] = -300.0                       # more than 126 below the maximum: the library exponential
    vals[1, :, total // 2] = 200.0
    vals[1, seq - 1, : total // 3] = -60000.0 if dt == "f16" else -3e38
    if batch > 1 and seq > 2:
        vals[1, 1, 2] = np.inf                   # +inf in the kept part: that row is NaN, the others are not
    y = oracle.encode(vals, dt)
    want = oracle.causal_softmax(y.copy(), dt).reshape(shape)
    buf = torch.zeros(start + batch * seq * total + 8, dtype=torch.float16 if dt == "f16" else torch.bfloat16, device="cuda")
    view = buf[start:start + batch * seq * total].view(shape)
    view.copy_(to_torch(y, dt).reshape(shape))
    ctx.causal_softmax(view)
    torch.cuda.synchronize()
    got = to_codes(view).reshape(shape)
    nan_want, nan_got = np.isnan(oracle.decode(want.ravel(), dt)).reshape(shape), np.isnan(oracle.decode(got.ravel(), dt)).reshape(shape)
    assert np.array_equal(nan_want, nan_got), "NaN in other places than on the CPU"
    assert nan_got[0, 0, 0]
    check(np.where(nan_got, 0, got).astype(np.uint16), np.where(nan_want, 0, want).astype(np.uint16), dt, f"specials {start} {shape} {dt}", max_frac=2e-2)
    assert not buf[:start].any() and not buf[start + batch * seq * total:].any()


@pytest.mark.parametrize("use_workspace", [False, True])
def test_infinities_and_long_tails_in_long_rows(ctx, use_workspace):
    """The same special values in rows of 50 000 elements (held in registers)."""
    rng = np.random.default_rng(79)
    vals = rng.standard_normal((2, 6, 50000)).astype(np.float32) * 2
    vals[0, :, 3] = -np.inf
    vals[0, 4, :] = -np.inf
    vals[1, :, 49990] = -300.0
    vals[1, 3, 0] = 200.0
    vals[1, 5, :30000] = -60000.0
    y = oracle.encode(vals, "f16")
    want = oracle.causal_softmax(y.copy(), "f16")
    got, _, _ = run(ctx, y, y.shape, None, "f16", use_workspace)
    check(got, want, "f16", "infinities and tails, long rows", max_frac=2e-2)
    assert np.isnan(oracle.decode(got, "f16")[0, 4, 0])


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(8, 1, 131072), (32, 1, 131072), (3, 2, 262144), (5, 1, 131072), (2, 1, 200000), (1, 20, 147456), (16, 2, 163848),
                                   (1, 40, 131080)])  # the last part holds 8 columns, all of them masked in the first 31 rows
def test_few_long_rows_split_over_workgroups(ctx, dt, shape):
    """Decoding over a long context (131 072 keys and more): one query row, or a few, per head.  With the workspace the
    library asks for, every row is split into parts of 16 384 (or 4096) columns on workgroups of their own (two launches);
    without it a workgroup takes a row.  Both against the oracle, and against each other: within one unit, nearly all equal."""
    from operators_amd.ops import CausalSoftmaxPlan

    rng = np.random.default_rng(shape[0] * 131 + shape[2])
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 3, dt)
    with CausalSoftmaxPlan(ctx, to_torch(y, dt).reshape(shape)) as plan:
        rows, of_16k = shape[0] * shape[1], -(-shape[2] // 16384)
        columns = 4096 if shape[2] <= 262144 and rows * of_16k <= 64 else 16384  # per workgroup
        assert plan.workspace_size == rows * -(-shape[2] // columns) * 16
    b, s_, t = shape
    want = oracle.causal_softmax(y.copy(), dt)
    split, _, _ = run(ctx, y, shape, None, dt, True)
    whole, _, _ = run(ctx, y, shape, None, dt, False)
    # the CPU path adds a row's exponentials one after the other in fp32: the longer the row, the more of its
    # quotients land on the other side of a rounding boundary (3 % of bf16 outputs at 131 072 columns, 8 % at
    # 262 144) - one unit at most, and the float64 quotient below says which side is right
    loose = 0.2
    check(split, want, dt, f"{shape} {dt} split", max_frac=loose)
    check(whole, want, dt, f"{shape} {dt} a workgroup per row", max_frac=loose)
    check(split, whole, dt, f"{shape} {dt} split against a workgroup per row", max_frac=2e-3)
    # what both are held to: the float64 quotient narrowed by the type's rule
    keep = np.broadcast_to(np.arange(t)[None, :] <= t - s_ + np.arange(s_)[:, None], shape)
    x = np.where(keep, oracle.decode(y, dt).astype(np.float64).reshape(shape), -np.inf)
    e = np.exp(x - x.max(-1, keepdims=True))
    exact = oracle.encode((e / e.sum(-1, keepdims=True)).astype(np.float32).ravel(), dt).reshape(shape)
    frac, worst = check(split.reshape(shape), exact, dt, f"{shape} {dt} split against float64", max_frac=1e-3)
    assert worst <= 1
    for i in range(s_):
        assert not split.reshape(shape)[:, i, t - s_ + i + 1:].any(), "the masked part is exact zeros"


@pytest.mark.parametrize("use_workspace", [False, True])
def test_infinities_and_long_tails_in_few_very_long_rows(ctx, use_workspace):
    """Special values where rows are split over workgroups: parts that are -inf throughout, a row that is, a part that
    holds the row's only large value, parts more than 126 below the row's maximum, +inf, NaN."""
    rng = np.random.default_rng(83)
    vals = rng.standard_normal((2, 5, 140000)).astype(np.float32) * 2
    vals[0, :, 3] = -np.inf
    vals[0, 1, 16384:49152] = -np.inf
    vals[0, 4, :] = -np.inf
    vals[1, :, 139990] = -300.0
    vals[1, 3, 70000] = 200.0
    vals[1, 2, :100000] = -60000.0
    vals[1, 0, 20000] = np.inf
    vals[1, 1, 90000] = np.nan
    y = oracle.encode(vals, "f16")
    want = oracle.causal_softmax(y.copy(), "f16")
    got, _, _ = run(ctx, y, y.shape, None, "f16", use_workspace)
    check(got, want, "f16", "infinities and tails, few very long rows", max_frac=0.2)
    out = oracle.decode(got, "f16")
    assert np.isnan(out[0, 4, 0]) and np.isnan(out[1, 0, 5]) and np.isnan(out[1, 1, 5])


def test_split_form_is_for_few_long_rows_only(ctx):
    """No workspace is asked for where a workgroup per row fills the chip, where rows are short, or where rows are
    not whole 16-byte vectors; and a strided view of few long rows takes the split form like a dense one."""
    import torch

    from operators_amd.ops import CausalSoftmaxPlan

    for shape in [(32, 4096, 4096), (200, 1, 262144), (64, 1, 131072), (8, 1, 131064), (8, 1, 140001), (8, 1, 65536)]:
        with CausalSoftmaxPlan(ctx, torch.empty(shape, dtype=torch.float16, device="cuda")) as plan:
            assert plan.workspace_size == 0, shape
    rng = np.random.default_rng(5)
    shape, strides = (6, 2, 140000), (2 * 140008 + 16, 140008, 1)
    y = oracle.encode(rng.standard_normal(shape).astype(np.float32) * 2, "f16")
    want = oracle.causal_softmax(y.copy(), "f16")
    got, before, after = run(ctx, y, shape, strides, "f16", True)
    check(got, want, "f16", "strided few long rows, split", max_frac=0.2)
    mask = np.zeros(before.size, bool)
    idx = (np.arange(6)[:, None, None] * strides[0] + np.arange(2)[None, :, None] * strides[1] + np.arange(140000)[None, None, :]).ravel()
    mask[idx] = True
    assert np.array_equal(before[~mask], after[~mask]), "the gaps between the rows are left alone"


def test_short_rows_give_the_bits_of_a_wavefront_per_row(ctx):
    """Rows of up to 1024 elements share a wavefront (8, 16 or 32 lanes each) when
    the rows of a group lie within 2 GiB of each other; rows 256 MiB apart get a
    wavefront each.  Both forms add in the same order: same data, same bits."""
    import torch

    for dt, tdt in (("f16", torch.float16), ("bf16", torch.bfloat16)):
        for total in (64, 72, 128, 136, 192, 200, 256, 264, 320, 384, 512, 520, 576, 640, 768, 896, 1000, 1024):
            seq = 8
            rng = np.random.default_rng(900 + total)
            vals = rng.standard_normal((1, seq, total)).astype(np.float32) * 3
            vals[0, 2, 1] = -np.inf
            vals[0, 5, :3] = 400.0
            codes = oracle.encode(vals, dt)
            dense = to_torch(codes, dt).reshape(1, seq, total)
            far = torch.zeros(seq << 27, dtype=tdt, device="cuda").as_strided((1, seq, total), (seq << 27, 1 << 27, 1))
            far.copy_(dense)
            ctx.causal_softmax(dense)
            ctx.causal_softmax(far)
            torch.cuda.synchronize()
            assert torch.equal(dense.view(torch.int16), far.contiguous().view(torch.int16)), (dt, total)
            del far


def test_status_codes_match_reference(ctx):
    import ctypes

    from operators_amd import infiniopCausalSoftmaxDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    for case in golden_json()["status"]:
        if case["op"] != "causal_softmax":
            continue
        t = case["tensors"][0]
        desc = make_descriptor(lib, t[1], t[2], LAYOUT[t[0]])
        d = infiniopCausalSoftmaxDescriptor_t()
        st = lib.infiniopCreateCausalSoftmaxDescriptor(ctx.handle, ctypes.byref(d), desc)
        want = 0 if case.get("bf16_extension") else (5 if case.get("cpu_only_layout") else case["status"])
        assert st == want, (case, st)
        if st == 0:
            assert lib.infiniopDestroyCausalSoftmaxDescriptor(d) == 0
        lib.infiniopDestroyTensorDescriptor(desc)
