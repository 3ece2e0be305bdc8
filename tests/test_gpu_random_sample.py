"""RandomSample on the GPU through the C ABI, against the compiled reference's
golden indices and the oracle.

Bar: the returned index is the oracle's, or - where equal logits exist - an
index holding the same logit value (the reference's own criterion,
operatorspy/tests/random_sample.py: `indices == ans or data[indices] ==
data[ans]`; the CPU's order among equal values depends on the swap history of
its selection sort, the GPU orders them by index).  For logits without ties
the index itself must agree.  Where the reference leaves the result unwritten
(random_val >= 1) the GPU must leave it unwritten too."""
import numpy as np
import pytest

import oracle
from helpers import golden, golden_json, to_torch

pytestmark = pytest.mark.gpu
CASES = golden_json()["random_sample_cases"]
SENTINEL = -12345


def gpu_sample(ctx, codes, rv, topp, topk, temp, offset=0, dt="f16"):
    """offset (elements) places the logits at an address that is not 16-byte
    aligned.  Every case runs twice: with the workspace the library asks for
    (vocabularies of 4096 and more then take the two-launch form) and without
    it (one workgroup); the two must give the same index."""
    with_ws = gpu_sample_once(ctx, codes, rv, topp, topk, temp, offset, True, dt)
    without = gpu_sample_once(ctx, codes, rv, topp, topk, temp, offset, False, dt)
    assert with_ws == without, ("with workspace", with_ws, "without", without)
    return with_ws


def gpu_sample_once(ctx, codes, rv, topp, topk, temp, offset, use_workspace, dt="f16"):
    import torch

    codes = np.ascontiguousarray(codes, np.uint16)
    if offset:
        buf = to_torch(np.concatenate([np.zeros(offset, np.uint16), codes]), dt)
        probs = buf[offset:]
    else:
        probs = to_torch(codes, dt)
    result = torch.full((1,), SENTINEL, dtype=torch.int64, device="cuda")  # the bits of a uint64
    view = result.view(torch.uint64)
    ctx.random_sample(view, probs, rv, topp, topk, temp, use_workspace=use_workspace)
    torch.cuda.synchronize()
    got = int(result.item())
    return None if got == SENTINEL else got


def same_choice(codes, got, want, dt="f16"):
    if got == want:
        return True
    if got is None or want is None:
        return False
    v = oracle.decode(np.asarray(codes, np.uint16), dt)
    return 0 <= got < v.size and float(v[got]) == float(v[want])


@pytest.mark.parametrize("i", range(len(CASES)))
def test_golden_cases(ctx, i):
    voc, rv, topp, topk, temp, kind = CASES[i]
    g = golden("random_sample")
    x = g[f"rs{i}_logits"]
    want = int(g["rs_index"][i])
    want = None if want < 0 else want
    got = gpu_sample(ctx, x, rv, topp, topk, temp)
    assert same_choice(x, got, want), (CASES[i], got, want)
    if kind in ("uniform", "normal") and np.unique(x).size == x.size:
        assert got == want


@pytest.mark.parametrize("offset", [0, 3])
def test_against_oracle_distinct_logits(ctx, offset):
    """No two logits equal: the index itself must be the oracle's."""
    rng = np.random.default_rng(21 + offset)
    pool = np.arange(0x0400, 0x7C00, dtype=np.uint16)  # every positive normal fp16 code
    pool = np.concatenate([pool, pool | 0x8000])
    bad = []
    for trial in range(120):
        voc = int(rng.choice([2, 7, 8, 9, 63, 500, 1024, 4096, 8191, 8200, 32000, 50257]))
        x = rng.choice(pool, voc, replace=False)
        scale = rng.choice([0, 1, 2])  # squeeze the range so several candidates carry weight
        if scale:
            v = x.view(np.float16).astype(np.float32)
            v = np.sign(v) * np.log1p(np.abs(v)) * (1.0 if scale == 1 else 0.3)
            x = np.unique(v.astype(np.float16).view(np.uint16))
            x = x[(x & 0x7FFF) != 0]
            rng.shuffle(x)
            voc = x.size
        args = (float(rng.random()), float(rng.choice([0.0, 0.3, 0.8, 0.95, 1.0])), int(rng.choice([1, 2, 3, 5, 20, 50, 200, 1024])),
                float(rng.choice([0.5, 1.0, 2.0, 10.0])))
        want = oracle.random_sample(x, *args)
        got = gpu_sample(ctx, x, *args, offset=offset)
        if got != want:
            bad.append((trial, voc, args, got, want))
    assert not bad, bad[:5]


def test_against_oracle_with_ties(ctx):
    rng = np.random.default_rng(77)
    bad = []
    for trial in range(80):
        voc = int(rng.choice([5, 64, 777, 4096, 32000, 151936]))
        kind = trial % 3
        if kind == 0:
            x = rng.random(voc, dtype=np.float32).astype(np.float16)  # the reference test's distribution: many ties at 32000
        elif kind == 1:
            x = (rng.standard_normal(voc, dtype=np.float32) * 2.5).astype(np.float16)
        else:
            x = rng.choice(np.array([-3.0, -0.0, 0.0, 0.5, 0.5009765625, 4.0], np.float16), voc)
        codes = x.view(np.uint16)
        args = (float(rng.random()), float(rng.choice([0.0, 0.5, 0.9, 1.0])), int(rng.choice([1, 2, 4, 10, 50, 300, 1024, 5000])),
                float(rng.choice([0.5, 1.0, 2.0])))
        want = oracle.random_sample(codes, *args)
        got = gpu_sample(ctx, codes, *args)
        if not same_choice(codes, got, want):
            bad.append((trial, voc, args, got, want))
    assert not bad, bad[:5]


def test_equal_logits_come_in_index_order(ctx):
    """A flat distribution over the candidates (huge temperature, topp = 1):
    random_val picks by rank, and equal logits are ranked by ascending index."""
    x = np.full(4000, 1.0, np.float16)
    x[[17, 1800, 3999]] = 2.0
    codes = x.view(np.uint16)
    k = 8
    expect = [17, 1800, 3999, 0, 1, 2, 3, 4]
    for r in range(k):
        assert gpu_sample(ctx, codes, (r + 0.5) / k, 1.0, k, 1e9) == expect[r]


def test_greedy_special_values(ctx):
    x = (np.random.default_rng(1).standard_normal(5000) * 2).astype(np.float16)
    codes = x.view(np.uint16).copy()
    assert gpu_sample(ctx, codes, 0.5, 0.0, 5, 1.0) == int(np.argmax(x))
    assert gpu_sample(ctx, codes, 0.5, 0.9, 1, 1.0) == int(np.argmax(x))
    assert gpu_sample(ctx, codes, 0.5, 0.9, -7, 1.0) == int(np.argmax(x))
    c = codes.copy()
    c[2500] = 0x7E00  # a NaN further back is never greater than anything
    assert gpu_sample(ctx, c, 0.5, 0.0, 1, 1.0) == oracle.random_sample(c, 0.5, 0.0, 1, 1.0) == int(np.argmax(x))
    c[0] = 0x7E00     # a NaN in front is never beaten
    assert gpu_sample(ctx, c, 0.5, 0.0, 1, 1.0) == oracle.random_sample(c, 0.5, 0.0, 1, 1.0) == 0
    c = np.full(300, 0xFC00, np.uint16)  # all -Inf: the first
    assert gpu_sample(ctx, c, 0.5, 0.0, 1, 1.0) == 0
    c[123] = 0x8000
    c[200] = 0x0000   # -0 and +0 are equal: the first of them
    assert gpu_sample(ctx, c, 0.5, 0.0, 1, 1.0) == oracle.random_sample(c, 0.5, 0.0, 1, 1.0) == 123


def test_limits(ctx):
    import torch

    from operators_amd.ops import RandomSamplePlan
    from operators_amd.utils import InfiniopError

    probs = to_torch((np.random.default_rng(2).standard_normal(4096)).astype(np.float16).view(np.uint16), "f16")
    result = torch.zeros(1, dtype=torch.int64, device="cuda").view(torch.uint64)
    with RandomSamplePlan(ctx, result, probs) as plan:
        assert 0 < plan.workspace_size <= 48 * 16 + 65536 * 4  # headers + a count per 16-bit key, whatever the vocabulary
        plan(result, probs, 0.5, 0.9, 256, 1.0)           # the largest candidate count ranked in LDS
        plan(result, probs, 0.5, 0.9, 257, 1.0)           # beyond it: the histogram walk, no limit on topk
        plan(result, probs, 0.5, 0.9, 1025, 1.0)
        plan(result, probs, 0.5, 0.9, 2 ** 31 - 1, 1.0)   # clamped to the vocabulary, as in the reference
        torch.cuda.synchronize()
        plan(result, probs, 0.5, 0.0, 100000, 1.0)        # greedy form: topk is not looked at
        torch.cuda.synchronize()
    # random_val = 1: the reference writes nothing, neither does the kernel
    codes = (np.random.default_rng(3).standard_normal(640)).astype(np.float16).view(np.uint16)
    assert oracle.random_sample(codes, 1.0, 0.9, 6, 1.0) is None
    assert gpu_sample(ctx, codes, 1.0, 0.9, 6, 1.0) is None
    # one logit
    assert gpu_sample(ctx, codes[:1], 0.5, 0.9, 4, 1.0) == 0
    assert gpu_sample(ctx, codes[:1], 0.5, 0.0, 1, 1.0) == 0


def test_lists_that_overflow_fall_back_to_the_full_path(ctx):
    """More equal logits at the top than a workgroup's candidate list holds,
    and candidate counts close to the two-launch form's limit: the second
    launch notices and works from the logits itself."""
    rng = np.random.default_rng(13)
    x = (rng.standard_normal(32000, dtype=np.float32)).astype(np.float16)
    x[rng.choice(32000, 9000, replace=False)] = 6.0   # 9000 equal maxima: every list overflows
    codes = x.view(np.uint16)
    for args in ((0.4, 0.9, 50, 1.0), (0.77, 1.0, 256, 2.0), (0.1, 0.5, 2, 0.5)):
        want = oracle.random_sample(codes, *args)
        assert same_choice(codes, gpu_sample(ctx, codes, *args), want), args
    y = (rng.standard_normal(20000, dtype=np.float32) * 2).astype(np.float16).view(np.uint16)
    for topk in (200, 255, 256, 257):
        args = (0.63, 0.97, topk, 1.3)
        assert same_choice(y, gpu_sample(ctx, y, *args), oracle.random_sample(y, *args)), args
    # the last workgroup holds fewer lanes with data than topk
    z = (rng.standard_normal(4096 + 8 * 30 + 3, dtype=np.float32) * 2).astype(np.float16).view(np.uint16)
    for topk in (20, 40, 100):
        args = (0.5, 0.9, topk, 1.0)
        assert same_choice(z, gpu_sample(ctx, z, *args), oracle.random_sample(z, *args)), args


def test_bf16_extension_against_oracle(ctx):
    """bf16 logits (accepted here, refused by the reference): against the
    oracle's bf16 form - same arithmetic, probabilities rounded to nearest
    even.  Parity unpinned by the reference."""
    rng = np.random.default_rng(31)
    bad = []
    for trial in range(60):
        voc = int(rng.choice([3, 100, 4096, 5000, 32000, 128256]))
        x = oracle.f32_to_bf16((rng.standard_normal(voc, dtype=np.float32) * (3.0 if trial % 2 else 0.7)).astype(np.float32))
        if trial % 3 == 0:  # distinct codes only
            x = np.unique(x)
            x = x[(x & 0x7FFF) != 0]
            rng.shuffle(x)
            voc = x.size
        args = (float(rng.random()), float(rng.choice([0.0, 0.5, 0.9, 1.0])), int(rng.choice([1, 2, 8, 50, 256, 600])), float(rng.choice([0.5, 1.0, 2.0])))
        want = oracle.random_sample(x, *args, dtype="bf16")
        got = gpu_sample(ctx, x, *args, dt="bf16")
        if not same_choice(x, got, want, "bf16") or (trial % 3 == 0 and got != want):
            bad.append((trial, voc, args, got, want))
    assert not bad, bad[:5]
    # the codes are read as bf16, not as fp16: 1.0, 2.0, then fp16's 1.0 (bf16 0.0078125)
    assert gpu_sample(ctx, np.array([0x3F80, 0x4000, 0x3C00], np.uint16), 0.5, 0.0, 1, 1.0, dt="bf16") == 1


def test_large_vocabulary(ctx):
    rng = np.random.default_rng(8)
    for voc in (151936, 1_000_003):
        x = (rng.standard_normal(voc, dtype=np.float32) * 3).astype(np.float16).view(np.uint16)
        for args in ((0.37, 0.9, 40, 0.8), (0.9, 0.0, 1, 1.0)):
            want = oracle.random_sample(x, *args)
            got = gpu_sample(ctx, x, *args)
            assert same_choice(x, got, want), (voc, args, got, want)


@pytest.mark.parametrize("voc,topk", [(1025, 1025), (5000, 1025), (5000, 5000), (8191, 3000), (20000, 100000), (34000, 2048)])
def test_more_candidates_than_lds_ranks_distinct_logits(ctx, voc, topk):
    """topk beyond 1024 (the reference has no limit, random_sample.cc:67-74): no
    two logits equal, so the index itself must be the oracle's - for top-p
    values that stop the walk early, late and never.

    The draw compares a running sum of thousands of fp16 probabilities with a
    limit; the GPU's expf and the order in which it adds up the softmax
    denominator differ from the host's in the last bit, which can move one
    probability by an fp16 unit and with it the crossing point by one rank.
    For the nearly flat distributions (hundreds to thousands of entries kept)
    a result one rank away from the oracle's is therefore accepted, at most
    once per case; the peaked ones must agree exactly."""
    rng = np.random.default_rng(500 + voc + topk)
    pool = np.arange(0x0400, 0x4801, dtype=np.uint16)  # every normal fp16 code up to 8.0, so that the distribution is not one spike
    pool = np.concatenate([pool, pool | 0x8000])
    codes = rng.choice(pool, voc, replace=False)
    order = np.argsort(-oracle.decode(codes, "f16"), kind="stable")
    rank = np.empty(voc, np.int64)
    rank[order] = np.arange(voc)
    bad, near = [], []
    for rv, topp, temp, flat in [(0.37, 0.9, 1.0, False), (0.999, 1.0, 2.0, True), (0.05, 0.5, 0.7, False), (0.93, 0.9999, 5.0, True),
                                 (0.5, 1e-4, 1.0, False), (0.71, 1.0, 50.0, True)]:
        want = oracle.random_sample(codes, rv, topp, topk, temp)
        got = gpu_sample(ctx, codes, rv, topp, topk, temp)
        if got == want:
            continue
        if flat and got is not None and want is not None and abs(int(rank[got]) - int(rank[want])) <= 1:
            near.append((rv, topp, temp, got, want))
        else:
            bad.append((rv, topp, temp, got, want))
    assert not bad, bad
    assert len(near) <= 1, near


def test_more_candidates_than_lds_ranks_with_ties(ctx):
    """The reference test's own distribution (uniform [0, 1) in fp16: a few
    thousand distinct values) with topk up to the whole vocabulary: an index
    holding the same logit as the oracle's."""
    rng = np.random.default_rng(91)
    bad = []
    for trial in range(24):
        voc = int(rng.choice([2000, 4096, 16000]))
        x = rng.random(voc, dtype=np.float32).astype(np.float16) if trial % 2 else (rng.standard_normal(voc, dtype=np.float32) * 3).astype(np.float16)
        codes = x.view(np.uint16)
        args = (float(rng.random()), float(rng.choice([0.3, 0.9, 1.0])), int(rng.choice([1025, 1500, 4096, voc, 10 ** 6])), float(rng.choice([0.5, 1.0, 3.0])))
        want = oracle.random_sample(codes, *args)
        got = gpu_sample(ctx, codes, *args)
        if not same_choice(codes, got, want):
            bad.append((trial, voc, args, got, want))
    assert not bad, bad[:5]


def test_more_candidates_few_distinct_logits(ctx):
    """The walk over more than 1024 candidates takes 64 keys at a time while the
    running sum stays below 1.0 and entry by entry beyond it.  Distributions
    that put both to work: every logit equal (one key holding the whole
    vocabulary: the entry inside the key comes from a division), two and
    three levels, one dominant logit (the running sum is 1.0 after the first
    entry and everything after it adds nothing or a last unit), logits so far
    apart that most probabilities are zero, and the entry limit (topk) falling
    inside a key.  All ties, so the logit at the drawn index must be the
    oracle's; where the oracle leaves the result unwritten, so must the GPU."""
    rng = np.random.default_rng(7)
    f = lambda *v: np.asarray(v, np.float16).view(np.uint16)  # noqa: E731
    bad = []
    cases = []
    for voc in (1500, 4100, 9000):
        cases.append(("all equal", np.full(voc, f(0.25)[0], np.uint16)))
        cases.append(("two levels", rng.choice(f(1.0, -1.0), voc)))
        cases.append(("three levels", rng.choice(f(2.0, 1.5, -3.0), voc, p=[0.01, 0.09, 0.9])))
        one = np.full(voc, f(-20.0)[0], np.uint16)
        one[voc // 3] = f(12.0)[0]
        cases.append(("one dominant", one))
        far = rng.choice(f(30.0, 0.0, -40.0), voc, p=[0.002, 0.5, 0.498])
        cases.append(("far apart", far))
        cases.append(("eight values", rng.choice(f(0.0, 0.5, 1.0, 1.5, 2.0, 2.5, 3.0, 3.5), voc)))
    for what, codes in cases:
        voc = codes.size
        for rv, topp, topk, temp in [(0.37, 0.9, voc, 1.0), (0.999, 1.0, voc, 1.0), (0.0, 1.0, voc, 0.5), (0.6, 0.5, 1025, 2.0),
                                     (0.95, 1.0, voc - 7, 1.0), (0.5, 1e-3, voc, 1.0), (0.9999, 0.99, 2 * voc, 4.0), (1.0, 1.0, voc, 1.0)]:
            want = oracle.random_sample(codes, rv, topp, topk, temp)
            got = gpu_sample(ctx, codes, rv, topp, topk, temp)
            if not same_choice(codes, got, want):
                bad.append((what, voc, (rv, topp, topk, temp), got, want))
    assert not bad, bad[:6]


def test_more_candidates_bf16_still_adds_entry_by_entry(ctx):
    """bf16 probabilities are finer than the 2^-24 units the fast walk counts
    in, so bf16 logits keep the one-by-one chain: against the oracle's bf16
    extension on tie-heavy inputs."""
    rng = np.random.default_rng(8)
    bad = []
    for voc in (1400, 5000):
        x = rng.integers(-24, 24, voc).astype(np.float32) / 4
        codes = oracle.encode(x, "bf16")
        for rv, topp, topk, temp in [(0.37, 0.9, voc, 1.0), (0.99, 1.0, voc, 2.0), (0.2, 0.6, 2000, 0.7)]:
            want = oracle.random_sample(codes, rv, topp, topk, temp, "bf16")
            got = gpu_sample(ctx, codes, rv, topp, topk, temp, dt="bf16")
            if not same_choice(codes, got, want, "bf16"):
                bad.append((voc, (rv, topp, topk, temp), got, want))
    assert not bad, bad
