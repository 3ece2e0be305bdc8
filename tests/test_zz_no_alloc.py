"""infiniopRandomSampleNoAlloc - the one entry point that takes no workspace and
allocates nothing (what its first launches leave for the drawing workgroup -
candidate lists, or a count per key - lives in an array the library keeps on
the GPU) - against infiniopRandomSample with a workspace, through the C ABI.

Bar: the same index, exactly (both run the same kernels on the same logits).
Two calls in a row, the second on a smaller vocabulary, so that whatever the
first left behind in the shared array would show; then the size limit."""
import ctypes

import numpy as np
import pytest

import oracle
from helpers import to_torch

pytestmark = pytest.mark.gpu
SENTINEL = -777


def draw(ctx, codes, rv, topp, topk, temp, entry, dtype="f16"):
    import torch

    from operators_amd.ops import RandomSamplePlan

    probs = to_torch(np.ascontiguousarray(codes, np.uint16), dtype)
    result = torch.full((1,), SENTINEL, dtype=torch.int64, device="cuda")
    view = result.view(torch.uint64)
    with RandomSamplePlan(ctx, view, probs, use_workspace=True) as plan:
        if entry == "no_alloc":
            plan.no_alloc(view, probs, rv, topp, topk, temp)
        else:
            plan(view, probs, rv, topp, topk, temp)
        torch.cuda.synchronize()
    return int(result.item())


def logits(rng, voc):
    return oracle.encode((rng.standard_normal(voc) * 3).astype(np.float32), "f16")


def test_two_calls_in_a_row_second_one_smaller(ctx):
    rng = np.random.default_rng(77)
    # 151 936 logits fill 38 of the 48 lists; 32 000 fill 16; 5 000 three; 1 000 take the one-workgroup form
    for voc in (151936, 32000, 5000, 1000):
        x = logits(rng, voc)
        # top-k 50 and 256: candidate lists in the array; 257 and "off": a count per key in the same array;
        # alternating, so that each form finds what the other left there
        for rv, topp, topk, temp in ((0.37, 0.9, 50, 0.8), (0.41, 0.9, voc, 0.8), (0.92, 0.95, 256, 1.3), (0.77, 1.0, 257, 1.0),
                                     (0.05, 1.0, 7, 0.5), (0.3, 0.99, 2 ** 31 - 1, 2.0), (0.5, 0.0, 1, 1.0)):
            want = draw(ctx, x, rv, topp, topk, temp, "workspace")
            got = draw(ctx, x, rv, topp, topk, temp, "no_alloc")
            assert got == want != SENTINEL, (voc, rv, topp, topk, temp, got, want)
            if min(topk, voc) * voc <= 2 * 10 ** 8:  # the oracle's selection loop is O(topk * voc): seconds beyond this
                ref = oracle.random_sample(x, rv, topp, topk, temp)
                assert got == ref or x[got] == x[ref], (voc, rv, topp, topk, temp, got, ref)


def test_bf16_logits_and_a_random_value_of_one(ctx):
    """The extension type, and the draw that falls off the end of the cumulative distribution (random_val = 1: the
    reference's loop then finds no candidate and leaves the result as it was; with one logit, sampling asked for,
    nothing is launched at all)."""
    rng = np.random.default_rng(79)
    for voc in (40000, 6000, 700):
        x = oracle.encode((rng.standard_normal(voc) * 3).astype(np.float32), "bf16")
        for rv, topp, topk, temp in ((0.37, 0.9, 50, 0.8), (0.66, 1.0, 300, 1.0), (1.0, 0.9, 50, 0.8), (0.5, 0.0, 1, 1.0)):
            want = draw(ctx, x, rv, topp, topk, temp, "workspace", "bf16")
            got = draw(ctx, x, rv, topp, topk, temp, "no_alloc", "bf16")
            assert got == want, (voc, rv, topp, topk, temp, got, want)
    x16 = logits(rng, 33000)
    for rv in (1.0, 1.5):
        want = draw(ctx, x16, rv, 0.9, 50, 0.8, "workspace")
        assert draw(ctx, x16, rv, 0.9, 50, 0.8, "no_alloc") == want
        ref = oracle.random_sample(x16, rv, 0.9, 50, 0.8)  # None: the reference leaves the result unwritten
        assert (want == SENTINEL) if ref is None else (want == ref or x16[want] == x16[ref]), (rv, want, ref)
    one = logits(rng, 1)
    for entry in ("workspace", "no_alloc"):
        assert draw(ctx, one, 1.0, 0.9, 2, 1.0, entry) == SENTINEL  # nothing wins, nothing is written
        assert draw(ctx, one, 0.3, 0.9, 2, 1.0, entry) == 0


def test_repeated_calls_share_the_array_in_stream_order(ctx):
    """Back-to-back calls on one stream without a host wait in between: each
    one's two launches are ordered behind the previous one's."""
    import torch

    from operators_amd.ops import RandomSamplePlan

    rng = np.random.default_rng(78)
    xs = [logits(rng, voc) for voc in (40000, 9000, 33000, 4096)]
    probs = [to_torch(x, "f16") for x in xs]
    results = [torch.full((1,), SENTINEL, dtype=torch.int64, device="cuda") for _ in xs]
    plans = [RandomSamplePlan(ctx, r.view(torch.uint64), p, use_workspace=True) for r, p in zip(results, probs)]
    for plan, r, p in zip(plans, results, probs):
        plan.no_alloc(r.view(torch.uint64), p, 0.61, 0.9, 40, 0.9)
    torch.cuda.synchronize()
    for plan, r, p, x in zip(plans, results, probs, xs):
        want = torch.full((1,), SENTINEL, dtype=torch.int64, device="cuda")
        plan(want.view(torch.uint64), p, 0.61, 0.9, 40, 0.9)
        torch.cuda.synchronize()
        assert int(r.item()) == int(want.item()) != SENTINEL
        plan.close()


def test_size_limit_is_an_error_not_a_fault(ctx):
    import torch

    from operators_amd.ops import RandomSamplePlan

    voc = (1 << 20) + 8
    probs = torch.zeros(voc, dtype=torch.float16, device="cuda")
    result = torch.full((1,), SENTINEL, dtype=torch.int64, device="cuda")
    with RandomSamplePlan(ctx, result.view(torch.uint64), probs, use_workspace=False) as plan:
        st = ctx.lib.infiniopRandomSampleNoAlloc(plan.desc, result.data_ptr(), probs.data_ptr(), ctypes.c_float(0.3), ctypes.c_float(0.9), 50,
                                                 ctypes.c_float(1.0), None)
        assert st == 2  # STATUS_BAD_PARAM
        torch.cuda.synchronize()
        assert int(result.item()) == SENTINEL
