"""The oracle's RandomSample against what pins it (no GPU):
  * the golden indices written by the compiled reference
    (tests/golden/random_sample.npz, cases in status_cases.json),
  * the compiled reference itself on fresh inputs, where it is present,
  * an independent model for logits without ties: numpy's argsort instead of
    the selection sort, float64 softmax with an error margin instead of the
    fp32 one,
  * closed forms: a tiny topp or random_val = 0 returns the maximum, a huge
    temperature makes the kept candidates equally likely so random_val picks
    by rank, the greedy form is numpy's argmax.
"""
import numpy as np
import pytest

import oracle
from helpers import golden, golden_json
from oracle import ref

CASES = golden_json()["random_sample_cases"]


def f16(codes, dt="f16"):
    return oracle.decode(np.asarray(codes, np.uint16), dt).astype(np.float64)


@pytest.mark.parametrize("i", range(len(CASES)))
def test_golden(i):
    voc, rv, topp, topk, temp, _kind = CASES[i]
    g = golden("random_sample")
    want = int(g["rs_index"][i])
    got = oracle.random_sample(g[f"rs{i}_logits"], rv, topp, topk, temp)
    assert (-1 if got is None else got) == want


@pytest.mark.skipif(not ref.available(), reason="compiled reference not built")
def test_vs_compiled_reference_on_fresh_inputs():
    rng = np.random.default_rng(5)
    for trial in range(60):
        voc = int(rng.integers(1, 3000))
        kind = trial % 3
        if kind == 0:
            x = rng.random(voc, dtype=np.float32).astype(np.float16)
        elif kind == 1:
            x = (rng.standard_normal(voc, dtype=np.float32) * 4).astype(np.float16)
        else:
            x = rng.choice(np.array([-2.0, 0.5, 0.75, 1.0], np.float16), voc)
        args = (float(rng.random()), float(rng.choice([0.0, 0.5, 0.9, 1.0])), int(rng.integers(0, 40)), float(rng.choice([0.5, 1.0, 2.0])))
        assert oracle.random_sample(x.view(np.uint16), *args) == ref.random_sample(x.view(np.uint16), *args), (trial, voc, args)


def model_without_ties(x, rv, topp, topk, temp, dt="f16"):
    """Candidates by argsort; probabilities in float64.  Returns the set of
    indices the fp32/fp16 arithmetic of the operator may land on: the float64
    answer and its neighbours in the sorted order when a threshold falls
    within rounding distance of a running sum."""
    v = f16(x, dt)
    order = np.argsort(-v, kind="stable")
    k = min(topk, v.size)
    p = np.exp((v - v[order[0]]) / temp)
    p = (p / p.sum())[order[:k]]
    cum = np.cumsum(p)
    slack = 4e-3  # rounding of each probability to 11 (fp16) or 8 (bf16) bits, summed over the candidates: below 2^-9

    def first_above(limit, upto):
        hit = np.flatnonzero(limit < cum[:upto])
        return int(hit[0]) if hit.size else None

    def first_reaching(bound):
        hit = np.flatnonzero(cum >= bound)
        return int(hit[0]) if hit.size else k

    ends = set()
    for e in range(first_reaching(topp - slack), first_reaching(topp + slack) + 1):
        ends.add(e + 1 if e < k - 1 else k)
    allowed = set()
    for end in ends:
        lo, hi = first_above(rv * cum[end - 1] - slack, end), first_above(rv * cum[end - 1] + slack, end)
        if lo is not None:
            allowed.update(int(order[i]) for i in range(lo, (hi if hi is not None else end - 1) + 1))
    return allowed


def test_model_without_ties():
    rng = np.random.default_rng(11)
    for trial in range(40):
        voc = int(rng.integers(50, 5000))
        x = rng.permutation(np.arange(-voc // 2, voc - voc // 2)).astype(np.float32)  # all distinct
        x = (x * (12.0 / voc)).astype(np.float16)
        if np.unique(x).size != voc:
            x = np.unique(rng.standard_normal(4 * voc).astype(np.float16))[:voc].copy()
            rng.shuffle(x)
            voc = x.size
        rv, topp, topk, temp = float(rng.random() * 0.98), float(rng.choice([0.3, 0.7, 0.95])), int(rng.integers(2, 30)), float(rng.choice([0.7, 1.0, 1.8]))
        got = oracle.random_sample(x.view(np.uint16), rv, topp, topk, temp)
        assert got in model_without_ties(x.view(np.uint16), rv, topp, topk, temp), (trial, voc, rv, topp, topk, temp, got)


def test_closed_forms():
    rng = np.random.default_rng(3)
    x = np.unique((rng.standard_normal(3000) * 3).astype(np.float16))
    rng.shuffle(x)
    codes = x.view(np.uint16)
    top = int(np.argmax(x))
    # the first running sum already reaches a tiny topp: one candidate is kept
    assert oracle.random_sample(codes, 0.999, 1e-6, 10, 1.0) == top
    # random_val = 0 is below the first running sum whatever is kept
    assert oracle.random_sample(codes, 0.0, 0.9, 10, 1.0) == top
    # greedy form
    assert oracle.random_sample(codes, 0.5, 0.0, 10, 1.0) == top
    assert oracle.random_sample(codes, 0.5, 0.9, 1, 1.0) == top
    assert oracle.random_sample(codes, 0.5, 0.9, -3, 1.0) == top
    # random_val = 1 never lies below a running sum: nothing is written
    assert oracle.random_sample(codes, 1.0, 0.9, 10, 1.0) is None
    # a huge temperature flattens the distribution: with topp = 1 all topk candidates are kept with
    # equal probabilities, so random_val chooses by rank
    order = np.argsort(-x.astype(np.float64), kind="stable")
    k = 8
    for r in range(k):
        assert oracle.random_sample(codes, (r + 0.5) / k, 1.0, k, 1e9) == int(order[r])
    # topk beyond the vocabulary is clamped to it
    small = codes[:5]
    assert oracle.random_sample(small, 0.0, 0.9, 50, 1.0) == int(np.argmax(x[:5]))


def test_equal_logits_choose_among_the_equal():
    """With ties the reference's order among equal values depends on the swap
    history; whatever it is, the chosen logit has the value the rank demands."""
    x = np.array([1.0] * 6 + [3.0] * 3 + [2.0] * 4, np.float16)
    rng = np.random.default_rng(0)
    rng.shuffle(x)
    codes = x.view(np.uint16)
    srt = np.sort(x.astype(np.float64))[::-1]
    for r in range(10):
        got = oracle.random_sample(codes, (r + 0.5) / 10, 1.0, 10, 1e9)
        assert float(x[got]) == srt[r]


def test_bf16_extension():
    """bf16 logits are this project's extension (the reference refuses them):
    PARITY UNPINNED by the reference.  Pinned here by the same closed forms
    and the same independent model as fp16."""
    rng = np.random.default_rng(17)
    vals = np.unique(oracle.f32_to_bf16((rng.standard_normal(6000) * 3).astype(np.float32)))
    vals = vals[(vals & 0x7FFF) != 0]
    rng.shuffle(vals)
    x = oracle.decode(vals, "bf16").astype(np.float64)
    top = int(np.argmax(x))
    assert oracle.random_sample(vals, 0.999, 1e-6, 10, 1.0, "bf16") == top
    assert oracle.random_sample(vals, 0.0, 0.9, 10, 1.0, "bf16") == top
    assert oracle.random_sample(vals, 0.5, 0.0, 10, 1.0, "bf16") == top
    assert oracle.random_sample(vals, 1.0, 0.9, 10, 1.0, "bf16") is None
    order = np.argsort(-x, kind="stable")
    for r in range(8):
        assert oracle.random_sample(vals, (r + 0.5) / 8, 1.0, 8, 1e9, "bf16") == int(order[r])
    for trial in range(30):
        rv, topp, topk, temp = float(rng.random() * 0.98), float(rng.choice([0.3, 0.7, 0.95])), int(rng.integers(2, 30)), float(rng.choice([0.7, 1.0, 1.8]))
        got = oracle.random_sample(vals, rv, topp, topk, temp, "bf16")
        assert got in model_without_ties(vals, rv, topp, topk, temp, "bf16"), (trial, rv, topp, topk, temp, got)
    # the same codes read as fp16 mean other values: the type argument matters
    assert oracle.random_sample(np.array([0x3F80, 0x4000, 0x3C00], np.uint16), 0.5, 0.0, 1, 1.0, "bf16") == 1
