"""The Attention composite (KV-cache write, q K^T, causal softmax, P V, head
transpose) on the GPU through the C ABI, against the oracle's composition of
the reference's CPU operators (which matches the compiled reference's own
infiniopAttention bit for bit, tests/test_oracle_ops.py).

Bar: the reference's test tolerance rtol 1e-2 (operatorspy/tests/attention.py:179)
plus an absolute term of four output ulps at the magnitude of v - the two
GEMMs round to nearest on the GPU and truncate on the CPU, and the result is a
weighted mean of v, so elements near zero carry the rounding of ones that are
not.  The caches must hold k and v exactly (a copy)."""
import numpy as np
import pytest

import oracle
from helpers import strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
ULP = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7}

CASES = [
    # n_q_head, n_kv_head, seq, head_dim, pos, capacity, q/k/v strides, cache strides   (first three: operatorspy/tests/attention.py:310-358)
    (32, 4, 5, 64, 0, 2048, (64, 2560, 1), (64, 11264, 1)),
    (32, 4, 1, 64, 3, 2048, (64, 2560, 1), (64, 11264, 1)),
    (8, 4, 2, 16, 1, 8, None, None),
    (64, 8, 200, 128, 56, 256, (128, 80 * 128, 1), None),  # a Llama-70B-shaped layer: q, k, v views of one fused qkv buffer
    (16, 16, 33, 64, 0, 40, None, (64, 16 * 64, 1)),         # no grouping, token-major caches
]


def strided_np(x, strides):
    span = 1 + sum((n - 1) * s for n, s in zip(x.shape, strides))
    buf = np.zeros(span, x.dtype)
    view = np.lib.stride_tricks.as_strided(buf, x.shape, [s * x.itemsize for s in strides])
    view[...] = x
    return view


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(CASES)))
def test_against_oracle(ctx, dt, case):
    import torch

    heads, kv_heads, seq, hd, pos, cap, qkv_st, cache_st = CASES[case]
    rng = np.random.default_rng(500 + case)
    enc = lambda s: oracle.encode(rng.standard_normal(s).astype(np.float32), dt)  # noqa: E731
    q, k, v = enc((heads, seq, hd)), enc((kv_heads, seq, hd)), enc((kv_heads, seq, hd))
    kc, vc = enc((kv_heads, cap, hd)), enc((kv_heads, cap, hd))

    dev = lambda x, st: strided_like(x, x.shape, st, dt)[0] if st else to_torch(x, dt)  # noqa: E731
    tq, tk, tv = dev(q, qkv_st), dev(k, qkv_st), dev(v, qkv_st)
    tkc, tvc = dev(kc, cache_st), dev(vc, cache_st)
    tout = torch.zeros((seq, heads, hd), dtype=tq.dtype, device="cuda")
    ctx.attention(tout, tq, tk, tv, tkc, tvc, pos)
    torch.cuda.synchronize()

    want_kc, want_vc = kc.copy(), vc.copy()
    want = oracle.attention(np.zeros((seq, heads, hd), np.uint16), q, k, v, want_kc, want_vc, pos, dt)
    assert np.array_equal(to_codes(tkc), want_kc) and np.array_equal(to_codes(tvc), want_vc), "cache contents"
    g, r = oracle.decode(to_codes(tout), dt).astype(np.float64), oracle.decode(want, dt).astype(np.float64)
    vmax = float(np.abs(oracle.decode(want_vc[:, : pos + seq], dt)).max())
    tol = 1e-2 * np.abs(r) + 4 * ULP[dt] * vmax
    assert np.all(np.abs(g - r) <= tol), (float(np.max(np.abs(g - r) - tol)), case, dt)


def test_against_float64_attention(ctx):
    """Independent of the oracle: plain float64 attention over the cache."""
    import torch

    heads, kv_heads, seq, hd, pos, cap = 8, 2, 16, 32, 5, 32
    rng = np.random.default_rng(77)
    enc = lambda s: oracle.encode(rng.standard_normal(s).astype(np.float32), "f16")  # noqa: E731
    q, k, v, kc, vc = enc((heads, seq, hd)), enc((kv_heads, seq, hd)), enc((kv_heads, seq, hd)), enc((kv_heads, cap, hd)), enc((kv_heads, cap, hd))
    tout = torch.zeros((seq, heads, hd), dtype=torch.float16, device="cuda")
    ctx.attention(tout, to_torch(q, "f16"), to_torch(k, "f16"), to_torch(v, "f16"), to_torch(kc, "f16"), to_torch(vc, "f16"), pos)
    torch.cuda.synchronize()
    f = lambda x: oracle.decode(x, "f16").astype(np.float64)  # noqa: E731
    K, V = f(kc), f(vc)
    K[:, pos:pos + seq], V[:, pos:pos + seq] = f(k), f(v)
    total = pos + seq
    out = np.zeros((seq, heads, hd))
    for h in range(heads):
        s = f(q)[h] @ K[h // (heads // kv_heads), :total].T / np.sqrt(hd)
        s = np.where(np.arange(total)[None, :] <= pos + np.arange(seq)[:, None], s, -np.inf)
        p = np.exp(s - s.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        out[:, h] = p @ V[h // (heads // kv_heads), :total]
    got = f(to_codes(tout))
    assert np.all(np.abs(got - out) <= 1e-2 * np.abs(out) + 6 * 2.0 ** -10 * np.abs(V).max())


def test_decoding_over_a_long_context(ctx):
    """One new token against 131 071 cached ones: the scores are 8 rows of 131 072 columns, which CausalSoftmax
    splits over workgroups through its share of Attention's workspace; both products are this library's own kernels
    (the second through its share of the workspace).  Against plain float64 attention."""
    import torch

    from operators_amd.ops import AttentionPlan

    heads, kv_heads, seq, hd, pos, cap = 8, 2, 1, 64, 131071, 131072
    rng = np.random.default_rng(78)
    enc = lambda s: oracle.encode(rng.standard_normal(s).astype(np.float32), "f16")  # noqa: E731
    q, k, v, kc, vc = enc((heads, seq, hd)), enc((kv_heads, seq, hd)), enc((kv_heads, seq, hd)), enc((kv_heads, cap, hd)), enc((kv_heads, cap, hd))
    tout = torch.zeros((seq, heads, hd), dtype=torch.float16, device="cuda")
    tq, tk, tv, tkc, tvc = (to_torch(x, "f16") for x in (q, k, v, kc, vc))
    with AttentionPlan(ctx, tout, tq, tk, tv, tkc, tvc, pos) as plan:
        scores, result, parts = heads * seq * cap * 2, heads * seq * hd * 2, heads * seq * (cap // 4096) * 16
        weighted = kv_heads * (cap // 512) * hd * 8 * 4  # the second Matmul's partial sums: chunks of 512 keys, 8 columns of fp32 per chunk
        assert result % 16 == 0  # (one token: the head-major result is out itself and takes no workspace)
        assert plan.workspace_size == scores + parts + weighted  # (every part is a multiple of 16 here)
    ctx.attention(tout, tq, tk, tv, tkc, tvc, pos)
    torch.cuda.synchronize()
    f = lambda x: oracle.decode(x, "f16").astype(np.float64)  # noqa: E731
    K, V = f(kc), f(vc)
    K[:, pos:pos + seq], V[:, pos:pos + seq] = f(k), f(v)
    assert np.array_equal(to_codes(tkc)[:, pos], k[:, 0]) and np.array_equal(to_codes(tvc)[:, pos], v[:, 0]), "cache contents"
    out = np.zeros((seq, heads, hd))
    for h in range(heads):
        s_ = f(q)[h] @ K[h // (heads // kv_heads)].T / np.sqrt(hd)
        s_ = oracle.decode(oracle.encode(s_.astype(np.float32), "f16"), "f16").astype(np.float64)  # the scores are stored as fp16
        p = np.exp(s_ - s_.max(-1, keepdims=True))
        p /= p.sum(-1, keepdims=True)
        p = oracle.decode(oracle.encode(p.astype(np.float32), "f16"), "f16").astype(np.float64)  # and so are the weights
        out[:, h] = p @ V[h // (heads // kv_heads)]
    got = f(to_codes(tout))
    assert np.all(np.abs(got - out) <= 1e-2 * np.abs(out) + 6 * 2.0 ** -10 * np.abs(V).max())


def test_status_codes_and_workspace(ctx):
    import torch

    from operators_amd import InfiniopError
    from operators_amd.ops import AttentionPlan

    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")  # noqa: E731
    out, q, k, v, kc, vc = z(5, 8, 16), z(8, 5, 16), z(2, 5, 16), z(2, 5, 16), z(2, 32, 16), z(2, 32, 16)
    with AttentionPlan(ctx, out, q, k, v, kc, vc, 3) as plan:
        assert plan.workspace_size == (8 * 5 * 8 + 8 * 5 * 16) * 2  # scores + head-major result; q is used where it lies
        st = ctx.lib.infiniopAttention(plan.desc, plan.workspace.data_ptr(), plan.workspace_size - 1, out.data_ptr(), q.data_ptr(),
                                       k.data_ptr(), v.data_ptr(), kc.data_ptr(), vc.data_ptr(), None)
        assert st == 6
    bad = [
        ((z(5, 8), q, k, v, kc, vc, 0), 4),               # rank
        ((z(5, 8, 32)[:, :, ::2], q, k, v, kc, vc, 0), 5), # out not contiguous
        ((z(5, 4, 16), q, k, v, kc, vc, 0), 2),            # out does not match q
        ((out, q, k, v, z(2, 6, 16), vc, 3), 2),           # cache shorter than pos + seq
        ((out, z(9, 5, 16), k, v, kc, vc, 0), 2),          # (q heads are out's heads, so out mismatches)
    ]
    for args, code in bad:
        with pytest.raises(InfiniopError) as err:
            AttentionPlan(ctx, *args)
        assert err.value.status == code, (err.value.status, code)
