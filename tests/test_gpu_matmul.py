"""Matmul and the MLP composite on the GPU through the C ABI.

The product is a library GEMM with fp32 accumulation and round-to-nearest
output; the reference's CPU path accumulates in fp32 in index order and
truncates.  Bar: the reference's own test tolerance, rtol 1e-2
(operatorspy/tests/matmul.py:127), applied as
    |gpu - ref| <= 1e-2 * |ref| + slack,
where slack is what the two summation orders may differ by,
4 * k * 2^-24 * sum|a||b|; and, tighter, both results within rounding of the
float64 product."""
import numpy as np
import pytest

import oracle
from helpers import strided_like, to_codes, to_torch

pytestmark = pytest.mark.gpu
ULP = {"f16": 2.0 ** -10, "bf16": 2.0 ** -7, "f32": 2.0 ** -23}


def as_f64(x, dt):
    return (x if dt == "f32" else oracle.decode(x, dt)).astype(np.float64)


def make(shape, dt, rng, positive):
    v = rng.random(shape, dtype=np.float32) if positive else rng.standard_normal(shape).astype(np.float32)
    return v if dt == "f32" else oracle.encode(v, dt)


def device(x, dt, strides=None):
    if strides is None:
        return to_torch(x, dt)
    return strided_like(x, x.shape, strides, dt)[0]


def check(got, ref, exact, mag, k, dt, what):
    g, r = as_f64(got, dt), as_f64(ref, dt)
    order_slack = 4 * k * 2.0 ** -24 * mag
    assert np.all(np.abs(g - r) <= 1e-2 * np.abs(r) + order_slack + 1e-30), what
    # each within rounding (gpu: nearest, half an ulp; reference: truncation, one ulp) of the float64 product
    assert np.all(np.abs(g - exact) <= 0.5 * ULP[dt] * np.abs(exact) + order_slack + 1e-30), what + " (gpu vs float64)"
    assert np.all(np.abs(r - exact) <= 1.0 * ULP[dt] * np.abs(exact) + order_slack + 1e-30), what + " (oracle vs float64)"


REFERENCE_CASES = [
    # alpha, beta, a_shape, b_shape, c_shape, a_stride, b_stride, c_stride   (operatorspy/tests/matmul.py:297-306)
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), None, None, None),
    (1.0, 0.0, (2, 4, 2048), (2, 2048, 2048), (2, 4, 2048), None, None, None),
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), (4096, 1), (4096, 1), (4096, 1)),
    (1.0, 1.0, (6, 2048), (2048, 2560), (6, 2560), (2048, 1), (1, 2048), (2560, 1)),
    (1.0 / 8.0, 0.0, (4, 8 * 6, 64), (4, 64, 6), (4, 8 * 6, 6), None, None, None),
]
MORE_CASES = [
    (0.5, -1.5, (33, 100), (100, 17), (33, 17), (1, 33), (1, 100), (1, 33)),          # everything column-major
    (1.0, 0.0, (40, 72), (72, 56), (40, 56), (1, 40), (56, 1), (56, 1)),               # a column-major, b and c row-major
    (2.0, 1.0, (3, 16, 32), (32, 24), (3, 16, 24), None, None, None),                  # one b for every batch
    (1.0, 0.0, (5, 8, 64), (5, 64, 8), (5, 8, 8), (1024, 64, 1), (1024, 1, 64), None), # padded batch strides
    (1.0, 0.0, (128, 256), (256, 512), (128, 512), None, None, None),
]


@pytest.mark.parametrize("dt", ["f16", "f32", "bf16"])
@pytest.mark.parametrize("case", range(len(REFERENCE_CASES) + len(MORE_CASES)))
def test_against_oracle(ctx, dt, case):
    import torch

    alpha, beta, a_shape, b_shape, c_shape, a_st, b_st, c_st = (REFERENCE_CASES + MORE_CASES)[case]
    rng = np.random.default_rng(1000 + case)
    positive = case < len(REFERENCE_CASES)  # the reference's test draws from [0, 1)
    a, b = make(a_shape, dt, rng, positive), make(b_shape, dt, rng, positive)
    c0 = make(c_shape, dt, rng, positive)
    ta, tb, tc = device(a, dt, a_st), device(b, dt, b_st), device(c0, dt, c_st)
    ctx.matmul(tc, ta, tb, alpha, beta)
    torch.cuda.synchronize()
    got = tc.cpu().numpy() if dt == "f32" else to_codes(tc)
    ref = oracle.matmul(c0.copy(), a, b, alpha, beta, dt)
    fa, fb, fc = as_f64(a, dt), as_f64(b, dt), as_f64(c0, dt)
    exact = alpha * np.matmul(fa, fb) + beta * fc
    mag = abs(alpha) * np.matmul(np.abs(fa), np.abs(fb)) + abs(beta) * np.abs(fc)
    check(got, ref, exact, mag, a_shape[-1], dt, f"case {case} {dt}")


# The two products of an attention while decoding, which this library serves with kernels of its own instead of the
# BLAS library's: scores = q @ K^T (few queries against many keys: matmul_skinny) and out = weights @ V (a sum over many
# keys: matmul_long_k, through the workspace Matmul then asks for).
# batch, queries, head_dim, keys, cache rows (the caches are [batch, rows, head_dim]: K^T and V are views of them)
DECODE_CASES = [(8, 8, 128, 4096, 4096), (2, 8, 128, 33000, 33008), (3, 5, 64, 1031, 2048), (2, 16, 256, 2049, 2056), (1, 1, 32, 1024, 1024),
                (2, 3, 96, 3001, 3008), (2, 8, 512, 1500, 1504), (2, 7, 16, 50001, 50008), (1, 8, 8, 1500, 1504), (4, 4, 128, 131072, 131072)]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(DECODE_CASES)))
@pytest.mark.parametrize("alpha,beta", [(0.125, 0.0), (0.5, 0.25)])
def test_the_products_of_a_decoding_attention(ctx, dt, case, alpha, beta):
    import torch

    from operators_amd.ops import MatmulPlan

    batch, nq, hd, keys, rows = DECODE_CASES[case]
    rng = np.random.default_rng(3000 + case)
    q = make((batch, nq, hd), dt, rng, False)
    cache = make((batch, rows, hd), dt, rng, False)
    weights = make((batch, nq, keys), dt, rng, True)
    tq, tcache, tw = to_torch(q, dt), to_torch(cache, dt), to_torch(weights, dt)
    fq, fc, fw = as_f64(q, dt), as_f64(cache, dt)[:, :keys], as_f64(weights, dt)

    # scores [batch, queries, keys] = alpha * q @ K^T + beta * scores, K^T a view of the cache
    s0 = make((batch, nq, keys), dt, rng, False)
    ts = to_torch(s0, dt)
    k_t = tcache[:, :keys, :].transpose(1, 2)
    ctx.matmul(ts, tq, k_t, alpha, beta)
    torch.cuda.synchronize()
    exact = alpha * np.matmul(fq, fc.transpose(0, 2, 1)) + beta * as_f64(s0, dt)
    mag = abs(alpha) * np.matmul(np.abs(fq), np.abs(fc).transpose(0, 2, 1)) + abs(beta) * np.abs(as_f64(s0, dt))
    g = as_f64(to_codes(ts), dt)
    assert np.all(np.abs(g - exact) <= 0.5 * ULP[dt] * np.abs(exact) + 4 * hd * 2.0 ** -24 * mag + 1e-30), f"scores case {case} {dt}"

    # out [batch, queries, head_dim] = alpha * weights @ V + beta * out, with the workspace and without (the BLAS library then)
    o0 = make((batch, nq, hd), dt, rng, False)
    v = tcache[:, :keys, :]
    exact = alpha * np.matmul(fw, fc) + beta * as_f64(o0, dt)
    mag = abs(alpha) * np.matmul(np.abs(fw), np.abs(fc)) + abs(beta) * np.abs(as_f64(o0, dt))
    for use_workspace in (True, False):
        to = to_torch(o0, dt)
        with MatmulPlan(ctx, to, tw, v, alpha, beta) as plan:
            fits = hd in (8, 16, 32, 64, 128, 256) and nq <= 8 and keys >= 1024
            assert (plan.workspace_size > 0) == fits, (case, plan.workspace_size)
            plan(to, tw, v, None, use_workspace)
        torch.cuda.synchronize()
        g = as_f64(to_codes(to), dt)
        assert np.all(np.abs(g - exact) <= 0.5 * ULP[dt] * np.abs(exact) + 4 * keys * 2.0 ** -24 * mag + 1e-30), f"weighted values case {case} {dt} workspace {use_workspace}"


# tokens, input width, output width, row pitch of the weight matrix (a few tokens through a layer's weights while decoding:
# the sum over the input width is split over workgroups, matmul_long_k_wide, through the workspace Matmul asks for)
WEIGHT_CASES = [(1, 1024, 1024, 1024), (8, 4096, 2048, 2048), (3, 1031, 1544, 1544), (5, 2050, 8200, 8208), (8, 8192, 10240, 10240),
                (2, 28672, 8192, 8192), (7, 1500, 1024, 4096), (9, 2048, 2048, 2048), (4, 2048, 1028, 1032)]


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("case", range(len(WEIGHT_CASES)))
@pytest.mark.parametrize("alpha,beta", [(1.0, 0.0), (0.5, 0.25)])
def test_few_tokens_through_a_weight_matrix(ctx, dt, case, alpha, beta):
    import torch

    from operators_amd.ops import MatmulPlan

    tokens, d, n, pitch = WEIGHT_CASES[case]
    rng = np.random.default_rng(4000 + case)
    x = make((tokens, d), dt, rng, False)
    w = (rng.standard_normal((d, n)).astype(np.float32) * 0.05)
    w = oracle.encode(w, dt)
    y0 = make((tokens, n), dt, rng, False)
    tx = to_torch(x, dt)
    tw = device(w, dt, (pitch, 1)) if pitch != n else to_torch(w, dt)
    exact = alpha * np.matmul(as_f64(x, dt), as_f64(w, dt)) + beta * as_f64(y0, dt)
    mag = abs(alpha) * np.matmul(np.abs(as_f64(x, dt)), np.abs(as_f64(w, dt))) + abs(beta) * np.abs(as_f64(y0, dt))
    for use_workspace in (True, False):
        ty = to_torch(y0, dt)
        with MatmulPlan(ctx, ty, tx, tw, alpha, beta) as plan:
            fits = tokens <= 8 and n % 8 == 0 and n >= 1024 and d >= 1024 and pitch % 8 == 0
            assert (plan.workspace_size > 0) == fits, (case, plan.workspace_size)
            plan(ty, tx, tw, None, use_workspace)
        torch.cuda.synchronize()
        g = as_f64(to_codes(ty), dt)
        assert np.all(np.abs(g - exact) <= 0.5 * ULP[dt] * np.abs(exact) + 4 * d * 2.0 ** -24 * mag + 1e-30), f"case {case} {dt} workspace {use_workspace}"


@pytest.mark.parametrize("seed", range(48))
def test_random_decoding_products(ctx, seed):
    """Random shapes, strides, scales and types around the three products this library serves itself (and just outside
    them, where the BLAS library takes the call): each output within rounding of the float64 product."""
    import torch

    from operators_amd.ops import MatmulPlan

    rng = np.random.default_rng(7000 + seed)
    gen = torch.Generator(device="cuda")
    gen.manual_seed(7000 + seed)
    dt = torch.bfloat16 if rng.random() < 0.5 else torch.float16
    ulp = 2.0 ** -7 if dt == torch.bfloat16 else 2.0 ** -10
    randn = lambda *shape, scale=1.0: (torch.randn(shape, device="cuda", generator=gen) * scale).to(dt)  # noqa: E731
    kind = seed % 3
    batch = int(rng.choice([1, 1, 2, 3, 8]))
    nq = int(rng.integers(1, 18))
    alpha, beta = (1.0, 0.0) if rng.random() < 0.5 else (float(rng.choice([0.5, -1.25, 0.125])), float(rng.choice([0.0, 1.0, 0.25])))
    if kind == 0:  # scores = q K^T
        hd = int(rng.choice([32, 64, 96, 128, 160, 256, 384, 512, 48, 1024]))
        keys = int(rng.integers(900, 40000))
        rows = (keys + int(rng.integers(0, 9)) + 7) // 8 * 8
        cache = randn(batch, rows, hd)
        a, b, c, kk = randn(batch, nq, hd), cache[:, :keys, :].transpose(1, 2), randn(batch, nq, keys), hd
    elif kind == 1:  # out = weights V
        hd = int(rng.choice([8, 16, 32, 64, 128, 256, 96, 512]))
        keys = int(rng.integers(900, 60000))
        cache = randn(batch, keys + 3, hd)
        a, b, c, kk = torch.rand((batch, nq, keys), device="cuda", generator=gen).to(dt), cache[:, :keys, :], randn(batch, nq, hd), keys
    else:  # tokens through weights
        d = int(rng.integers(900, 9000))
        n = int(rng.choice([1024, 1536, 2048, 4096, 8200, 1000, 1028, 22016]))
        wbuf = randn(d, n + int(rng.choice([0, 0, 8, 24, 4])), scale=0.05)
        a, b, c, kk = randn(nq, d), wbuf[:, :n], randn(nq, n), d
    c0 = c.clone()
    with MatmulPlan(ctx, c, a, b, alpha, beta) as plan:
        plan(c, a, b)
    torch.cuda.synchronize()
    want = alpha * torch.matmul(a.double(), b.double()) + beta * c0.double()
    mag = abs(alpha) * torch.matmul(a.double().abs(), b.double().abs()) + abs(beta) * c0.double().abs()
    outside = (c.double() - want).abs() > want.abs() * ulp * 0.5 + 4 * kk * 2.0 ** -24 * mag + 1e-30
    assert not bool(outside.any()), f"seed {seed}: kind {kind} {dt} a {tuple(a.shape)} b {tuple(b.shape)} alpha {alpha} beta {beta}: {int(outside.sum())} outside rounding"


def test_decoding_products_with_special_values(ctx):
    """An infinity or a NaN in one key's values, or in one weight, reaches exactly the outputs it reaches in the float64
    product - also where the key count is odd and the last pair of keys is half empty."""
    import torch

    rng = np.random.default_rng(9)
    batch, nq, hd, keys = 2, 5, 128, 2047
    cache = rng.standard_normal((batch, keys, hd)).astype(np.float32)
    weights = rng.random((batch, nq, keys), dtype=np.float32)
    cache[0, 2046, 3] = np.inf   # the last key (odd count: alone in its pair)
    cache[1, 100, 7] = np.nan
    weights[1, 2, 5] = np.inf
    tc, tw = to_torch(oracle.encode(cache, "f16"), "f16"), to_torch(oracle.encode(weights, "f16"), "f16")
    to = torch.zeros((batch, nq, hd), dtype=torch.float16, device="cuda")
    ctx.matmul(to, tw, tc)
    torch.cuda.synchronize()
    with np.errstate(invalid="ignore", over="ignore"):
        exact = np.matmul(as_f64(oracle.encode(weights, "f16"), "f16"), as_f64(oracle.encode(cache, "f16"), "f16"))
    got = as_f64(to_codes(to), "f16")
    assert np.array_equal(np.isnan(got), np.isnan(exact)) and np.array_equal(np.isinf(got), np.isinf(exact))


def test_identity_and_permutation_are_exact(ctx):
    """a @ I = a and a @ P = a with its columns permuted: no rounding anywhere."""
    import torch

    rng = np.random.default_rng(7)
    a = oracle.encode(rng.standard_normal((48, 64)).astype(np.float32), "f16")
    perm = rng.permutation(64)
    p = np.zeros((64, 64), np.float32)
    p[perm, np.arange(64)] = 1
    for mat, want in ((np.eye(64, dtype=np.float32), a), (p, a[:, perm])):
        tc = torch.zeros((48, 64), dtype=torch.float16, device="cuda")
        ctx.matmul(tc, to_torch(a, "f16"), to_torch(oracle.encode(mat, "f16"), "f16"))
        torch.cuda.synchronize()
        assert np.array_equal(to_codes(tc), want)


def test_status_codes(ctx):
    import torch

    from operators_amd import InfiniopError
    from operators_amd.ops import MatmulPlan

    z = lambda *s, dtype=torch.float16: torch.zeros(s, dtype=dtype, device="cuda")  # noqa: E731
    MatmulPlan(ctx, z(4, 6), z(4, 5), z(5, 6)).close()
    bad = [
        ((z(4, 6), z(4, 5), z(7, 6)), 4),                      # inner extents differ (the reference ends the process here)
        ((z(2, 2, 4, 6), z(4, 5), z(5, 6)), 4),                # rank 4
        ((z(4, 12)[:, ::2], z(8, 5)[::2], z(5, 6)), 5),        # c with neither stride 1
        ((z(3, 4, 6), z(2, 4, 5), z(5, 6)), 2),                # batch of a is neither c's nor 1
        ((z(4, 6, dtype=torch.int32), z(4, 5, dtype=torch.int32), z(5, 6, dtype=torch.int32)), 3),
    ]
    for tensors, code in bad:
        with pytest.raises(InfiniopError) as err:
            MatmulPlan(ctx, *tensors)
        assert err.value.status == code, (err.value.status, code)


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("residual", [False, True])
def test_mlp_against_oracle(ctx, dt, residual):
    """tokens 64, d 256, di 384: the reference's composite, stage by stage."""
    import torch

    rng = np.random.default_rng(31)
    n, d, di = 64, 256, 384
    x = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    w12 = oracle.encode(rng.standard_normal((d, 2 * di)).astype(np.float32) * d ** -0.5, dt)
    w3 = oracle.encode(rng.standard_normal((di, d)).astype(np.float32) * di ** -0.5, dt)
    y0 = oracle.encode(rng.standard_normal((n, d)).astype(np.float32), dt)
    want = oracle.mlp(y0.copy(), x, w12, w3, 0.5, residual, dt)
    ty = to_torch(y0, dt)
    ctx.mlp(ty, to_torch(x, dt), to_torch(w12, dt), to_torch(w3, dt), 0.5, residual)
    torch.cuda.synchronize()
    g, r = as_f64(to_codes(ty), dt), as_f64(want, dt)
    # rounding of the two intermediates differs (nearest vs truncation): a few ulps of the values that enter the second product
    tol = 1e-2 * np.abs(r) + 8 * ULP[dt] * np.sqrt(di) * 0.5
    assert np.all(np.abs(g - r) <= tol), float(np.max(np.abs(g - r) - tol))


def test_mlp_workspace_contract(ctx):
    import torch

    from operators_amd.ops import MLPPlan

    f16 = torch.float16
    y, x = torch.zeros((8, 64), dtype=f16, device="cuda"), torch.zeros((8, 64), dtype=f16, device="cuda")
    w12, w3 = torch.zeros((64, 256), dtype=f16, device="cuda"), torch.zeros((128, 64), dtype=f16, device="cuda")
    with MLPPlan(ctx, y, x, w12, w3) as plan:
        assert plan.workspace_size == 8 * 256 * 2 + 8 * 128 * 2
        st = ctx.lib.infiniopMLP(plan.desc, plan.workspace.data_ptr(), plan.workspace_size - 1, y.data_ptr(), x.data_ptr(),
                                 w12.data_ptr(), w3.data_ptr(), None)
        assert st == 6  # a short workspace: STATUS_MEMORY_NOT_ALLOCATED, as in the reference
