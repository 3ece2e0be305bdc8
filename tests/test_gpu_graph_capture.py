"""The five launches of the prefill chain recorded into a HIP graph and
replayed: stage 4 of every operator only enqueues kernels on the caller's
stream (no allocation, no memset, no synchronisation), so a capture holds
exactly those kernels.  Every replay, with eager work and synchronisations in
between, must reproduce the eager results bit for bit."""
import pytest

pytestmark = pytest.mark.gpu


def test_chain_replays_from_a_hip_graph(ctx):
    import torch

    from operators_amd.ops import AddPlan, RMSNormPlan, RoPEPlan, SwiGLUPlan, sin_cos_table

    tokens, bf16 = 512, torch.bfloat16
    gen = torch.Generator(device="cuda")
    gen.manual_seed(11)
    rnd = lambda *s: torch.randn(s, device="cuda", dtype=torch.float32, generator=gen).to(bf16)  # noqa: E731
    x, w = rnd(tokens, 8192), torch.rand(8192, device="cuda", generator=gen) + 0.5
    qkv0 = rnd(tokens, 80, 128)
    gate_up, a, b = rnd(tokens, 2 * 4096), rnd(tokens, 8192), rnd(tokens, 8192)
    pos = torch.arange(tokens, device="cuda", dtype=torch.int64).view(torch.uint64)
    sin_t, cos_t = sin_cos_table(tokens, 128, 5e5, device="cuda")

    y, qkv = torch.empty_like(x), qkv0.clone()
    h, c = torch.empty((tokens, 4096), dtype=bf16, device="cuda"), torch.empty_like(a)
    q, k = qkv[:, :64, :], qkv[:, 64:72, :]
    plans = [RMSNormPlan(ctx, y, x, w, 1e-5), RoPEPlan(ctx, q, pos, sin_t, cos_t), RoPEPlan(ctx, k, pos, sin_t, cos_t),
             SwiGLUPlan(ctx, h, gate_up[:, 4096:], gate_up[:, :4096]), AddPlan(ctx, c, a, b)]

    def chain(stream):
        plans[0](y, x, w, stream)
        plans[1](q, pos, sin_t, cos_t, stream)
        plans[2](k, pos, sin_t, cos_t, stream)
        plans[3](h, gate_up[:, 4096:], gate_up[:, :4096], stream)
        plans[4](c, a, b, stream)

    # eager results (RoPE works in place: start every run from the same qkv)
    chain(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = [t.clone() for t in (y, qkv, h, c)]

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        qkv.copy_(qkv0)
        with torch.cuda.graph(graph, stream=side):
            chain(torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    for replay in range(4):
        for t in (y, h, c):
            t.zero_()  # eager work between replays, and proof that the replay rewrites the outputs
        qkv.copy_(qkv0)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, ref, name in zip((y, qkv, h, c), want, ("rms_norm", "rope", "swiglu", "add")):
            assert torch.equal(got.view(torch.int16), ref.view(torch.int16)), (replay, name)
    for p in plans:
        p.close()


def test_random_sample_replays_from_a_hip_graph(ctx):
    """The two launches of the sampling form, captured once: every replay
    draws from whatever the logits buffer holds at that moment and must give
    the index an eager call gives for the same logits."""
    import torch

    from operators_amd.ops import RandomSamplePlan

    gen = torch.Generator(device="cuda")
    gen.manual_seed(5)
    draws = [(torch.randn(32000, device="cuda", generator=gen) * 3).to(torch.float16) for _ in range(4)]
    logits = draws[0].clone()
    result = torch.full((1,), -1, dtype=torch.int64, device="cuda")
    plan = RandomSamplePlan(ctx, result.view(torch.uint64), logits)
    assert plan.workspace_size > 0
    args = (0.61, 0.9, 40, 0.9)

    want = []
    for d in draws:
        logits.copy_(d)
        plan(result.view(torch.uint64), logits, *args, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want.append(int(result.item()))
    assert len(set(want)) > 1  # the draws differ, so a replay that ignored the buffer would show

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            plan(result.view(torch.uint64), logits, *args, torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()

    for replay, d in enumerate(draws):
        logits.copy_(d)
        result.fill_(-1)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert int(result.item()) == want[replay], replay
    plan.close()


def test_split_causal_softmax_replays_from_a_hip_graph(ctx):
    """The two launches that share very few very long rows among workgroups (their partial maxima and sums meet in
    the workspace), captured once: every replay works on whatever the scores buffer holds and must give the bits of
    an eager call on the same scores."""
    import torch

    from operators_amd.ops import CausalSoftmaxPlan

    gen = torch.Generator(device="cuda")
    gen.manual_seed(6)
    draws = [(torch.randn((8, 1, 131072), device="cuda", generator=gen) * 3).to(torch.float16) for _ in range(3)]
    scores = draws[0].clone()
    plan = CausalSoftmaxPlan(ctx, scores)
    assert plan.workspace_size > 0
    want = []
    for d in draws:
        scores.copy_(d)
        plan(scores)
        torch.cuda.synchronize()
        want.append(scores.clone())

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        scores.copy_(draws[0])
        with torch.cuda.graph(graph, stream=side):
            plan(scores, torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for replay in range(6):
        i = replay % len(draws)
        plan.workspace.random_(0, 256)  # eager work between replays: the parts of the replay before are gone
        scores.copy_(draws[i])
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(scores.view(torch.int16), want[i].view(torch.int16)), replay
    plan.close()


def test_decoding_mlp_replays_from_a_hip_graph(ctx):
    """One token through the MLP composite: both products are this library's own kernels (partial sums through the
    composite's workspace), so the capture holds five kernels of this library and nothing else."""
    import torch

    from operators_amd.ops import MLPPlan

    gen = torch.Generator(device="cuda")
    gen.manual_seed(8)
    d, di, bf16 = 2048, 4096, torch.bfloat16
    rnd = lambda *s, scale=1.0: (torch.randn(s, device="cuda", dtype=torch.float32, generator=gen) * scale).to(bf16)  # noqa: E731
    xs = [rnd(1, d) for _ in range(3)]
    w12, w3 = rnd(d, 2 * di, scale=d ** -0.5), rnd(di, d, scale=di ** -0.5)
    x, y = xs[0].clone(), torch.zeros((1, d), dtype=bf16, device="cuda")
    plan = MLPPlan(ctx, y, x, w12, w3, 1.0, False)
    want = []
    for v in xs:
        x.copy_(v)
        plan(y, x, w12, w3)
        torch.cuda.synchronize()
        want.append(y.clone())

    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            plan(y, x, w12, w3, torch.cuda.current_stream().cuda_stream)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    for replay in range(6):
        i = replay % len(xs)
        y.zero_()
        plan.workspace.random_(0, 256)
        x.copy_(xs[i])
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), want[i].view(torch.int16)), replay
    plan.close()
