"""One handle and one set of descriptors used from several host threads at
once, each thread on a stream of its own with buffers of its own.

The library keeps no state between calls: descriptors are written once at
create time and only read afterwards, stage 4 binds the device and enqueues on
the stream it is handed (reference contract: handles may be shared between
threads, src/devices/cuda/cuda_handle.h keeps its pools lock-free for that
reason).  The one piece of shared state is Matmul's pool of BLAS handles, which
is taken from under a lock.  Every thread must get, bit for bit, what a single
thread gets."""
import threading

import pytest

pytestmark = pytest.mark.gpu

THREADS = 4
ROUNDS = 12


def test_shared_descriptors_on_four_threads_and_streams(ctx):
    import torch

    from operators_amd.ops import (AddPlan, AddRMSNormPlan, CausalSoftmaxPlan, MatmulPlan, RearrangePlan, RMSNormPlan, RoPEPlan,
                                   SwiGLUPlan, sin_cos_table)

    tokens, f16 = 384, torch.float16
    sin_t, cos_t = sin_cos_table(tokens, 128, 1e4, device="cuda")
    pos = torch.arange(tokens, device="cuda", dtype=torch.int64).view(torch.uint64)

    def make(seed):
        gen = torch.Generator(device="cuda")
        gen.manual_seed(seed)
        rnd = lambda *s: torch.randn(s, device="cuda", dtype=torch.float32, generator=gen).to(f16)  # noqa: E731
        t = {"x": rnd(tokens, 4096), "w": torch.rand(4096, device="cuda", generator=gen) + 0.5, "qkv0": rnd(tokens, 48, 128),
             "gate_up": rnd(tokens, 2 * 2816), "a": rnd(tokens, 4096), "b": rnd(tokens, 4096), "scores0": rnd(8, tokens, tokens),
             "m_a": rnd(tokens, 512), "m_b": rnd(512, 768)}
        t.update(y=torch.empty_like(t["x"]), qkv=t["qkv0"].clone(), h=torch.empty((tokens, 2816), dtype=f16, device="cuda"),
                 c=torch.empty_like(t["a"]), fy=torch.empty_like(t["a"]), fc=torch.empty_like(t["a"]), scores=t["scores0"].clone(),
                 heads=torch.empty((32, tokens, 128), dtype=f16, device="cuda"), m_c=torch.empty((tokens, 768), dtype=f16, device="cuda"))
        return t

    sets = [make(100 + i) for i in range(THREADS)]
    t0 = sets[0]
    # descriptors are made once, from the first set's tensors (all sets have the same shapes and strides), and shared
    plans = {
        "rms": RMSNormPlan(ctx, t0["y"], t0["x"], t0["w"], 1e-5),
        "rope": RoPEPlan(ctx, t0["qkv"][:, :32, :], pos, sin_t, cos_t),
        "swiglu": SwiGLUPlan(ctx, t0["h"], t0["gate_up"][:, 2816:], t0["gate_up"][:, :2816]),
        "add": AddPlan(ctx, t0["c"], t0["a"], t0["b"]),
        "fused": AddRMSNormPlan(ctx, t0["fy"], t0["fc"], t0["a"], t0["b"], t0["w"], 1e-5),
        "softmax": CausalSoftmaxPlan(ctx, t0["scores"]),
        "rearrange": RearrangePlan(ctx, t0["heads"].permute(1, 0, 2), t0["qkv"][:, :32, :]),
        "matmul": MatmulPlan(ctx, t0["m_c"], t0["m_a"], t0["m_b"]),
    }

    def chain(t, stream):
        plans["rms"](t["y"], t["x"], t["w"], stream)
        plans["rope"](t["qkv"][:, :32, :], pos, sin_t, cos_t, stream)
        plans["swiglu"](t["h"], t["gate_up"][:, 2816:], t["gate_up"][:, :2816], stream)
        plans["add"](t["c"], t["a"], t["b"], stream)
        plans["fused"](t["fy"], t["fc"], t["a"], t["b"], t["w"], stream)
        plans["softmax"](t["scores"], stream)
        plans["rearrange"](t["heads"].permute(1, 0, 2), t["qkv"][:, :32, :], stream)
        plans["matmul"](t["m_c"], t["m_a"], t["m_b"], stream)

    outputs = ("y", "qkv", "h", "c", "fy", "fc", "scores", "heads", "m_c")
    # what one thread gets
    want = []
    for t in sets:
        chain(t, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        want.append({k: t[k].clone() for k in outputs})

    failures = []
    barrier = threading.Barrier(THREADS)

    def worker(i):
        try:
            t, stream = sets[i], torch.cuda.Stream()
            with torch.cuda.stream(stream):
                for r in range(ROUNDS):
                    for k in ("y", "h", "c", "fy", "fc", "heads", "m_c"):
                        t[k].zero_()
                    t["qkv"].copy_(t["qkv0"])  # RoPE and the softmax work in place
                    t["scores"].copy_(t["scores0"])
                    if r == 0:
                        barrier.wait()  # all threads launch at the same time
                    chain(t, stream.cuda_stream)
                    stream.synchronize()
                    for k in outputs:
                        if not torch.equal(t[k].view(torch.int16), want[i][k].view(torch.int16)):
                            failures.append((i, r, k))
        except Exception as e:  # a thread's exception must fail the test, not vanish
            failures.append((i, "exception", repr(e)))
            try:
                barrier.abort()
            except Exception:
                pass

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(THREADS)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    torch.cuda.synchronize()
    for p in plans.values():
        p.close()
    assert not failures, failures[:8]
