"""A caller written in C, linked against libinfiniop.so and the HIP runtime,
run as a process of its own: tests/c_client/client (built beside the library
by `python -m operators_amd.build`).  It follows the calling sequence the
reference documents for C callers (reference README.md:10-40) - handle,
descriptors, workspace sizes, one call of RMSNorm, RoPE, SwiGLU and Add on a
stream of its own, destroy - on device buffers it allocates itself; this test
writes its input file, runs it, and compares the bytes it wrote with the CPU
oracle on the same input: RoPE and Add bit for bit, RMSNorm and SwiGLU within
one unit in the last place."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from helpers import assert_codes_close, assert_codes_equal
from operators_amd.ops import sin_cos_table

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CLIENT = os.path.join(ROOT, "tests", "c_client", "client")


def fnv1a(data):
    h = 14695981039346656037
    # the same sum the client prints, over the same bytes (vectorised: xor-multiply is sequential, so fold in Python ints per chunk)
    for byte in data:
        h = ((h ^ byte) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return h


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_c_client_runs_the_four_operators(tmp_path, dtype):
    assert os.path.isfile(CLIENT), "build the C client first: python -m operators_amd.build"
    tokens, hidden, heads, buf_heads, head_dim, ffn, rows = 24, 512, 3, 5, 64, 384, 40
    rng = np.random.default_rng(5 if dtype == "f16" else 6)
    x = oracle.encode(rng.standard_normal((tokens, hidden)).astype(np.float32), dtype)
    w = rng.uniform(0.5, 1.5, hidden).astype(np.float32)
    qkv = oracle.encode(rng.standard_normal((tokens, buf_heads, head_dim)).astype(np.float32), dtype)
    pos = rng.integers(0, rows, tokens).astype(np.uint64)
    sin_t, cos_t = (t.numpy() for t in sin_cos_table(rows, head_dim, 1e4))
    gate_up = oracle.encode(rng.standard_normal((tokens, 2 * ffn)).astype(np.float32), dtype)

    src, dst = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(src, "wb") as f:
        f.write(np.array([0 if dtype == "f16" else 1, tokens, hidden, heads, buf_heads, head_dim, ffn, rows], np.uint64).tobytes())
        for arr in (x, w, qkv, pos, sin_t.astype(np.float32), cos_t.astype(np.float32), gate_up):
            f.write(np.ascontiguousarray(arr).tobytes())

    res = subprocess.run([CLIENT, str(src), str(dst)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 0, (res.returncode, res.stdout, res.stderr)
    raw = dst.read_bytes()
    assert res.stdout.split() == ["checksum", f"{fnv1a(raw):016x}"]

    out = np.frombuffer(raw, np.uint16)
    n_x, n_qkv, n_act = tokens * hidden, tokens * buf_heads * head_dim, tokens * ffn
    assert out.size == 2 * n_x + n_qkv + n_act
    y = out[:n_x].reshape(tokens, hidden)
    qkv_out = out[n_x:n_x + n_qkv].reshape(tokens, buf_heads, head_dim)
    act = out[n_x + n_qkv:n_x + n_qkv + n_act].reshape(tokens, ffn)
    resid = out[n_x + n_qkv + n_act:].reshape(tokens, hidden)

    assert_codes_close(y, oracle.rms_norm(x, w, 1e-5, dtype, "f32"), dtype, max_ulp=1, max_frac=5e-3, what="RMSNorm from C")
    want_qkv = qkv.copy()
    oracle.rope(want_qkv[:, :heads, :], pos, sin_t, cos_t, dtype)
    assert_codes_equal(qkv_out, want_qkv, dtype, what="RoPE from C (heads behind the rotated ones untouched)")
    assert_codes_close(act, oracle.swiglu(gate_up[:, ffn:], gate_up[:, :ffn], dtype), dtype, max_ulp=1, max_frac=5e-3, what="SwiGLU from C")
    assert_codes_equal(resid, oracle.add(x, np.ascontiguousarray(y), (tokens, hidden), dtype), dtype, what="Add from C")


def test_c_client_reports_a_bad_call(tmp_path):
    """A head width the operator does not take (odd) comes back as a status, not as a crash."""
    src, dst = tmp_path / "in.bin", tmp_path / "out.bin"
    tokens, hidden, heads, buf_heads, head_dim, ffn, rows = 4, 64, 1, 1, 7, 16, 8
    with open(src, "wb") as f:
        f.write(np.array([0, tokens, hidden, heads, buf_heads, head_dim, ffn, rows], np.uint64).tobytes())
        f.write(bytes(tokens * hidden * 2 + hidden * 4 + tokens * buf_heads * head_dim * 2 + tokens * 8 + 2 * rows * head_dim * 4 + tokens * 2 * ffn * 2))
    res = subprocess.run([CLIENT, str(src), str(dst)], capture_output=True, text=True, timeout=120)
    assert res.returncode == 10 + 4, (res.returncode, res.stderr)  # 10 + STATUS_BAD_TENSOR_SHAPE
    assert "infiniopCreateRoPEDescriptor" in res.stderr
