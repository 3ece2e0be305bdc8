"""The note oracle/upstream_bf16.md lists the dtype guards of the reference's
CPU back end that refuse BF16.  This test compiles the reference as it is
(make -C oracle ref: its own sources, where they lie) and checks that each of
those guards still answers STATUS_BAD_TENSOR_DTYPE, at the stage the note
says, while the oracle - the same path with the guards opened - accepts the
same descriptors.  Skipped where there is neither a checkout of the reference
nor a built oracle/_ref."""
import os
import subprocess

import numpy as np
import pytest

import oracle
from oracle import ref

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BAD_DTYPE = 3


@pytest.fixture(scope="module", autouse=True)
def reference_library():
    if not ref.available():
        if not os.path.isdir("/root/reference/src"):
            pytest.skip("no checkout of the reference and no oracle/_ref")
        subprocess.run(["make", "-C", os.path.join(ROOT, "oracle"), "ref"], check=True, capture_output=True)
    assert ref.available()


def T(dt, shape, strides=None):
    return (dt, tuple(shape), strides)


def test_add_refuses_bf16_at_create():
    assert ref.add_status(T("bf16", (4, 8)), T("bf16", (4, 8)), T("bf16", (4, 8))) == BAD_DTYPE
    assert ref.add_status(T("f16", (4, 8)), T("f16", (4, 8)), T("f16", (4, 8))) == 0
    s = oracle.Spec("bf16", (4, 8))
    assert oracle.add_check(s, s, s, allow_bf16=True) == 0 and oracle.add_check(s, s, s, allow_bf16=False) == BAD_DTYPE


def test_swiglu_refuses_bf16_at_create():
    assert ref.swiglu_status(T("bf16", (4, 8)), T("bf16", (4, 8)), T("bf16", (4, 8))) == BAD_DTYPE
    assert ref.swiglu_status(T("f16", (4, 8)), T("f16", (4, 8)), T("f16", (4, 8))) == 0
    s = oracle.Spec("bf16", (4, 8))
    assert oracle.swiglu_check(s, s, s, allow_bf16=True) == 0


def test_rope_refuses_bf16_at_create():
    args = lambda dt: (T(dt, (4, 2, 8)), T("u64", (4,)), T("f32", (16, 8)), T("f32", (16, 8)))  # noqa: E731
    assert ref.rope_status(*args("bf16")) == BAD_DTYPE
    assert ref.rope_status(*args("f16")) == 0
    specs = [oracle.Spec(*t) for t in args("bf16")]
    assert oracle.rope_check(*specs, allow_bf16=True) == 0


def test_rms_norm_accepts_the_descriptor_and_refuses_bf16_at_compute():
    y, x, w = T("bf16", (4, 64)), T("bf16", (4, 64)), T("f32", (64,))
    assert ref.rms_norm_status(y, x, w) == 0
    assert ref.rms_norm_status(y, x, w, run=True) == BAD_DTYPE
    assert ref.rms_norm_status(T("f16", (4, 64)), T("f16", (4, 64)), w, run=True) == 0
    # the oracle, same call, bf16 admitted
    codes = oracle.f32_to_bf16(np.ones((4, 64), np.float32))
    out = oracle.rms_norm(codes, np.ones(64, np.float32), 1e-5, "bf16", "f32")
    assert out.shape == (4, 64)


def test_causal_softmax_and_random_sample_refuse_bf16_at_create():
    assert ref.causal_softmax_status(T("bf16", (4, 8))) == BAD_DTYPE
    assert ref.causal_softmax_status(T("f16", (4, 8))) == 0
    assert ref.random_sample_status(T("u64", (1,)), T("bf16", (512,))) == BAD_DTYPE
    assert ref.random_sample_status(T("u64", (1,)), T("f16", (512,))) == 0


def test_the_note_names_every_guard():
    note = open(os.path.join(ROOT, "oracle", "upstream_bf16.md")).read()
    for path in ("src/devices/cpu/common_cpu", "src/ops/add/cpu/add_cpu.cc", "src/ops/swiglu/cpu/swiglu_cpu.cc",
                 "src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc", "src/ops/rms_norm/cpu/rms_norm_cpu.cc",
                 "src/ops/causal_softmax/cpu/causal_softmax_cpu.cc", "src/ops/random_sample/cpu/random_sample.cc"):
        assert path in note, path
    if os.path.isdir("/root/reference/src"):
        for path in ("src/ops/add/cpu/add_cpu.cc", "src/ops/swiglu/cpu/swiglu_cpu.cc", "src/ops/rotary_embedding/cpu/rotary_embedding_cpu.cc",
                     "src/ops/rms_norm/cpu/rms_norm_cpu.cc"):
            assert os.path.isfile(os.path.join("/root/reference", path)), path
