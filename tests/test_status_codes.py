"""Create-time checks, without a GPU: the status codes recorded from the
compiled reference (tests/golden/status_cases.json) against
  * the oracle's restatement of the checks, and
  * the shipped library's own host-side validation, reached through the public
    C entry points with a hand-made handle (a handle is a plain struct whose
    fields the create functions only read; no GPU call is made before stage 4).
bf16 cases are this project's extension: the reference answers BAD_TENSOR_DTYPE,
the oracle (with the extension switched on) and the library accept them."""
import ctypes

import pytest

import operators_amd as oa
import oracle
from helpers import golden_json
from oracle.ref import LAYOUT

CASES = golden_json()["status"]


def spec(t):
    return oracle.Spec(t[0], t[1], t[2])


@pytest.mark.parametrize("i", range(len(CASES)))
def test_oracle_checks_reproduce_reference_status(i):
    case = CASES[i]
    specs = [spec(t) for t in case["tensors"]]
    if case["op"] == "add":
        st = oracle.add_check(*specs, allow_bf16=False)
    elif case["op"] == "swiglu":
        st = oracle.swiglu_check(*specs, allow_bf16=False)
    elif case["op"] == "rope":
        st = oracle.rope_check(*specs, allow_bf16=False)
    elif case["op"] == "rearrange":
        assert oracle.rearrange_check(*specs) == case["status"], case
        return
    elif case["op"] == "random_sample":
        assert oracle.random_sample_check(*specs) == case["status"], case
        if case.get("bf16_extension"):
            assert oracle.random_sample_check(*specs, allow_bf16=True) == 0
        return
    elif case["op"] == "causal_softmax":
        st = oracle.causal_softmax_check(specs[0], allow_bf16=False, unit_inner=False)
        assert st == case["status"], case
        if case.get("bf16_extension"):
            assert oracle.causal_softmax_check(specs[0], allow_bf16=True, unit_inner=True) == 0
        if case.get("cpu_only_layout"):
            assert oracle.causal_softmax_check(specs[0], allow_bf16=False, unit_inner=True) == 5
        return
    else:
        st = oracle.rms_norm_check(*specs)
        if st == 0 and case.get("run"):  # the reference reports unsupported data types at compute time
            import numpy as np
            n, d = case["tensors"][0][1]
            buf = np.zeros(n * d * 4, np.uint8)
            st = oracle.lib().oracle_rms_norm(oracle.DT[case["tensors"][0][0]], oracle.DT[case["tensors"][2][0]], n, d, d, d,
                                             ctypes.c_float(1e-5), buf.ctypes.data, buf.ctypes.data, buf.ctypes.data)
            if case.get("bf16_extension"):
                assert st == 0
                return
    assert st == case["status"], case
    if case.get("bf16_extension") and case["op"] != "rms_norm":
        again = {"add": oracle.add_check, "swiglu": oracle.swiglu_check, "rope": oracle.rope_check}[case["op"]](*specs, allow_bf16=True)
        assert again == 0


class FakeAmdContext(ctypes.Structure):
    """Layout of the library's handle (operators_amd/csrc/devices/amd/amd_handle.h)."""
    _fields_ = [("device", ctypes.c_int), ("device_id", ctypes.c_int), ("cu_count", ctypes.c_int),
                ("lds_per_block", ctypes.c_int), ("max_grid_x", ctypes.c_int), ("wave_size", ctypes.c_int)]


@pytest.fixture(scope="module")
def fake_handle():
    ctxt = FakeAmdContext(oa.DeviceEnum.DEVICE_AMD, 0, 256, 65536, 2 ** 31 - 1, 64)
    return ctypes.cast(ctypes.pointer(ctxt), oa.infiniopHandle_t), ctxt


CREATE = {
    "add": ("infiniopCreateAddDescriptor", "infiniopDestroyAddDescriptor", oa.infiniopAddDescriptor_t),
    "swiglu": ("infiniopCreateSwiGLUDescriptor", "infiniopDestroySwiGLUDescriptor", oa.infiniopSwiGLUDescriptor_t),
    "rope": ("infiniopCreateRoPEDescriptor", "infiniopDestroyRoPEDescriptor", oa.infiniopRoPEDescriptor_t),
    "rms_norm": ("infiniopCreateRMSNormDescriptor", "infiniopDestroyRMSNormDescriptor", oa.infiniopRMSNormDescriptor_t),
    "rearrange": ("infiniopCreateRearrangeDescriptor", "infiniopDestroyRearrangeDescriptor", oa.infiniopRearrangeDescriptor_t),
    "causal_softmax": ("infiniopCreateCausalSoftmaxDescriptor", "infiniopDestroyCausalSoftmaxDescriptor", oa.infiniopCausalSoftmaxDescriptor_t),
    "random_sample": ("infiniopCreateRandomSampleDescriptor", "infiniopDestroyRandomSampleDescriptor", oa.infiniopRandomSampleDescriptor_t),
}


@pytest.mark.parametrize("i", range(len(CASES)))
def test_library_host_validation_reproduces_reference_status(fake_handle, i):
    case = CASES[i]
    lib = oa.open_lib()
    handle, _keep = fake_handle
    create, destroy, dtype = CREATE[case["op"]]
    descs = [oa.make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
    d = dtype()
    extra = (ctypes.c_float(1e-5),) if case["op"] == "rms_norm" else ()
    st = getattr(lib, create)(handle, ctypes.byref(d), *descs, *extra)
    if case["op"] == "rms_norm" and case.get("run"):
        # the dtype verdict comes at compute time, as in the reference; on a
        # machine without a GPU only the "unsupported type" answer can be
        # observed, because it is given before anything touches the device
        assert st == 0
        if case["status"] == 3 and not case.get("bf16_extension"):
            assert lib.infiniopRMSNorm(d, None, 0, None, None, None, None) == 3
        want = 0
    else:
        want = 0 if case.get("bf16_extension") else case["status"]
        if case.get("cpu_only_layout"):
            want = 5  # non-unit inner stride: accepted by the reference's CPU back end only, refused here as by its GPU back end
    assert st == want, (case, st)
    if st == 0:
        size = ctypes.c_uint64(7)
        if case["op"] == "causal_softmax":
            assert lib.infiniopGetCausalSoftmaxWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0
        if case["op"] == "rms_norm":
            assert lib.infiniopGetRMSNormWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0
        if case["op"] == "rope":
            assert lib.infiniopGetRoPEWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0
        if case["op"] == "random_sample":
            assert lib.infiniopGetRandomSampleWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0  # 512 logits: one workgroup
        assert getattr(lib, destroy)(d) == 0
    for x in descs:
        lib.infiniopDestroyTensorDescriptor(x)


FUSED_CASES = [
    # (y, c, a, b, w) as (dtype, shape, strides) -> create status; the fused Add + RMSNorm has no reference
    # counterpart, so the expectations are RMSNorm's and Add's own rules (shape 4, strides 5, type at compute time)
    ([("f16", (4, 64), None)] * 4 + [("f32", (64,), None)], 0),
    ([("f16", (4, 64), (128, 1))] * 4 + [("f16", (64,), None)], 0),
    ([("f16", (4, 64), None)] * 3 + [("f16", (4, 32), None), ("f32", (64,), None)], 4),
    ([("f16", (4, 64), None)] * 4 + [("f32", (32,), None)], 4),
    ([("f16", (4, 64), None)] * 2 + [("f16", (64,), None), ("f16", (4, 64), None), ("f32", (64,), None)], 4),
    ([("f16", (4, 64), None)] * 3 + [("f16", (4, 64), (128, 2)), ("f32", (64,), None)], 5),
    ([("f16", (4, 64), None)] * 4 + [("f32", (64,), (2,))], 5),
]


@pytest.mark.parametrize("i", range(len(FUSED_CASES)))
def test_fused_add_rms_norm_host_validation(fake_handle, i):
    tensors, want = FUSED_CASES[i]
    lib = oa.open_lib()
    handle, _keep = fake_handle
    descs = [oa.make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in tensors]
    d = oa.infiniopAddRMSNormDescriptor_t()
    st = lib.infiniopCreateAddRMSNormDescriptor(handle, ctypes.byref(d), *descs, ctypes.c_float(1e-5))
    assert st == want, (tensors, st)
    if st == 0:
        size = ctypes.c_uint64(7)
        assert lib.infiniopGetAddRMSNormWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0
        assert lib.infiniopDestroyAddRMSNormDescriptor(d) == 0
    for x in descs:
        lib.infiniopDestroyTensorDescriptor(x)


def test_fused_add_rms_norm_refuses_mixed_types_at_compute_time(fake_handle):
    lib = oa.open_lib()
    handle, _keep = fake_handle
    descs = [oa.make_descriptor(lib, (4, 64), None, oa.F16 if k != 2 else oa.F32) for k in range(4)] + [oa.make_descriptor(lib, (64,), None, oa.F32)]
    d = oa.infiniopAddRMSNormDescriptor_t()
    assert lib.infiniopCreateAddRMSNormDescriptor(handle, ctypes.byref(d), *descs, ctypes.c_float(1e-5)) == 0
    assert lib.infiniopAddRMSNorm(d, None, 0, None, None, None, None, None, None) == 3  # answered before anything touches a device
    assert lib.infiniopDestroyAddRMSNormDescriptor(d) == 0
    for x in descs:
        lib.infiniopDestroyTensorDescriptor(x)


MATMUL_CASES = [
    # (c, a, b) as (dtype, shape, strides) -> create status; the table the reference's own back end is held to
    # in test_oracle_ops.py, plus what this back end answers where the reference ends the process (mismatched extents)
    ((("f16", (4, 6), None), ("f16", (4, 5), None), ("f16", (5, 6), None)), 0),
    ((("f32", (2, 4, 6), None), ("f32", (2, 4, 5), None), ("f32", (5, 6), None)), 0),
    ((("f16", (4, 6), (1, 4)), ("f16", (4, 5), (1, 4)), ("f16", (5, 6), (1, 5))), 0),
    ((("f16", (2, 2, 4, 6), None), ("f16", (4, 5), None), ("f16", (5, 6), None)), 4),
    ((("f16", (4, 6), (12, 2)), ("f16", (4, 5), None), ("f16", (5, 6), None)), 5),
    ((("f16", (3, 4, 6), None), ("f16", (2, 4, 5), None), ("f16", (5, 6), None)), 2),
    ((("u8", (4, 6), None), ("u8", (4, 5), None), ("u8", (5, 6), None)), 3),
    ((("f16", (4, 6), None), ("f16", (4, 5), None), ("f16", (7, 6), None)), 4),
]


@pytest.mark.parametrize("i", range(len(MATMUL_CASES)))
def test_matmul_host_validation(fake_handle, i):
    tensors, want = MATMUL_CASES[i]
    lib = oa.open_lib()
    handle, _keep = fake_handle
    descs = [oa.make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in tensors]
    d = oa.infiniopMatmulDescriptor_t()
    st = lib.infiniopCreateMatmulDescriptor(handle, ctypes.byref(d), descs[0], ctypes.c_float(1.0), descs[1], descs[2], ctypes.c_float(0.0))
    assert st == want, (tensors, st)
    if st == 0:
        size = ctypes.c_uint64(7)
        assert lib.infiniopGetMatmulWorkspaceSize(d, ctypes.byref(size)) == 0 and size.value == 0
        assert lib.infiniopDestroyMatmulDescriptor(d) == 0
    for x in descs:
        lib.infiniopDestroyTensorDescriptor(x)


def test_mlp_host_validation_and_workspace_size(fake_handle):
    lib = oa.open_lib()
    handle, _keep = fake_handle
    mk = lambda shape, strides=None: oa.make_descriptor(lib, shape, strides, oa.F16)  # noqa: E731
    y, x, w12, w3 = mk((8, 64)), mk((8, 64)), mk((64, 256)), mk((128, 64))
    d = oa.infiniopMLPDescriptor_t()
    assert lib.infiniopCreateMLPDescriptor(handle, ctypes.byref(d), y, x, w12, w3, ctypes.c_float(1.0), ctypes.c_char(b"\x00")) == 0
    size = ctypes.c_uint64(0)
    assert lib.infiniopGetMLPWorkspaceSize(d, ctypes.byref(size)) == 0
    assert size.value == 8 * 256 * 2 + 8 * 128 * 2  # the two intermediates; the reference reserves the same (mlp/operator.cc:62-65)
    assert lib.infiniopMLP(d, None, 0, None, None, None, None, None) == 6  # short workspace
    assert lib.infiniopDestroyMLPDescriptor(d) == 0
    bad_x = mk((8, 64), (128, 2))
    assert lib.infiniopCreateMLPDescriptor(handle, ctypes.byref(d), y, bad_x, w12, w3, ctypes.c_float(1.0), ctypes.c_char(b"\x00")) == 5
    w3_bad = mk((100, 64))
    assert lib.infiniopCreateMLPDescriptor(handle, ctypes.byref(d), y, x, w12, w3_bad, ctypes.c_float(1.0), ctypes.c_char(b"\x00")) == 4
    for t in (y, x, w12, w3, bad_x, w3_bad):
        lib.infiniopDestroyTensorDescriptor(t)


def test_descriptor_starts_with_device_number(fake_handle):
    lib = oa.open_lib()
    handle, _keep = fake_handle
    descs = [oa.make_descriptor(lib, (4, 8), None, oa.F16) for _ in range(3)]
    d = oa.infiniopAddDescriptor_t()
    assert lib.infiniopCreateAddDescriptor(handle, ctypes.byref(d), *descs) == 0
    assert d.contents.device == oa.DeviceEnum.DEVICE_AMD
    assert lib.infiniopDestroyAddDescriptor(d) == 0
    # a handle of another device is refused by every create function
    other = FakeAmdContext(oa.DeviceEnum.DEVICE_CPU, 0, 1, 1, 1, 1)
    assert lib.infiniopCreateAddDescriptor(ctypes.cast(ctypes.pointer(other), oa.infiniopHandle_t), ctypes.byref(d), *descs) == 8
    d2 = oa.infiniopSwiGLUDescriptor_t()
    assert lib.infiniopCreateSwiGLUDescriptor(ctypes.cast(ctypes.pointer(other), oa.infiniopHandle_t), ctypes.byref(d2), *descs) == 8
    for x in descs:
        lib.infiniopDestroyTensorDescriptor(x)


def test_causal_softmax_refuses_fewer_columns_than_rows(fake_handle):
    """The reference's column bound wraps around for total < seq and its CPU
    loops then leave the row; this library refuses the shape instead."""
    lib = oa.open_lib()
    handle, _keep = fake_handle
    y = oa.make_descriptor(lib, (8, 4), None, oa.F16)
    d = oa.infiniopCausalSoftmaxDescriptor_t()
    assert lib.infiniopCreateCausalSoftmaxDescriptor(handle, ctypes.byref(d), y) == 4
    lib.infiniopDestroyTensorDescriptor(y)


def test_null_output_pointer_is_memory_not_allocated(fake_handle):
    lib = oa.open_lib()
    handle, _keep = fake_handle
    t = oa.make_descriptor(lib, (4, 2, 8), None, oa.F16)
    p = oa.make_descriptor(lib, (4,), None, oa.U64)
    s = oa.make_descriptor(lib, (16, 8), None, oa.F32)
    assert lib.infiniopCreateRoPEDescriptor(handle, None, t, p, s, s) == 6  # rotary_embedding_cpu.cc:54-55
    for x in (t, p, s):
        lib.infiniopDestroyTensorDescriptor(x)


def test_random_sample_host_rules_beyond_the_reference(fake_handle):
    """A strided or empty logits vector is refused at create time; null
    pointers are refused at stage 4 before anything touches the device, and
    the entry point without workspace refuses vocabularies beyond its limit
    the same way.  topk has no upper limit (the reference has none)."""
    lib = oa.open_lib()
    handle, _keep = fake_handle

    def create(result, probs):
        descs = [oa.make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in (result, probs)]
        d = oa.infiniopRandomSampleDescriptor_t()
        st = lib.infiniopCreateRandomSampleDescriptor(handle, ctypes.byref(d), *descs)
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)
        return st, d

    assert create(("u64", (1,), None), ("f16", (512,), (2,)))[0] == 5
    assert create(("u64", (1,), None), ("f16", (0,), None))[0] == 4
    assert create(("u64", (), None), ("f16", (512,), None))[0] == 0
    st, d = create(("u64", (1,), None), ("f16", (4096,), None))
    assert st == 0
    f = ctypes.c_float
    assert lib.infiniopRandomSample(d, None, 0, None, None, f(0.5), f(0.9), 4, f(1.0), None) == 2
    assert lib.infiniopRandomSampleNoAlloc(d, None, None, f(0.5), f(0.9), 4, f(1.0), None) == 2
    assert lib.infiniopDestroyRandomSampleDescriptor(d) == 0
    st, d = create(("u64", (1,), None), ("f16", ((1 << 20) + 1,), None))
    assert st == 0
    assert lib.infiniopRandomSampleNoAlloc(d, 8, 8, f(0.5), f(0.9), 4, f(1.0), None) == 2  # more logits than its lists serve
    assert lib.infiniopDestroyRandomSampleDescriptor(d) == 0
