"""The C-ABI library loads and exports exactly what include/infiniop.h
declares; argument checks that need no GPU behave as documented."""
import ctypes
import os
import re

import pytest

import operators_amd as oa
from operators_amd.liboperators import EXPORTED_SYMBOLS, TensorDescriptor, library_path

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_in_header():
    text = open(os.path.join(ROOT, "include", "infiniop.h")).read()
    return sorted(set(re.findall(r"INFINIOP_EXPORT\s+infiniopStatus_t\s+(infiniop\w+)\s*\(", text)))


def test_header_declares_every_entry_point():
    names = declared_in_header()
    assert len(names) == 46  # handle 2 + tensor 2 + add 3 + rms_norm 4 + rope 4 + swiglu 3 + causal_softmax 4 + rearrange 3 + add_rms_norm 4 + matmul 4 + mlp 4 + attention 4 + random_sample 4 + its allocation-free form 1
    assert sorted(EXPORTED_SYMBOLS) == names


def test_library_exports_every_declared_symbol():
    assert os.path.isfile(library_path()), "build the library first: python -m operators_amd.build"
    lib = oa.open_lib()
    for name in declared_in_header():
        assert hasattr(lib, name), name


def test_every_declaration_cites_the_reference():
    text = open(os.path.join(ROOT, "include", "infiniop.h")).read()
    for name in declared_in_header():
        before = text[:re.search(r"infiniopStatus_t\s+" + name + r"\s*\(", text).start()]
        comment = before[before.rindex("/*"):]
        if "AddRMSNorm" in name:  # the fused operator: the reference has none, and the header must say so
            assert "no counterpart in the reference" in comment and "include/ops/" in comment, name
        elif "NoAlloc" in name:  # no counterpart either; the header names the callers it is for
            assert "no counterpart in the reference" in comment and "cannot allocate" in comment, name
        else:
            assert "replaces include/" in comment, name


def test_data_layout_is_four_bytes_and_matches_c_bitfield():
    assert ctypes.sizeof(oa.DataLayout) == 4
    raw = lambda d: int.from_bytes(bytes(d), "little")  # noqa: E731
    # packed | sign<<8 | size<<9 | mantissa<<16 | exponent<<24
    assert raw(oa.F16) == 1 | (1 << 8) | (2 << 9) | (10 << 16) | (5 << 24)
    assert raw(oa.BF16) == 1 | (1 << 8) | (2 << 9) | (7 << 16) | (8 << 24)
    assert raw(oa.U64) == 1 | (0 << 8) | (8 << 9) | (64 << 16)
    assert ctypes.sizeof(TensorDescriptor) == 32


def test_tensor_descriptor_round_trip():
    lib = oa.open_lib()
    d = oa.make_descriptor(lib, (3, 4, 5), None, oa.F16)
    assert d.contents.ndim == 3
    assert [d.contents.shape[i] for i in range(3)] == [3, 4, 5]
    assert [d.contents.strides[i] for i in range(3)] == [20, 5, 1]  # NULL strides = contiguous
    assert lib.infiniopDestroyTensorDescriptor(d) == 0
    d = oa.make_descriptor(lib, (3, 4), (100, 2), oa.BF16)
    assert [d.contents.strides[i] for i in range(2)] == [100, 2]
    assert d.contents.dt == oa.BF16
    assert lib.infiniopDestroyTensorDescriptor(d) == 0
    d = oa.make_descriptor(lib, (), None, oa.F32)  # rank 0
    assert d.contents.ndim == 0
    assert lib.infiniopDestroyTensorDescriptor(d) == 0


def test_create_handle_argument_checks():
    lib = oa.open_lib()
    h = oa.infiniopHandle_t()
    assert lib.infiniopCreateHandle(None, oa.DeviceEnum.DEVICE_AMD, 0) == 6   # MEMORY_NOT_ALLOCATED
    assert lib.infiniopCreateHandle(ctypes.byref(h), oa.DeviceEnum.DEVICE_AMD, -1) == 2  # BAD_PARAM
    for other in (oa.DeviceEnum.DEVICE_CPU, oa.DeviceEnum.DEVICE_CUDA, oa.DeviceEnum.DEVICE_BANG, oa.DeviceEnum.DEVICE_ASCEND, 17):
        assert lib.infiniopCreateHandle(ctypes.byref(h), other, 0) == 8    # BAD_DEVICE: no CPU or other path inside
    assert lib.infiniopCreateHandle(ctypes.byref(h), oa.DeviceEnum.DEVICE_AMD, 4096) == 8  # no such GPU (or no GPU at all)


def test_no_cpu_fallback_in_python_layer():
    """The package must fail loudly, not compute on the host, when the library is absent."""
    with pytest.raises(FileNotFoundError):
        oa.open_lib("/nonexistent/libinfiniop.so")
    import operators_amd.ops as ops
    src = open(ops.__file__).read() + open(oa.__file__).read()
    assert "oracle" not in src
