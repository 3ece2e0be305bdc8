"""Loader and ctypes prototypes for libinfiniop.so (amd-gpu build).

Counterpart of the reference's operatorspy/liboperators.py:11-73: the library is
looked up under $INFINI_ROOT/lib when INFINI_ROOT is set, otherwise in this
package's own lib/ directory (where `python -m operators_amd.build` puts it).
There is no fallback implementation: if the library is missing, `open_lib`
raises.
"""
import ctypes
import os
from ctypes import POINTER, Structure, c_char, c_float, c_int, c_int32, c_int64, c_uint64, c_void_p

from .data_layout import DataLayout

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libinfiniop.so"


class TensorDescriptor(Structure):
    _fields_ = [
        ("dt", DataLayout),
        ("ndim", c_uint64),
        ("shape", POINTER(c_uint64)),
        ("strides", POINTER(c_int64)),
    ]


infiniopTensorDescriptor_t = POINTER(TensorDescriptor)


class Handle(Structure):
    _fields_ = [("device", c_int)]


infiniopHandle_t = POINTER(Handle)


class _OpDescriptor(Structure):
    """Every operator descriptor starts with its device number; nothing else
    of it is visible to callers."""
    _fields_ = [("device", c_int32)]


class AddDescriptor(_OpDescriptor):
    pass


class RMSNormDescriptor(_OpDescriptor):
    pass


class RoPEDescriptor(_OpDescriptor):
    pass


class SwiGLUDescriptor(_OpDescriptor):
    pass


class CausalSoftmaxDescriptor(_OpDescriptor):
    pass


class RearrangeDescriptor(_OpDescriptor):
    pass


class AddRMSNormDescriptor(_OpDescriptor):
    pass


class MatmulDescriptor(_OpDescriptor):
    pass


class MLPDescriptor(_OpDescriptor):
    pass


class AttentionDescriptor(_OpDescriptor):
    pass


class RandomSampleDescriptor(_OpDescriptor):
    pass


infiniopAddDescriptor_t = POINTER(AddDescriptor)
infiniopRMSNormDescriptor_t = POINTER(RMSNormDescriptor)
infiniopRoPEDescriptor_t = POINTER(RoPEDescriptor)
infiniopSwiGLUDescriptor_t = POINTER(SwiGLUDescriptor)
infiniopCausalSoftmaxDescriptor_t = POINTER(CausalSoftmaxDescriptor)
infiniopRearrangeDescriptor_t = POINTER(RearrangeDescriptor)
infiniopAddRMSNormDescriptor_t = POINTER(AddRMSNormDescriptor)
infiniopMatmulDescriptor_t = POINTER(MatmulDescriptor)
infiniopMLPDescriptor_t = POINTER(MLPDescriptor)
infiniopAttentionDescriptor_t = POINTER(AttentionDescriptor)
infiniopRandomSampleDescriptor_t = POINTER(RandomSampleDescriptor)


class CTensor:
    """A tensor descriptor together with the address of its data."""

    def __init__(self, desc, data):
        self.descriptor = desc
        self.data = data


def library_path():
    root = os.environ.get("INFINI_ROOT")
    if root:
        return os.path.join(root, "lib", LIB_NAME)
    return os.path.join(_PKG_DIR, "lib", LIB_NAME)


# name -> (argtypes); every entry point returns an infiniopStatus_t (int32)
_PROTOTYPES = {
    "infiniopCreateHandle": [POINTER(infiniopHandle_t), c_int, c_int],
    "infiniopDestroyHandle": [infiniopHandle_t],
    "infiniopCreateTensorDescriptor": [POINTER(infiniopTensorDescriptor_t), c_uint64, POINTER(c_uint64), POINTER(c_int64), DataLayout],
    "infiniopDestroyTensorDescriptor": [infiniopTensorDescriptor_t],
    "infiniopCreateAddDescriptor": [infiniopHandle_t, POINTER(infiniopAddDescriptor_t)] + [infiniopTensorDescriptor_t] * 3,
    "infiniopAdd": [infiniopAddDescriptor_t, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyAddDescriptor": [infiniopAddDescriptor_t],
    "infiniopCreateRMSNormDescriptor": [infiniopHandle_t, POINTER(infiniopRMSNormDescriptor_t)] + [infiniopTensorDescriptor_t] * 3 + [c_float],
    "infiniopGetRMSNormWorkspaceSize": [infiniopRMSNormDescriptor_t, POINTER(c_uint64)],
    "infiniopRMSNorm": [infiniopRMSNormDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyRMSNormDescriptor": [infiniopRMSNormDescriptor_t],
    "infiniopCreateRoPEDescriptor": [infiniopHandle_t, POINTER(infiniopRoPEDescriptor_t)] + [infiniopTensorDescriptor_t] * 4,
    "infiniopGetRoPEWorkspaceSize": [infiniopRoPEDescriptor_t, POINTER(c_uint64)],
    "infiniopRoPE": [infiniopRoPEDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyRoPEDescriptor": [infiniopRoPEDescriptor_t],
    "infiniopCreateSwiGLUDescriptor": [infiniopHandle_t, POINTER(infiniopSwiGLUDescriptor_t)] + [infiniopTensorDescriptor_t] * 3,
    "infiniopSwiGLU": [infiniopSwiGLUDescriptor_t, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroySwiGLUDescriptor": [infiniopSwiGLUDescriptor_t],
    "infiniopCreateCausalSoftmaxDescriptor": [infiniopHandle_t, POINTER(infiniopCausalSoftmaxDescriptor_t), infiniopTensorDescriptor_t],
    "infiniopGetCausalSoftmaxWorkspaceSize": [infiniopCausalSoftmaxDescriptor_t, POINTER(c_uint64)],
    "infiniopCausalSoftmax": [infiniopCausalSoftmaxDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p],
    "infiniopDestroyCausalSoftmaxDescriptor": [infiniopCausalSoftmaxDescriptor_t],
    "infiniopCreateRearrangeDescriptor": [infiniopHandle_t, POINTER(infiniopRearrangeDescriptor_t), infiniopTensorDescriptor_t, infiniopTensorDescriptor_t],
    "infiniopRearrange": [infiniopRearrangeDescriptor_t, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyRearrangeDescriptor": [infiniopRearrangeDescriptor_t],
    "infiniopCreateMatmulDescriptor": [infiniopHandle_t, POINTER(infiniopMatmulDescriptor_t), infiniopTensorDescriptor_t, c_float,
                                       infiniopTensorDescriptor_t, infiniopTensorDescriptor_t, c_float],
    "infiniopGetMatmulWorkspaceSize": [infiniopMatmulDescriptor_t, POINTER(c_uint64)],
    "infiniopMatmul": [infiniopMatmulDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyMatmulDescriptor": [infiniopMatmulDescriptor_t],
    "infiniopCreateMLPDescriptor": [infiniopHandle_t, POINTER(infiniopMLPDescriptor_t)] + [infiniopTensorDescriptor_t] * 4 + [c_float, c_char],
    "infiniopGetMLPWorkspaceSize": [infiniopMLPDescriptor_t, POINTER(c_uint64)],
    "infiniopMLP": [infiniopMLPDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyMLPDescriptor": [infiniopMLPDescriptor_t],
    "infiniopCreateAttentionDescriptor": [infiniopHandle_t, POINTER(infiniopAttentionDescriptor_t)] + [infiniopTensorDescriptor_t] * 6 + [c_uint64],
    "infiniopGetAttentionWorkspaceSize": [infiniopAttentionDescriptor_t, POINTER(c_uint64)],
    "infiniopAttention": [infiniopAttentionDescriptor_t, c_void_p, c_uint64] + [c_void_p] * 7,
    "infiniopDestroyAttentionDescriptor": [infiniopAttentionDescriptor_t],
    "infiniopCreateRandomSampleDescriptor": [infiniopHandle_t, POINTER(infiniopRandomSampleDescriptor_t), infiniopTensorDescriptor_t, infiniopTensorDescriptor_t],
    "infiniopGetRandomSampleWorkspaceSize": [infiniopRandomSampleDescriptor_t, POINTER(c_uint64)],
    "infiniopRandomSample": [infiniopRandomSampleDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_float, c_float, c_int, c_float, c_void_p],
    "infiniopRandomSampleNoAlloc": [infiniopRandomSampleDescriptor_t, c_void_p, c_void_p, c_float, c_float, c_int, c_float, c_void_p],
    "infiniopDestroyRandomSampleDescriptor": [infiniopRandomSampleDescriptor_t],
    "infiniopCreateAddRMSNormDescriptor": [infiniopHandle_t, POINTER(infiniopAddRMSNormDescriptor_t)] + [infiniopTensorDescriptor_t] * 5 + [c_float],
    "infiniopGetAddRMSNormWorkspaceSize": [infiniopAddRMSNormDescriptor_t, POINTER(c_uint64)],
    "infiniopAddRMSNorm": [infiniopAddRMSNormDescriptor_t, c_void_p, c_uint64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "infiniopDestroyAddRMSNormDescriptor": [infiniopAddRMSNormDescriptor_t],
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)


# Entry points of this library that the reference does not have.
EXTENSION_SYMBOLS = tuple(n for n in _PROTOTYPES if "AddRMSNorm" in n or "NoAlloc" in n)


def bind_prototypes(lib, extensions=True):
    """Attach argument and result types for every entry point.  Works on any
    library exporting the same C ABI: this one, or (with extensions=False) a
    build of the reference, which lacks the fused operator."""
    for name, argtypes in _PROTOTYPES.items():
        if not extensions and name in EXTENSION_SYMBOLS:
            continue
        fn = getattr(lib, name)  # AttributeError names the missing symbol
        fn.argtypes = argtypes
        fn.restype = c_int32
    return lib


_cached = {}


def open_lib(path=None):
    path = path or library_path()
    if path in _cached:
        return _cached[path]
    # PyTorch-ROCm ships its own copy of the HIP runtime (same SONAME as the
    # system one).  Two HIP runtimes in one process cannot both own the GPU, so
    # when torch is going to be used in this process it has to be loaded first:
    # the dynamic linker then binds this library to the copy torch brought.
    try:
        import torch  # noqa: F401
    except ImportError:
        pass
    if not os.path.isfile(path):
        raise FileNotFoundError(
            f"{path} not found: build it with `python -m operators_amd.build` "
            "or point INFINI_ROOT at an installed copy")
    lib = bind_prototypes(ctypes.CDLL(path))
    _cached[path] = lib
    return lib
