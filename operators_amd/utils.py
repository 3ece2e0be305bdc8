"""Helpers for driving the C ABI from PyTorch tensors.

Same helper names and meaning as the reference's operatorspy/utils.py:6-108
(check_error, to_tensor, create_workspace, create_handle, destroy_handle,
rearrange_tensor), written for this library.
"""
import ctypes

from . import data_layout as dl
from .liboperators import CTensor, infiniopHandle_t, infiniopTensorDescriptor_t

STATUS_NAMES = {
    0: "STATUS_SUCCESS",
    1: "STATUS_EXECUTION_FAILED",
    2: "STATUS_BAD_PARAM",
    3: "STATUS_BAD_TENSOR_DTYPE",
    4: "STATUS_BAD_TENSOR_SHAPE",
    5: "STATUS_BAD_TENSOR_STRIDES",
    6: "STATUS_MEMORY_NOT_ALLOCATED",
    7: "STATUS_INSUFFICIENT_WORKSPACE",
    8: "STATUS_BAD_DEVICE",
}


class InfiniopError(Exception):
    def __init__(self, status):
        self.status = status
        super().__init__(f"Error code {status} ({STATUS_NAMES.get(status, 'unknown')})")


def check_error(status):
    if status != 0:
        raise InfiniopError(status)


def torch_dtype_to_layout(dtype):
    import torch

    table = {
        torch.int8: dl.I8, torch.int16: dl.I16, torch.int32: dl.I32, torch.int64: dl.I64,
        torch.uint8: dl.U8, torch.float16: dl.F16, torch.bfloat16: dl.BF16,
        torch.float32: dl.F32, torch.float64: dl.F64,
    }
    for name, layout in (("uint16", dl.U16), ("uint32", dl.U32), ("uint64", dl.U64)):
        if hasattr(torch, name):
            table[getattr(torch, name)] = layout
    if dtype not in table:
        raise TypeError(f"no DataLayout for {dtype}")
    return table[dtype]


def make_descriptor(lib, shape, strides, layout):
    """infiniopCreateTensorDescriptor from Python sequences; strides=None means contiguous."""
    ndim = len(shape)
    c_shape = (ctypes.c_uint64 * ndim)(*shape)
    c_strides = None if strides is None else (ctypes.c_int64 * ndim)(*strides)
    desc = infiniopTensorDescriptor_t()
    check_error(lib.infiniopCreateTensorDescriptor(ctypes.byref(desc), ndim, c_shape, c_strides, layout))
    return desc


def to_tensor(tensor, lib):
    """Describe a torch tensor (shape, strides in elements, dtype) and pair the
    descriptor with the tensor's data address."""
    desc = make_descriptor(lib, tuple(tensor.shape), tuple(tensor.stride()), torch_dtype_to_layout(tensor.dtype))
    return CTensor(desc, tensor.data_ptr())


def destroy_tensor(lib, ctensor):
    check_error(lib.infiniopDestroyTensorDescriptor(ctensor.descriptor))


def create_workspace(size, torch_device):
    if size == 0:
        return None
    import torch

    return torch.zeros(size=(size,), dtype=torch.uint8, device=torch_device)


def create_handle(lib, device, id=0):
    handle = infiniopHandle_t()
    check_error(lib.infiniopCreateHandle(ctypes.byref(handle), device, id))
    return handle


def destroy_handle(lib, handle):
    check_error(lib.infiniopDestroyHandle(handle))


def rearrange_tensor(tensor, new_strides):
    """A tensor with the values of `tensor` laid out with the given positive
    strides (in elements) inside a fresh zero-filled buffer."""
    import torch

    shape = tuple(tensor.shape)
    if any(s <= 0 for s in new_strides):
        raise ValueError("only positive strides are supported")
    span = 1 + sum((n - 1) * s for n, s in zip(shape, new_strides))
    buf = torch.zeros((span,), dtype=tensor.dtype, device=tensor.device)
    view = torch.as_strided(buf, shape, tuple(new_strides))
    view.copy_(tensor)
    return view
