"""RMSNorm on the amd-gpu device, the reference's cases (operatorspy/tests/rms_norm.py:117-121)
against its torch formula (:32-37) at its tolerance (:81, atol 1e-3, rtol 1e-3)."""
import ctypes
import sys

import torch

from operators_amd import check_error, create_workspace, destroy_tensor, infiniopRMSNormDescriptor_t, to_tensor
from operators_amd.tests.test_utils import run


def rms_norm(x, w, eps):
    h = x.to(torch.float32)
    h = h * torch.rsqrt(h.pow(2).mean(-1, keepdim=True) + eps)
    return w * h.to(x.dtype)


def test(lib, handle, torch_device, y_shape, x_shape, w_shape, dtype=torch.float16, w_dtype=torch.float16):
    print(f"Testing RMS_Norm on {torch_device} with y_shape:{y_shape} x_shape:{x_shape} w_shape:{w_shape} dtype:{dtype} w_dtype:{w_dtype}")
    y = torch.zeros(y_shape, dtype=dtype).to(torch_device)
    x = torch.rand(x_shape, dtype=dtype).to(torch_device)
    w = torch.ones(w_shape, dtype=w_dtype).to(torch_device)
    eps = 1e-5
    ans = rms_norm(x, w, eps)
    ty, tx, tw = to_tensor(y, lib), to_tensor(x, lib), to_tensor(w, lib)
    desc = infiniopRMSNormDescriptor_t()
    check_error(lib.infiniopCreateRMSNormDescriptor(handle, ctypes.byref(desc), ty.descriptor, tx.descriptor, tw.descriptor, eps))
    size = ctypes.c_uint64(0)
    check_error(lib.infiniopGetRMSNormWorkspaceSize(desc, ctypes.byref(size)))
    workspace = create_workspace(size.value, y.device)
    check_error(lib.infiniopRMSNorm(desc, workspace.data_ptr() if workspace is not None else None, size.value, ty.data, tx.data, tw.data, None))
    torch.cuda.synchronize()
    tol = 1e-3 if dtype == torch.float16 else 1e-2
    assert torch.allclose(y.to(dtype), ans.to(dtype), atol=tol, rtol=tol)
    check_error(lib.infiniopDestroyRMSNormDescriptor(desc))
    for t in (ty, tx, tw):
        destroy_tensor(lib, t)


TEST_CASES = [
    ((16, 2048), (16, 2048), (2048,), torch.float16, torch.float16),
    ((16, 2048), (16, 2048), (2048,), torch.float16, torch.float32),
    ((64, 8192), (64, 8192), (8192,), torch.bfloat16, torch.float32),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
