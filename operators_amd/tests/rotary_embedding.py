"""RoPE on the amd-gpu device, the reference's cases (operatorspy/tests/rotary_embedding.py:169-178)
against its complex-multiplication formula (:41-52) at its tolerance (:129, atol 1e-4, rtol 1e-2)."""
import ctypes
import sys

import torch

from operators_amd import check_error, create_workspace, destroy_tensor, infiniopRoPEDescriptor_t, rearrange_tensor, to_tensor
from operators_amd.ops import sin_cos_table
from operators_amd.tests.test_utils import run


def rotary_embedding(t, pos, theta):
    dh = t.shape[2]
    freqs = 1.0 / (theta ** (torch.arange(0, dh, 2)[: dh // 2].float() / dh))
    cis = torch.polar(torch.ones(pos.numel(), dh // 2), torch.outer(pos.float(), freqs))
    t_ = torch.view_as_complex(t.float().reshape(*t.shape[:-1], -1, 2))
    return torch.view_as_real(t_ * cis[:, None, :]).flatten(2).to(t.dtype)


def test(lib, handle, torch_device, shape, strides=None, dtype=torch.float16):
    print(f"Testing Rotary Positional Embedding on {torch_device} with shape:{shape} strides:{strides} and dtype:{dtype}")
    t = torch.rand(shape, dtype=dtype)
    if strides is not None:
        t = rearrange_tensor(t, strides)
    pos = torch.arange(0, t.shape[0])
    theta = 1e4
    ans = rotary_embedding(t, pos, theta)
    t = t.to(torch_device)
    pos = pos.to(torch.int64).to(torch_device).view(torch.uint64)
    sin_t, cos_t = sin_cos_table(t.shape[0] * 2, t.shape[2], theta, device=torch_device)
    tt, tp, ts, tcos = to_tensor(t, lib), to_tensor(pos, lib), to_tensor(sin_t, lib), to_tensor(cos_t, lib)
    desc = infiniopRoPEDescriptor_t()
    check_error(lib.infiniopCreateRoPEDescriptor(handle, ctypes.byref(desc), tt.descriptor, tp.descriptor, ts.descriptor, tcos.descriptor))
    size = ctypes.c_uint64(0)
    check_error(lib.infiniopGetRoPEWorkspaceSize(desc, ctypes.byref(size)))
    workspace = create_workspace(size.value, t.device)
    check_error(lib.infiniopRoPE(desc, workspace.data_ptr() if workspace is not None else None, size.value, tt.data, tp.data, ts.data, tcos.data, None))
    torch.cuda.synchronize()
    tol = (1e-4, 1e-2) if dtype == torch.float16 else (1e-2, 2e-2)
    assert torch.allclose(t.cpu(), ans, atol=tol[0], rtol=tol[1])
    check_error(lib.infiniopDestroyRoPEDescriptor(desc))
    for x in (tt, tp, ts, tcos):
        destroy_tensor(lib, x)


TEST_CASES = [
    ((1, 32, 128), None, torch.float16),
    ((1, 32, 64), None, torch.float16),
    ((4, 1, 32), None, torch.float16),
    ((1, 32, 128), None, torch.float16),
    ((3, 32, 128), (8000, 200, 1), torch.float16),
    ((64, 8, 128), (10240, 128, 1), torch.bfloat16),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
