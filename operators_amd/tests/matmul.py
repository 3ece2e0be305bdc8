"""Matmul on the amd-gpu device: the reference's cases (operatorspy/tests/matmul.py:296-308) against torch's
fp32 product at the reference's tolerance (:120, rtol 1e-2), plus bf16."""
import ctypes
import sys

import torch

from operators_amd import check_error, infiniopMatmulDescriptor_t
from operators_amd.tests.test_utils import described, laid_out, run, workspace_for


def test(lib, handle, torch_device, alpha, beta, a_shape, b_shape, c_shape, a_strides=None, b_strides=None, c_strides=None, dtype=torch.float16):
    print(f"Testing Matmul on {torch_device} with a_shape:{a_shape} b_shape:{b_shape} c_shape:{c_shape}"
          f" a_stride:{a_strides} b_stride:{b_strides} c_stride:{c_strides} alpha:{alpha} beta:{beta} dtype:{dtype}")
    a = torch.rand(a_shape, dtype=dtype).to(torch_device)
    b = torch.rand(b_shape, dtype=dtype).to(torch_device)
    c = torch.ones(c_shape, dtype=dtype).to(torch_device)
    want = alpha * torch.matmul(a.to(torch.float32), b.to(torch.float32)).to(dtype) + beta * c
    a, b, c = laid_out(a, a_strides), laid_out(b, b_strides), laid_out(c, c_strides)
    with described(lib, c, a, b) as (tc, ta, tb):
        desc = infiniopMatmulDescriptor_t()
        check_error(lib.infiniopCreateMatmulDescriptor(handle, ctypes.byref(desc), tc.descriptor, alpha, ta.descriptor, tb.descriptor, beta))
        ws, size, owner = workspace_for(lib, lib.infiniopGetMatmulWorkspaceSize, desc, a.device)
        check_error(lib.infiniopMatmul(desc, ws, size, tc.data, ta.data, tb.data, None))
        torch.cuda.synchronize()
        check_error(lib.infiniopDestroyMatmulDescriptor(desc))
    assert torch.allclose(c, want, atol=0, rtol=1e-2)


_SHAPES = [
    # alpha, beta, a, b, c, strides of a, b, c (elements)
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), None, None, None),
    (1.0, 0.0, (2, 4, 2048), (2, 2048, 2048), (2, 4, 2048), None, None, None),
    (1.0, 0.0, (1, 2048), (2048, 2048), (1, 2048), (4096, 1), (4096, 1), (4096, 1)),
    (1.0, 1.0, (6, 2048), (2048, 2560), (6, 2560), (2048, 1), (1, 2048), (2560, 1)),
    (1.0 / 8.0, 0.0, (4, 8 * 6, 64), (4, 64, 6), (4, 8 * 6, 6), None, None, None),
]
TEST_CASES = [case + (dt,) for case in _SHAPES for dt in (torch.float16, torch.float32)] + [_SHAPES[3] + (torch.bfloat16,)]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
