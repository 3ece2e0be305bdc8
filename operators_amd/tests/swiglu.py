"""SwiGLU on the amd-gpu device, the reference's cases (operatorspy/tests/swiglu.py:240-246),
out of place and in place on either operand, against its torch formula (:30-32) at its
tolerance (:83, atol 1e-4, rtol 1e-2)."""
import ctypes
import sys

import torch

from operators_amd import check_error, destroy_tensor, infiniopSwiGLUDescriptor_t, rearrange_tensor, to_tensor
from operators_amd.tests.test_utils import run


def swiglu(a, b):
    return a * b / (1 + torch.exp(-b.float()).to(b.dtype))


def test(lib, handle, torch_device, shape, a_stride=None, b_stride=None, c_stride=None, dtype=torch.float16):
    for mode in ("out of place", "in place on a", "in place on b"):
        print(f"Testing SwiGLU on {torch_device} with shape:{shape} a_stride:{a_stride} b_stride:{b_stride} c_stride:{c_stride} dtype:{dtype} {mode}")
        a = torch.rand(shape, dtype=dtype).to(torch_device)
        b = torch.rand(shape, dtype=dtype).to(torch_device)
        if a_stride is not None:
            a = rearrange_tensor(a, a_stride)
        if b_stride is not None:
            b = rearrange_tensor(b, b_stride)
        ans = swiglu(a, b)
        if mode == "out of place":
            c = torch.rand(shape, dtype=dtype).to(torch_device)
            if c_stride is not None:
                c = rearrange_tensor(c, c_stride)
        else:
            c = a if mode == "in place on a" else b
        ta, tb = to_tensor(a, lib), to_tensor(b, lib)
        tc = to_tensor(c, lib) if mode == "out of place" else (ta if mode == "in place on a" else tb)
        desc = infiniopSwiGLUDescriptor_t()
        check_error(lib.infiniopCreateSwiGLUDescriptor(handle, ctypes.byref(desc), tc.descriptor, ta.descriptor, tb.descriptor))
        check_error(lib.infiniopSwiGLU(desc, tc.data, ta.data, tb.data, None))
        torch.cuda.synchronize()
        tol = (1e-4, 1e-2) if dtype == torch.float16 else (1e-2, 2e-2)
        assert torch.allclose(c, ans, atol=tol[0], rtol=tol[1])
        check_error(lib.infiniopDestroySwiGLUDescriptor(desc))
        for t in {id(x): x for x in (ta, tb, tc)}.values():
            destroy_tensor(lib, t)


TEST_CASES = [
    ((13, 4), None, None, None, torch.float16),
    ((13, 4), (10, 1), (10, 1), (10, 1), torch.float16),
    ((16, 5632), None, None, None, torch.float16),
    ((16, 5632), (13312, 1), (13312, 1), (13312, 1), torch.float16),
    ((16, 5632), (13312, 1), (13312, 1), None, torch.bfloat16),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
