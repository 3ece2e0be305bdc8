"""Rearrange on the amd-gpu device: the reference's cases (operatorspy/tests/rearrange.py:109-117), compared
exactly (a copy has no tolerance; the reference's :56 allows rtol 1e-3)."""
import ctypes
import sys

import torch

from operators_amd import check_error, infiniopRearrangeDescriptor_t
from operators_amd.tests.test_utils import described, laid_out, run


def test(lib, handle, torch_device, src, dst, dtype=torch.float16):
    (src_shape, src_strides), (dst_shape, dst_strides) = src, dst
    print(f"Testing Rearrange on {torch_device} with x_shape:{src_shape} x_stride:{src_strides} y_shape:{dst_shape} y_stride:{dst_strides} dtype:{dtype}")
    x = laid_out(torch.rand(src_shape, dtype=dtype).to(torch_device), src_strides)
    y = laid_out(torch.zeros(dst_shape, dtype=dtype).to(torch_device), dst_strides)
    with described(lib, y, x) as (ty, tx):
        desc = infiniopRearrangeDescriptor_t()
        check_error(lib.infiniopCreateRearrangeDescriptor(handle, ctypes.byref(desc), ty.descriptor, tx.descriptor))
        check_error(lib.infiniopRearrange(desc, ty.data, tx.data, None))
        torch.cuda.synchronize()
        check_error(lib.infiniopDestroyRearrangeDescriptor(desc))
    assert torch.equal(x, y)


TEST_CASES = [
    # (source shape, source strides), (destination shape, destination strides)
    (((2, 4, 32), None), ((2, 4, 32), (256, 64, 1))),
    (((32, 6, 64), (64, 2560, 1)), ((32, 6, 64), None)),
    (((4, 6, 64), (64, 2560, 1)), ((4, 6, 64), (131072, 64, 1))),
    (((1, 32, 64), (2048, 64, 1)), ((1, 32, 64), (2048, 64, 1))),
    (((32, 1, 64), (64, 2560, 1)), ((32, 1, 64), (64, 64, 1))),
    (((4, 1, 64), (64, 2560, 1)), ((4, 1, 64), (64, 11264, 1))),
    # the head transpose of attention, bf16
    (((64, 8, 128), (1024, 128, 1)), ((64, 8, 128), (128, 8192, 1)), torch.bfloat16),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
