"""Add on the amd-gpu device, the reference's cases (operatorspy/tests/add.py:114-127)
against torch.add at its tolerance (:80, atol 0, rtol 1e-3)."""
import ctypes
import sys

import torch

from operators_amd import check_error, destroy_tensor, infiniopAddDescriptor_t, to_tensor
from operators_amd.tests.test_utils import run

OUT_OF_PLACE, INPLACE_A, INPLACE_B = "out of place", "in place on a", "in place on b"


def test(lib, handle, torch_device, c_shape, a_shape, b_shape, inplace=OUT_OF_PLACE, dtype=torch.float16):
    print(f"Testing Add on {torch_device} with c_shape:{c_shape} a_shape:{a_shape} b_shape:{b_shape} dtype:{dtype} {inplace}")
    a = torch.rand(a_shape, dtype=dtype).to(torch_device)
    b = torch.rand(b_shape, dtype=dtype).to(torch_device)
    c = torch.rand(c_shape, dtype=dtype).to(torch_device) if inplace == OUT_OF_PLACE else (a if inplace == INPLACE_A else b)
    ans = torch.add(a, b)
    ta, tb = to_tensor(a, lib), to_tensor(b, lib)
    tc = to_tensor(c, lib) if inplace == OUT_OF_PLACE else (ta if inplace == INPLACE_A else tb)
    desc = infiniopAddDescriptor_t()
    check_error(lib.infiniopCreateAddDescriptor(handle, ctypes.byref(desc), tc.descriptor, ta.descriptor, tb.descriptor))
    check_error(lib.infiniopAdd(desc, tc.data, ta.data, tb.data, None))
    torch.cuda.synchronize()
    assert torch.allclose(c, ans, atol=0, rtol=1e-3)
    check_error(lib.infiniopDestroyAddDescriptor(desc))
    for t in {id(x): x for x in (ta, tb, tc)}.values():
        destroy_tensor(lib, t)


TEST_CASES = [
    ((1, 3), (1, 3), (1, 3), OUT_OF_PLACE),
    ((), (), (), OUT_OF_PLACE),
    ((3, 3), (3, 3), (3, 3), OUT_OF_PLACE),
    ((2, 20, 3), (2, 1, 3), (2, 20, 3), OUT_OF_PLACE),
    ((32, 20, 512), (32, 20, 512), (32, 20, 512), INPLACE_A),
    ((32, 20, 512), (32, 20, 512), (32, 20, 512), INPLACE_B),
    ((32, 256, 112, 112), (32, 256, 112, 1), (32, 256, 112, 112), OUT_OF_PLACE),
    ((32, 256, 112, 112), (32, 256, 112, 112), (32, 256, 112, 112), OUT_OF_PLACE),
    ((2, 4, 3), (2, 1, 3), (4, 3), OUT_OF_PLACE),
    ((2, 3, 4, 5), (2, 3, 4, 5), (5,), OUT_OF_PLACE),
    ((3, 2, 4, 5), (4, 5), (3, 2, 1, 1), OUT_OF_PLACE),
]
TEST_CASES += [c + (torch.float32,) for c in TEST_CASES[:4]] + [c + (torch.bfloat16,) for c in TEST_CASES[:4]]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
