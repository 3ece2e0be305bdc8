"""CausalSoftmax on the amd-gpu device: the reference's cases (operatorspy/tests/causal_softmax.py:111-115) and a
few of this back end's launch forms, against a torch formula at the reference's tolerance (:73, rtol 1e-2)."""
import ctypes
import sys

import torch

from operators_amd import check_error, infiniopCausalSoftmaxDescriptor_t
from operators_amd.tests.test_utils import described, laid_out, run, workspace_for


def expected(x):
    """Row i of each [seq, total] matrix keeps columns j <= total - seq + i."""
    seq, total = x.shape[-2], x.shape[-1]
    cols = torch.arange(total, device=x.device)
    keep = cols[None, :] <= (total - seq) + torch.arange(seq, device=x.device)[:, None]
    scores = x.to(torch.float32).masked_fill(~keep, float("-inf"))
    return torch.softmax(scores, dim=-1).to(x.dtype)


def test(lib, handle, torch_device, shape, strides=None, dtype=torch.float16):
    print(f"Testing CausalSoftmax on {torch_device} with x_shape:{shape} x_stride:{strides} dtype:{dtype}")
    x = laid_out(torch.rand(shape, dtype=dtype).to(torch_device), strides)
    want = expected(x)
    with described(lib, x) as (tx,):
        desc = infiniopCausalSoftmaxDescriptor_t()
        check_error(lib.infiniopCreateCausalSoftmaxDescriptor(handle, ctypes.byref(desc), tx.descriptor))
        ws, size, owner = workspace_for(lib, lib.infiniopGetCausalSoftmaxWorkspaceSize, desc, x.device)
        check_error(lib.infiniopCausalSoftmax(desc, ws, size, tx.data, None))
        torch.cuda.synchronize()
        check_error(lib.infiniopDestroyCausalSoftmaxDescriptor(desc))
    assert torch.allclose(x, want, atol=0, rtol=1e-2)
    assert bool((x.masked_select(want == 0) == 0).all())  # the masked part is exact zeros


TEST_CASES = [
    # shape, strides (elements)
    ((32, 20, 512), None),
    ((32, 20, 512), (20480, 512, 1)),
    # this back end's other forms: several rows per wavefront, ragged rows, rows of 512 lanes, rows held as raw words
    ((64, 128, 128), None, torch.float16),
    ((3, 33, 333), None, torch.float16),
    ((2, 16, 20480), None, torch.bfloat16),
    ((1, 8, 40000), None, torch.float16),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
