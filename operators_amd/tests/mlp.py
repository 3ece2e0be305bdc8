"""The MLP composite on the amd-gpu device: the reference's cases (operatorspy/tests/mlp.py:245-263) against its
torch formula (:36-55: gate = x @ w12[:, :di], up = x @ w12[:, di:], each rounded to the element type, SwiGLU, the
second product with alpha folded into w3, the residual) at the reference's tolerance (:133, rtol 2e-2)."""
import ctypes
import sys

import torch

from operators_amd import check_error, infiniopMLPDescriptor_t
from operators_amd.tests.test_utils import described, laid_out, run, workspace_for


def expected(y, x, w12, w3, alpha, residual):
    dt, di = x.dtype, w3.shape[0]
    x32 = x.to(torch.float32)
    gate = (x32 @ w12[:, :di].to(torch.float32)).to(dt)
    up = (x32 @ w12[:, di:].to(torch.float32)).to(dt)
    act = up * gate / (1 + torch.exp(-gate.float()).to(dt))
    out = (act.to(torch.float32) @ (alpha * w3.to(torch.float32))).to(dt)
    return out + y if residual else out


def test(lib, handle, torch_device, tokens, hidden, inter, alpha, residual, dtype=torch.float16, x_strides=None, y_strides=None,
         w12_strides=None, w3_strides=None):
    print(f"Testing MLP on {torch_device} with num_tokens:{tokens} hidden_size:{hidden} intermediate_size:{inter} alpha:{alpha} residual:{residual}"
          f" dtype:{dtype} x_stride:{x_strides} y_stride:{y_strides} w12_stride:{w12_strides} w3_stride:{w3_strides}")
    y = torch.rand([tokens, hidden], dtype=dtype).to(torch_device) * 0.01
    x = torch.rand([tokens, hidden], dtype=dtype).to(torch_device) * 0.01
    w12 = torch.rand([hidden, 2 * inter], dtype=dtype).to(torch_device) * 0.01
    w3 = torch.rand([inter, hidden], dtype=dtype).to(torch_device) * 0.01
    want = expected(y, x, w12, w3, alpha, residual)
    y, x, w12, w3 = laid_out(y, y_strides), laid_out(x, x_strides), laid_out(w12, w12_strides), laid_out(w3, w3_strides)
    with described(lib, y, x, w12, w3) as (ty, tx, t12, t3):
        desc = infiniopMLPDescriptor_t()
        check_error(lib.infiniopCreateMLPDescriptor(handle, ctypes.byref(desc), ty.descriptor, tx.descriptor, t12.descriptor, t3.descriptor,
                                                    alpha, ctypes.c_char(b"\x01" if residual else b"\x00")))
        ws, size, owner = workspace_for(lib, lib.infiniopGetMLPWorkspaceSize, desc, x.device)
        check_error(lib.infiniopMLP(desc, ws, size, ty.data, tx.data, t12.data, t3.data, None))
        torch.cuda.synchronize()
        check_error(lib.infiniopDestroyMLPDescriptor(desc))
    assert torch.allclose(y, want, atol=0, rtol=2e-2)


TEST_CASES = [
    # tokens, hidden, intermediate, alpha, residual, dtype, strides of x, y, w12, w3 (elements)
    (4, 4096, 11008, 1.0, True, torch.float16, None, None, None, None),
    (4, 4096, 11008, 1.0, True, torch.float16, [8192, 1], [8192, 1], None, None),
    (4, 4096, 11008, 1.0, True, torch.float16, None, None, [1, 4096], [1, 11008]),
    (4, 4096, 11008, 1.0, False, torch.float16, None, None, None, None),
    (4, 4096, 11008, 1.0, False, torch.float16, [8192, 1], [8192, 1], None, None),
    (16, 4096, 11008, 1.0, True, torch.bfloat16, None, None, None, None),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
