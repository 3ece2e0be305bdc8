"""The script-form tests (`python -m operators_amd.tests.<op> --amd`, the
reference's own case tables against torch at the reference's tolerances) run
in-process: every case of every script must pass on the amd-gpu device."""
import importlib

import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("op", ["add", "rms_norm", "rotary_embedding", "swiglu", "causal_softmax", "rearrange", "random_sample", "matmul", "mlp"])
def test_reference_style_cases(ctx, op, capsys):
    import torch

    mod = importlib.import_module(f"operators_amd.tests.{op}")
    torch.manual_seed(0)
    for case in mod.TEST_CASES:
        mod.test(ctx.lib, ctx.handle, "cuda", *case)
    out = capsys.readouterr().out
    assert out.count("Testing") >= len(mod.TEST_CASES)
