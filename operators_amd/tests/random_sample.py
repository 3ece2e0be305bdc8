"""RandomSample on the amd-gpu device: the reference's cases (operatorspy/tests/random_sample.py:177-189).
The expected index follows the reference's CPU back end (src/ops/random_sample/cpu/random_sample.cc:80-158): the
topk largest logits in descending order, softmax with temperature over ALL logits, the shortest prefix of the
candidates whose probability reaches topp, and the first candidate whose running sum exceeds random_val times that
prefix's mass.  Equal logits may come in any order (the reference's own test accepts an index of equal value, :133)."""
import ctypes
import sys

import torch

from operators_amd import check_error, infiniopRandomSampleDescriptor_t
from operators_amd.tests.test_utils import described, run, workspace_for


def narrowed(p, dtype):
    """fp32 probabilities as the library stores them: fp16 by truncation (the reference's conversion), bf16 to nearest even."""
    if dtype == torch.bfloat16:
        return p.to(torch.bfloat16).to(torch.float32)
    h = p.to(torch.float16)
    bits = h.view(torch.int16) - (h.to(torch.float32) > p).to(torch.int16)  # positive values: one step towards zero
    return bits.view(torch.float16).to(torch.float32)


def expected(logits, random_val, topp, topk, temperature):
    if not (topp > 0 and topk > 1):
        return int(torch.argmax(logits))
    x = logits.to(torch.float32).cpu()
    k = min(topk, x.numel())
    top, idx = torch.sort(x, descending=True, stable=True)
    e = torch.exp((top - top[0]) / temperature)
    probs = narrowed(e / e.sum(), logits.dtype)[:k].tolist()
    run, last = 0.0, k
    for i, p in enumerate(probs):
        run = float(torch.tensor(run, dtype=torch.float32) + torch.tensor(p, dtype=torch.float32))
        if run >= topp:
            last = i + 1 if i < k - 1 else k
            break
    kept = torch.tensor(probs[:last], dtype=torch.float32)
    total = torch.tensor(0.0)
    for p in kept:
        total = total + p
    threshold, run = torch.tensor(random_val, dtype=torch.float32) * total, torch.tensor(0.0)
    for i, p in enumerate(kept):
        run = run + p
        if threshold < run:
            return int(idx[i])
    return None


def test(lib, handle, torch_device, voc, random_val, topp, topk, temperature, dtype=torch.float16):
    print(f"Testing RandomSample on {torch_device} with voc:{voc} random_val:{random_val} topp:{topp} topk:{topk} temperature:{temperature} dtype:{dtype}")
    logits = torch.rand(voc, dtype=dtype).to(torch_device)
    want = expected(logits, random_val, topp, topk, temperature)
    result = torch.zeros(1, dtype=torch.int64, device=torch_device).view(torch.uint64)
    with described(lib, result, logits) as (tr, tl):
        desc = infiniopRandomSampleDescriptor_t()
        check_error(lib.infiniopCreateRandomSampleDescriptor(handle, ctypes.byref(desc), tr.descriptor, tl.descriptor))
        ws, size, owner = workspace_for(lib, lib.infiniopGetRandomSampleWorkspaceSize, desc, logits.device)
        check_error(lib.infiniopRandomSample(desc, ws, size, tr.data, tl.data, random_val, topp, topk, temperature, None))
        torch.cuda.synchronize()
        check_error(lib.infiniopDestroyRandomSampleDescriptor(desc))
    got = int(result.view(torch.int64).item())
    assert want is not None and (got == want or logits[got] == logits[want]), (got, want)


TEST_CASES = [
    # voc, random_val, topp, topk, temperature
    (512, 0.92, 0.8, 3, 0.5),
    (4096, 0.95, 0.9, 5, 1.0),
    (16384, 0.85, 0.85, 10, 2.0),
    (512, 0.92, 0, 3, 0.5),
    (4096, 0.95, 0.9, 1, 1.0),
    (16384, 0.85, 0, 1, 2.0),
    (16384, 0.85, 0, 1, 2.0),
    (32000, 0.8, 0.8, 50, 1.0),
    (32000, 0.8, 1.0, 25, 1.0),
    # beyond the reference's: the histogram form (more than 256 candidates) and bf16 logits
    (151936, 0.4, 0.95, 1000, 0.7),
    (32000, 0.6, 0.9, 40, 1.0, torch.bfloat16),
]

if __name__ == "__main__":
    sys.exit(run(TEST_CASES, test))
