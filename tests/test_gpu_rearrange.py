"""Rearrange on the GPU through the C ABI: byte-exact against the reference's
golden vectors and the oracle, including the bytes it must not touch."""
import numpy as np
import pytest

import oracle
from helpers import golden, golden_json

pytestmark = pytest.mark.gpu
NP_OF = {"f16": np.uint16, "f32": np.float32, "u8": np.uint8, "f64": np.float64, "bf16": np.uint16}


def torch_dtype(dt):
    import torch

    return {"f16": torch.float16, "bf16": torch.bfloat16, "f32": torch.float32, "u8": torch.uint8, "f64": torch.float64}[dt]


def contig(shape):
    out, run = [], 1
    for n in reversed(shape):
        out.append(run)
        run *= n
    return list(reversed(out))


def device_view(buf_np, dt, shape, strides):
    """Upload a flat numpy buffer bit for bit and view it with the given strides."""
    import torch

    raw = torch.from_numpy(np.ascontiguousarray(buf_np).view(np.uint8).copy()).cuda()
    typed = raw.view(torch_dtype(dt))
    return torch.as_strided(typed, tuple(shape), tuple(strides)), raw


def run_case(ctx, dt, shape, ss, sd, src_buf, dst_buf):
    import torch

    ss, sd = ss or contig(shape), sd or contig(shape)
    src, _ = device_view(src_buf, dt, shape, ss)
    dst, dst_raw = device_view(dst_buf, dt, shape, sd)
    ctx.rearrange(dst, src)
    torch.cuda.synchronize()
    return dst_raw.cpu().numpy()


def test_golden_cases(ctx):
    g = golden("rearrange")
    for i, (dt, shape, ss, sd) in enumerate(golden_json()["rearrange_cases"]):
        got = run_case(ctx, dt, shape, ss, sd, g[f"rearrange{i}_src"], g[f"rearrange{i}_dst_before"])
        assert np.array_equal(got, g[f"rearrange{i}_dst_after"].view(np.uint8)), (i, dt, shape, ss, sd)


CASES = [
    # dtype, shape, src strides, dst strides
    ("f16", (2048, 8, 128), (80 * 128, 128, 1), (128, 2048 * 128, 1)),       # k heads of a fused qkv buffer -> [head, token, dim] cache
    ("bf16", (512, 64, 128), (64 * 128, 128, 1), (128, 512 * 128, 1)),       # [token, head, dim] -> [head, token, dim]
    ("f16", (64, 1000), (1000, 1), (1024, 1)),                               # row padding
    ("f16", (33, 7, 5), (40, 5, 1), (35, 5, 1)),                             # odd row length: 2-byte units
    ("u8", (9, 77), (80, 1), (77, 1)),                                       # 1-byte units
    ("f32", (4, 3, 2, 50), (3 * 128, 128, 64, 1), (300, 100, 50, 1)),
    ("f16", (1 << 20,), None, None),                                         # one contiguous row
    ("f16", (3, 5, 7, 2, 16), (5 * 7 * 64, 7 * 64, 64, 32, 1), (5 * 7 * 32, 7 * 32, 32, 16, 1)),
    ("f64", (100, 10), (16, 1), None),
    # 128 MiB outputs: large enough for the write-through store path of both kernels
    ("bf16", (8192, 64, 128), (80 * 128, 128, 1), (128, 8192 * 128, 1)),     # q heads -> [head, token, dim], 256-byte rows
    ("f16", (4096, 16384), (16384, 1), (16392, 1)),                          # long rows into a padded destination
    # rows of 16 bytes and more that do not lie on 16-byte boundaries: 16-byte units at any boundary, the last one overlapping
    ("u8", (37, 17), (19, 1), (23, 1)),                                      # one whole unit and an overlapping one, odd pitches
    ("u8", (5, 3, 16), (3 * 17, 17, 1), (48, 16, 1)),                        # rows of exactly one unit at odd addresses
    ("u8", (11, 255), (300, 1), (257, 1)),
    ("f16", (513, 127), (131, 1), (127, 1)),                                 # 254-byte rows, the flat form
    ("bf16", (64, 8, 127), (10 * 127, 127, 1), (127, 64 * 127, 1)),          # heads of odd width -> [head, token, dim]
    ("f16", (9, 4095), (4099, 1), (4095, 1)),                                # rows of more than a wavefront of units: the row form
    ("f16", (3, 20001), (20003, 1), (20001, 1)),
    ("f16", (300, 120), (128, 1), (120, 1)),                                 # on 16-byte but not on 128-byte boundaries
    ("f32", (70, 33), (35, 1), (33, 1)),
]


@pytest.mark.parametrize("case", range(len(CASES)))
def test_against_oracle(ctx, case):
    dt, shape, ss, sd = CASES[case]
    ss, sd = ss or contig(shape), sd or contig(shape)
    item = np.dtype(NP_OF[dt]).itemsize
    rng = np.random.default_rng(900 + case)
    span = lambda st: 1 + sum((n - 1) * s for n, s in zip(shape, st))  # noqa: E731
    src_buf = rng.integers(0, 256, span(ss) * item, dtype=np.uint8).view(NP_OF[dt])
    dst_buf = rng.integers(0, 256, span(sd) * item, dtype=np.uint8).view(NP_OF[dt])
    want_buf = dst_buf.copy()
    src = np.lib.stride_tricks.as_strided(src_buf, shape, [s * item for s in ss])
    dst = np.lib.stride_tricks.as_strided(want_buf, shape, [s * item for s in sd])
    oracle.rearrange(dst, src)
    got = run_case(ctx, dt, shape, ss, sd, src_buf, dst_buf)
    assert np.array_equal(got, want_buf.view(np.uint8)), (dt, shape, ss, sd)


def test_misaligned_base_pointers(ctx):
    """Views that start 2 bytes into their buffers: 16-byte units at that boundary; what lies in front of and between the rows stays."""
    import torch

    rng = np.random.default_rng(950)
    src_np = rng.integers(0, 65536, 4096 * 3 + 1, dtype=np.uint16)
    src_all = torch.from_numpy(src_np.view(np.int16)).cuda().view(torch.float16)
    dst_all = torch.zeros(64 * 200 + 1, dtype=torch.float16, device="cuda")
    src = torch.as_strided(src_all[1:], (64, 128), (192, 1))
    dst = torch.as_strided(dst_all[1:], (64, 128), (200, 1))
    ctx.rearrange(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst.view(torch.int16), src.view(torch.int16))
    assert dst_all[0] == 0 and not dst_all[1:].view(64, 200)[:, 128:].any()


def test_status_codes_match_reference(ctx):
    import ctypes

    from operators_amd import infiniopRearrangeDescriptor_t, make_descriptor
    from oracle.ref import LAYOUT

    lib = ctx.lib
    for case in golden_json()["status"]:
        if case["op"] != "rearrange":
            continue
        descs = [make_descriptor(lib, t[1], t[2], LAYOUT[t[0]]) for t in case["tensors"]]
        d = infiniopRearrangeDescriptor_t()
        st = lib.infiniopCreateRearrangeDescriptor(ctx.handle, ctypes.byref(d), *descs)
        assert st == case["status"], (case, st)
        if st == 0:
            assert lib.infiniopDestroyRearrangeDescriptor(d) == 0
        for x in descs:
            lib.infiniopDestroyTensorDescriptor(x)


@pytest.mark.parametrize("shape,strides", [((0, 4), None), ((3, 0, 8), (64, 8, 1)), ((4, 0), None), ((2, 3, 0, 8), (96, 32, 8, 1))])
def test_zero_extent_copies_nothing(ctx, shape, strides):
    """An extent of zero anywhere: the descriptor is accepted (as by the
    reference, whose loops then run zero times) and the call leaves the
    destination as it was."""
    import ctypes

    import torch

    from operators_amd import F16, infiniopRearrangeDescriptor_t, make_descriptor

    lib = ctx.lib
    dst_d, src_d = make_descriptor(lib, shape, None, F16), make_descriptor(lib, shape, strides, F16)
    d = infiniopRearrangeDescriptor_t()
    assert lib.infiniopCreateRearrangeDescriptor(ctx.handle, ctypes.byref(d), dst_d, src_d) == 0
    dst = torch.full((64,), 7.0, dtype=torch.float16, device="cuda")
    src = torch.full((64,), 3.0, dtype=torch.float16, device="cuda")
    assert lib.infiniopRearrange(d, dst.data_ptr(), src.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert bool((dst == 7.0).all())
    assert lib.infiniopDestroyRearrangeDescriptor(d) == 0
    lib.infiniopDestroyTensorDescriptor(dst_d)
    lib.infiniopDestroyTensorDescriptor(src_d)
