"""Pins the oracle's scalar conversions (oracle.c) independently of the oracle:
golden vectors from the compiled reference, numpy's exact widening, an ideal
round-toward-zero narrowing assembled from numpy primitives, and hand probes
whose answers follow from the reference's text
(src/devices/cpu/common_cpu.cc:3-64)."""
import numpy as np
import pytest

import oracle
from helpers import golden


def test_f16_to_f32_every_code_matches_reference_golden():
    g = golden("conversions")
    got = oracle.f16_to_f32(np.arange(65536, dtype=np.uint16)).view(np.uint32)
    want = g["all_f16_as_f32_bits"]
    # The fixture was read from the reference's scalar function through a C
    # `float` return value widened to a Python float, which sets the quiet bit
    # of signalling NaNs; the function itself leaves it clear (checked in the
    # next test).  Compare NaNs with that bit set on both sides.
    nan = (want & 0x7FFFFFFF) > 0x7F800000
    assert np.array_equal(got[~nan], want[~nan])
    assert np.array_equal(got[nan] | 0x00400000, want[nan] | 0x00400000)


def test_f16_to_f32_every_code_is_numpy_widening():
    codes = np.arange(65536, dtype=np.uint16)
    got = oracle.f16_to_f32(codes)
    want = codes.view(np.float16).astype(np.float32)
    nan = np.isnan(want)
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got.view(np.uint32)[~nan], want.view(np.uint32)[~nan])
    # NaN payloads are moved up by 13 bits and not quieted
    assert np.array_equal(got.view(np.uint32)[nan] & 0x7FFFFF, (codes[nan].astype(np.uint32) & 0x3FF) << 13)


def test_f32_to_f16_matches_reference_golden():
    g = golden("conversions")
    got = oracle.f32_to_f16(g["f32_bits"].view(np.float32))
    assert np.array_equal(got, g["f16_codes"])


def _ideal_rtz(values):
    """fp32 -> fp16 toward zero for |v| < 65536, from numpy's round-to-nearest
    conversion and nextafter: step back when rounding moved away from zero."""
    v = values.astype(np.float32)
    with np.errstate(over="ignore"):
        h = v.astype(np.float16)
    # values in (65504, 65536) round to inf under RNE but truncate to 65504
    h = np.where(np.isinf(h) & np.isfinite(v), np.copysign(np.float16(65504), v).astype(np.float16), h)
    away = np.abs(h.astype(np.float32)) > np.abs(v)
    h = np.where(away, np.nextafter(h, np.float16(0)), h)
    # nextafter towards +0 from the smallest negative subnormal yields -0 in IEEE; numpy gives -0 as well
    out = h.view(np.uint16).copy()
    # keep the sign of zero results
    zero = (out & 0x7FFF) == 0
    out[zero] = (v.view(np.uint32)[zero] >> 16).astype(np.uint16) & 0x8000
    return out


def test_f32_to_f16_is_round_toward_zero_below_65536():
    rng = np.random.default_rng(7)
    n = 600_000
    expo = rng.integers(127 - 30, 127 + 16, n, dtype=np.uint32)
    bits = (rng.integers(0, 2, n, dtype=np.uint32) << 31) | (expo << 23) | rng.integers(0, 1 << 23, n, dtype=np.uint32)
    vals = bits.view(np.float32)
    # plus both fp32 neighbours of every finite fp16 value
    finite = np.arange(65536, dtype=np.uint16)
    finite = finite[(finite & 0x7C00) != 0x7C00].view(np.float16).astype(np.float32)
    vals = np.concatenate([vals, finite, np.nextafter(finite, np.float32(np.inf)), np.nextafter(finite, np.float32(-np.inf))])
    vals = vals[np.abs(vals) < 65536]
    assert np.array_equal(oracle.f32_to_f16(vals), _ideal_rtz(vals))


@pytest.mark.parametrize("value,code", [
    (1.0 + 1.5 * 2.0 ** -10, 0x3C01),      # truncation, not rounding (RNE would give 0x3C02)
    (65504.0 + 65504.0, 0x7FFF),           # exponent 16 is unguarded: lands on a NaN pattern
    (65536.0, 0x7C00),                     # ... or on the infinity pattern
    (-65536.0, 0xFC00),
    (131072.0, 0x8000),                    # exponent 17: (17+15)<<10 = bit 15, exponent field 0
    (-131072.0, 0x8000),
    (2.0 ** 30, 0xB400),                   # exponent 30: (45 & 31) << 10 = 0x3400, plus bit 15
    (2.0 ** 31, 0x7C00),                   # exponent 31 and above: infinity
    (float("inf"), 0x7C00),
    (float("-inf"), 0xFC00),
    (2.0 ** -24, 0x0001),
    (2.0 ** -25, 0x0000),
    (-(2.0 ** -25), 0x8000),
    (2.0 ** -14 - 2.0 ** -25, 0x03FF),     # largest subnormal, by truncation
])
def test_f32_to_f16_probes(value, code):
    assert int(oracle.f32_to_f16(np.array([value], np.float32))[0]) == code


def test_f32_to_f16_nan_is_canonical_with_sign():
    bits = np.array([0x7FC00000, 0xFFC00000, 0x7F800001, 0xFF800001, 0x7FFFFFFF], np.uint32)
    got = oracle.f32_to_f16(bits.view(np.float32))
    assert got.tolist() == [0x7E00, 0xFE00, 0x7E00, 0xFE00, 0x7E00]


def test_round_trip_is_identity_on_all_non_nan_codes():
    codes = np.arange(65536, dtype=np.uint16)
    back = oracle.f32_to_f16(oracle.f16_to_f32(codes))
    nan = ((codes & 0x7C00) == 0x7C00) & ((codes & 0x3FF) != 0)
    assert np.array_equal(back[~nan], codes[~nan])
    assert np.array_equal(back[nan], (codes[nan] & 0x8000) | 0x7E00)


def test_bf16_conversions_are_torch_cpu():
    """bf16 is this project's extension; torch's CPU conversion is its pin."""
    import torch

    rng = np.random.default_rng(3)
    bits = rng.integers(0, 1 << 32, 400_000, dtype=np.uint64).astype(np.uint32)
    vals = bits.view(np.float32)
    want = torch.from_numpy(vals.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.f32_to_bf16(vals)
    nan = np.isnan(vals)
    assert np.array_equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7F80) == 0x7F80).all() and ((got[nan] & 0x7F) != 0).all()
    codes = np.arange(65536, dtype=np.uint16)
    wide = oracle.bf16_to_f32(codes)
    assert np.array_equal(wide.view(np.uint32), codes.astype(np.uint32) << 16)
