"""The kernels divide by numbers the host knows (row lengths, head counts,
sequence lengths) with a multiplication and a shift; the constants are made by
`amd::fast_div` on the host and applied by `amd::fast_quotient` on the device
(operators_amd/csrc/devices/amd/kernel_amd.h).  Both are plain integer
arithmetic, so the pair is compiled for the host and checked there against `/`:
every divisor up to 70 000, the neighbours of every power of two, 200 000 random
divisors below 2^31, each with edge operands and random ones."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.skipif(shutil.which("hipcc") is None, reason="needs hipcc to compile the header")
def test_multiply_and_shift_division_equals_division(tmp_path):
    exe = tmp_path / "fast_div_check"
    subprocess.run(["hipcc", "--offload-arch=gfx950", "-O2", "-std=c++17", "-I", os.path.join(ROOT, "operators_amd", "csrc"),
                    os.path.join(ROOT, "tests", "c_client", "fast_div_check.hip"), "-o", str(exe)], check=True, capture_output=True, timeout=300)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True, timeout=300).stdout
    assert out.startswith("ok "), out
    assert int(out.split()[1]) > 19_000_000
