"""The drop-in boundary as a C client and a dynamic linker see it (no GPU):
  * a C11 translation unit that includes the reference's header paths and calls
    the hot path compiles against include/ as plain C;
  * every reference-style header path resolves on its own;
  * the shared library's dynamic symbol table holds exactly the entry points
    include/infiniop.h declares - nothing of the back end leaks out."""
import os
import re
import shutil
import subprocess

import pytest

from operators_amd.liboperators import EXPORTED_SYMBOLS, library_path

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
INCLUDE = os.path.join(ROOT, "include")

# reference include/infini_operators.h:1-19 and include/operators.h:4-7, minus the CNN-family operators
REFERENCE_PATHS = [
    "infini_operators.h", "operators.h", "export.h", "device.h", "status.h", "data_type.h", "tensor.h", "handle.h",
    "handle/handle_export.h", "tensor/tensor_descriptor.h",
    "ops/add/add.h", "ops/attention/attention.h", "ops/causal_softmax/causal_softmax.h", "ops/matmul/matmul.h",
    "ops/mlp/mlp.h", "ops/random_sample/random_sample.h", "ops/rearrange/rearrange.h", "ops/rms_norm/rms_norm.h",
    "ops/rotary_embedding/rotary_embedding.h", "ops/swiglu/swiglu.h",
]

needs_gcc = pytest.mark.skipif(shutil.which("gcc") is None, reason="no C compiler")


@needs_gcc
def test_c_client_compiles_as_c11():
    src = os.path.join(ROOT, "tests", "c_client", "client.c")
    res = subprocess.run(["gcc", "-std=c11", "-Wall", "-Wextra", "-Werror", "-pedantic", "-fsyntax-only", "-I", INCLUDE, src],
                         capture_output=True, text=True)
    assert res.returncode == 0, res.stderr


@needs_gcc
@pytest.mark.parametrize("path", REFERENCE_PATHS)
def test_reference_header_path_stands_alone(path, tmp_path):
    assert os.path.isfile(os.path.join(INCLUDE, path)), path
    tu = tmp_path / "one.c"
    tu.write_text(f'#include "{path}"\nstatic infiniopStatus_t ok(void) {{ return STATUS_SUCCESS; }}\n'
                  "int main(void) { Device d = DevAmdGpu; DataLayout t = F16; (void) t; return (int) ok() + (d != 4); }\n")
    for compiler, std in (("gcc", "-std=c11"), ("g++", "-std=c++17")):
        if shutil.which(compiler) is None:
            continue
        res = subprocess.run([compiler, std, "-x", "c" if compiler == "gcc" else "c++", "-fsyntax-only", "-I", INCLUDE, str(tu)],
                             capture_output=True, text=True)
        assert res.returncode == 0, (path, compiler, res.stderr)


@needs_gcc
def test_export_header_gives_the_reference_macros(tmp_path):
    """reference include/export.h:4-16: every operator header of the reference starts from `__export` and `__C`."""
    tu = tmp_path / "macros.c"
    tu.write_text('#include "ops/swiglu/swiglu.h"\n__C __export int mine(void);\nint mine(void) { return 0; }\n')
    for compiler, lang in (("gcc", "c"), ("g++", "c++")):
        res = subprocess.run([compiler, "-x", lang, "-Wall", "-Werror", "-fsyntax-only", "-I", INCLUDE, str(tu)], capture_output=True, text=True)
        assert res.returncode == 0, (compiler, res.stderr)


@needs_gcc
def test_c_client_links_against_the_library(tmp_path):
    """The program form of the C client (what tests/test_gpu_c_client.py runs on the GPU) links with the plain C compiler."""
    from operators_amd import build as lib_build

    assert os.path.isfile(library_path())
    out = lib_build.build_c_client(verbose=False)
    assert os.access(out, os.X_OK)
    needed = subprocess.run(["readelf", "-d", out], capture_output=True, text=True, check=True).stdout
    assert "libinfiniop.so" in needed and "libamdhip64.so" in needed


def test_dynamic_symbol_table_is_exactly_the_header():
    lib = library_path()
    assert os.path.isfile(lib), "build the library first: python -m operators_amd.build"
    out = subprocess.run(["nm", "-D", "--defined-only", lib], capture_output=True, text=True, check=True).stdout
    exported = sorted(line.split()[-1] for line in out.splitlines() if re.search(r"\s[TtDdBbWwVv]\s", line))
    ours = [s for s in exported if s.startswith("infiniop")]
    assert sorted(ours) == sorted(EXPORTED_SYMBOLS)
    # hidden visibility: no C++ symbol of the back end is visible, only what the toolchain itself adds
    leaked = [s for s in exported if not s.startswith("infiniop") and not s.startswith(("_init", "_fini", "__hip", "_edata", "_end", "__bss_start"))]
    assert leaked == [], leaked


def test_xmake_file_names_the_gfx950_option():
    text = open(os.path.join(ROOT, "xmake.lua")).read()
    assert 'option("amd-gpu")' in text and 'target("amd-gpu")' in text and 'target("infiniop")' in text
    assert "--offload-arch=gfx950" in text and "ENABLE_AMD_GPU" in text
    # one architecture only, and no CUDA toolchain anywhere
    assert re.findall(r"offload-arch=(\w+)", text) == ["gfx950"] * len(re.findall(r"offload-arch=", text))
    assert "cuda" not in text.lower().replace("no cuda headers", "")


def test_bench_reads_its_traffic_figure_from_the_committed_profile(tmp_path):
    """roofline.traffic is the swiglu row of profiles/c5_kernels_hbm_traffic_pmc.txt, byte for byte, and its absence is an error."""
    import sys

    sys.path.insert(0, ROOT)
    import bench

    text = open(bench.TRAFFIC_PROFILE).read()
    row = [l for l in text.splitlines() if bench.DOMINANT_KERNEL in l and l.startswith("C5 swiglu")]
    assert len(row) == 1
    assert bench.measured_traffic() == int(row[0].split()[-3])
    # every row of the table carries the algorithmic bytes of its own bench row: no ratio is 0, none is far from 1
    ratios = [float(l.split()[-1]) for l in text.splitlines() if re.search(r"\(\d+\)\s+[\d.]+\s+[\d.]+\s+\d+\s+\d+\s+[\d.]+$", l)]
    assert len(ratios) >= 15 and all(0.99 < r < 1.06 for r in ratios), ratios
    assert 0.99 < bench.measured_traffic() / 1409286144 < 1.01  # the counters see the algorithmic bytes, no more
    with pytest.raises(FileNotFoundError):
        bench.measured_traffic(str(tmp_path / "absent.txt"))
    empty = tmp_path / "empty.txt"
    empty.write_text("no such kernel here\n")
    with pytest.raises(LookupError):
        bench.measured_traffic(str(empty))
