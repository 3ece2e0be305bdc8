"""What the compiler reports for every kernel of the library (registers,
scratch memory, spills), as recorded by `python -m operators_amd.build` in
operators_amd/lib/kernel_resources.json.  A kernel that spills vector registers
writes them to memory and reads them back - traffic that no byte count of the
operator explains - so none may: the build itself refuses such a kernel, and
this test checks the record of the library that is there."""
import json
import os

from operators_amd import build as lib_build


def _record():
    if not os.path.isfile(lib_build.RESOURCES_PATH):
        lib_build.build(verbose=False)  # no library yet: build it (and with it the record)
    with open(lib_build.RESOURCES_PATH) as f:
        return json.load(f)


def test_no_kernel_spills_vector_registers():
    record = _record()
    assert len(record) > 100  # every .hip translation unit reported
    spilling = {name: fig["vgpr_spill"] for name, fig in record.items() if fig.get("vgpr_spill", 0) != 0}
    assert spilling == {}


def test_every_operator_reports_its_kernels():
    names = " ".join(_record())
    for kernel in ("add_", "swiglu_rows", "rope_once", "rms_norm_rows", "rms_norm_once", "rms_norm_wide", "causal_softmax_rows",
                   "causal_softmax_held", "rearrange", "random_sample"):
        assert kernel in names, kernel


def test_remark_parser_reads_the_compiler_format():
    text = """
a.hip:5:1: remark: Function Name: _Z3foov [-Rpass-analysis=kernel-resource-usage]
    5 | void foo() {
      | ^
a.hip:5:1: remark:     TotalSGPRs: 20 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     VGPRs: 128 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     AGPRs: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     ScratchSize [bytes/lane]: 48 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     Occupancy [waves/SIMD]: 4 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     SGPRs Spill: 0 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     VGPRs Spill: 3 [-Rpass-analysis=kernel-resource-usage]
a.hip:5:1: remark:     LDS Size [bytes/block]: 128 [-Rpass-analysis=kernel-resource-usage]
"""
    got = lib_build.kernel_resources(text)
    assert got == {"_Z3foov": {"sgprs": 20, "vgprs": 128, "agprs": 0, "scratch_bytes": 48, "occupancy": 4, "sgpr_spill": 0,
                               "vgpr_spill": 3, "lds_bytes": 128}}
