"""Build libinfiniop.so (amd-gpu device, gfx950 only) with hipcc.

    python -m operators_amd.build            # compile everything, link in-tree
    python -m operators_amd.build --install  # also copy lib + headers to $INFINI_ROOT

Stands in for the reference's xmake targets (xmake.lua:215-238: one shared
library `infiniop` installed under $INFINI_ROOT/{lib,include}); xmake itself is
not required.  The library is written for CDNA4 only, so there is exactly one
offload architecture and no host-compiler fallback.
"""
import argparse
import concurrent.futures
import json
import os
import re
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
REPO_DIR = os.path.dirname(PKG_DIR)
CSRC = os.path.join(PKG_DIR, "csrc")
INCLUDE = os.path.join(REPO_DIR, "include")
OBJ_DIR = os.path.join(PKG_DIR, "build")
LIB_DIR = os.path.join(PKG_DIR, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libinfiniop.so")

ARCH = "gfx950"

# -ffp-contract=off: RoPE's products must round before the add that follows
#   them, as in the reference's CPU build (baseline x86-64 has no FMA).
# -packed-fp32-ops off: no v_pk_{add,mul,fma}_f32 from auto-vectorisation.
COMMON_FLAGS = [
    "-std=c++17", "-O3", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off",
    "-I", INCLUDE, "-Wall", "-Wno-unused-const-variable",
]
# -Rpass-analysis=kernel-resource-usage: the back end reports every kernel's
#   registers, scratch and spills; build() records them and refuses a kernel
#   that spills vector registers (a spill is HBM traffic nobody asked for).
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Rpass-analysis=kernel-resource-usage",
]
RESOURCES_PATH = os.path.join(LIB_DIR, "kernel_resources.json")
_REMARK = re.compile(r"remark:\s+(.*?)\s+\[-Rpass-analysis=kernel-resource-usage\]")
_FIELDS = {
    "VGPRs": "vgprs", "AGPRs": "agprs", "TotalSGPRs": "sgprs", "VGPRs Spill": "vgpr_spill", "SGPRs Spill": "sgpr_spill",
    "ScratchSize [bytes/lane]": "scratch_bytes", "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds_bytes",
}


def kernel_resources(stderr):
    """The per-kernel figures out of one compilation's remarks: {mangled name: {...}}."""
    out, cur = {}, None
    for line in stderr.splitlines():
        m = _REMARK.search(line)
        if not m:
            continue
        key, _, val = m.group(1).rpartition(":")
        key, val = key.strip(), val.strip()
        if key == "Function Name":
            cur = out.setdefault(val, {})
        elif cur is not None and key in _FIELDS:
            cur[_FIELDS[key]] = int(val)
    return out


def demangle(names):
    res = subprocess.run(["c++filt"], input="\n".join(names), capture_output=True, text=True)
    got = res.stdout.splitlines() if res.returncode == 0 else []
    return got if len(got) == len(names) else list(names)


def hipcc():
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cand = os.path.join(rocm, "bin", "hipcc")
    return cand if os.path.exists(cand) else "hipcc"


def sources():
    out = []
    for root, _dirs, files in os.walk(CSRC):
        for f in sorted(files):
            if f.endswith((".cc", ".hip")):
                out.append(os.path.join(root, f))
    return sorted(out)


def _compile(src):
    rel = os.path.relpath(src, CSRC)
    obj = os.path.join(OBJ_DIR, rel.replace(os.sep, "__") + ".o")
    cmd = [hipcc()] + COMMON_FLAGS
    if src.endswith(".hip"):
        cmd += HIP_FLAGS
    else:
        # host-only translation units still go through hipcc so that they see
        # the HIP runtime headers; no device code is generated for them
        cmd += ["-x", "c++", "-D__HIP_PLATFORM_AMD__", "-I", os.path.join(os.environ.get("ROCM_PATH", "/opt/rocm"), "include")]
    cmd += ["-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    # the host pass of hipcc does not know the packed-fp32 feature name and says so; drop that line
    resources = kernel_resources(res.stderr) if src.endswith(".hip") else {}
    keep, held, skip = [], [], 0
    for l in res.stderr.splitlines():
        # a remark is three lines (the message, the source line it points at and a caret), with the
        # chain of includes that leads to its file in front
        if "-Rpass-analysis=kernel-resource-usage" in l:
            held, skip = [], 2
        elif skip and re.match(r"\s*(\d+\s*)?\|", l):
            skip -= 1
        elif l.startswith("In file included from"):
            held.append(l)
        elif "packed-fp32-ops" not in l:
            skip = 0
            keep += held + [l]
            held = []
    return src, obj, res.returncode, "\n".join(keep), resources


def build(verbose=True, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs, resources = [], {}
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, obj, rc, err, res_of in pool.map(_compile, srcs):
            if verbose:
                print(f"[hipcc {ARCH}] {os.path.relpath(src, REPO_DIR)}", flush=True)
            if err.strip():
                print(err, file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"compilation failed: {src}")
            objs.append(obj)
            for name, fig in res_of.items():
                resources[name] = dict(fig, source=os.path.relpath(src, REPO_DIR))
    names = sorted(resources)
    record = {pretty: dict(resources[name], mangled=name) for name, pretty in zip(names, demangle(names))}
    with open(RESOURCES_PATH, "w") as f:
        json.dump(record, f, indent=1, sort_keys=True)
    spilling = {k: v["vgpr_spill"] for k, v in record.items() if v.get("vgpr_spill", 0) != 0}
    if spilling:
        for k, v in sorted(spilling.items()):
            print(f"[spill] {v} vector registers: {k}", file=sys.stderr)
        raise RuntimeError(f"{len(spilling)} kernels spill vector registers to scratch memory (see {RESOURCES_PATH})")
    if verbose:
        print(f"[resources] {len(record)} kernels, none spills; {os.path.relpath(RESOURCES_PATH, REPO_DIR)}", flush=True)
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        print(res.stderr, file=sys.stderr)
        raise RuntimeError("link failed")
    if verbose:
        print(f"[link] {os.path.relpath(LIB_PATH, REPO_DIR)}", flush=True)
    return LIB_PATH


def build_c_client(verbose=True):
    """The C11 caller under tests/c_client, linked against the library and the HIP
    runtime with the plain C compiler: tests/c_client/client (run on the GPU by
    tests/test_gpu_c_client.py).  It finds both libraries through its run path."""
    src = os.path.join(REPO_DIR, "tests", "c_client", "client.c")
    out = os.path.join(REPO_DIR, "tests", "c_client", "client")
    rocm = os.environ.get("ROCM_PATH", "/opt/rocm")
    cmd = ["gcc", "-std=c11", "-O2", "-Wall", "-Wextra", "-Werror", "-DCLIENT_WITH_HIP_RUNTIME", "-D__HIP_PLATFORM_AMD__",
           "-I", INCLUDE, "-isystem", os.path.join(rocm, "include"), src, "-o", out,
           "-L", LIB_DIR, "-linfiniop", "-L", os.path.join(rocm, "lib"), "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../operators_amd/lib", "-Wl,-rpath," + os.path.join(rocm, "lib")]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        print(res.stderr, file=sys.stderr)
        raise RuntimeError("the C client does not build")
    if verbose:
        print(f"[gcc] {os.path.relpath(out, REPO_DIR)}", flush=True)
    return out


def install(root):
    """Copy the library and headers where the reference's loader looks
    ($INFINI_ROOT/lib/libinfiniop.so, operatorspy/liboperators.py:11,55)."""
    os.makedirs(os.path.join(root, "lib"), exist_ok=True)
    shutil.copy2(LIB_PATH, os.path.join(root, "lib", "libinfiniop.so"))
    shutil.copytree(INCLUDE, os.path.join(root, "include"), dirs_exist_ok=True)


if __name__ == "__main__":
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--install", action="store_true", help="copy to $INFINI_ROOT (default ~/.infini)")
    ap.add_argument("-j", "--jobs", type=int, default=None)
    args = ap.parse_args()
    build(jobs=args.jobs)
    build_c_client()
    if args.install:
        install(os.environ.get("INFINI_ROOT") or os.path.join(os.path.expanduser("~"), ".infini"))
