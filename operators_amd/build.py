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
import os
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
HIP_FLAGS = [
    f"--offload-arch={ARCH}", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


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
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    return src, obj, res.returncode, err


def build(verbose=True, jobs=None):
    os.makedirs(OBJ_DIR, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, os.cpu_count() or 1)
    objs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=jobs) as pool:
        for src, obj, rc, err in pool.map(_compile, srcs):
            if verbose:
                print(f"[hipcc {ARCH}] {os.path.relpath(src, REPO_DIR)}", flush=True)
            if err.strip():
                print(err, file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"compilation failed: {src}")
            objs.append(obj)
    cmd = [hipcc(), "-shared", "-fPIC", f"--offload-arch={ARCH}", "-o", LIB_PATH] + objs
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        print(res.stderr, file=sys.stderr)
        raise RuntimeError("link failed")
    if verbose:
        print(f"[link] {os.path.relpath(LIB_PATH, REPO_DIR)}", flush=True)
    return LIB_PATH


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
    if args.install:
        install(os.environ.get("INFINI_ROOT") or os.path.join(os.path.expanduser("~"), ".infini"))
