"""Builds libdifflogic_hip.so (the C-ABI kernel library) in-tree with hipcc for gfx950.

    python difflogic_amd/build.py
"""
import os
import shutil
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
INCLUDE = os.path.join(os.path.dirname(HERE), "include")
LIB_NAME = "libdifflogic_hip.so"
LIB_PATH = os.path.join(HERE, LIB_NAME)
SOURCES = ("packed.hip", "lds_net.hip", "train.hip", "schedule.cpp")
# streaming / gather microbenchmarks for `bench.py --ceilings`: a library of their own, never
# loaded by the package
CEILINGS_LIB_PATH = os.path.join(HERE, "libdl_ceilings.so")
CEILINGS_SOURCES = ("ceilings.hip",)

HIPCC_FLAGS = (
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared", "-fvisibility=default",
    # no automatic mul+add fusion: kernels that state the same arithmetic give the same bits
    # (the chained and unchained training kernels are checked for equality); fma is written out
    "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
)


def hipcc_path():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found (set HIPCC or install ROCm under /opt/rocm)")


def build_library(verbose=False):
    """Compiles every kernel source into one shared library next to this file, and the
    measurement helpers into a second one."""
    _compile(SOURCES, LIB_PATH, verbose)
    _compile(CEILINGS_SOURCES, CEILINGS_LIB_PATH, verbose)
    return LIB_PATH


def _compile(sources, out_path, verbose):
    cmd = [hipcc_path(), *HIPCC_FLAGS, f"-I{INCLUDE}", f"-I{CSRC}",
           *[os.path.join(CSRC, s) for s in sources], "-o", out_path + ".tmp"]
    if verbose:
        print(" ".join(cmd))
    proc = subprocess.run(cmd, capture_output=True, text=True)
    # hipcc's host pass warns that it does not know the packed-fp32 feature; that is expected.
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err, file=sys.stderr)
    os.replace(out_path + ".tmp", out_path)
    return out_path


if __name__ == "__main__":
    print(build_library(verbose=True))
