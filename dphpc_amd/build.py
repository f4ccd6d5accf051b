"""Compile the HIP library for gfx950 with hipcc (cross-compiles without a GPU)."""
import os
import shutil
import subprocess

PKG = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG, "csrc")
LIB_DIR = os.path.join(PKG, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libsddmm_amd.so")

HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",          # FMAs are written explicitly; the exact kernel needs mul and add apart
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc():
    for cand in (os.environ.get("HIPCC"), shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and os.path.exists(cand):
            return cand
    raise RuntimeError("hipcc not found")


def sources():
    return [os.path.join(CSRC, "sddmm_amd.hip")]


def build_library(verbose=False, extra_flags=(), out=None):
    """(Re)build dphpc_amd/lib/libsddmm_amd.so; returns its path."""
    os.makedirs(LIB_DIR, exist_ok=True)
    cmd = [hipcc()] + HIPCC_FLAGS + list(extra_flags) + ["-o", out or LIB_PATH] + sources()
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.check_call(cmd)
    return LIB_PATH


if __name__ == "__main__":
    print(build_library(verbose=True))
