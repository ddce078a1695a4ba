"""Builds the gfx950 shared libraries of this package in-tree with hipcc.

    python -m pimaicompiler_amd.build        # libpimhip.so (the C ABI of include/pimhip.h)

hipcc cross-compiles for gfx950 without a GPU, so this runs on any host that has ROCm installed.
"""
import os
import shutil
import subprocess
import sys

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(PKG_DIR, "csrc")
LIB_PATH = os.path.join(PKG_DIR, "libpimhip.so")

# -packed-fp32-ops is switched off for every device compilation of this package.
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-result", "-Wno-unused-value",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build libpimhip.so")
    return exe


def build_pimhip(verbose=True):
    src = [os.path.join(CSRC, "pimhip_api.hip")]
    cmd = [hipcc()] + HIP_FLAGS + src + ["-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out)
    if verbose and out.strip():
        print(out)
    return LIB_PATH


def build_all(verbose=True):
    return [build_pimhip(verbose)]


if __name__ == "__main__":
    build_all()
    sys.exit(0)
