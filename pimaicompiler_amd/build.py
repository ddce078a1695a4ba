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
    # the first 16 dwords of a kernel's plain arguments arrive in scalar registers instead of through a load at its start
    # (about 0.1 us off every launch whose first instructions need them; kernels that take a struct are unaffected)
    "-mllvm", "-amdgpu-kernarg-preload-count=16",
    "-Wno-unused-result", "-Wno-unused-value",
]


def hipcc():
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build libpimhip.so")
    return exe


# One translation unit per kernel family (each kernel header is compiled once); api_common.h is what they share.
SOURCES = ["api_core.hip", "api_gemv.hip", "api_xproj.hip", "api_lstm.hip", "api_decoder.hip", "api_moe.hip", "api_rnnt.hip", "api_blas.hip"]
OBJ_DIR = os.path.join(PKG_DIR, "build")


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l)
    return res.returncode, out


def build_pimhip(verbose=True, jobs=None):
    """Compiles the translation units side by side (hipcc -c), then links libpimhip.so."""
    from concurrent.futures import ThreadPoolExecutor

    os.makedirs(OBJ_DIR, exist_ok=True)
    compile_flags = [f for f in HIP_FLAGS if f != "-shared"]
    objs = [os.path.join(OBJ_DIR, os.path.splitext(f)[0] + ".o") for f in SOURCES]
    cmds = [[hipcc()] + compile_flags + ["-c", os.path.join(CSRC, f), "-o", o] for f, o in zip(SOURCES, objs)]
    jobs = jobs or min(len(cmds), max(1, (os.cpu_count() or 2) - 1), 8)
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda c: _run(c, verbose), cmds))
    for (rc, out), cmd in zip(results, cmds):
        if rc != 0:
            raise RuntimeError("hipcc failed: " + " ".join(cmd) + "\n" + out)
        if verbose and out.strip():
            print(out)
    rc, out = _run([hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC"] + objs + ["-o", LIB_PATH], verbose)
    if rc != 0:
        raise RuntimeError("linking libpimhip.so failed:\n" + out)
    return LIB_PATH


ATEN_LIB_PATH = os.path.join(PKG_DIR, "_aten_ops_pimhip.so")
ROCM_HOME = os.environ.get("ROCM_HOME") or os.environ.get("ROCM_PATH") or "/opt/rocm"


def build_aten_ops(verbose=True):
    """The C++ operator bodies with the reference's signatures (cpp/aten_ops_pimhip.cpp) plus their pybind module,
    compiled with g++ against this image's LibTorch and linked to libpimhip.so next to it."""
    import sysconfig

    from torch.utils import cpp_extension as ce
    import torch

    cpp = os.path.join(PKG_DIR, "cpp")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-w",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-DTORCH_EXTENSION_NAME=_aten_ops_pimhip",
           "-DTORCH_API_INCLUDE_EXTENSION_H"]
    # c10/hip/HIPStream.h (torch's current stream) pulls in the HIP runtime API headers; host compiler only.
    cmd += ["-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", f"-I{ROCM_HOME}/include"]
    cmd += [f"-I{p}" for p in ce.include_paths()] + [f"-I{sysconfig.get_paths()['include']}"]
    cmd += [os.path.join(cpp, "aten_ops_pimhip.cpp"), os.path.join(cpp, "aten_ops_pybind.cpp"), "-o", ATEN_LIB_PATH]
    cmd += [f"-L{p}" for p in ce.library_paths()] + ["-lc10", "-lc10_hip", "-ltorch", "-ltorch_cpu", "-ltorch_python"]
    cmd += [f"-L{PKG_DIR}", "-lpimhip", "-Wl,-rpath,$ORIGIN"] + [f"-Wl,-rpath,{p}" for p in ce.library_paths()]
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed:\n" + res.stdout)
    return ATEN_LIB_PATH


def build_all(verbose=True):
    return [build_pimhip(verbose), build_aten_ops(verbose)]


if __name__ == "__main__":
    build_all()
    sys.exit(0)
