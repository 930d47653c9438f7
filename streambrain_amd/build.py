"""Builds the native parts of the package for gfx950, in-tree:

  streambrain_amd/libsbhip.so                           HIP kernels + C ABI (include/sbhip.h), hipcc
  streambrain_amd/_bcpnn_backend_hip_internals*.so      pybind11 module over the C ABI, g++

Usage: python -m streambrain_amd.build [-v]
"""
import concurrent.futures
import os
import subprocess
import sys
import sysconfig

PKG = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(PKG)
CSRC = os.path.join(PKG, "csrc")
OBJ = os.path.join(PKG, "csrc", "build")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
HIP_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    # packed-FP32 VALU forms are kept out of every kernel of this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]
HIP_SOURCES = ["sb_kernels_f32.hip", "sb_kernels_f64.hip", "sbhip_api.hip"]
LIB = os.path.join(PKG, "libsbhip.so")
PYMOD_SRC = os.path.join(CSRC, "pybind_module.cpp")


def pymod_path():
    return os.path.join(PKG, "_bcpnn_backend_hip_internals" + sysconfig.get_config_var("EXT_SUFFIX"))


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        raise RuntimeError("build step failed:\n" + " ".join(cmd) + "\n" + res.stdout)
    # hipcc's host pass does not know the packed-fp32 feature flag and says so; nothing else is expected
    out = "\n".join(l for l in res.stdout.splitlines() if "packed-fp32-ops" not in l).strip()
    if out and verbose:
        print(out, flush=True)


def build_lib(verbose=False):
    os.makedirs(OBJ, exist_ok=True)
    objs = []
    jobs = []
    with concurrent.futures.ThreadPoolExecutor(max_workers=len(HIP_SOURCES)) as pool:
        for src in HIP_SOURCES:
            obj = os.path.join(OBJ, src.replace(".hip", ".o"))
            objs.append(obj)
            cmd = [HIPCC, *HIP_FLAGS, "-I", os.path.join(ROOT, "include"), "-c",
                   os.path.join(CSRC, src), "-o", obj]
            jobs.append(pool.submit(_run, cmd, verbose))
        for j in jobs:
            j.result()
    _run([HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB, *objs], verbose)
    return LIB


def build_pymod(verbose=False):
    import pybind11
    inc = sysconfig.get_paths()["include"]
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden",
           "-I", pybind11.get_include(), "-I", inc, "-I", os.path.join(ROOT, "include"),
           PYMOD_SRC, "-o", pymod_path(), "-L", PKG, "-lsbhip", "-Wl,-rpath,$ORIGIN"]
    _run(cmd, verbose)
    return pymod_path()


def build(verbose=False):
    build_lib(verbose)
    if os.path.exists(PYMOD_SRC):
        build_pymod(verbose)


if __name__ == "__main__":
    build(verbose="-v" in sys.argv[1:])
