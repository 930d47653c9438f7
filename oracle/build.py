"""Build the CPU oracle (test infrastructure) with gcc.

  libbcpnn_oracle.so       strict IEEE restatement (the checker)
  libbcpnn_oracle_fast.so  the reference's flag set (CMakeLists.txt:18-24,39-40), timed as the CPU baseline

-march=x86-64-v3 stands in for the reference's -march=native so that a library built on one host
still runs on another; build_native() builds the reference's own -march=native variant for the host it
runs on (the bench's CPU baseline calls it on the machine it times, and falls back to the portable library
where there is no gcc).

The reference's own kernels_openmp_internal.cc is NOT built: it includes <cblas.h>, which this image
does not provide, and writing a substitute header is not a reference build.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
SRC = os.path.join(HERE, "bcpnn_oracle.c")

VARIANTS = {
    "libbcpnn_oracle.so": ["-O2", "-ffp-contract=off", "-fopenmp"],
    "libbcpnn_oracle_fast.so": ["-O3", "-march=x86-64-v3", "-ffast-math", "-fopenmp"],
}


def build(verbose=False):
    for name, flags in VARIANTS.items():
        cmd = ["gcc", "-std=c11", "-fPIC", "-shared", "-Wall", "-Wextra", *flags, "-o",
               os.path.join(HERE, name), SRC, "-lm"]
        if verbose:
            print(" ".join(cmd), flush=True)
        subprocess.run(cmd, check=True, cwd=HERE)


def build_native(out_dir):
    """libbcpnn_oracle_native.so in out_dir: the reference's flag set with -march=native, for this host only.
    Returns its path, or None when gcc is missing or fails."""
    path = os.path.join(out_dir, "libbcpnn_oracle_native.so")
    cmd = ["gcc", "-std=c11", "-fPIC", "-shared", "-O3", "-march=native", "-ffast-math", "-fopenmp", "-o", path, SRC,
           "-lm"]
    try:
        subprocess.run(cmd, check=True, cwd=HERE, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
    except (OSError, subprocess.CalledProcessError):
        return None
    return path


if __name__ == "__main__":
    build(verbose=True)
    sys.exit(0)
