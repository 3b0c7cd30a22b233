"""Builds the C port of the oracle (oracle/woq_ref.c) into oracle/libwoq_oracle.so with gcc.

The reference's own sources are not built here: its WOQ kernels sit behind `#ifdef USE_LIBXSMM`
and need libxsmm / ideep / sleef, whose submodule directories are empty in the mount, a
generated version header, and gcc >= 12.3 (this image has 11.4), so oracle/_ref/ stays empty.
"""
import os
import subprocess

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libwoq_oracle.so")


def build(verbose=True):
    cmd = ["gcc", "-O3", "-march=x86-64-v3", "-fopenmp", "-fPIC", "-shared", "-fno-fast-math",
           os.path.join(HERE, "woq_ref.c"), "-o", LIB, "-lm"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("gcc failed:\n" + res.stderr)
    if verbose:
        print("built", LIB)
    return LIB


if __name__ == "__main__":
    build()
