"""Builds libwoq_hip.so (gfx950) from the .hip sources in this directory.

Usage: python build.py [--jobs N] [--incremental]
--incremental recompiles only the sources that are newer than their object file (or older than a
header); the default compiles everything.
The library is written to ../lib/libwoq_hip.so, in-tree, so that a copy of the
repository carries it to a machine that has no compiler cache.
"""
import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_DIR = os.path.join(os.path.dirname(HERE), "lib")
OBJ_DIR = os.path.join(HERE, "build")
SOURCES = ["woq_api.hip", "woq_pack.hip", "woq_small_m.hip", "woq_decode.hip", "woq_decode_dq.hip", "woq_gemm.hip", "woq_gemm_w4.hip", "woq_gemm_w4s.hip", "woq_gemm_dense.hip", "woq_int8.hip", "woq_moe.hip", "woq_gemm_w4i8.hip", "woq_act_quant.hip", "woq_fp32.hip"]
# measurement probes of bench.py: a library of their own, so that the product library carries none
PROBE_SOURCE = "bench_probes.hip"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def lib_path():
    return os.path.join(LIB_DIR, "libwoq_hip.so")


def torch_lib_path():
    return os.path.join(LIB_DIR, "libwoq_torch.so")


def probe_lib_path():
    return os.path.join(LIB_DIR, "libwoq_bench_probes.so")


def build_probes(verbose=True, incremental=False):
    """hipcc on bench_probes.hip -> ../lib/libwoq_bench_probes.so (loaded by bench.py only)."""
    src, out = os.path.join(HERE, PROBE_SOURCE), probe_lib_path()
    if incremental and os.path.exists(out) and os.path.getmtime(out) > max(
            os.path.getmtime(src), os.path.getmtime(os.path.join(HERE, "woq_common.h"))):
        return out
    res = subprocess.run([HIPCC, *FLAGS, "-shared", src, "-o", out], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("hipcc failed for bench_probes.hip:\n" + res.stderr[-4000:])
    if verbose:
        print("built", out)
    return out


def build_torch_binding(verbose=True, incremental=False):
    """g++ on torch_binding.cpp (host code only: the operator / custom-class registrations over the C ABI)
    -> ../lib/libwoq_torch.so, linked against libwoq_hip.so beside it and the libraries of the installed
    PyTorch (ROCm build).  No hipify step: the source is written against the HIP headers of PyTorch."""
    import torch
    from torch.utils import cpp_extension

    src = os.path.join(HERE, "torch_binding.cpp")
    out = torch_lib_path()
    if incremental and os.path.exists(out) and os.path.getmtime(out) > max(
            os.path.getmtime(src), os.path.getmtime(os.path.join(os.path.dirname(os.path.dirname(HERE)), "include", "woq_hip.h"))):
        return out
    tlib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1",
           f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}", "-Wno-deprecated-declarations"]
    for inc in cpp_extension.include_paths() + ["/opt/rocm/include"]:
        cmd += ["-isystem", inc]
    cmd += [src, "-o", out, f"-L{LIB_DIR}", "-lwoq_hip", f"-L{tlib}", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch",
            "-lamdhip64", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{tlib}"]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("g++ failed for torch_binding.cpp:\n" + res.stderr[-6000:])
    if verbose:
        print("built", out)
    return out


def _stale(src, obj):
    if not os.path.exists(obj):
        return True
    t = os.path.getmtime(obj)
    deps = [os.path.join(HERE, src)] + [os.path.join(HERE, h) for h in os.listdir(HERE) if h.endswith(".h")]
    deps.append(os.path.join(os.path.dirname(os.path.dirname(HERE)), "include", "woq_hip.h"))
    return any(os.path.getmtime(d) > t for d in deps)


def _compile(src, incremental=False):
    obj = os.path.join(OBJ_DIR, src.replace(".hip", ".o"))
    if incremental and not _stale(src, obj):
        return obj
    cmd = [HIPCC, *FLAGS, "-c", os.path.join(HERE, src), "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in res.stderr.splitlines() if "packed-fp32-ops" not in l)
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err.strip():
        sys.stderr.write(err + "\n")
    return obj


def build(jobs=4, verbose=True, incremental=False):
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda src: _compile(src, incremental), SOURCES))
    cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib_path(), *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("link failed:\n" + res.stderr)
    if verbose:
        print("built", lib_path())
    build_torch_binding(verbose, incremental)
    build_probes(verbose, incremental)
    return lib_path()


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=4)
    ap.add_argument("--incremental", action="store_true")
    args = ap.parse_args()
    build(args.jobs, incremental=args.incremental)
