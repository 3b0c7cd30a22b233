"""Static check of the compiled split-K kernels (no GPU).  Workgroups that share the K range of a tile hand their fp32
partial tiles through memory with relaxed device-scope atomics and one counter, without fences: the scheme is correct
only for the instructions the compiler emits today (the argument is written out in the kernels' sources).  This test
compiles the three sources to device assembly and asserts, in every kernel that moves the counter, exactly that form:

* the partial-tile stores are ``global_store_dword ... sc1`` (written through to the device-coherent level);
* between the last of them and the counter's ``global_atomic_add ... sc0`` stand an ``s_waitcnt vmcnt(0)`` (the
  stores are acknowledged) and an ``s_barrier`` (of every wave), in that order;
* the workgroup that draws the last count passes a barrier and then reads the other tiles with
  ``global_load_dword ... sc1`` (not from its own stale cache lines);
* no cache-wide write-back or invalidate was inserted (what fences would cost).

A compiler that drops a cache bit or moves the wait fails here, before a run can go wrong only now and then."""
import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "intel-extension-for-pytorch_amd", "csrc")
sys.path.insert(0, CSRC)
SOURCES = ["woq_decode_dq.hip", "woq_gemm_w4.hip", "woq_gemm_w4i8.hip"]


def _functions(asm):
    lines = asm.split("\n")
    for s in [i for i, l in enumerate(lines) if re.match(r"^_ZN3woq\w+:", l)]:
        e = next((i for i in range(s + 1, len(lines)) if lines[i].startswith(".Lfunc_end")), None)
        if e is None:  # a data symbol behind the last function
            continue
        body = [l.split(";")[0].strip() for l in lines[s:e]]
        yield lines[s].split(":")[0], [l for l in body if l]


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_partial_tiles_and_counter_of_split_k_compile_to_the_coherent_instruction_forms(tmp_path):
    import build as woq_build

    def compile_one(src):
        out = tmp_path / (src + ".s")
        cmd = [woq_build.HIPCC, *woq_build.FLAGS, "-I", os.path.join(ROOT, "include"), "--cuda-device-only", "-S",
               os.path.join(CSRC, src), "-o", str(out)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        assert res.returncode == 0, res.stderr[-2000:]
        return out.read_text()

    with ThreadPoolExecutor(max_workers=3) as pool:
        texts = list(pool.map(compile_one, SOURCES))
    for src, asm in zip(SOURCES, texts):
        checked = 0
        for name, body in _functions(asm):
            adds = [i for i, l in enumerate(body) if l.startswith("global_atomic_add")]
            if not adds:
                continue
            checked += 1
            assert not any(l.startswith(("buffer_wbl2", "buffer_inv")) for l in body), name
            for i in adds:
                assert re.search(r"\bsc0\b", body[i]), (name, body[i])
            first = adds[0]
            stores = [i for i in range(first) if body[i].startswith("global_store_dword") and re.search(r"\bsc1\b", body[i])]
            assert stores, name
            between = body[stores[-1] + 1:first]
            waits = [i for i, l in enumerate(between) if l.startswith("s_waitcnt") and "vmcnt(0)" in l]
            assert waits, name
            assert any(l.startswith("s_barrier") for l in between[waits[0]:]), name
            after = body[adds[-1] + 1:]
            loads = [i for i, l in enumerate(after) if l.startswith("global_load_dword") and re.search(r"\bsc1\b", l)]
            assert loads, name
            assert any(l.startswith("s_barrier") for l in after[:loads[0]]), name
            # the counter is set back to zero with the coherent store form as well
            assert any(l.startswith("global_store_dword") and re.search(r"\bsc1\b", l) for l in after[loads[0]:]), name
        assert checked >= 2, (src, checked)
