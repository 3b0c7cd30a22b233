"""Static check of the compiled dense-copy GEMM kernel (no GPU): its weight fragments are requested by inline
``global_load_dwordx4`` instructions whose completion the program tracks by hand (``s_waitcnt vmcnt(N)`` with
hand-counted N), which the compiler cannot verify.  The check walks the device assembly of every instance -- prologue,
the K loop twice, the rest -- with a queue of the loads in flight and asserts what the scheme rests on:

* no instruction reads or writes the destination registers of a fragment load that may still be in flight;
* the K loop never drains the queue (no ``vmcnt(0)`` inside it), so the ring of fragments stays in flight;
* the K loop holds no accumulator copies (``v_accvgpr_*``, ``v_mov`` of whole tiles).

A compiler that reorders the loads against their waits, or reuses a fragment register early, fails here before any
run does."""
import os
import re
import shutil
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "intel-extension-for-pytorch_amd", "csrc")
sys.path.insert(0, CSRC)


def _registers(text):
    out = set()
    for m in re.finditer(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b", text):
        if m.group(1):
            out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def _kernels(asm):
    lines = asm.split("\n")
    starts = [i for i, l in enumerate(lines) if re.match(r"^_ZN.*woq_gemm_dense_kernel.*:", l)]
    for s in starts:
        e = next(i for i in range(s + 1, len(lines)) if lines[i].startswith(".Lfunc_end"))
        body = [l.split(";")[0].strip() for l in lines[s:e]]
        yield lines[s].split(":")[0], [l for l in body if l]


def _k_loop(body):
    """The backward branch that encloses the most MFMAs: (first, last) instruction index."""
    labels = {m.group(1): i for i, l in enumerate(body) if (m := re.match(r"^(\.LBB\d+_\d+):", l))}
    best = None
    for i, l in enumerate(body):
        m = re.match(r"s_c?branch\w* (\.LBB\d+_\d+)", l)
        if m and labels.get(m.group(1), i) < i:
            a = labels[m.group(1)]
            n = sum(1 for x in body[a:i] if x.startswith("v_mfma"))
            if best is None or n > best[2]:
                best = (a, i, n)
    return best


@pytest.mark.skipif(shutil.which("hipcc") is None and not os.path.exists("/opt/rocm/bin/hipcc"), reason="no hipcc")
def test_fragment_loads_of_the_dense_kernel_are_waited_for_before_their_registers_are_touched(tmp_path):
    import build as woq_build

    out = tmp_path / "dense.s"
    cmd = [woq_build.HIPCC, *woq_build.FLAGS, "-I", os.path.join(ROOT, "include"), "--cuda-device-only", "-S",
           os.path.join(CSRC, "woq_gemm_dense.hip"), "-o", str(out)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr[-2000:]
    seen = 0
    for name, body in _kernels(out.read_text()):
        seen += 1
        a, b, mfmas = _k_loop(body)
        assert mfmas >= 64, (name, mfmas)
        loop = body[a:b + 1]
        assert not any(re.match(r"s_waitcnt.*vmcnt\(0\)", l) for l in loop), name
        assert not any(l.startswith(("v_accvgpr", "v_mov_b32", "scratch_")) for l in loop), name
        in_flight, touched_in_flight, deepest = [], [], 0
        for l in body[:b + 1] + loop + body[b + 1:]:
            if l.endswith(":") or l.startswith("."):
                continue
            op = l.split()[0]
            if op == "s_waitcnt":
                m = re.search(r"vmcnt\((\d+)\)", l)
                if m:
                    del in_flight[:max(0, len(in_flight) - int(m.group(1)))]
                continue
            regs = _registers(l)
            touched_in_flight += [l for d in in_flight if d & regs]
            if op.startswith(("global_load", "buffer_load")):
                # the fragment loads carry registers; the activation loads go to LDS and carry none
                in_flight.append(_registers(l.split(",")[0]) if op == "global_load_dwordx4" else set())
                deepest = max(deepest, len(in_flight))
            elif op.startswith(("global_store", "buffer_store", "global_atomic")):
                in_flight.append(set())
        assert not touched_in_flight, (name, touched_in_flight[:3])
        assert deepest >= 16, (name, deepest)  # a whole K step of fragments is kept in flight
    assert seen >= 4, seen  # three workgroup shapes, the narrowest twice
