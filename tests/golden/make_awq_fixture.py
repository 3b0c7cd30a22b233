"""Writes tests/golden/awq_fixture.pt from the AutoAWQ tensors the reference's own test holds
(tests/cpu/data/awq/{qweight,scales,qzeros,bias,act}.pt; used by
tests/cpu/test_ipex_llm_quantization.py:112-151).  Data only: the files are tensor archives
loaded with weights_only=True; the activation is cut to its first 48 rows to keep the
fixture small.  Run once in a container that mounts the reference:

    python tests/golden/make_awq_fixture.py /root/reference
"""
import os
import sys

import torch


def main(ref_root):
    src = os.path.join(ref_root, "tests", "cpu", "data", "awq")
    out = {}
    for name in ("qweight", "scales", "qzeros", "bias", "act"):
        out[name] = torch.load(os.path.join(src, name + ".pt"), weights_only=True)
    out["act"] = out["act"][:48].clone()
    dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "awq_fixture.pt")
    torch.save(out, dst)
    print({k: (tuple(v.shape), v.dtype) for k, v in out.items()})


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
