"""Writes tests/golden/blob_muladd_fp32.bin (+ .json): the device VM program of out = x * y + 0.5 over 5000 fp32
elements as the host compiler emits it, for tests/cc/device_blob.cc, which launches it through the device layer's C
ABI alone. No GPU needed: the kernel is compiled in disassembly mode (tensor addresses are placeholders, the test
fills in real ones). Run from the repository root: python tests/golden/make_blob_fixture.py"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
N = 5000


def build():
    from dvm_amd.tester import Tester
    t = Tester("vector", run_mode="das")
    x, y = t.load(np.zeros([N], np.float32)), t.load(np.zeros([N], np.float32))
    t.store(t.add(t.mul(x, y), 0.5))
    t.codegen()
    programs = t.programs()
    assert len(programs) == 1 and programs[0][2] == []
    return programs[0]


if __name__ == "__main__":
    blob, geometry, _ = build()
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "blob_muladd_fp32.bin"), "wb") as f:
        f.write(blob)
    with open(os.path.join(here, "blob_muladd_fp32.json"), "w") as f:
        json.dump({"elements": N, "workgroups": geometry[0], "threads": geometry[1], "lds_bytes": geometry[2]}, f)
    print("wrote", len(blob), "bytes, geometry", geometry)
