#!/usr/bin/env python3
"""Writes tests/golden/golden.npz: the output of the REFERENCE's own compiled ggml-cpu flash_attn_ext
(oracle/_ref, built by oracle/Makefile from /root/reference) for the cases of tests/golden/cases.py.
V := K (576 wide), which is the only form that op accepts; all 576 output columns are stored as float32.
Run in the build container:  python tests/golden/gen_golden.py"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import oracle as O  # noqa: E402
from tests.golden import cases  # noqa: E402


def main():
    if not O.ref_available():
        O.build()
    out = {}
    for name in cases.CASES:
        inp = cases.make_inputs(name)
        y = O.ref_flash_attn_ext(inp["q"], inp["k"], inp["k_type"], mask=inp["mask"], scale=inp["scale"], n_threads=4)
        out[name] = y
        out[name + "/digest"] = np.frombuffer(inp["digest"].encode(), dtype=np.uint8)
        print(name, y.shape, float(np.abs(y).max()))
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "golden.npz"), **out)


if __name__ == "__main__":
    main()
