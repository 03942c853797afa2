#!/usr/bin/env python3
"""Writes tests/golden/golden.npz: the output of the REFERENCE's own compiled ggml-cpu flash_attn_ext
(oracle/_ref, built by oracle/Makefile from /root/reference) for the cases of tests/golden/cases.py.
V := K (576 wide), which is the only form that op accepts; all 576 output columns are stored as float32.
Also tests/golden/front_golden.npz (the same for the nodes either side of the attention node: ROPE, and the query-side /
output-side sub-graphs of llm_attn_mla, cases.FRONT_CASES) and tests/golden/ggml_abi_table.json (struct sizes, offsets and
enum ordinals of the reference's headers as its compiler sees them).
Run in the build container:  python tests/golden/gen_golden.py"""
import json
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
        y = O.ref_flash_attn_ext(inp["q"], inp["k"], inp["k_type"], mask=inp["mask"], scale=inp["scale"], max_bias=inp["max_bias"],
                                 softcap=inp["softcap"], n_threads=4)
        out[name] = y
        out[name + "/digest"] = np.frombuffer(inp["digest"].encode(), dtype=np.uint8)
        print(name, y.shape, float(np.abs(y).max()))
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "golden.npz"), **out)
    out = {}
    for name in cases.FRONT_CASES:
        inp = cases.make_front_inputs(name)
        if inp["kind"] == "rope":
            y = O.ref_rope(inp["x"], inp["pos"], inp["p"])
        elif inp["kind"] == "q_states":
            y = O.ref_mla_q_states(inp["x"], inp["wkv_b"], inp["w_type"], inp["pos"], inp["p"], inp["n_head"])
        else:
            y = O.ref_mla_unabsorb(inp["x"], inp["wkv_b"], inp["w_type"], inp["n_head"])
        out[name] = y
        out[name + "/digest"] = np.frombuffer(inp["digest"].encode(), dtype=np.uint8)
        print(name, y.shape, float(np.abs(y).max()))
    np.savez_compressed(os.path.join(ROOT, "tests", "golden", "front_golden.npz"), **out)
    # sizeof / offsetof / enum ordinals of the reference's headers, as its own compiler sees them
    with open(os.path.join(ROOT, "tests", "golden", "ggml_abi_table.json"), "w") as f:
        json.dump(O.ref_abi_table(), f, indent=1, sort_keys=True)
        f.write("\n")


if __name__ == "__main__":
    main()
