#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/: small seeded inputs and the CPU oracle's outputs.

    python tests/golden/make_golden.py

The reference holds no numeric fixtures for this path (its tests regenerate inputs from
SeedTree / SplitMix64), so these vectors come from this repository's own oracle
(oracle/attn_oracle.c), which is pinned independently in tests/test_oracle_pinning.py.  Inputs
are not stored: they are regenerated from the seed by tinytitan_amd.synthetic, whose stream is
pinned against published SplitMix64 / FNV-1a answers.  Outputs are stored as fp16 bit patterns.
"""
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from tests.helpers import oracle_workload  # noqa: E402
from tinytitan_amd import synthetic  # noqa: E402

CASES = {
    "c1_full": ("decode_c1", {}),
    "c2_ctx777": ("decode_c2", {"context": 777}),
    "c3_4seq": ("decode_c3", {"n_seq": 4, "lo": 3, "hi": 400}),
    "c4_t40_start50": ("prefill_c4", {"tokens": 40, "start": 50}),
    "c5_2seq_ctx300_rows4": ("verify_c5", {"n_seq": 2, "context": 300, "rows": 4}),
}


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    index = {}
    for name, (builder, kwargs) in CASES.items():
        w = getattr(synthetic, builder)(**kwargs)
        outs = oracle_workload(w)
        arrays = {f"out{i}": o.astype(np.float16).view(np.uint16) for i, o in enumerate(outs)}
        np.savez_compressed(os.path.join(here, name + ".npz"), **arrays)
        index[name] = {"builder": builder, "kwargs": kwargs, "sequences": len(outs)}
    with open(os.path.join(here, "index.json"), "w") as f:
        json.dump(index, f, indent=1, sort_keys=True)
    print("wrote", sorted(index))


if __name__ == "__main__":
    main()
