#!/usr/bin/env python3
"""Writes the golden fixtures of tests/golden/: small seeded inputs and the CPU oracle's outputs.

    python tests/golden/make_golden.py

The reference holds no numeric fixtures for this path (its tests regenerate inputs from
SeedTree / SplitMix64), so the attention vectors come from this repository's own oracle
(oracle/attn_oracle.c), which is pinned independently in tests/test_oracle_pinning.py; the o_proj
vectors are the outputs of the reference's own C kernels as built into oracle/_ref.  Inputs
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


# Pre-attention epilogue: (tokens, heads, kv_heads, dim, rotary_dim, base position)
EPILOGUE_CASES = {
    "epilogue_t37_pos41": {"tokens": 37, "heads": 16, "kv_heads": 2, "dim": 256, "rotary_dim": 64, "position": 41},
    "epilogue_t5_pos40000_d128": {"tokens": 5, "heads": 8, "kv_heads": 2, "dim": 128, "rotary_dim": 32, "position": 40000},
}
EPILOGUE_EPS, EPILOGUE_THETA = 1e-6, 1e7


def epilogue_outputs(case):
    import oracle
    x = synthetic.epilogue_inputs(case["tokens"], case["heads"], case["kv_heads"], case["dim"])
    return oracle.qkv_epilogue(x["packed"].astype(np.float32), x["k"].astype(np.float32), case["tokens"], case["heads"],
                               case["kv_heads"], case["dim"], x["q_weight"], x["k_weight"], EPILOGUE_EPS,
                               case["rotary_dim"], EPILOGUE_THETA, case["position"])


# Quantised KV rows: (tokens, kv_heads, dim, bits); the rows are the seeded N(0,1) stream below, every
# third token scaled down (small scales), token 1's first group constant (scale 0).
QUANT_CASES = {
    "kvq_t19_2x256_8bit": {"tokens": 19, "kv_heads": 2, "dim": 256, "bits": 8},
    "kvq_t19_2x256_4bit": {"tokens": 19, "kv_heads": 2, "dim": 256, "bits": 4},
    "kvq_t7_3x64_8bit": {"tokens": 7, "kv_heads": 3, "dim": 64, "bits": 8},
    "kvq_t7_3x64_4bit": {"tokens": 7, "kv_heads": 3, "dim": 64, "bits": 4},
}


def quant_inputs(case):
    n = case["tokens"] * case["kv_heads"] * case["dim"]
    rows = synthetic.normal(0x4B51, f"kvq-{case['kv_heads']}x{case['dim']}", n).reshape(case["tokens"], -1).astype(np.float32)
    rows[::3] *= 0.01
    rows[1, :64] = 0.75
    return rows.astype(np.float16)


def quant_outputs(case):
    import oracle
    return oracle.kv_quantize_rows(quant_inputs(case).astype(np.float32), case["bits"])


# o_proj: (rows, columns, bits, tokens).  The outputs stored for these are NOT this repository's oracle's: they are
# what the reference's own C kernels (tinytitan_int4_affine_gemv / tinytitan_int8_affine_gemv, compiled from the
# reference checkout into oracle/_ref by `make -C oracle`) return for the regenerated inputs, as raw fp32.
OPROJ_CASES = {
    "oproj_m48_n704_4bit": {"rows": 48, "columns": 704, "bits": 4, "tokens": 3},
    "oproj_m48_n704_8bit": {"rows": 48, "columns": 704, "bits": 8, "tokens": 3},
    "oproj_m7_n64_4bit": {"rows": 7, "columns": 64, "bits": 4, "tokens": 2},
}


def oproj_inputs(case):
    """(packed, scales, biases, x fp16): weights uniform(-0.5, 0.5) quantised per row, x uniform(-1, 1), as the
    reference's GEMV tests draw them (DequantInt4GEMVTests.swift:52-66)."""
    import oracle
    label = f"oproj-m{case['rows']}-n{case['columns']}"
    raw = oracle.fill_uniform(0x0B, label, -0.5, 0.5, case["rows"] * case["columns"]).reshape(case["rows"], case["columns"])
    x = oracle.fill_uniform(0x0B, label + "-x", -1.0, 1.0, case["tokens"] * case["columns"]).reshape(case["tokens"], -1)
    return oracle.affine_quantize_rows(raw, case["bits"]) + (x.astype(np.float16),)


def oproj_reference_outputs(case):
    import oracle
    packed, scales, biases, x = oproj_inputs(case)
    lines = [oracle.reference_affine_gemv(packed, scales, biases, row.astype(np.float32), case["bits"]) for row in x]
    if any(line is None for line in lines):
        raise RuntimeError("oracle/_ref is not built: run `make -C oracle` where the reference checkout is present")
    return np.stack(lines)


# The sparse attention's indexer: (raw keys cached, heads, dim, ratio, budget).  Stored: the pooled blocks (plain
# means), the scores of one query row over them, and the selection of that row as mask, index list and count.
QSA_CASES = {
    "qsa_t1003_r4_b64": {"cells": 1003, "heads": 4, "dim": 128, "ratio": 4, "budget": 64},
    "qsa_t700_r8_b128": {"cells": 700, "heads": 2, "dim": 128, "ratio": 8, "budget": 128},
}


def qsa_inputs(case):
    """(raw keys fp16 [cells][dim], query fp16 [1][heads][dim]); every fifth key is repeated so that pooled blocks,
    and with them scores, tie."""
    label = f"qsa-{case['cells']}-{case['ratio']}"
    raw = synthetic.normal(0x05A, label, case["cells"] * case["dim"]).reshape(case["cells"], case["dim"]).astype(np.float16)
    group = 5 * case["ratio"]
    for first in range(0, case["cells"] - 2 * group, 7 * group):
        raw[first + group:first + 2 * group] = raw[first:first + group]
    q = synthetic.normal(0x05A, label + "-q", case["heads"] * case["dim"]).reshape(1, case["heads"], case["dim"]).astype(np.float16)
    return raw, q


def qsa_outputs(case):
    import oracle
    raw, q = qsa_inputs(case)
    cells, ratio, dim = case["cells"], case["ratio"], case["dim"]
    blocks = (cells - 1) // ratio + 1
    pooled = np.zeros((blocks, dim), np.uint16)
    oracle.qsa_pool_blocks(raw.view(np.uint16), pooled, dim, 0, blocks, ratio, cells)
    scores = oracle.qsa_block_scores(q.view(np.uint16), pooled, dim, case["heads"], blocks, 1)
    _, keep, indices = oracle.qsa_select_keys(scores[0], cells, ratio, case["budget"] + ratio - 1)
    return pooled, scores, keep, indices


def main():
    here = os.path.dirname(os.path.abspath(__file__))
    for name, case in QSA_CASES.items():
        pooled, scores, keep, indices = qsa_outputs(case)
        np.savez_compressed(os.path.join(here, name + ".npz"), pooled=pooled, scores=scores, keep=keep, indices=indices)
    with open(os.path.join(here, "qsa_index.json"), "w") as f:
        json.dump(QSA_CASES, f, indent=1, sort_keys=True)
    for name, case in OPROJ_CASES.items():
        np.savez_compressed(os.path.join(here, name + ".npz"), y=oproj_reference_outputs(case))
    with open(os.path.join(here, "oproj_index.json"), "w") as f:
        json.dump(OPROJ_CASES, f, indent=1, sort_keys=True)
    for name, case in QUANT_CASES.items():
        np.savez_compressed(os.path.join(here, name + ".npz"), rows=quant_outputs(case))
    with open(os.path.join(here, "kvq_index.json"), "w") as f:
        json.dump(QUANT_CASES, f, indent=1, sort_keys=True)
    for name, case in EPILOGUE_CASES.items():
        q, g, k = epilogue_outputs(case)
        np.savez_compressed(os.path.join(here, name + ".npz"), q=q.astype(np.float16).view(np.uint16),
                            gate=g.astype(np.float16).view(np.uint16), k=k.astype(np.float16).view(np.uint16))
    with open(os.path.join(here, "epilogue_index.json"), "w") as f:
        json.dump(EPILOGUE_CASES, f, indent=1, sort_keys=True)
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
