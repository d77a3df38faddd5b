"""Golden fixtures: the oracle must still reproduce them bit for bit (CPU), and the GPU path must
match them to the parity bar (GPU) -- so a drifting oracle and a drifting kernel are told apart."""
import json
import os

import numpy as np
import pytest

from tests.helpers import assert_parity, gpu_workload, oracle_workload
from tinytitan_amd import synthetic

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INDEX = json.load(open(os.path.join(HERE, "index.json")))


def _load(name):
    entry = INDEX[name]
    w = getattr(synthetic, entry["builder"])(**entry["kwargs"])
    data = np.load(os.path.join(HERE, name + ".npz"))
    outs = [data[f"out{i}"].view(np.float16).astype(np.float32) for i in range(entry["sequences"])]
    return w, outs


@pytest.mark.parametrize("name", sorted(INDEX))
def test_oracle_reproduces_golden(name):
    w, golden = _load(name)
    for got, want in zip(oracle_workload(w), golden):
        # fp16-rounded outputs; one ulp of slack for libm differences between build hosts
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 2.0 ** -10 * max(1.0, np.abs(want).max())
        assert (got != want).mean() < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(INDEX))
def test_gpu_matches_golden(gpu_ctx, name):
    w, golden = _load(name)
    assert_parity(gpu_workload(gpu_ctx, w), golden, name)
