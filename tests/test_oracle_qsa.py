"""Pins the oracle of the sparse-attention block indexer (pool, score, select) on the CPU.

The selection rule is checked against the cases and expected cells of the reference's own tests
(tests/TinyTitan/Kernels/Attention/QSAIndexerTests.swift, tests/TinyTitan/Runtime/QSAExactnessTests.swift)
and against an independent restatement over cells; pooling and scoring against closed forms that a
plausible mistake fails, and float64 numpy."""
import numpy as np
import pytest

import oracle
from tinytitan_amd.engine import QSAExactness, QSAIndexerRequired

RATIO, BUDGET = 4, 64          # QSAIndexerTests.swift:19-21
WIDTH = BUDGET + RATIO - 1     # selectionWidth, QSAIndexer.swift:91


def kept(keep):
    return [int(i) for i in np.flatnonzero(keep)]


def select_over_cells(scores, visible, ratio, width):
    """The rule as the reference words it: cells ordered by (score descending, index ascending), every cell
    carrying its block's score, the tail biased above everything (QSAIndexer+Scratch.swift:216-246)."""
    keep = np.zeros(visible, dtype=np.uint8)
    if visible <= width:
        keep[:] = 1
        return keep
    complete = visible // ratio * ratio
    keep[complete:] = 1
    remaining = width - (visible - complete)
    cell_scores = np.repeat(np.asarray(scores[:complete // ratio], dtype=np.float64), ratio)
    order = np.argsort(-cell_scores, kind="stable")  # stable: equal scores stay in index order
    keep[order[:max(remaining, 0)]] = 1
    return keep


# --- the reference's own selection cases ------------------------------------------------------

def test_dense_window_skips_selection():
    # QSAIndexerTests.swift:42-50
    assert WIDTH == 67
    selected, keep, idx = oracle.qsa_select_keys(np.zeros(20, np.float32), 67, RATIO, WIDTH)
    assert not selected and keep.all() and list(idx) == list(range(67))
    selected, _, _ = oracle.qsa_select_keys(np.zeros(20, np.float32), 68, RATIO, WIDTH)
    assert selected


def test_tail_always_survives():
    # QSAIndexerTests.swift:52-68: 25 complete blocks + 3 tail cells, every block far above zero
    visible = 103
    selected, keep, idx = oracle.qsa_select_keys(np.full(visible // 4 + 1, 1000.0, np.float32), visible, RATIO, WIDTH)
    cells = kept(keep)
    assert selected and {100, 101, 102} <= set(cells) and len(cells) == WIDTH
    assert list(idx) == cells


def test_budget_cuts_the_last_block():
    # QSAIndexerTests.swift:70-90: 17 complete blocks, block 0 best; 16 whole, the worst gives 3 of 4
    scores = np.zeros(18, np.float32)
    scores[:17] = [17 - b for b in range(17)]
    _, keep, _ = oracle.qsa_select_keys(scores, 68, RATIO, WIDTH)
    cells = kept(keep)
    assert len(cells) == 67 and 64 in cells and 66 in cells and 67 not in cells


def test_ties_favour_lower_index():
    # QSAIndexerTests.swift:92-106
    _, keep, _ = oracle.qsa_select_keys(np.full(19, 5.0, np.float32), 72, RATIO, WIDTH)
    cells = kept(keep)
    assert len(cells) == 67 and cells[0] == 0 and cells[-1] == 66


@pytest.mark.parametrize("seed", range(12))
def test_selection_against_the_rule_over_cells(seed):
    rng = np.random.default_rng(seed)
    ratio = int(rng.choice([1, 2, 4, 8]))
    budget = int(rng.integers(1, 40)) * ratio
    width = budget + ratio - 1
    visible = int(rng.integers(1, 6 * width))
    blocks = visible // ratio + 1
    # few distinct values: ties everywhere; both zeros
    scores = rng.choice(np.array([0.0, -0.0, 0.5, 1.0, 3.0, -2.0], np.float32), size=blocks).astype(np.float32)
    selected, keep, idx = oracle.qsa_select_keys(scores, visible, ratio, width)
    want = select_over_cells(scores, visible, ratio, width)
    assert selected == (visible > width)
    assert np.array_equal(keep, want)
    assert list(idx) == kept(want)
    if selected:
        assert keep.sum() == width


def test_selection_width_below_tail_keeps_only_the_tail():
    # qsa_select_decode's `width <= tail` branch (qsa.metal:170-173)
    _, keep, _ = oracle.qsa_select_keys(np.ones(4, np.float32), 11, 4, 2)
    assert kept(keep) == [8, 9, 10]


# --- the dense-exact window -------------------------------------------------------------------

def test_exactness_window_of_the_production_geometry():
    # QSAExactnessTests.swift:14-59
    q = QSAExactness(2048, 4)
    assert q.kept_blocks == 512
    assert q.maximum_exact_visible_keys == 2051 and q.indexer_required_from_context == 2052
    for v in (0, 1, 4, 1000, 2048, 2049, 2050, 2051):
        assert q.is_dense_exact(v)
    for v in (2052, 2053, 4096, 262_144):
        assert not q.is_dense_exact(v)
    assert q.is_dense_exact_for_context(2051) and not q.is_dense_exact_for_context(2052)
    assert q.is_dense_exact_for_context(0)


def test_exactness_tracks_the_geometry():
    # QSAExactnessTests.swift:82-91
    assert QSAExactness(64, 1).maximum_exact_visible_keys == 64
    wide = QSAExactness(512, 8)
    assert wide.kept_blocks == 64 and wide.maximum_exact_visible_keys == 64 * 8 + 7


def test_refusal_carries_the_numbers():
    # QSAExactnessTests.swift:61-80
    text = str(QSAIndexerRequired(2052, 2051))
    assert "2052" in text and "2051" in text and "--max-new" in text
    assert "was not built" in text and "not implemented" not in text


def test_exact_window_is_where_the_selection_is_vacuous():
    # the window derived from block accounting is exactly where the selection keeps everything visible
    for budget, ratio in ((64, 4), (16, 8), (12, 1), (2048, 4)):
        q = QSAExactness(budget, ratio)
        width = budget + ratio - 1
        rng = np.random.default_rng(budget)
        for visible in (q.maximum_exact_visible_keys - 1, q.maximum_exact_visible_keys, q.indexer_required_from_context,
                        q.indexer_required_from_context + ratio):
            scores = rng.standard_normal(visible // ratio + 1).astype(np.float32)
            _, keep, _ = oracle.qsa_select_keys(scores, visible, ratio, width)
            assert bool(keep.all()) == q.is_dense_exact(visible), (budget, ratio, visible)


# --- pooling ------------------------------------------------------------------------------------

def half_bits(a):
    return np.asarray(a, dtype=np.float16).view(np.uint16)


def test_pool_of_equal_rows_is_that_row_and_the_tail_divides_by_its_members():
    dim, ratio, n_kv = 128, 4, 14  # blocks 0..2 whole, block 3 has 2 members
    rng = np.random.default_rng(3)
    rows = rng.standard_normal((4, dim)).astype(np.float16)
    raw = np.repeat(rows, ratio, axis=0)[:n_kv]
    pooled = np.zeros((4, dim), np.uint16)
    oracle.qsa_pool_blocks(raw.view(np.uint16), pooled, dim, 0, 4, ratio, n_kv)
    assert np.array_equal(pooled.view(np.float16), rows)  # dividing the tail by the ratio would halve block 3


def test_pool_against_float64_and_untouched_blocks():
    dim, ratio, n_kv = 128, 4, 203
    rng = np.random.default_rng(4)
    raw = rng.standard_normal((n_kv, dim)).astype(np.float16)
    blocks = (n_kv + ratio - 1) // ratio
    pooled = np.full((blocks + 2, dim), 0x7E00, np.uint16)
    oracle.qsa_pool_blocks(raw.view(np.uint16), pooled, dim, 5, blocks - 5 + 2, ratio, n_kv)  # two blocks past the end: skipped
    got = pooled.view(np.float16).astype(np.float64)
    for b in range(5, blocks):
        members = raw[b * ratio:min((b + 1) * ratio, n_kv)].astype(np.float64)
        assert np.abs(got[b] - members.mean(axis=0)).max() <= 1e-3
    assert (pooled[:5] == 0x7E00).all() and (pooled[blocks:] == 0x7E00).all()


# --- scoring ------------------------------------------------------------------------------------

def test_scores_of_one_hot_queries_read_single_elements():
    dim, heads, blocks = 128, 4, 9
    rng = np.random.default_rng(5)
    pooled = rng.standard_normal((blocks, dim)).astype(np.float16)
    q = np.zeros((1, heads, dim), np.float16)
    picks = [3, 40, 77, 127]
    for h, d in enumerate(picks):
        q[0, h, d] = 1.0
    got = oracle.qsa_block_scores(q.view(np.uint16), pooled.view(np.uint16), dim, heads, blocks, 1)
    want = np.maximum(pooled[:, picks].astype(np.float32), 0).sum(axis=1)
    assert np.allclose(got[0], want, rtol=0, atol=1e-6)


def test_scores_rectify_each_head_before_the_sum():
    dim, blocks = 128, 3
    pooled = np.zeros((blocks, dim), np.float16)
    pooled[:, 0] = [1.0, 2.0, -3.0]
    q = np.zeros((1, 2, dim), np.float16)
    q[0, 0, 0], q[0, 1, 0] = 1.0, -1.0  # the heads disagree: summing first would give zero everywhere
    got = oracle.qsa_block_scores(q.view(np.uint16), pooled.view(np.uint16), dim, 2, blocks, 1)
    assert list(got[0]) == [1.0, 2.0, 3.0]


def test_scores_against_float64():
    dim, heads, blocks, tokens = 128, 4, 50, 7
    rng = np.random.default_rng(6)
    pooled = rng.standard_normal((blocks, dim)).astype(np.float16)
    q = rng.standard_normal((tokens, heads, dim)).astype(np.float16)
    got = oracle.qsa_block_scores(q.view(np.uint16), pooled.view(np.uint16), dim, heads, blocks, tokens)
    want = np.maximum(np.einsum("thd,bd->thb", q.astype(np.float64), pooled.astype(np.float64)), 0).sum(axis=1)
    assert np.abs(got - want).max() <= 1e-4


# --- norm and rotation of the pooled rows -----------------------------------------------------

def test_norm_rope_rows_positions_advance_by_the_stride():
    dim, ratio, theta = 128, 4, 1e7
    rng = np.random.default_rng(7)
    rows = rng.standard_normal((6, dim)).astype(np.float16)
    gamma = (1 + 0.1 * rng.standard_normal(dim)).astype(np.float32)
    got = oracle.qsa_norm_rope_rows(rows.view(np.uint16), 1, dim, gamma, 1e-6, theta, 8, ratio).view(np.float16)
    x = rows.astype(np.float64)
    normed = (x / np.sqrt((x * x).mean(axis=1, keepdims=True) + 1e-6) * gamma).astype(np.float16).astype(np.float64)
    half = dim // 2
    freq = theta ** (-2.0 * np.arange(half) / dim)
    for t in range(6):
        angle = (8 + t * ratio) * freq  # block b sits at the position of its first member
        lo, hi = normed[t, :half], normed[t, half:]
        want = np.concatenate([lo * np.cos(angle) - hi * np.sin(angle), lo * np.sin(angle) + hi * np.cos(angle)])
        assert np.abs(got[t].astype(np.float64) - want).max() <= 4e-3
    # position 0 does not rotate: the norm alone, rounded once
    at0 = oracle.qsa_norm_rope_rows(rows[:1].view(np.uint16), 1, dim, gamma, 1e-6, theta, 0, ratio).view(np.float16)
    assert np.abs(at0[0].astype(np.float64) - normed[0]).max() <= 2e-3
