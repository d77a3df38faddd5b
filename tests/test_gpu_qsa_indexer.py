"""The sparse-attention block indexer (pool, norm and rotation, score, select) through the C ABI.

Bars: pooling and the selection are bit-exact against the oracle (the selection on the same scores);
scores agree to fp32 rounding (another summation order on the matrix cores: |diff| <= 2e-5 * sum |q||k|
per head, far below what separates two scores that are not ties); the norm-and-rotation chain, whose
stages round to fp16, to 2 ulp of fp16 at the value's magnitude plus 1e-3 absolute."""
import ctypes

import numpy as np
import pytest

import oracle
from tests.test_gpu_attention_api import _check, _dev
from tests.test_gpu_keep_mask import _decode_keep, _oracle_kept
from tests.test_gpu_kv_quant import _append, _cache

pytestmark = pytest.mark.gpu

RATIO, BUDGET = 4, 64  # the reference's test geometry (QSAIndexerTests.swift:19-21)
WIDTH = BUDGET + RATIO - 1


def _lib(ctx):
    return ctx._lib


def _select(ctx, scores, rows, first_visible, ratio, width, compact=True, keep_stride=None, score_stride=None, mask=True):
    """tt_hip_qsa_select on host scores [rows][score_stride]; returns (keep [rows][keep_stride], indices, counts);
    mask=False passes no mask rows and returns None for them."""
    import torch
    scores = np.ascontiguousarray(scores, dtype=np.float32).reshape(rows, -1)
    score_stride = score_stride or scores.shape[1]
    last = first_visible + rows - 1
    keep_stride = keep_stride or (last + 3) // 4 * 4
    sd = torch.from_numpy(scores).cuda()
    keep = torch.full((rows, keep_stride), 7, dtype=torch.uint8, device="cuda")
    idx = torch.full((rows, max(width, 1)), -1, dtype=torch.int32, device="cuda") if compact else None
    cnt = torch.full((rows,), -1, dtype=torch.int32, device="cuda") if compact else None
    torch.cuda.synchronize()
    ctx._check(_lib(ctx).tt_hip_qsa_select(ctx.handle, sd.data_ptr(), score_stride, rows, first_visible, ratio, width,
                                           keep.data_ptr() if mask else None, keep_stride, idx.data_ptr() if compact else None,
                                           max(width, 1), cnt.data_ptr() if compact else None), "tt_hip_qsa_select")
    ctx.synchronize()
    if not mask:
        assert (keep.cpu().numpy() == 7).all()
    return (keep.cpu().numpy() if mask else None), (idx.cpu().numpy() if compact else None), (cnt.cpu().numpy() if compact else None)


def _check_rows(got, scores, rows, first_visible, ratio, width):
    keep, idx, cnt = got
    scores = np.asarray(scores, dtype=np.float32).reshape(rows, -1)
    for r in range(rows):
        visible = first_visible + r
        _, want, want_idx = oracle.qsa_select_keys(scores[r], visible, ratio, width)
        assert np.array_equal(keep[r, :visible], want), (r, visible)
        assert not keep[r, visible:].any(), "the mask row is zero past the visible keys"
        if idx is not None:
            assert cnt[r] == len(want_idx), (r, visible, cnt[r], len(want_idx))
            assert np.array_equal(idx[r, :cnt[r]].astype(np.uint32), want_idx), (r, visible)


# --- selection: the reference's own cases -----------------------------------------------------

def test_reference_selection_cases(gpu_ctx):
    # QSAIndexerTests.swift:52-106
    keep, idx, cnt = _select(gpu_ctx, np.full(26, 1000.0), 1, 103, RATIO, WIDTH)
    cells = list(np.flatnonzero(keep[0]))
    assert {100, 101, 102} <= set(cells) and len(cells) == WIDTH and cnt[0] == WIDTH and list(idx[0, :WIDTH]) == cells
    scores = np.zeros(18, np.float32)
    scores[:17] = [17 - b for b in range(17)]
    keep, _, _ = _select(gpu_ctx, scores, 1, 68, RATIO, WIDTH)
    cells = list(np.flatnonzero(keep[0]))
    assert len(cells) == 67 and 64 in cells and 66 in cells and 67 not in cells
    keep, _, _ = _select(gpu_ctx, np.full(19, 5.0), 1, 72, RATIO, WIDTH)
    cells = list(np.flatnonzero(keep[0]))
    assert len(cells) == 67 and cells[0] == 0 and cells[-1] == 66
    # inside the window (67 visible) everything is kept; the host mirror hands out no mask there
    keep, idx, cnt = _select(gpu_ctx, np.zeros(20), 1, 67, RATIO, WIDTH)
    assert keep[0, :67].all() and not keep[0, 67:].any() and cnt[0] == 67 and list(idx[0]) == list(range(67))


@pytest.mark.parametrize("seed", range(10))
def test_selection_with_ties_zeros_and_ragged_geometry(gpu_ctx, seed):
    rng = np.random.default_rng(100 + seed)
    ratio = int(rng.choice([1, 2, 3, 4, 8]))
    budget = int(rng.integers(1, 60)) * ratio
    width = budget + ratio - 1
    visible = int(rng.integers(width + 1, 8 * width))
    blocks = visible // ratio + 1
    values = np.array([0.0, -0.0, 0.5, 1.0, 3.0, -2.0, 1e-30, -1e-30, 65504.0], np.float32)
    scores = rng.choice(values, size=blocks).astype(np.float32)
    got = _select(gpu_ctx, scores, 1, visible, ratio, width)
    _check_rows(got, scores, 1, visible, ratio, width)
    assert got[0][0].sum() == width


@pytest.mark.parametrize("blocks,seed", [(1, 0), (2, 1), (255, 2), (1024, 3), (1025, 4), (4097, 7), (16385, 8), (32768, 9),
                                         (40000, 5), (65536, 6), (70000, 10), (300000, 11)])
def test_selection_over_many_blocks(gpu_ctx, blocks, seed):
    # distinct scores (the early exit after the score's passes), then scores that share their upper bytes; the block
    # counts walk through every register-resident size of the kernel and, past 65536, the form that re-reads memory
    rng = np.random.default_rng(200 + seed)
    ratio, width = 4, 2051
    visible = blocks * ratio + int(rng.integers(0, ratio))
    if visible <= width:
        width = max(ratio, visible - 2)
    for scores in (rng.standard_normal(blocks + 1).astype(np.float32),
                   (1.0 + rng.integers(0, 300, blocks + 1) * 2.0 ** -23).astype(np.float32)):
        got = _select(gpu_ctx, scores, 1, visible, ratio, width)
        _check_rows(got, scores, 1, visible, ratio, width)


@pytest.mark.parametrize("blocks,rows", [(5000, 9), (20000, 9), (40000, 10), (70000, 9), (30000, 3), (6000, 8), (30000, 8), (40000, 8),
                                         (900, 64), (1500, 66), (3000, 70), (6000, 64), (12000, 65), (17000, 64),
                                         (1800, 5), (7000, 3), (900, 1024), (1500, 1030), (3000, 1100), (6000, 1024),
                                         (12000, 1024)])
def test_selection_rows_with_many_blocks(gpu_ctx, blocks, rows):
    # more than 8 rows: one workgroup per row with its scores in registers (16, 32 or 64 per thread) or, past 65536
    # blocks, re-read from memory; from 1024 rows on workgroups of 256 threads (4 - 64 scores per thread) while the
    # blocks fit them; up to 8 rows: every row spread over many workgroups
    rng = np.random.default_rng(blocks + rows)
    ratio, width = 4, 2051
    first = blocks * ratio - 2
    last_blocks = (first + rows - 1) // ratio
    scores = (np.abs(rng.standard_normal((rows, last_blocks + 1))) * 30).astype(np.float32)
    scores[:, ::7] = 0.0  # blocks every head dislikes
    got = _select(gpu_ctx, scores, rows, first, ratio, width)
    _check_rows(got, scores, rows, first, ratio, width)


@pytest.mark.parametrize("kind", ["equal", "mostly_zero", "two_values", "negative"])
def test_spread_selection_with_degenerate_scores(gpu_ctx, kind):
    # one row over many workgroups when the scores tie: every block shares the answer's upper bits and the last
    # workgroup resolves them all; and calls of different sizes one after the other (the workspace is left clean)
    rng = np.random.default_rng(len(kind))
    ratio, width = 4, 2051
    for blocks in (20000, 33000, 5000, 17000):
        visible = blocks * ratio + 3
        if kind == "equal":
            scores = np.full(blocks + 1, 2.5, np.float32)
        elif kind == "mostly_zero":
            scores = np.where(rng.random(blocks + 1) < 0.01, rng.random(blocks + 1), 0.0).astype(np.float32)  # fewer positive than the budget
        elif kind == "two_values":
            scores = rng.choice(np.array([1.0, 1.0000001], np.float32), blocks + 1).astype(np.float32)
        else:
            scores = (-np.abs(rng.standard_normal(blocks + 1)) - 0.0).astype(np.float32)
        got = _select(gpu_ctx, scores, 1, visible, ratio, width)
        _check_rows(got, scores, 1, visible, ratio, width)
        mask_only = _select(gpu_ctx, scores, 1, visible, ratio, width, compact=False)
        assert np.array_equal(mask_only[0], got[0])


@pytest.mark.parametrize("shared", [1, 2, 63, 64, 65, 200, 3000])
def test_selection_rank_among_blocks_that_share_their_upper_bits(gpu_ctx, shared):
    # The register-resident kernel finds the rank's upper 16 bits in one pass and, when at most 64 blocks share
    # them, ranks those in one wavefront; more of them go through the 8-bit passes.  `shared` blocks around the rank
    # differ only below those bits; 100 distinct larger scores sit above them, smaller ones below.
    rng = np.random.default_rng(300 + shared)
    ratio, budget = 4, 4 * (100 + shared // 2)
    width = budget + ratio - 1
    for blocks, rows in ((5000, 1), (9000, 12)):
        first = blocks * ratio + 1
        scores = (rng.random((rows, blocks + rows)) * 0.4).astype(np.float32)
        for r in range(rows):
            at = rng.permutation(blocks)[:100 + shared]
            scores[r, at[:100]] = (2.0 + np.arange(100)).astype(np.float32)
            scores[r, at[100:]] = (1.0 + rng.permutation(shared) * 2.0 ** -20).astype(np.float32)
        got = _select(gpu_ctx, scores, rows, first, ratio, width)
        _check_rows(got, scores, rows, first, ratio, width)


@pytest.mark.parametrize("budget_blocks", [40, 700, 2500])
def test_selection_over_scores_of_every_magnitude(gpu_ctx, budget_blocks):
    # scores spread over 120 binades: only a part of a row lies within the 2,048 upper-16-bit values below its largest
    # score that the first pass counts; a rank below them falls back to the passes over single bytes
    rng = np.random.default_rng(budget_blocks)
    ratio = 4
    width = budget_blocks * ratio + ratio - 1
    for blocks, rows in ((6000, 1), (4000, 9)):
        first = blocks * ratio + 2
        scores = np.exp2(-120.0 * rng.random((rows, blocks + rows))).astype(np.float32)
        scores[:, ::11] = 0.0
        got = _select(gpu_ctx, scores, rows, first, ratio, width)
        _check_rows(got, scores, rows, first, ratio, width)


@pytest.mark.parametrize("blocks,rows", [(40, 1), (10, 3), (3000, 1), (9000, 5), (20000, 2), (70000, 1), (70000, 9), (2000, 1100)])
def test_selection_as_lists_alone(gpu_ctx, blocks, rows):
    # no mask rows asked for (selectKeysCompact's answer, QSAIndexer+Scratch.swift:191-217): the lists and counts are
    # those of the call that writes both -- through every form of the kernel: a row inside the dense window, one
    # workgroup per row with the scores in registers or re-read, a row spread over many workgroups
    rng = np.random.default_rng(blocks * 7 + rows)
    ratio, width = 4, 2051
    first = blocks * ratio - 1
    scores = np.abs(rng.standard_normal((rows, (first + rows - 1) // ratio + 1))).astype(np.float32)
    scores[:, ::5] = 0.0
    both = _select(gpu_ctx, scores, rows, first, ratio, width)
    _check_rows(both, scores, rows, first, ratio, width)
    none, idx, cnt = _select(gpu_ctx, scores, rows, first, ratio, width, mask=False)
    assert none is None and np.array_equal(cnt, both[2])
    for r in range(rows):
        assert np.array_equal(idx[r, :cnt[r]], both[1][r, :cnt[r]]), r


def test_selection_rows_of_a_chunk(gpu_ctx):
    # every row of a chunk: its own visible keys, its own scores, rows inside the dense window among them
    rng = np.random.default_rng(300)
    ratio, width, start, tokens = 4, 67, 40, 200
    blocks = (start + tokens - 1) // ratio + 1
    scores = np.round(rng.standard_normal((tokens, blocks)) * 4).astype(np.float32) / 4  # many ties
    got = _select(gpu_ctx, scores, tokens, start + 1, ratio, width)
    _check_rows(got, scores, tokens, start + 1, ratio, width)
    # the mask alone, padded strides
    keep, idx, cnt = _select(gpu_ctx, np.pad(scores, ((0, 0), (0, 5))), tokens, start + 1, ratio, width, compact=False,
                             keep_stride=260)
    assert idx is None and cnt is None and np.array_equal(keep[:, :240], got[0][:, :240]) and not keep[:, 240:].any()


def test_selection_width_below_the_tail_and_budget_beyond_the_blocks(gpu_ctx):
    # qsa_select_decode's side branches (qsa.metal:170-182)
    got = _select(gpu_ctx, np.ones(4), 1, 11, 4, 2)
    _check_rows(got, np.ones(4), 1, 11, 4, 2)
    assert list(np.flatnonzero(got[0][0])) == [8, 9, 10] and got[2][0] == 2
    scores = np.arange(5, dtype=np.float32)
    got = _select(gpu_ctx, scores, 1, 18, 4, 17)  # remaining 15 = 3 whole blocks + 3 cells of 4 complete ones
    _check_rows(got, scores, 1, 18, 4, 17)


def test_selection_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd.engine import TinyTitanHIPError
    L, h = _lib(gpu_ctx), gpu_ctx.handle
    s = torch.zeros(64, dtype=torch.float32, device="cuda")
    k = torch.zeros(256, dtype=torch.uint8, device="cuda")
    i = torch.zeros(256, dtype=torch.int32, device="cuda")
    assert L.tt_hip_qsa_select(h, None, 64, 1, 100, 4, 67, k.data_ptr(), 100, None, 0, None) == 1
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 0, 67, k.data_ptr(), 100, None, 0, None) == 1
    shape = L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 4, 67, k.data_ptr(), 99, None, 0, None)
    assert shape not in (0, 1) and "shape" in str(TinyTitanHIPError(shape, "x")).lower()
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 4, 67, k.data_ptr(), 100, i.data_ptr(), 66, None) == shape
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 10, 2, 100, 4, 67, k.data_ptr(), 128, None, 0, None) == shape
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 0, 100, 4, 67, k.data_ptr(), 0, None, 0, None) == 0
    # no mask: then a list and its counts
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 4, 67, None, 0, None, 0, None) == 1
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 4, 67, None, 0, i.data_ptr(), 67, None) == 1
    assert L.tt_hip_qsa_select(h, s.data_ptr(), 64, 1, 100, 4, 67, None, 0, i.data_ptr(), 67, i.data_ptr() + 4 * 128) == 0
    gpu_ctx.synchronize()


# --- pooling ------------------------------------------------------------------------------------

def _pool(ctx, raw, pooled, dim, first_block, count, ratio, n_kv, gamma_bits=None, eps=1e-6, theta=1e7):
    import torch
    rd = torch.from_numpy(np.ascontiguousarray(raw).view(np.float16)).cuda()
    pd = torch.from_numpy(np.ascontiguousarray(pooled).view(np.float16)).cuda()
    gd = torch.from_numpy(gamma_bits.view(np.int16)).cuda() if gamma_bits is not None else None
    torch.cuda.synchronize()
    ctx._check(_lib(ctx).tt_hip_qsa_pool_blocks(ctx.handle, rd.data_ptr(), pd.data_ptr(), dim, first_block, count, ratio,
                                                n_kv, gd.data_ptr() if gd is not None else None, eps, theta),
               "tt_hip_qsa_pool_blocks")
    ctx.synchronize()
    return pd.cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("dim,ratio,n_kv,first", [(128, 4, 203, 0), (128, 4, 8192, 1000), (256, 8, 77, 2), (128, 1, 50, 0),
                                                  (128, 3, 100, 31)])
def test_pooling_is_bit_exact(gpu_ctx, dim, ratio, n_kv, first):
    rng = np.random.default_rng(dim + n_kv)
    raw = rng.standard_normal((n_kv, dim)).astype(np.float16).view(np.uint16)
    blocks = (n_kv + ratio - 1) // ratio
    want = np.full((blocks + 3, dim), 0x7E00, np.uint16)
    got = _pool(gpu_ctx, raw, want, dim, first, blocks - first + 3, ratio, n_kv)  # three blocks past the end: left alone
    oracle.qsa_pool_blocks(raw, want, dim, first, blocks - first + 3, ratio, n_kv)
    assert np.array_equal(got, want)
    assert (got[:first] == 0x7E00).all() and (got[blocks:] == 0x7E00).all()


def _bf16_bits(values):
    return np.array([oracle.bf16_bits(float(v)) for v in values], dtype=np.uint16)


def _close_f16(got_bits, want_bits, what):
    got, want = got_bits.view(np.float16).astype(np.float64), want_bits.view(np.float16).astype(np.float64)
    bound = 2 * np.maximum(np.abs(want), 2.0 ** -14) * 2.0 ** -10 + 1e-3
    assert (np.abs(got - want) <= bound).all(), (what, float(np.abs(got - want).max()))


@pytest.mark.parametrize("dim,ratio,n_kv", [(128, 4, 4099), (256, 4, 530)])
def test_pooled_blocks_with_norm_and_rotation(gpu_ctx, dim, ratio, n_kv):
    rng = np.random.default_rng(dim)
    raw = rng.standard_normal((n_kv, dim)).astype(np.float16).view(np.uint16)
    gamma_bits = _bf16_bits(1 + 0.2 * rng.standard_normal(dim))
    gamma = np.array([oracle.bf16_to_f32(int(b)) for b in gamma_bits], dtype=np.float32)
    blocks = (n_kv + ratio - 1) // ratio
    first = 7
    got = _pool(gpu_ctx, raw, np.zeros((blocks, dim), np.uint16), dim, first, blocks - first, ratio, n_kv, gamma_bits)
    plain = np.zeros((blocks, dim), np.uint16)
    oracle.qsa_pool_blocks(raw, plain, dim, first, blocks - first, ratio, n_kv)
    want = oracle.qsa_norm_rope_rows(plain[first:], 1, dim, gamma, 1e-6, 1e7, first * ratio, ratio)
    _close_f16(got[first:], want, "pooled + norm + rotation")
    assert not got[:first].any()


@pytest.mark.parametrize("dim,heads,tokens,position", [(128, 4, 1, 131071), (128, 4, 77, 5000), (256, 2, 9, 0),
                                                       # a chunk's rows (4,096 and more): four to a wavefront, the angles
                                                       # of a token computed once -- with 2 heads a wavefront spans two
                                                       # tokens, with 1 head four; the last wavefront ragged
                                                       (128, 4, 1100, 5000), (128, 2, 2101, 100), (256, 8, 520, 7),
                                                       (128, 1, 4099, 60000)])
def test_norm_and_rotation_of_query_rows(gpu_ctx, dim, heads, tokens, position):
    import torch
    rng = np.random.default_rng(tokens)
    rows = rng.standard_normal((tokens, heads, dim)).astype(np.float16)
    gamma_bits = _bf16_bits(1 + 0.2 * rng.standard_normal(dim))
    gamma = np.array([oracle.bf16_to_f32(int(b)) for b in gamma_bits], dtype=np.float32)
    rd, gd = torch.from_numpy(rows).cuda(), torch.from_numpy(gamma_bits.view(np.int16)).cuda()
    torch.cuda.synchronize()
    gpu_ctx._check(_lib(gpu_ctx).tt_hip_qsa_norm_rope_rows(gpu_ctx.handle, rd.data_ptr(), tokens, heads, dim, gd.data_ptr(),
                                                           1e-6, 1e7, position, 1), "tt_hip_qsa_norm_rope_rows")
    gpu_ctx.synchronize()
    want = oracle.qsa_norm_rope_rows(rows.view(np.uint16), heads, dim, gamma, 1e-6, 1e7, position, 1)
    _close_f16(rd.cpu().numpy().view(np.uint16).reshape(tokens, -1), want, "query rows")


# --- scoring ------------------------------------------------------------------------------------

def _scores(ctx, q, pooled, dim, heads, blocks, tokens, stride=None):
    import torch
    stride = stride or blocks
    qd, pd = torch.from_numpy(q).cuda(), torch.from_numpy(pooled).cuda()
    out = torch.full((tokens, stride), -5.0, dtype=torch.float32, device="cuda")
    torch.cuda.synchronize()
    ctx._check(_lib(ctx).tt_hip_qsa_block_scores(ctx.handle, qd.data_ptr(), pd.data_ptr(), out.data_ptr(), stride, dim, heads,
                                                 blocks, tokens), "tt_hip_qsa_block_scores")
    ctx.synchronize()
    return out.cpu().numpy()


@pytest.mark.parametrize("dim,heads,blocks,tokens", [(128, 4, 32768, 1), (128, 4, 1000, 1), (128, 4, 517, 300), (128, 4, 33, 2048),
                                                     (128, 1, 70, 45), (128, 2, 100, 17), (128, 8, 65, 13), (256, 4, 129, 40),
                                                     (256, 8, 31, 5), (128, 4, 1, 1),
                                                     # a chunk over many blocks: two block tiles per wavefront
                                                     (128, 4, 4100, 80), (128, 8, 4200, 40), (128, 1, 4097, 300), (128, 2, 8191, 130),
                                                     # workgroups that walk six row tiles and more: the LDS ring of three
                                                     # tiles goes round, the last tile ragged
                                                     (128, 4, 1500, 2100), (256, 8, 1500, 1050), (128, 2, 4200, 2500)])
def test_scores_against_the_oracle(gpu_ctx, dim, heads, blocks, tokens):
    rng = np.random.default_rng(dim + heads + blocks + tokens)
    pooled = rng.standard_normal((blocks, dim)).astype(np.float16)
    q = rng.standard_normal((tokens, heads, dim)).astype(np.float16)
    got = _scores(gpu_ctx, q, pooled, dim, heads, blocks, tokens, stride=blocks + 3)
    assert (got[:, blocks:] == -5.0).all(), "nothing is written past a row's blocks"
    want = oracle.qsa_block_scores(q.view(np.uint16), pooled.view(np.uint16), dim, heads, blocks, tokens)
    bound = 2e-5 * np.einsum("thd,bd->tb", np.abs(q.astype(np.float32)), np.abs(pooled.astype(np.float32)))
    assert (np.abs(got[:, :blocks] - want) <= bound + 1e-6).all(), float(np.abs(got[:, :blocks] - want).max())


def test_scores_closed_forms(gpu_ctx):
    dim, blocks = 128, 40
    rng = np.random.default_rng(9)
    pooled = rng.standard_normal((blocks, dim)).astype(np.float16)
    q = np.zeros((1, 4, dim), np.float16)
    picks = [3, 40, 77, 127]
    for h, d in enumerate(picks):
        q[0, h, d] = 1.0
    got = _scores(gpu_ctx, q, pooled, dim, 4, blocks, 1)
    assert np.array_equal(got[0], np.maximum(pooled[:, picks].astype(np.float32), 0).sum(axis=1, dtype=np.float32))
    # rectified per head before the sum: two heads that disagree do not cancel
    pooled2 = np.zeros((3, dim), np.float16)
    pooled2[:, 0] = [1.0, 2.0, -3.0]
    q2 = np.zeros((1, 2, dim), np.float16)
    q2[0, 0, 0], q2[0, 1, 0] = 1.0, -1.0
    assert list(_scores(gpu_ctx, q2, pooled2, dim, 2, 3, 1)[0]) == [1.0, 2.0, 3.0]


def test_pool_and_score_argument_errors(gpu_ctx):
    import torch
    L, h = _lib(gpu_ctx), gpu_ctx.handle
    a = torch.zeros(64 * 128, dtype=torch.float16, device="cuda")
    s = torch.zeros(64, dtype=torch.float32, device="cuda")
    assert L.tt_hip_qsa_pool_blocks(h, None, a.data_ptr(), 128, 0, 1, 4, 4, None, 1e-6, 1e7) == 1
    shape = L.tt_hip_qsa_pool_blocks(h, a.data_ptr(), a.data_ptr(), 96, 0, 1, 4, 4, None, 1e-6, 1e7)
    assert shape not in (0, 1)
    assert L.tt_hip_qsa_pool_blocks(h, a.data_ptr(), a.data_ptr(), 128, 0, 0, 4, 4, None, 1e-6, 1e7) == 0
    assert L.tt_hip_qsa_block_scores(h, a.data_ptr(), a.data_ptr(), s.data_ptr(), 64, 128, 3, 8, 1) == shape  # heads
    assert L.tt_hip_qsa_block_scores(h, a.data_ptr(), a.data_ptr(), s.data_ptr(), 7, 128, 4, 8, 1) == shape   # stride
    assert L.tt_hip_qsa_block_scores(h, a.data_ptr() + 2, a.data_ptr(), s.data_ptr(), 64, 128, 4, 8, 1) == shape
    assert L.tt_hip_qsa_norm_rope_rows(h, a.data_ptr(), 1, 4, 64, a.data_ptr(), 1e-6, 1e7, 0, 1) == shape
    assert L.tt_hip_qsa_norm_rope_rows(h, a.data_ptr(), 1, 4, 128, None, 1e-6, 1e7, 0, 1) == 1


# --- the indexer in front of the attention ----------------------------------------------------

def test_indexer_drives_the_sparse_decode(gpu_ctx):
    # A chunk fills the caches, then a decode step: append its key, repool its block, score, select, attend.
    # The attention over the indexer's mask equals the oracle's attention over the oracle's selection on the
    # same scores, and the gathered index form agrees with the mask form.
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager, QSAIndexer
    H, KH, D, T = 16, 2, 256, 1500
    IH, ID, ratio, budget = 4, 128, 4, 256
    rng = np.random.default_rng(77)
    k, v = (rng.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (rng.standard_normal((1, 1, H, D)).astype(np.float16) for _ in range(2))
    raw = rng.standard_normal((T, ID)).astype(np.float16)
    iq = rng.standard_normal((1, IH, ID)).astype(np.float16)
    gamma_bits = _bf16_bits(1 + 0.1 * rng.standard_normal(ID))
    gamma = np.array([oracle.bf16_to_f32(int(b)) for b in gamma_bits], dtype=np.float32)
    gd = torch.from_numpy(gamma_bits.view(np.int16)).cuda()

    indexer = QSAIndexer(gpu_ctx, IH, ID, ratio, budget, 1e7, capacity=2048)
    assert indexer.selection_width == budget + ratio - 1
    indexer.raw_key_destination(0, 0, T - 1).copy_(torch.from_numpy(raw[:T - 1]).cuda())
    torch.cuda.synchronize()
    indexer.encode_pool_prefill(0, 0, T - 1, gd, 1e-6)
    # the decode step's token joins block (T - 1) / ratio
    indexer.raw_key_destination(0, T - 1, 1).copy_(torch.from_numpy(raw[T - 1:]).cuda())
    torch.cuda.synchronize()
    indexer.encode_pool_prefill(0, T - 1, 1, gd, 1e-6)
    iqd = torch.from_numpy(iq).cuda()
    torch.cuda.synchronize()
    scores = indexer.encode_scores(0, iqd, gd, T - 1, 1, 1e-6)
    mask, indices, count = indexer.select_keys_compact(T)
    gpu_ctx.synchronize()
    scores_h = scores.cpu().numpy()

    blocks = (T - 1) // ratio + 1
    plain = np.zeros((blocks, ID), np.uint16)
    oracle.qsa_pool_blocks(raw.view(np.uint16), plain, ID, 0, blocks, ratio, T)
    pooled_want = oracle.qsa_norm_rope_rows(plain, 1, ID, gamma, 1e-6, 1e7, 0, ratio)
    _close_f16(indexer.pooled[0][:blocks].cpu().numpy().view(np.uint16), pooled_want, "pooled cache")
    # scores on the device's own pooled rows and query: the scoring kernel alone
    q_dev = iqd.cpu().numpy().view(np.uint16)
    want_scores = oracle.qsa_block_scores(q_dev, indexer.pooled[0][:blocks].cpu().numpy().view(np.uint16), ID, IH, blocks, 1)
    assert np.abs(scores_h - want_scores).max() <= 1e-3
    _, want_keep, want_idx = oracle.qsa_select_keys(scores_h[0], T, ratio, indexer.selection_width)
    assert count == indexer.selection_width == len(want_idx)
    assert np.array_equal(mask[:T].cpu().numpy(), want_keep)
    assert np.array_equal(indices[:count].cpu().numpy().astype(np.uint32), want_idx)

    kv = _cache(gpu_ctx, 16, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    qd, gated = _dev(q), _dev(gate)
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_full_keep(kv, 0, qd, out, H, [T], mask, 0.0625, slot=[0], gate=gated,
                                        keep_stride=(T + 3) // 4 * 4)
    gpu_ctx.synchronize()
    got = out.float().cpu().numpy()[0, 0]
    want = _oracle_kept(q[0, 0], k, v, want_keep, H, KH, D, 0.0625, gate=gate[0, 0])
    _check(got, want, "decode over the indexer's selection")
    # index form: gather the listed rows, attend densely over them
    scratch = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=count + 32, initial_capacity=count + 32)
    kd = torch.zeros((count, KH * D), dtype=torch.float16, device="cuda")
    vd = torch.zeros_like(kd)
    torch.cuda.synchronize()
    kv.gather(0, 0, indices[:count], kd, vd)
    gpu_ctx.synchronize()
    scratch.append(0, 0, 0, kd, vd)
    out2 = torch.zeros_like(qd)
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_full(scratch, 0, qd, out2, H, [count], 0.0625, gate=gated)
    gpu_ctx.synchronize()
    _check(out2.float().cpu().numpy()[0, 0], want, "decode over the gathered selection")
    scratch.close()
    kv.close()


@pytest.mark.parametrize("dim,heads,ratio,position", [(128, 4, 4, 1499), (128, 4, 4, 1500), (128, 4, 4, 127), (256, 8, 3, 4000),
                                                      (128, 1, 4, 5), (128, 2, 5, 70001), (256, 4, 4, 0)])
def test_decode_step_in_one_launch_equals_the_three(gpu_ctx, dim, heads, ratio, position):
    # tt_hip_qsa_decode_scores: the newest key's block pooled again, the query rows normed and rotated, every
    # block scored -- bit for bit what pool_blocks (that block), norm_rope_rows and block_scores give in a row;
    # the query rows are left as they came; blocks before the newest key's are not touched.
    import torch
    from tinytitan_amd.engine import QSAIndexer
    rng = np.random.default_rng(position * 31 + dim + heads)
    T = position + 1
    raw = rng.standard_normal((T, dim)).astype(np.float16)
    iq = rng.standard_normal((1, heads, dim)).astype(np.float16)
    key_bits, query_bits = _bf16_bits(1 + 0.1 * rng.standard_normal(dim)), _bf16_bits(1 + 0.1 * rng.standard_normal(dim))
    kd, qd = (torch.from_numpy(b.view(np.int16)).cuda() for b in (key_bits, query_bits))
    results = []
    for fused in (False, True):
        indexer = QSAIndexer(gpu_ctx, heads, dim, ratio, 64, 1e7, capacity=T + 8)
        indexer.raw_key_destination(0, 0, T).copy_(torch.from_numpy(raw).cuda())
        torch.cuda.synchronize()
        if position > 0:
            indexer.encode_pool_prefill(0, 0, position, kd, 1e-6)  # the state before the step
        iqd = torch.from_numpy(iq).cuda()
        torch.cuda.synchronize()
        if fused:
            scores = indexer.encode_decode_step(0, position, iqd, kd, qd, 1e-6)
            gpu_ctx.synchronize()
            assert torch.equal(iqd.cpu(), torch.from_numpy(iq)), "the query rows are read only"
        else:
            indexer.encode_pool_prefill(0, position, 1, kd, 1e-6)
            scores = indexer.encode_scores(0, iqd, qd, position, 1, 1e-6)
            gpu_ctx.synchronize()
        blocks = position // ratio + 1
        assert scores.shape == (1, blocks)
        results.append((scores.cpu().numpy().copy(), indexer.pooled[0][:blocks + 1].cpu().numpy().view(np.uint16).copy()))
    assert np.array_equal(results[0][0].view(np.uint32), results[1][0].view(np.uint32)), "scores differ bit-wise"
    assert np.array_equal(results[0][1], results[1][1]), "pooled blocks differ"


def test_indexer_drives_a_sparse_prefill_chunk(gpu_ctx):
    # per-query selections of a chunk from the indexer, handed to the chunk attention as the per-row mask
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams, QSAIndexer
    H, KH, D = 8, 2, 128
    IH, ID, ratio, budget = 4, 128, 4, 64
    start, tokens = 160, 96
    total = start + tokens
    rng = np.random.default_rng(78)
    k, v = (rng.standard_normal((total, KH, D)).astype(np.float16) for _ in range(2))
    q = rng.standard_normal((tokens, H, D)).astype(np.float16)
    raw = rng.standard_normal((total, ID)).astype(np.float16)
    iq = rng.standard_normal((tokens, IH, ID)).astype(np.float16)
    gamma_bits = _bf16_bits(1 + 0.1 * rng.standard_normal(ID))
    gd = torch.from_numpy(gamma_bits.view(np.int16)).cuda()
    indexer = QSAIndexer(gpu_ctx, IH, ID, ratio, budget, 1e7, capacity=512)
    indexer.raw_key_destination(0, 0, total).copy_(torch.from_numpy(raw).cuda())
    torch.cuda.synchronize()
    indexer.encode_pool_prefill(0, 0, start, gd, 1e-6)
    indexer.encode_pool_prefill(0, start, tokens, gd, 1e-6)  # the chunk repools from its first block on
    iqd = torch.from_numpy(iq).cuda()
    torch.cuda.synchronize()
    scores = indexer.encode_scores(0, iqd, gd, start, tokens, 1e-6)
    selection = indexer.select_keys_prefill(start, tokens)
    gpu_ctx.synchronize()
    assert selection is not None and selection.mask_stride % 4 == 0 and selection.index_stride == indexer.selection_width
    scores_h = scores.cpu().numpy()
    mask = selection.mask[:tokens * selection.mask_stride].view(tokens, selection.mask_stride).cpu().numpy()
    idx = selection.indices[:tokens * selection.index_stride].view(tokens, -1).cpu().numpy()
    cnt = selection.counts[:tokens].cpu().numpy()
    _check_rows((mask, idx, cnt), scores_h, tokens, start + 1, ratio, indexer.selection_width)
    assert indexer.select_keys_prefill(0, 60) is None  # a chunk inside the dense window has no selection

    kv = _cache(gpu_ctx, 16, KH, D, total)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    qd = torch.from_numpy(q).cuda()
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    PrefillAttention(gpu_ctx).encode_causal(kv, 0, 0, qd, out, PrefillAttentionParams(start, tokens, total, H, 0.0625, H * D, H * D),
                                            keep_mask=selection.mask, keep_stride=selection.mask_stride)
    gpu_ctx.synchronize()
    got = out.float().cpu().numpy()
    for t in (0, 17, tokens - 1):
        want = _oracle_kept(q[t], k[:start + t + 1], v[:start + t + 1], mask[t, :start + t + 1], H, KH, D, 0.0625)
        _check(got[t], want, f"chunk row {t} over its selection")
    kv.close()


def test_indexer_step_in_a_graph(gpu_ctx):
    # a decode step's four calls captured in one graph, at a context the one-workgroup selection serves and at one
    # the multi-workgroup form serves (whose workspace every replay must leave clean for the next): replays equal
    # the eager results, with eager calls in between.  The first use allocates (scores, mask, workspace), which a
    # capture refuses: the eager pass comes first.
    import torch
    from tinytitan_amd.engine import HIPContext, QSAIndexer
    ctx = HIPContext(gpu_ctx.device)
    IH, ID, ratio, budget = 4, 128, 4, 2048
    rng = np.random.default_rng(91)
    gamma = torch.from_numpy(_bf16_bits(1 + 0.1 * rng.standard_normal(ID)).view(np.int16)).cuda()
    setups = []
    for cells in (20000, 100001):
        ix = QSAIndexer(ctx, IH, ID, ratio, budget, 1e7, capacity=cells + 3)
        ix.raw_key_destination(0, 0, cells).copy_(torch.from_numpy(rng.standard_normal((cells, ID)).astype(np.float16)).cuda())
        torch.cuda.synchronize()
        ix.encode_pool_prefill(0, 0, cells - 1, gamma, 1e-6)
        q0 = torch.from_numpy(rng.standard_normal((1, IH, ID)).astype(np.float16)).cuda()
        setups.append((ix, cells, q0, q0.clone()))

    def step():
        for ix, cells, q0, q in setups:
            ix.encode_pool_prefill(0, cells - 1, 1, gamma, 1e-6)
            ix.encode_scores(0, q, gamma, cells - 1, 1, 1e-6)
            ix._select(1, cells, ix.scored_blocks_per_row, (cells + 3) // 4 * 4, True)

    def outputs():
        return [(ix.keep_buf[:cells].clone(), ix.keep_index_buf[:ix.selection_width].clone(), ix.keep_count_buf[:1].clone())
                for ix, cells, _, _ in setups]

    def reset():
        for ix, _, q0, q in setups:
            q.copy_(q0)  # the norm and rotation work in place
            ix.keep_buf.fill_(9)
            ix.keep_index_buf.fill_(-1)
            ix.keep_count_buf.fill_(-1)
        torch.cuda.synchronize()

    step()  # allocates the indexers' buffers and the selection workspace
    ctx.synchronize()
    reset()
    step()
    ctx.synchronize()
    eager = outputs()
    for (ix, cells, _, _), (mask, idx, cnt) in zip(setups, eager):
        blocks = (cells - 1) // ratio + 1
        scores = ix.scores_buf[:blocks].cpu().numpy()
        _, want_keep, want_idx = oracle.qsa_select_keys(scores, cells, ratio, ix.selection_width)
        assert np.array_equal(mask.cpu().numpy(), want_keep) and int(cnt[0]) == len(want_idx)
        assert np.array_equal(idx[:len(want_idx)].cpu().numpy().astype(np.uint32), want_idx)
    reset()
    ctx.graph_begin()
    step()
    graph = ctx.graph_end()
    for replay in range(3):
        reset()
        graph.launch()
        ctx.synchronize()
        for got, want in zip(outputs(), eager):
            assert all(torch.equal(g, w) for g, w in zip(got, want)), f"replay {replay}"
        reset()
        step()  # eager work between replays
        ctx.synchronize()
    graph.close()
    ctx.close()


def test_indexer_snapshot_payload(gpu_ctx):
    # QSAIndexer+State.swift:11-113: per layer the pooled blocks and the raw keys of the last block, in the
    # reference's wire format; a restored indexer scores and selects the next step exactly as the original does
    import torch
    from tinytitan_amd.engine import QSAIndexer
    IH, ID, ratio, budget, position = 4, 128, 4, 64, 1022  # a partial last block: 2 members
    rng = np.random.default_rng(55)
    gamma = torch.from_numpy(_bf16_bits(1 + 0.1 * rng.standard_normal(ID)).view(np.int16)).cuda()
    raw = {layer: rng.standard_normal((position + 1, ID)).astype(np.float16) for layer in (3, 7)}

    def filled():
        ix = QSAIndexer(gpu_ctx, IH, ID, ratio, budget, 1e7, capacity=2048)
        for layer in (7, 3):
            ix.raw_key_destination(layer, 0, position).copy_(torch.from_numpy(raw[layer][:position]).cuda())
            torch.cuda.synchronize()
            ix.encode_pool_prefill(layer, 0, position, gamma, 1e-6)
        gpu_ctx.synchronize()
        return ix

    source = filled()
    payload = bytearray(b"head")
    source.append_snapshot_payload(payload, position)
    blocks, tail = 256, 2
    assert len(payload) == 4 + 4 + 2 * (12 + blocks * ID * 2 + tail * ID * 2)
    assert int.from_bytes(payload[4:8], "little") == 2 and int.from_bytes(payload[8:12], "little") == 3  # layers ascending
    assert [int.from_bytes(payload[12 + 4 * k:16 + 4 * k], "little") for k in range(2)] == [blocks, tail]
    assert bytes(payload[20:20 + blocks * ID * 2]) == source.pooled[3][:blocks].cpu().numpy().tobytes()

    restored = QSAIndexer(gpu_ctx, IH, ID, ratio, budget, 1e7, capacity=2048)
    end = restored.restore_snapshot_payload(bytes(payload), 4, position)
    assert end == len(payload)
    results = []
    for ix in (source, restored):
        step = []
        for layer in (3, 7):  # the next token joins the partial block: repooling reads the restored raw tail
            ix.raw_key_destination(layer, position, 1).copy_(torch.from_numpy(raw[layer][position:]).cuda())
            q = torch.from_numpy(raw[layer][:IH].reshape(1, IH, ID).copy()).cuda()
            torch.cuda.synchronize()
            ix.encode_pool_prefill(layer, position, 1, gamma, 1e-6)
            scores = ix.encode_scores(layer, q, gamma, position, 1, 1e-6).clone()
            mask, idx, count = ix.select_keys_compact(position + 1)
            gpu_ctx.synchronize()
            step.append((scores.cpu(), mask[:position + 1].clone().cpu(), idx[:count].clone().cpu()))
        results.append(step)
    for (s0, m0, i0), (s1, m1, i1) in zip(*results):
        assert torch.equal(s0, s1) and torch.equal(m0, m1) and torch.equal(i0, i1)
    with pytest.raises(ValueError):
        restored.restore_snapshot_payload(bytes(payload), 4, position + 4)   # other blocks than the position implies
    with pytest.raises(ValueError):
        restored.restore_snapshot_payload(bytes(payload[:-10]), 4, position)  # truncated
