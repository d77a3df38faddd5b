"""Decode attention over a sparse key selection (the keepMask of Attention.encodeFull) through the C ABI.

Semantics, as the reference's test states them (SimdPartialAttentionTests.swift:103-123): masking a key out
is the same as its absence, so the oracle is the decode oracle over the kept rows alone.  Bar: the attention
path's own (max-abs 2e-3, mean-abs 2e-4 against the fp16-rounded oracle output); for the reference's own
cases also its bar (max-abs / max|ref| < 0.02 against the fp32 reference over the unquantised inputs)."""
import numpy as np
import pytest

import oracle
from tests.helpers import f16_round
from tests.test_gpu_attention_api import _check, _decode, _dev
from tests.test_gpu_kv_quant import _append, _cache, _dequantised

pytestmark = pytest.mark.gpu


def _decode_keep(ctx, kv, q, seq_lens, keep, heads, scale, slots=None, gate=None, keep_stride=None):
    import torch
    from tinytitan_amd.engine import Attention
    qd, kd = _dev(q), _dev(keep)
    gd = _dev(gate) if gate is not None else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(ctx).encode_full_keep(kv, 0, qd, out, heads, list(seq_lens), kd, scale,
                                    slot=list(slots if slots is not None else range(len(seq_lens))), gate=gd,
                                    keep_stride=keep_stride)
    ctx.synchronize()
    return out.float().cpu().numpy()


def _oracle_kept(q, k, v, keep, heads, kv_heads, dim, scale, gate=None):
    kept = np.flatnonzero(keep)
    kf = k.astype(np.float32).reshape(k.shape[0], -1)[kept]
    vf = v.astype(np.float32).reshape(v.shape[0], -1)[kept]
    return oracle.decode(q.astype(np.float32), kf, vf, heads, kv_heads, dim, scale,
                         gate=gate.astype(np.float32) if gate is not None else None)


@pytest.mark.parametrize("seq_len,fraction,seed", [(4096, 0.55, 0x51AD), (700, 1.0, 0x51AE), (2048, 0.02, 0x51AF)])
def test_reference_cases_int8_cache(gpu_ctx, seq_len, fraction, seed):
    # SimdPartialAttentionTests.swift:15-37, :128-158: Qwen3.8 full-attention geometry (24 q heads, 2 KV heads,
    # dim 256, int8 KV); one stream draws q, k uniform(-0.5, 0.5), v uniform(0, 1), then the selection; the
    # query's own position is always kept; 2 % kept leaves whole key ranges empty.
    H, KH, D = 24, 2, 256
    scale = 1.0 / np.sqrt(np.float32(D))  # encodeFull's default
    n_q, n_kv = H * D, seq_len * KH * D
    u = oracle.fill_uniform(seed, f"simd-partial-{seq_len}", 0.0, 1.0, n_q + 2 * n_kv + seq_len)
    q = (np.float32(-0.5) + np.float32(1.0) * u[:n_q]).astype(np.float16).reshape(H, D)
    k = (np.float32(-0.5) + np.float32(1.0) * u[n_q:n_q + n_kv]).astype(np.float16).reshape(seq_len, KH, D)
    v = u[n_q + n_kv:n_q + 2 * n_kv].astype(np.float16).reshape(seq_len, KH, D)
    keep = (u[n_q + 2 * n_kv:] < np.float32(fraction)).astype(np.uint8)
    keep[seq_len - 1] = 1
    kv = _cache(gpu_ctx, 8, KH, D, seq_len)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    got = _decode_keep(gpu_ctx, kv, q[None, None], [seq_len], keep, H, float(scale))[0, 0]
    kv.close()
    assert np.isfinite(got).all()
    want = _oracle_kept(q, _dequantised(k, 8), _dequantised(v, 8), keep, H, KH, D, float(scale))
    _check(got, want, f"keep {fraction} over {seq_len} keys, 8-bit cache")
    reference = _oracle_kept(q, k, v, keep, H, KH, D, float(scale))  # fp32 reference over the unquantised inputs
    assert np.abs(got - reference).max() / np.abs(reference).max() < 0.02


@pytest.mark.parametrize("bits", [16, 8, 4])
@pytest.mark.parametrize("D,H,KH,T,fraction", [(256, 16, 2, 1187, 0.3), (128, 8, 4, 333, 0.6), (64, 24, 2, 70, 0.5),
                                               (256, 16, 2, 32768, 0.1), (128, 32, 1, 4100, 0.9)])
def test_shapes_precisions_and_splits(gpu_ctx, bits, D, H, KH, T, fraction):
    r = np.random.default_rng(D + T + bits)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((H, D)).astype(np.float16) for _ in range(2))
    keep = (r.random(T) < fraction).astype(np.uint8)
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    got = _decode_keep(gpu_ctx, kv, q[None, None], [T], keep, H, 0.0625, gate=gate[None, None])[0, 0]
    kv.close()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    _check(got, _oracle_kept(q, ks, vs, keep, H, KH, D, 0.0625, gate=gate), f"D={D} H={H}/{KH} T={T} keep {fraction} bits {bits}")


def test_full_mask_is_the_plain_decode_and_empty_mask_gives_zeros(gpu_ctx):
    H, KH, D, T = 16, 2, 256, 900
    r = np.random.default_rng(3)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q = r.standard_normal((1, 1, H, D)).astype(np.float16)
    kv = _cache(gpu_ctx, 16, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    plain = _decode(gpu_ctx, kv, q, [T], H, 0.0625)
    assert np.array_equal(_decode_keep(gpu_ctx, kv, q, [T], np.ones(T, np.uint8), H, 0.0625), plain)
    assert np.array_equal(_decode_keep(gpu_ctx, kv, q, [T], np.full(T, 7, np.uint8), H, 0.0625), plain)  # any non-zero byte keeps
    assert not _decode_keep(gpu_ctx, kv, q, [T], np.zeros(T, np.uint8), H, 0.0625).any()
    one = np.zeros(T, np.uint8)
    one[517] = 1  # a single kept key: the output is that key's V row for every head of its group
    got = _decode_keep(gpu_ctx, kv, q, [T], one, H, 0.0625)[0, 0]
    for h in range(H):
        assert np.array_equal(got[h], v[517, h // (H // KH)].astype(np.float32))
    # bytes past the sequence's end are not read as keys
    longer = np.ones(T + 64, np.uint8)
    assert np.array_equal(_decode_keep(gpu_ctx, kv, q, [T - 100], longer, H, 0.0625), _decode(gpu_ctx, kv, q, [T - 100], H, 0.0625))
    kv.close()


def test_batched_sequences_with_their_own_masks(gpu_ctx):
    H, KH, D = 16, 2, 128
    lengths = [700, 33, 1500]
    r = np.random.default_rng(4)
    kv = _cache(gpu_ctx, 16, KH, D, max(lengths), slots=3)
    rows, masks = [], np.zeros((3, 1536), np.uint8)
    for i, n in enumerate(lengths):
        k, v = (r.standard_normal((n, KH, D)).astype(np.float16) for _ in range(2))
        _append(gpu_ctx, kv, 0, i, 0, k, v)
        masks[i, :n] = r.random(n) < 0.4
        rows.append((k, v))
    q = r.standard_normal((3, 1, H, D)).astype(np.float16)
    got = _decode_keep(gpu_ctx, kv, q, lengths, masks, H, 0.09, keep_stride=1536)
    kv.close()
    for i, (k, v) in enumerate(rows):
        _check(got[i, 0], _oracle_kept(q[i, 0], k, v, masks[i, :lengths[i]], H, KH, D, 0.09), f"sequence {i}")


def test_ring_cache_while_the_sequence_fits_the_ring(gpu_ctx):
    # keep[p] is indexed by the key's position (attention.metal:229-230); without a window a ring serves a sequence
    # only while it fits, so every position is still where it was stored
    import torch
    from tinytitan_amd.engine import KVCacheManager
    H, KH, D, ring, total = 8, 2, 128, 256, 200
    r = np.random.default_rng(5)
    k, v = (r.standard_normal((total, KH, D)).astype(np.float16) for _ in range(2))
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=4096, ring_capacity=ring)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    keep = (r.random(total) < 0.5).astype(np.uint8)
    q = r.standard_normal((1, 1, H, D)).astype(np.float16)
    got = _decode_keep(gpu_ctx, kv, q, [total], keep, H, 0.0884)[0, 0]
    kv.close()
    _check(got, _oracle_kept(q[0, 0], k, v, keep, H, KH, D, 0.0884), "ring cache")


def test_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    H, KH, D, T = 8, 2, 64, 64
    kv = _cache(gpu_ctx, 16, KH, D, T, slots=2)
    q = torch.zeros((2, 1, H, D), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    keep = torch.ones(128, dtype=torch.uint8, device="cuda")
    lib, h = gpu_ctx._lib, gpu_ctx.handle
    slots, lens = capi.int_array([0, 1]), capi.int_array([40, 50])
    call = lambda mask, stride: lib.tt_hip_attn_decode_keep(h, kv.handle, 0, 2, slots, lens, mask, stride, H, q.data_ptr(), None,
                                                            0.125, out.data_ptr())
    assert call(None, 64) == capi.ERR_INVALID_ARGUMENT
    assert call(keep.data_ptr(), 45) == capi.ERR_SHAPE  # the second sequence's mask would start inside the first's
    assert call(keep.data_ptr(), 64) == capi.OK
    gpu_ctx.synchronize()
    kv.close()


# ---- per-query selections of a prefill chunk (mask form) ---------------------------------------

def _prefill_keep(ctx, kv, q, start, kv_valid, keep, heads, scale, gate=None):
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    rows, width = q.shape
    qd, kd = _dev(q), _dev(keep)
    gd = _dev(gate) if gate is not None else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    PrefillAttention(ctx).encode_causal(kv, 0, 0, qd, out, PrefillAttentionParams(start, rows, kv_valid, heads, scale, width, width, width),
                                        gate=gd, keep_mask=kd, keep_stride=keep.shape[1])
    ctx.synchronize()
    return out.float().cpu().numpy()


def _oracle_rows_kept(q, k, v, start, keep, heads, kv_heads, dim, scale, gate=None):
    """Row t over the keys p <= start + t with keep[t][p] != 0: the decode oracle over those rows alone."""
    rows = q.shape[0]
    out = np.zeros((rows, heads * dim), np.float32)
    for t in range(rows):
        visible = keep[t, :start + t + 1]
        if not visible.any():
            continue
        g = gate[t].reshape(heads, dim) if gate is not None else None
        out[t] = _oracle_kept(q[t].reshape(heads, dim), k[:start + t + 1], v[:start + t + 1], visible, heads, kv_heads, dim, scale,
                              gate=g).reshape(-1)
    return out


@pytest.mark.parametrize("bits", [16, 8])
@pytest.mark.parametrize("D,H,KH,start,rows,fraction", [(256, 16, 2, 300, 70, 0.4), (128, 8, 4, 0, 45, 0.7), (64, 4, 4, 1000, 33, 0.2),
                                                        (256, 16, 2, 5000, 2, 0.5), (128, 8, 8, 77, 130, 0.05)])
def test_prefill_chunk_with_per_query_selections(gpu_ctx, bits, D, H, KH, start, rows, fraction):
    # GQA-packed 32-row tiles, the 16-row tile (2 rows of 8 heads), one head per KV head; 5 % kept leaves rows with
    # nothing but (sometimes) their own key, and some rows with no key at all
    r = np.random.default_rng(D + start + rows + bits)
    T = start + rows + 9  # a few keys past the chunk: no row sees them
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((rows, H * D)).astype(np.float16) for _ in range(2))
    stride = ((T + 3) // 4) * 4 + 8
    keep = (r.random((rows, stride)) < fraction).astype(np.uint8)
    keep[1, :] = 0  # one row with no kept key: zeros
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    got = _prefill_keep(gpu_ctx, kv, q, start, T, keep, H, 1.0 / np.sqrt(D), gate=gate)
    kv.close()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    want = _oracle_rows_kept(q, ks, vs, start, keep, H, KH, D, 1.0 / np.sqrt(D), gate=gate)
    assert not got[1].any()
    _check(got, want, f"chunk D={D} {H}/{KH} start {start} rows {rows} keep {fraction} bits {bits}")


@pytest.mark.parametrize("bits", [16, 8])
@pytest.mark.parametrize("D,H,KH,rows,split_tokens", [(256, 16, 2, 13, 0), (256, 16, 2, 13, 4096), (256, 16, 2, 13, 32768),
                                                      (256, 16, 2, 13, 65536), (256, 16, 2, 2, 32768), (128, 8, 2, 9, 32768),
                                                      (64, 4, 4, 40, 16384)])
def test_prefill_chunk_over_a_long_context_lists_the_touched_blocks(gpu_ctx, bits, D, H, KH, rows, split_tokens):
    # Long splits: the workgroup lists the key blocks that any row of its tile keeps a key of -- over one window of 64
    # blocks a wavefront (the planner's own splits; 4096 keys), over four and eight windows (32768, 65536 keys) -- and
    # its wavefronts walk the list in turn.  Rows share a cluster of cells, draw others of their own, keep their own
    # key, and one row keeps nothing.
    # (also the 16-row tile -- 2 rows of 8 heads --, other head sizes, and one head per KV head: 32 tokens a tile)
    start = 70000
    r = np.random.default_rng(7000 + bits + split_tokens + rows)
    T = start + rows
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((rows, H * D)).astype(np.float16) for _ in range(2))
    stride = ((T + 3) // 4) * 4
    keep = np.zeros((rows, stride), np.uint8)
    shared = r.choice(start // 4, 150, replace=False)
    for t in range(rows):
        cells = np.concatenate([shared, r.choice(start // 4, 60, replace=False)])
        keep[t, (cells[:, None] * 4 + np.arange(4)[None, :]).reshape(-1)] = 1
        keep[t, start + t] = 1
    keep[:, 0:3] = 1  # the first block of the first wavefront, which is read before the selection is known
    empty = min(5, rows - 1)
    keep[empty, :] = 0
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    gpu_ctx.set_split_tokens(split_tokens)
    try:
        got = _prefill_keep(gpu_ctx, kv, q, start, T, keep, H, 0.0625, gate=gate)
    finally:
        gpu_ctx.set_split_tokens(0)
        kv.close()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    want = _oracle_rows_kept(q, ks, vs, start, keep, H, KH, D, 0.0625, gate=gate)
    assert not got[empty].any()
    _check(got, want, f"long chunk D={D} {H}/{KH} rows {rows} bits {bits} split {split_tokens}")


@pytest.mark.parametrize("bits,D,H,KH", [(16, 256, 16, 2), (8, 128, 8, 2)])
def test_prefill_chunk_of_many_tiles_in_few_splits_merges_by_half_tiles(gpu_ctx, bits, D, H, KH):
    # 140 rows of 8 heads per KV head are 35 token tiles x 2 KV heads = 70 tiles; with four key ranges each they are
    # launched XCD-major and merged by the combine that takes half a tile per workgroup.
    start, rows = 9000, 140
    r = np.random.default_rng(140 + bits)
    T = start + rows
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((rows, H * D)).astype(np.float16) for _ in range(2))
    stride = ((T + 3) // 4) * 4
    keep = (r.random((rows, stride)) < 0.04).astype(np.uint8)
    keep[np.arange(rows), start + np.arange(rows)] = 1
    keep[17, :] = 0
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    gpu_ctx.set_split_tokens(2560)
    try:
        got = _prefill_keep(gpu_ctx, kv, q, start, T, keep, H, 0.0625, gate=gate)
    finally:
        gpu_ctx.set_split_tokens(0)
        kv.close()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    want = _oracle_rows_kept(q, ks, vs, start, keep, H, KH, D, 0.0625, gate=gate)
    assert not got[17].any()
    _check(got, want, f"many tiles, few splits: D={D} {H}/{KH} bits {bits}")


@pytest.mark.parametrize("bits,D,H,KH,start,rows", [(16, 256, 16, 2, 20000, 37), (8, 128, 8, 2, 3000, 70), (16, 64, 4, 4, 100, 9)])
def test_prefill_chunk_over_index_lists_equals_the_mask_form(gpu_ctx, bits, D, H, KH, start, rows):
    # The compacted form of a chunk's selection (keepIndices / keepIndexStride / keepCounts, prefill.metal:1069-1117):
    # per row a list of key ids -- here unsorted, with a repeat, with ids the row cannot see yet and one past the
    # cache, a row with an empty list and a list as long as its stride.  The oracle's result over the listed keys,
    # and the mask form's up to the order of the additions (the lists are walked as lists: a tile's touched blocks
    # come off a plan made of them, not off rows of bytes).
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    r = np.random.default_rng(start + rows + bits)
    T = start + rows
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((rows, H * D)).astype(np.float16) for _ in range(2))
    stride = ((T + 3) // 4) * 4
    keep = np.zeros((rows, stride), np.uint8)
    index_stride = min(300, T)
    indices = r.integers(0, 2 ** 31, size=(rows, index_stride), dtype=np.int64).astype(np.uint32)  # garbage past the counts
    counts = np.zeros(rows, np.uint32)
    for t in range(rows):
        n = index_stride if t == 1 else int(r.integers(5, min(200, T)))
        ids = r.choice(T, n, replace=False).astype(np.uint32)  # some of them at or past the row's own position
        ids[0] = start + t                                      # its own key
        if n > 3:
            ids[2] = ids[1]                                     # a repeat
            ids[3] = T + 7                                      # past the cache
        r.shuffle(ids)
        if t == 4:
            n = 0
        indices[t, :n] = ids[:n]
        counts[t] = n
        seen = ids[:n][ids[:n] <= start + t]
        keep[t, seen] = 1
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    by_mask = _prefill_keep(gpu_ctx, kv, q, start, T, keep, H, 0.0625, gate=gate)
    qd, gd = _dev(q), _dev(gate)
    idx_d, cnt_d = _dev(indices.view(np.int32)), _dev(counts.view(np.int32))
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    width = H * D
    att = PrefillAttention(gpu_ctx)
    params = PrefillAttentionParams(start, rows, T, H, 0.0625, width, width, width)
    att.encode_causal(kv, 0, 0, qd, out, params, gate=gd, keep_indices=idx_d, keep_index_stride=index_stride, keep_counts=cnt_d)
    gpu_ctx.synchronize()
    by_list = out.float().cpu().numpy()
    # a second, shorter chunk through the same store (its rows are cleared again)
    out2 = torch.full((5, width), float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    att.encode_causal(kv, 0, 0, qd[:5], out2, PrefillAttentionParams(start, 5, start + 5, H, 0.0625, width, width, width),
                      gate=gd[:5], keep_indices=idx_d, keep_index_stride=index_stride, keep_counts=cnt_d)
    gpu_ctx.synchronize()
    again = out2.float().cpu().numpy()
    kv.close()
    assert np.isfinite(by_list).all() and np.abs(by_list - by_mask).max() <= 2e-3
    assert not by_list[4].any()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    want = _oracle_rows_kept(q, ks, vs, start, keep, H, KH, D, 0.0625, gate=gate)
    _check(by_list, want, f"index lists D={D} {H}/{KH} bits {bits}")
    # (a row of the shorter chunk sees the same keys: ids at or past its position were dropped in both)
    _check(again, want[:5], "index lists, second call")


@pytest.mark.parametrize("bits,split_tokens", [(16, 0), (8, 0), (16, 8192)])
def test_prefill_chunk_over_index_lists_deep_in_a_long_context(gpu_ctx, bits, split_tokens):
    # 256 rows behind 128k keys (the sparse chunk's benchmark shape), every row its own ascending list of 512 cells of
    # 4 keys plus its own block: 64 token tiles x 2 KV heads over two key ranges (or sixteen), each walking a few
    # hundred of the 4,096 key blocks.  Against the oracle on rows spread over the chunk, and against the mask form.
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    H, KH, D, rows, start = 16, 2, 256, 256, 131072 - 256
    T = start + rows
    r = np.random.default_rng(4096 + bits + split_tokens)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((rows, H * D)).astype(np.float16) for _ in range(2))
    index_stride = 2048 + 64
    indices = np.zeros((rows, index_stride), np.uint32)
    counts = np.zeros(rows, np.uint32)
    keep = np.zeros((rows, T), np.uint8)
    for t in range(rows):
        cells = np.sort(r.choice(start // 4, 512, replace=False)).astype(np.uint32)
        ids = (cells[:, None] * 4 + np.arange(4, dtype=np.uint32)[None]).reshape(-1)
        own = np.arange((start + t) & ~31, start + t + 1, dtype=np.uint32)  # its own block, up to its own key
        ids = np.concatenate([ids, own])
        indices[t, :ids.size] = ids
        counts[t] = ids.size
        keep[t, ids] = 1
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    gpu_ctx.set_split_tokens(split_tokens)
    try:
        by_mask = _prefill_keep(gpu_ctx, kv, q, start, T, keep, H, 0.0625, gate=gate)
        qd, gd = _dev(q), _dev(gate)
        idx_d, cnt_d = _dev(indices.view(np.int32)), _dev(counts.view(np.int32))
        out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        width = H * D
        PrefillAttention(gpu_ctx).encode_causal(kv, 0, 0, qd, out, PrefillAttentionParams(start, rows, T, H, 0.0625, width, width, width),
                                                gate=gd, keep_indices=idx_d, keep_index_stride=index_stride, keep_counts=cnt_d)
        gpu_ctx.synchronize()
    finally:
        gpu_ctx.set_split_tokens(0)
    by_list = out.float().cpu().numpy()
    kv.close()
    assert np.isfinite(by_list).all() and np.abs(by_list - by_mask).max() <= 2e-3
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    some = [0, 1, 2, 3, 4, 31, 32, 100, 127, 128, 200, 254, 255]
    for t in some:
        want = _oracle_rows_kept(q[t:t + 1], ks, vs, start + t, keep[t:t + 1], H, KH, D, 0.0625, gate=gate[t:t + 1])
        _check(by_list[t:t + 1], want, f"index lists at 128k keys, row {t}, bits {bits}, split {split_tokens}")


def test_prefill_chunk_over_index_lists_goes_in_pieces_of_rows_when_its_plan_is_large(gpu_ctx):
    # One head per KV head: a tile is 32 tokens, and behind 262k keys a tile's plan has room for all 8,192 key blocks
    # times 33 words -- 124 tiles fill the 128 MiB a piece may take, so 4,100 rows go as two pieces.  Random lists of
    # 40 to 300 ids per row (unsorted); the mask form is the comparison (its rows are 1.07 GB here), the oracle on a few rows.
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    H, KH, D, rows, start = 1, 1, 64, 4100, 262144 - 4100
    T = start + rows
    r = np.random.default_rng(262144)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q = r.standard_normal((rows, H * D)).astype(np.float16)
    index_stride = 300
    indices = r.integers(0, T, size=(rows, index_stride), dtype=np.int64).astype(np.uint32)
    counts = r.integers(40, index_stride + 1, size=rows).astype(np.uint32)
    indices[:, 0] = start + np.arange(rows)  # every row lists its own key
    kv = _cache(gpu_ctx, 16, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    keep_d = torch.zeros((rows, T), dtype=torch.uint8, device="cuda")
    idx_t = torch.from_numpy(indices.astype(np.int64)).cuda()
    cnt_t = torch.from_numpy(counts.astype(np.int64)).cuda()
    listed = torch.arange(index_stride, device="cuda")[None, :] < cnt_t[:, None]
    visible = idx_t <= (start + torch.arange(rows, device="cuda"))[:, None]
    rr = torch.arange(rows, device="cuda")[:, None].expand(-1, index_stride)
    sel = listed & visible
    keep_d[rr[sel], idx_t[sel]] = 1
    qd = _dev(q)
    width = H * D
    outs = []
    torch.cuda.synchronize()
    att = PrefillAttention(gpu_ctx)
    params = PrefillAttentionParams(start, rows, T, H, 0.125, width, width, width)
    for form in ("mask", "lists"):
        out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        if form == "mask":
            att.encode_causal(kv, 0, 0, qd, out, params, keep_mask=keep_d, keep_stride=T)
        else:
            att.encode_causal(kv, 0, 0, qd, out, params, keep_indices=_dev(indices.view(np.int32)), keep_index_stride=index_stride,
                              keep_counts=_dev(counts.view(np.int32)))
        gpu_ctx.synchronize()
        outs.append(out.float().cpu().numpy())
    kv.close()
    by_mask, by_list = outs
    assert np.isfinite(by_list).all() and np.abs(by_list - by_mask).max() <= 2e-3
    keep = keep_d.cpu().numpy()
    for t in (0, 31, 32, 3967, 3968, 3969, 4099):  # (3,968 rows is where the first piece ends)
        want = _oracle_rows_kept(q[t:t + 1], k, v, start + t, keep[t:t + 1], H, KH, D, 0.125)
        _check(by_list[t:t + 1], want, f"index lists in pieces, row {t}")


def test_prefill_keep_indices_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    H, KH, D, T = 8, 2, 64, 96
    kv = _cache(gpu_ctx, 16, KH, D, T)
    q = torch.zeros((16, H * D), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    idx = torch.zeros(16 * 8, dtype=torch.int32, device="cuda")
    cnt = torch.zeros(16, dtype=torch.int32, device="cuda")
    lib, h = gpu_ctx._lib, gpu_ctx.handle
    call = lambda i, stride, c, q_len=16, kv_valid=80: lib.tt_hip_attn_prefill_keep_indices(
        h, kv.handle, 0, 0, 40, q_len, kv_valid, i, stride, c, H, q.data_ptr(), H * D, None, 0, 0.125, out.data_ptr(), H * D)
    assert call(idx.data_ptr(), 8, cnt.data_ptr()) == capi.OK
    assert call(None, 8, cnt.data_ptr()) == capi.ERR_INVALID_ARGUMENT
    assert call(idx.data_ptr(), 8, None) == capi.ERR_INVALID_ARGUMENT
    assert call(idx.data_ptr(), 0, cnt.data_ptr()) == capi.ERR_SHAPE
    assert call(idx.data_ptr(), 8, cnt.data_ptr(), kv_valid=50) == capi.ERR_INVALID_ARGUMENT  # the chunk ends past the valid keys
    gpu_ctx.synchronize()
    assert not out.float().abs().sum().item()  # every list is empty: zeros
    kv.close()


@pytest.mark.parametrize("bits,lengths", [(16, [40000]), (8, [9001, 77, 5000, 1]), (16, [300, 2047])])
def test_decode_over_index_lists_equals_the_mask_form(gpu_ctx, bits, lengths):
    # DecodeKeySelection.indices / .count: per sequence a list of key ids (unsorted, a repeat, ids at or past the
    # sequence's length, an empty list) -- the same rows as the mask form, bit for bit.
    import torch
    from tinytitan_amd.engine import Attention
    H, KH, D = 16, 2, 256
    n = len(lengths)
    r = np.random.default_rng(sum(lengths) + bits)
    kv = _cache(gpu_ctx, bits, KH, D, max(lengths), slots=n)
    for i, L in enumerate(lengths):
        k, v = (r.standard_normal((L, KH, D)).astype(np.float16) for _ in range(2))
        _append(gpu_ctx, kv, 0, i, 0, k, v)
    q, gate = (r.standard_normal((n, H, D)).astype(np.float16) for _ in range(2))
    stride = (max(lengths) + 3) // 4 * 4
    keep = np.zeros((n, stride), np.uint8)
    index_stride = 2100
    indices = r.integers(0, 2 ** 31, size=(n, index_stride), dtype=np.int64).astype(np.uint32)
    counts = np.zeros(n, np.uint32)
    for i, L in enumerate(lengths):
        m = 0 if i == 1 else min(L, int(r.integers(1, 2051)))
        ids = r.choice(L, m, replace=False).astype(np.uint32)
        if m > 3:
            ids[1] = ids[0]
            ids[2] = L + 5
            ids[3] = L
        r.shuffle(ids)
        indices[i, :m] = ids
        counts[i] = m
        keep[i, ids[ids < L]] = 1
    qd, gd, kd = _dev(q), _dev(gate), _dev(keep)
    by_mask = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    by_list = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    idx_d, cnt_d = _dev(indices.view(np.int32)), _dev(counts.view(np.int32))
    torch.cuda.synchronize()
    att = Attention(gpu_ctx)
    att.encode_full_keep(kv, 0, qd, by_mask, H, lengths, kd, 0.0625, slot=list(range(n)), gate=gd, keep_stride=stride)
    att.encode_full_keep_indices(kv, 0, qd, by_list, H, lengths, idx_d, cnt_d, 0.0625, slot=list(range(n)), gate=gd)
    gpu_ctx.synchronize()
    kv.close()
    a, b = by_mask.float().cpu().numpy(), by_list.float().cpu().numpy()
    assert np.isfinite(b).all() and np.array_equal(a, b)
    if n > 1:
        assert not b[1].any()


def test_index_lists_inside_a_graph_capture():
    # The rows the lists are written out to live in a store the context owns: it cannot grow inside a capture
    # (BUSY, and the capture survives), and once it is large enough the call is captured and replays.
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, HIPContext, TinyTitanHIPError
    ctx = HIPContext(0)
    H, KH, D, L = 8, 2, 128, 5000
    r = np.random.default_rng(5)
    kv = _cache(ctx, 16, KH, D, L)
    k, v = (r.standard_normal((L, KH, D)).astype(np.float16) for _ in range(2))
    _append(ctx, kv, 0, 0, 0, k, v)
    ids = np.sort(r.choice(L, 700, replace=False)).astype(np.int32)
    keep = np.zeros((1, L + (-L) % 4), np.uint8)
    keep[0, ids] = 1
    qd = _dev(r.standard_normal((1, H, D)).astype(np.float16))
    idx_d, cnt_d, kd = _dev(ids[None]), _dev(np.array([700], np.int32)), _dev(keep)
    want = torch.zeros_like(qd)
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    att = Attention(ctx)
    att.encode_full_keep(kv, 0, qd, want, H, [L], kd, 0.09, keep_stride=keep.shape[1])
    ctx.synchronize()
    ctx.graph_begin()
    with pytest.raises(TinyTitanHIPError) as e:
        att.encode_full_keep_indices(kv, 0, qd, out, H, [L], idx_d, cnt_d, 0.09)
    assert e.value.status == capi.ERR_BUSY
    graph = ctx.graph_end()
    graph.close()
    att.encode_full_keep_indices(kv, 0, qd, out, H, [L], idx_d, cnt_d, 0.09)  # eager: the store grows
    ctx.synchronize()
    assert torch.equal(out, want)
    ctx.graph_begin()
    att.encode_full_keep_indices(kv, 0, qd, out, H, [L], idx_d, cnt_d, 0.09)
    graph = ctx.graph_end()
    for replay in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.launch()
        ctx.synchronize()
        assert torch.equal(out, want), f"replay {replay}"
    graph.close()
    kv.close()
    ctx.close()


def test_prefill_full_selection_is_the_plain_chunk(gpu_ctx):
    from tests.test_gpu_attention_api import _prefill
    H, KH, D, start, rows = 16, 2, 256, 130, 50  # a chunk the plain call also sends through the split-K tiles
    r = np.random.default_rng(9)
    T = start + rows
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q = r.standard_normal((rows, H * D)).astype(np.float16)
    kv = _cache(gpu_ctx, 16, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    plain = _prefill(gpu_ctx, kv, q, start, rows, T, H, 0.0625)
    kept = _prefill_keep(gpu_ctx, kv, q, start, T, np.ones((rows, T), np.uint8), H, 0.0625)
    kv.close()
    assert np.abs(kept - plain).max() <= 2.0 ** -10 * np.abs(plain).max()  # the plain call may take the chunk kernel


def test_prefill_keep_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    H, KH, D, T = 8, 2, 64, 96
    kv = _cache(gpu_ctx, 16, KH, D, T)
    q = torch.zeros((16, H * D), dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    keep = torch.ones(16 * 128, dtype=torch.uint8, device="cuda")
    lib, h = gpu_ctx._lib, gpu_ctx.handle
    call = lambda mask, stride: lib.tt_hip_attn_prefill_keep(h, kv.handle, 0, 0, 40, 16, 80, mask, stride, H, q.data_ptr(), H * D, None, 0,
                                                             0.125, out.data_ptr(), H * D)
    assert call(None, 128) == capi.ERR_INVALID_ARGUMENT
    assert call(keep.data_ptr(), 52) == capi.ERR_SHAPE         # a row shorter than the positions the chunk sees (56)
    assert call(keep.data_ptr(), 58) == capi.ERR_SHAPE         # rows are read a word at a time
    assert call(keep.data_ptr() + 2, 128) == capi.ERR_SHAPE
    assert call(keep.data_ptr(), 128) == capi.OK
    gpu_ctx.synchronize()
    kv.close()


# ---- the compacted form: gather the selected rows, attend densely ----------------------------------

@pytest.mark.parametrize("bits,ring", [(16, 0), (8, 0), (4, 0), (16, 512)])
def test_gathered_selection_equals_the_masked_decode(gpu_ctx, bits, ring):
    # DecodeKeySelection.indices / count: the selected rows gathered into a scratch cache and attended over as
    # `count` keys give what the mask form gives over the whole context (same rows: a quantised cache hands out
    # level * scale + bias, which is what its attention kernels multiply)
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, T = 16, 2, 256, 3000 if not ring else 400
    r = np.random.default_rng(50 + bits + ring)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((1, 1, H, D)).astype(np.float16) for _ in range(2))
    keep = (r.random(T) < 0.15).astype(np.uint8)
    keep[T - 1] = 1
    indices = np.flatnonzero(keep).astype(np.int32)
    if ring:
        kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=4096, ring_capacity=ring, precision_bits=bits)
    else:
        kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    masked = _decode_keep(gpu_ctx, kv, q, [T], keep, H, 0.0625, gate=gate)
    n = len(indices)
    scratch = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=n + 32, initial_capacity=n + 32)
    kd = torch.full((n, KH * D + 8), 9.0, dtype=torch.float16, device="cuda")  # padded rows: the stride is honoured
    vd = torch.full_like(kd, 9.0)
    pos = _dev(indices)
    bad = _dev(np.array([-1, 10 ** 6, int(indices[3])], dtype=np.int32))  # outside the cache: zero rows
    kb = torch.full((3, KH * D), 5.0, dtype=torch.float16, device="cuda")
    vb = torch.full_like(kb, 5.0)
    torch.cuda.synchronize()
    kv.gather(0, 0, pos, kd, vd)
    kv.gather(0, 0, bad, kb, vb)
    gpu_ctx.synchronize()
    rows_k, rows_v = kv.read(0, 0, 0, T)
    assert torch.equal(kd[:, :KH * D], rows_k.reshape(T, -1)[torch.from_numpy(indices).cuda().long()])
    assert torch.equal(vd[:, :KH * D], rows_v.reshape(T, -1)[torch.from_numpy(indices).cuda().long()])
    assert (kd[:, KH * D:] == 9.0).all() and (vd[:, KH * D:] == 9.0).all()
    assert not kb[:2].any() and not vb[:2].any() and torch.equal(kb[2], kd[3, :KH * D])
    scratch.append(0, 0, 0, kd[:, :KH * D].contiguous(), vd[:, :KH * D].contiguous())
    gpu_ctx.synchronize()
    qd, gd = _dev(q), _dev(gate)
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_full(scratch, 0, qd, out, H, [n], 0.0625, gate=gd)
    gpu_ctx.synchronize()
    dense = out.float().cpu().numpy()
    scratch.close()
    kv.close()
    ks, vs = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    want = _oracle_kept(q[0, 0], ks, vs, keep, H, KH, D, 0.0625, gate=gate[0, 0])
    _check(dense[0, 0], want, f"gathered selection, bits {bits}")
    _check(masked[0, 0], want, f"masked selection, bits {bits}")
    assert np.abs(dense - masked).max() <= 2e-3


def _indexer_shaped(r, n, blocks_kept, ratio=4):
    """A selection as the block indexer makes it: random complete blocks of `ratio` keys and the query's own tail."""
    keep = np.zeros(n, np.uint8)
    chosen = r.choice(n // ratio - 1, size=blocks_kept, replace=False)
    keep[(chosen[:, None] * ratio + np.arange(ratio)[None, :]).ravel()] = 1
    keep[n // ratio * ratio - ratio:] = 1
    return keep


@pytest.mark.parametrize("bits", [16, 8])
@pytest.mark.parametrize("offset", [0, 1])
def test_long_context_walks_only_the_touched_blocks(gpu_ctx, bits, offset):
    # 140,000 keys: splits of nine blocks a wavefront, where a wavefront finds its touched blocks up front and walks
    # only those (offset 0: the mask starts on a word boundary) or tests block by block (offset 1); most wavefronts
    # have no touched block but their first, whole splits have none
    import torch
    H, KH, D, T = 16, 2, 256, 140000
    r = np.random.default_rng(60 + bits)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((1, 1, H, D)).astype(np.float16) for _ in range(2))
    keep = _indexer_shaped(r, T, 512)
    keep[30000:90000] = 0  # a long stretch without a kept key
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    from tinytitan_amd.engine import Attention
    qd, gd = _dev(q), _dev(gate)
    held = torch.zeros(T + 8, dtype=torch.uint8, device="cuda")
    held[offset:offset + T] = torch.from_numpy(keep).cuda()
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_full_keep(kv, 0, qd, out, H, [T], held[offset:offset + T], 0.0625, slot=[0], gate=gd)
    gpu_ctx.synchronize()
    got = out.float().cpu().numpy()[0, 0]
    kv.close()
    kk, vv = (k, v) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    _check(got, _oracle_kept(q[0, 0], kk, vv, keep, H, KH, D, 0.0625, gate=gate[0, 0]), f"140k keys, {bits}-bit cache, offset {offset}")


def test_many_long_sequences_keep_a_split_to_64_blocks_a_wavefront(gpu_ctx):
    # 16 sequences of 70,000 keys on two KV heads: 32 (sequence, tile) pairs share the chip, 8 splits each, which
    # would be 8,832 keys (69 blocks a wavefront); the word of blocks a wavefront walks holds 64, so the host
    # shortens the splits
    H, KH, D, T, S = 8, 2, 64, 70000, 16
    r = np.random.default_rng(61)
    kv = _cache(gpu_ctx, 16, KH, D, T, slots=S)
    rows, masks = [], np.zeros((S, T), np.uint8)
    for i in range(S):
        k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
        _append(gpu_ctx, kv, 0, i, 0, k, v)
        masks[i] = _indexer_shaped(r, T, 64 + 8 * i)
        rows.append((k, v))
    q = r.standard_normal((S, 1, H, D)).astype(np.float16)
    got = _decode_keep(gpu_ctx, kv, q, [T] * S, masks, H, 0.125, keep_stride=T)
    kv.close()
    for i, (k, v) in enumerate(rows):
        _check(got[i, 0], _oracle_kept(q[i, 0], k, v, masks[i], H, KH, D, 0.125), f"sequence {i}")


def _tail_only(r, n, blocks_kept):
    """Random complete blocks of 4 keys well before the end; in the last 32-key block only the keys of the mask's
    last, partial 4-byte word."""
    keep = np.zeros(n, np.uint8)
    chosen = r.choice((n - 64) // 4, size=blocks_kept, replace=False)
    keep[(chosen[:, None] * 4 + np.arange(4)[None, :]).ravel()] = 1
    keep[(n - 1) // 32 * 32:] = 0
    keep[n // 4 * 4:] = 1
    assert keep[n // 4 * 4:].size == n % 4
    return keep


@pytest.mark.parametrize("T", [140001, 140002, 140003])
def test_word_path_keeps_the_tail_of_a_length_that_is_not_a_multiple_of_four(gpu_ctx, T):
    # The wavefronts read their blocks' mask bytes as words (splits of nine blocks a wavefront); the mask is exactly
    # T bytes, so its last word straddles the end.  The only kept keys of the last block sit in that word, and the
    # last block is not its wavefront's first.
    import torch
    H, KH, D = 16, 2, 64
    r = np.random.default_rng(T)
    k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
    q = r.standard_normal((1, 1, H, D)).astype(np.float16)
    keep = _tail_only(r, T, 300)
    kv = _cache(gpu_ctx, 16, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    from tinytitan_amd.engine import Attention
    qd = _dev(q)
    held = torch.from_numpy(keep).cuda()  # exactly T bytes
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_full_keep(kv, 0, qd, out, H, [T], held, 0.125, slot=[0])
    gpu_ctx.synchronize()
    got = out.float().cpu().numpy()[0, 0]
    kv.close()
    _check(got, _oracle_kept(q[0, 0], k, v, keep, H, KH, D, 0.125), f"{T} keys, tail word only")


@pytest.mark.parametrize("T", [9001, 9002, 9003])
def test_word_path_keeps_the_tails_of_batched_sequences(gpu_ctx, T):
    # 16 sequences of equal length on two KV heads: 8 splits of 36 blocks each, read as words; every sequence's
    # last block holds kept keys only in the mask's last, partial word
    H, KH, D, S = 8, 2, 64, 16
    r = np.random.default_rng(T)
    stride = (T + 3) // 4 * 4
    kv = _cache(gpu_ctx, 16, KH, D, T, slots=S)
    rows, masks = [], np.zeros((S, stride), np.uint8)
    for i in range(S):
        k, v = (r.standard_normal((T, KH, D)).astype(np.float16) for _ in range(2))
        _append(gpu_ctx, kv, 0, i, 0, k, v)
        masks[i, :T] = _tail_only(r, T, 20 + i)
        rows.append((k, v))
    q = r.standard_normal((S, 1, H, D)).astype(np.float16)
    got = _decode_keep(gpu_ctx, kv, q, [T] * S, masks, H, 0.125, keep_stride=stride)
    kv.close()
    for i, (k, v) in enumerate(rows):
        _check(got[i, 0], _oracle_kept(q[i, 0], k, v, masks[i, :T], H, KH, D, 0.125), f"sequence {i} of {T} keys")
