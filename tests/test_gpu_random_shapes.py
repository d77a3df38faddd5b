"""Seeded sweep over head counts, head dims, chunk positions and lengths: the prefill kernel (and
the split-K kernel behind it for head groups it does not serve), a decode and a verify over the same
cache, each against the oracle at the attention bar.  Seeds 24-35 run over 8- and 4-bit caches (the
oracle then attends over the rows its own quantiser and loader give); seeds 36-47 add a sliding
window to the prefill chunk and the decode, over caches of all three precisions."""
import numpy as np
import pytest

import oracle
from tests.helpers import MAX_ABS, MEAN_ABS, f16_round

pytestmark = pytest.mark.gpu


def _close(got, want, what):
    diff = np.abs(got.astype(np.float64) - f16_round(want.astype(np.float32)).astype(np.float64))
    assert np.isfinite(got).all(), what
    assert diff.max() <= MAX_ABS and diff.mean() <= MEAN_ABS, f"{what}: max-abs {diff.max():.3e} mean-abs {diff.mean():.3e}"


@pytest.mark.parametrize("seed", range(48))
def test_random_shape(gpu_ctx, seed):
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager, PrefillAttention, PrefillAttentionParams
    rng = np.random.default_rng(1000 + seed)
    D = int(rng.choice([64, 128, 256]))
    KH = int(rng.choice([1, 2, 4]))
    H = KH * int(rng.choice([1, 2, 4, 8]))
    start, q_len, extra = int(rng.integers(0, 300)), int(rng.integers(1, 260)), int(rng.integers(0, 40))
    kv_valid = start + q_len + extra  # rows still see only their causal prefix
    gated = bool(rng.integers(0, 2))
    scale = float(1.0 / np.sqrt(D))
    k = rng.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = rng.standard_normal((kv_valid, KH, D)).astype(np.float16)
    q = rng.standard_normal((q_len, H * D)).astype(np.float16)
    g = rng.standard_normal((q_len, H * D)).astype(np.float16) if gated else None
    cap = ((kv_valid + 31) // 32) * 32 + int(rng.choice([0, 32, 64]))
    bits = 16 if seed < 24 else (8, 4, 16)[seed % 3 if seed >= 36 else seed % 2]  # the first 24 seeds keep their shapes
    window = int(rng.integers(1, 200)) if seed >= 36 else 0
    what = f"D{D} {H}q/{KH}kv start {start} rows {q_len} valid {kv_valid} gate {gated} bits {bits} window {window}"
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=cap, initial_capacity=cap, precision_bits=bits)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    kd, vd = dev(k), dev(v)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    gpu_ctx.synchronize()
    kv.advance(0, kv_valid)
    k32, v32 = k.astype(np.float32).reshape(kv_valid, -1), v.astype(np.float32).reshape(kv_valid, -1)
    if bits != 16:
        k32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(k32, bits), KH * D, bits)
        v32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(v32, bits), KH * D, bits)

    qd, gd = dev(q), dev(g) if gated else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    PrefillAttention(gpu_ctx).encode_causal(kv, 0, 0, qd, out, PrefillAttentionParams(start, q_len, kv_valid, H, scale, H * D,
                                                                                     H * D, H * D, sliding_window=window), gate=gd)
    gpu_ctx.synchronize()
    want = oracle.prefill_ref(q.astype(np.float32), k32, v32, H * D, KH * D, D, H, KH, start, q_len, kv_valid, window,
                              scale).reshape(q_len, -1)
    if gated:
        want = want / (1 + np.exp(-g.astype(np.float64)))
    _close(out.float().cpu().numpy(), want, "prefill " + what)

    L = int(rng.integers(1, kv_valid + 1))
    q1 = dev(q[:1].reshape(1, 1, H, D))
    o1 = torch.empty_like(q1)
    torch.cuda.synchronize()
    if window:
        Attention(gpu_ctx).encode_swa(kv, 0, q1, o1, H, L, window, scale)
    else:
        Attention(gpu_ctx).encode_full(kv, 0, q1, o1, H, L, scale)
    gpu_ctx.synchronize()
    first = max(0, L - window) if window else 0
    _close(o1.float().cpu().numpy().reshape(H, D),
           oracle.decode(q[0].astype(np.float32), k32[first:L], v32[first:L], H, KH, D, scale), f"decode over {L} keys, " + what)

    rows = int(rng.integers(1, min(5, kv_valid) + 1))
    s0 = int(rng.integers(0, kv_valid - rows + 1))
    qv = dev(q[:rows].reshape(1, rows, H, D))
    ov = torch.empty_like(qv)
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qv, ov, H, [s0], rows, scale, [0])
    gpu_ctx.synchronize()
    want = oracle.attention_batch(q[:rows].astype(np.float32), k32[:s0 + rows], v32[:s0 + rows], rows, s0, H, KH, D, scale)
    _close(ov.float().cpu().numpy().reshape(rows, -1), want.reshape(rows, -1), f"verify {rows} rows at {s0}, " + what)
    kv.close()


@pytest.mark.parametrize("seed", range(32))
def test_random_shape_with_selections(gpu_ctx, seed):
    """The same sweep over sparse key selections: a chunk with one selection per query row in both of its forms
    (rows of bytes; index lists) and a decode with one, over caches of all three precisions and split lengths from
    the planner's own down to 128 keys."""
    import torch
    from tests.test_gpu_keep_mask import _oracle_kept, _oracle_rows_kept
    from tinytitan_amd.engine import Attention, KVCacheManager, PrefillAttention, PrefillAttentionParams
    rng = np.random.default_rng(5000 + seed)
    D = int(rng.choice([64, 128, 256]))
    KH = int(rng.choice([1, 2, 4]))
    H = KH * int(rng.choice([1, 2, 4, 8]))
    deep = seed >= 16  # the second half: deep in a long context, where a tile's workgroup lists the blocks it touches
    start, q_len = int(rng.integers(8000, 24000) if deep else rng.integers(0, 3000)), int(rng.integers(1, 90))
    kv_valid = start + q_len
    gated = bool(rng.integers(0, 2))
    bits = (16, 8, 4)[seed % 3]
    fraction = float(rng.choice([0.005, 0.05, 0.2] if deep else [0.02, 0.2, 0.7]))
    split_tokens = int(rng.choice([0, 4096, 32768] if deep else [0, 128, 1024]))
    scale = float(1.0 / np.sqrt(D))
    what = f"D{D} {H}q/{KH}kv start {start} rows {q_len} gate {gated} bits {bits} kept {fraction} split {split_tokens}"
    k = rng.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = rng.standard_normal((kv_valid, KH, D)).astype(np.float16)
    q = rng.standard_normal((q_len, H * D)).astype(np.float16)
    g = rng.standard_normal((q_len, H * D)).astype(np.float16) if gated else None
    stride = (kv_valid + 3) // 4 * 4
    keep = (rng.random((q_len, stride)) < fraction).astype(np.uint8)
    keep[:, kv_valid:] = 0
    if q_len > 2:
        keep[q_len // 2] = 0  # a row that keeps nothing
    counts = np.array([int(keep[t, :start + t + 1].sum()) for t in range(q_len)], np.uint32)
    width = max(1, int(counts.max()))
    indices = np.full((q_len, width), 0x7fffffff, np.uint32)
    for t in range(q_len):
        ids = np.flatnonzero(keep[t, :start + t + 1]).astype(np.uint32)
        rng.shuffle(ids)
        indices[t, :len(ids)] = ids
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=kv_valid + 32, initial_capacity=kv_valid + 32, precision_bits=bits)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    kd, vd = dev(k), dev(v)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    gpu_ctx.synchronize()
    k32, v32 = k.astype(np.float32).reshape(kv_valid, -1), v.astype(np.float32).reshape(kv_valid, -1)
    if bits != 16:
        k32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(k32, bits), KH * D, bits)
        v32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(v32, bits), KH * D, bits)
    k3, v3 = k32.reshape(kv_valid, KH, D), v32.reshape(kv_valid, KH, D)
    qd, gd = dev(q), dev(g) if gated else None
    by_mask = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    by_list = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    keep_d, idx_d, cnt_d = dev(keep), dev(indices.view(np.int32)), dev(counts.view(np.int32))
    params = PrefillAttentionParams(start, q_len, kv_valid, H, scale, H * D, H * D, H * D)
    att = PrefillAttention(gpu_ctx)
    gpu_ctx.set_split_tokens(split_tokens)
    try:
        torch.cuda.synchronize()
        att.encode_causal(kv, 0, 0, qd, by_mask, params, gate=gd, keep_mask=keep_d, keep_stride=stride)
        att.encode_causal(kv, 0, 0, qd, by_list, params, gate=gd, keep_indices=idx_d, keep_index_stride=width, keep_counts=cnt_d)
        gpu_ctx.synchronize()
        want = _oracle_rows_kept(q, k3, v3, start, keep, H, KH, D, scale, gate=g)
        _close(by_mask.float().cpu().numpy(), want, "chunk, mask form, " + what)
        # (the lists are walked as lists: the same keys, dealt to the wavefronts in another order than the mask form's)
        _close(by_list.float().cpu().numpy(), want, "chunk, index lists, " + what)
        assert (by_list.float() - by_mask.float()).abs().max().item() <= 2e-3, "chunk, index lists against the mask form, " + what

        L = int(rng.integers(1, kv_valid + 1))
        row = (rng.random(stride) < fraction).astype(np.uint8)
        row[L - 1] = 1
        q1 = dev(q[:1].reshape(1, 1, H, D))
        o1 = torch.full(q1.shape, float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        Attention(gpu_ctx).encode_full_keep(kv, 0, q1, o1, H, L, dev(row[None]), scale, keep_stride=stride)
        gpu_ctx.synchronize()
        want1 = _oracle_kept(q[0].reshape(H, D), k3[:L], v3[:L], row[:L], H, KH, D, scale)
        _close(o1.float().cpu().numpy().reshape(H, D), want1.reshape(H, D), f"decode over {L} keys with a selection, " + what)
    finally:
        gpu_ctx.set_split_tokens(0)
        kv.close()
