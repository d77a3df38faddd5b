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
