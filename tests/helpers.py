"""Shared helpers of the parity tests: run a workload through the C ABI and through the oracle."""
from __future__ import annotations

import numpy as np

MAX_ABS = 2e-3   # parity bar: max |gpu - oracle| after both are rounded to fp16
MEAN_ABS = 2e-4  # parity bar: mean |gpu - oracle|


def f16_round(x: np.ndarray) -> np.ndarray:
    return x.astype(np.float16).astype(np.float32)


def oracle_workload(w, threads: int = 1):
    """Oracle outputs per sequence, fp16-rounded: decode via a1, multi-row via a3."""
    import oracle
    outs = []
    for s in w.sequences:
        k = s.k.astype(np.float32).reshape(s.k.shape[0], -1)
        v = s.v.astype(np.float32).reshape(s.v.shape[0], -1)
        q = s.q.astype(np.float32)
        g = s.gate.astype(np.float32) if s.gate is not None else None
        rows = q.shape[0]
        if w.kind == "decode":
            o = oracle.decode(q[0], k, v, w.heads, w.kv_heads, w.dim, w.scale, gate=g[0] if g is not None else None)[None]
        else:
            positions = s.start + rows
            o = oracle.attention_batch(q.reshape(rows, -1), k[:positions], v[:positions], rows, s.start, w.heads,
                                       w.kv_heads, w.dim, w.scale, gate=g.reshape(rows, -1) if g is not None else None,
                                       threads=threads)
        outs.append(f16_round(o))
    return outs


def gpu_workload(ctx, w, layers: int = 1, layer: int = 0, capacity=None, split_tokens: int = 0):
    """Runs a synthetic Workload through the C ABI; returns per-sequence fp32 arrays [rows][heads][dim]."""
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager, PrefillAttention, PrefillAttentionParams
    dev = torch.device("cuda", ctx.device)
    n = len(w.sequences)
    longest = max(s.k.shape[0] for s in w.sequences)
    cap = capacity or max(32, longest)
    kv = KVCacheManager(ctx, layers, w.kv_heads, w.dim, slots=n, max_context=max(cap, longest), initial_capacity=cap)
    try:
        kv.reserve(longest)
        for i, s in enumerate(w.sequences):
            kd = torch.from_numpy(s.k).to(dev)
            vd = torch.from_numpy(s.v).to(dev)
            torch.cuda.synchronize(dev)
            kv.append(layer, i, 0, kd, vd)
            ctx.synchronize()
            kv.advance(i, s.k.shape[0])
        ctx.set_split_tokens(split_tokens)
        rows = w.sequences[0].q.shape[0]
        q = torch.from_numpy(np.stack([s.q for s in w.sequences])).to(dev)
        gate = None
        if w.sequences[0].gate is not None:
            gate = torch.from_numpy(np.stack([s.gate for s in w.sequences])).to(dev)
        out = torch.full(q.shape, float("nan"), dtype=torch.float16, device=dev)
        torch.cuda.synchronize(dev)
        if w.kind == "decode":
            Attention(ctx).encode_full(kv, layer, q, out, w.heads, [s.k.shape[0] for s in w.sequences], w.scale,
                                       slot=list(range(n)), gate=gate)
        elif w.kind == "verify":
            Attention(ctx).encode_verify_rows(kv, layer, q, out, w.heads, [s.start for s in w.sequences], rows,
                                              w.scale, list(range(n)), gate=gate)
        else:
            assert n == 1
            s = w.sequences[0]
            width = w.heads * w.dim
            PrefillAttention(ctx).encode_causal(
                kv, layer, 0, q, out,
                PrefillAttentionParams(s.start, rows, s.start + rows, w.heads, w.scale, width, width, width), gate=gate)
        ctx.synchronize()
        ctx.set_split_tokens(0)
        res = out.float().cpu().numpy()
        return [res[i] for i in range(n)]
    finally:
        kv.close()


def assert_parity(gpu, ref, what: str = ""):
    worst, total, count = 0.0, 0.0, 0
    for a, b in zip(gpu, ref):
        assert a.shape == b.shape, (a.shape, b.shape)
        assert np.isfinite(a).all(), f"{what}: non-finite GPU output"
        diff = np.abs(a.astype(np.float64) - b.astype(np.float64))
        worst = max(worst, float(diff.max()))
        total += float(diff.sum())
        count += diff.size
    mean = total / max(count, 1)
    assert worst <= MAX_ABS, f"{what}: max-abs {worst:.3e} > {MAX_ABS}"
    assert mean <= MEAN_ABS, f"{what}: mean-abs {mean:.3e} > {MEAN_ABS}"
    return worst, mean
