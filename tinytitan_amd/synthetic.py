"""Seeded synthetic inputs for the five benchmark configurations.

The stream is the reference's test PRNG -- SplitMix64 seeded through
``SeedTree.key(label)`` (sources/TinyTitanValidation/Support/PRNG/
SplitMix64.swift:11-23, SeedTree.swift:12-19) -- vectorised in numpy, with a
Box-Muller transform on top for the N(0,1) draws the configurations ask for
(the reference's own kernel tests draw uniform(-0.5, 0.5); both are offered).
Every tensor is rounded to fp16 once, here, so the GPU path and any checker
see identical bits.

Layouts are the caller's: queries ``[rows][heads][dim]`` and token-major K/V
rows ``[positions][kv_heads][dim]`` (1024 B per token for 2 x 256 fp16, as in
tests/TinyTitan/Runtime/KVCache/KVCacheManagerTests.swift:105-115).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

_MASK = np.uint64(0xFFFFFFFFFFFFFFFF)
_GAMMA = 0x9E3779B97F4A7C15


def fnv1a64(label: str) -> int:
    h = 0xCBF29CE484222325
    for byte in label.encode("utf-8"):
        h ^= byte
        h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def seed_key(root: int, label: str) -> int:
    """``SeedTree(root).key(label)``: the child stream's SplitMix64 seed."""
    return (root ^ fnv1a64(label)) & 0xFFFFFFFFFFFFFFFF


def splitmix64(seed: int, count: int, offset: int = 0) -> np.ndarray:
    """Outputs ``offset .. offset+count-1`` of the SplitMix64 stream seeded with ``seed``."""
    with np.errstate(over="ignore"):
        index = np.arange(offset + 1, offset + count + 1, dtype=np.uint64)
        z = np.uint64(seed) + index * np.uint64(_GAMMA)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform(root: int, label: str, count: int, lo: float = -0.5, hi: float = 0.5) -> np.ndarray:
    """``SplitMix64.uniform(lo, hi)`` drawn ``count`` times (24-bit mantissa)."""
    raw = splitmix64(seed_key(root, label), count)
    u = (raw >> np.uint64(40)).astype(np.float32) / np.float32(1 << 24)
    return (np.float32(lo) + (np.float32(hi) - np.float32(lo)) * u).astype(np.float32)


def normal(root: int, label: str, count: int, chunk: int = 1 << 22) -> np.ndarray:
    """N(0,1) draws: Box-Muller over consecutive pairs of 24-bit uniforms of one stream."""
    seed = seed_key(root, label)
    out = np.empty(count, dtype=np.float32)
    done = 0
    while done < count:
        n = min(chunk, count - done)
        pairs = (n + 1) // 2
        raw = splitmix64(seed, 2 * pairs, offset=2 * (done // 2))
        u1 = ((raw[0::2] >> np.uint64(40)).astype(np.float64) + 1.0) / float(1 << 24)  # (0, 1]
        u2 = (raw[1::2] >> np.uint64(40)).astype(np.float64) / float(1 << 24)  # [0, 1)
        radius = np.sqrt(-2.0 * np.log(u1))
        z = np.empty(2 * pairs, dtype=np.float64)
        z[0::2] = radius * np.cos(2.0 * np.pi * u2)
        z[1::2] = radius * np.sin(2.0 * np.pi * u2)
        out[done:done + n] = z[:n].astype(np.float32)
        done += n
        assert done % 2 == 0 or done == count
    return out


def rope_neox_rows(rows: np.ndarray, positions: np.ndarray, rotary_dim: int, theta: float) -> np.ndarray:
    """NeoX half-split rotation of the first ``rotary_dim`` dims of every head.

    ``rows`` is ``[tokens][heads][dim]`` fp32, ``positions`` ``[tokens]``.  Pairs
    ``(i, i + rotary_dim/2)``, frequency ``theta**(-2i/rotary_dim)``, angle =
    position * frequency in fp32 (sources/TinyTitan/CPUEngine/CPUTensorOps.swift:120-139).
    """
    half = rotary_dim // 2
    idx = np.arange(half, dtype=np.float32)
    exponent = (-idx * np.float32(2.0) / np.float32(rotary_dim)).astype(np.float32)
    freq = np.power(np.float64(np.float32(theta)), exponent.astype(np.float64)).astype(np.float32)  # powf, rounded once
    angle = (positions.astype(np.float32)[:, None] * freq[None, :]).astype(np.float32)
    cos = np.cos(angle).astype(np.float32)[:, None, :]
    sin = np.sin(angle).astype(np.float32)[:, None, :]
    out = rows.astype(np.float32).copy()
    a = rows[..., :half].astype(np.float32)
    b = rows[..., half:rotary_dim].astype(np.float32)
    out[..., :half] = a * cos - b * sin
    out[..., half:rotary_dim] = a * sin + b * cos
    return out


@dataclass
class Sequence:
    """One sequence's tensors, all fp16 and in the caller's token-major layout."""
    k: np.ndarray  # [positions][kv_heads][dim]
    v: np.ndarray
    q: np.ndarray  # [rows][heads][dim]; rows = 1 for decode
    gate: Optional[np.ndarray]  # like q, or None
    start: int  # absolute position of q row 0 (row r sees keys < start + r + 1)


@dataclass
class Workload:
    name: str
    kind: str  # "decode" | "prefill" | "verify"
    heads: int
    kv_heads: int
    dim: int
    scale: float
    sequences: List[Sequence] = field(default_factory=list)
    note: str = ""

    @property
    def kv_bytes(self) -> int:
        """Algorithmic KV bytes: every cached K and V row read exactly once per sequence."""
        return sum(s.k.shape[0] * self.kv_heads * self.dim * 2 * 2 for s in self.sequences)

    @property
    def flops(self) -> int:
        """4 * dim * heads * (visible query-key pairs)."""
        pairs = 0
        for s in self.sequences:
            rows = s.q.shape[0]
            pairs += sum(min(s.k.shape[0], s.start + r + 1) for r in range(rows))
        return 4 * self.dim * self.heads * pairs


SEEDS: Dict[str, int] = {"C1": 0xC1, "C2": 0xC2, "C3": 0xC3, "C4": 0xC4, "C5": 0xC5}
ROPE_THETA = 1.0e7
ROTARY_DIM = 64


def _draw(root: int, label: str, shape, dist: str) -> np.ndarray:
    count = int(np.prod(shape))
    raw = normal(root, label, count) if dist == "normal" else uniform(root, label, count)
    return raw.reshape(shape)


def decode_c1(context: int = 2048, dist: str = "normal") -> Workload:
    """C1: batch 1, 8 q heads / 2 KV heads, dim 256, context 2048, no gate."""
    root, H, KH, D = SEEDS["C1"], 8, 2, 256
    w = Workload("C1", "decode", H, KH, D, 1.0 / 16.0)
    w.sequences.append(Sequence(
        k=_draw(root, "k", (context, KH, D), dist).astype(np.float16),
        v=_draw(root, "v", (context, KH, D), dist).astype(np.float16),
        q=_draw(root, "q", (1, H, D), dist).astype(np.float16),
        gate=None, start=context - 1))
    return w


def decode_c2(context: int = 32768, dist: str = "normal") -> Workload:
    """C2: batch 1, 16/2/256, context 32768, K rotated (NeoX, 64 dims, theta 1e7) at its row index, gated."""
    root, H, KH, D = SEEDS["C2"], 16, 2, 256
    w = Workload("C2", "decode", H, KH, D, 1.0 / 16.0)
    k = _draw(root, "k", (context, KH, D), dist)
    k = rope_neox_rows(k, np.arange(context), ROTARY_DIM, ROPE_THETA)
    w.sequences.append(Sequence(
        k=k.astype(np.float16),
        v=_draw(root, "v", (context, KH, D), dist).astype(np.float16),
        q=_draw(root, "q", (1, H, D), dist).astype(np.float16),
        gate=_draw(root, "gate", (1, H, D), dist).astype(np.float16),
        start=context - 1))
    return w


def c3_lengths(n_seq: int = 32, lo: int = 512, hi: int = 16384) -> List[int]:
    """Per-sequence context lengths: lo + next() mod (hi - lo + 1) on the ``lengths`` stream."""
    raw = splitmix64(seed_key(SEEDS["C3"], "lengths"), n_seq)
    return [int(lo + int(x) % (hi - lo + 1)) for x in raw]


def decode_c3(n_seq: int = 32, lo: int = 512, hi: int = 16384, dist: str = "normal") -> Workload:
    """C3: 32 sequences, 16/2/256, lengths uniform in [512, 16384], one query token each, no gate."""
    root, H, KH, D = SEEDS["C3"], 16, 2, 256
    w = Workload("C3", "decode", H, KH, D, 1.0 / 16.0)
    for i, length in enumerate(c3_lengths(n_seq, lo, hi)):
        w.sequences.append(Sequence(
            k=_draw(root, f"k{i}", (length, KH, D), dist).astype(np.float16),
            v=_draw(root, f"v{i}", (length, KH, D), dist).astype(np.float16),
            q=_draw(root, f"q{i}", (1, H, D), dist).astype(np.float16),
            gate=None, start=length - 1))
    return w


def prefill_c4(tokens: int = 4096, start: int = 0, dist: str = "normal") -> Workload:
    """C4: one causal chunk of 4096 tokens from position 0, 16/2/256, no gate."""
    root, H, KH, D = SEEDS["C4"], 16, 2, 256
    w = Workload("C4", "prefill", H, KH, D, 1.0 / 16.0)
    w.sequences.append(Sequence(
        k=_draw(root, "k", (start + tokens, KH, D), dist).astype(np.float16),
        v=_draw(root, "v", (start + tokens, KH, D), dist).astype(np.float16),
        q=_draw(root, "q", (tokens, H, D), dist).astype(np.float16),
        gate=None, start=start))
    return w


def verify_c5(n_seq: int = 8, context: int = 65536, rows: int = 4, dist: str = "normal") -> Workload:
    """C5: 8 sequences x 4 draft rows over a 65536-token cache plus their own 4 rows, 16/2/256, gated."""
    root, H, KH, D = SEEDS["C5"], 16, 2, 256
    w = Workload("C5", "verify", H, KH, D, 1.0 / 16.0)
    for i in range(n_seq):
        w.sequences.append(Sequence(
            k=_draw(root, f"k{i}", (context + rows, KH, D), dist).astype(np.float16),
            v=_draw(root, f"v{i}", (context + rows, KH, D), dist).astype(np.float16),
            q=_draw(root, f"q{i}", (rows, H, D), dist).astype(np.float16),
            gate=_draw(root, f"gate{i}", (rows, H, D), dist).astype(np.float16),
            start=context))
    return w


BUILDERS = {"C1": decode_c1, "C2": decode_c2, "C3": decode_c3, "C4": prefill_c4, "C5": verify_c5}


def epilogue_inputs(tokens: int = 37, heads: int = 16, kv_heads: int = 2, dim: int = 256, seed: int = 0xE4):
    """Seeded inputs of the pre-attention epilogue: packed [query ; gate] rows, K and V projection
    rows (fp16) and the two per-head norm weights as bfloat16 bit patterns with their fp32 values."""
    packed = normal(seed, "packed", tokens * heads * 2 * dim).reshape(tokens, heads, 2 * dim).astype(np.float16)
    k = (2.0 * normal(seed, "k_proj", tokens * kv_heads * dim)).reshape(tokens, kv_heads * dim).astype(np.float16)
    v = normal(seed, "v_proj", tokens * kv_heads * dim).reshape(tokens, kv_heads * dim).astype(np.float16)

    def bf16(x):
        u = x.astype(np.float32).view(np.uint32)
        bits = ((u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) >> np.uint32(16)).astype(np.uint16)
        return bits, (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)

    qw_bits, qw = bf16(1.0 + 0.25 * normal(seed, "q_norm", dim))
    kw_bits, kw = bf16(1.0 + 0.25 * normal(seed, "k_norm", dim))
    return {"packed": packed, "k": k, "v": v, "q_weight_bits": qw_bits, "q_weight": qw, "k_weight_bits": kw_bits,
            "k_weight": kw}
