"""Behaviour of the attention entry points through the C ABI: the reference's own kernel-test
shapes and edge cases (tests/TinyTitan/Kernels/Attention/AttentionTests.swift,
PrefillAttentionTests.swift), equivalences between the entry points, error codes, graphs."""
import numpy as np
import pytest

import oracle
from tests.helpers import MAX_ABS, MEAN_ABS, f16_round
from tinytitan_amd import synthetic

pytestmark = pytest.mark.gpu


def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


class Cache:
    """A KV cache filled from token-major numpy rows, plus the fp32 copies the oracle wants."""

    def __init__(self, ctx, k, v, slots=1, layers=1, capacity=None):
        import torch
        from tinytitan_amd.engine import KVCacheManager
        self.ctx = ctx
        n, kh, d = k.shape
        cap = capacity or max(32, n)
        self.kv = KVCacheManager(ctx, layers, kh, d, slots=slots, max_context=max(cap, n), initial_capacity=cap)
        self.put(0, 0, 0, k, v)
        self.k32 = k.astype(np.float32)
        self.v32 = v.astype(np.float32)

    def put(self, layer, slot, position, k, v):
        import torch
        kd, vd = _dev(k), _dev(v)
        torch.cuda.synchronize()
        self.kv.append(layer, slot, position, kd, vd)
        self.ctx.synchronize()

    def close(self):
        self.kv.close()


def _decode(ctx, kv, q, seq_lens, heads, scale, slots=None, gate=None, layer=0):
    import torch
    from tinytitan_amd.engine import Attention
    qd = _dev(q)
    gd = _dev(gate) if gate is not None else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(ctx).encode_full(kv, layer, qd, out, heads, list(seq_lens), scale,
                               slot=list(slots if slots is not None else range(len(seq_lens))), gate=gd)
    ctx.synchronize()
    return out.float().cpu().numpy()


def _check(got, want, what, max_abs=MAX_ABS, mean_abs=MEAN_ABS):
    assert np.isfinite(got).all(), what
    diff = np.abs(got.astype(np.float64) - f16_round(want).astype(np.float64))
    assert diff.max() <= max_abs, f"{what}: max-abs {diff.max():.3e}"
    assert diff.mean() <= mean_abs, f"{what}: mean-abs {diff.mean():.3e}"


# ---- the reference's decode kernel-test shapes ------------------------------------------------

@pytest.mark.parametrize("D,H,KH,T", [(64, 4, 2, 128), (256, 16, 8, 256), (256, 16, 2, 128), (64, 8, 1, 128),
                                      (128, 8, 4, 64), (256, 8, 2, 1187), (128, 32, 1, 70), (64, 24, 2, 333)])
def test_decode_reference_shapes_uniform_inputs(gpu_ctx, D, H, KH, T):
    # AttentionTests.swift:125-222,405-409: q/k/v uniform(-0.5, 0.5) from SeedTree(seed).key(label),
    # rounded to fp16, compared with AttentionRef at RelError < 1e-2 (Tolerances.swift:15).
    seed = 1000 + D + H + T
    q = synthetic.uniform(seed, "q", H * D).reshape(1, H, D).astype(np.float16)
    k = synthetic.uniform(seed, "k", T * KH * D).reshape(T, KH, D).astype(np.float16)
    v = synthetic.uniform(seed, "v", T * KH * D).reshape(T, KH, D).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    got = _decode(gpu_ctx, c.kv, q[None], [T], H, 1.0 / np.sqrt(D))[0, 0]
    want = oracle.attention_ref(q[0].astype(np.float32), c.k32, c.v32, D, H, KH, T)
    rel = np.abs(got - want).max() / max(np.abs(want).max(), 1e-6)
    assert rel < 1e-2
    _check(got, want, f"decode {D}/{H}/{KH}/{T}")
    c.close()


def test_decode_k_equals_v_aliasing(gpu_ctx):
    # AttentionTests: V may alias K; the math is unchanged.
    D, H, KH, T = 64, 4, 2, 96
    q = synthetic.uniform(7, "q", H * D).reshape(1, H, D).astype(np.float16)
    k = synthetic.uniform(7, "k", T * KH * D).reshape(T, KH, D).astype(np.float16)
    c = Cache(gpu_ctx, k, k)
    got = _decode(gpu_ctx, c.kv, q[None], [T], H, 0.125)[0, 0]
    _check(got, oracle.attention_ref(q[0].astype(np.float32), c.k32, c.k32, D, H, KH, T), "K==V")
    c.close()


def test_decode_empty_sequence_and_gate(gpu_ctx):
    w = synthetic.decode_c2(context=200)
    s = w.sequences[0]
    c = Cache(gpu_ctx, s.k, s.v)
    q = s.q[None]
    # seq_len 0: zeros, never NaN (attention.metal:418-427; Attention.swift reference :72)
    zero = _decode(gpu_ctx, c.kv, q, [0], w.heads, w.scale)
    assert np.array_equal(zero, np.zeros_like(zero))
    base = _decode(gpu_ctx, c.kv, q, [200], w.heads, w.scale)
    half = _decode(gpu_ctx, c.kv, q, [200], w.heads, w.scale, gate=np.zeros_like(s.q)[None])
    _check(half, base * 0.5, "gate 0 halves the output", max_abs=1e-3)
    # a shorter seq_len ignores the rows behind it
    want = oracle.decode(s.q[0].astype(np.float32), c.k32[:77].reshape(77, -1), c.v32[:77].reshape(77, -1),
                         w.heads, w.kv_heads, w.dim, w.scale, gate=s.gate[0].astype(np.float32))
    got = _decode(gpu_ctx, c.kv, q, [77], w.heads, w.scale, gate=s.gate[None])[0, 0]
    _check(got, want, "seq_len 77 of 200")
    c.close()


# ---- batched decode == per-row decode ----------------------------------------------------------

def test_batch_equals_per_row(gpu_ctx):
    # BatchAttentionTests.swift:67-231: rows at positions [17, 9, 23, 5] in 4 slots, abs diff < 1e-3.
    import torch
    from tinytitan_amd.engine import KVCacheManager
    H, KH, D = 16, 2, 256
    lens = [18, 10, 24, 6]
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=4, max_context=64, initial_capacity=64)
    r = np.random.default_rng(5)
    q = r.standard_normal((4, 1, H, D)).astype(np.float16)
    caches = []
    for slot, n in enumerate(lens):
        k = r.standard_normal((n, KH, D)).astype(np.float16)
        v = r.standard_normal((n, KH, D)).astype(np.float16)
        kd, vd = _dev(k), _dev(v)
        torch.cuda.synchronize()
        kv.append(0, slot, 0, kd, vd)
        gpu_ctx.synchronize()
        caches.append((k, v))
    batch = _decode(gpu_ctx, kv, q, lens, H, 0.0625)
    order = [2, 0, 3, 1]  # slots need not be in order
    shuffled = _decode(gpu_ctx, kv, q[order], [lens[i] for i in order], H, 0.0625, slots=order)
    for i, slot in enumerate(order):
        assert np.array_equal(shuffled[i], batch[slot])
    for slot, n in enumerate(lens):
        single = _decode(gpu_ctx, kv, q[slot:slot + 1], [n], H, 0.0625, slots=[slot])
        assert np.abs(single[0] - batch[slot]).max() < 1e-3
        k, v = caches[slot]
        want = oracle.decode(q[slot, 0].astype(np.float32), k.astype(np.float32).reshape(n, -1),
                             v.astype(np.float32).reshape(n, -1), H, KH, D, 0.0625)
        _check(batch[slot, 0], want, f"slot {slot}")
    kv.close()


def test_more_sequences_than_one_launch_holds(gpu_ctx):
    # 70 sequences: the library splits them over launches of at most 64
    import torch
    from tinytitan_amd.engine import KVCacheManager
    H, KH, D, n = 8, 2, 64, 70
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=n, max_context=64, initial_capacity=64)
    r = np.random.default_rng(6)
    k = r.standard_normal((n, 40, KH, D)).astype(np.float16)
    v = r.standard_normal((n, 40, KH, D)).astype(np.float16)
    q = r.standard_normal((n, 1, H, D)).astype(np.float16)
    lens = [1 + (7 * i) % 40 for i in range(n)]
    for slot in range(n):
        kd, vd = _dev(k[slot]), _dev(v[slot])
        torch.cuda.synchronize()
        kv.append(0, slot, 0, kd, vd)
        gpu_ctx.synchronize()
    got = _decode(gpu_ctx, kv, q, lens, H, 0.125)
    for slot in (0, 1, 63, 64, 69):
        L = lens[slot]
        want = oracle.decode(q[slot, 0].astype(np.float32), k[slot, :L].astype(np.float32).reshape(L, -1),
                             v[slot, :L].astype(np.float32).reshape(L, -1), H, KH, D, 0.125)
        _check(got[slot, 0], want, f"sequence {slot}")
    kv.close()


# ---- prefill: strides, offsets, future rows, tile edges ----------------------------------------

def _prefill(ctx, kv, q, start, q_len, kv_valid, heads, scale, q_stride=None, o_stride=None, gate=None, gate_stride=None,
             slot=0, prefix=(0, 0, 0)):
    """q is [q_len][heads*dim]; optional padded strides and non-zero buffer prefixes (in halves)."""
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    width = q.shape[1]
    qs, os_, gs = q_stride or width, o_stride or width, gate_stride or width
    qbuf = np.full(prefix[0] + q_len * qs, 5.0, np.float16)
    qbuf[prefix[0]:].reshape(q_len, qs)[:, :width] = q
    qd = _dev(qbuf)
    out = torch.full((prefix[1] + q_len * os_,), float("nan"), dtype=torch.float16, device="cuda")
    gd = None
    if gate is not None:
        gbuf = np.full(prefix[2] + q_len * gs, -5.0, np.float16)
        gbuf[prefix[2]:].reshape(q_len, gs)[:, :width] = gate
        gd = _dev(gbuf)
    torch.cuda.synchronize()
    PrefillAttention(ctx).encode_causal(
        kv, 0, slot, qd[prefix[0]:], out[prefix[1]:],
        PrefillAttentionParams(start, q_len, kv_valid, heads, scale, qs, os_, gs), gate=gd[prefix[2]:] if gd is not None else None)
    ctx.synchronize()
    res = out.float().cpu().numpy()
    body = res[prefix[1]:].reshape(q_len, os_)
    # nothing outside the packed rows was written
    assert np.isnan(res[:prefix[1]]).all() and np.isnan(body[:, width:]).all()
    return body[:, :width]


@pytest.mark.parametrize("H,KH,D,start,chunk", [(4, 2, 64, 0, 37), (4, 2, 64, 41, 37), (16, 2, 256, 0, 96),
                                                 (16, 2, 256, 70, 45), (8, 2, 128, 5, 130), (8, 1, 64, 0, 64)])
def test_prefill_padded_strides_and_offset_buffers(gpu_ctx, H, KH, D, start, chunk):
    # PrefillAttentionTests.swift:306-375: strides +3 / +5 / +7 and buffer prefixes of 17/19/23/29 halves.
    # Rows that are not 16-byte aligned take the split-K kernel; aligned ones the LDS-staged kernel.
    kv_valid = start + chunk
    r = np.random.default_rng(H * D + start)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    g = r.standard_normal((chunk, H * D)).astype(np.float16)
    k = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    scale = 1.0 / np.sqrt(D)
    want = oracle.prefill_ref(q.astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, start, chunk, kv_valid, 0, scale)
    want_gated = want.reshape(chunk, -1) / (1 + np.exp(-g.astype(np.float64)))
    for qs, os_, gs, prefix in ((H * D, H * D, H * D, (0, 0, 0)), (H * D + 3, H * D + 7, H * D + 5, (17, 19, 23)),
                                (H * D + 8, H * D + 16, H * D + 24, (8, 16, 24))):
        got = _prefill(gpu_ctx, c.kv, q, start, chunk, kv_valid, H, scale, q_stride=qs, o_stride=os_, prefix=prefix)
        _check(got, want.reshape(chunk, -1), f"prefill strides {qs}/{os_}")
        got = _prefill(gpu_ctx, c.kv, q, start, chunk, kv_valid, H, scale, q_stride=qs, o_stride=os_, gate=g,
                       gate_stride=gs, prefix=prefix)
        _check(got, want_gated, f"gated prefill strides {qs}/{os_}/{gs}")
    c.close()


@pytest.mark.parametrize("start,chunk,gated", [(2100, 70, False), (4000, 130, True), (3000, 32, True),
                                               (8064, 128, True), (8500, 333, False), (9001, 130, True),
                                               (12000, 64, True)])
def test_short_chunk_deep_in_a_long_context(gpu_ctx, start, chunk, gated):
    # The reference's default prefillChunkTokens is 128 (PrefillRuntimeConfig.swift:151-157): a short
    # chunk far into a context, which the chunk kernel alone would serve with 8 workgroups.  The
    # entry point cuts the keys over the chip instead: below 64 rows or 4096 keys through the
    # split-K kernel, above through the chunk kernel over key ranges plus the combine pass (the
    # cases here sit on both sides, with whole and ragged last blocks); same semantics, same bar.
    H, KH, D = 16, 2, 256
    kv_valid = start + chunk
    r = np.random.default_rng(start + chunk)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    g = r.standard_normal((chunk, H * D)).astype(np.float16) if gated else None
    k = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    got = _prefill(gpu_ctx, c.kv, q, start, chunk, kv_valid, H, 0.0625, gate=g)
    # CPUQwen35.attentionBatch restated (the chunk's rows are the cache's last): minutes faster than the scalar reference
    want = oracle.attention_batch(q.astype(np.float32), c.k32, c.v32, chunk, start, H, KH, D, 0.0625, threads=4)
    want = want.reshape(chunk, -1)
    if gated:
        want = want / (1 + np.exp(-g.astype(np.float64)))
    _check(got, want, f"chunk of {chunk} at {start}")
    c.close()


@pytest.mark.parametrize("H,KH,D,start,chunk", [(8, 2, 128, 4100, 200), (16, 4, 64, 6000, 129), (8, 1, 256, 4500, 1100),
                                                (16, 2, 256, 30000, 160)])
def test_chunk_over_key_ranges_other_shapes(gpu_ctx, H, KH, D, start, chunk):
    # The key-range route at other head sizes and group sizes, with an odd number of tiles, a ragged last tile, and
    # enough rows that the ranges are few (1100 rows: 35 tiles of 8 heads over two or three ranges): a workgroup
    # takes one tile over one range, the combine pass all of a row's ranges at once.
    kv_valid = start + chunk
    r = np.random.default_rng(start * 7 + chunk)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    g = r.standard_normal((chunk, H * D)).astype(np.float16)
    k = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    scale = float(D) ** -0.5
    got = _prefill(gpu_ctx, c.kv, q, start, chunk, kv_valid, H, scale, gate=g)
    want = oracle.attention_batch(q.astype(np.float32), c.k32, c.v32, chunk, start, H, KH, D, scale, threads=4)
    want = want.reshape(chunk, -1) / (1 + np.exp(-g.astype(np.float64)))
    _check(got, want, f"chunk of {chunk} at {start}, {H}q/{KH}kv/{D}")
    c.close()


def test_prefill_ignores_future_rows(gpu_ctx):
    # PrefillAttentionTests.swift:74-93: adversarial K/V behind each row's position must not leak.
    H, KH, D, chunk = 16, 2, 256, 64
    r = np.random.default_rng(9)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    k = r.standard_normal((chunk + 32, KH, D)).astype(np.float16)
    v = r.standard_normal((chunk + 32, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    clean = _prefill(gpu_ctx, c.kv, q[:1], 0, 1, 1, H, 0.0625)
    assert np.array_equal(clean[0].reshape(H, D), np.repeat(v[0], H // KH, axis=0).astype(np.float32))  # one key: its V row
    # poison everything after row 10, then attend rows 0..10 only
    k2, v2 = k.copy(), v.copy()
    k2[11:] = 60000.0
    v2[11:] = -60000.0
    c.put(0, 0, 0, k2, v2)
    got = _prefill(gpu_ctx, c.kv, q[:11], 0, 11, 11, H, 0.0625)
    want = oracle.prefill_ref(q[:11].astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, 0, 11, 11, 0, 0.0625)
    _check(got, want.reshape(11, -1), "future rows")
    c.close()


@pytest.mark.parametrize("keys", [1, 63, 64, 65, 127, 128, 129, 255, 256, 257, 1023, 1024, 1025])
def test_prefill_tile_boundary_key_counts(gpu_ctx, keys):
    # PrefillAttentionTests.swift:144-180: the last 3 rows of a chunk ending at `keys` keys.
    H, KH, D = 16, 2, 256
    rows = min(3, keys)
    r = np.random.default_rng(keys)
    q = r.standard_normal((rows, H * D)).astype(np.float16)
    k = r.standard_normal((keys, KH, D)).astype(np.float16)
    v = r.standard_normal((keys, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    got = _prefill(gpu_ctx, c.kv, q, keys - rows, rows, keys, H, 0.0625)
    want = oracle.prefill_ref(q.astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, keys - rows, rows, keys, 0, 0.0625)
    _check(got, want.reshape(rows, -1), f"{keys} keys")
    c.close()


@pytest.mark.parametrize("scale", [-0.0625, 0.0])
def test_prefill_scale_that_is_not_positive(gpu_ctx, scale):
    # `scale` is an argument (AttentionRef.apply: `scale ?? 1/sqrt(D)`): a negative one turns the ranking of the keys
    # round, zero gives the mean of the visible V rows.  A chunk that fills the chip, aligned, fp16 pages.
    H, KH, D, chunk = 16, 2, 256, 512
    r = np.random.default_rng(77)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    k = r.standard_normal((chunk, KH, D)).astype(np.float16)
    v = r.standard_normal((chunk, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    got = _prefill(gpu_ctx, c.kv, q, 0, chunk, chunk, H, scale)
    want = oracle.prefill_ref(q.astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, 0, chunk, chunk, 0, scale)
    _check(got, want.reshape(chunk, -1), f"scale {scale}")
    if scale == 0.0:
        mean = np.cumsum(c.v32.reshape(chunk, KH, D), axis=0) / np.arange(1, chunk + 1)[:, None, None]
        assert np.abs(got.reshape(chunk, KH, H // KH, D) - mean[:, :, None, :]).max() <= 2e-3
    c.close()


def test_chunked_prefill_equals_unchunked(gpu_ctx):
    w = synthetic.prefill_c4(tokens=300)
    s = w.sequences[0]
    c = Cache(gpu_ctx, s.k, s.v)
    q = s.q.reshape(300, -1)
    whole = _prefill(gpu_ctx, c.kv, q, 0, 300, 300, w.heads, w.scale)
    a = _prefill(gpu_ctx, c.kv, q[:101], 0, 101, 101, w.heads, w.scale)
    b = _prefill(gpu_ctx, c.kv, q[101:], 101, 199, 300, w.heads, w.scale)
    assert np.abs(np.concatenate([a, b]) - whole).max() <= 1e-3
    c.close()


# ---- verify == decode --------------------------------------------------------------------------

@pytest.mark.parametrize("W", [2, 5, 9])
def test_verify_rows_equal_decode_steps(gpu_ctx, W):
    # WideVerifyIdentityTests.swift:60-121: row r of a W-row pass == a decode at start + r.
    import torch
    from tinytitan_amd.engine import Attention
    w = synthetic.verify_c5(n_seq=2, context=777, rows=W)
    c = None
    from tinytitan_amd.engine import KVCacheManager
    kv = KVCacheManager(gpu_ctx, 1, w.kv_heads, w.dim, slots=2, max_context=1024, initial_capacity=1024)
    for i, s in enumerate(w.sequences):
        kd, vd = _dev(s.k), _dev(s.v)
        torch.cuda.synchronize()
        kv.append(0, i, 0, kd, vd)
        gpu_ctx.synchronize()
    q = np.stack([s.q for s in w.sequences])
    g = np.stack([s.gate for s in w.sequences])
    qd, gd = _dev(q), _dev(g)
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qd, out, w.heads, [777, 777], W, w.scale, [0, 1], gate=gd)
    gpu_ctx.synchronize()
    ver = out.float().cpu().numpy()
    for r in range(W):
        dec = _decode(gpu_ctx, kv, q[:, r:r + 1], [777 + r + 1] * 2, w.heads, w.scale, gate=g[:, r:r + 1])
        assert np.abs(dec[:, 0] - ver[:, r]).max() <= 1e-3, f"row {r}"
    kv.close()


def test_verify_full_batch_identity(gpu_ctx):
    # C5 at full size (8 sequences x 65540 keys) with device-generated data: every verify row
    # must equal the decode step at that position (the cache is far too large for the CPU oracle
    # to be the routine check; two of its sequences are checked against it in the config tests).
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, n, ctxlen, W = 16, 2, 256, 8, 65536, 4
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=n, max_context=ctxlen + 32, initial_capacity=ctxlen + 32)
    gen = torch.Generator(device="cuda").manual_seed(55)
    for i in range(n):
        k = torch.randn(ctxlen + W, KH, D, generator=gen, device="cuda").to(torch.float16)
        v = torch.randn(ctxlen + W, KH, D, generator=gen, device="cuda").to(torch.float16)
        torch.cuda.synchronize()
        kv.append(0, i, 0, k, v)
        gpu_ctx.synchronize()
    q = torch.randn(n, W, H, D, generator=gen, device="cuda").to(torch.float16)
    g = torch.randn(n, W, H, D, generator=gen, device="cuda").to(torch.float16)
    out = torch.zeros_like(q)
    dec = torch.zeros(n, 1, H, D, dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, q, out, H, [ctxlen] * n, W, 0.0625, list(range(n)), gate=g)
    gpu_ctx.synchronize()
    assert torch.isfinite(out).all()
    for r in (0, W - 1):
        qr, gr = q[:, r:r + 1].contiguous(), g[:, r:r + 1].contiguous()
        torch.cuda.synchronize()
        Attention(gpu_ctx).encode_full(kv, 0, qr, dec, H, [ctxlen + r + 1] * n, 0.0625, slot=list(range(n)), gate=gr)
        gpu_ctx.synchronize()
        diff = (dec[:, 0].float() - out[:, r].float()).abs()
        assert diff.max().item() <= 1e-3 and diff.mean().item() <= 2e-5
    kv.close()


@pytest.mark.gpu
@pytest.mark.parametrize("heads", [(16, 2, 256, 4), (32, 8, 128, 8), (32, 4, 64, 4)])
@pytest.mark.parametrize("bits", [16, 8])
def test_verify_rows_on_both_sides_of_the_tile_rule(gpu_ctx, bits, heads):
    # A few verify rows take tiles of 16 rows while the launch reads little (the planner's rule: keys x tiles of 16 x
    # KV heads up to 144 Ki at fp16, 288 Ki over quantised pages) and one tile of 32 beyond: the same rows either way,
    # each equal to the decode step at its position (WideVerifyIdentityTests.swift:60-121).
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, W = heads
    limit = (144 if bits == 16 else 288) * 1024 // (2 * KH)  # the rows fill two tiles of 16 per KV head
    below, above = limit - 40, limit + 40
    if bits == 16:
        small, large = gpu_ctx.split_geometry(1, H, KH, D, W, below), gpu_ctx.split_geometry(1, H, KH, D, W, above)
        assert small[2] == 2 * KH * small[1] and large[2] == KH * large[1]  # workgroups = splits x tiles
    gen = torch.Generator(device="cuda").manual_seed(91 + bits)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=above + 32, initial_capacity=above + 32, precision_bits=bits)
    k = torch.randn(above + W, KH, D, generator=gen, device="cuda").to(torch.float16)
    v = torch.randn(above + W, KH, D, generator=gen, device="cuda").to(torch.float16)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, k, v)
    gpu_ctx.synchronize()
    q = torch.randn(1, W, H, D, generator=gen, device="cuda").to(torch.float16)
    g = torch.randn(1, W, H, D, generator=gen, device="cuda").to(torch.float16)
    out = torch.zeros_like(q)
    dec = torch.zeros(1, 1, H, D, dtype=torch.float16, device="cuda")
    for start in (below - W, above - W):
        torch.cuda.synchronize()
        Attention(gpu_ctx).encode_verify_rows(kv, 0, q, out, H, [start], W, D ** -0.5, [0], gate=g)
        gpu_ctx.synchronize()
        assert torch.isfinite(out).all()
        for r in range(W):
            qr, gr = q[:, r:r + 1].contiguous(), g[:, r:r + 1].contiguous()
            torch.cuda.synchronize()
            Attention(gpu_ctx).encode_full(kv, 0, qr, dec, H, [start + r + 1], D ** -0.5, slot=[0], gate=gr)
            gpu_ctx.synchronize()
            diff = (dec[:, 0].float() - out[:, r].float()).abs()
            assert diff.max().item() <= 1e-3 and diff.mean().item() <= 2e-5, f"start {start} row {r}"
    kv.close()


# ---- a runner-shaped sequence: prefill chunks, decode steps, verify + rewind ---------------------

def test_runner_sequence_prefill_decode_verify_rewind(gpu_ctx):
    # The order of calls of RealForwardRunner: reserve, write K/V at the cursor, attend, advance
    # (RealForwardRunner+Decode.swift:211-439, +PrefillLayer.swift:240, +WideVerify.swift:74-139).
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, scale = 16, 2, 256, 0.0625
    r = np.random.default_rng(21)
    total = 150
    k = r.standard_normal((total, KH, D)).astype(np.float16)
    v = r.standard_normal((total, KH, D)).astype(np.float16)
    q = r.standard_normal((total, H * D)).astype(np.float16)
    g = r.standard_normal((total, H * D)).astype(np.float16)
    k32, v32 = k.astype(np.float32), v.astype(np.float32)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=4096, initial_capacity=64)

    def put(pos, n):
        kd, vd = _dev(k[pos:pos + n]), _dev(v[pos:pos + n])
        torch.cuda.synchronize()
        kv.append(0, 0, pos, kd, vd)
        gpu_ctx.synchronize()

    def want_rows(pos, n):
        o = oracle.attention_batch(q[pos:pos + n].astype(np.float32), k32[:pos + n], v32[:pos + n], n, pos, H, KH, D,
                                   scale, gate=g[pos:pos + n].astype(np.float32))
        return o.reshape(n, -1)

    pos = 0
    for chunk in (40, 37):  # two prefill chunks; the second one forces a capacity growth (64 -> 128)
        kv.expect_position(0, pos)
        kv.reserve(pos + chunk)
        put(pos, chunk)
        got = _prefill(gpu_ctx, kv, q[pos:pos + chunk], pos, chunk, pos + chunk, H, scale, gate=g[pos:pos + chunk])
        _check(got, want_rows(pos, chunk), f"prefill chunk at {pos}")
        kv.advance(0, chunk)
        pos += chunk
    assert kv.capacity_tokens == 128
    for _ in range(3):  # decode steps
        kv.expect_position(0, pos)
        kv.reserve(pos + 1)
        put(pos, 1)
        got = _decode(gpu_ctx, kv, q[pos].reshape(1, 1, H, D), [pos + 1], H, scale, gate=g[pos].reshape(1, 1, H, D))
        _check(got[0, 0].reshape(-1), want_rows(pos, 1)[0], f"decode at {pos}")
        kv.advance(0, 1)
        pos += 1
    # verify 4 draft rows, accept 2, rewind, and carry on decoding over the accepted prefix
    W = 4
    kv.reserve(pos + W)
    put(pos, W)
    qd, gd = _dev(q[pos:pos + W].reshape(1, W, H, D)), _dev(g[pos:pos + W].reshape(1, W, H, D))
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qd, out, H, [pos], W, scale, [0], gate=gd)
    gpu_ctx.synchronize()
    _check(out.float().cpu().numpy().reshape(W, -1), want_rows(pos, W), "verify rows")
    kv.advance(0, W)
    kv.rewind(0, pos + 2)
    pos += 2
    assert kv.position(0) == pos
    # the rejected rows are overwritten by the next token
    k[pos], v[pos] = k[pos + 20], v[pos + 20]
    k32, v32 = k.astype(np.float32), v.astype(np.float32)
    put(pos, 1)
    got = _decode(gpu_ctx, kv, q[pos].reshape(1, 1, H, D), [pos + 1], H, scale, gate=g[pos].reshape(1, 1, H, D))
    _check(got[0, 0].reshape(-1), want_rows(pos, 1)[0], "decode after rewind")
    kv.close()


# ---- error codes, geometry, graphs, timing -----------------------------------------------------

def test_error_codes(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import (Attention, KVCacheManager, PrefillAttention, PrefillAttentionParams,
                                      TinyTitanHIPError)
    kv = KVCacheManager(gpu_ctx, 1, 2, 64, slots=2, max_context=64)
    q = torch.zeros(1, 1, 8, 64, dtype=torch.float16, device="cuda")
    out = torch.zeros_like(q)
    att, pre = Attention(gpu_ctx), PrefillAttention(gpu_ctx)

    def status(fn):
        with pytest.raises(TinyTitanHIPError) as e:
            fn()
        return e.value.status

    assert status(lambda: att.encode_full(kv, 0, q, out, 7, [4], 0.125)) == capi.ERR_SHAPE        # 7 heads over 2 KV heads
    assert status(lambda: att.encode_full(kv, 1, q, out, 8, [4], 0.125)) == capi.ERR_INVALID_ARGUMENT  # layer
    assert status(lambda: att.encode_full(kv, 0, q, out, 8, [4], 0.125, slot=[2])) == capi.ERR_INVALID_ARGUMENT
    assert status(lambda: att.encode_full(kv, 0, q, out, 8, [65], 0.125)) == capi.ERR_CAPACITY    # beyond capacity
    assert status(lambda: att.encode_full(kv, 0, q, out, 8, [-1], 0.125)) == capi.ERR_INVALID_ARGUMENT
    assert status(lambda: att.encode_verify_rows(kv, 0, q, out, 8, [62], 4, 0.125, [0])) == capi.ERR_CAPACITY
    p = PrefillAttentionParams(10, 4, 13, 8, 0.125, 512, 512, 512)  # start + q_len > kv_valid
    assert status(lambda: pre.encode_causal(kv, 0, 0, q, out, p)) == capi.ERR_INVALID_ARGUMENT
    p = PrefillAttentionParams(0, 1, 1, 8, 0.125, 511, 512, 512)  # stride below the packed width
    assert status(lambda: pre.encode_causal(kv, 0, 0, q, out, p)) == capi.ERR_SHAPE
    p = PrefillAttentionParams(0, 1, 65, 8, 0.125, 512, 512, 512)  # kv_valid beyond capacity
    assert status(lambda: pre.encode_causal(kv, 0, 0, q, out, p)) == capi.ERR_CAPACITY
    lib = capi.lib()
    assert lib.tt_hip_attn_decode(gpu_ctx.handle, kv.handle, 0, 1, capi.int_array([0]), capi.int_array([1]), 8, None,
                                  None, 0.125, out.data_ptr()) == capi.ERR_INVALID_ARGUMENT  # null q
    assert lib.tt_hip_attn_decode(None, kv.handle, 0, 1, capi.int_array([0]), capi.int_array([1]), 8, q.data_ptr(),
                                  None, 0.125, out.data_ptr()) == capi.ERR_INVALID_ARGUMENT  # null context
    assert capi.strerror(capi.ERR_CURSOR) == "KV cursor mismatch"
    kv.close()


def test_split_geometry_reports_dispatch_shape(gpu_ctx):
    # cf. attentionSplitGeometry_reportsEffectiveDispatchShape (AttentionTests.swift:27-51)
    split, n_splits, wgs = gpu_ctx.split_geometry(1, 16, 2, 256, 1, 32768)
    assert split % 32 == 0 and n_splits == -(-32768 // split) and wgs == n_splits * 2
    assert 256 <= wgs <= 1024  # enough workgroups to cover 256 CUs
    split1, n1, wgs1 = gpu_ctx.split_geometry(1, 16, 2, 256, 1, 20)
    assert n1 == 1 and wgs1 == 2  # a short sequence is a single pass, no combine
    gpu_ctx.set_split_tokens(100)
    assert gpu_ctx.split_geometry(1, 16, 2, 256, 1, 1000)[0] == 128  # overrides round up to whole blocks
    gpu_ctx.set_split_tokens(0)


def test_graph_replay_matches_eager(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, TinyTitanHIPError
    w = synthetic.decode_c2(context=2000)
    s = w.sequences[0]
    c = Cache(gpu_ctx, s.k, s.v, layers=2)
    c.put(1, 0, 0, s.k[::-1].copy(), s.v[::-1].copy())
    qd, gd = _dev(s.q[None]), _dev(s.gate[None])
    outs = [torch.zeros_like(qd), torch.zeros_like(qd)]
    att = Attention(gpu_ctx)
    eager = []
    for layer in range(2):
        torch.cuda.synchronize()
        att.encode_full(c.kv, layer, qd, outs[layer], w.heads, [2000], w.scale, gate=gd)
        gpu_ctx.synchronize()
        eager.append(outs[layer].clone())
    gpu_ctx.graph_begin()
    for layer in range(2):
        att.encode_full(c.kv, layer, qd, outs[layer], w.heads, [2000], w.scale, gate=gd)
    graph = gpu_ctx.graph_end()
    for replay in range(4):
        for o in outs:
            o.zero_()
        torch.cuda.synchronize()
        graph.launch()
        gpu_ctx.synchronize()
        for layer in range(2):
            assert torch.equal(outs[layer], eager[layer]), f"replay {replay} layer {layer}"
        # eager work of the program's own between replays
        att.encode_full(c.kv, 0, qd, outs[0], w.heads, [1999 - replay], w.scale, gate=gd)
        gpu_ctx.synchronize()
    graph.close()
    c.close()
    # a call that would have to allocate while capturing is refused (run it once eagerly first);
    # on a context of its own, whose split scratch no earlier test has grown
    from tinytitan_amd.engine import HIPContext
    fresh = HIPContext(gpu_ctx.device)
    big = Cache(fresh, np.zeros((4000, 2, 256), np.float16), np.zeros((4000, 2, 256), np.float16))
    fresh.graph_begin()
    with pytest.raises(TinyTitanHIPError) as e:
        Attention(fresh).encode_full(big.kv, 0, qd, outs[0], w.heads, [4000], w.scale, gate=gd)
    assert e.value.status == capi.ERR_BUSY
    fresh.graph_end().close()
    big.close()
    fresh.close()


def test_growth_and_creation_inside_a_capture_are_refused_and_the_capture_survives():
    # tt_hip_kv_reserve past capacity and tt_hip_kv_create* would allocate, copy and synchronise on the capturing
    # stream: both answer BUSY, the capture ends cleanly and its graph replays.
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, HIPContext, KVCacheManager, TinyTitanHIPError
    ctx = HIPContext(0)
    w = synthetic.decode_c2(context=600)
    s = w.sequences[0]
    kv = KVCacheManager(ctx, 1, w.kv_heads, w.dim, slots=1, max_context=4096, initial_capacity=640)
    kd, vd = _dev(s.k), _dev(s.v)
    qd, gd = _dev(s.q[None]), _dev(s.gate[None])
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    kv.advance(0, 600)  # growth moves a slot's rows up to its cursor
    att = Attention(ctx)
    att.encode_full(kv, 0, qd, out, w.heads, [600], w.scale, gate=gd)
    ctx.synchronize()
    eager = out.clone()
    ctx.graph_begin()
    with pytest.raises(TinyTitanHIPError) as e:
        kv.reserve(2000)
    assert e.value.status == capi.ERR_BUSY and kv.capacity_tokens == 640
    with pytest.raises(TinyTitanHIPError) as e:
        KVCacheManager(ctx, 1, 2, 64, slots=1, max_context=64, initial_capacity=64)
    assert e.value.status == capi.ERR_BUSY
    kv.reserve(600)  # no growth: fine inside a capture
    att.encode_full(kv, 0, qd, out, w.heads, [600], w.scale, gate=gd)
    graph = ctx.graph_end()
    for replay in range(3):
        out.zero_()
        torch.cuda.synchronize()
        graph.launch()
        ctx.synchronize()
        assert torch.equal(out, eager), f"replay {replay}"
    # growth outside the capture frees the stores the graph's kernels address: the graph refuses to replay
    kv.reserve(2000)
    assert kv.capacity_tokens >= 2000
    with pytest.raises(TinyTitanHIPError) as e:
        graph.launch()
    assert e.value.status == capi.ERR_STALE
    graph.close()
    # the grown cache holds the same rows: a fresh capture replays
    ctx.graph_begin()
    att.encode_full(kv, 0, qd, out, w.heads, [600], w.scale, gate=gd)
    graph = ctx.graph_end()
    out.zero_()
    torch.cuda.synchronize()
    graph.launch()
    ctx.synchronize()
    assert torch.equal(out, eager)
    # a later eager call that grows the split scratch stales it as well
    big = KVCacheManager(ctx, 1, 2, 256, slots=8, max_context=8192, initial_capacity=8192)
    torch.cuda.synchronize()
    att.encode_verify_rows(big, 0, torch.zeros((8, 4, 16, 256), dtype=torch.float16, device="cuda"),
                           torch.zeros((8, 4, 16, 256), dtype=torch.float16, device="cuda"), 16, [8000] * 8, 4, 0.0625,
                           list(range(8)))
    ctx.synchronize()
    with pytest.raises(TinyTitanHIPError) as e:
        graph.launch()
    assert e.value.status == capi.ERR_STALE
    graph.close()
    big.close()
    kv.close()
    ctx.close()


def test_default_stream_orders_with_the_callers_work(gpu_ctx):
    # torch's default stream is HIP's null stream (handle 0): use_torch_stream selects it, and a decode enqueued
    # right behind torch kernels that produce its inputs sees them without any synchronisation in between
    import torch
    from tinytitan_amd.engine import Attention
    w = synthetic.decode_c2(context=900)
    s = w.sequences[0]
    c = Cache(gpu_ctx, s.k, s.v)
    want = _decode(gpu_ctx, c.kv, s.q[None], [900], w.heads, w.scale, gate=s.gate[None])
    try:
        gpu_ctx.use_torch_stream()
        assert gpu_ctx._lib.tt_hip_ctx_stream(gpu_ctx.handle) in (None, 0)
        host_q, host_g = torch.from_numpy(s.q[None]).pin_memory(), torch.from_numpy(s.gate[None]).pin_memory()
        for _ in range(3):
            qd = torch.empty(host_q.shape, dtype=torch.float16, device="cuda")
            gd = torch.empty_like(qd)
            out = torch.full(host_q.shape, float("nan"), dtype=torch.float16, device="cuda")
            qd.copy_(host_q, non_blocking=True)
            gd.copy_(host_g, non_blocking=True)
            qd.mul_(1.0)  # a kernel on the same stream
            Attention(gpu_ctx).encode_full(c.kv, 0, qd, out, w.heads, [900], w.scale, gate=gd)
            got = out.float().cpu().numpy()  # torch's copy is ordered behind the decode on the same stream
            assert np.array_equal(got, want)
    finally:
        gpu_ctx.set_stream(None)
    c.close()


def test_profile_and_timer(gpu_ctx):
    import torch
    from tinytitan_amd.engine import Attention
    w = synthetic.decode_c1()
    s = w.sequences[0]
    c = Cache(gpu_ctx, s.k, s.v)
    qd = _dev(s.q[None])
    out = torch.zeros_like(qd)
    att = Attention(gpu_ctx)
    torch.cuda.synchronize()
    att.encode_full(c.kv, 0, qd, out, w.heads, [2048], w.scale)
    gpu_ctx.synchronize()
    gpu_ctx.profile_enable(8)
    gpu_ctx.timer_begin()
    for _ in range(5):
        att.encode_full(c.kv, 0, qd, out, w.heads, [2048], w.scale)
    total_ns = gpu_ctx.timer_end_ns()
    launches, kernel_ns = gpu_ctx.profile_read()
    gpu_ctx.profile_disable()
    assert launches == 5 and 0 < kernel_ns <= total_ns * 1.05
    assert gpu_ctx.profile_read() == (0, 0)
    c.close()


def test_prefill_head_groups_the_staged_kernel_does_not_serve(gpu_ctx):
    # 2 q heads per KV head (not a multiple of 4) takes the split-K kernel; results must not differ.
    H, KH, D, chunk = 4, 2, 128, 70
    r = np.random.default_rng(31)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    k = r.standard_normal((chunk, KH, D)).astype(np.float16)
    v = r.standard_normal((chunk, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    got = _prefill(gpu_ctx, c.kv, q, 0, chunk, chunk, H, 0.0884)
    want = oracle.prefill_ref(q.astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, 0, chunk, chunk, 0, 0.0884)
    _check(got, want.reshape(chunk, -1), "group of 2")
    c.close()


def test_kernel_variant_switches_are_explicit_calls_and_change_no_result():
    # tt_hip_set_option (the reference's TINYTITAN_ATTN_* switches, Attention.swift:186-188, as calls): the cache
    # policy of the K/V loads and the order a chunk's workgroups are dealt out in change timing only -- the
    # outputs are bit for bit those of the defaults; unknown options and values are refused.
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, HIPContext, PrefillAttention, PrefillAttentionParams, TinyTitanHIPError
    ctx = HIPContext(0)
    w = synthetic.decode_c2(context=3000)
    s = w.sequences[0]
    c = Cache(ctx, s.k, s.v)
    qd, gd = _dev(s.q[None]), _dev(s.gate[None])
    outs = {}
    for mode in (-1, 0, 1):
        ctx.set_option(capi.OPT_KV_STREAM, mode)
        out = torch.zeros_like(qd)
        Attention(ctx).encode_full(c.kv, 0, qd, out, w.heads, [3000], w.scale, gate=gd)
        ctx.synchronize()
        outs[mode] = out
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[-1])
    # the measurement control: the pass over K/V without its combine pass -- nothing is written -- and back
    ctx.set_option(capi.OPT_MEASURE_PASS_ONLY, 1)
    marked = torch.full_like(qd, 7.0)
    Attention(ctx).encode_full(c.kv, 0, qd, marked, w.heads, [3000], w.scale, gate=gd)
    ctx.synchronize()
    assert (marked == 7.0).all()
    ctx.set_option(capi.OPT_MEASURE_PASS_ONLY, 0)
    Attention(ctx).encode_full(c.kv, 0, qd, marked, w.heads, [3000], w.scale, gate=gd)
    ctx.synchronize()
    assert torch.equal(marked, outs[-1])
    # a chunk of a few rows deep in the sequence goes through the split-K tiles over several key ranges
    r = np.random.default_rng(97)
    rows, H, D = 40, w.heads, w.dim
    q = _dev(r.standard_normal((rows, H * D)).astype(np.float16))
    ctx.set_split_tokens(512)
    chunk = {}
    for mode in (1, 0):
        ctx.set_option(capi.OPT_XCD_GRID, mode)
        out = torch.zeros_like(q)
        PrefillAttention(ctx).encode_causal(c.kv, 0, 0, q, out, PrefillAttentionParams(3000 - rows, rows, 3000, H, w.scale, H * D, H * D, H * D))
        ctx.synchronize()
        chunk[mode] = out
    ctx.set_split_tokens(0)
    assert torch.equal(chunk[0], chunk[1])
    for option, value in ((0, 0), (99, 1), (capi.OPT_KV_STREAM, 2), (capi.OPT_KV_STREAM, -2), (capi.OPT_XCD_GRID, 2),
                          (capi.OPT_MEASURE_PASS_ONLY, 2)):
        with pytest.raises(TinyTitanHIPError) as e:
            ctx.set_option(option, value)
        assert e.value.status == capi.ERR_INVALID_ARGUMENT
    ctx.graph_begin()
    with pytest.raises(TinyTitanHIPError) as e:
        ctx.set_option(capi.OPT_XCD_GRID, 1)
    assert e.value.status == capi.ERR_BUSY
    ctx.graph_end().close()
    c.close()
    ctx.close()
