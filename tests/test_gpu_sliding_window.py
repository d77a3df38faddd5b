"""Sliding-window attention through the C ABI against the oracle's windowed references
(AttentionRef.apply with `window`, sources/TinyTitanValidation/Support/Reference/Attention/Attention.swift:14-114;
PrefillAttentionRef with `slidingWindow`, PrefillAttentionRef.swift:59-101), at the attention bar."""
import numpy as np
import pytest

import oracle
from tests.test_gpu_attention_api import Cache, _check, _dev

pytestmark = pytest.mark.gpu


def _swa(ctx, kv, q, seq_lens, window, heads, scale, gate=None):
    import torch
    from tinytitan_amd.engine import Attention
    qd, gd = _dev(q), _dev(gate) if gate is not None else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(ctx).encode_swa(kv, 0, qd, out, heads, list(seq_lens), window, scale, slot=list(range(len(seq_lens))), gate=gd)
    ctx.synchronize()
    return out.float().cpu().numpy()


@pytest.mark.parametrize("H,KH,D,T,window", [(16, 2, 256, 1187, 256), (16, 2, 256, 1187, 100), (8, 2, 128, 700, 33),
                                             (4, 1, 64, 300, 1), (16, 2, 256, 5000, 4096), (16, 2, 256, 200, 4096),
                                             (16, 2, 256, 4200, 31)])
def test_decode_window(gpu_ctx, H, KH, D, T, window):
    r = np.random.default_rng(T + window)
    q = r.standard_normal((1, H, D)).astype(np.float16)
    k = r.standard_normal((T, KH, D)).astype(np.float16)
    v = r.standard_normal((T, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    scale = D ** -0.5
    for length in (T, T - 37 if T > 40 else T, min(T, window), 1):
        got = _swa(gpu_ctx, c.kv, q, [length], window, H, scale)[0]
        want = oracle.attention_ref(q[0].astype(np.float32), c.k32[:length], c.v32[:length], D, H, KH, length, window, scale)
        _check(got, want.reshape(H, D), f"window {window} over {length} keys")
    # the window matters, and window 0 is the plain decode
    if T > 2 * window:
        plain = _swa(gpu_ctx, c.kv, q, [T], 0, H, scale)[0]
        full = oracle.attention_ref(q[0].astype(np.float32), c.k32, c.v32, D, H, KH, T, 0, scale)
        _check(plain, full.reshape(H, D), "window 0")
        assert np.abs(full.reshape(H, D) - _swa(gpu_ctx, c.kv, q, [T], window, H, scale)[0]).max() > 1e-3
    c.close()


def test_decode_window_batch_and_gate(gpu_ctx):
    H, KH, D, window = 16, 2, 256, 500
    lengths = [1500, 499, 501, 3000, 1]
    r = np.random.default_rng(3)
    from tinytitan_amd.engine import KVCacheManager
    import torch
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=len(lengths), max_context=3008, initial_capacity=3008)
    ks, vs = [], []
    for s, n in enumerate(lengths):
        k = r.standard_normal((n, KH, D)).astype(np.float16)
        v = r.standard_normal((n, KH, D)).astype(np.float16)
        kd, vd = _dev(k), _dev(v)
        torch.cuda.synchronize()
        kv.append(0, s, 0, kd, vd)
        gpu_ctx.synchronize()
        ks.append(k.astype(np.float32).reshape(n, -1))
        vs.append(v.astype(np.float32).reshape(n, -1))
    q = r.standard_normal((len(lengths), 1, H, D)).astype(np.float16)
    g = r.standard_normal((len(lengths), 1, H, D)).astype(np.float16)
    got = _swa(gpu_ctx, kv, q, lengths, window, H, 0.0625, gate=g)
    for s, n in enumerate(lengths):
        want = oracle.attention_ref(q[s, 0].astype(np.float32), ks[s], vs[s], D, H, KH, n, window, 0.0625).reshape(H, D)
        want = want / (1 + np.exp(-g[s, 0].astype(np.float64)))
        _check(got[s, 0], want, f"sequence {s} of {n} keys")
    kv.close()


@pytest.mark.parametrize("start,chunk,window,gated", [(0, 200, 64, False), (300, 70, 100, True), (1000, 129, 333, True),
                                                      (50, 40, 1000, False), (4000, 257, 2048, True), (90, 10, 1, False),
                                                      (0, 2100, 512, True), (700, 1000, 900, False), (33, 2500, 31, True),
                                                      (5000, 64, 4096, False)])
def test_prefill_window(gpu_ctx, start, chunk, window, gated):
    # chunks whose window and rows stay within 2048 keys run the MFMA chunk kernel from each tile's window
    # block on, as do the chunks of 2048+ rows (half a chip of workgroups); (4000, 257, 2048) and
    # (5000, 64, 4096) -- few rows over a long window -- run the split-K kernel
    import torch
    from tinytitan_amd.engine import PrefillAttention, PrefillAttentionParams
    H, KH, D = 16, 2, 256
    kv_valid = start + chunk
    r = np.random.default_rng(start + chunk + window)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    g = r.standard_normal((chunk, H * D)).astype(np.float16) if gated else None
    k = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    c = Cache(gpu_ctx, k, v)
    qd, gd = _dev(q), _dev(g) if gated else None
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    PrefillAttention(gpu_ctx).encode_causal(c.kv, 0, 0, qd, out, PrefillAttentionParams(start, chunk, kv_valid, H, 0.0625, H * D,
                                                                                       H * D, H * D, sliding_window=window), gate=gd)
    gpu_ctx.synchronize()
    want = oracle.prefill_ref(q.astype(np.float32), c.k32, c.v32, H * D, KH * D, D, H, KH, start, chunk, kv_valid, window, 0.0625)
    want = want.reshape(chunk, -1)
    if gated:
        want = want / (1 + np.exp(-g.astype(np.float64)))
    _check(out.float().cpu().numpy(), want, f"prefill of {chunk} at {start}, window {window}")
    c.close()


def test_window_over_a_quantised_cache(gpu_ctx):
    from tinytitan_amd.engine import KVCacheManager
    import torch
    H, KH, D, T, window = 16, 2, 256, 2000, 300
    r = np.random.default_rng(8)
    k = r.standard_normal((T, KH, D)).astype(np.float16)
    v = r.standard_normal((T, KH, D)).astype(np.float16)
    q = r.standard_normal((1, 1, H, D)).astype(np.float16)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=T, initial_capacity=T, precision_bits=8)
    kd, vd = _dev(k), _dev(v)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    gpu_ctx.synchronize()
    deq = lambda x: oracle.kv_dequantize_rows(oracle.kv_quantize_rows(x.reshape(T, -1).astype(np.float32), 8), KH * D, 8)
    got = _swa(gpu_ctx, kv, q, [T], window, H, 0.0625)[0, 0]
    want = oracle.attention_ref(q[0, 0].astype(np.float32), deq(k), deq(v), D, H, KH, T, window, 0.0625)
    _check(got, want.reshape(H, D), "8-bit cache, window 300")
    kv.close()


def test_window_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, KVCacheManager, TinyTitanHIPError
    kv = KVCacheManager(gpu_ctx, 1, 2, 256, slots=1, max_context=64, initial_capacity=64)
    q = torch.zeros((1, 1, 16, 256), dtype=torch.float16, device="cuda")
    with pytest.raises(TinyTitanHIPError) as e:
        Attention(gpu_ctx).encode_swa(kv, 0, q, torch.zeros_like(q), 16, [10], -1, 0.0625)
    assert e.value.status == capi.ERR_INVALID_ARGUMENT
    kv.close()


@pytest.mark.parametrize("bits", [16, 8])
def test_ring_cache_streams_a_long_sequence(gpu_ctx, bits):
    # A sliding-window layer kept as a ring of 256 rows (position p at row p % 256) while the sequence
    # runs to 1000 tokens: chunks of 64 are appended (never wrapping), each chunk's windowed prefill and a
    # windowed decode at its end are checked against the oracle over the whole, linear K/V.
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, PrefillAttention, PrefillAttentionParams, TinyTitanHIPError
    H, KH, D, total, cap, window, chunk = 8, 2, 128, 1000, 256, 150, 64
    r = np.random.default_rng(bits)
    k = r.standard_normal((total, KH, D)).astype(np.float16)
    v = r.standard_normal((total, KH, D)).astype(np.float16)
    q = r.standard_normal((total, H * D)).astype(np.float16)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=1024, precision_bits=bits, ring_capacity=cap)
    assert kv.capacity_tokens == cap
    kv.reserve(1000)
    assert kv.capacity_tokens == cap  # a ring does not grow
    if bits == 16:
        k32, v32 = k.astype(np.float32).reshape(total, -1), v.astype(np.float32).reshape(total, -1)
    else:
        k32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(k.reshape(total, -1).astype(np.float32), bits), KH * D, bits)
        v32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(v.reshape(total, -1).astype(np.float32), bits), KH * D, bits)
    scale = D ** -0.5
    for start in range(0, total, chunk):
        n = min(chunk, total - start)
        kd, vd = _dev(k[start:start + n]), _dev(v[start:start + n])
        torch.cuda.synchronize()
        kv.append(0, 0, start, kd, vd)
        gpu_ctx.synchronize()
        kv.advance(0, n)
        qd = _dev(q[start:start + n])
        out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        PrefillAttention(gpu_ctx).encode_causal(kv, 0, 0, qd, out, PrefillAttentionParams(start, n, start + n, H, scale, H * D, H * D,
                                                                                         H * D, sliding_window=window))
        gpu_ctx.synchronize()
        want = oracle.prefill_ref(q[start:start + n].astype(np.float32), k32, v32, H * D, KH * D, D, H, KH, start, n, start + n,
                                  window, scale).reshape(n, -1)
        _check(out.float().cpu().numpy(), want, f"chunk at {start}")
        L = start + n
        got = _swa(gpu_ctx, kv, q[L - 1].reshape(1, 1, H, D), [L], window, H, scale)[0, 0]
        first = max(0, L - window)
        _check(got, oracle.decode(q[L - 1].astype(np.float32), k32[first:L], v32[first:L], H, KH, D, scale), f"decode at {L}")
    # the last rows read back from where the ring put them
    rk, rv = kv.read(0, 0, total - 40, 40)
    if bits == 16:
        assert np.array_equal(rk.cpu().numpy(), k[total - 40:]) and np.array_equal(rv.cpu().numpy(), v[total - 40:])
    # what a ring refuses: a range that wraps, keys it no longer holds, rows past max_context
    z = _dev(np.zeros((64, KH * D), np.float16))
    for call, status in ((lambda: kv.append(0, 0, 1000 - 40 + 24, z, z), capi.ERR_CAPACITY),  # 984 % 256 + 64 > 256
                         (lambda: _swa(gpu_ctx, kv, q[:1].reshape(1, 1, H, D), [1000], 400, H, scale), capi.ERR_CAPACITY),
                         (lambda: _swa(gpu_ctx, kv, q[:1].reshape(1, 1, H, D), [1000], 0, H, scale), capi.ERR_CAPACITY),
                         (lambda: kv.append(0, 0, 1000, z, z), capi.ERR_CAPACITY)):
        with pytest.raises(TinyTitanHIPError) as e:
            call()
        assert e.value.status == status
    kv.close()


def test_ring_cache_through_the_fused_epilogue(gpu_ctx):
    # rows written by the fused epilogue land at position % capacity and are rotated by their position
    import torch
    from tinytitan_amd.engine import KVCacheManager, QKVEpilogue
    H, KH, D, cap = 8, 2, 128, 128
    r = np.random.default_rng(11)
    ring = KVCacheManager(gpu_ctx, 1, KH, D, slots=2, max_context=4096, ring_capacity=cap)
    flat = KVCacheManager(gpu_ctx, 1, KH, D, slots=2, max_context=4096, initial_capacity=4096)
    w = torch.from_numpy(((1.0 + 0.2 * r.standard_normal(D)).astype(np.float32).view(np.uint32) >> 16).astype(np.int16)).cuda()
    for n_seq, rows, positions in ((1, 70, [300]), (2, 1, [1000, 2047]), (1, 33, [3 * cap - 33])):
        T = n_seq * rows
        packed = _dev(r.standard_normal((T, H, 2 * D)).astype(np.float16))
        kp = _dev(r.standard_normal((T, KH * D)).astype(np.float16))
        vp = _dev(r.standard_normal((T, KH * D)).astype(np.float16))
        res = []
        for cache in (ring, flat):
            qo = torch.empty((T, H * D), dtype=torch.float16, device="cuda")
            go = torch.empty_like(qo)
            torch.cuda.synchronize()
            QKVEpilogue(gpu_ctx).encode(cache, 0, packed, kp, vp, w, w, qo, go, H, positions, rows, 1e-6, 32, 1e7,
                                        slots=list(range(n_seq)))
            gpu_ctx.synchronize()
            res.append([cache.read(0, s, positions[s], rows) for s in range(n_seq)] + [qo, go])
        for a, b in zip(res[0][:-2], res[1][:-2]):
            assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
        assert torch.equal(res[0][-2], res[1][-2]) and torch.equal(res[0][-1], res[1][-1])
    ring.close()
    flat.close()


@pytest.mark.parametrize("ring", [False, True])
def test_verify_rows_with_a_window_equal_windowed_decodes(gpu_ctx, ring):
    # row r of a windowed verify pass == a windowed decode at start + r, on a linear cache and on a ring
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, W, start, window, cap = 16, 2, 256, 4, 700, 200, 256
    r = np.random.default_rng(5 + ring)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=2, max_context=1024, initial_capacity=1024, ring_capacity=cap if ring else 0)
    ks, vs = [], []
    for s in range(2):
        k = r.standard_normal((start + W, KH, D)).astype(np.float16)
        v = r.standard_normal((start + W, KH, D)).astype(np.float16)
        for at in range(0, start + W, 64):  # appends of 64 never wrap a 256-row ring
            kd, vd = _dev(k[at:at + 64]), _dev(v[at:at + 64])
            torch.cuda.synchronize()
            kv.append(0, s, at, kd, vd)
            gpu_ctx.synchronize()
        ks.append(k.astype(np.float32).reshape(start + W, -1))
        vs.append(v.astype(np.float32).reshape(start + W, -1))
    q = r.standard_normal((2, W, H, D)).astype(np.float16)
    g = r.standard_normal((2, W, H, D)).astype(np.float16)
    qd, gd = _dev(q), _dev(g)
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qd, out, H, [start, start], W, 0.0625, [0, 1], gate=gd, window=window)
    gpu_ctx.synchronize()
    ver = out.float().cpu().numpy()
    for s in range(2):
        for row in range(W):
            n = start + row + 1
            want = oracle.attention_ref(q[s, row].astype(np.float32), ks[s][:n], vs[s][:n], D, H, KH, n, window, 0.0625)
            want = want.reshape(H, D) / (1 + np.exp(-g[s, row].astype(np.float64)))
            _check(ver[s, row], want, f"sequence {s} row {row}")
    dec = _swa(gpu_ctx, kv, q[:, :1], [start + 1, start + 1], window, H, 0.0625, gate=g[:, :1])
    assert np.abs(dec[:, 0] - ver[:, 0]).max() <= 1e-3
    kv.close()
