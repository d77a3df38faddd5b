"""Quantised KV caches (8 and 4 bits) through the C ABI.

Byte work -- the quantiser fused into the append, the stored rows, their round trip -- is held
bit-exact against the oracle's restatement of kv_cache_quantize_affine
(sources/TinyTitanCore/Metal/Quant/kv_cache_quantize.metal:7-73).  Attention over a quantised
cache is held to the attention path's own bar (max-abs 2e-3, mean-abs 2e-4) against the oracle's
attention over the rows its loader (attention.metal:89-117) gives back, and to the reference
test's bar (KVCacheQuantizedAttentionTests.swift) against the fp16 result."""
import numpy as np
import pytest

import oracle
from tests.helpers import MAX_ABS, MEAN_ABS, f16_round
from tests.test_gpu_attention_api import _check, _decode, _dev, _prefill

pytestmark = pytest.mark.gpu


def _cache(ctx, bits, kh, d, tokens, slots=1, layers=1, capacity=None):
    from tinytitan_amd.engine import KVCacheManager
    cap = capacity or max(32, tokens)
    return KVCacheManager(ctx, layers, kh, d, slots=slots, max_context=max(cap, tokens), initial_capacity=cap,
                          precision_bits=bits)


def _append(ctx, kv, layer, slot, position, k, v):
    import torch
    kd, vd = _dev(k), _dev(v)
    torch.cuda.synchronize()
    kv.append(layer, slot, position, kd, vd)
    ctx.synchronize()


def _rows(n, kh, d, seed, spread=True):
    r = np.random.default_rng(seed)
    scale = r.uniform(0.05, 3.0, size=(n, 1, 1)) if spread else 1.0
    k = (r.standard_normal((n, kh, d)) * scale).astype(np.float16)
    v = (r.standard_normal((n, kh, d)) * scale).astype(np.float16)
    return k, v


def _dequantised(x, bits):
    """What the oracle's loader reads back from the oracle's quantiser, [n][kh][d] fp32."""
    n, kh, d = x.shape
    rows = oracle.kv_quantize_rows(x.reshape(n, kh * d).astype(np.float32), bits)
    return oracle.kv_dequantize_rows(rows, kh * d, bits).reshape(n, kh, d)


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("kh,d", [(2, 256), (4, 128), (3, 64)])
def test_appended_rows_are_the_oracles_bytes(gpu_ctx, bits, kh, d):
    # rows land at ragged positions across block edges, in two appends and a second slot
    n = 101
    k, v = _rows(n, kh, d, seed=bits * 1000 + d)
    k[5, 0, :64] = 0.25  # a constant group: scale 0
    kv = _cache(gpu_ctx, bits, kh, d, 160, slots=2)
    assert kv.precision_bits == bits and kv.token_stride_bytes == oracle.kv_row_layout(kh * d, bits)[0]
    _append(gpu_ctx, kv, 0, 1, 7, k[:40], v[:40])
    _append(gpu_ctx, kv, 0, 1, 47, k[40:], v[40:])
    got_k, got_v = kv.export_rows(0, 1, 7, n)
    want_k = oracle.kv_quantize_rows(k.reshape(n, -1).astype(np.float32), bits)
    want_v = oracle.kv_quantize_rows(v.reshape(n, -1).astype(np.float32), bits)
    assert np.array_equal(got_k.cpu().numpy(), want_k)
    assert np.array_equal(got_v.cpu().numpy(), want_v)
    # the other slot and the rows in front are untouched (zero levels, zero scale and bias)
    front_k, front_v = kv.export_rows(0, 1, 0, 7)
    other_k, _ = kv.export_rows(0, 0, 0, 128)
    assert not front_k.any() and not front_v.any() and not other_k.any()
    # dequantised read == the oracle's loader, rounded to fp16 (the product-sum may be fused: one ulp)
    rk, rv = kv.read(0, 1, 7, n)
    for got, want in ((rk, _dequantised(k, bits)), (rv, _dequantised(v, bits))):
        g = got.float().cpu().numpy()
        assert (np.abs(g - want) <= 2.0 ** -10 * np.abs(want) + 1e-7).all()
    kv.close()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("kh,d", [(2, 256), (4, 128), (3, 64)])
def test_a_chunks_whole_blocks_are_the_oracles_bytes(gpu_ctx, bits, kh, d):
    """A chunk's whole 32-token blocks are quantised a workgroup per block (its ragged ends a wavefront per group, like
    single rows): the same stored bytes as the oracle's quantiser either way, at a ragged start, at an aligned
    start, and from a source whose rows are not 16-byte aligned (everything by rows)."""
    import torch
    n, whole, cap = 2200, 1024, 4096  # (ragged chunks up to 2048 rows and aligned ones up to 768 go by rows altogether)
    k, v = _rows(n, kh, d, seed=bits * 77 + d)
    k[33, kh - 1, -64:] = -1.5  # constant groups inside whole blocks: scale 0
    v[64, 0, :64] = 0.0
    want_k = oracle.kv_quantize_rows(k.reshape(n, -1).astype(np.float32), bits)
    want_v = oracle.kv_quantize_rows(v.reshape(n, -1).astype(np.float32), bits)
    kv = _cache(gpu_ctx, bits, kh, d, cap, slots=3)
    _append(gpu_ctx, kv, 0, 0, 19, k, v)        # 13 rows, 68 blocks, 11 rows
    _append(gpu_ctx, kv, 0, 1, 64, k[:whole], v[:whole])  # 32 blocks, nothing else
    # rows at a 2-byte offset inside a wider buffer: the 16-byte pieces of the block form do not apply
    wide_k = torch.zeros((n, kh * d + 8), dtype=torch.float16, device="cuda")
    wide_v = torch.zeros_like(wide_k)
    wide_k[:, 1:1 + kh * d] = _dev(k).reshape(n, -1)
    wide_v[:, 1:1 + kh * d] = _dev(v).reshape(n, -1)
    torch.cuda.synchronize()
    kv.append(0, 2, 19, wide_k[:, 1:1 + kh * d], wide_v[:, 1:1 + kh * d], token_stride=kh * d + 8, n_tokens=n)
    gpu_ctx.synchronize()
    for slot, first, count in ((0, 19, n), (1, 64, whole), (2, 19, n)):
        got_k, got_v = kv.export_rows(0, slot, first, count)
        assert np.array_equal(got_k.cpu().numpy(), want_k[:count]), (slot, "K")
        assert np.array_equal(got_v.cpu().numpy(), want_v[:count]), (slot, "V")
    # what lies around the chunks is untouched
    for slot, first, count in ((0, 0, 19), (0, 19 + n, cap - 19 - n), (1, 0, 64), (1, 64 + whole, cap - 64 - whole)):
        around_k, around_v = kv.export_rows(0, slot, first, count)
        assert not around_k.any() and not around_v.any(), (slot, first)
    kv.close()


@pytest.mark.parametrize("bits", [8, 4])
def test_stored_rows_round_trip_and_growth(gpu_ctx, bits):
    kh, d, n = 2, 256, 77
    k, v = _rows(n, kh, d, seed=bits)
    a = _cache(gpu_ctx, bits, kh, d, 1024, capacity=96)
    _append(gpu_ctx, a, 0, 0, 3, k, v)
    a.advance(0, 3 + n)
    rows_k, rows_v = a.export_rows(0, 0, 3, n)
    a.reserve(1000)  # growth copies whole blocks
    assert a.capacity_tokens >= 1000
    again_k, again_v = a.export_rows(0, 0, 3, n)
    assert (again_k == rows_k).all() and (again_v == rows_v).all()
    b = _cache(gpu_ctx, bits, kh, d, 128)
    b.import_rows(0, 0, 20, rows_k, rows_v)  # other positions: other keys inside the blocks
    gpu_ctx.synchronize()
    back_k, back_v = b.export_rows(0, 0, 20, n)
    assert (back_k == rows_k).all() and (back_v == rows_v).all()
    a.close()
    b.close()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("H,KH,D,T", [(16, 2, 256, 1187), (8, 2, 256, 33), (8, 4, 128, 300), (24, 2, 64, 333),
                                      (32, 1, 128, 70)])
def test_decode_over_quantised_cache(gpu_ctx, bits, H, KH, D, T):
    k, v = _rows(T, KH, D, seed=T + bits, spread=False)
    r = np.random.default_rng(T)
    q = r.standard_normal((1, H, D)).astype(np.float16)
    g = r.standard_normal((1, H, D)).astype(np.float16)
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    scale = D ** -0.5
    kq, vq = _dequantised(k, bits), _dequantised(v, bits)
    for length in (T, T - 1, 1):
        got = _decode(gpu_ctx, kv, q, [length], H, scale, gate=g)
        want = oracle.decode(q[0].astype(np.float32), kq[:length], vq[:length], H, KH, D, scale, gate=g[0].astype(np.float32))
        _check(got[0], want, f"{bits}-bit decode over {length} keys")
    kv.close()


@pytest.mark.parametrize("bits,tolerance", [(8, 0.02), (4, 0.20)])
def test_reference_decode_case(gpu_ctx, bits, tolerance):
    # KVCacheQuantizedAttentionTests.swift:9-83 on its own seeded inputs, judged its way: against
    # the fp16-input reference at RelError < 0.02 (8 bits) / 0.20 (4 bits).
    H, KH, D, T = 16, 2, 256, 8
    draws = oracle.fill_uniform(0x4B56, f"kv-cache-{bits}", -0.5, 0.5, H * D + 2 * T * KH * D)
    q = f16_round(draws[:H * D]).reshape(1, H, D)
    k = f16_round(draws[H * D:H * D + T * KH * D]).reshape(T, KH, D)
    v = f16_round(draws[H * D + T * KH * D:]).reshape(T, KH, D)
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k.astype(np.float16), v.astype(np.float16))
    got = _decode(gpu_ctx, kv, q.astype(np.float16), [T], H, 0.0625)[0]
    want = oracle.attention_ref(q.reshape(-1), k.reshape(T, -1), v.reshape(T, -1), D, H, KH, T, 0, 0.0625).reshape(H, D)
    rel = np.abs(got - want).max() / max(np.abs(want).max(), 1e-6)
    assert rel < tolerance
    # and to our own bar against the oracle's loader
    want_q = oracle.decode(q[0], _dequantised(k, bits), _dequantised(v, bits), H, KH, D, 0.0625)
    _check(got, want_q, "reference decode case")
    kv.close()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("start,chunk", [(0, 70), (4, 4), (100, 129), (2100, 64), (0, 333), (8100, 200), (3000, 130),
                                         (0, 1100)])
def test_prefill_over_quantised_cache(gpu_ctx, bits, start, chunk):
    # quantizedChunkedPrefillTracksFP16Kernel (KVCacheQuantizedAttentionTests.swift:101-178) is the (4, 4) case.
    # Chunks of 128 rows and more over 2560 keys and more, or with enough rows to fill a quarter of the chip, go
    # through fp16 pages dequantised once per call and the MFMA chunk kernel (whole: (0, 1100); over key ranges:
    # (8100, 200), (3000, 130)); the others through the split-K kernel reading the levels.
    H, KH, D = 16, 2, 256
    kv_valid = start + chunk
    k, v = _rows(kv_valid, KH, D, seed=start + chunk + bits, spread=False)
    r = np.random.default_rng(start)
    q = r.standard_normal((chunk, H * D)).astype(np.float16)
    g = r.standard_normal((chunk, H * D)).astype(np.float16)
    kv = _cache(gpu_ctx, bits, KH, D, kv_valid)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    got = _prefill(gpu_ctx, kv, q, start, chunk, kv_valid, H, 0.0625, gate=g)
    kq, vq = _dequantised(k, bits).reshape(kv_valid, -1), _dequantised(v, bits).reshape(kv_valid, -1)
    sig = 1 + np.exp(-g.astype(np.float64))
    want = oracle.attention_batch(q.astype(np.float32), kq, vq, chunk, start, H, KH, D, 0.0625, threads=4).reshape(chunk, -1) / sig
    _check(got, want, f"{bits}-bit prefill of {chunk} at {start}")
    # the reference's bar for this path: within 0.025 / 0.20 of the fp16 kernel's result
    plain = oracle.attention_batch(q.astype(np.float32), k.reshape(kv_valid, -1).astype(np.float32),
                                   v.reshape(kv_valid, -1).astype(np.float32), chunk, start, H, KH, D, 0.0625,
                                   threads=4).reshape(chunk, -1) / sig
    assert np.abs(got - plain).max() / np.abs(plain).max() < (0.025 if bits == 8 else 0.20)
    kv.close()


@pytest.mark.parametrize("bits", [8, 4])
def test_verify_rows_equal_decode_steps_and_batch(gpu_ctx, bits):
    import torch
    from tinytitan_amd.engine import Attention
    H, KH, D, W, ctx_len = 16, 2, 256, 4, 700
    kv = _cache(gpu_ctx, bits, KH, D, 1024, slots=3)
    ks, vs = [], []
    for s in range(3):
        k, v = _rows(ctx_len + W, KH, D, seed=s + bits, spread=False)
        _append(gpu_ctx, kv, 0, s, 0, k, v)
        ks.append(k)
        vs.append(v)
    r = np.random.default_rng(bits)
    q = r.standard_normal((3, W, H, D)).astype(np.float16)
    g = r.standard_normal((3, W, H, D)).astype(np.float16)
    qd, gd = _dev(q), _dev(g)
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qd, out, H, [ctx_len] * 3, W, 0.0625, [0, 1, 2], gate=gd)
    gpu_ctx.synchronize()
    ver = out.float().cpu().numpy()
    for s in range(3):
        kq, vq = _dequantised(ks[s], bits), _dequantised(vs[s], bits)
        for row in range(W):
            n = ctx_len + row + 1
            want = oracle.decode(q[s, row].astype(np.float32), kq[:n], vq[:n], H, KH, D, 0.0625, gate=g[s, row].astype(np.float32))
            _check(ver[s, row], want, f"{bits}-bit verify row {row} of sequence {s}")
    dec = _decode(gpu_ctx, kv, q[:, 0], [ctx_len + 1] * 3, H, 0.0625, gate=g[:, 0])
    assert np.abs(dec - ver[:, 0]).max() <= 1e-3
    kv.close()


def test_long_context_decode_8_bit(gpu_ctx):
    # the metric's shape (16/2/256, 32768 keys) over an 8-bit cache
    H, KH, D, T = 16, 2, 256, 32768
    k, v = _rows(T, KH, D, seed=32768, spread=False)
    r = np.random.default_rng(1)
    q = r.standard_normal((1, H, D)).astype(np.float16)
    kv = _cache(gpu_ctx, 8, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    got = _decode(gpu_ctx, kv, q, [T], H, 0.0625)
    want = oracle.decode(q[0].astype(np.float32), _dequantised(k, 8), _dequantised(v, 8), H, KH, D, 0.0625)
    _check(got[0], want, "8-bit decode over 32768 keys")
    kv.close()


@pytest.mark.parametrize("bits", [8, 4])
def test_snapshot_carries_stored_rows(gpu_ctx, bits):
    kh, d, n, layers = 2, 256, 45, 2
    a = _cache(gpu_ctx, bits, kh, d, 256, layers=layers, capacity=64)
    data = [_rows(n, kh, d, seed=10 * bits + layer) for layer in range(layers)]
    for layer, (k, v) in enumerate(data):
        _append(gpu_ctx, a, layer, 0, 0, k, v)
    a.advance(0, n)
    lengths = a.snapshot_segment_lengths(n)
    stride = oracle.kv_row_layout(kh * d, bits)[0]
    assert lengths == [n * stride] * (2 * layers)
    payload = bytearray()
    a.append_snapshot_payload(payload, lengths)
    want = b"".join(oracle.kv_quantize_rows(x.reshape(n, -1).astype(np.float32), bits).tobytes()
                    for k, v in data for x in (k, v))
    assert bytes(payload) == want  # the wire format: K rows then V rows per layer, stored row format
    b = _cache(gpu_ctx, bits, kh, d, 256, layers=layers, capacity=32)
    b.restore_snapshot(n, lengths, payload)
    assert b.position(0) == n
    for layer in range(layers):
        ak, av = a.export_rows(layer, 0, 0, n)
        bk, bv = b.export_rows(layer, 0, 0, n)
        assert (ak == bk).all() and (av == bv).all()
    a.close()
    b.close()


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("H,KH,D,rot,n_seq,rows,positions", [
    (16, 2, 256, 64, 1, 1, [37]), (16, 2, 256, 64, 3, 1, [0, 31, 100]), (16, 2, 256, 64, 1, 75, [5]),
    (16, 2, 256, 64, 2, 4, [60, 30]), (8, 2, 128, 32, 1, 40, [0]), (4, 1, 64, 16, 2, 3, [7, 33])])
def test_fused_epilogue_writes_the_same_rows(gpu_ctx, bits, H, KH, D, rot, n_seq, rows, positions):
    # The fused epilogue on a quantised cache == the fused epilogue on an fp16 cache, its K/V rows read
    # back and appended to a quantised cache: the same fp16 rows through the same quantiser, so the
    # stored bytes are identical (and those of tt_hip_kv_append are the oracle's, tested above).
    import torch
    from tinytitan_amd.engine import KVCacheManager, QKVEpilogue
    r = np.random.default_rng(bits * 100 + D + rows)
    T = n_seq * rows
    packed = _dev(r.standard_normal((T, H, 2 * D)).astype(np.float16))
    k = _dev((2.0 * r.standard_normal((T, KH * D))).astype(np.float16))
    v = _dev(r.standard_normal((T, KH * D)).astype(np.float16))
    w = torch.from_numpy(((1.0 + 0.2 * r.standard_normal(D)).astype(np.float32).view(np.uint32) >> 16).astype(np.int16)).cuda()
    slots = list(range(n_seq))
    cap = 128
    plain = KVCacheManager(gpu_ctx, 1, KH, D, slots=n_seq, max_context=cap, initial_capacity=cap)
    quant = _cache(gpu_ctx, bits, KH, D, cap, slots=n_seq)
    want = _cache(gpu_ctx, bits, KH, D, cap, slots=n_seq)
    outs = []
    for cache in (plain, quant):
        q = torch.full((T, H * D), float("nan"), dtype=torch.float16, device="cuda")
        g = torch.full_like(q, float("nan"))
        torch.cuda.synchronize()
        QKVEpilogue(gpu_ctx).encode(cache, 0, packed, k, v, w, w, q, g, H, positions, rows, 1e-6, rot, 1e7, slots=slots)
        gpu_ctx.synchronize()
        outs.append((q, g))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])  # q and gate do not depend on the cache
    for s in range(n_seq):
        kr, vr = plain.read(0, s, positions[s], rows)
        want.append(0, s, positions[s], kr.reshape(rows, -1).contiguous(), vr.reshape(rows, -1).contiguous())
        gpu_ctx.synchronize()
        got_k, got_v = quant.export_rows(0, s, positions[s], rows)
        want_k, want_v = want.export_rows(0, s, positions[s], rows)
        assert torch.equal(got_k, want_k) and torch.equal(got_v, want_v), f"sequence {s}"
        if positions[s] > 0:  # rows in front stay untouched
            front_k, front_v = quant.export_rows(0, s, 0, positions[s])
            assert not front_k.any() and not front_v.any()
    for cache in (plain, quant, want):
        cache.close()


def test_graph_replay_over_a_quantised_cache(gpu_ctx):
    # a decode and a staged prefill chunk of an 8-bit cache captured in one graph: replays equal the
    # eager results; a chunk whose staging store would have to grow while capturing is refused
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import Attention, HIPContext, PrefillAttention, PrefillAttentionParams, TinyTitanHIPError
    H, KH, D, T, chunk = 16, 2, 256, 5200, 160  # (from 786,432 / 160 = 4,915 keys on such a chunk runs on dequantised pages)
    ctx = HIPContext(gpu_ctx.device)  # its own scratch and staging stores, whatever ran before
    k, v = _rows(T, KH, D, seed=77, spread=False)
    kv = _cache(ctx, 8, KH, D, T)
    _append(ctx, kv, 0, 0, 0, k, v)
    r = np.random.default_rng(7)
    q1, qc = _dev(r.standard_normal((1, 1, H, D)).astype(np.float16)), _dev(r.standard_normal((chunk, H * D)).astype(np.float16))
    o1, oc = torch.zeros_like(q1), torch.zeros_like(qc)
    params = PrefillAttentionParams(T - chunk, chunk, T, H, 0.0625, H * D, H * D, H * D)
    att, pre = Attention(ctx), PrefillAttention(ctx)

    def both():
        att.encode_full(kv, 0, q1, o1, H, [T], 0.0625)
        pre.encode_causal(kv, 0, 0, qc, oc, params)

    ctx.graph_begin()
    with pytest.raises(TinyTitanHIPError) as e:
        pre.encode_causal(kv, 0, 0, qc, oc, params)  # first use: the staging store does not exist yet
    assert e.value.status == capi.ERR_BUSY
    ctx.graph_end().close()
    torch.cuda.synchronize()
    both()
    ctx.synchronize()
    eager = (o1.clone(), oc.clone())
    ctx.graph_begin()
    both()
    graph = ctx.graph_end()
    for replay in range(3):
        o1.zero_()
        oc.zero_()
        torch.cuda.synchronize()
        graph.launch()
        ctx.synchronize()
        assert torch.equal(o1, eager[0]) and torch.equal(oc, eager[1]), f"replay {replay}"
        att.encode_full(kv, 0, q1, o1, H, [T - 1 - replay], 0.0625)  # eager work between replays
        ctx.synchronize()
    graph.close()
    kv.close()
    ctx.close()


def test_what_a_quantised_cache_refuses(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, TinyTitanHIPError
    with pytest.raises(TinyTitanHIPError) as e:
        KVCacheManager(gpu_ctx, 1, 2, 256, precision_bits=5)
    assert e.value.status == capi.ERR_INVALID_ARGUMENT
    kv = _cache(gpu_ctx, 8, 2, 256, 64)
    rows = torch.zeros((1, 542), dtype=torch.uint8, device="cuda")
    with pytest.raises(TinyTitanHIPError) as e:
        kv.import_rows(0, 0, 0, rows, rows)  # a stride below the stored row
    assert e.value.status == capi.ERR_SHAPE
    kv.close()


@pytest.mark.parametrize("bits", [16, 8, 4])
@pytest.mark.parametrize("D,H,KH", [(256, 16, 2), (128, 8, 2), (64, 4, 4)])
def test_row_maxima_that_keep_growing_rescale_the_accumulators(gpu_ctx, bits, D, H, KH):
    # Scores that rise along the context: every few key blocks a row's reference maximum moves again and the
    # accumulators -- by then far from zero -- are rescaled (random keys move it once or twice, in the first
    # blocks).  A decode row (16-row tiles) and a four-row verify pass (32-row tiles) over the same cache.
    import torch
    from tinytitan_amd.engine import Attention
    T, W = 2048 + 4, 4
    r = np.random.default_rng(D + bits)
    u = r.choice([-1.0, 1.0], size=D)
    ramp = np.linspace(0.0, 1.0, T)[:, None, None]
    k = (u[None, None, :] * ramp * 224.0 / D + 0.02 * r.standard_normal((T, KH, D))).astype(np.float16)
    v = r.standard_normal((T, KH, D)).astype(np.float16)
    # score of head h at key j: scale * D * (224 / D) * (j / T) * (0.5 + 1.5 h / H) = 7 .. 28 at the last key (10 .. 40 in
    # log2 units, against a threshold of 4; larger scores would test the rounding of a dequantised key instead)
    q = (u[None, None, :] * (0.5 + 1.5 * np.arange(H)[None, :, None] / H) * np.ones((W, 1, 1))
         + 0.02 * r.standard_normal((W, H, D))).astype(np.float16)
    kv = _cache(gpu_ctx, bits, KH, D, T)
    _append(gpu_ctx, kv, 0, 0, 0, k, v)
    kq, vq = (k.astype(np.float32), v.astype(np.float32)) if bits == 16 else (_dequantised(k, bits), _dequantised(v, bits))
    scale = 0.0625
    qd = _dev(q[None])
    out = torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    Attention(gpu_ctx).encode_verify_rows(kv, 0, qd, out, H, [T - W], W, scale, [0])
    gpu_ctx.synchronize()
    ver = out.float().cpu().numpy()[0]
    for row in range(W):
        n = T - W + row + 1
        want = oracle.decode(q[row].astype(np.float32), kq[:n].reshape(n, -1), vq[:n].reshape(n, -1), H, KH, D, scale)
        _check(ver[row], want, f"{bits}-bit verify row {row} under rising scores")
    dec = _decode(gpu_ctx, kv, q[W - 1:W], [T], H, scale)
    want = oracle.decode(q[W - 1].astype(np.float32), kq.reshape(T, -1), vq.reshape(T, -1), H, KH, D, scale)
    _check(dec[0], want, f"{bits}-bit decode under rising scores")
    kv.close()
