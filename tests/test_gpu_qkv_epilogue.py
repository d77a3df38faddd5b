"""The pre-attention epilogue (split [query ; gate], per-head q/k RMS norm, NeoX sub-dim RoPE, K/V
cache write) through the C ABI against the oracle's restatement of CPUQwen35.attention
(sources/TinyTitan/CPUEngine/CPUQwen35.swift:266-300).

Bar for this element-wise stage: the kernel computes in fp32 from the same fp16 inputs and rounds to
fp16 once, so it must land on the oracle's fp16-rounded value or its neighbour:
|gpu - oracle_fp32| <= 2^-10 * |oracle_fp32| + 1e-6 (one fp16 ulp; the fp32 differences -- order of
the sum of squares, cos/sin implementations -- are four orders of magnitude below that and only
matter at a rounding boundary).  The gate and V are copies: bit-exact.  The rotation frequencies are
computed on the host with the same C library powf as the oracle, so large positions need no slack."""
import numpy as np
import pytest

import oracle

pytestmark = pytest.mark.gpu

EPS = 1e-6
THETA = 1e7


def _bf16_bits(x32):
    """fp32 -> bfloat16 bit patterns (round to nearest even) and the fp32 values they stand for."""
    u = x32.astype(np.float32).view(np.uint32)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)
    return r, (r.astype(np.uint32) << 16).view(np.float32)


def _within_one_ulp(got, ref32, what):
    tol = 2.0 ** -10 * np.abs(ref32) + 1e-6
    bad = np.abs(got.astype(np.float64) - ref32.astype(np.float64)) > tol
    assert not bad.any(), f"{what}: {bad.sum()} elements off by more than one fp16 ulp, worst " \
                          f"{np.abs(got - ref32).max():.3e}"


def _run(gpu_ctx, H, KH, D, rot, n_seq, rows, positions, slots, seed, qp_pad=0, kv_pad=0, q_pad=0, g_pad=0, shift=0,
         capacity=None):
    import torch
    from tinytitan_amd.engine import KVCacheManager, QKVEpilogue
    r = np.random.default_rng(seed)
    T = n_seq * rows
    packed = r.standard_normal((T, H, 2 * D)).astype(np.float16)
    k = (2.5 * r.standard_normal((T, KH * D))).astype(np.float16)
    v = r.standard_normal((T, KH * D)).astype(np.float16)
    qw_bits, qw = _bf16_bits(1.0 + 0.3 * r.standard_normal(D))
    kw_bits, kw = _bf16_bits(1.0 + 0.3 * r.standard_normal(D))
    cap = capacity or max(64, max(positions) + rows)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=max(slots) + 1, max_context=cap, initial_capacity=cap)

    def padded(x, pad):  # token-major rows with `pad` extra halves per token and `shift` halves in front
        width = x.shape[1]
        buf = torch.full((T * (width + pad) + shift,), 77.0, dtype=torch.float16)
        buf[shift:].view(T, width + pad)[:, :width] = torch.from_numpy(x.reshape(T, width))
        return buf.cuda(), width + pad

    pd, qp_stride = padded(packed.reshape(T, -1), qp_pad)
    kd, kv_stride = padded(k, kv_pad)
    vd, _ = padded(v, kv_pad)
    q_stride, g_stride = H * D + q_pad, H * D + g_pad
    q_out = torch.full((T * q_stride + shift,), float("nan"), dtype=torch.float16, device="cuda")
    g_out = torch.full((T * g_stride + shift,), float("nan"), dtype=torch.float16, device="cuda")
    qwd = torch.from_numpy(qw_bits.view(np.int16)).cuda()
    kwd = torch.from_numpy(kw_bits.view(np.int16)).cuda()
    torch.cuda.synchronize()
    QKVEpilogue(gpu_ctx).encode(kv, 0, pd[shift:], kd[shift:], vd[shift:], qwd, kwd, q_out[shift:], g_out[shift:], H,
                                list(positions), rows, EPS, rot, THETA, slots=list(slots), q_packed_stride=qp_stride,
                                kv_stride=kv_stride, q_stride=q_stride, gate_stride=g_stride)
    gpu_ctx.synchronize()
    got_q = q_out[shift:].view(T, q_stride).float().cpu().numpy()
    got_g = g_out[shift:].view(T, g_stride).cpu().numpy()
    assert np.isnan(got_q[:, H * D:]).all() and np.isnan(got_g[:, H * D:].astype(np.float32)).all()  # padding untouched
    for s in range(n_seq):
        sl = slice(s * rows, (s + 1) * rows)
        want_q, want_g, want_k = oracle.qkv_epilogue(packed[sl].astype(np.float32), k[sl].astype(np.float32), rows, H, KH, D,
                                                     qw, kw, EPS, rot, THETA, positions[s])
        _within_one_ulp(got_q[sl, :H * D], want_q, f"q of sequence {s}")
        assert np.array_equal(got_g[sl, :H * D], packed[sl, :, D:].reshape(rows, H * D)), "gate is a copy"
        kr, vr = kv.read(0, slots[s], positions[s], rows)
        _within_one_ulp(kr.float().cpu().numpy().reshape(rows, KH * D), want_k, f"cached K of sequence {s}")
        assert np.array_equal(vr.cpu().numpy().reshape(rows, KH * D), v[sl]), "cached V is a copy"
    return kv


@pytest.mark.parametrize("H,KH,D,rot", [(16, 2, 256, 64), (8, 2, 128, 32), (4, 1, 64, 16), (16, 2, 256, 0),
                                        (8, 2, 256, 256)])
def test_decode_rows(gpu_ctx, H, KH, D, rot):
    # one token per sequence, scattered slots and positions (incl. 0: no rotation, and a block edge)
    kv = _run(gpu_ctx, H, KH, D, rot, 5, 1, [0, 31, 32, 1000, 4095], [3, 0, 4, 1, 2], seed=D + rot, capacity=4096)
    kv.close()


@pytest.mark.parametrize("position,rows", [(0, 128), (7, 200), (33, 31), (64, 64), (31, 2), (5, 40), (0, 384), (7, 500), (33, 415), (64, 383)])
def test_chunk_whole_blocks_and_ragged_edges(gpu_ctx, position, rows):
    # (from 384 rows on a chunk's whole 32-token blocks are written by the block path, below by the row path)
    kv = _run(gpu_ctx, 16, 2, 256, 64, 1, rows, [position], [1], seed=position * 131 + rows)
    # rows outside the chunk still hold the zeros they were allocated with
    if position > 0:
        kr, vr = kv.read(0, 1, 0, position)
        assert not kr.any() and not vr.any()
    kv.close()


def test_verify_rows_of_several_sequences(gpu_ctx):
    kv = _run(gpu_ctx, 16, 2, 256, 64, 3, 4, [100, 65, 30], [0, 2, 1], seed=5, capacity=256)
    kv.close()


def test_padded_strides_and_unaligned_buffers(gpu_ctx):
    # strides that are not multiples of 4 halves and buffers starting 1 half in: the scalar path
    kv = _run(gpu_ctx, 8, 2, 128, 32, 1, 70, [9], [0], seed=6, qp_pad=3, kv_pad=5, q_pad=7, g_pad=9, shift=1)
    kv.close()
    kv = _run(gpu_ctx, 16, 2, 256, 64, 1, 45, [20], [0], seed=7, qp_pad=8, kv_pad=16, q_pad=24, g_pad=4)
    kv.close()


def test_large_positions(gpu_ctx):
    # angle = position * frequency in fp32 at positions where one ulp of a frequency would move it by 4e-3
    kv = _run(gpu_ctx, 16, 2, 256, 64, 2, 2, [65534, 40000], [0, 1], seed=8, capacity=65536)
    kv.close()


def test_feeds_the_attention_kernels(gpu_ctx):
    # epilogue -> advance -> prefill attention, against the oracle's epilogue -> attention_batch
    import torch
    from tinytitan_amd.engine import KVCacheManager, PrefillAttention, PrefillAttentionParams, QKVEpilogue
    H, KH, D, T = 16, 2, 256, 96
    r = np.random.default_rng(9)
    packed = r.standard_normal((T, H, 2 * D)).astype(np.float16)
    k = r.standard_normal((T, KH * D)).astype(np.float16)
    v = r.standard_normal((T, KH * D)).astype(np.float16)
    qw_bits, qw = _bf16_bits(1.0 + 0.2 * r.standard_normal(D))
    kw_bits, kw = _bf16_bits(1.0 + 0.2 * r.standard_normal(D))
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=128, initial_capacity=128)
    q = torch.empty((T, H * D), dtype=torch.float16, device="cuda")
    g = torch.empty_like(q)
    out = torch.empty_like(q)
    args = [torch.from_numpy(x).cuda() for x in (packed, k, v)]
    qwd, kwd = torch.from_numpy(qw_bits.view(np.int16)).cuda(), torch.from_numpy(kw_bits.view(np.int16)).cuda()
    torch.cuda.synchronize()
    QKVEpilogue(gpu_ctx).encode(kv, 0, args[0], args[1], args[2], qwd, kwd, q, g, H, 0, T, EPS, 64, THETA)
    kv.advance(0, T)
    PrefillAttention(gpu_ctx).encode_causal(kv, 0, 0, q, out, PrefillAttentionParams(0, T, T, H, 0.0625, H * D, H * D), gate=g)
    gpu_ctx.synchronize()
    want_q, want_g, want_k = oracle.qkv_epilogue(packed.astype(np.float32), k.astype(np.float32), T, H, KH, D, qw, kw, EPS,
                                                 64, THETA, 0)
    f16 = lambda x: x.astype(np.float16).astype(np.float32)
    want = oracle.attention_batch(f16(want_q), f16(want_k), v.astype(np.float32), T, 0, H, KH, D, 0.0625, gate=want_g)
    diff = np.abs(out.float().cpu().numpy() - f16(want.reshape(T, -1)))
    assert diff.max() <= 2e-3 and diff.mean() <= 2e-4  # the attention path's own bar
    kv.close()


def test_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, QKVEpilogue, TinyTitanHIPError
    H, KH, D = 16, 2, 256
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=64, initial_capacity=64)
    z = lambda *s: torch.zeros(s, dtype=torch.float16, device="cuda")
    w = torch.zeros(D, dtype=torch.int16, device="cuda")
    ep = QKVEpilogue(gpu_ctx)

    def call(**kw):
        a = dict(num_q_heads=H, positions=0, rows=1, eps=EPS, rotary_dim=64, theta=THETA)
        a.update(kw)
        ep.encode(kv, 0, z(a["rows"], H * 2 * D), z(a["rows"], KH * D), z(a["rows"], KH * D), w, w, z(a["rows"], H * D),
                  z(a["rows"], H * D), **a)

    call()  # the valid baseline
    for bad, code in ((dict(rotary_dim=63), capi.ERR_SHAPE), (dict(rotary_dim=258), capi.ERR_SHAPE),
                      (dict(rotary_dim=4), capi.ERR_SHAPE),  # a pair would sit inside one lane (8 dims per lane)
                      (dict(num_q_heads=15), capi.ERR_SHAPE), (dict(q_stride=H * D - 1), capi.ERR_SHAPE),
                      (dict(kv_stride=KH * D - 1), capi.ERR_SHAPE), (dict(positions=64), capi.ERR_CAPACITY),
                      (dict(positions=-1), capi.ERR_INVALID_ARGUMENT), (dict(slots=1), capi.ERR_INVALID_ARGUMENT)):
        with pytest.raises(TinyTitanHIPError) as e:
            call(**bad)
        assert e.value.status == code, bad
    kv.close()
