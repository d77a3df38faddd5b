"""KV cache snapshots through the C ABI, following the reference's save/restore tests
(tests/TinyTitan/Runtime/KVCache/KVCacheManagerTests.swift:33-104) and its wire format
(sources/TinyTitan/Runtime/KVCache/KVCacheManager+Snapshot.swift:12-118): per layer, slot 0's rows
of K as token-major fp16 rows, then V -- byte-identical to what the reference writes from its own
token-major buffers, although the HBM pages here are swizzled."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

LAYERS, KH, D = 3, 2, 256


def _manager(ctx, max_context, slots=1, initial=None):
    from tinytitan_amd.engine import KVCacheManager
    return KVCacheManager(ctx, LAYERS, KH, D, slots=slots, max_context=max_context,
                          initial_capacity=initial or min(max_context, 8192))


def _fill(ctx, kv, tokens, seed, slot=0):
    import torch
    g = torch.Generator().manual_seed(seed)
    rows = []
    for layer in range(LAYERS):
        k = torch.randn(tokens, KH * D, generator=g).to(torch.float16)
        v = torch.randn(tokens, KH * D, generator=g).to(torch.float16)
        kd, vd = k.cuda(), v.cuda()
        torch.cuda.synchronize()
        kv.append(layer, slot, 0, kd, vd)
        ctx.synchronize()
        rows.append((k, v))
    kv.advance(slot, tokens)
    return rows


def test_a_snapshot_round_trips_through_restore(gpu_ctx):
    # KVCacheManagerTests.swift:79-104
    import torch
    saver = _manager(gpu_ctx, 128)
    rows = _fill(gpu_ctx, saver, 100, seed=1)
    lengths = saver.snapshot_segment_lengths(100)
    assert lengths == [100 * saver.token_stride_bytes] * (2 * LAYERS)
    payload = bytearray(b"hdr!")  # the payload is appended to, not overwritten
    saver.append_snapshot_payload(payload, lengths)
    assert len(payload) == 4 + LAYERS * 2 * 100 * saver.token_stride_bytes
    # wire format: token-major rows, K then V, layer by layer
    want = b"".join(k.numpy().tobytes() + v.numpy().tobytes() for k, v in rows)
    assert bytes(payload[4:]) == want

    receiver = _manager(gpu_ctx, 128, slots=2)
    receiver.advance(1, 7)  # restore resets every cursor
    offset = receiver.restore_snapshot(100, lengths, bytes(payload), offset=4)
    assert offset == len(payload)
    assert receiver.position(0) == 100 and receiver.position(1) == 0
    for layer, (k, v) in enumerate(rows):
        kr, vr = receiver.read(layer, 0, 0, 100)
        assert torch.equal(kr.cpu().reshape(100, -1), k) and torch.equal(vr.cpu().reshape(100, -1), v)
    saver.close()
    receiver.close()


def test_a_snapshot_past_the_initial_capacity_grows_the_receiver(gpu_ctx):
    # KVCacheManagerTests.swift:33-77: the restore must grow to the snapshot's position BEFORE it
    # compares lengths; with an empty payload the copy then fails, and the growth stays.
    from tinytitan_amd import capi
    from tinytitan_amd.engine import TinyTitanHIPError
    target = 8500
    saver = _manager(gpu_ctx, 9000)
    saver.reserve(target)
    saver.advance(0, target)
    lengths = saver.snapshot_segment_lengths(target)
    receiver = _manager(gpu_ctx, 9000)
    assert receiver.capacity_tokens == 8192
    with pytest.raises(TinyTitanHIPError) as e:
        receiver.restore_snapshot(target, lengths, b"")
    assert e.value.status == capi.ERR_SHAPE  # invalidLayout
    assert receiver.capacity_tokens >= target
    saver.close()
    receiver.close()


def test_invalid_positions_and_layouts(gpu_ctx):
    from tinytitan_amd import capi
    from tinytitan_amd.engine import TinyTitanHIPError
    kv = _manager(gpu_ctx, 128)
    for bad in (0, -3, 129):  # snapshotSegmentLengths guard (:13-15)
        with pytest.raises(TinyTitanHIPError) as e:
            kv.snapshot_segment_lengths(bad)
        assert e.value.status == capi.ERR_CURSOR
    _fill(gpu_ctx, kv, 40, seed=2)
    good = kv.snapshot_segment_lengths(40)
    payload = bytearray()
    for wrong in (kv.snapshot_segment_lengths(41), good[:-1], [good[0] + 2] + good[1:]):
        with pytest.raises(TinyTitanHIPError) as e:  # appendSnapshotPayload checks against the cursor (:42-45)
            kv.append_snapshot_payload(payload, wrong)
        assert e.value.status == capi.ERR_SHAPE
    assert len(payload) == 0
    kv.append_snapshot_payload(payload, good)
    other = _manager(gpu_ctx, 128)
    for position, lengths, data in ((41, good, bytes(payload)), (40, good, bytes(payload[:-1])), (40, good[:-2], bytes(payload))):
        with pytest.raises(TinyTitanHIPError) as e:
            other.restore_snapshot(position, lengths, data)
        assert e.value.status == capi.ERR_SHAPE
    with pytest.raises(TinyTitanHIPError) as e:
        other.restore_snapshot(0, good, bytes(payload))
    assert e.value.status == capi.ERR_CURSOR
    kv.close()
    other.close()


def test_restored_cache_attends_like_the_original(gpu_ctx):
    import torch
    from tinytitan_amd.engine import Attention
    H, tokens = 16, 777
    saver = _manager(gpu_ctx, 1024)
    _fill(gpu_ctx, saver, tokens, seed=3)
    payload = bytearray()
    lengths = saver.snapshot_segment_lengths(tokens)
    saver.append_snapshot_payload(payload, lengths)
    receiver = _manager(gpu_ctx, 1024)
    receiver.restore_snapshot(tokens, lengths, bytes(payload))
    q = torch.randn(1, 1, H, D, generator=torch.Generator().manual_seed(4)).to(torch.float16).cuda()
    outs = []
    for kv in (saver, receiver):
        out = torch.empty_like(q)
        torch.cuda.synchronize()
        Attention(gpu_ctx).encode_full(kv, 1, q, out, H, tokens, 0.0625)
        gpu_ctx.synchronize()
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])
    saver.close()
    receiver.close()
