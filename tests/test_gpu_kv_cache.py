"""KV cache behaviour through the C ABI, following the reference's KVCacheManagerTests and
KVCacheGrowthTests (tests/TinyTitan/Runtime/KVCache/)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _rows(seed, n, kv_heads=2, dim=256):
    import torch
    g = torch.Generator().manual_seed(seed)
    k = torch.randn(n, kv_heads, dim, generator=g).to(torch.float16)
    v = torch.randn(n, kv_heads, dim, generator=g).to(torch.float16)
    return k, v


def _put(ctx, kv, layer, slot, position, k, v, **kw):
    import torch
    kd, vd = k.cuda(), v.cuda()
    torch.cuda.synchronize()
    kv.append(layer, slot, position, kd, vd, **kw)
    ctx.synchronize()


def test_token_stride_is_1024_bytes_for_2x256(gpu_ctx):
    # KVCacheManagerTests.swift:105-115
    from tinytitan_amd.engine import KVCacheManager
    kv = KVCacheManager(gpu_ctx, 1, 2, 256, slots=1, max_context=4096)
    assert kv.token_stride_bytes == 1024
    assert kv.capacity_tokens == 4096 and kv.bytes == 2 * 4096 * 1024
    kv.close()


def test_append_read_round_trip_is_bit_exact(gpu_ctx):
    from tinytitan_amd.engine import KVCacheManager
    import torch
    kv = KVCacheManager(gpu_ctx, 2, 2, 256, slots=2, max_context=1024, initial_capacity=1024)
    k, v = _rows(1, 300)
    # ragged pieces crossing 32-token block edges, into layer 1 / slot 1
    pos = 0
    for n in (1, 30, 2, 65, 202):
        _put(gpu_ctx, kv, 1, 1, pos, k[pos:pos + n], v[pos:pos + n])
        pos += n
    kr, vr = kv.read(1, 1, 0, 300)
    assert torch.equal(kr.cpu(), k) and torch.equal(vr.cpu(), v)
    # a window in the middle
    kr, vr = kv.read(1, 1, 31, 70)
    assert torch.equal(kr.cpu(), k[31:101]) and torch.equal(vr.cpu(), v[31:101])
    # other layer / slot untouched (stores start zero-filled)
    kr, vr = kv.read(0, 0, 0, 64)
    assert not kr.any() and not vr.any()
    kr, vr = kv.read(1, 0, 0, 64)
    assert not kr.any() and not vr.any()
    kv.close()


def test_append_from_padded_source_rows(gpu_ctx):
    # the caller's projection output may be wider than kv_heads*dim (src_token_stride in elements)
    from tinytitan_amd.engine import KVCacheManager
    import torch
    kv = KVCacheManager(gpu_ctx, 1, 2, 64, slots=1, max_context=256, initial_capacity=256)
    k, v = _rows(2, 40, 2, 64)
    stride = 2 * 64 + 24
    kp = torch.full((40, stride), 7.0, dtype=torch.float16)
    vp = torch.full((40, stride), -3.0, dtype=torch.float16)
    kp[:, :128] = k.reshape(40, 128)
    vp[:, :128] = v.reshape(40, 128)
    _put(gpu_ctx, kv, 0, 0, 5, kp, vp, token_stride=stride, n_tokens=40)
    kr, vr = kv.read(0, 0, 5, 40)
    assert torch.equal(kr.cpu(), k) and torch.equal(vr.cpu(), v)
    kv.close()


@pytest.mark.parametrize("kv_heads,dim,position,n,pad,shift", [(2, 256, 7, 200, 0, 0), (3, 128, 33, 191, 40, 0),
                                                               (1, 64, 0, 96, 8, 0), (2, 256, 31, 130, 0, 1),
                                                               (2, 128, 64, 64, 3, 0), (2, 256, 7, 1100, 0, 0),
                                                               (2, 128, 64, 320, 8, 0), (1, 64, 32, 288, 0, 0)])
def test_chunk_append_whole_blocks_and_ragged_edges(gpu_ctx, kv_heads, dim, position, n, pad, shift):
    # Whole 32-token blocks of a longer chunk (more than 256 rows, more than 1024 with ragged ends) go through the
    # block kernel, the ragged head/tail, short chunks and sources that are not 16-byte aligned (odd stride, shifted
    # base) element by element: same bytes either way, and rows before/after the range keep what they held.
    from tinytitan_amd.engine import KVCacheManager
    import torch
    cap = 512 if position + n <= 480 else 1536
    kv = KVCacheManager(gpu_ctx, 1, kv_heads, dim, slots=2, max_context=cap, initial_capacity=cap)
    old_k, old_v = _rows(11, cap, kv_heads, dim)
    _put(gpu_ctx, kv, 0, 1, 0, old_k, old_v)
    k, v = _rows(12, n, kv_heads, dim)
    width = kv_heads * dim
    stride = width + pad
    kp = torch.full((n * stride + shift,), 9.0, dtype=torch.float16)
    vp = torch.full((n * stride + shift,), -9.0, dtype=torch.float16)
    kp[shift:].view(n, stride)[:, :width] = k.reshape(n, width)
    vp[shift:].view(n, stride)[:, :width] = v.reshape(n, width)
    kd, vd = kp.cuda(), vp.cuda()
    torch.cuda.synchronize()
    kv.append(0, 1, position, kd[shift:], vd[shift:], token_stride=stride, n_tokens=n)
    gpu_ctx.synchronize()
    kr, vr = kv.read(0, 1, 0, cap)
    want_k, want_v = old_k.clone(), old_v.clone()
    want_k[position:position + n], want_v[position:position + n] = k, v
    assert torch.equal(kr.cpu(), want_k) and torch.equal(vr.cpu(), want_v)
    kr, vr = kv.read(0, 0, 0, 512)
    assert not kr.any() and not vr.any()
    kv.close()


def test_slots_are_disjoint_and_cursors_independent(gpu_ctx):
    # KVCacheManagerTests.swift:240-271
    from tinytitan_amd.engine import KVCacheManager
    import torch
    kv = KVCacheManager(gpu_ctx, 1, 2, 256, slots=4, max_context=512, initial_capacity=512)
    data = {}
    for slot, n in enumerate((17, 9, 23, 5)):
        data[slot] = _rows(10 + slot, n)
        _put(gpu_ctx, kv, 0, slot, 0, *data[slot])
        kv.advance(slot, n)
    assert [kv.position(s) for s in range(4)] == [17, 9, 23, 5]
    for slot, n in enumerate((17, 9, 23, 5)):
        kr, vr = kv.read(0, slot, 0, n)
        assert torch.equal(kr.cpu(), data[slot][0]) and torch.equal(vr.cpu(), data[slot][1])
    kv.reset(2)
    assert [kv.position(s) for s in range(4)] == [17, 9, 0, 5]
    kv.reset()
    assert [kv.position(s) for s in range(4)] == [0, 0, 0, 0]
    kv.close()


def test_rewind_only_moves_the_cursor(gpu_ctx):
    # KVCacheManagerTests.swift:209-221; KVCacheManager+Storage.swift:299-309
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, TinyTitanHIPError
    import torch
    kv = KVCacheManager(gpu_ctx, 1, 2, 256, slots=1, max_context=256, initial_capacity=256)
    k, v = _rows(3, 12)
    _put(gpu_ctx, kv, 0, 0, 0, k, v)
    kv.advance(0, 12)
    kv.rewind(0, 8)
    assert kv.position(0) == 8
    kr, _ = kv.read(0, 0, 0, 12)
    assert torch.equal(kr.cpu(), k)  # rows past the cursor are unreachable, not erased
    with pytest.raises(TinyTitanHIPError) as e:
        kv.rewind(0, 9)  # beyond the cursor
    assert e.value.status == capi.ERR_CURSOR
    with pytest.raises(TinyTitanHIPError) as e:
        kv.rewind(0, -1)
    assert e.value.status == capi.ERR_CURSOR
    kv.expect_position(0, 8)
    with pytest.raises(TinyTitanHIPError) as e:
        kv.expect_position(0, 7)
    assert e.value.status == capi.ERR_CURSOR
    kv.close()


def test_capacity_starts_at_min_of_max_context_and_8192(gpu_ctx):
    # KVCacheGrowthTests.swift:41-52
    from tinytitan_amd.engine import KVCacheManager
    a = KVCacheManager(gpu_ctx, 1, 2, 64, slots=1, max_context=262144)
    assert a.capacity_tokens == 8192
    a.close()
    b = KVCacheManager(gpu_ctx, 1, 2, 64, slots=1, max_context=1000)
    assert b.capacity_tokens == 1024 and b.max_context == 1024  # rounded up to whole 32-token blocks
    b.close()


def test_reserve_doubles_clamps_and_preserves_rows(gpu_ctx):
    # KVCacheGrowthTests.swift:54-113
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, TinyTitanHIPError
    import torch
    kv = KVCacheManager(gpu_ctx, 2, 2, 128, slots=2, max_context=1024, initial_capacity=128)
    k0, v0 = _rows(4, 100, 2, 128)
    k1, v1 = _rows(5, 77, 2, 128)
    for layer in range(2):
        _put(gpu_ctx, kv, layer, 0, 0, k0, v0)
        _put(gpu_ctx, kv, layer, 1, 0, k1, v1)
    kv.advance(0, 100)
    kv.advance(1, 77)
    with pytest.raises(TinyTitanHIPError) as e:  # append past capacity: the caller must reserve first
        _put(gpu_ctx, kv, 0, 0, 100, k0[:40], v0[:40])
    assert e.value.status == capi.ERR_CAPACITY
    kv.reserve(100)
    assert kv.capacity_tokens == 128  # below capacity: no-op
    kv.reserve(129)
    assert kv.capacity_tokens == 256  # doubles
    kv.reserve(700)
    assert kv.capacity_tokens == 1024  # 256 -> 512 -> 1024
    kv.reserve(10 ** 6)
    assert kv.capacity_tokens == 1024  # clamps at max_context without failing
    kv.reserve(1024)
    assert kv.capacity_tokens == 1024  # idempotent
    assert kv.token_stride_bytes == 2 * 128 * 2
    for layer in range(2):
        kr, vr = kv.read(layer, 0, 0, 100)
        assert torch.equal(kr.cpu(), k0) and torch.equal(vr.cpu(), v0)
        kr, vr = kv.read(layer, 1, 0, 77)
        assert torch.equal(kr.cpu(), k1) and torch.equal(vr.cpu(), v1)
    assert kv.position(0) == 100 and kv.position(1) == 77
    kv.close()


def test_argument_errors(gpu_ctx):
    from tinytitan_amd import capi
    from tinytitan_amd.engine import KVCacheManager, TinyTitanHIPError
    with pytest.raises(TinyTitanHIPError) as e:
        KVCacheManager(gpu_ctx, 1, 2, 96, slots=1, max_context=64)  # head_dim the kernels do not serve
    assert e.value.status == capi.ERR_SHAPE
    with pytest.raises(TinyTitanHIPError) as e:
        KVCacheManager(gpu_ctx, 1, 2, 64, slots=257, max_context=64)  # more than 256 slots
    assert e.value.status == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(TinyTitanHIPError) as e:
        KVCacheManager(gpu_ctx, 1, 2, 256, slots=1, max_context=5_000_000, initial_capacity=64)  # a page beyond 32-bit reach
    assert e.value.status == capi.ERR_CAPACITY
    ok = KVCacheManager(gpu_ctx, 1, 2, 256, slots=1, max_context=5_000_000, initial_capacity=64, precision_bits=8)  # 8 bit: fits
    ok.close()
    kv = KVCacheManager(gpu_ctx, 1, 2, 64, slots=2, max_context=64)
    k, v = _rows(6, 4, 2, 64)
    for bad in (dict(layer=1, slot=0), dict(layer=0, slot=2), dict(layer=-1, slot=0)):
        with pytest.raises(TinyTitanHIPError) as e:
            _put(gpu_ctx, kv, bad["layer"], bad["slot"], 0, k, v)
        assert e.value.status == capi.ERR_INVALID_ARGUMENT
    with pytest.raises(TinyTitanHIPError) as e:
        _put(gpu_ctx, kv, 0, 0, 0, k, v, token_stride=100, n_tokens=4)  # stride below the packed width
    assert e.value.status == capi.ERR_SHAPE
    with pytest.raises(TinyTitanHIPError) as e:
        kv.advance(0, 65)
    assert e.value.status == capi.ERR_CAPACITY
    kv.close()
