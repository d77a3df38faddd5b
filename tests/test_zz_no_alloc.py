"""tt_hip_attn_decode_noalloc through the C ABI: the decode for callers that cannot allocate.

Its split-K partials live in a fixed array of the library's device image instead of the context's grown-on-demand
buffers.  Bar: bit-equal to tt_hip_attn_decode on the same inputs (same kernels, same geometry), on two calls in a
row of which the second is smaller (so stale partials of the first would show), and within the attention bar of the
CPU oracle.  Sizes beyond the array are refused with TT_HIP_ERR_SCRATCH.  And the property it exists for: as the first
attention call of a fresh context it leaves the device's free memory as it was, where the allocating entry point
has to grow the context's partial buffers."""
import ctypes

import numpy as np
import pytest

import oracle
from tests.helpers import MAX_ABS, MEAN_ABS, f16_round

pytestmark = pytest.mark.gpu


def _decode_both(lib, ctx, kv, lens, heads, q, gate, scale):
    """The same decode through both entry points; returns (allocating, no-allocation) outputs as numpy."""
    import torch
    from tinytitan_amd import capi
    n = len(lens)
    slots, seq_lens = capi.int_array(list(range(n))), capi.int_array(list(lens))
    outs = []
    for fn in (lib.tt_hip_attn_decode, lib.tt_hip_attn_decode_noalloc):
        out = torch.full(q.shape, float("nan"), dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        status = fn(ctx.handle, kv.handle, 0, n, slots, seq_lens, heads, q.data_ptr(), gate.data_ptr() if gate is not None else None,
                    ctypes.c_float(scale), out.data_ptr())
        assert status == capi.OK, capi.strerror(status)
        ctx.synchronize()
        outs.append(out.cpu().numpy())
    return outs


def test_no_alloc_decode_equals_the_allocating_decode_twice_in_a_row():
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import HIPContext, KVCacheManager
    ctx = HIPContext(0)  # a context of its own: its grown-on-demand partial buffers start empty
    lib = ctx._lib
    H, KH, D, scale = 16, 2, 256, 0.0625
    r = np.random.default_rng(0x7A)
    # first call: 3 ragged sequences, the longest 9,000 keys (many splits); second call: one sequence of 1,500 keys
    # (fewer, shorter splits) -- what the first left in the array lies beyond and between the second's partials
    for lens in ([9000, 4100, 777], [1500]):
        n, longest = len(lens), max(lens)
        kv = KVCacheManager(ctx, 1, KH, D, slots=n, max_context=longest, initial_capacity=longest)
        ks, vs = [], []
        for i, length in enumerate(lens):
            k, v = (r.standard_normal((length, KH, D)).astype(np.float16) for _ in range(2))
            kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
            torch.cuda.synchronize()
            kv.append(0, i, 0, kd, vd)
            ctx.synchronize()
            ks.append(k)
            vs.append(v)
        q, gate = (r.standard_normal((n, 1, H, D)).astype(np.float16) for _ in range(2))
        qd, gd = torch.from_numpy(q).cuda(), torch.from_numpy(gate).cuda()
        want, got = _decode_both(lib, ctx, kv, lens, H, qd, gd, scale)
        assert np.isfinite(got.astype(np.float32)).all()
        assert np.array_equal(want.view(np.uint16), got.view(np.uint16)), f"lengths {lens}: outputs differ bit-wise"
        for i, length in enumerate(lens):
            ref = oracle.decode(q[i, 0].astype(np.float32), ks[i].astype(np.float32).reshape(length, -1),
                                vs[i].astype(np.float32).reshape(length, -1), H, KH, D, scale, gate=gate[i, 0].astype(np.float32))
            diff = np.abs(got[i, 0].astype(np.float64) - f16_round(ref).astype(np.float64))
            assert diff.max() <= MAX_ABS and diff.mean() <= MEAN_ABS, f"lengths {lens}, sequence {i}: {diff.max():.2e}"
        kv.close()
    # beyond the fixed array: with the planner's own splits every decode of up to 64 sequences fits; a split override
    # of 32 keys makes one sequence of 40,000 keys take 1,250 splits on each of two KV heads -- 40,000 partial rows --
    # and more than 64 sequences do not fit one launch's tables.  Both are refused before anything is launched.
    kv = KVCacheManager(ctx, 1, KH, 64, slots=65, max_context=40000, initial_capacity=40000)
    qd = torch.zeros((65, 1, H, 64), dtype=torch.float16, device="cuda")
    out = torch.full_like(qd, 7.0)
    torch.cuda.synchronize()
    ctx.set_split_tokens(32)
    status = lib.tt_hip_attn_decode_noalloc(ctx.handle, kv.handle, 0, 1, capi.int_array([0]), capi.int_array([40000]), H,
                                            qd.data_ptr(), None, ctypes.c_float(0.125), out.data_ptr())
    assert status == capi.ERR_SCRATCH, capi.strerror(status)
    ctx.set_split_tokens(0)
    status = lib.tt_hip_attn_decode_noalloc(ctx.handle, kv.handle, 0, 65, capi.int_array(list(range(65))),
                                            capi.int_array([40000] + [32] * 64), H, qd.data_ptr(), None,
                                            ctypes.c_float(0.125), out.data_ptr())
    assert status == capi.ERR_SCRATCH, capi.strerror(status)
    ctx.synchronize()
    assert (out == 7.0).all()
    # one long sequence beside 63 short ones: every sequence takes the splits its own keys need, which fits
    status = lib.tt_hip_attn_decode_noalloc(ctx.handle, kv.handle, 0, 64, capi.int_array(list(range(64))),
                                            capi.int_array([40000] + [32] * 63), H, qd.data_ptr(), None,
                                            ctypes.c_float(0.125), out.data_ptr())
    assert status == capi.OK, capi.strerror(status)
    ctx.synchronize()
    assert (out[:64] == 0.0).all()  # an all-zero cache and query: zeros, written for every sequence
    kv.close()
    ctx.close()


def test_no_alloc_decode_is_the_first_call_of_a_fresh_context_and_allocates_nothing():
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import HIPContext, KVCacheManager
    H, KH, D, scale, lens = 16, 2, 256, 0.0625, [6000, 2500]
    r = np.random.default_rng(0x7B)
    n, longest = len(lens), max(lens)
    q, gate = (r.standard_normal((n, 1, H, D)).astype(np.float16) for _ in range(2))
    qd, gd = torch.from_numpy(q).cuda(), torch.from_numpy(gate).cuda()
    slots, seq_lens = capi.int_array(list(range(n))), capi.int_array(lens)

    def cache(ctx):
        kv = KVCacheManager(ctx, 1, KH, D, slots=n, max_context=longest, initial_capacity=longest)
        rr = np.random.default_rng(0x7C)
        for i, length in enumerate(lens):
            kd, vd = (torch.from_numpy(rr.standard_normal((length, KH, D)).astype(np.float16)).cuda() for _ in range(2))
            torch.cuda.synchronize()
            kv.append(0, i, 0, kd, vd)
            ctx.synchronize()
        return kv

    def call(fn, ctx, kv, out):
        status = fn(ctx.handle, kv.handle, 0, n, slots, seq_lens, H, qd.data_ptr(), gd.data_ptr(), ctypes.c_float(scale), out.data_ptr())
        assert status == capi.OK, capi.strerror(status)
        ctx.synchronize()

    # Another context runs the same step first, so that the kernels' code is on the device before anything is measured
    # (a kernel's first launch in a process loads its code object, which is device memory too).
    warm = HIPContext(0)
    warm_kv = cache(warm)
    outs = [torch.full(qd.shape, float("nan"), dtype=torch.float16, device="cuda") for _ in range(3)]
    call(warm._lib.tt_hip_attn_decode, warm, warm_kv, outs[0])
    call(warm._lib.tt_hip_attn_decode_noalloc, warm, warm_kv, outs[0])
    ctx = HIPContext(0)  # fresh: its grown-on-demand partial buffers do not exist yet
    kv = cache(ctx)
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    call(ctx._lib.tt_hip_attn_decode_noalloc, ctx, kv, outs[1])
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert free_after == free_before, f"the no-allocation decode changed free device memory by {free_before - free_after} bytes"
    # the same step through the allocating entry point has to create the context's partial buffers: the measure sees it
    call(ctx._lib.tt_hip_attn_decode, ctx, kv, outs[2])
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] < free_after, "the allocating decode was expected to grow the partial buffers"
    assert torch.equal(outs[1], outs[2]) and torch.equal(outs[0], outs[1])
    assert torch.isfinite(outs[1].float()).all()
    for c in (kv, warm_kv):
        c.close()
    ctx.close()
    warm.close()
