"""CPU-side checks of the C-ABI library: it loads, exports everything the header declares, and its
pure host arithmetic (page layout, status strings) is right.  No compute call is made."""
import ctypes
import os

import numpy as np
import pytest

from tinytitan_amd import capi

pytestmark = pytest.mark.skipif(not os.path.exists(capi.LIB_PATH) and not os.path.exists("/opt/rocm/bin/hipcc"),
                                reason="library not built and no hipcc to build it")


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(capi.LIB_PATH):
        from tinytitan_amd import build
        build.build()
    return capi.lib()


def test_exports_every_declared_symbol(lib):
    declared = capi.declared_symbols()
    assert len(declared) >= 35
    assert {"tt_hip_kv_append", "tt_hip_attn_decode", "tt_hip_attn_prefill", "tt_hip_attn_verify"} <= set(declared)
    missing = [name for name in declared if not hasattr(lib, name)]
    assert not missing
    # and the ctypes table covers the header exactly
    assert sorted(capi._SIGNATURES) == declared


def test_status_strings(lib):
    assert capi.strerror(capi.OK) == "ok"
    texts = {capi.strerror(code) for code in range(0, 9)}
    assert len(texts) == 9 and "unknown status" not in texts
    assert capi.strerror(99) == "unknown status"


def test_null_handles_are_errors_not_crashes(lib):
    assert lib.tt_hip_kv_capacity(None) == -1
    assert lib.tt_hip_kv_position(None, 0) == -1
    assert lib.tt_hip_kv_bytes(None) == 0
    assert lib.tt_hip_sync(None) == capi.ERR_INVALID_ARGUMENT
    assert lib.tt_hip_kv_advance(None, 0, 1) == capi.ERR_INVALID_ARGUMENT
    assert lib.tt_hip_kv_reserve(None, 10) == capi.ERR_INVALID_ARGUMENT
    assert lib.tt_hip_attn_decode(None, None, 0, 1, None, None, 8, None, None, 1.0, None) == capi.ERR_INVALID_ARGUMENT
    assert lib.tt_hip_attn_prefill(None, None, 0, 0, 0, 1, 1, 8, None, 0, None, 0, 1.0, None, 0) == capi.ERR_INVALID_ARGUMENT
    assert lib.tt_hip_attn_verify(None, None, 0, 1, None, None, 4, 8, None, None, 1.0, None) == capi.ERR_INVALID_ARGUMENT
    lib.tt_hip_ctx_destroy(None)
    lib.tt_hip_kv_destroy(None)
    lib.tt_hip_graph_destroy(None)
    err = ctypes.c_int(0)
    assert not lib.tt_hip_kv_create(None, 1, 2, 256, 1, 64, 64, ctypes.byref(err))
    assert err.value == capi.ERR_INVALID_ARGUMENT


def test_context_create_without_a_device_reports_it(lib):
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    err = ctypes.c_int(0)
    assert not lib.tt_hip_ctx_create(0, ctypes.byref(err))
    assert err.value == capi.ERR_NO_DEVICE


@pytest.mark.parametrize("D", [64, 128, 256])
def test_page_layout_is_a_bijection_per_block(lib, D):
    # every (position, d) of a block maps to a distinct offset inside that block's 32*D halves
    for base in (0, 32 * 7):
        k = np.array([[lib.tt_hip_kv_k_offset(D, base + p, d) for d in range(D)] for p in range(32)])
        v = np.array([[lib.tt_hip_kv_v_offset(D, base + p, d) for d in range(D)] for p in range(32)])
        lo, hi = (base // 32) * 32 * D, (base // 32 + 1) * 32 * D
        for off in (k, v):
            assert off.min() == lo and off.max() == hi - 1
            assert len(np.unique(off)) == 32 * D


def test_k_layout_is_the_mfma_a_fragment_order(lib):
    # v_mfma_f32_32x32x16_f16 A fragment of k-step s: lane (key = l % 32, g = l / 32) holds
    # d = 16 s + 8 g + j at 16-byte-per-lane consecutive addresses.
    D = 256
    for s in range(D // 16):
        for lane in range(64):
            key, g = lane % 32, lane // 32
            for j in range(8):
                assert lib.tt_hip_kv_k_offset(D, key, 16 * s + 8 * g + j) == (s * 64 + lane) * 8 + j


def test_v_layout_matches_the_score_register_order(lib):
    # S^T result register v of lane (n, g) is key 8 (v / 4) + 4 g + v % 4 (32x32 C layout); the
    # P.V k-step t of that lane takes registers 8 t .. 8 t + 7.  Those 8 keys must be the 8
    # consecutive halves of V chunk (d, 2 t + g).
    D = 128
    for d in (0, 5, 127):
        for t in range(2):
            for g in range(2):
                keys = [8 * ((8 * t + j) // 4) + 4 * g + (8 * t + j) % 4 for j in range(8)]
                offs = [lib.tt_hip_kv_v_offset(D, key, d) for key in keys]
                assert offs == [(d * 4 + 2 * t + g) * 8 + j for j in range(8)]
    # 16x16x32 variant: lane group g4 owns tile-a keys {0,4,16,20}[g4] + (0..3) and tile-b keys + 8
    for g4 in range(4):
        first = (g4 & 1) * 4 + (g4 >> 1) * 16
        keys = [first + i for i in range(4)] + [first + 8 + i for i in range(4)]
        offs = [lib.tt_hip_kv_v_offset(D, key, 9) for key in keys]
        assert offs == [(9 * 4 + g4) * 8 + j for j in range(8)]
