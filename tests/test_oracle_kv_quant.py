"""Pins the oracle's quantised KV rows (row layout, affine quantiser, loader) against the reference's
own known answers, closed forms, hand-packed rows, an independent numpy statement and the
reference test's own bar on its own seeded inputs."""
import numpy as np
import pytest

import oracle

G = oracle.KV_GROUP_SIZE


def f16(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


def split_row(row, elements, bits):
    """(levels, scales, biases) of one stored row, unpacked by hand (not through the oracle's loader)."""
    stride, value_bytes = oracle.kv_row_layout(elements, bits)
    groups = (elements + G - 1) // G
    if bits == 8:
        levels = row[:elements].astype(np.int64)
    else:
        packed = row[:(elements + 1) // 2]
        levels = np.stack([packed & 0x0F, packed >> 4], axis=1).reshape(-1)[:elements].astype(np.int64)
    halves = row[value_bytes:value_bytes + 4 * groups].copy().view(np.float16).astype(np.float32)
    return levels, halves[:groups], halves[groups:]


def test_row_layout_known_answers():
    # KVCacheQuantizedAttentionTests.swift:96-98: stride of the 2 x 256 row at each precision.
    assert oracle.kv_row_layout(512, 16) == (1024, 1024)
    assert oracle.kv_row_layout(512, 8) == (544, 512)
    assert oracle.kv_row_layout(512, 4) == (288, 256)
    # odd packed byte counts round up to 2; a ragged last group still gets its scale and bias
    assert oracle.kv_row_layout(65, 8) == (66 + 2 * 2 * 2, 66)
    assert oracle.kv_row_layout(70, 4) == (36 + 2 * 2 * 2, 36)
    with pytest.raises(oracle.OracleError):
        oracle.kv_row_layout(512, 5)


@pytest.mark.parametrize("bits", [8, 4])
def test_constant_group_has_scale_zero_and_exact_values(bits):
    row = np.full((1, 128), 0.375, dtype=np.float32)
    row[0, 64:] = -1.5
    q = oracle.kv_quantize_rows(row, bits)
    levels, scales, biases = split_row(q[0], 128, bits)
    assert not levels.any() and not scales.any()
    assert list(biases) == [0.375, -1.5]
    assert np.array_equal(oracle.kv_dequantize_rows(q, 128, bits), row)


@pytest.mark.parametrize("bits", [8, 4])
def test_exact_ramp_maps_to_its_own_indices(bits):
    # bias + k * scale with a power-of-two scale: every value is a level, the round trip is exact
    top = 255 if bits == 8 else 15
    k = (np.arange(64) * 37) % (top + 1)
    k[5], k[17] = 0, top  # the group holds both ends
    scale, bias = 2.0 ** -6, -1.25
    row = (bias + k * scale).astype(np.float32)[None, :]
    assert np.array_equal(f16(row), row)
    q = oracle.kv_quantize_rows(row, bits)
    levels, scales, biases = split_row(q[0], 64, bits)
    assert np.array_equal(levels, k) and scales[0] == scale and biases[0] == bias
    assert np.array_equal(oracle.kv_dequantize_rows(q, 64, bits), row)


def test_minimum_and_maximum_take_the_end_levels_and_halves_round_away_from_zero():
    # group of 0 .. 255 scaled so that scale == 1: x.5 cannot occur; then a group where it does:
    # values {0, 2.5, 5} at 4 bits: scale = 1/3 ... instead use 8 bits with range 510 -> scale 2,
    # value 1 -> 0.5 -> rounds away from zero to 1, value 3 -> 1.5 -> 2.
    row = np.zeros((1, 64), dtype=np.float32)
    row[0, :4] = [0.0, 510.0, 1.0, 3.0]
    q = oracle.kv_quantize_rows(row, 8)
    levels, scales, biases = split_row(q[0], 64, 8)
    assert list(levels[:4]) == [0, 255, 1, 2] and scales[0] == 2.0 and biases[0] == 0.0


def test_nibble_order_by_hand():
    # even element in the low nibble (kv_cache_quantize.metal:63-72, attention.metal:104-106)
    row = np.zeros((1, 64), dtype=np.float32)
    row[0, :4] = [0.0, 15.0, 3.0, 9.0]
    q = oracle.kv_quantize_rows(row, 4)
    assert q[0, 0] == (0 | (15 << 4)) and q[0, 1] == (3 | (9 << 4))
    back = oracle.kv_dequantize_rows(q, 64, 4)
    assert list(back[0, :4]) == [0.0, 15.0, 3.0, 9.0]


def numpy_quantize(rows, bits):
    """Independent vectorised statement of the same quantiser (whole groups only)."""
    tokens, elements = rows.shape
    top = np.float32(255 if bits == 8 else 15)
    g = rows.reshape(tokens, elements // G, G).astype(np.float32)
    lo, hi = g.min(axis=2, keepdims=True), g.max(axis=2, keepdims=True)
    scale = np.where(hi > lo, (hi - lo) / top, np.float32(0)).astype(np.float32)
    with np.errstate(divide="ignore", invalid="ignore"):
        x = np.clip((g - lo) / scale, 0, top)
    levels = np.where(scale > 0, np.floor(x + np.float32(0.5)), 0).astype(np.int64)  # x >= 0: half away from zero
    return levels.reshape(tokens, elements), scale[..., 0].astype(np.float16), lo[..., 0].astype(np.float16)


@pytest.mark.parametrize("bits", [8, 4])
def test_against_numpy_statement_and_error_bound(bits):
    r = np.random.default_rng(bits)
    rows = f16(r.standard_normal((37, 512)) * r.uniform(0.01, 4.0, size=(37, 1)))
    q = oracle.kv_quantize_rows(rows, bits)
    want_levels, want_scale, want_bias = numpy_quantize(rows, bits)
    top = 255 if bits == 8 else 15
    for t in range(rows.shape[0]):
        levels, scales, biases = split_row(q[t], 512, bits)
        assert np.array_equal(levels, want_levels[t])
        assert np.array_equal(scales, want_scale[t].astype(np.float32))
        assert np.array_equal(biases, want_bias[t].astype(np.float32))
    back = oracle.kv_dequantize_rows(q, 512, bits)
    # half a step from rounding the level, plus what rounding the scale to fp16 moves the top level
    scale32 = np.repeat(want_scale.astype(np.float32), G, axis=1)
    bound = 0.5 * scale32 * (1 + 2.0 ** -10) + top * scale32 * 2.0 ** -11 + 1e-7
    assert (np.abs(back - rows) <= bound).all()
    # the loader is level * scale + bias with the STORED halves
    manual = want_levels * scale32 + np.repeat(want_bias.astype(np.float32), G, axis=1)
    assert np.array_equal(back, manual.astype(np.float32))


def test_ragged_last_group_and_row_padding():
    r = np.random.default_rng(3)
    rows = f16(r.standard_normal((3, 70)))
    for bits in (8, 4):
        q = oracle.kv_quantize_rows(rows, bits)
        levels, scales, biases = split_row(q[0], 70, bits)
        assert biases[1] == rows[0, 64:].min() and levels[64:].max() == (255 if bits == 8 else 15)
        back = oracle.kv_dequantize_rows(q, 70, bits)
        assert np.abs(back - rows).max() <= 0.51 * max(scales) + 1e-3


def rel_error(actual, reference):
    # RelError.compute (sources/TinyTitanValidation/Support/Tolerance/RelError.swift:7-16)
    return np.abs(actual - reference).max() / max(np.abs(reference).max(), 1e-6)


@pytest.mark.parametrize("bits,tolerance", [(8, 0.02), (4, 0.20)])
def test_reference_decode_case_meets_the_reference_bar(bits, tolerance):
    # KVCacheQuantizedAttentionTests.swift:9-83 on its own inputs: SeedTree(0x4B56).key("kv-cache-<bits>"),
    # q then k then v from one stream, uniform(-0.5, 0.5) rounded to fp16, 16/2/256, 8 keys, scale 1/16.
    H, KH, D, T = 16, 2, 256, 8
    draws = oracle.fill_uniform(0x4B56, f"kv-cache-{bits}", -0.5, 0.5, H * D + 2 * T * KH * D)
    q, k, v = f16(draws[:H * D]), f16(draws[H * D:H * D + T * KH * D]), f16(draws[H * D + T * KH * D:])
    k, v = k.reshape(T, KH * D), v.reshape(T, KH * D)
    kq = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(k, bits), KH * D, bits)
    vq = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(v, bits), KH * D, bits)
    want = oracle.attention_ref(q, k, v, D, H, KH, T, 0, 0.0625)
    got = f16(oracle.attention_ref(q, kq, vq, D, H, KH, T, 0, 0.0625))
    err = rel_error(got.reshape(-1), want.reshape(-1))
    assert err < tolerance
    assert err > 1e-5  # and the quantiser did change something
