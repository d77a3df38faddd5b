"""Pins the oracle's affine-quantised projection (o_proj) -- bf16 conversion, the group quantiser, the
GEMV and its fp16-rounded multi-token form -- against the reference's own C kernels compiled into
``oracle/_ref``, the reference tests' closed forms and recorded value, hand-packed rows and a float64
numpy statement."""
import os

import numpy as np
import pytest

import oracle

G = oracle.AFFINE_GROUP_SIZE


def lcg_floats(count, seed):
    """``Int8AffineGEMVTests.pseudorandom`` (tests/TinyTitan/Kernels/CPU/Int8AffineGEMVTests.swift:17-24)."""
    state, out = seed, []
    for _ in range(count):
        state = (state * 6364136223846793005 + 1442695040888963407) & 0xFFFFFFFFFFFFFFFF
        value = (state >> 33) & 0xFFFFFFFF
        value = value - (1 << 32) if value >= 1 << 31 else value
        out.append(np.float32(value) / np.float32(2147483647))
    return np.array(out, dtype=np.float32)


def unpack_levels(packed, bits):
    """Levels of hand-unpacked rows (not through the oracle's dequantiser)."""
    if bits == 8:
        return packed.astype(np.int64)
    return np.stack([packed & 0x0F, packed >> 4], axis=-1).reshape(packed.shape[0], -1).astype(np.int64)


def bf16_array(bits):
    return (np.asarray(bits, dtype=np.uint32) << 16).view(np.float32)


def test_bf16_known_bit_patterns_and_ties():
    assert oracle.bf16_bits(1.0) == 0x3F80 and oracle.bf16_bits(0.375) == 0x3EC0 and oracle.bf16_bits(-2.0) == 0xC000
    # round to nearest even at the half-way points of the dropped 16 bits
    even = np.array([0x3F808000], dtype=np.uint32).view(np.float32)[0]   # tie, kept mantissa even -> down
    odd = np.array([0x3F818000], dtype=np.uint32).view(np.float32)[0]    # tie, kept mantissa odd -> up
    above = np.array([0x3F808001], dtype=np.uint32).view(np.float32)[0]
    assert oracle.bf16_bits(even) == 0x3F80 and oracle.bf16_bits(odd) == 0x3F82 and oracle.bf16_bits(above) == 0x3F81
    for bits in list(range(0, 0x7F80, 97)) + list(range(0x8000, 0xFF80, 101)):
        assert oracle.bf16_bits(oracle.bf16_to_f32(bits)) == bits


@pytest.mark.parametrize("bits", [4, 8])
def test_quantiser_closed_forms(bits):
    top = (1 << bits) - 1
    row = np.full((1, 2 * G), 0.375, dtype=np.float32)   # constant group: scale 1, bias = value (Quantization.swift:78-83)
    ramp = -1.25 + ((np.arange(G) * 37) % (top + 1)) * 2.0 ** -6
    ramp[3], ramp[9] = -1.25, -1.25 + top * 2.0 ** -6
    row[0, G:] = ramp                                     # exact ramp with a power-of-two step: its own indices
    packed, scales, biases = oracle.affine_quantize_rows(row, bits)
    levels = unpack_levels(packed, bits)[0]
    assert scales[0, 0] == 0x3F80 and biases[0, 0] == 0x3EC0 and not levels[:G].any()
    assert oracle.bf16_to_f32(scales[0, 1]) == 2.0 ** -6 and oracle.bf16_to_f32(biases[0, 1]) == -1.25
    assert np.array_equal(levels[G:], np.round((ramp + 1.25) * 64).astype(np.int64))
    assert levels[G + 3] == 0 and levels[G + 9] == top
    assert np.array_equal(oracle.affine_dequantize_rows(packed, scales, biases, bits), row)


def test_nibble_order_is_low_first():
    # element 2 k in the low nibble of byte k (tinytitan_kernels.h:12-14)
    packed = np.array([[0x21, 0x43] + [0] * 30], dtype=np.uint8)
    scales = np.array([[0x3F80]], dtype=np.uint16)
    biases = np.zeros((1, 1), dtype=np.uint16)
    assert list(oracle.affine_dequantize_rows(packed, scales, biases, 4)[0, :5]) == [1.0, 2.0, 3.0, 4.0, 0.0]
    x = np.zeros(G, dtype=np.float32)
    x[1] = 1.0
    assert oracle.affine_gemv(packed, scales, biases, x, 4)[0] == 2.0


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("n", [128, 256, 2816])
def test_round_trip_stays_within_the_reference_bound(bits, n):
    # DequantInt4GEMVReferenceTests.swift:62-80: |recovered - raw| <= scale + 1e-4 per group
    raw = oracle.fill_uniform(0xF5, f"int4-affine-roundtrip-n{n}", -1.0, 1.0, n)[None, :]
    packed, scales, biases = oracle.affine_quantize_rows(raw, bits)
    recovered = oracle.affine_dequantize_rows(packed, scales, biases, bits)
    bound = np.repeat(bf16_array(scales[0]), G) + 1e-4
    assert (np.abs(recovered[0] - raw[0]) <= bound).all()
    if bits == 8:  # the finer grid: half a step plus the bf16 rounding of the bias
        assert (np.abs(recovered[0] - raw[0]) <= 0.5 * bound + 2.0 ** -8).all()


@pytest.mark.parametrize("bits", [4, 8])
def test_constant_row_is_carried_by_the_bias_term(bits):
    # Int8AffineGEMVTests.swift:104-110
    x = lcg_floats(128, 3)
    packed, scales, biases = oracle.affine_quantize_rows(np.full((1, 128), 0.375, dtype=np.float32), bits)
    got = oracle.affine_gemv(packed, scales, biases, x, bits)[0]
    want = 0.375 * float(x.astype(np.float64).sum())
    assert abs(got - want) <= 1e-3 * max(1.0, abs(want))


def test_recorded_value_of_the_reference_test():
    # Int8AffineGEMVTests.swift:172-186: lanes i % 16, scale 1, bias 0, x from its generator with seed 5;
    # "Measured here: 955.4322 against 955.43225" for the two widths on the reference's machine.
    x = lcg_floats(256, 5)
    lanes = (np.arange(3 * 256) % 16).astype(np.uint8).reshape(3, 256)
    scales = np.full((3, 4), 0x3F80, dtype=np.uint16)
    biases = np.zeros((3, 4), dtype=np.uint16)
    four = oracle.affine_gemv((lanes[:, 0::2] | (lanes[:, 1::2] << 4)).astype(np.uint8), scales, biases, x, 4)
    eight = oracle.affine_gemv(lanes, scales, biases, x, 8)
    for got in list(four) + list(eight):
        assert abs(float(got) - 955.4322) <= 2e-4


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("rows,n", [(3, 64), (37, 2816), (64, 4096), (5, 6144)])
def test_gemv_matches_the_reference_c_kernel_bit_for_bit(bits, rows, n):
    r = np.random.default_rng(rows * 131 + n + bits)
    packed, scales, biases = oracle.affine_quantize_rows(r.uniform(-0.5, 0.5, (rows, n)).astype(np.float32), bits)
    x = r.uniform(-1.0, 1.0, n).astype(np.float32)
    got = oracle.affine_gemv(packed, scales, biases, x, bits)
    reference = oracle.reference_affine_gemv(packed, scales, biases, x, bits)
    if reference is None:
        assert not os.path.isdir("/root/reference"), "the reference checkout is here but oracle/_ref was not built"
        pytest.skip("oracle/_ref is not built (no reference checkout on this machine)")
    assert np.array_equal(got, reference)


@pytest.mark.parametrize("bits", [4, 8])
def test_gemv_matches_float64_dequantise_then_dot(bits):
    # the formulation of DequantInt4GemvRef (sources/TinyTitanValidation/Support/Reference/Quant/DequantInt4Gemv.swift:12-41)
    r = np.random.default_rng(40 + bits)
    rows, n = 96, 2816
    packed, scales, biases = oracle.affine_quantize_rows(r.uniform(-0.5, 0.5, (rows, n)).astype(np.float32), bits)
    x = r.uniform(-1.0, 1.0, n).astype(np.float16).astype(np.float32)
    levels = unpack_levels(packed, bits).astype(np.float64)
    dense = levels * np.repeat(bf16_array(scales), G, axis=1) + np.repeat(bf16_array(biases), G, axis=1)
    want = dense @ x.astype(np.float64)
    got = oracle.affine_gemv(packed, scales, biases, x, bits)
    magnitude = np.abs(dense) @ np.abs(x.astype(np.float64))
    assert (np.abs(got - want) <= 1e-5 * magnitude).all()
    # and the reference's own bar for this comparison (Tolerances.swift:10, RelError.compute)
    assert np.abs(got - want).max() / np.abs(want).max() < 5e-3


@pytest.mark.parametrize("bits", [4, 8])
def test_projection_is_the_gemv_per_token_rounded_to_fp16(bits):
    r = np.random.default_rng(60 + bits)
    rows, n, tokens = 40, 256, 5
    packed, scales, biases = oracle.affine_quantize_rows(r.uniform(-0.5, 0.5, (rows, n)).astype(np.float32), bits)
    x = r.standard_normal((tokens, n)).astype(np.float16).astype(np.float32)
    y = oracle.affine_projection(packed, scales, biases, x, bits)
    for t in range(tokens):
        line = oracle.affine_gemv(packed, scales, biases, x[t], bits)
        assert np.array_equal(y[t], line.astype(np.float16).astype(np.float32))


@pytest.mark.parametrize("bits", [4, 8])
def test_half_weight_projection_matches_float64_over_rounded_weights(bits):
    # tensorops.metal:93-97: weightTile = half(fma(float(q), scale, bias)); an independent numpy statement
    r = np.random.default_rng(80 + bits)
    rows, n, tokens = 70, 704, 9
    packed, scales, biases = oracle.affine_quantize_rows(r.uniform(-0.5, 0.5, (rows, n)).astype(np.float32), bits)
    x = r.standard_normal((tokens, n)).astype(np.float16).astype(np.float32)
    levels = unpack_levels(packed, bits).astype(np.float64)
    exact = levels * np.repeat(bf16_array(scales), G, axis=1).astype(np.float64) + np.repeat(bf16_array(biases), G, axis=1)
    dense = exact.astype(np.float32).astype(np.float16).astype(np.float64)  # through fp32 (the fma's rounding), then half
    want = x.astype(np.float64) @ dense.T
    got = oracle.affine_projection(packed, scales, biases, x, bits, half_weights=True)
    magnitude = np.abs(x.astype(np.float64)) @ np.abs(dense).T
    assert (np.abs(got - want) <= 2.0 ** -11 * np.abs(want) + 1e-5 * magnitude).all()
    # against the exactly factored projection: the weights moved by at most half an fp16 ulp each
    plain = oracle.affine_projection(packed, scales, biases, x, bits)
    assert (np.abs(got - plain) <= 2.0 ** -10 * np.abs(plain) + 2.0 ** -11 * magnitude).all()


def test_half_weight_projection_equals_the_factored_one_when_weights_are_halves():
    # power-of-two scale, short bias: every level * scale + bias is an fp16 number, so rounding the tile changes nothing
    r = np.random.default_rng(9)
    rows, n = 33, 256
    packed = r.integers(0, 256, (rows, n), dtype=np.uint8)
    scales = np.full((rows, n // G), oracle.bf16_bits(2.0 ** -7), dtype=np.uint16)
    biases = np.full((rows, n // G), oracle.bf16_bits(-1.0), dtype=np.uint16)
    x = r.integers(-8, 9, (4, n)).astype(np.float32) / 8.0  # sums exact in fp32 whatever their order
    assert np.array_equal(oracle.affine_projection(packed, scales, biases, x, 8, half_weights=True),
                          oracle.affine_projection(packed, scales, biases, x, 8))


def test_shapes_the_format_does_not_allow_are_refused():
    packed = np.zeros((2, 50), dtype=np.uint8)
    params = np.zeros((2, 1), dtype=np.uint16)
    with pytest.raises(oracle.OracleError):
        oracle.affine_gemv(packed, params, params, np.zeros(100, dtype=np.float32), 4)  # 100 columns: not a multiple of 64
    with pytest.raises(oracle.OracleError):
        oracle.affine_quantize_rows(np.zeros((1, 64), dtype=np.float32), 5)
