"""The projection behind the gate (o_proj over affine-quantised weights) through the C ABI.

The oracle is the restatement of the reference's C kernels (bit for bit equal to them, see
tests/test_oracle_affine.py) followed by the Metal kernels' one fp16 rounding.  The HIP kernel does
the same factored arithmetic -- scale * sum(level * x) + bias * sum(x) per group, in fp32 -- and
differs only in the order of the fp32 sums, so the bar is: within one fp16 ulp of the oracle's
value plus 1e-5 of the row's absolute magnitude sum(|w| |x|) (the room fp32 reordering needs),
and nearly all outputs bit-equal.  The reference's own bar between its kernel and its fp32
reference (max-abs / max|ref| < 5e-3, DequantInt4GEMVTests.swift:107-112) is asserted as well."""
import numpy as np
import pytest

import oracle
from tests.test_gpu_attention_api import _dev

pytestmark = pytest.mark.gpu

G = oracle.AFFINE_GROUP_SIZE


def _weights(rows, n, bits, seed, label=None):
    if label is None:
        raw = np.random.default_rng(seed).uniform(-0.5, 0.5, (rows, n)).astype(np.float32)
    else:  # the reference tests' generator: one stream, row after row, then x
        raw = oracle.fill_uniform(seed, label, -0.5, 0.5, rows * n).reshape(rows, n)
    return oracle.affine_quantize_rows(raw, bits)


def _magnitude(packed, scales, biases, x, bits):
    dense = np.abs(oracle.affine_dequantize_rows(packed, scales, biases, bits).astype(np.float64))
    return np.abs(x.astype(np.float64)) @ dense.T


def _project(ctx, bits, packed, scales, biases, x, x_stride=None, y_stride=None, weights_offset=0):
    import torch
    from tinytitan_amd.engine import AffineProjection
    rows, n = packed.shape[0], packed.shape[1] * 8 // bits
    tokens = x.shape[0]
    xs, ys = x_stride or n, y_stride or rows
    xd = torch.full((tokens, xs), 7.0, dtype=torch.float16, device="cuda")
    xd[:, :n] = _dev(x)
    yd = torch.full((tokens, ys), -3.0, dtype=torch.float16, device="cuda")
    raw = np.zeros(packed.size + 16 + weights_offset, dtype=np.uint8)
    raw[weights_offset:weights_offset + packed.size] = packed.reshape(-1)
    wd = _dev(raw)
    assert wd.data_ptr() % 16 == 0
    sd, bd = _dev(scales.view(np.int16)), _dev(biases.view(np.int16))
    torch.cuda.synchronize()
    AffineProjection(ctx).encode(bits, wd, sd, bd, xd, yd, rows, n, tokens, xs, ys, weights_offset=weights_offset)
    ctx.synchronize()
    out = yd.cpu().numpy()
    assert (out[:, rows:] == np.float16(-3.0)).all(), "wrote beyond a row of y"
    return out[:, :rows].astype(np.float32)


def _assert_parity(got, want, magnitude, what):
    assert np.isfinite(got).all(), what
    diff = np.abs(got.astype(np.float64) - want.astype(np.float64))
    ulp = 2.0 ** -10 * np.maximum(np.abs(want.astype(np.float64)), 2.0 ** -14)
    worst = (diff - ulp - 1e-5 * magnitude).max()
    assert worst <= 0, f"{what}: {worst:.3e} beyond one fp16 ulp + fp32 reordering room"
    assert (got == want).mean() >= 0.97, f"{what}: only {(got == want).mean():.4f} of the outputs bit-equal"
    assert diff.max() / max(np.abs(want).max(), 1e-6) < 5e-3, what  # Tolerance.fp16Reduction


def _case(ctx, bits, rows, n, tokens, seed, label=None, **kw):
    packed, scales, biases = _weights(rows, n, bits, seed, label)
    if label is None:
        x = np.random.default_rng(seed + 1).uniform(-1.0, 1.0, (tokens, n)).astype(np.float16)
    else:
        x = oracle.fill_uniform(seed, label + "-x", -1.0, 1.0, tokens * n).reshape(tokens, n).astype(np.float16)
    got = _project(ctx, bits, packed, scales, biases, x, **kw)
    want = oracle.affine_projection(packed, scales, biases, x.astype(np.float32), bits)
    _assert_parity(got, want, _magnitude(packed, scales, biases, x, bits), f"bits={bits} m={rows} n={n} T={tokens}")
    return got


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,n,seed", [(128, 128, 0xC1), (1024, 2816, 0xC2), (64, 64, 0xC3)])
def test_reference_gemv_shapes(gpu_ctx, bits, m, n, seed):
    # DequantInt4GEMVTests.swift:114-124: weights uniform(-0.5, 0.5) quantised per row, x uniform(-1, 1) in fp16
    _case(gpu_ctx, bits, m, n, 1, seed, label=f"int4-gemv-kernel-m{m}-n{n}")


@pytest.mark.parametrize("bits", [4, 8])
def test_weights_at_a_2_aligned_not_4_aligned_offset(gpu_ctx, bits):
    # DequantInt4GEMVTests.swift:126-133: the resident layout leaves tensors 2-byte aligned only
    _case(gpu_ctx, bits, 128, 2816, 1, 0xC4, label="int4-gemv-kernel-m128-n2816-off2", weights_offset=2)
    _case(gpu_ctx, bits, 65, 192, 3, 0xC5, weights_offset=6)


@pytest.mark.parametrize("m", [64, 65, 128, 129])
@pytest.mark.parametrize("n", [64, 128, 192, 256, 320, 512])
def test_reference_sweep(gpu_ctx, m, n):
    # DequantInt4GEMVTests.swift:135-141 (OffByMultiples.multiplesOfGroup up to 512)
    _case(gpu_ctx, 4, m, n, 1, m * 0x9E37 + n)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("tokens", [1, 2, 4, 5, 8, 9, 10, 31, 32, 33, 100])
def test_o_proj_shape_over_token_counts(gpu_ctx, bits, tokens):
    # Qwen3.6-35B-A3B o_proj: hidden 2048 x (16 heads * 256); decode 1 row, two-row and wide verify, a batch
    rows, n = 2048, 4096
    packed, scales, biases = _weights(rows, n, bits, 11 + bits)
    x = np.random.default_rng(tokens).standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x)
    want = oracle.affine_projection(packed, scales, biases, x.astype(np.float32), bits)
    _assert_parity(got, want, _magnitude(packed, scales, biases, x, bits), f"o_proj bits={bits} T={tokens}")


@pytest.mark.parametrize("bits,m,n,tokens", [(4, 96, 8192, 40), (8, 33, 6144, 7), (4, 2816, 4096, 5), (8, 1000, 704, 70)])
def test_other_shapes_and_padded_strides(gpu_ctx, bits, m, n, tokens):
    # 8192 columns: more groups than a wavefront keeps in registers; row counts off the 32-row tile
    _case(gpu_ctx, bits, m, n, tokens, 1000 + m + n, x_stride=n + 24, y_stride=m + 5)


def test_rows_are_independent_of_their_neighbours(gpu_ctx):
    # a token's row does not depend on where it sits in the batch: permuting x permutes y bit for bit, and a
    # sub-batch gives the same bits as the full one (up to 9 tokens take a different kernel with another order
    # of the fp32 sums: there the same row agrees to the rounding of that order)
    bits, rows, n, tokens = 4, 512, 1024, 70
    packed, scales, biases = _weights(rows, n, bits, 5)
    x = np.random.default_rng(6).standard_normal((tokens, n)).astype(np.float16)
    perm = np.random.default_rng(7).permutation(tokens)
    base = _project(gpu_ctx, bits, packed, scales, biases, x)
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[perm]), base[perm])
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[37:50]), base[37:50])
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x), base)  # and the same bits every time
    few = _project(gpu_ctx, bits, packed, scales, biases, x[40:43])
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[41:42]), few[1:2])
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[[42, 40, 41, 42]])[1:], few)
    _assert_parity(few, base[40:43], _magnitude(packed, scales, biases, x[40:43], bits), "3 tokens against the same rows in a batch")


GEMM_MIN_TOKENS = 513  # from here on a chunk takes the GEMM kernel, whose weights are rounded to fp16 like the reference's tensor-op tile


def _sampled(tokens):
    return np.unique(np.concatenate([[0, 31, 32, 33, 127, 128, tokens - 129, tokens - 33, tokens - 32, tokens - 1],
                                     np.random.default_rng(79).integers(0, tokens, 38)]))


@pytest.mark.parametrize("bits,m,n,tokens", [(4, 2048, 512, 512), (4, 2048, 8192, 512), (8, 1024, 1024, 500), (4, 130, 4096, GEMM_MIN_TOKENS - 1)])
def test_batches_below_the_gemm_threshold_on_sampled_tokens(gpu_ctx, bits, m, n, tokens):
    # many 32-token slabs: workgroups walk several row tiles with their x fragments kept (or, at 8192 columns,
    # reloaded); same arithmetic and same bar as a single row
    packed, scales, biases = _weights(m, n, bits, 70 + bits)
    x = np.random.default_rng(71).standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x)
    pick = _sampled(tokens)
    want = oracle.affine_projection(packed, scales, biases, x[pick].astype(np.float32), bits)
    _assert_parity(got[pick], want, _magnitude(packed, scales, biases, x[pick], bits), f"batch bits={bits} m={m} n={n}")
    assert np.isfinite(got).all()
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[pick[3]:pick[3] + 12])[0], got[pick[3]])


@pytest.mark.parametrize("bits,m,n,tokens", [(4, 2048, 4096, 4096), (8, 2048, 4096, GEMM_MIN_TOKENS), (4, 1000, 8192, 1400), (8, 300, 512, 2047),
                                              (4, 256, 64, GEMM_MIN_TOKENS)])
def test_chunks_take_the_gemm_with_half_weights(gpu_ctx, bits, m, n, tokens):
    # a prefill chunk's o_proj (4096 tokens at the model's shape) and shapes off the 128 x 256 tile.  The oracle
    # is the reference's tensor-op arithmetic (weights rounded to half, tensorops.metal:80-125) on sampled tokens
    # that cover tile edges; against the exactly factored result the two stay inside the reference's own bar.
    packed, scales, biases = _weights(m, n, bits, 77 + bits)
    x = np.random.default_rng(78).standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x)
    pick = _sampled(tokens)
    want = oracle.affine_projection(packed, scales, biases, x[pick].astype(np.float32), bits, half_weights=True)
    _assert_parity(got[pick], want, _magnitude(packed, scales, biases, x[pick], bits), f"chunk bits={bits} m={m} n={n}")
    exact = oracle.affine_projection(packed, scales, biases, x[pick].astype(np.float32), bits)
    assert np.abs(got[pick] - exact).max() / np.abs(exact).max() < 5e-3  # Tolerance.fp16Reduction
    assert np.isfinite(got).all()
    # a token's row does not depend on its neighbours or its place in the tile
    perm = np.random.default_rng(80).permutation(tokens)
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[perm]), got[perm])


def test_gemm_with_padded_strides_and_unaligned_weights(gpu_ctx):
    packed, scales, biases = _weights(200, 320, 4, 90)
    x = np.random.default_rng(91).standard_normal((GEMM_MIN_TOKENS + 10, 320)).astype(np.float16)
    want = oracle.affine_projection(packed, scales, biases, x.astype(np.float32), 4, half_weights=True)
    for kw in ({"x_stride": 328, "y_stride": 203}, {"weights_offset": 2}):
        got = _project(gpu_ctx, 4, packed, scales, biases, x, **kw)
        _assert_parity(got, want, _magnitude(packed, scales, biases, x, 4), f"gemm {kw}")


@pytest.mark.parametrize("bits,m,n,tokens,kw", [(4, 200, 1152, 600, {"x_stride": 1160, "y_stride": 203}), (4, 200, 1152, 600, {"weights_offset": 2}),
                                                 (8, 260, 1088, 700, {}), (4, 2048, 4096, 2048, {}), (4, 384, 8192, 2000, {"y_stride": 392})])
def test_gemm_with_the_columns_in_two_parts(gpu_ctx, bits, m, n, tokens, kw):
    # no more tiles of 128 tokens x 128 rows than the card has CUs, 16 groups of columns or more: the workgroup's
    # eight wavefronts take the columns in two parts and add their accumulators.  18 and 17 groups: a last span
    # that is partly (or, for the second part, mostly) past the matrix; 128 groups: the scales and biases are
    # staged a second time on the way.
    packed, scales, biases = _weights(m, n, bits, 95 + bits)
    x = np.random.default_rng(96).standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x, **kw)
    pick = _sampled(tokens)
    want = oracle.affine_projection(packed, scales, biases, x[pick].astype(np.float32), bits, half_weights=True)
    _assert_parity(got[pick], want, _magnitude(packed, scales, biases, x[pick], bits), f"two parts bits={bits} m={m} n={n} {kw}")
    assert np.isfinite(got).all()
    perm = np.random.default_rng(97).permutation(tokens)
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[perm], **kw), got[perm])


@pytest.mark.parametrize("bits,m,n,tokens,kw", [(8, 2048, 512, 2176, {}), (4, 2000, 320, 2200, {"x_stride": 328, "y_stride": 2003}),
                                                 (4, 2000, 320, 2200, {"weights_offset": 2}), (4, 300, 4096, 16500, {})])
def test_gemm_in_tiles_of_256_rows(gpu_ctx, bits, m, n, tokens, kw):
    # more tiles of 128 tokens x 128 rows than the card has CUs, and tiles of 256 rows whose last round fills most of
    # the chip: eight wavefronts share one x tile.  Row counts off the tile, 5 groups of columns (a last span partly
    # past the matrix), padded strides, weights at a 2-byte offset, 8-bit levels, and two rounds of workgroups less one.
    packed, scales, biases = _weights(m, n, bits, 85 + bits)
    x = np.random.default_rng(86).standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x, **kw)
    pick = _sampled(tokens)
    want = oracle.affine_projection(packed, scales, biases, x[pick].astype(np.float32), bits, half_weights=True)
    _assert_parity(got[pick], want, _magnitude(packed, scales, biases, x[pick], bits), f"256-row tiles bits={bits} m={m} n={n} {kw}")
    assert np.isfinite(got).all()
    perm = np.random.default_rng(87).permutation(tokens)
    assert np.array_equal(_project(gpu_ctx, bits, packed, scales, biases, x[perm], **kw), got[perm])


def test_closed_forms(gpu_ctx):
    # constant rows are carried by the bias term alone (Int8AffineGEMVTests.swift:104-110); a one-hot x picks a column
    for bits in (4, 8):
        raw = np.full((40, 128), 0.375, dtype=np.float32)
        packed, scales, biases = oracle.affine_quantize_rows(raw, bits)
        x = np.random.default_rng(3).uniform(-1, 1, (2, 128)).astype(np.float16)
        got = _project(gpu_ctx, bits, packed, scales, biases, x)
        want = 0.375 * x.astype(np.float64).sum(axis=1, keepdims=True)
        assert (np.abs(got - want) <= 2.0 ** -10 * np.abs(want) + 1e-6).all()
        raw = np.random.default_rng(4).uniform(-0.5, 0.5, (70, 192)).astype(np.float32)
        packed, scales, biases = oracle.affine_quantize_rows(raw, bits)
        dense = oracle.affine_dequantize_rows(packed, scales, biases, bits)
        x = np.zeros((3, 192), dtype=np.float16)
        x[0, 0], x[1, 77], x[2, 191] = 1.0, 1.0, 1.0
        got = _project(gpu_ctx, bits, packed, scales, biases, x)
        for t, column in enumerate((0, 77, 191)):
            assert np.array_equal(got[t], dense[:, column].astype(np.float16).astype(np.float32))


def test_behind_the_gate(gpu_ctx):
    # the runner's sequence: gated decode attention, then o_proj on its output, against the oracle's same chain
    import torch
    from tinytitan_amd.engine import Attention, KVCacheManager
    H, KH, D, T, hidden = 16, 2, 256, 700, 2048
    r = np.random.default_rng(21)
    k, v = (r.standard_normal((T, KH * D)).astype(np.float16) for _ in range(2))
    q, gate = (r.standard_normal((1, 1, H, D)).astype(np.float16) for _ in range(2))
    packed, scales, biases = _weights(hidden, H * D, 4, 22)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=T, initial_capacity=T)
    kd, vd, qd, gd = _dev(k), _dev(v), _dev(q), _dev(gate)
    out = torch.zeros_like(qd)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    Attention(gpu_ctx).encode_full(kv, 0, qd, out, H, [T], 0.0625, gate=gd)
    gpu_ctx.synchronize()
    attn = out.cpu().numpy().reshape(1, H * D)
    got = _project(gpu_ctx, 4, packed, scales, biases, attn)
    want_attn = oracle.decode(q.reshape(H, D), k, v, H, KH, D, 0.0625, gate=gate.reshape(H, D))
    want_attn = want_attn.reshape(1, -1).astype(np.float16)
    want = oracle.affine_projection(packed, scales, biases, want_attn.astype(np.float32), 4)
    # attention carries its own bar (2e-3 per element of x); through 4096 columns of |w| <= 0.5 that is
    # far below the projection's output scale
    spread = np.abs(want).max()
    assert np.abs(got - want).max() <= 2e-2 * spread
    same_x = oracle.affine_projection(packed, scales, biases, attn.astype(np.float32), 4)
    _assert_parity(got, same_x, _magnitude(packed, scales, biases, attn, 4), "o_proj on the GPU's own attention output")
    kv.close()


def test_graph_replay(gpu_ctx):
    # a decode row and a 40-token batch captured in one graph: replays equal the eager results.  The larger
    # kernels set their LDS limit on first use in a process, which a capture refuses: the first use is eager.
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import AffineProjection, HIPContext, TinyTitanHIPError
    ctx = HIPContext(gpu_ctx.device)
    rows, n, tokens = 2048, 4096, 40
    packed, scales, biases = _weights(rows, n, 4, 31)
    x = np.random.default_rng(32).standard_normal((tokens, n)).astype(np.float16)
    wd, sd, bd, xd = _dev(packed), _dev(scales.view(np.int16)), _dev(biases.view(np.int16)), _dev(x)
    yd = torch.zeros((tokens, rows), dtype=torch.float16, device="cuda")
    y1 = torch.zeros((1, rows), dtype=torch.float16, device="cuda")
    proj = AffineProjection(ctx)

    chunk = GEMM_MIN_TOKENS + 20  # and a chunk through the GEMM kernel, on a smaller matrix
    packed_c, scales_c, biases_c = _weights(256, 512, 8, 33)
    wc, sc, bc = _dev(packed_c), _dev(scales_c.view(np.int16)), _dev(biases_c.view(np.int16))
    xc = _dev(np.random.default_rng(34).standard_normal((chunk, 512)).astype(np.float16))
    yc = torch.zeros((chunk, 256), dtype=torch.float16, device="cuda")

    def both():
        proj.encode(4, wd, sd, bd, xd, yd, rows, n, tokens)
        proj.encode(4, wd, sd, bd, xd[7:8], y1, rows, n, 1)
        proj.encode(8, wc, sc, bc, xc, yc, 256, 512, chunk)

    torch.cuda.synchronize()
    both()
    ctx.synchronize()
    eager = (yd.clone(), y1.clone(), yc.clone())
    ctx.graph_begin()
    both()
    graph = ctx.graph_end()
    for replay in range(3):
        yd.zero_()
        y1.zero_()
        yc.zero_()
        torch.cuda.synchronize()
        graph.launch()
        ctx.synchronize()
        assert torch.equal(yd, eager[0]) and torch.equal(y1, eager[1]) and torch.equal(yc, eager[2]), f"replay {replay}"
        proj.encode(4, wd, sd, bd, xd[:9], yd[:9], rows, n, 9)  # eager work between replays
        ctx.synchronize()
    graph.close()
    ctx.close()


def test_argument_errors(gpu_ctx):
    import torch
    from tinytitan_amd import capi
    from tinytitan_amd.engine import AffineProjection, TinyTitanHIPError
    proj = AffineProjection(gpu_ctx)
    w = torch.zeros(64 * 128 + 16, dtype=torch.uint8, device="cuda")
    s = torch.zeros((64, 4), dtype=torch.int16, device="cuda")
    x = torch.zeros((2, 264), dtype=torch.float16, device="cuda")
    y = torch.full((2, 64), 5.0, dtype=torch.float16, device="cuda")

    def status(*args, **kw):
        with pytest.raises(TinyTitanHIPError) as e:
            proj.encode(*args, **kw)
        return e.value.status

    assert status(5, w, s, s, x, y, 64, 256, 2, 264, 64) == capi.ERR_SHAPE            # bits
    assert status(4, w, s, s, x, y, 64, 200, 2, 264, 64) == capi.ERR_SHAPE            # columns % 64
    assert status(4, w, s, s, x, y, 64, 256, 2, 248, 64) == capi.ERR_SHAPE            # x stride below the row
    assert status(4, w, s, s, x, y, 64, 256, 2, 264, 60) == capi.ERR_SHAPE            # y stride below the row
    assert status(4, w, s, s, x, y, 64, 256, 2, 260, 64) == capi.ERR_SHAPE            # x rows off 16 bytes
    assert status(4, w, s, s, x.view(-1)[4:260].view(1, 256), y, 64, 256, 1, 256, 64) == capi.ERR_SHAPE
    assert status(4, w, s, s, x, y, 64, 256, 2, 264, 64, weights_offset=1) == capi.ERR_SHAPE  # odd address
    assert status(4, w, s, s, x, y, 0, 256, 2, 264, 64) == capi.ERR_INVALID_ARGUMENT
    assert status(4, w, s, s, x, y, 64, 256, -1, 264, 64) == capi.ERR_INVALID_ARGUMENT
    proj.encode(4, w, s, s, x, y, 64, 256, 0, 264, 64)  # no tokens: nothing to do, nothing written
    gpu_ctx.synchronize()
    assert (y == 5.0).all()
    lib = gpu_ctx._lib
    assert lib.tt_hip_affine_projection(gpu_ctx.handle, 4, None, s.data_ptr(), s.data_ptr(), x.data_ptr(), y.data_ptr(),
                                        64, 256, 1, 264, 64) == capi.ERR_INVALID_ARGUMENT


@pytest.mark.parametrize("seed", range(32))
def test_random_shapes(gpu_ctx, seed):
    # row counts off every tile size (8, 32, 128), column counts from one group to more than a wavefront holds,
    # token counts across the three kernels' ranges, padded strides, weights at 2-byte-aligned offsets
    rng = np.random.default_rng(7000 + seed)
    bits = int(rng.choice([4, 8]))
    rows = int(rng.integers(1, 700))
    n = 64 * int(rng.choice([1, 2, 3, 5, 8, 11, 16, 44, 64, 96, 130]))
    tokens = int(rng.choice([1, 2, 3, 4, 5, 17, 32, 33, 70, 200])) if seed % 4 else int(rng.integers(GEMM_MIN_TOKENS, GEMM_MIN_TOKENS + 300))
    if tokens >= GEMM_MIN_TOKENS:
        rows, n = min(rows, 300), min(n, 64 * 16)  # keeps the oracle's share of the test short
    kw = {}
    if rng.integers(0, 2):
        kw["x_stride"] = n + 8 * int(rng.integers(1, 5))
        kw["y_stride"] = rows + int(rng.integers(1, 9))
    if rng.integers(0, 3) == 0:
        kw["weights_offset"] = 2 * int(rng.integers(1, 8))
    packed, scales, biases = _weights(rows, n, bits, 7100 + seed)
    x = rng.standard_normal((tokens, n)).astype(np.float16)
    got = _project(gpu_ctx, bits, packed, scales, biases, x, **kw)
    want = oracle.affine_projection(packed, scales, biases, x.astype(np.float32), bits, half_weights=tokens >= GEMM_MIN_TOKENS)
    _assert_parity(got, want, _magnitude(packed, scales, biases, x, bits), f"seed {seed}: bits {bits} m {rows} n {n} T {tokens} {kw}")
