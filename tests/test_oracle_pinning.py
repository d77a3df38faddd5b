"""Pins the CPU oracle: known answers, closed forms, an independent numpy
restatement and the equivalences the reference's own tests assert."""
import numpy as np
import pytest

import oracle
from tests.np_reference import attention_rows
from tinytitan_amd import synthetic


def rng(seed):
    return np.random.default_rng(seed)


# ---- PRNG ---------------------------------------------------------------------------------

def test_splitmix64_known_answers():
    # Published SplitMix64 test vector (Vigna's reference implementation, seed 1234567).
    g = oracle.SplitMix64(1234567)
    assert [g.next() for _ in range(5)] == [
        6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]
    assert list(synthetic.splitmix64(1234567, 5)) == [
        6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431, 16408922859458223821]


def test_fnv1a_known_answers():
    # FNV-1a 64 published vectors: "" -> offset basis, "a", "foobar".
    assert oracle.seedtree_key(0, "") == 0xCBF29CE484222325
    assert oracle.seedtree_key(0, "a") == 0xAF63DC4C8601EC8C
    assert oracle.seedtree_key(0, "foobar") == 0x85944171F73967E8
    assert synthetic.fnv1a64("foobar") == 0x85944171F73967E8
    assert oracle.seedtree_key(0xDEADBEEF, "q") == synthetic.seed_key(0xDEADBEEF, "q")


def test_uniform_matches_numpy_generator_and_range():
    a = oracle.fill_uniform(0xC1, "q", -0.5, 0.5, 4096)
    b = synthetic.uniform(0xC1, "q", 4096)
    assert np.array_equal(a, b)
    assert a.min() >= -0.5 and a.max() < 0.5
    assert abs(a.mean()) < 0.02


def test_normal_stream_is_chunk_invariant_and_standard():
    a = synthetic.normal(7, "x", 100001, chunk=1 << 22)
    b = synthetic.normal(7, "x", 100001, chunk=4096)
    assert np.array_equal(a, b)
    assert abs(a.mean()) < 0.02 and abs(a.std() - 1.0) < 0.02


# ---- fp16 ---------------------------------------------------------------------------------

def test_f16_to_f32_exhaustive():
    bits = np.arange(65536, dtype=np.uint16)
    ours = oracle.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    both_nan = np.isnan(ours) & np.isnan(ref)
    assert np.array_equal(ours[~both_nan].view(np.uint32), ref[~both_nan].view(np.uint32))


def test_f32_to_f16_round_to_nearest_even():
    r = rng(1)
    x = np.concatenate([
        r.standard_normal(200000).astype(np.float32) * 4,
        (r.standard_normal(50000) * 1e-6).astype(np.float32),       # subnormal halves
        (r.standard_normal(50000) * 3e4).astype(np.float32),        # near overflow
        np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, -1e9, 2.0 ** -24, 2.0 ** -25, 1.5 * 2.0 ** -25,
                  np.inf, -np.inf], dtype=np.float32),
    ])
    # every exact midpoint between adjacent normal halves -> ties must go to even
    h = np.arange(0x0400, 0x7BFF, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float32)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float32)
    x = np.concatenate([x, (lo + hi) / 2])
    with np.errstate(over="ignore"):
        expect = x.astype(np.float16).view(np.uint16)
    assert np.array_equal(oracle.f32_to_f16_bits(x), expect)


# ---- CPUOps -------------------------------------------------------------------------------

def test_softmax_closed_forms():
    # sums to one, shift invariant (tests/TinyTitan/CPUEngine/CPUEngineTests.swift:909-916)
    x = np.array([1.0, 2.0, 3.0, 4.0], dtype=np.float32)
    p = oracle.softmax(x)
    assert abs(p.sum() - 1.0) < 1e-6
    assert np.allclose(p, oracle.softmax(x + 100.0), atol=1e-6)
    e = np.exp(x.astype(np.float64) - 4.0)
    assert np.allclose(p, e / e.sum(), atol=1e-7)
    assert np.allclose(oracle.softmax(np.zeros(7, np.float32)), 1.0 / 7.0)
    big = oracle.softmax(np.array([1000.0, 0.0], np.float32))
    assert big[0] == 1.0 and big[1] == 0.0  # no overflow, exact saturation


def test_sigmoid_closed_forms():
    # CPUEngineTests.swift:948-956
    assert oracle.sigmoid(0.0) == 0.5
    assert abs(oracle.sigmoid(2.0) + oracle.sigmoid(-2.0) - 1.0) < 1e-7
    assert abs(oracle.sigmoid(1.0) - 0.7310585786300049) < 1e-7
    assert oracle.sigmoid(100.0) == 1.0 and oracle.sigmoid(-100.0) < 1e-40


def test_rope_identities():
    # CPUEngineTests.swift:921-946
    r = rng(2)
    x = r.standard_normal(2 * 256).astype(np.float32)
    assert np.array_equal(oracle.rope_neox(x, 256, 64, 0, 1e7), x)  # position 0 is the identity
    y = oracle.rope_neox(x, 256, 64, 12345, 1e7).reshape(2, 256)
    xr = x.reshape(2, 256)
    assert np.array_equal(y[:, 64:], xr[:, 64:])  # tail untouched
    # pairs are (i, i + 32): each pair's norm is preserved, adjacent pairing would not hold this
    assert np.allclose(y[:, :32] ** 2 + y[:, 32:64] ** 2, xr[:, :32] ** 2 + xr[:, 32:64] ** 2, rtol=1e-5)
    # pair 0 has frequency theta^0 = 1: a plain rotation by `position` radians
    pos = 3
    z = oracle.rope_neox(x, 256, 64, pos, 1e7).reshape(2, 256)
    assert np.allclose(z[:, 0], xr[:, 0] * np.cos(3.0) - xr[:, 32] * np.sin(3.0), atol=1e-6)
    assert np.allclose(z[:, 32], xr[:, 0] * np.sin(3.0) + xr[:, 32] * np.cos(3.0), atol=1e-6)
    # pair i rotates by pos * theta^(-2i/64)
    i = 5
    ang = pos * (1e7 ** (-2 * i / 64))
    assert np.allclose(z[:, i], xr[:, i] * np.cos(ang) - xr[:, 32 + i] * np.sin(ang), atol=1e-6)
    # the vectorised generator used for C2's K agrees with the oracle row by row
    rows = r.standard_normal((5, 2, 256)).astype(np.float32)
    positions = np.array([0, 1, 17, 4096, 32767])
    got = synthetic.rope_neox_rows(rows, positions, 64, 1e7)
    for t, p in enumerate(positions):
        want = oracle.rope_neox(rows[t].reshape(-1), 256, 64, int(p), 1e7).reshape(2, 256)
        # angle = position * frequency in fp32: one ulp of the frequency moves the angle by
        # position * 2^-24, so large positions are compared at that sensitivity
        assert np.allclose(got[t], want, atol=2e-6 + 8.0 * float(p) * 2.0 ** -24)


def test_rms_norm_per_slice_closed_forms():
    # CPUEngineTests.swift:886-901: unit root-mean-square; every slice takes its OWN statistics.
    y = oracle.rms_norm_per_slice(np.array([3, 4, 0, 0], np.float32), 4, np.ones(4, np.float32), 0.0)
    assert abs(np.mean(y ** 2) - 1) < 1e-5
    y = oracle.rms_norm_per_slice(np.array([1, 1, 100, 100], np.float32), 2, np.ones(2, np.float32), 0.0)
    assert abs(y[0] - 1) < 1e-4 and abs(y[2] - 1) < 1e-4
    # a constant slice c normalises to sign(c) * gamma; scaling the input changes nothing (eps = 0)
    r = rng(3)
    gamma = r.standard_normal(256).astype(np.float32)
    y = oracle.rms_norm_per_slice(np.full(256, -7.5, np.float32), 256, gamma, 0.0)
    assert np.allclose(y, -gamma, rtol=1e-6)
    x = r.standard_normal(3 * 256).astype(np.float32)
    a = oracle.rms_norm_per_slice(x, 256, gamma, 0.0)
    b = oracle.rms_norm_per_slice(x * 37.0, 256, gamma, 0.0)
    assert np.allclose(a, b, rtol=2e-6, atol=1e-7)
    # against the formula written out independently in float64, with epsilon inside the root
    x64 = x.reshape(3, 256).astype(np.float64)
    want = x64 / np.sqrt((x64 ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma.astype(np.float64)
    got = oracle.rms_norm_per_slice(x, 256, gamma, 1e-6).reshape(3, 256)
    assert np.allclose(got, want, rtol=3e-6, atol=1e-7)
    # epsilon is added to the MEAN of squares, not to the sum and not outside the root
    tiny = np.full(4, 1e-3, np.float32)
    y = oracle.rms_norm_per_slice(tiny, 4, np.ones(4, np.float32), 1e-6)
    assert np.allclose(y, 1e-3 / np.sqrt(1e-6 + 1e-6), rtol=1e-5)


def test_qkv_epilogue_composition():
    # CPUQwen35.swift:266-300: split [query ; gate] per head, norm q and k per head, rotate q and k.
    H, KH, D, T, base = 4, 2, 64, 5, 11
    r = rng(4)
    packed = r.standard_normal((T, H, 2 * D)).astype(np.float32)
    k = r.standard_normal((T, KH * D)).astype(np.float32)
    qg, kg = r.standard_normal(D).astype(np.float32), r.standard_normal(D).astype(np.float32)
    q_out, g_out, k_out = oracle.qkv_epilogue(packed, k, T, H, KH, D, qg, kg, 1e-6, 16, 1e7, base)
    # the gate is the second half of every head's packed row, bit for bit; a strided (even/odd) or
    # halves-of-the-whole-row split would fail here
    assert np.array_equal(g_out.reshape(T, H, D), packed[:, :, D:])
    # independent float64 statement: norm, then NeoX rotation of the first 16 dims, pairs (i, i+8)
    def ref(x, gamma, pos):  # x [heads][D]
        x = x.astype(np.float64)
        y = x / np.sqrt((x ** 2).mean(axis=1, keepdims=True) + 1e-6) * gamma.astype(np.float64)
        i = np.arange(8)
        ang = pos * (1e7 ** (-2.0 * i / 16))
        a, b = y[:, :8].copy(), y[:, 8:16].copy()
        y[:, :8] = a * np.cos(ang) - b * np.sin(ang)
        y[:, 8:16] = a * np.sin(ang) + b * np.cos(ang)
        return y
    for t in range(T):
        assert np.allclose(q_out[t].reshape(H, D), ref(packed[t, :, :D], qg, base + t), rtol=2e-5, atol=2e-6)
        assert np.allclose(k_out[t].reshape(KH, D), ref(k[t].reshape(KH, D), kg, base + t), rtol=2e-5, atol=2e-6)
    # position 0: no rotation, the norm alone
    q0, _, k0 = oracle.qkv_epilogue(packed[:1], k[:1], 1, H, KH, D, qg, kg, 1e-6, 16, 1e7, 0)
    assert np.array_equal(q0.reshape(-1), oracle.rms_norm_per_slice(packed[0, :, :D].reshape(-1), D, qg, 1e-6))
    assert np.array_equal(k0.reshape(-1), oracle.rms_norm_per_slice(k[0], D, kg, 1e-6))
    # a chunk is its rows one at a time (CPUQwen35+BatchAttention.swift:49-86 vs CPUQwen35.swift:266-300)
    for t in range(T):
        q1, g1, k1 = oracle.qkv_epilogue(packed[t:t + 1], k[t:t + 1], 1, H, KH, D, qg, kg, 1e-6, 16, 1e7, base + t)
        assert np.array_equal(q1[0], q_out[t]) and np.array_equal(g1[0], g_out[t]) and np.array_equal(k1[0], k_out[t])
    # the norm comes BEFORE the rotation (they do not commute when gamma differs inside a pair)
    swapped = oracle.rms_norm_per_slice(oracle.rope_neox(packed[2, :, :D].reshape(-1), D, 16, base + 2, 1e7), D, qg, 1e-6)
    assert not np.allclose(swapped, q_out[2], atol=1e-3)


# ---- decode oracle ------------------------------------------------------------------------

def _decode_inputs(seed, H, KH, D, T, dist="uniform"):
    r = rng(seed)
    f = (lambda *s: (r.random(s) - 0.5)) if dist == "uniform" else (lambda *s: r.standard_normal(s))
    q = f(H, D).astype(np.float16).astype(np.float32)
    k = f(T, KH, D).astype(np.float16).astype(np.float32)
    v = f(T, KH, D).astype(np.float16).astype(np.float32)
    return q, k, v


# shapes of tests/TinyTitan/Validation/Reference/AttentionReferenceTests.swift:48-79 plus the configs' geometry
@pytest.mark.parametrize("D,H,KH,T", [(64, 4, 2, 128), (64, 4, 2, 32), (64, 8, 1, 128), (128, 8, 4, 64),
                                      (256, 8, 2, 300), (256, 16, 2, 257)])
def test_decode_two_formulations_and_numpy(D, H, KH, T):
    q, k, v = _decode_inputs(D + T, H, KH, D, T, "normal")
    scale = 1.0 / np.sqrt(D)
    a = oracle.decode(q, k, v, H, KH, D, scale)
    b = oracle.attention_ref(q, k, v, D, H, KH, T)  # scale defaults to 1/sqrt(D)
    n = attention_rows(q[None], k, v, T - 1, scale)[0]
    ref_norm = np.abs(n).max()
    assert np.abs(a - b).max() / ref_norm < 1e-5
    assert np.abs(a - n).max() / ref_norm < 1e-5
    assert np.abs(b - n).max() / ref_norm < 1e-5


def test_attention_ref_window():
    q, k, v = _decode_inputs(9, 4, 2, 64, 128)
    a = oracle.attention_ref(q, k, v, 64, 4, 2, 128, window=64)
    n = attention_rows(q[None], k, v, 127, 1 / 8.0, window=64)[0]
    assert np.abs(a - n).max() < 1e-6
    assert np.abs(a - oracle.attention_ref(q, k, v, 64, 4, 2, 128)).max() > 1e-4  # the window matters
    full = oracle.attention_ref(q, k, v, 64, 4, 2, 128, window=128)  # window >= seq: no clipping
    assert np.array_equal(full, oracle.attention_ref(q, k, v, 64, 4, 2, 128))


def test_decode_closed_forms():
    H, KH, D, T = 8, 2, 256, 50
    q, k, v = _decode_inputs(3, H, KH, D, T, "normal")
    # single key: the output is that V row, whatever the score
    one = oracle.decode(q, k[:1], v[:1], H, KH, D, 0.0625)
    for h in range(H):
        assert np.array_equal(one[h], v[0, h // 4])
    # q = 0: uniform weights -> mean of V
    uni = oracle.decode(np.zeros_like(q), k, v, H, KH, D, 0.0625)
    for h in range(H):
        assert np.allclose(uni[h], v[:, h // 4].mean(axis=0), atol=1e-6)
    # empty cache: zeros, no NaN
    empty = oracle.decode(q, k[:0], v[:0], H, KH, D, 0.0625)
    assert np.array_equal(empty, np.zeros((H, D), np.float32))
    # gate 0 halves the output exactly; the gate applies after normalisation
    base = oracle.decode(q, k, v, H, KH, D, 0.0625)
    assert np.array_equal(oracle.decode(q, k, v, H, KH, D, 0.0625, gate=np.zeros((H, D), np.float32)), base * 0.5)
    g = rng(4).standard_normal((H, D)).astype(np.float32)
    gated = oracle.decode(q, k, v, H, KH, D, 0.0625, gate=g)
    assert np.allclose(gated, base / (1 + np.exp(-g.astype(np.float64))), rtol=1e-6, atol=1e-7)
    # one dominant key saturates to its V row
    k2 = k.copy()
    k2[7, 0] = q[0] * 50
    assert np.allclose(oracle.decode(q, k2, v, H, KH, D, 0.0625)[0], v[7, 0], atol=1e-6)


def test_gqa_mapping_is_head_div_group():
    # Design of CPUEngineTests.swift:788-818: shared KV heads == written-out duplicate heads,
    # and the strided pairing (head % kvHeads) gives a different answer.
    H, KH, D, T = 8, 2, 64, 40
    q, k, v = _decode_inputs(5, H, KH, D, T, "normal")
    shared = oracle.decode(q, k, v, H, KH, D, 0.125)
    k_dup = np.repeat(k, H // KH, axis=1)  # [T][H][D]: kv head h//group written out per q head
    v_dup = np.repeat(v, H // KH, axis=1)
    assert np.allclose(shared, oracle.decode(q, k_dup, v_dup, H, H, D, 0.125), atol=1e-7)
    k_str = np.tile(k, (1, H // KH, 1))  # head % kvHeads pairing
    v_str = np.tile(v, (1, H // KH, 1))
    assert np.abs(shared - oracle.decode(q, k_str, v_str, H, H, D, 0.125)).max() > 1e-3


# ---- prefill / verify oracle --------------------------------------------------------------

def _batch_inputs(seed, H, KH, D, positions, tokens):
    r = rng(seed)
    q = r.standard_normal((tokens, H, D)).astype(np.float16).astype(np.float32)
    k = r.standard_normal((positions, KH, D)).astype(np.float16).astype(np.float32)
    v = r.standard_normal((positions, KH, D)).astype(np.float16).astype(np.float32)
    g = r.standard_normal((tokens, H, D)).astype(np.float16).astype(np.float32)
    return q, k, v, g


@pytest.mark.parametrize("H,KH,D,base,tokens", [(4, 2, 8, 0, 3), (4, 2, 8, 5, 4), (16, 2, 256, 60, 4), (8, 2, 64, 0, 70)])
def test_attention_batch_row_equals_decode_step(H, KH, D, base, tokens):
    # Row r of a chunk == a decode step at base + r over base + r + 1 keys
    # (WideVerifyIdentityTests.swift:60-121 asserts this of the GPU paths).
    positions = base + tokens
    q, k, v, g = _batch_inputs(H * D + base, H, KH, D, positions, tokens)
    scale = 1.0 / np.sqrt(D)
    batch = oracle.attention_batch(q, k, v, tokens, base, H, KH, D, scale, gate=g)
    for r in range(tokens):
        step = oracle.decode(q[r], k[:base + r + 1], v[:base + r + 1], H, KH, D, scale, gate=g[r])
        assert np.abs(batch[r] - step).max() < 2e-6
    n = attention_rows(q, k, v, base, scale, gate=g)
    assert np.abs(batch - n).max() / np.abs(n).max() < 1e-5
    # threads only changes who computes a head
    assert np.array_equal(batch, oracle.attention_batch(q, k, v, tokens, base, H, KH, D, scale, gate=g, threads=4))


def test_attention_batch_chunking_invariance_and_limit_error():
    H, KH, D = 4, 2, 16
    q, k, v, _ = _batch_inputs(11, H, KH, D, 24, 24)
    whole = oracle.attention_batch(q, k, v, 24, 0, H, KH, D, 0.25)
    a = oracle.attention_batch(q[:10], k[:10], v[:10], 10, 0, H, KH, D, 0.25)
    b = oracle.attention_batch(q[10:], k, v, 14, 10, H, KH, D, 0.25)
    assert np.abs(np.concatenate([a, b]) - whole).max() < 1e-6
    with pytest.raises(oracle.OracleError):  # limit past the cache: the reference throws (BatchAttention.swift:149-152)
        oracle.attention_batch(q[:4], k[:3], v[:3], 4, 0, H, KH, D, 0.25)


def test_prefill_ref_strides_offsets_and_future_rows():
    # PrefillAttentionTests.swift:306-346: padded strides; :74-93: adversarial future K/V must not leak.
    H, KH, D, start, chunk = 4, 2, 8, 5, 4
    kv_valid = start + chunk
    q, k, v, _ = _batch_inputs(13, H, KH, D, kv_valid + 3, chunk)
    qs, ks = H * D + 3, KH * D + 5
    qp = np.full((chunk, qs), 7.0, np.float32)
    qp[:, :H * D] = q.reshape(chunk, -1)
    kp = np.full((kv_valid + 3, ks), -9.0, np.float32)
    vp = np.full((kv_valid + 3, ks), 1e30, np.float32)
    kp[:, :KH * D] = k.reshape(k.shape[0], -1)
    vp[:, :KH * D] = v.reshape(v.shape[0], -1)
    kp[kv_valid:, :] = 1e4   # rows past kv_valid: huge scores if they leaked
    vp[kv_valid:, :] = 1e30
    got = oracle.prefill_ref(qp, kp, vp, qs, ks, D, H, KH, start, chunk, kv_valid, 0, 0.35)
    want = attention_rows(q, k, v, start, 0.35, kv_valid=kv_valid)
    assert np.abs(got - want).max() < 1e-5
    batch = oracle.attention_batch(q, k[:kv_valid], v[:kv_valid], chunk, start, H, KH, D, 0.35)
    assert np.abs(got - batch).max() < 1e-5
    # future rows inside the chunk are adversarial too: row t must ignore rows > start + t
    k2, v2 = k.copy(), v.copy()
    k2[start + 1:] *= 100
    v2[start + 1:] = 1e6
    a = oracle.prefill_ref(q, k2, v2, H * D, KH * D, D, H, KH, start, chunk, kv_valid, 0, 0.35)
    assert np.abs(a[0] - want[0]).max() < 1e-5
    # sliding window and an empty range (kv_valid = 0 -> zeros)
    w = oracle.prefill_ref(q, k, v, H * D, KH * D, D, H, KH, start, chunk, kv_valid, 3, 0.35)
    assert np.abs(w - attention_rows(q, k, v, start, 0.35, window=3, kv_valid=kv_valid)).max() < 1e-5
    z = oracle.prefill_ref(q, k, v, H * D, KH * D, D, H, KH, 0, chunk, 0, 0, 0.35)
    assert np.array_equal(z, np.zeros_like(z))


@pytest.mark.parametrize("keys", [1, 63, 64, 65, 127, 128, 129, 255, 256, 257])
def test_batch_tile_boundary_key_counts(keys):
    # Key counts around tile edges (PrefillAttentionTests.swift:146-152), oracle vs numpy.
    H, KH, D = 4, 2, 64
    q, k, v, _ = _batch_inputs(keys, H, KH, D, keys, 1)
    got = oracle.attention_batch(q, k, v, 1, keys - 1, H, KH, D, 0.125)
    assert np.abs(got - attention_rows(q, k, v, keys - 1, 0.125)).max() < 2e-6
