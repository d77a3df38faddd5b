"""ctypes binding of the CPU oracle (``oracle/attn_oracle.c``).

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``.  Nothing under ``tinytitan_amd/``
may import this package.

All arrays are numpy ``float32`` in the reference's own CPU layouts
(token-major caches ``[positions][kv_heads*dim]``, queries ``[tokens][heads*dim]``).
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libtt_oracle.so")
_lib = None

_f32p = ctypes.POINTER(ctypes.c_float)
_u16p = ctypes.POINTER(ctypes.c_uint16)


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = ctypes.CDLL(_LIB_PATH)
        L.tt_oracle_splitmix64_next.restype = ctypes.c_uint64
        L.tt_oracle_splitmix64_next.argtypes = [ctypes.POINTER(ctypes.c_uint64)]
        L.tt_oracle_splitmix64_uniform.restype = ctypes.c_float
        L.tt_oracle_splitmix64_uniform.argtypes = [ctypes.POINTER(ctypes.c_uint64), ctypes.c_float, ctypes.c_float]
        L.tt_oracle_seedtree_key.restype = ctypes.c_uint64
        L.tt_oracle_seedtree_key.argtypes = [ctypes.c_uint64, ctypes.c_char_p]
        L.tt_oracle_fill_uniform.restype = None
        L.tt_oracle_fill_uniform.argtypes = [ctypes.c_uint64, ctypes.c_char_p, ctypes.c_float, ctypes.c_float, _f32p, ctypes.c_size_t]
        L.tt_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.tt_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.tt_oracle_f16_to_f32.restype = ctypes.c_float
        L.tt_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.tt_oracle_round_through_f16.restype = None
        L.tt_oracle_round_through_f16.argtypes = [_f32p, ctypes.c_size_t]
        L.tt_oracle_f32_to_f16_array.restype = None
        L.tt_oracle_f32_to_f16_array.argtypes = [_f32p, _u16p, ctypes.c_size_t]
        L.tt_oracle_f16_to_f32_array.restype = None
        L.tt_oracle_f16_to_f32_array.argtypes = [_u16p, _f32p, ctypes.c_size_t]
        L.tt_oracle_sigmoid.restype = ctypes.c_float
        L.tt_oracle_sigmoid.argtypes = [ctypes.c_float]
        L.tt_oracle_softmax_inplace.restype = None
        L.tt_oracle_softmax_inplace.argtypes = [_f32p, ctypes.c_int]
        L.tt_oracle_rope_neox.restype = None
        L.tt_oracle_rope_neox.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_float]
        L.tt_oracle_rms_norm_per_slice.restype = None
        L.tt_oracle_rms_norm_per_slice.argtypes = [_f32p, ctypes.c_int, ctypes.c_int, _f32p, ctypes.c_float]
        L.tt_oracle_qkv_epilogue.restype = ctypes.c_int
        L.tt_oracle_qkv_epilogue.argtypes = ([_f32p, _f32p] + [ctypes.c_int] * 4 + [_f32p, _f32p, ctypes.c_float, ctypes.c_int,
                                              ctypes.c_float, ctypes.c_int, _f32p, _f32p, _f32p])
        L.tt_oracle_decode.restype = ctypes.c_int
        L.tt_oracle_decode.argtypes = [_f32p, _f32p, _f32p, _f32p] + [ctypes.c_int] * 4 + [ctypes.c_float, _f32p]
        L.tt_oracle_attention_batch.restype = ctypes.c_int
        L.tt_oracle_attention_batch.argtypes = [_f32p, _f32p, _f32p, _f32p] + [ctypes.c_int] * 6 + [ctypes.c_float, ctypes.c_int, _f32p]
        L.tt_oracle_attention_ref.restype = ctypes.c_int
        L.tt_oracle_attention_ref.argtypes = [_f32p, _f32p, _f32p] + [ctypes.c_int] * 5 + [ctypes.c_float, _f32p]
        L.tt_oracle_prefill_ref.restype = ctypes.c_int
        L.tt_oracle_prefill_ref.argtypes = [_f32p, _f32p, _f32p] + [ctypes.c_int] * 9 + [ctypes.c_float, _f32p]
        _u8p, _ip = ctypes.POINTER(ctypes.c_uint8), ctypes.POINTER(ctypes.c_int)
        L.tt_oracle_kv_row_layout.restype = ctypes.c_int
        L.tt_oracle_kv_row_layout.argtypes = [ctypes.c_int] * 3 + [_ip, _ip]
        L.tt_oracle_kv_quantize_rows.restype = ctypes.c_int
        L.tt_oracle_kv_quantize_rows.argtypes = [_f32p, ctypes.c_size_t] + [ctypes.c_int] * 4 + [_u8p, ctypes.c_size_t]
        L.tt_oracle_kv_dequantize_rows.restype = ctypes.c_int
        L.tt_oracle_kv_dequantize_rows.argtypes = [_u8p, ctypes.c_size_t] + [ctypes.c_int] * 4 + [_f32p]
        _z = ctypes.c_size_t
        L.tt_oracle_bf16_bits.restype = ctypes.c_uint16
        L.tt_oracle_bf16_bits.argtypes = [ctypes.c_float]
        L.tt_oracle_bf16_to_f32.restype = ctypes.c_float
        L.tt_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.tt_oracle_affine_quantize_rows.restype = ctypes.c_int
        L.tt_oracle_affine_quantize_rows.argtypes = [ctypes.c_int, _f32p, _z, _z, _u8p, _u16p, _u16p]
        L.tt_oracle_affine_dequantize_rows.restype = ctypes.c_int
        L.tt_oracle_affine_dequantize_rows.argtypes = [ctypes.c_int, _u8p, _u16p, _u16p, _z, _z, _f32p]
        L.tt_oracle_affine_gemv.restype = ctypes.c_int
        L.tt_oracle_affine_gemv.argtypes = [ctypes.c_int, _u8p, _u16p, _u16p, _f32p, _z, _z, _f32p]
        L.tt_oracle_affine_projection.restype = ctypes.c_int
        L.tt_oracle_affine_projection.argtypes = [ctypes.c_int, _u8p, _u16p, _u16p, _f32p] + [_z] * 5 + [_f32p]
        L.tt_oracle_affine_projection_half_weights.restype = ctypes.c_int
        L.tt_oracle_affine_projection_half_weights.argtypes = L.tt_oracle_affine_projection.argtypes
        _u32p = ctypes.POINTER(ctypes.c_uint32)
        L.tt_oracle_qsa_pool_blocks.restype = ctypes.c_int
        L.tt_oracle_qsa_pool_blocks.argtypes = [_u16p, _u16p] + [ctypes.c_int] * 5
        L.tt_oracle_qsa_block_scores.restype = ctypes.c_int
        L.tt_oracle_qsa_block_scores.argtypes = [_u16p, _u16p, _f32p] + [ctypes.c_int] * 4
        L.tt_oracle_qsa_select_keys.restype = ctypes.c_int
        L.tt_oracle_qsa_select_keys.argtypes = [_f32p] + [ctypes.c_int] * 3 + [_u8p, _u32p, _u32p]
        L.tt_oracle_max_threads.restype = ctypes.c_int
        L.tt_oracle_max_threads.argtypes = []
        _lib = L
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _ptr(a: np.ndarray):
    return a.ctypes.data_as(_f32p)


class OracleError(RuntimeError):
    pass


def _check(status: int, what: str) -> None:
    if status != 0:
        raise OracleError(f"{what}: oracle status {status}")


# --- PRNG -----------------------------------------------------------------

class SplitMix64:
    def __init__(self, seed: int):
        self._state = ctypes.c_uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next(self) -> int:
        return int(lib().tt_oracle_splitmix64_next(ctypes.byref(self._state)))

    def uniform(self, lo: float, hi: float) -> float:
        return float(lib().tt_oracle_splitmix64_uniform(ctypes.byref(self._state), lo, hi))


def seedtree_key(root: int, label: str) -> int:
    return int(lib().tt_oracle_seedtree_key(root & 0xFFFFFFFFFFFFFFFF, label.encode("utf-8")))


def fill_uniform(root: int, label: str, lo: float, hi: float, count: int) -> np.ndarray:
    out = np.empty(count, dtype=np.float32)
    lib().tt_oracle_fill_uniform(root & 0xFFFFFFFFFFFFFFFF, label.encode("utf-8"), lo, hi, _ptr(out), count)
    return out


# --- fp16 -----------------------------------------------------------------

def round_through_f16(values) -> np.ndarray:
    out = _f32(values).copy()
    lib().tt_oracle_round_through_f16(_ptr(out), out.size)
    return out


def f32_to_f16_bits(values) -> np.ndarray:
    src = _f32(values)
    out = np.empty(src.shape, dtype=np.uint16)
    lib().tt_oracle_f32_to_f16_array(_ptr(src), out.ctypes.data_as(_u16p), src.size)
    return out


def f16_bits_to_f32(bits) -> np.ndarray:
    src = np.ascontiguousarray(bits, dtype=np.uint16)
    out = np.empty(src.shape, dtype=np.float32)
    lib().tt_oracle_f16_to_f32_array(src.ctypes.data_as(_u16p), _ptr(out), src.size)
    return out


# --- ops ------------------------------------------------------------------

def sigmoid(x: float) -> float:
    return float(lib().tt_oracle_sigmoid(x))


def softmax(values) -> np.ndarray:
    out = _f32(values).copy()
    lib().tt_oracle_softmax_inplace(_ptr(out), out.size)
    return out


def rope_neox(values, head_dim: int, rotary_dim: int, position: int, theta: float) -> np.ndarray:
    out = _f32(values).copy()
    lib().tt_oracle_rope_neox(_ptr(out), out.size, head_dim, rotary_dim, position, theta)
    return out


def rms_norm_per_slice(values, width: int, gamma, epsilon: float) -> np.ndarray:
    """``CPUOps.rmsNormPerSlice`` (CPUTensorOps.swift:70-84)."""
    out = _f32(values).copy()
    g = _f32(gamma).reshape(-1)
    assert g.size == width and out.size % width == 0
    lib().tt_oracle_rms_norm_per_slice(_ptr(out), out.size, width, _ptr(g), epsilon)
    return out


def qkv_epilogue(packed, k_rows, tokens: int, heads: int, kv_heads: int, dim: int, q_gamma, k_gamma,
                 epsilon: float, rotary_dim: int, theta: float, base_position: int):
    """Split [query ; gate], per-head RMS norm of q and k, NeoX sub-dim RoPE (CPUQwen35.swift:266-300).

    Returns ``(q [tokens][heads*dim], gate likewise, k [tokens][kv_heads*dim])`` in fp32."""
    p = _f32(packed).reshape(-1)
    k = _f32(k_rows).reshape(-1)
    qg, kg = _f32(q_gamma).reshape(-1), _f32(k_gamma).reshape(-1)
    assert p.size == tokens * heads * 2 * dim and k.size == tokens * kv_heads * dim
    assert qg.size == dim and kg.size == dim
    q_out = np.empty(tokens * heads * dim, dtype=np.float32)
    g_out = np.empty_like(q_out)
    k_out = np.empty(tokens * kv_heads * dim, dtype=np.float32)
    _check(lib().tt_oracle_qkv_epilogue(_ptr(p), _ptr(k), tokens, heads, kv_heads, dim, _ptr(qg), _ptr(kg), epsilon,
                                        rotary_dim, theta, base_position, _ptr(q_out), _ptr(g_out), _ptr(k_out)),
           "qkv_epilogue")
    return (q_out.reshape(tokens, heads * dim), g_out.reshape(tokens, heads * dim),
            k_out.reshape(tokens, kv_heads * dim))


KV_GROUP_SIZE = 64  # KVCacheManager.quantizationGroupSize


def kv_row_layout(elements: int, bits: int, group_size: int = KV_GROUP_SIZE):
    """``KVCacheManager.rowLayout`` (KVCacheManager+Validation.swift:30-41): (stride, value_bytes) in bytes."""
    stride, value_bytes = ctypes.c_int(), ctypes.c_int()
    _check(lib().tt_oracle_kv_row_layout(elements, bits, group_size, ctypes.byref(stride), ctypes.byref(value_bytes)),
           "kv_row_layout")
    return stride.value, value_bytes.value


def kv_quantize_rows(rows, bits: int, group_size: int = KV_GROUP_SIZE) -> np.ndarray:
    """``kv_cache_quantize_affine`` (kv_cache_quantize.metal:7-73): [tokens][elements] fp16-representable
    values -> uint8 rows [tokens][stride] (packed levels, fp16 scales, fp16 biases; padding bytes zero)."""
    src = _f32(rows)
    tokens, elements = src.shape
    stride, _ = kv_row_layout(elements, bits, group_size)
    out = np.zeros((tokens, stride), dtype=np.uint8)
    _check(lib().tt_oracle_kv_quantize_rows(_ptr(src), elements, tokens, elements, bits, group_size,
                                            out.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), stride), "kv_quantize_rows")
    return out


def kv_dequantize_rows(rows: np.ndarray, elements: int, bits: int, group_size: int = KV_GROUP_SIZE) -> np.ndarray:
    """``attn_load_kv`` (attention.metal:89-117) over whole rows: uint8 [tokens][stride] -> fp32 [tokens][elements]."""
    r = np.ascontiguousarray(rows, dtype=np.uint8)
    tokens, stride = r.shape
    out = np.empty((tokens, elements), dtype=np.float32)
    _check(lib().tt_oracle_kv_dequantize_rows(r.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8)), stride, tokens, elements,
                                              bits, group_size, _ptr(out)), "kv_dequantize_rows")
    return out


def decode(query, keys, values, heads: int, kv_heads: int, dim: int, scale: float, gate=None) -> np.ndarray:
    """``CPUQwen35.attention`` inner block.  keys/values ``[cached][kv_heads*dim]``."""
    q = _f32(query).reshape(-1)
    k = _f32(keys).reshape(-1)
    v = _f32(values).reshape(-1)
    cached = k.size // (kv_heads * dim)
    assert q.size == heads * dim and v.size == k.size
    g = _f32(gate).reshape(-1) if gate is not None else None
    out = np.empty(heads * dim, dtype=np.float32)
    _check(lib().tt_oracle_decode(_ptr(q), _ptr(g) if g is not None else None, _ptr(k), _ptr(v),
                                  cached, heads, kv_heads, dim, scale, _ptr(out)), "decode")
    return out.reshape(heads, dim)


def attention_batch(query, keys, values, tokens: int, base_position: int, heads: int, kv_heads: int,
                    dim: int, scale: float, gate=None, threads: int = 1) -> np.ndarray:
    """``CPUQwen35.attentionBatch`` attention part.  keys/values already hold the chunk's rows."""
    q = _f32(query).reshape(-1)
    k = _f32(keys).reshape(-1)
    v = _f32(values).reshape(-1)
    positions = k.size // (kv_heads * dim)
    assert q.size == tokens * heads * dim and v.size == k.size
    g = _f32(gate).reshape(-1) if gate is not None else None
    out = np.empty(tokens * heads * dim, dtype=np.float32)
    _check(lib().tt_oracle_attention_batch(_ptr(q), _ptr(g) if g is not None else None, _ptr(k), _ptr(v),
                                           tokens, positions, base_position, heads, kv_heads, dim, scale,
                                           threads, _ptr(out)), "attention_batch")
    return out.reshape(tokens, heads, dim)


def attention_ref(q, k, v, head_dim: int, num_q_heads: int, num_kv_heads: int, seq_len: int,
                  window: int = 0, scale: float = -1.0) -> np.ndarray:
    """``AttentionRef.apply``.  k/v ``[seq][kv_heads][dim]``; ``scale < 0`` means 1/sqrt(dim)."""
    qa, ka, va = _f32(q).reshape(-1), _f32(k).reshape(-1), _f32(v).reshape(-1)
    assert qa.size == num_q_heads * head_dim
    assert ka.size == seq_len * num_kv_heads * head_dim and va.size == ka.size
    out = np.empty(num_q_heads * head_dim, dtype=np.float32)
    _check(lib().tt_oracle_attention_ref(_ptr(qa), _ptr(ka), _ptr(va), head_dim, num_q_heads, num_kv_heads,
                                         seq_len, window, scale, _ptr(out)), "attention_ref")
    return out.reshape(num_q_heads, head_dim)


def prefill_ref(q, k, v, q_stride: int, kv_stride: int, head_dim: int, q_heads: int, kv_heads: int,
                start: int, chunk: int, kv_valid: int, window: int, scale: float) -> np.ndarray:
    """``PrefillAttentionRef.apply`` with explicit (possibly padded) strides."""
    qa, ka, va = _f32(q).reshape(-1), _f32(k).reshape(-1), _f32(v).reshape(-1)
    out = np.empty(chunk * q_heads * head_dim, dtype=np.float32)
    _check(lib().tt_oracle_prefill_ref(_ptr(qa), _ptr(ka), _ptr(va), q_stride, kv_stride, head_dim, q_heads,
                                       kv_heads, start, chunk, kv_valid, window, scale, _ptr(out)),
           "prefill_ref")
    return out.reshape(chunk, q_heads, head_dim)


# --- affine-quantised projection (o_proj) -----------------------------------

AFFINE_GROUP_SIZE = 64  # Quantization.groupSize


def _u8(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_uint8))


def _u16(a):
    return a.ctypes.data_as(_u16p)


def bf16_bits(value: float) -> int:
    return int(lib().tt_oracle_bf16_bits(float(value)))


def bf16_to_f32(bits: int) -> float:
    return float(lib().tt_oracle_bf16_to_f32(int(bits)))


def affine_quantize_rows(weights, bits: int):
    """``Quantization.quantizeInt4Affine`` / ``quantizeInt8Affine`` (Quantization.swift:60-113, :158-199) over the
    rows of a [rows][n] matrix -> (packed uint8 [rows][n*bits/8], scales uint16 [rows][n/64], biases likewise)."""
    w = _f32(weights)
    rows, n = w.shape
    packed = np.zeros((rows, n * bits // 8), dtype=np.uint8)
    scales = np.zeros((rows, n // AFFINE_GROUP_SIZE), dtype=np.uint16)
    biases = np.zeros_like(scales)
    _check(lib().tt_oracle_affine_quantize_rows(bits, _ptr(w), rows, n, _u8(packed), _u16(scales), _u16(biases)),
           "affine_quantize_rows")
    return packed, scales, biases


def affine_dequantize_rows(packed, scales, biases, bits: int) -> np.ndarray:
    """``Quantization.dequantizeInt4Affine`` / ``dequantizeInt8Affine`` (:119-136, :205-220) -> fp32 [rows][n]."""
    packed, scales, biases = (np.ascontiguousarray(a) for a in (packed, scales, biases))
    rows, n = packed.shape[0], packed.shape[1] * 8 // bits
    out = np.empty((rows, n), dtype=np.float32)
    _check(lib().tt_oracle_affine_dequantize_rows(bits, _u8(packed), _u16(scales), _u16(biases), rows, n, _ptr(out)),
           "affine_dequantize_rows")
    return out


def affine_gemv(packed, scales, biases, x, bits: int) -> np.ndarray:
    """``tinytitan_int4_affine_gemv`` / ``tinytitan_int8_affine_gemv`` (TinyTitanKernelsC, portable branch): fp32 in,
    fp32 out, one vector."""
    packed, scales, biases = (np.ascontiguousarray(a) for a in (packed, scales, biases))
    vec = _f32(x)
    rows, n = packed.shape[0], packed.shape[1] * 8 // bits
    assert vec.shape == (n,), (vec.shape, n)
    out = np.empty(rows, dtype=np.float32)
    _check(lib().tt_oracle_affine_gemv(bits, _u8(packed), _u16(scales), _u16(biases), _ptr(vec), rows, n, _ptr(out)),
           "affine_gemv")
    return out


def affine_projection(packed, scales, biases, x, bits: int, half_weights: bool = False) -> np.ndarray:
    """``encodeAffineProjection`` for o_proj (RealForwardRunner+PrefillProjection.swift:53-66): x [tokens][n]
    fp16-representable values -> y [tokens][rows], rounded to fp16 and returned as fp32.  ``half_weights``: the
    tensor-operation path for chunks, whose weight tile is rounded to half (tensorops.metal:80-125)."""
    packed, scales, biases = (np.ascontiguousarray(a) for a in (packed, scales, biases))
    act = _f32(x)
    rows, n = packed.shape[0], packed.shape[1] * 8 // bits
    tokens = act.shape[0]
    assert act.shape == (tokens, n), (act.shape, n)
    out = np.empty((tokens, rows), dtype=np.float32)
    fn = lib().tt_oracle_affine_projection_half_weights if half_weights else lib().tt_oracle_affine_projection
    _check(fn(bits, _u8(packed), _u16(scales), _u16(biases), _ptr(act), rows, n, tokens, n, rows, _ptr(out)),
           "affine_projection")
    return out


_REF_AFFINE_PATH = os.path.join(_HERE, "_ref", "libtt_ref_affine.so")


def reference_affine_gemv(packed, scales, biases, x, bits: int):
    """The reference's own C kernel (``tinytitan_int4_affine_gemv`` / ``tinytitan_int8_affine_gemv``) as compiled
    from the reference checkout into ``oracle/_ref``; ``None`` where that build is absent."""
    if not os.path.exists(_REF_AFFINE_PATH):
        return None
    ref = ctypes.CDLL(_REF_AFFINE_PATH)
    fn = ref.tinytitan_int4_affine_gemv if bits == 4 else ref.tinytitan_int8_affine_gemv
    fn.restype = None
    fn.argtypes = [ctypes.POINTER(ctypes.c_uint8), _u16p, _u16p, _f32p, ctypes.c_size_t, ctypes.c_size_t, _f32p]
    packed, scales, biases = (np.ascontiguousarray(a) for a in (packed, scales, biases))
    vec = _f32(x)
    rows, n = packed.shape[0], packed.shape[1] * 8 // bits
    out = np.full(rows, np.nan, dtype=np.float32)
    fn(_u8(packed), _u16(scales), _u16(biases), _ptr(vec), rows, n, _ptr(out))
    return out


def qsa_pool_blocks(raw_bits, pooled_bits, dim: int, first_block: int, block_count: int, ratio: int, n_kv: int) -> None:
    """``qsa_pool_blocks`` (qsa.metal:44-66) on fp16 bit patterns; ``pooled_bits`` ([blocks][dim] uint16) is updated in place."""
    raw = np.ascontiguousarray(raw_bits, dtype=np.uint16)
    assert pooled_bits.dtype == np.uint16 and pooled_bits.flags.c_contiguous
    assert raw.size >= n_kv * dim and pooled_bits.size >= (first_block + block_count) * dim
    _check(lib().tt_oracle_qsa_pool_blocks(_u16(raw), _u16(pooled_bits), dim, first_block, block_count, ratio, n_kv),
           "qsa_pool_blocks")


def qsa_norm_rope_rows(rows_bits, heads: int, dim: int, gamma, epsilon: float, theta: float, position: int,
                       position_stride: int) -> np.ndarray:
    """The indexer's norm and rotation of fp16 rows ``[tokens][heads][dim]``: per-head RMS norm, a rounding to
    fp16, NeoX rotation over the whole head at ``position + token * position_stride``, a rounding to fp16
    (QSAIndexer.swift:213-232 for pooled blocks: heads 1, stride = the ratio; :343-357 for query rows: stride 1)."""
    bits = np.ascontiguousarray(rows_bits, dtype=np.uint16).reshape(-1, heads * dim)
    out = np.empty_like(bits)
    for t in range(bits.shape[0]):
        x = f16_bits_to_f32(bits[t])
        x = round_through_f16(rms_norm_per_slice(x, dim, gamma, epsilon))
        x = rope_neox(x, dim, dim, position + t * position_stride, theta)
        out[t] = f32_to_f16_bits(x)
    return out


def qsa_block_scores(query_bits, pooled_bits, dim: int, heads: int, blocks: int, tokens: int) -> np.ndarray:
    """``qsa_block_scores_rows`` (qsa.metal:106-130): fp32 ``[tokens][blocks]``."""
    q = np.ascontiguousarray(query_bits, dtype=np.uint16)
    p = np.ascontiguousarray(pooled_bits, dtype=np.uint16)
    assert q.size == tokens * heads * dim and p.size >= blocks * dim
    out = np.empty((tokens, blocks), dtype=np.float32)
    _check(lib().tt_oracle_qsa_block_scores(_u16(q), _u16(p), _ptr(out), dim, heads, blocks, tokens), "qsa_block_scores")
    return out


def qsa_select_keys(scores, visible: int, ratio: int, width: int):
    """``QSAIndexer.selectKeys`` (QSAIndexer+Scratch.swift:228-262) with the compacted list of
    ``selectKeysPrefill`` (QSAIndexer.swift:484-492).  Returns ``(selected, keep [visible] uint8, indices)``;
    ``selected`` is False inside the dense window, where everything visible is kept."""
    s = _f32(scores).reshape(-1) if scores is not None else np.zeros(1, dtype=np.float32)
    keep = np.zeros(max(visible, 1), dtype=np.uint8)
    indices = np.zeros(max(width, visible, 1), dtype=np.uint32)
    count = ctypes.c_uint32(0)
    st = lib().tt_oracle_qsa_select_keys(_ptr(s), visible, ratio, width, _u8(keep),
                                         indices.ctypes.data_as(ctypes.POINTER(ctypes.c_uint32)), ctypes.byref(count))
    if st < 0:
        raise ValueError("qsa_select_keys: bad arguments")
    return bool(st), keep[:visible], indices[:count.value].copy()


def max_threads() -> int:
    return int(lib().tt_oracle_max_threads())
