"""tt_hip_attn_prefill at the edges of its routes.

The entry point serves a chunk by one of several kernels, chosen from the chunk's rows, the keys before it, the
cache's precision and the head shape (the chunk kernel whole or over key ranges, the split-K kernel with one-head or
GQA-packed tiles).  Same semantics and the same bar (max-abs 2e-3, mean-abs 2e-4 against the CPU oracle) whichever
serves: the cases sit on both sides of every threshold -- 31 / 32, 63 / 64 rows, 2559 / 2560, 4095 / 4096,
32767 / 32768 keys, 786,432 / rows keys (where the key ranges take over from the split-K tiles), and the keys up to
which the split-K tiles are 16 rows high -- over fp16 and over 8-bit pages, for head groups the chunk kernel takes and
one it does not."""
import numpy as np
import pytest

import oracle
from tests.test_gpu_attention_api import _check, _dev, _prefill

pytestmark = pytest.mark.gpu


def _chunk(gpu_ctx, bits, H, KH, D, rows, kv_valid):
    from tinytitan_amd.engine import KVCacheManager
    import torch
    start = kv_valid - rows
    r = np.random.default_rng(rows * 1000003 + kv_valid * 7 + bits)
    k = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    v = r.standard_normal((kv_valid, KH, D)).astype(np.float16)
    q = r.standard_normal((rows, H * D)).astype(np.float16)
    g = r.standard_normal((rows, H * D)).astype(np.float16)
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=kv_valid, initial_capacity=kv_valid, precision_bits=bits)
    kd, vd = _dev(k), _dev(v)
    torch.cuda.synchronize()
    kv.append(0, 0, 0, kd, vd)
    gpu_ctx.synchronize()
    if bits == 16:
        k32, v32 = k.astype(np.float32), v.astype(np.float32)
    else:  # what the oracle's loader reads back from the oracle's quantiser
        k32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(k.reshape(kv_valid, -1).astype(np.float32), bits), KH * D, bits)
        v32 = oracle.kv_dequantize_rows(oracle.kv_quantize_rows(v.reshape(kv_valid, -1).astype(np.float32), bits), KH * D, bits)
    scale = float(D) ** -0.5
    got = _prefill(gpu_ctx, kv, q, start, rows, kv_valid, H, scale, gate=g)
    want = oracle.attention_batch(q.astype(np.float32), k32.reshape(kv_valid, -1), v32.reshape(kv_valid, -1), rows, start, H, KH, D,
                                  scale, threads=4)
    want = want.reshape(rows, -1) / (1 + np.exp(-g.astype(np.float64)))
    _check(got, want, f"{rows} rows behind {start} keys, {H}q/{KH}kv/{D}, {bits} bits")
    kv.close()


@pytest.mark.parametrize("bits", [16, 8])
@pytest.mark.parametrize("rows,kv_valid", [(8, 2560), (9, 2559), (9, 2560), (31, 32768), (32, 32767), (32, 32768), (63, 4096),
                                           (64, 4095), (64, 4096), (65, 8200), (130, 2047), (130, 2049), (257, 300),
                                           (1030, 1030), (520, 1600), (64, 12287), (64, 12288), (128, 6143), (128, 6144),
                                           (200, 4095), (200, 4096), (310, 2559), (310, 2560), (32, 20480), (32, 20481),
                                           (48, 16384), (96, 1700), (96, 1720)])
def test_rows_and_keys_on_both_sides_of_every_threshold(gpu_ctx, bits, rows, kv_valid):
    _chunk(gpu_ctx, bits, 8, 2, 128, rows, kv_valid)


@pytest.mark.parametrize("bits", [16, 8])
@pytest.mark.parametrize("H,KH,D,rows,kv_valid", [(6, 2, 128, 5, 9000), (6, 2, 128, 300, 5000), (6, 2, 64, 1100, 1100),
                                                   (4, 4, 128, 40, 20000), (16, 2, 256, 3, 33000)])
def test_head_groups_the_chunk_kernel_does_not_take_and_few_rows(gpu_ctx, bits, H, KH, D, rows, kv_valid):
    _chunk(gpu_ctx, bits, H, KH, D, rows, kv_valid)
