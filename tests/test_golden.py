"""Golden fixtures: the oracle must still reproduce them bit for bit (CPU), and the GPU path must
match them to the parity bar (GPU) -- so a drifting oracle and a drifting kernel are told apart."""
import json
import os

import numpy as np
import pytest

from tests.helpers import assert_parity, gpu_workload, oracle_workload
from tinytitan_amd import synthetic

HERE = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
INDEX = json.load(open(os.path.join(HERE, "index.json")))


def _load(name):
    entry = INDEX[name]
    w = getattr(synthetic, entry["builder"])(**entry["kwargs"])
    data = np.load(os.path.join(HERE, name + ".npz"))
    outs = [data[f"out{i}"].view(np.float16).astype(np.float32) for i in range(entry["sequences"])]
    return w, outs


@pytest.mark.parametrize("name", sorted(INDEX))
def test_oracle_reproduces_golden(name):
    w, golden = _load(name)
    for got, want in zip(oracle_workload(w), golden):
        # fp16-rounded outputs; one ulp of slack for libm differences between build hosts
        assert got.shape == want.shape
        assert np.abs(got - want).max() <= 2.0 ** -10 * max(1.0, np.abs(want).max())
        assert (got != want).mean() < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(INDEX))
def test_gpu_matches_golden(gpu_ctx, name):
    w, golden = _load(name)
    assert_parity(gpu_workload(gpu_ctx, w), golden, name)


# ---- pre-attention epilogue ---------------------------------------------------------------

EPILOGUE_INDEX = json.load(open(os.path.join(HERE, "epilogue_index.json")))


def _epilogue_golden(name):
    data = np.load(os.path.join(HERE, name + ".npz"))
    return {key: data[key].view(np.float16).astype(np.float32) for key in ("q", "gate", "k")}


@pytest.mark.parametrize("name", sorted(EPILOGUE_INDEX))
def test_oracle_reproduces_epilogue_golden(name):
    from tests.golden.make_golden import epilogue_outputs
    case, golden = EPILOGUE_INDEX[name], _epilogue_golden(name)
    q, g, k = epilogue_outputs(case)
    for got, want in ((q, golden["q"]), (g, golden["gate"]), (k, golden["k"])):
        got = got.astype(np.float16).astype(np.float32)
        # one fp16 ulp of slack for libm (powf / cosf / sinf) differences between build hosts
        assert np.abs(got - want).max() <= 2.0 ** -10 * max(1.0, np.abs(want).max())
        assert (got != want).mean() < 1e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(EPILOGUE_INDEX))
def test_gpu_matches_epilogue_golden(gpu_ctx, name):
    import torch
    from tests.golden.make_golden import EPILOGUE_EPS, EPILOGUE_THETA
    from tinytitan_amd.engine import KVCacheManager, QKVEpilogue
    case, golden = EPILOGUE_INDEX[name], _epilogue_golden(name)
    T, H, KH, D = case["tokens"], case["heads"], case["kv_heads"], case["dim"]
    x = synthetic.epilogue_inputs(T, H, KH, D)
    cap = case["position"] + T
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=cap, initial_capacity=cap)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    q = torch.empty((T, H * D), dtype=torch.float16, device="cuda")
    g = torch.empty_like(q)
    args = (dev(x["packed"]), dev(x["k"]), dev(x["v"]), dev(x["q_weight_bits"].view(np.int16)),
            dev(x["k_weight_bits"].view(np.int16)))
    torch.cuda.synchronize()
    QKVEpilogue(gpu_ctx).encode(kv, 0, *args, q, g, H, case["position"], T, EPILOGUE_EPS, case["rotary_dim"], EPILOGUE_THETA)
    gpu_ctx.synchronize()
    kr, vr = kv.read(0, 0, case["position"], T)
    for got, want in ((q.float().cpu().numpy(), golden["q"]), (kr.float().cpu().numpy().reshape(T, -1), golden["k"])):
        # the golden values are fp16-rounded: the kernel may land on the neighbouring half
        assert np.abs(got - want).max() <= 2.0 ** -10 * max(1.0, np.abs(want).max())
        assert (got != want).mean() < 2e-2
    assert np.array_equal(g.float().cpu().numpy(), golden["gate"])
    assert np.array_equal(vr.cpu().numpy().reshape(T, -1), x["v"])
    kv.close()


# ---- quantised KV rows (byte work: bit-exact) ---------------------------------------------

QUANT_INDEX = json.load(open(os.path.join(HERE, "kvq_index.json")))


@pytest.mark.parametrize("name", sorted(QUANT_INDEX))
def test_oracle_reproduces_quantised_rows_golden(name):
    from tests.golden.make_golden import quant_outputs
    golden = np.load(os.path.join(HERE, name + ".npz"))["rows"]
    assert np.array_equal(quant_outputs(QUANT_INDEX[name]), golden)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(QUANT_INDEX))
def test_gpu_matches_quantised_rows_golden(gpu_ctx, name):
    import torch
    from tests.golden.make_golden import quant_inputs
    from tinytitan_amd.engine import KVCacheManager
    case = QUANT_INDEX[name]
    golden = np.load(os.path.join(HERE, name + ".npz"))["rows"]
    T, KH, D = case["tokens"], case["kv_heads"], case["dim"]
    rows = torch.from_numpy(quant_inputs(case)).cuda()
    kv = KVCacheManager(gpu_ctx, 1, KH, D, slots=1, max_context=64, initial_capacity=64, precision_bits=case["bits"])
    torch.cuda.synchronize()
    kv.append(0, 0, 5, rows, rows)  # K and V both from the same rows: both layouts must give the golden bytes back
    gpu_ctx.synchronize()
    got_k, got_v = kv.export_rows(0, 0, 5, T)
    assert np.array_equal(got_k.cpu().numpy(), golden) and np.array_equal(got_v.cpu().numpy(), golden)
    kv.close()


# ---- o_proj: outputs of the reference's own C kernels ----------------------------------------

OPROJ_INDEX = json.load(open(os.path.join(HERE, "oproj_index.json")))


@pytest.mark.parametrize("name", sorted(OPROJ_INDEX))
def test_oracle_reproduces_the_reference_kernels_outputs(name):
    # the stored vectors were written by tinytitan_int4_affine_gemv / tinytitan_int8_affine_gemv (oracle/_ref);
    # the oracle's restatement gives the same fp32 bits without that build
    import oracle
    from tests.golden.make_golden import oproj_inputs
    case = OPROJ_INDEX[name]
    golden = np.load(os.path.join(HERE, name + ".npz"))["y"]
    packed, scales, biases, x = oproj_inputs(case)
    got = np.stack([oracle.affine_gemv(packed, scales, biases, row.astype(np.float32), case["bits"]) for row in x])
    assert np.array_equal(got, golden)


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(OPROJ_INDEX))
def test_gpu_matches_the_reference_kernels_outputs(gpu_ctx, name):
    import torch
    from tests.golden.make_golden import oproj_inputs
    from tinytitan_amd.engine import AffineProjection
    case = OPROJ_INDEX[name]
    golden = np.load(os.path.join(HERE, name + ".npz"))["y"].astype(np.float16).astype(np.float32)  # the kernels' one rounding
    packed, scales, biases, x = oproj_inputs(case)
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()
    wd, sd, bd, xd = dev(packed), dev(scales.view(np.int16)), dev(biases.view(np.int16)), dev(x)
    yd = torch.empty((case["tokens"], case["rows"]), dtype=torch.float16, device="cuda")
    torch.cuda.synchronize()
    AffineProjection(gpu_ctx).encode(case["bits"], wd, sd, bd, xd, yd, case["rows"], case["columns"], case["tokens"])
    gpu_ctx.synchronize()
    got = yd.float().cpu().numpy()
    assert (np.abs(got - golden) <= 2.0 ** -10 * np.abs(golden) + 1e-4).all()  # one fp16 ulp; fp32 summation order near zero
    assert (got == golden).mean() >= 0.97


# --- the sparse attention's indexer -------------------------------------------------------------

QSA_INDEX = json.load(open(os.path.join(HERE, "qsa_index.json")))


def _qsa(name):
    from tests.golden import make_golden
    case = QSA_INDEX[name]
    return case, make_golden.qsa_inputs(case), np.load(os.path.join(HERE, name + ".npz"))


@pytest.mark.parametrize("name", sorted(QSA_INDEX))
def test_oracle_reproduces_golden_indexer(name):
    from tests.golden import make_golden
    case, _, golden = _qsa(name)
    pooled, scores, keep, indices = make_golden.qsa_outputs(case)
    assert np.array_equal(pooled, golden["pooled"]) and np.array_equal(scores, golden["scores"])
    assert np.array_equal(keep, golden["keep"]) and np.array_equal(indices, golden["indices"])
    width = case["budget"] + case["ratio"] - 1
    assert keep.sum() == width == len(indices), "the fixtures lie past the dense window"
    assert len(np.unique(golden["scores"])) < golden["scores"].size, "the fixtures hold tied scores"


@pytest.mark.gpu
@pytest.mark.parametrize("name", sorted(QSA_INDEX))
def test_gpu_matches_golden_indexer(gpu_ctx, name):
    import torch
    case, (raw, q), golden = _qsa(name)
    cells, ratio, dim, heads = case["cells"], case["ratio"], case["dim"], case["heads"]
    blocks, width = (cells - 1) // ratio + 1, case["budget"] + case["ratio"] - 1
    L, h = gpu_ctx._lib, gpu_ctx.handle
    rd, qd = torch.from_numpy(raw).cuda(), torch.from_numpy(q).cuda()
    pooled = torch.zeros((blocks, dim), dtype=torch.float16, device="cuda")
    scores = torch.zeros((1, blocks), dtype=torch.float32, device="cuda")
    stride = (cells + 3) // 4 * 4
    keep = torch.zeros(stride, dtype=torch.uint8, device="cuda")
    idx = torch.zeros(width, dtype=torch.int32, device="cuda")
    cnt = torch.zeros(1, dtype=torch.int32, device="cuda")
    torch.cuda.synchronize()
    gpu_ctx._check(L.tt_hip_qsa_pool_blocks(h, rd.data_ptr(), pooled.data_ptr(), dim, 0, blocks, ratio, cells, None, 0.0, 0.0), "pool")
    gpu_ctx._check(L.tt_hip_qsa_block_scores(h, qd.data_ptr(), pooled.data_ptr(), scores.data_ptr(), blocks, dim, heads, blocks, 1), "scores")
    gpu_ctx.synchronize()
    assert np.array_equal(pooled.cpu().numpy().view(np.uint16), golden["pooled"])
    assert np.abs(scores.cpu().numpy() - golden["scores"]).max() <= 1e-3
    # the selection on the fixture's scores, so that a last-bit difference of a score cannot move a tie
    gs = torch.from_numpy(golden["scores"]).cuda()
    torch.cuda.synchronize()
    gpu_ctx._check(L.tt_hip_qsa_select(h, gs.data_ptr(), blocks, 1, cells, ratio, width, keep.data_ptr(), stride, idx.data_ptr(),
                                       width, cnt.data_ptr()), "select")
    gpu_ctx.synchronize()
    assert np.array_equal(keep[:cells].cpu().numpy(), golden["keep"]) and int(cnt[0]) == len(golden["indices"])
    assert np.array_equal(idx.cpu().numpy().astype(np.uint32), golden["indices"])
