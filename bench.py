#!/usr/bin/env python3
"""Benchmark of the KV-cache attention path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload C2] [--all]

A step is one pass of the hot path over one batch of synthetic input: for the
default workload C2, one GQA decode attention (16 q heads / 2 KV heads, dim 256,
gated) over a 32768-token fp16 KV cache that is already resident in HBM.  Steps
rotate over `--layers` separate layer caches of the same shape (as a model's
decode step does), so that every step reads its 64 MiB from HBM rather than
from the 256 MiB last-level cache.

Prints ONE JSON line: KV GB/s for the workload, the roofline of the dominant
kernel (its own HIP-event duration, measured live) and the CPU oracle timed on
this host beside it.  With --all the other four configurations are measured
too and reported under "workloads".
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_FP16_PEAK_TFLOPS = 2500.0  # MI355X dense fp16
# o_proj behind the gate, tokens per step: a decode row, the 8 x 4 rows of a C5 verify pass, the C4 chunk
PROJECTION_TOKENS = {"O1": 1, "O5": 32, "O4": 4096}
PROJECTION_DEFAULT_TOKENS = dict(PROJECTION_TOKENS)
# The sparse attention's block indexer at the reference's production geometry (4 heads of 128, blocks of 4 keys,
# budget 2048): (keys already cached, tokens of the step).  Q2: a decode step at C2's context; Q6: at the
# reference's largest context; Q4: the 4096-token chunk of C4; Q3: a 4096-token chunk behind 28,672 cached keys.
INDEXER_SHAPES = {"Q2": (32767, 1), "Q6": (262143, 1), "Q4": (0, 4096), "Q3": (28672, 4096)}
INDEXER_HEADS, INDEXER_DIM, INDEXER_RATIO, INDEXER_BUDGET = 4, 128, 4, 2048
INDEXER_SEPARATE_LAUNCHES = False  # --indexer-separate-launches
INDEXER_LISTS_ONLY = False         # --indexer-lists-only


def indexer_bytes(context: int, tokens: int) -> int:
    """Algorithmic bytes of one indexer step: pooled blocks and query rows read, scores written and read once, per
    row the mask written (its visible keys; none with --indexer-lists-only) and the index list (at most the selection
    width)."""
    total = context + tokens
    blocks = (total - 1) // INDEXER_RATIO + 1
    width = INDEXER_BUDGET + INDEXER_RATIO - 1
    visible = 0 if INDEXER_LISTS_ONLY else sum(context + r + 1 for r in range(tokens))
    return (blocks * INDEXER_DIM * 2 + tokens * INDEXER_HEADS * INDEXER_DIM * 2 + 2 * tokens * blocks * 4 + visible
            + tokens * min(width, total) * 4)

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# (two runs), each scaled by what the same counter reads for a plain 64 MiB -> 64 MiB copy
# (profiles/attn_splitk_c2_traffic.md, attn_prefill_c4_counters.md, qkv_epilogue_e4.md,
# attn_splitk_c1_c3_c5_trace_and_traffic.md, attn_splitk_kv8_quantised.md, affine_proj_o1_o5_o4.md; "C2/8" is C2
# over an 8-bit cache).  None: not measured
# for that workload.
MEASURED_TRAFFIC_BYTES = {"C1": 4477212, "C2": 69383103, "C3": 598966317, "C4": 113935667, "C5": 1114007952,
                          "E4": 151546501, "C2/8": 37988966, "O1": 4868151, "O5": 7137478, "O4": 96536529}


def _load_engine():
    from tinytitan_amd import capi
    if not os.path.exists(capi.LIB_PATH):
        from tinytitan_amd import build
        build.build()
    from tinytitan_amd import engine
    return engine


class DeviceWorkload:
    """A workload resident in HBM: KV caches filled through the ABI, q/gate/out on device."""

    def __init__(self, eng, ctx, name, layers, seeded, data_scale=1.0, kv_bits=16, window=0, weight_bits=4, keep_fraction=0.0,
                 keep_budget=0, keep_rows="shared", keep_form="mask"):
        import numpy as np
        import torch
        from tinytitan_amd import synthetic
        self.eng, self.ctx, self.name, self.layers = eng, ctx, name, layers
        dev = torch.device("cuda", ctx.device)
        self.dev = dev
        H, KH, D = (8, 2, 256) if name == "C1" else (16, 2, 256)
        self.H, self.KH, self.D, self.scale = H, KH, D, 1.0 / 16.0
        self.host = None  # numpy Workload when the inputs are the seeded ones
        gen = torch.Generator(device=dev)
        gen.manual_seed(synthetic.SEEDS.get(name, 0xE4))

        def randn(*shape):
            return (torch.randn(*shape, generator=gen, device=dev, dtype=torch.float32) * data_scale).to(torch.float16)

        self.bits = kv_bits
        self.window = window
        self.keep = None  # sparse key selection of the decode workloads: one byte per key position
        self.sparse_step = False  # S2 / S6: a step is the indexer's step, the selection and the decode over it
        if name in INDEXER_SHAPES:
            # One layer's indexer caches filled to `context` keys; a step appends `tokens` raw keys' worth of pooled
            # blocks, norms and rotates the query rows, scores every block and selects (mask and index list).
            self.kind = "indexer"
            self.context, self.rows = INDEXER_SHAPES[name]
            self.lengths, self.starts = [self.context + self.rows], [self.context]
            total = self.context + self.rows
            self.indexer = eng.QSAIndexer(ctx, INDEXER_HEADS, INDEXER_DIM, INDEXER_RATIO, INDEXER_BUDGET, 1e7, capacity=total)
            self.indexer.raw_key_destination(0, 0, total).copy_(randn(total, INDEXER_DIM))
            self.norm = (1.0 + 0.1 * torch.randn(INDEXER_DIM, generator=gen, device=dev)).to(torch.bfloat16)
            torch.cuda.synchronize(dev)
            if self.context:
                self.indexer.encode_pool_prefill(0, 0, self.context, self.norm, 1e-6)
            self.q = randn(self.rows, INDEXER_HEADS, INDEXER_DIM)
            self.kv = None
            blocks = (total - 1) // INDEXER_RATIO + 1
            self.kv_bytes = indexer_bytes(self.context, self.rows)
            self.flops = 2 * self.rows * INDEXER_HEADS * blocks * INDEXER_DIM
            ctx.synchronize()
            torch.cuda.synchronize(dev)
            return
        if name in PROJECTION_TOKENS:
            # o_proj behind the gate at the model's shape: hidden 2048 x (16 heads * 256), affine levels with a
            # bf16 scale and bias per group of 64 columns; one weight set per rotated layer
            self.kind, self.rows = "projection", PROJECTION_TOKENS[name]
            self.lengths, self.starts = [self.rows], [0]
            self.weight_bits = weight_bits
            m, n = 2048, H * D
            self.m, self.n = m, n
            self.weights = torch.randint(0, 256, (layers, m, n * weight_bits // 8), generator=gen, device=dev, dtype=torch.uint8)
            top = float((1 << weight_bits) - 1)
            span = 0.02 + 0.08 * torch.rand(layers, m, n // 64, generator=gen, device=dev)
            self.w_scales = (span / top).to(torch.bfloat16)
            self.w_biases = (-0.5 * span).to(torch.bfloat16)
            self.q = randn(self.rows, n)
            self.out = torch.zeros(self.rows, m, dtype=torch.float16, device=dev)
            self.projection = eng.AffineProjection(ctx)
            self.kv = None
            # the matrix as stored: levels + scales + biases (x and y are 1/500 of it at one token)
            self.kv_bytes = m * n * weight_bits // 8 + 2 * m * (n // 64) * 2
            self.flops = 2 * self.rows * m * n
            torch.cuda.synchronize(dev)
            return
        if name in ("C1", "C2", "S2", "S6"):
            self.kind, self.rows = "decode", 1
            ctxlen = {"C1": 2048, "C2": 32768, "S2": 32768, "S6": 262144}[name]
            self.lengths, self.starts = [ctxlen], [ctxlen - 1]
            gated = name != "C1"
        elif name == "C3":
            self.kind, self.rows = "decode", 1
            self.lengths = synthetic.c3_lengths()
            self.starts = [n - 1 for n in self.lengths]
            gated = False
        elif name == "C4":
            self.kind, self.rows = "prefill", 4096
            self.lengths, self.starts = [4096], [0]
            gated = False
        elif name in ("D1", "D2", "D6", "P2", "P6"):
            # the reference's default prefill chunk (prefillChunkTokens = 128) behind 8k / 32k / 128k cached keys
            self.kind, self.rows = "prefill", 128
            total = {"D1": 8192, "D2": 32768, "D6": 131072, "P2": 32768, "P6": 131072}[name]
            self.lengths, self.starts = [total], [total - 128]
            gated = False
        elif name == "K4":
            # a chunk late in a long context whose rows each keep a sparse selection of the cached keys
            self.kind, self.rows = "prefill_keep", 256
            self.lengths, self.starts = [131072], [131072 - 256]
            gated = False
        elif name == "C5":
            self.kind, self.rows = "verify", 4
            self.lengths, self.starts = [65536 + 4] * 8, [65536] * 8
            gated = True
        elif name == "E4":
            # the stage in front of C4: raw QKV projections of the 4096-token chunk -> q, gate, cached K/V
            self.kind, self.rows = "epilogue", 4096
            self.lengths, self.starts = [4096], [0]
            gated = True
        else:
            raise ValueError(name)
        n = len(self.lengths)
        longest = max(self.lengths)
        self.kv = eng.KVCacheManager(ctx, layers, KH, D, slots=n, max_context=longest, initial_capacity=longest,
                                     precision_bits=self.bits)
        if self.kind == "epilogue":
            T = self.rows
            self.packed = randn(T, H, 2 * D)
            self.k_proj, self.v_proj = randn(T, KH * D), randn(T, KH * D)
            self.q_weight = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
            self.k_weight = (1.0 + 0.1 * torch.randn(D, generator=gen, device=dev)).to(torch.bfloat16)
            self.q = torch.empty(T, H * D, dtype=torch.float16, device=dev)
            self.gate = torch.empty_like(self.q)
            self.out = self.q
            self.epilogue = eng.QKVEpilogue(ctx)
            # per token: 2 H D + 2 KH D halves in, H D + H D + 2 KH D halves out
            self.kv_bytes = T * (2 * H * D + 2 * KH * D) * 2 * 2
            self.flops = 0
            torch.cuda.synchronize(dev)
            return
        if seeded:
            self.host = synthetic.BUILDERS[name]()
        for i, length in enumerate(self.lengths):
            if self.host is not None:
                k = torch.from_numpy(self.host.sequences[i].k).to(dev)
                v = torch.from_numpy(self.host.sequences[i].v).to(dev)
            else:
                k, v = randn(length, KH, D), randn(length, KH, D)
            torch.cuda.synchronize(dev)
            for layer in range(layers):
                self.kv.append(layer, i, 0, k, v)
            ctx.synchronize()
            self.kv.advance(i, length)
            del k, v
        if self.host is not None:
            self.q = torch.from_numpy(np.stack([s.q for s in self.host.sequences])).to(dev)
            self.gate = torch.from_numpy(np.stack([s.gate for s in self.host.sequences])).to(dev) if gated else None
        else:
            self.q = randn(n, self.rows, H, D)
            self.gate = randn(n, self.rows, H, D) if gated else None
        self.out = torch.zeros_like(self.q)
        if keep_fraction > 0.0 and self.kind == "decode" and not window:
            self.keep = (torch.rand(n, longest, generator=gen, device=dev) < keep_fraction).to(torch.uint8)
            for i, length in enumerate(self.lengths):
                self.keep[i, length - 1] = 1  # the query's own position is always kept
        elif keep_budget > 0 and self.kind == "decode" and not window:
            # a selection as the block indexer makes it: random complete blocks of 4 keys up to the budget, and the
            # ragged tail of the query's own block
            self.keep = torch.zeros(n, longest, dtype=torch.uint8, device=dev)
            for i, length in enumerate(self.lengths):
                complete = length // INDEXER_RATIO
                chosen = torch.randperm(complete, generator=gen, device=dev)[:keep_budget // INDEXER_RATIO]
                cells = (chosen[:, None] * INDEXER_RATIO + torch.arange(INDEXER_RATIO, device=dev)[None, :]).flatten()
                self.keep[i, cells] = 1
                self.keep[i, complete * INDEXER_RATIO:length] = 1
                self.keep[i, length - 1] = 1
        if self.kind == "prefill_keep":
            # per query row: `budget` cells in complete blocks of 4 keys -- the same cells for every row ("shared": rows
            # of one chunk select much the same context) or drawn per row ("independent") -- and the row's own block
            budget = keep_budget or INDEXER_BUDGET
            start, total = self.starts[0], self.lengths[0]
            self.keep = torch.zeros(self.rows, total, dtype=torch.uint8, device=dev)
            complete = start // INDEXER_RATIO
            common = torch.randperm(complete, generator=gen, device=dev)[:budget // INDEXER_RATIO]
            offsets = torch.arange(INDEXER_RATIO, device=dev)[None, :]
            for r in range(self.rows):
                chosen = common if keep_rows == "shared" else torch.randperm(complete, generator=gen, device=dev)[:budget // INDEXER_RATIO]
                self.keep[r, (chosen[:, None] * INDEXER_RATIO + offsets).flatten()] = 1
                self.keep[r, (start + r) // INDEXER_RATIO * INDEXER_RATIO:start + r + 1] = 1
        self.keep_form = keep_form
        if self.keep is not None and keep_form == "indices":  # the same selection compacted: ascending key ids per row, and their counts
            counts = self.keep.sum(dim=1, dtype=torch.int32)
            width = max(1, int(counts.max().item()))
            order = torch.argsort(self.keep, dim=1, descending=True, stable=True)[:, :width]
            self.keep_indices = order.to(torch.int32).contiguous()
            self.keep_counts = counts.contiguous()
        if name in ("P2", "P6"):
            # The whole sparse step of the default chunk: the block indexer's chunk step (its caches filled to the chunk's
            # start, the chunk's raw keys already in them) -- pooling, query rows, block scores, per-row selection as
            # index lists alone -- and the chunk attention over those lists.  sparse_step = False runs the dense chunk
            # (workload D2 / D6) on the same cache.
            self.sparse_step = True
            total, start = self.lengths[0], self.starts[0]
            self.indexer = eng.QSAIndexer(ctx, INDEXER_HEADS, INDEXER_DIM, INDEXER_RATIO, INDEXER_BUDGET, 1e7, capacity=total)
            self.indexer.raw_key_destination(0, 0, total).copy_(randn(total, INDEXER_DIM))
            self.norm = (1.0 + 0.1 * torch.randn(INDEXER_DIM, generator=gen, device=dev)).to(torch.bfloat16)
            torch.cuda.synchronize(dev)
            self.indexer.encode_pool_prefill(0, 0, start, self.norm, 1e-6)
            self.iq = randn(self.rows, INDEXER_HEADS, INDEXER_DIM)
            ctx.synchronize()
        if name in ("S2", "S6"):
            # The whole sparse decode step: the block indexer's step (its caches filled to the context, the step's key
            # already in them) -- repooling, query rows, block scores in one launch, then the selection -- and the
            # attention over the mask it has just written.  sparse_step = False runs the dense step on the same cache.
            self.sparse_step = True
            length = self.lengths[0]
            self.indexer = eng.QSAIndexer(ctx, INDEXER_HEADS, INDEXER_DIM, INDEXER_RATIO, INDEXER_BUDGET, 1e7, capacity=length)
            self.indexer.raw_key_destination(0, 0, length).copy_(randn(length, INDEXER_DIM))
            self.norm = (1.0 + 0.1 * torch.randn(INDEXER_DIM, generator=gen, device=dev)).to(torch.bfloat16)
            torch.cuda.synchronize(dev)
            self.indexer.encode_pool_prefill(0, 0, length - 1, self.norm, 1e-6)
            self.iq = randn(1, INDEXER_HEADS, INDEXER_DIM)
            ctx.synchronize()
        self.attn = eng.Attention(ctx)
        self.prefill = eng.PrefillAttention(ctx)
        # stored K and V rows: 1024 / 544 / 288 B each; with a sliding window only the last `window` of a sequence
        windowed = window and self.kind in ("decode", "prefill")
        visible = [min(n, window) if windowed and self.kind == "decode" else n for n in self.lengths]
        self.kv_bytes = sum(visible) * self.kv.token_stride_bytes * 2
        if self.keep is not None and keep_budget > 0:
            # only the 32-key blocks that hold a kept key are read
            padded = torch.nn.functional.pad(self.keep, (0, -self.keep.shape[1] % 32))
            touched = int(padded.view(n, -1, 32).any(dim=-1).sum().item())
            self.kv_bytes = touched * 32 * self.kv.token_stride_bytes * 2
        pairs = sum(min(L, s + r + 1, window if windowed else L) for L, s in zip(self.lengths, self.starts)
                    for r in range(self.rows))
        if self.kind == "prefill_keep":
            # the 32-key blocks that any row keeps a key of cross HBM once; the arithmetic is the kept (row, key) pairs'
            touched = int(self.keep.view(self.rows, -1, 32).any(dim=-1).any(dim=0).sum().item())
            self.kv_bytes = touched * 32 * self.kv.token_stride_bytes * 2
            pairs = int(self.keep.sum().item())
        self.flops = 4 * D * H * pairs
        torch.cuda.synchronize(dev)

    def step(self, i: int) -> None:
        layer = i % self.layers
        n = len(self.lengths)
        if self.kind == "prefill" and self.sparse_step:
            ix, start, total = self.indexer, self.starts[0], self.lengths[0]
            ix.encode_pool_prefill(0, start, self.rows, self.norm, 1e-6)
            # (the norm and rotation work in place: every step norms the rows again, which keeps them bounded)
            ix.encode_scores(0, self.iq, self.norm, start, self.rows, 1e-6)
            ix._select(self.rows, start + 1, ix.scored_blocks_per_row, (total + 3) // 4 * 4, True, mask=False)
            w = self.H * self.D
            params = self.eng.PrefillAttentionParams(start, self.rows, total, self.H, self.scale, w, w, w)
            self.prefill.encode_causal(self.kv, layer, 0, self.q, self.out, params, keep_indices=ix.keep_index_buf,
                                       keep_index_stride=ix.selection_width, keep_counts=ix.keep_count_buf)
        elif self.kind == "decode" and self.sparse_step:
            ix, length = self.indexer, self.lengths[0]
            ix.encode_decode_step(0, length - 1, self.iq, self.norm, self.norm, 1e-6)
            stride = (length + 3) // 4 * 4
            ix._select(1, length, ix.scored_blocks_per_row, stride, False)
            self.attn.encode_full_keep(self.kv, layer, self.q, self.out, self.H, self.lengths, ix.keep_buf, self.scale,
                                       slot=[0], gate=self.gate, keep_stride=stride)
        elif self.kind == "decode" and self.keep is not None and self.keep_form == "indices":
            self.attn.encode_full_keep_indices(self.kv, layer, self.q, self.out, self.H, self.lengths, self.keep_indices,
                                               self.keep_counts, self.scale, slot=list(range(n)), gate=self.gate)
        elif self.kind == "decode" and self.keep is not None:
            self.attn.encode_full_keep(self.kv, layer, self.q, self.out, self.H, self.lengths, self.keep, self.scale,
                                       slot=list(range(n)), gate=self.gate, keep_stride=self.keep.shape[1])
        elif self.kind == "decode" and self.window:
            self.attn.encode_swa(self.kv, layer, self.q, self.out, self.H, self.lengths, self.window, self.scale,
                                 slot=list(range(n)), gate=self.gate)
        elif self.kind == "decode":
            self.attn.encode_full(self.kv, layer, self.q, self.out, self.H, self.lengths, self.scale,
                                  slot=list(range(n)), gate=self.gate)
        elif self.kind == "indexer":
            ix = self.indexer
            if self.rows == 1 and not INDEXER_SEPARATE_LAUNCHES:
                # a decode step: repooling, query norm + rotation and block scores in one launch
                ix.encode_decode_step(0, self.context, self.q, self.norm, self.norm, 1e-6)
            else:
                ix.encode_pool_prefill(0, self.context, self.rows, self.norm, 1e-6)
                # the norm and rotation work in place: every step norms the rows again, which keeps them bounded
                ix.encode_scores(0, self.q, self.norm, self.context, self.rows, 1e-6)
            blocks = ix.scored_blocks_per_row
            stride = (self.context + self.rows + 3) // 4 * 4
            ix._select(self.rows, self.context + 1, blocks, stride, True, mask=not INDEXER_LISTS_ONLY)
        elif self.kind == "projection":
            self.projection.encode(self.weight_bits, self.weights[layer], self.w_scales[layer], self.w_biases[layer], self.q,
                                   self.out, self.m, self.n, self.rows)
        elif self.kind == "epilogue":
            self.epilogue.encode(self.kv, layer, self.packed, self.k_proj, self.v_proj, self.q_weight, self.k_weight,
                                 self.q, self.gate, self.H, 0, self.rows, 1e-6, 64, 1e7)
        elif self.kind == "verify":
            self.attn.encode_verify_rows(self.kv, layer, self.q, self.out, self.H, self.starts, self.rows, self.scale,
                                         list(range(n)), gate=self.gate)
        elif self.kind == "prefill_keep":
            w = self.H * self.D
            params = self.eng.PrefillAttentionParams(self.starts[0], self.rows, self.lengths[0], self.H, self.scale, w, w, w)
            if self.keep_form == "indices":
                self.prefill.encode_causal(self.kv, layer, 0, self.q, self.out, params, keep_indices=self.keep_indices,
                                           keep_index_stride=self.keep_indices.shape[1], keep_counts=self.keep_counts)
            else:
                self.prefill.encode_causal(self.kv, layer, 0, self.q, self.out, params, keep_mask=self.keep,
                                           keep_stride=self.keep.shape[1])
        else:
            w = self.H * self.D
            self.prefill.encode_causal(self.kv, layer, 0, self.q, self.out,
                                       self.eng.PrefillAttentionParams(self.starts[0], self.rows, self.lengths[0], self.H, self.scale, w, w, w,
                                                                       sliding_window=self.window),
                                       gate=self.gate)

    def close(self):
        if self.kv is not None:
            self.kv.close()


def measure(wl: DeviceWorkload, steps: int, warmup: int, launch: str):
    """Times exactly `steps` steps; returns (wall ms/step, device ms/step, dominant-kernel us/launch, launches)."""
    import torch
    ctx = wl.ctx
    for i in range(warmup):
        wl.step(i)
    ctx.synchronize()
    graph = None
    if launch == "graph":
        ctx.graph_begin()
        for i in range(steps):
            wl.step(i)
        graph = ctx.graph_end()
        graph.launch()  # untimed: first replay uploads the graph
        ctx.synchronize()
    torch.cuda.synchronize(wl.dev)
    ctx.synchronize()
    t0 = time.perf_counter()
    ctx.timer_begin()
    if graph is not None:
        graph.launch()
    else:
        for i in range(steps):
            wl.step(i)
    dev_ns = ctx.timer_end_ns()  # blocks until the stream is idle
    ctx.synchronize()
    torch.cuda.synchronize(wl.dev)
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    if graph is not None:
        graph.close()
    # Second pass: the dominant kernel alone, by HIP events on the launch stream.  The library binds a start and a
    # stop event to that kernel's dispatch (hipExtLaunchKernelGGL): the pair reads the dispatch's own begin-to-end
    # time, which is what a kernel trace reports, and nothing is subtracted from it.  The indexer's entry points
    # span several launches each and record a pair AROUND them: there an empty pair's reading is taken off, and the
    # line says that its kernel time is an estimate.
    ctx.profile_enable(steps)
    for i in range(steps):
        wl.step(i)
    launches, total_ns = ctx.profile_read()
    overhead_us = ctx.profile_event_overhead_ns() / 1e3 if wl.kind == "indexer" else 0.0
    ctx.profile_disable()
    raw_us = total_ns / max(launches, 1) / 1e3
    kern_us = max(raw_us - overhead_us, 1e-3)
    # Third pass, for the kernels whose step is a pass over K/V plus a combine pass: `steps` launches of the pass ALONE
    # (the library's measurement control leaves the combine out; outputs are not written), replayed from one graph
    # between one pair of events: the kernel's sustained launch duration, launch-to-launch, with nothing subtracted.
    run_us = None
    if wl.kind in ("decode", "verify") and launch == "graph" and not getattr(wl, "sparse_step", False):
        from tinytitan_amd import capi
        ctx.set_option(capi.OPT_MEASURE_PASS_ONLY, 1)
        try:
            ctx.graph_begin()
            for i in range(steps):
                wl.step(i)
            run = ctx.graph_end()
            run.launch()
            ctx.synchronize()
            ctx.timer_begin()
            run.launch()
            run_us = ctx.timer_end_ns() / 1e3 / max(launches, 1)
            run.close()
        finally:
            ctx.set_option(capi.OPT_MEASURE_PASS_ONLY, 0)
        wl.step(0)  # (the outputs are whole again)
        ctx.synchronize()
    elif launch == "graph" and launches == steps and wl.kind in ("prefill", "projection", "epilogue") and \
            (wl.kind == "projection" or wl.bits == 16) and (wl.kind != "prefill" or wl.starts[0] == 0):
        run_us = dev_ns / 1e3 / steps  # a step IS one launch of the kernel: the timed replay above is that run
    return wall_ms, dev_ns / 1e6 / steps, (kern_us, raw_us, overhead_us, run_us), launches


def read_control(ctx, nbytes: int, steps: int, warmup: int):
    """The plain-read control: a kernel that only reads `nbytes`, timed like the dominant kernel (a HIP event pair bound
    to each dispatch), rotating over 1 GiB of regions so that every launch reads HBM."""
    import torch
    regions = max(2, -(-(1 << 30) // nbytes))
    buf = torch.empty(regions * nbytes, dtype=torch.uint8, device="cuda")
    buf.random_(0, 256)
    torch.cuda.synchronize()
    read = 0
    for i in range(warmup):
        read = ctx.calibrate_read(buf, (i % regions) * nbytes, nbytes)
    ctx.synchronize()
    ctx.profile_enable(steps)
    for i in range(steps):
        ctx.calibrate_read(buf, (i % regions) * nbytes, nbytes)
    launches, total_ns = ctx.profile_read()
    ctx.profile_disable()
    dispatch_us = max(total_ns / max(launches, 1) / 1e3, 1e-3)
    # ... and like the attention pass: the same launches replayed from one graph between one pair of events
    ctx.graph_begin()
    for i in range(steps):
        ctx.calibrate_read(buf, (i % regions) * nbytes, nbytes)
    run = ctx.graph_end()
    run.launch()
    ctx.synchronize()
    ctx.timer_begin()
    run.launch()
    kern_us = max(ctx.timer_end_ns() / 1e3 / steps, 1e-3)
    run.close()
    del buf
    return {"kernel": "calibrate_read_kernel", "bytes_per_launch": read, "kernel_us": round(kern_us, 2),
            "timed_by": "one HIP event pair around a graph replay of the launches, divided by their number",
            "dispatch_event_us": round(dispatch_us, 2),
            "achieved": round(read / (kern_us * 1e-6) / 1e9, 1), "unit": "GB/s",
            "frac": round(read / (kern_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4), "launches": launches}


def oracle_table_row(wl, threads_all: int):
    """One row of the five-configuration table: the CPU oracle over the WHOLE seeded configuration on one thread (the
    reference's attention loop is single-threaded) and head-parallel on `threads_all` threads (labelled non-reference),
    and the GPU output's distance from it after both are rounded to fp16."""
    import numpy as np
    import oracle
    w = wl.host
    got = wl.out.float().cpu().numpy()
    worst, total, count = 0.0, 0.0, 0
    cpu_s = {1: 0.0, threads_all: 0.0}
    for i, s in enumerate(w.sequences):
        k = s.k.astype(np.float32).reshape(s.k.shape[0], -1)
        v = s.v.astype(np.float32).reshape(s.v.shape[0], -1)
        rows = s.q.shape[0]
        q = s.q.astype(np.float32).reshape(rows, -1)
        g = s.gate.astype(np.float32).reshape(rows, -1) if s.gate is not None else None
        positions = s.start + rows
        ref = None
        for threads in (1, threads_all):
            t0 = time.perf_counter()
            if w.kind == "decode" and threads == 1:  # CPUQwen35.attention, as the reference runs a decode row
                ref = oracle.decode(q[0], k, v, w.heads, w.kv_heads, w.dim, w.scale, gate=g[0] if g is not None else None)[None]
            else:
                o = oracle.attention_batch(q, k[:positions], v[:positions], rows, s.start, w.heads, w.kv_heads, w.dim, w.scale,
                                           gate=g, threads=threads)
                if threads == 1:
                    ref = o
            cpu_s[threads] += time.perf_counter() - t0
        ref = ref.reshape(rows, w.heads, w.dim).astype(np.float16).astype(np.float64)
        diff = np.abs(got[i].reshape(rows, w.heads, w.dim).astype(np.float64) - ref)
        worst = max(worst, float(diff.max()))
        total += float(diff.sum())
        count += diff.size
    return {"cpu_ms_1_thread": round(cpu_s[1] * 1e3, 2), "cpu_ms_all_threads": round(cpu_s[threads_all] * 1e3, 2),
            "cpu_threads_all": threads_all, "max_abs": worst, "mean_abs": total / max(count, 1)}


def projection_kernel(tokens: int) -> str:
    """Which of the three o_proj kernels a token count takes (tt_hip_affine_projection's own thresholds)."""
    return "affine_gemv_kernel" if tokens <= 9 else ("affine_proj_kernel" if tokens < 513 else "affine_gemm_kernel")


def flop_bound(wl) -> bool:
    return wl.kind == "prefill" or (wl.kind == "projection" and wl.rows > 256)


def roofline_for(wl: DeviceWorkload, timing):
    kern_us, raw_us, overhead_us, run_us = timing
    if wl.kind == "indexer":
        kern_us *= 2  # two timed entry points per step: the block scores and the selection
    res = _roofline_for(wl, run_us if run_us is not None else kern_us)
    if wl.kind == "indexer":
        res["timed_by"] = "HIP event pairs recorded around each entry point's launches, less an empty pair's reading: an estimate"
        res["event_pair_us"] = round(raw_us, 2)
        res["empty_event_pair_us"] = round(overhead_us, 2)
    elif run_us is not None:
        if wl.kind in ("decode", "verify"):
            res["timed_by"] = ("one HIP event pair around a graph replay of nothing but this kernel's launches (the steps without "
                               "their combine pass), divided by their number: launch to launch, nothing subtracted")
        else:
            res["timed_by"] = ("one HIP event pair around a graph replay of the steps, each of which is one launch of this "
                               "kernel, divided by their number: launch to launch, nothing subtracted")
        res["dispatch_event_us"] = round(kern_us, 2)  # a pair bound to each dispatch: includes the command processor's work around the kernel
    else:
        res["timed_by"] = "HIP events bound to the dispatch (its begin to its end), nothing subtracted"
    key = wl.name if wl.bits == 16 else f"{wl.name}/{wl.bits}"
    if wl.kind == "projection":
        key = wl.name if wl.weight_bits == 4 else f"{wl.name}/{wl.weight_bits}"
    if (wl.kind == "projection" and wl.rows != PROJECTION_DEFAULT_TOKENS[wl.name]) or wl.keep is not None:
        key = None  # --tokens / --keep-fraction: not the measured shape
    res["traffic"] = None if wl.window else MEASURED_TRAFFIC_BYTES.get(key)
    return res


def _roofline_for(wl: DeviceWorkload, kern_us: float):
    if wl.kind == "projection" and wl.rows > 256:
        achieved = wl.flops / (kern_us * 1e-6) / 1e12
        return {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None,
                "kernel": projection_kernel(wl.rows), "kernel_us": round(kern_us, 2), "flops_per_launch": wl.flops}
    if wl.kind == "prefill":
        achieved = wl.flops / (kern_us * 1e-6) / 1e12
        return {"bound": "mfma", "achieved": round(achieved, 2), "peak": MFMA_FP16_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / MFMA_FP16_PEAK_TFLOPS, 4), "traffic": None,
                "kernel": "attn_prefill_kernel", "kernel_us": round(kern_us, 2), "flops_per_launch": wl.flops}
    achieved = wl.kv_bytes / (kern_us * 1e-6) / 1e9
    return {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": None,
            "kernel": {"epilogue": "qkv_epilogue_kernel", "projection": projection_kernel(wl.rows),
                       "indexer": "qsa_scores_kernel + the qsa_select kernels"}.get(wl.kind, "attn_splitk_kernel"),
            "kernel_us": round(kern_us, 2), "bytes_per_launch": wl.kv_bytes}


def cpu_baseline(name: str, budget_s: float = 12.0, kv_bits: int = 16, window: int = 0, weight_bits: int = 4,
                 keep_fraction: float = 0.0):
    """The CPU oracle (a scalar restatement of the reference's CPU attention) on this host, one thread."""
    import numpy as np
    import oracle
    from tinytitan_amd import synthetic
    if name in PROJECTION_TOKENS:
        # The reference's own C kernel (tinytitan_int4_affine_gemv / tinytitan_int8_affine_gemv, compiled from the
        # reference checkout into oracle/_ref) where that build is present, else the oracle's restatement of it:
        # one vector against the 2048 x 4096 matrix, one thread, repeated.
        m, n = 2048, 4096
        r = np.random.default_rng(0x0A)
        packed, scales, biases = oracle.affine_quantize_rows(r.uniform(-0.5, 0.5, (m, n)).astype(np.float32), weight_bits)
        x = r.standard_normal(n).astype(np.float16).astype(np.float32)
        have_ref = oracle.reference_affine_gemv(packed, scales, biases, x, weight_bits) is not None
        run_once = (lambda: oracle.reference_affine_gemv(packed, scales, biases, x, weight_bits)) if have_ref else \
                   (lambda: oracle.affine_gemv(packed, scales, biases, x, weight_bits))
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            run_once()
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        fn = f"tinytitan_int{weight_bits}_affine_gemv built from the reference's C source" if have_ref else "tt_oracle_affine_gemv"
        sample = f"{reps} x one token against the {m} x {n} {weight_bits}-bit matrix ({fn}, 1 thread, {dt * 1e3:.2f} ms each)"
        if PROJECTION_TOKENS[name] > 256:
            return {"value": round(2 * m * n / dt / 1e12, 6), "unit": "TFLOP/s", "cores": 1,
                    "kind": "reference" if have_ref else "port", "sample": sample}
        stored = packed.nbytes + scales.nbytes + biases.nbytes
        return {"value": round(stored / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "reference" if have_ref else "port",
                "sample": sample}
    if name in INDEXER_SHAPES:
        # The oracle's restatement of the Metal scoring kernel (all host threads) and of the host selection (a sort
        # per row, one thread): a decode step whole, a chunk on its last 64 rows (the ones that see most).
        context, tokens = INDEXER_SHAPES[name]
        rows = min(tokens, 64)
        context += tokens - rows
        blocks = (context + rows - 1) // INDEXER_RATIO + 1
        r = np.random.default_rng(0x0B)
        pooled = r.standard_normal((blocks, INDEXER_DIM)).astype(np.float16).view(np.uint16)
        q = r.standard_normal((rows, INDEXER_HEADS, INDEXER_DIM)).astype(np.float16).view(np.uint16)
        width = INDEXER_BUDGET + INDEXER_RATIO - 1
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            scores = oracle.qsa_block_scores(q, pooled, INDEXER_DIM, INDEXER_HEADS, blocks, rows)
            for row in range(rows):
                oracle.qsa_select_keys(scores[row], context + row + 1, INDEXER_RATIO, width)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        share = indexer_bytes(*INDEXER_SHAPES[name]) * rows / tokens  # the sampled rows' share of a step's bytes
        return {"value": round(share / dt / 1e9, 4), "unit": "GB/s", "cores": oracle.max_threads(), "kind": "port",
                "sample": f"{reps} x scoring and selection of {rows} query rows over {blocks} blocks "
                          f"(tt_oracle_qsa_block_scores on {oracle.max_threads()} threads, tt_oracle_qsa_select_keys on 1; "
                          f"{dt * 1e3:.2f} ms each)"}
    if window or keep_fraction > 0.0:
        return None  # the baselines below walk every key
    if kv_bits != 16 and name != "C2":
        return None  # the quantised baseline below is the C2 shape; the other shapes report the fp16 one without --kv-bits
    if kv_bits != 16:
        # The reference's CPU engine keeps fp32 K/V; what stands beside the quantised GPU path is the
        # Metal loader's arithmetic restated (tt_oracle_kv_dequantize_rows over the stored rows of K
        # and of V) followed by the decode oracle: one step over the C2-shaped cache.
        bits = kv_bits
        H, KH, D, T = 16, 2, 256, 32768
        r = np.random.default_rng(0xC8)
        q = r.standard_normal((H, D)).astype(np.float32)
        rows = [oracle.kv_quantize_rows(r.standard_normal((T, KH * D)).astype(np.float16).astype(np.float32), bits)
                for _ in range(2)]
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            k, v = (oracle.kv_dequantize_rows(x, KH * D, bits) for x in rows)
            oracle.decode(q, k, v, H, KH, D, 1.0 / 16.0)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": round(2 * rows[0].nbytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} full decode steps over 32768 stored {bits}-bit rows (tt_oracle_kv_dequantize_rows + "
                          f"tt_oracle_decode, 1 thread, {dt * 1e3:.1f} ms each)"}
    if name in ("C1", "C2"):
        w = synthetic.BUILDERS[name]()
        s = w.sequences[0]
        k = s.k.astype(np.float32).reshape(s.k.shape[0], -1)
        v = s.v.astype(np.float32).reshape(s.v.shape[0], -1)
        q = s.q.astype(np.float32)[0]
        g = s.gate.astype(np.float32)[0] if s.gate is not None else None
        oracle.decode(q, k, v, w.heads, w.kv_heads, w.dim, w.scale, gate=g)  # warm-up
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            oracle.decode(q, k, v, w.heads, w.kv_heads, w.dim, w.scale, gate=g)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": round(w.kv_bytes / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} full {name} decode steps (tt_oracle_decode, 1 thread, {dt * 1e3:.1f} ms each)"}
    if name in ("C3", "C4", "C5"):
        # CPUQwen35.attentionBatch restated (tt_oracle_attention_batch, one thread) on a bounded sample of
        # the workload: C4 its first 512 tokens; C5 one of its 8 sequences; C3 one decode step
        # (tt_oracle_decode) over its shortest sequence.  Reported in the workload's own unit over the
        # sample's own work.
        H, KH, D, scale = 16, 2, 256, 1.0 / 16.0
        r = np.random.default_rng(0xC0)
        if name == "C4":
            rows, base, what = 512, 0, "first 512 tokens of the chunk"
        elif name == "C5":
            rows, base, what = 4, 65536, "one of the 8 sequences (4 rows over 65540 keys)"
        else:
            rows, base = 1, min(synthetic.c3_lengths()) - 1
            what = f"the shortest of the 32 sequences ({base + 1} keys)"
        keys = base + rows
        q = r.standard_normal((rows, H * D)).astype(np.float32)
        k = r.standard_normal((keys, KH * D)).astype(np.float32)
        v = r.standard_normal((keys, KH * D)).astype(np.float32)
        if name == "C3":  # a decode step: the decode oracle, as for C1 / C2
            run_once = lambda: oracle.decode(q[0], k, v, H, KH, D, scale)
        else:
            run_once = lambda: oracle.attention_batch(q, k, v, rows, base, H, KH, D, scale)
        run_once()  # warm-up
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            run_once()
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        if name == "C4":
            pairs = sum(base + t + 1 for t in range(rows))
            return {"value": round(4 * D * H * pairs / dt / 1e12, 5), "unit": "TFLOP/s", "cores": 1, "kind": "port",
                    "sample": f"{reps} x {what} (tt_oracle_attention_batch, 1 thread, {dt * 1e3:.1f} ms each)"}
        return {"value": round(keys * KH * D * 2 * 2 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} x {what} ({'tt_oracle_decode' if name == 'C3' else 'tt_oracle_attention_batch'}, 1 thread, "
                          f"{dt * 1e3:.1f} ms each; bytes counted at the GPU path's fp16 widths)"}
    if name == "K4":
        # Each row is the decode oracle over the rows of K and V that it keeps (a masked-out key is an absent one): a
        # sample of 32 of the chunk's 256 rows, 2048 + 4 kept keys each.
        H, KH, D, rows, kept = 16, 2, 256, 32, INDEXER_BUDGET + INDEXER_RATIO
        r = np.random.default_rng(0x4B)
        q = r.standard_normal((rows, H, D)).astype(np.float32)
        k, v = (r.standard_normal((kept, KH * D)).astype(np.float32) for _ in range(2))
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            for t in range(rows):
                oracle.decode(q[t], k, v, H, KH, D, 1.0 / 16.0)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        # in the GPU path's unit: the touched blocks' bytes, of which the sampled rows do an eighth of the arithmetic
        blocks = INDEXER_BUDGET // INDEXER_RATIO + 8
        return {"value": round(blocks * 32 * KH * D * 2 * 2 * (rows / 256) / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} x 32 of the 256 rows, each over its {kept} kept keys (tt_oracle_decode, 1 thread, {dt * 1e3:.1f} ms each; "
                          f"bytes: the sample's share of the touched blocks at fp16 widths)"}
    if name == "E4":
        H, KH, D, T = 16, 2, 256, 512
        r = np.random.default_rng(0xE4)
        packed = r.standard_normal((T, H, 2 * D)).astype(np.float32)
        k = r.standard_normal((T, KH * D)).astype(np.float32)
        w = np.ones(D, np.float32)
        reps, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < budget_s:
            oracle.qkv_epilogue(packed, k, T, H, KH, D, w, w, 1e-6, 64, 1e7, 0)
            reps += 1
        dt = (time.perf_counter() - t0) / reps
        return {"value": round(T * (2 * H * D + 2 * KH * D) * 4 / dt / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
                "sample": f"{reps} x 512 tokens of the 4096-token chunk (tt_oracle_qkv_epilogue, 1 thread, "
                          f"{dt * 1e3:.1f} ms each; bytes counted at the GPU path's fp16 widths)"}
    return None


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="C2", choices=["C1", "C2", "C3", "C4", "C5", "K4", "E4", "O1", "O5", "O4", "Q2", "Q6", "Q4", "Q3", "S2", "S6", "D1", "D2", "D6",
                                                              "P2", "P6"])
    ap.add_argument("--weight-bits", type=int, default=4, choices=[4, 8],
                    help="width of the o_proj levels of the O workloads (the reference stores q_proj / o_proj at 4 bits)")
    ap.add_argument("--kv-bits", type=int, default=16, choices=[16, 8, 4],
                    help="precision of the KV cache the attention workloads read: fp16, or the 8 / 4-bit affine rows "
                         "(bytes are then counted at the stored row widths, 544 / 288 B per token and side at 2 x 256)")
    ap.add_argument("--window", type=int, default=0,
                    help="sliding window of the decode and prefill workloads (C1-C4): a row sees its last WINDOW keys (0: all)")
    ap.add_argument("--keep-fraction", type=float, default=0.0,
                    help="decode workloads (C1-C3): attend over a random sparse key selection that keeps this fraction "
                         "of the keys (the keepMask of the reference's decode); at random nearly every 32-key block holds a kept "
                         "key and is read")
    ap.add_argument("--keep-budget", type=int, default=0,
                    help="decode workloads (C1-C3): attend over a selection shaped like the block indexer's: this many "
                         "cells in random complete blocks of 4 keys, plus the query's own ragged tail; key blocks "
                         "without a kept key are not read")
    ap.add_argument("--keep-rows", default="shared", choices=["shared", "independent"],
                    help="K4: every row keeps the same cells, or each row draws its own")
    ap.add_argument("--indexer-separate-launches", action="store_true",
                    help="Q2 / Q6: the decode step's repooling, query rows and block scores as three launches (the A/B of the fused one)")
    ap.add_argument("--indexer-lists-only", action="store_true",
                    help="Q workloads: the selection writes the index lists and their counts and no mask rows")
    ap.add_argument("--keep-form", default="mask", choices=["mask", "indices"],
                    help="K4, and decode workloads with a selection: rows of bytes, or compacted into per-row lists of key ids")
    ap.add_argument("--tokens", type=int, default=0,
                    help="token count of an O workload instead of its own (e.g. 128, the reference's default prefill chunk)")
    ap.add_argument("--layers", type=int, default=0, help="layer caches to rotate over (0: enough for >= 1 GiB of KV)")
    ap.add_argument("--launch", default="graph", choices=["graph", "eager"])
    ap.add_argument("--all", action="store_true", help="also measure the other configurations")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true")
    ap.add_argument("--split-tokens", type=int, default=0, help="override the split-K planner (keys per split)")
    ap.add_argument("--data-scale", type=float, default=1.0,
                    help="multiply the synthetic q/K/V by this (0: all zeros).  Not a benchmark setting: it shows how far "
                         "the card's power limit, i.e. the operand data, sets the MFMA-bound kernel's time")
    ap.add_argument("--no-calibrate-read", action="store_true",
                    help="skip the plain-read control (a kernel that only reads the workload's KV bytes, timed the same way; "
                         "run by default beside the HBM-bound attention workloads)")
    ap.add_argument("--table", action="store_true",
                    help="measure the five configurations C1-C5 on their seeded inputs at full size, run the CPU oracle over the "
                         "whole of each (one thread, and head-parallel on every host thread) and report the table: CPU ms, "
                         "GPU us, rate, fraction of peak, max-abs and mean-abs against the oracle (takes a few minutes)")
    ap.add_argument("--no-prefill", action="store_true",
                    help="default run only: skip the C4 causal-prefill block (the second half of the metric)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run a plain 64 MiB -> 64 MiB elementwise copy 10 times (the known-size kernel that "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings are scaled by)")
    args = ap.parse_args()
    global INDEXER_SEPARATE_LAUNCHES, INDEXER_LISTS_ONLY
    INDEXER_SEPARATE_LAUNCHES = args.indexer_separate_launches
    INDEXER_LISTS_ONLY = args.indexer_lists_only
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (no collectives, no sharding); use --gpus 1", file=sys.stderr)
        return 2
    import numpy as np
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the attention path has no CPU fallback", file=sys.stderr)
        return 3
    if args.tokens > 0 and args.workload in PROJECTION_TOKENS:
        PROJECTION_TOKENS[args.workload] = args.tokens
    eng = _load_engine()
    ctx = eng.HIPContext(0)
    ctx.set_split_tokens(args.split_tokens)

    def layers_for(name):
        if args.layers > 0:
            return args.layers
        if name in INDEXER_SHAPES:
            return 1
        if name in PROJECTION_TOKENS:
            return 128  # 128 weight sets of 4.5 / 8.5 MiB: more than the 256 MiB last-level cache holds
        per_layer = {"C1": 4 << 20, "C2": 64 << 20, "C3": 600 << 20, "C4": 8 << 20, "C5": 1 << 30, "K4": 256 << 20, "E4": 8 << 20,
                     "S2": 64 << 20, "S6": 512 << 20, "D1": 16 << 20, "D2": 64 << 20, "D6": 256 << 20, "P2": 64 << 20,
                     "P6": 256 << 20}[name]
        if name != "E4":
            per_layer = per_layer * kv_bits_for(name) // 16
        return max(2, min(64, -(-(1 << 30) // per_layer)))

    def kv_bits_for(name):
        return 16 if name == "E4" else args.kv_bits

    def run(name, seeded):
        wl = DeviceWorkload(eng, ctx, name, layers_for(name), seeded and args.data_scale == 1.0, args.data_scale,
                            kv_bits_for(name), args.window, args.weight_bits, args.keep_fraction, args.keep_budget, args.keep_rows, args.keep_form)
        steps = args.steps if name in ("C1", "C2", "O1", "O5", "Q2", "Q6", "S2", "S6") else max(10, args.steps // 10)
        wall_ms, dev_ms, kern_us, launches = measure(wl, steps, args.warmup, args.launch)
        res = {"steps": steps, "ms_per_step": round(wall_ms, 5), "device_ms_per_step": round(dev_ms, 5),
               "kv_GBps": round(wl.kv_bytes / (wall_ms * 1e-3) / 1e9, 1),
               "TFLOPps": round(wl.flops / (wall_ms * 1e-3) / 1e12, 2),
               "layers": wl.layers, "roofline": None if wl.sparse_step else roofline_for(wl, kern_us)}
        if wl.sparse_step:
            # the dense step over the same caches, timed the same way: what the sparse step has to beat
            wl.sparse_step = False
            d_wall, d_dev, _, _ = measure(wl, steps, args.warmup, args.launch)
            wl.sparse_step = True
            res["dense_step"] = {"ms_per_step": round(d_wall, 5), "device_ms_per_step": round(d_dev, 5),
                                 "kv_GBps": round(wl.kv_bytes / (d_wall * 1e-3) / 1e9, 1)}
        parity = None
        if seeded and not args.no_parity and wl.host is not None and name in ("C1", "C2") and wl.bits == 16 and not wl.window \
                and wl.keep is None:
            import oracle
            s = wl.host.sequences[0]
            ref = oracle.decode(s.q.astype(np.float32)[0], s.k.astype(np.float32).reshape(s.k.shape[0], -1),
                                s.v.astype(np.float32).reshape(s.v.shape[0], -1), wl.H, wl.KH, wl.D, wl.scale,
                                gate=s.gate.astype(np.float32)[0] if s.gate is not None else None)
            ref = ref.astype(np.float16).astype(np.float32)
            got = wl.out.float().cpu().numpy()[0, 0]
            parity = {"max_abs": float(np.abs(got - ref).max()), "mean_abs": float(np.abs(got - ref).mean())}
            res["parity_vs_oracle"] = parity
        wl.close()
        return wl, res

    if args.table:
        import oracle
        rows = {}
        for name in ("C1", "C2", "C3", "C4", "C5"):
            t0 = time.perf_counter()
            wl = DeviceWorkload(eng, ctx, name, layers_for(name), True)
            steps = args.steps if name in ("C1", "C2") else max(10, args.steps // 10)
            wall_ms, dev_ms, kern, launches = measure(wl, steps, args.warmup, args.launch)
            roof = roofline_for(wl, kern)
            row = {"gpu_step_us": round(wall_ms * 1e3, 2), "gpu_kernel_us": roof["kernel_us"], "kernel": roof["kernel"],
                   "rate": roof["achieved"], "unit": roof["unit"], "frac_of_peak": roof["frac"],
                   "step_rate": round((wl.flops / 1e12 if flop_bound(wl) else wl.kv_bytes / 1e9) / (wall_ms * 1e-3), 1)}
            row.update(oracle_table_row(wl, oracle.max_threads()))
            wl.close()
            rows[name] = row
            print(f"bench.py --table: {name} done in {time.perf_counter() - t0:.0f} s: {row}", file=sys.stderr, flush=True)
        print(json.dumps({"table": rows, "data": "synthetic, seeded (tinytitan_amd/synthetic.py)", "n_gpus": 1,
                          "parity_bar": {"max_abs": 2e-3, "mean_abs": 2e-4}}))
        ctx.close()
        return 0
    wl, main_res = run(args.workload, seeded=args.workload in ("C1", "C2"))
    line = {
        "metric": "decode attn KV GB/s @32k ctx" if args.workload == "C2" else (
            "sparse prefill chunk step (indexer + selection + attention over it): the dense chunk's flops per step time, TFLOP/s"
            if wl.sparse_step and wl.kind == "prefill" else (
            "sparse decode step (indexer + selection + attention over it): the context's KV bytes per step time, GB/s" if wl.sparse_step else (
            "epilogue bytes GB/s" if args.workload == "E4" else (
                f"o_proj throughput {args.workload}" if wl.kind == "projection" else (
                    f"indexer bytes GB/s {args.workload}" if wl.kind == "indexer" else f"attention throughput {args.workload}"))))),
        "value": main_res["TFLOPps"] if flop_bound(wl) else main_res["kv_GBps"],
        "unit": "TFLOP/s" if flop_bound(wl) else "GB/s",
        "n_gpus": 1, "steps": main_res["steps"], "warmup": args.warmup, "ms_per_step": main_res["ms_per_step"],
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 rows, f32 scores, u64 selection keys" if wl.kind == "indexer" else f"u{wl.weight_bits} levels + bf16 scale/bias, f16 activations, f32 accumulate" if wl.kind == "projection" else "f16 storage, f32 accumulate" if wl.bits == 16 else f"u{wl.bits} levels + f16 scale/bias storage, f16 operands, f32 accumulate",
        "data": "synthetic" if args.data_scale == 1.0 else "synthetic x %g (NOT the benchmark setting)" % args.data_scale,
        "config": {"workload": {
            "C1": "C1 decode B1 8q/2kv heads dim256 ctx2048",
            "C2": "C2 decode B1 16q/2kv heads dim256 ctx32768, K RoPE-rotated, sigmoid gate",
            "C3": "C3 decode B32 16q/2kv heads dim256 ctx U[512,16384]",
            "C4": "C4 causal prefill T4096 16q/2kv heads dim256 from position 0",
            "C5": "C5 verify B8 x 4 rows over 65536+4 keys 16q/2kv heads dim256, sigmoid gate",
            "K4": "K4 sparse prefill chunk: 256 rows behind 130816 cached keys, 16q/2kv heads dim256, every row keeping its own selection of cells in blocks of 4 (one byte per key) and its own block",
            "E4": "E4 pre-attention epilogue + KV append of the C4 chunk: T4096 16q/2kv heads dim256, rotary 64",
            "O1": "O1 o_proj behind the gate, 1 decode row: 2048 x 4096 affine matrix, group 64",
            "O5": "O5 o_proj behind the gate, the 32 rows of a C5 verify pass: 2048 x 4096 affine matrix, group 64",
            "O4": "O4 o_proj behind the gate, the 4096-token C4 chunk: 2048 x 4096 affine matrix, group 64",
            "Q2": "Q2 sparse-attention indexer, decode step at 32768 keys: repool, query norm + rotation, block scores, selection (4 heads of 128, blocks of 4, budget 2048)",
            "Q6": "Q6 sparse-attention indexer, decode step at 262144 keys: repool, query norm + rotation, block scores, selection (4 heads of 128, blocks of 4, budget 2048)",
            "Q4": "Q4 sparse-attention indexer, the 4096-token C4 chunk: pooling, query norm + rotation, block scores, per-row selection (4 heads of 128, blocks of 4, budget 2048)",
            "Q3": "Q3 sparse-attention indexer, a 4096-token chunk behind 28672 cached keys: pooling, query norm + rotation, block scores, per-row selection (4 heads of 128, blocks of 4, budget 2048)",
            "D1": "D1 the reference's default prefill chunk, 128 rows, behind 8064 cached keys, 16q/2kv heads dim256",
            "D2": "D2 the reference's default prefill chunk, 128 rows, behind 32640 cached keys, 16q/2kv heads dim256",
            "D6": "D6 the reference's default prefill chunk, 128 rows, behind 130944 cached keys, 16q/2kv heads dim256",
            "P2": "P2 whole sparse step of the default prefill chunk, 128 rows behind 32640 cached keys: the indexer's chunk step (pooling, query rows, block scores, per-row selection as index lists, budget 2048 in blocks of 4) and the chunk attention over the lists; `dense_step` = the D2 chunk over the same cache",
            "P6": "P6 whole sparse step of the default prefill chunk, 128 rows behind 130944 cached keys: the indexer's chunk step and the chunk attention over its index lists; `dense_step` = the D6 chunk over the same cache",
            "S2": "S2 whole sparse decode step at 32768 keys: the indexer's step in one launch, the selection (budget 2048, blocks of 4), the decode over the mask it wrote; `dense_step` = the C2 decode over the same cache",
            "S6": "S6 whole sparse decode step at 262144 keys: the indexer's step in one launch, the selection (budget 2048, blocks of 4), the decode over the mask it wrote; `dense_step` = the dense decode over the same cache"}[args.workload]
            + (f", {wl.weight_bits}-bit levels" if wl.kind == "projection" else "")
            + (f", {wl.rows} tokens (--tokens)" if wl.kind == "projection" and args.tokens > 0 else "")
            + ("" if wl.bits == 16 else f", {wl.bits}-bit KV cache")
            + (f", sliding window {wl.window}" if wl.window and wl.kind in ("decode", "prefill") else "")
            + (f", sparse selection keeping {args.keep_fraction:g} of the keys" if wl.keep is not None and args.keep_fraction > 0 else "")
            + (f", sparse selection of {args.keep_budget} cells in blocks of 4" if wl.keep is not None and args.keep_budget > 0 else "")
            + (f", {args.keep_budget or INDEXER_BUDGET} cells a row, {args.keep_rows}, as {args.keep_form}" if wl.kind == "prefill_keep" else ""),
            "layer_caches_rotated": main_res["layers"], "launch": args.launch,
            "kv_bytes_per_step": wl.kv_bytes, "flops_per_step": wl.flops},
        "device_ms_per_step": main_res["device_ms_per_step"],
        "roofline": main_res["roofline"],
    }
    if "parity_vs_oracle" in main_res:
        line["parity_vs_oracle"] = main_res["parity_vs_oracle"]
    if "dense_step" in main_res:
        line["dense_step"] = main_res["dense_step"]
    # (the read kernel gives every CU 64 KiB a turn: a cache smaller than one turn -- C1's 4 MiB -- has no such control)
    if wl.kind in ("decode", "verify") and wl.keep is None and not wl.window and not args.no_calibrate_read and not wl.sparse_step \
            and wl.kv_bytes >= 256 * 65536:
        # the same bytes through a kernel that only reads them
        line["read_control"] = read_control(ctx, wl.kv_bytes, main_res["steps"], args.warmup)
    default_run = args.workload == "C2" and args.kv_bits == 16 and not args.window and args.keep_fraction == 0.0 \
        and args.keep_budget == 0 and args.data_scale == 1.0 and args.split_tokens == 0
    if default_run and not args.no_prefill and not args.all:
        # The metric's second half: causal prefill of a 4096-token chunk (C4), TFLOP/s against the fp16 MFMA peak.
        wl4, res4 = run("C4", seeded=False)
        line["prefill"] = {
            "metric": "prefill attn TFLOP/s (% MFMA)", "value": res4["TFLOPps"], "unit": "TFLOP/s", "steps": res4["steps"],
            "warmup": args.warmup, "ms_per_step": res4["ms_per_step"], "device_ms_per_step": res4["device_ms_per_step"],
            "dtype": "f16 storage and MFMA operands, f32 accumulate", "data": "synthetic",
            "config": {"workload": "C4 causal prefill T4096 16q/2kv heads dim256 from position 0",
                       "layer_caches_rotated": res4["layers"], "launch": args.launch, "flops_per_step": wl4.flops},
            "roofline": res4["roofline"],
            "cpu_baseline": None if args.no_cpu_baseline else cpu_baseline("C4"),
        }
    if args.all:
        others = {}
        for name in ["C1", "C2", "C3", "C4", "C5", "E4", "O1", "O5", "O4", "Q2", "Q6", "Q4", "Q3"]:
            if name == args.workload:
                continue
            _, res = run(name, seeded=name in ("C1", "C2"))
            others[name] = res
        line["workloads"] = others
    if args.calibrate_copy:
        src = torch.ones(32 << 20, dtype=torch.float16, device="cuda")  # 64 MiB read, 64 MiB written
        dst = torch.empty_like(src)
        for _ in range(10):
            torch.mul(src, 1.0, out=dst)
        torch.cuda.synchronize()
    line["cpu_baseline"] = None if args.no_cpu_baseline else cpu_baseline(
        args.workload, kv_bits=kv_bits_for(args.workload), window=args.window, weight_bits=args.weight_bits,
        keep_fraction=args.keep_fraction if args.keep_budget == 0 else 1.0)
    ctx.close()
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
