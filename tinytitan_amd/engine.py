"""Host-side mirror of the reference's attention operator interface, over the C ABI.

Names and argument meaning follow the Swift types this path replaces:

* ``KVCacheManager``   sources/TinyTitan/Runtime/KVCache/KVCacheManager.swift:62-333
* ``Attention``        sources/TinyTitan/Kernels/Attention/Attention.swift:270-307
* ``PrefillAttention`` sources/TinyTitan/Kernels/Attention/PrefillAttention.swift:5-55,165-258
* ``verify rows``      sources/TinyTitan/Runtime/Inference/RealForwardRunner+VerifyDecodeOrderAttention.swift:52-110
* ``QSAIndexer``       sources/TinyTitan/Kernels/Attention/QSAIndexer.swift, QSAIndexer+Scratch.swift
* ``QSAExactness``     sources/TinyTitan/Runtime/Family/QSAExactness.swift:22-65

Tensors are torch fp16 CUDA(HIP) tensors; torch is only the owner of device
memory here -- every computation happens inside libctinytitan_hip.so.  Swift
``throws`` / ``precondition`` failures surface as ``TinyTitanHIPError`` carrying
the ABI status code.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Optional, Sequence

import torch

from . import capi


class TinyTitanHIPError(RuntimeError):
    def __init__(self, status: int, where: str, detail: str = ""):
        self.status = status
        msg = f"{where}: {capi.strerror(status)} (status {status})"
        if detail:
            msg += f" [{detail}]"
        super().__init__(msg)


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    if t is None:
        return None
    if not t.is_cuda or t.dtype != torch.float16:
        raise TypeError("expected an fp16 device tensor")
    return t.data_ptr()


def _ptr_raw(t: torch.Tensor) -> int:
    """Device tensor passed as raw bytes (stored cache rows)."""
    if not t.is_cuda or not t.is_contiguous():
        raise TypeError("expected a contiguous device tensor")
    return t.data_ptr()


def _ptr16(t: torch.Tensor) -> int:
    """Device tensor of 16-bit elements passed as raw bit patterns (bfloat16 weights)."""
    if not t.is_cuda or t.element_size() != 2:
        raise TypeError("expected a device tensor of 16-bit elements")
    return t.data_ptr()


class HIPContext:
    """Owns the HIP stream, split-K scratch and timing events (``tt_hip_ctx``)."""

    def __init__(self, device: int = 0):
        err = ctypes.c_int(0)
        self._lib = capi.lib()
        self.handle = self._lib.tt_hip_ctx_create(device, ctypes.byref(err))
        if not self.handle:
            raise TinyTitanHIPError(err.value, "tt_hip_ctx_create")
        self.device = device

    def _check(self, status: int, where: str) -> None:
        if status != capi.OK:
            detail = self._lib.tt_hip_last_hip_error(self.handle).decode() if status == capi.ERR_HIP else ""
            raise TinyTitanHIPError(status, where, detail)

    def synchronize(self) -> None:
        self._check(self._lib.tt_hip_sync(self.handle), "tt_hip_sync")

    def set_stream(self, hip_stream: Optional[int]) -> None:
        self._check(self._lib.tt_hip_ctx_set_stream(self.handle, hip_stream), "tt_hip_ctx_set_stream")

    def use_torch_stream(self) -> None:
        """Enqueue on torch's current stream of this device (its default stream is HIP's null stream, handle 0)."""
        handle = torch.cuda.current_stream(self.device).cuda_stream
        if handle:
            self.set_stream(handle)
        else:
            self._check(self._lib.tt_hip_ctx_set_default_stream(self.handle), "tt_hip_ctx_set_default_stream")

    def timer_begin(self) -> None:
        self._check(self._lib.tt_hip_timer_begin(self.handle), "tt_hip_timer_begin")

    def timer_end_ns(self) -> int:
        ns = ctypes.c_uint64(0)
        self._check(self._lib.tt_hip_timer_end(self.handle, ctypes.byref(ns)), "tt_hip_timer_end")
        return ns.value

    def profile_enable(self, max_launches: int) -> None:
        self._check(self._lib.tt_hip_profile_enable(self.handle, max_launches), "tt_hip_profile_enable")

    def profile_disable(self) -> None:
        self._check(self._lib.tt_hip_profile_disable(self.handle), "tt_hip_profile_disable")

    def profile_read(self):
        """(launches, total_ns) of the dominant kernel since the last read."""
        n, ns = ctypes.c_int(0), ctypes.c_uint64(0)
        self._check(self._lib.tt_hip_profile_read(self.handle, ctypes.byref(n), ctypes.byref(ns)), "tt_hip_profile_read")
        return n.value, ns.value

    def profile_event_overhead_ns(self) -> int:
        ns = ctypes.c_uint64(0)
        self._check(self._lib.tt_hip_profile_event_overhead_ns(self.handle, ctypes.byref(ns)),
                    "tt_hip_profile_event_overhead_ns")
        return ns.value

    def calibrate_read(self, buf: torch.Tensor, offset_bytes: int = 0, nbytes: Optional[int] = None) -> int:
        """A plain streaming read of `buf` (the control a decode pass is compared with); returns the bytes read."""
        total = buf.numel() * buf.element_size()
        n = total - offset_bytes if nbytes is None else nbytes
        read = ctypes.c_size_t(0)
        self._check(self._lib.tt_hip_calibrate_read(self.handle, buf.data_ptr() + offset_bytes, n, None, ctypes.byref(read)),
                    "tt_hip_calibrate_read")
        return read.value

    def graph_begin(self) -> None:
        self._check(self._lib.tt_hip_graph_begin(self.handle), "tt_hip_graph_begin")

    def graph_end(self) -> "HIPGraph":
        g = ctypes.c_void_p(None)
        self._check(self._lib.tt_hip_graph_end(self.handle, ctypes.byref(g)), "tt_hip_graph_end")
        return HIPGraph(self, g)

    def set_split_tokens(self, tokens: int) -> None:
        self._check(self._lib.tt_hip_set_split_tokens(self.handle, tokens), "tt_hip_set_split_tokens")

    def set_option(self, option: int, value: int) -> None:
        """A kernel-variant switch (``capi.OPT_*``), cf. the reference's TINYTITAN_ATTN_* (Attention.swift:186-188)."""
        self._check(self._lib.tt_hip_set_option(self.handle, option, value), "tt_hip_set_option")

    def split_geometry(self, n_seq: int, n_q_heads: int, n_kv_heads: int, head_dim: int, rows: int, seq_len: int):
        """(split_tokens, splits, workgroups) -- cf. ``Attention.splitGeometry`` (Attention.swift:202-227)."""
        a, b, c = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
        self._check(self._lib.tt_hip_split_geometry(self.handle, n_seq, n_q_heads, n_kv_heads, head_dim, rows,
                                                    seq_len, ctypes.byref(a), ctypes.byref(b), ctypes.byref(c)),
                    "tt_hip_split_geometry")
        return a.value, b.value, c.value

    def close(self) -> None:
        if getattr(self, "handle", None):
            self._lib.tt_hip_ctx_destroy(self.handle)
            self.handle = None

    def __del__(self):  # pragma: no cover - best effort
        try:
            self.close()
        except Exception:
            pass


class HIPGraph:
    """A captured sequence of calls (``tt_hip_graph``); ``launch`` replays it on the context's stream."""

    def __init__(self, ctx: HIPContext, handle):
        self.ctx, self.handle = ctx, handle

    def launch(self) -> None:
        self.ctx._check(self.ctx._lib.tt_hip_graph_launch(self.ctx.handle, self.handle), "tt_hip_graph_launch")

    def close(self) -> None:
        if self.handle:
            self.ctx._lib.tt_hip_graph_destroy(self.handle)
            self.handle = None


def kv_row_layout(elements: int, bits: int):
    """``KVCacheManager.rowLayout`` (KVCacheManager+Validation.swift:30-41): (stride, value_bytes) in bytes."""
    stride, values = ctypes.c_size_t(0), ctypes.c_size_t(0)
    status = capi.lib().tt_hip_kv_row_layout(elements, bits, ctypes.byref(stride), ctypes.byref(values))
    if status != capi.OK:
        raise TinyTitanHIPError(status, "tt_hip_kv_row_layout")
    return stride.value, values.value


class KVCacheManager:
    """KV cache in HBM: per-layer stores, a region per slot, a cursor per slot.  ``precision_bits`` 16 keeps
    fp16 values, 8 / 4 the reference's affine levels with a scale and a bias per token and group of 64."""

    def __init__(self, ctx: HIPContext, layers: int, kv_heads: int, head_dim: int, slots: int = 1,
                 max_context: int = 262144, initial_capacity: Optional[int] = None, precision_bits: int = 16,
                 ring_capacity: int = 0):
        """``ring_capacity`` > 0: a ring for sliding-window layers (row of position p at p % capacity)."""
        self.ctx = ctx
        self._lib = ctx._lib
        if initial_capacity is None:
            initial_capacity = min(max_context, 8192)  # KVCacheManager.swift:270-285
        err = ctypes.c_int(0)
        if ring_capacity > 0:
            self.handle = self._lib.tt_hip_kv_create_ring(ctx.handle, layers, kv_heads, head_dim, slots, ring_capacity,
                                                          max_context, precision_bits, ctypes.byref(err))
        else:
            self.handle = self._lib.tt_hip_kv_create_quantized(ctx.handle, layers, kv_heads, head_dim, slots,
                                                               initial_capacity, max_context, precision_bits, ctypes.byref(err))
        if not self.handle:
            raise TinyTitanHIPError(err.value, "tt_hip_kv_create_ring" if ring_capacity > 0 else "tt_hip_kv_create_quantized")
        self.layers, self.kv_heads, self.head_dim, self.slots = layers, kv_heads, head_dim, slots
        self.precision_bits = precision_bits

    # -- bookkeeping ---------------------------------------------------------
    @property
    def capacity_tokens(self) -> int:
        return self._lib.tt_hip_kv_capacity(self.handle)

    @property
    def max_context(self) -> int:
        return self._lib.tt_hip_kv_max_context(self.handle)

    @property
    def token_stride_bytes(self) -> int:
        return self._lib.tt_hip_kv_token_stride_bytes(self.handle)

    @property
    def bytes(self) -> int:
        return self._lib.tt_hip_kv_bytes(self.handle)

    def position(self, slot: int = 0) -> int:
        p = self._lib.tt_hip_kv_position(self.handle, slot)
        if p < 0:
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "tt_hip_kv_position")
        return p

    def advance(self, slot: int = 0, by: int = 1) -> None:
        self.ctx._check(self._lib.tt_hip_kv_advance(self.handle, slot, by), "tt_hip_kv_advance")

    def rewind(self, slot: int, to: int) -> None:
        self.ctx._check(self._lib.tt_hip_kv_rewind(self.handle, slot, to), "tt_hip_kv_rewind")

    def reset(self, slot: int = -1) -> None:
        self.ctx._check(self._lib.tt_hip_kv_reset(self.handle, slot), "tt_hip_kv_reset")

    def reserve(self, tokens: int) -> None:
        self.ctx._check(self._lib.tt_hip_kv_reserve(self.handle, tokens), "tt_hip_kv_reserve")

    def expect_position(self, slot: int, position: int) -> None:
        self.ctx._check(self._lib.tt_hip_kv_expect_position(self.handle, slot, position), "tt_hip_kv_expect_position")

    # -- rows ----------------------------------------------------------------
    def append(self, layer: int, slot: int, position: int, k: torch.Tensor, v: torch.Tensor,
               token_stride: Optional[int] = None, n_tokens: Optional[int] = None) -> None:
        """Write token-major rows ``[n_tokens][kv_heads*head_dim]`` at ``[position, position+n)``."""
        width = self.kv_heads * self.head_dim
        if n_tokens is None:
            n_tokens = k.numel() // width
        if token_stride is None:
            token_stride = width
        self.ctx._check(self._lib.tt_hip_kv_append(self.handle, layer, slot, position, n_tokens, _ptr(k), _ptr(v),
                                                   token_stride), "tt_hip_kv_append")

    def export_rows(self, layer: int, slot: int, position: int, n_tokens: int):
        """K and V rows in the stored row format, ``[n_tokens][token_stride_bytes]`` uint8 each."""
        dev = torch.device("cuda", self.ctx.device)
        stride = self.token_stride_bytes
        k = torch.zeros((n_tokens, stride), dtype=torch.uint8, device=dev)
        v = torch.zeros_like(k)
        torch.cuda.synchronize(dev)
        self.ctx._check(self._lib.tt_hip_kv_export_rows(self.handle, layer, slot, position, n_tokens, _ptr_raw(k),
                                                        _ptr_raw(v), stride), "tt_hip_kv_export_rows")
        self.ctx.synchronize()
        return k, v

    def import_rows(self, layer: int, slot: int, position: int, k_rows: torch.Tensor, v_rows: torch.Tensor) -> None:
        """Write stored rows (as ``export_rows`` returns them) at ``[position, position + n)``, as they are."""
        n_tokens, stride = k_rows.shape
        self.ctx._check(self._lib.tt_hip_kv_import_rows(self.handle, layer, slot, position, n_tokens, _ptr_raw(k_rows),
                                                        _ptr_raw(v_rows), stride), "tt_hip_kv_import_rows")

    def read(self, layer: int, slot: int, position: int, n_tokens: int):
        """Token-major copies ``[n_tokens][kv_heads][head_dim]`` of K and V rows (dequantised when the cache is)."""
        dev = torch.device("cuda", self.ctx.device)
        k = torch.empty((n_tokens, self.kv_heads, self.head_dim), dtype=torch.float16, device=dev)
        v = torch.empty_like(k)
        torch.cuda.synchronize(dev)
        self.ctx._check(self._lib.tt_hip_kv_read(self.handle, layer, slot, position, n_tokens, _ptr(k), _ptr(v),
                                                 self.kv_heads * self.head_dim), "tt_hip_kv_read")
        self.ctx.synchronize()
        return k, v

    def gather(self, layer: int, slot: int, positions: torch.Tensor, k_out: torch.Tensor, v_out: torch.Tensor) -> None:
        """Rows of the listed positions (an int32 device tensor) into token-major ``k_out`` / ``v_out``
        ``[n][kv_heads * head_dim]``: the compacted form of a sparse selection (``DecodeKeySelection.indices``),
        to be appended into a scratch cache and attended densely.  Enqueued on the context's stream."""
        if positions.dtype != torch.int32 or not positions.is_cuda or not positions.is_contiguous():
            raise TypeError("expected a contiguous int32 device tensor of positions")
        self.ctx._check(self._lib.tt_hip_kv_gather(self.handle, layer, slot, positions.data_ptr(), positions.numel(),
                                                   _ptr(k_out), _ptr(v_out), k_out.stride(0)), "tt_hip_kv_gather")

    # ---- inference-state snapshots (KVCacheManager+Snapshot.swift:12-118) ----

    def snapshot_segment_lengths(self, position: int):
        import ctypes
        n = self._lib.tt_hip_kv_snapshot_segment_count(self.handle)
        arr = (ctypes.c_size_t * n)()
        self.ctx._check(self._lib.tt_hip_kv_snapshot_segment_lengths(self.handle, position, arr, n),
                        "tt_hip_kv_snapshot_segment_lengths")
        return list(arr)

    def append_snapshot_payload(self, payload: bytearray, segment_lengths) -> None:
        """Appends slot 0's rows (token-major K then V per layer) to ``payload``."""
        import ctypes
        n = len(segment_lengths)
        arr = (ctypes.c_size_t * n)(*segment_lengths)
        total = sum(segment_lengths)
        buf = (ctypes.c_char * max(total, 1))()
        off = ctypes.c_size_t(0)
        self.ctx._check(self._lib.tt_hip_kv_snapshot_export(self.handle, arr, n, ctypes.addressof(buf), total,
                                                            ctypes.byref(off)), "tt_hip_kv_snapshot_export")
        payload += bytes(buf[:off.value])

    def restore_snapshot(self, position: int, segment_lengths, data: bytes, offset: int = 0) -> int:
        """Returns the offset behind the consumed bytes."""
        import ctypes
        n = len(segment_lengths)
        arr = (ctypes.c_size_t * n)(*segment_lengths)
        src = ctypes.create_string_buffer(bytes(data), len(data)) if len(data) else None
        off = ctypes.c_size_t(offset)
        self.ctx._check(self._lib.tt_hip_kv_snapshot_restore(self.handle, position, arr, n,
                                                             ctypes.addressof(src) if src is not None else None, len(data),
                                                             ctypes.byref(off)), "tt_hip_kv_snapshot_restore")
        return off.value

    def close(self) -> None:
        if getattr(self, "handle", None):
            self._lib.tt_hip_kv_destroy(self.handle)
            self.handle = None

    def __del__(self):  # pragma: no cover
        try:
            self.close()
        except Exception:
            pass


class Attention:
    """Decode attention over the cache (``Attention.encodeFull`` + the sigmoid gate pass)."""

    def __init__(self, ctx: HIPContext):
        self.ctx = ctx
        self._lib = ctx._lib

    def encode_full(self, kv: KVCacheManager, layer: int, q: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                    seq_len, scale: float, slot=0, gate: Optional[torch.Tensor] = None) -> None:
        """``seq_len`` is the exclusive key count (position + 1).  ``slot``/``seq_len`` may be
        lists for the batched form (one query token per sequence)."""
        slots = list(slot) if isinstance(slot, (list, tuple)) else [slot]
        lens = list(seq_len) if isinstance(seq_len, (list, tuple)) else [seq_len]
        if len(slots) != len(lens):
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "Attention.encode_full")
        self.ctx._check(self._lib.tt_hip_attn_decode(self.ctx.handle, kv.handle, layer, len(slots),
                                                     capi.int_array(slots), capi.int_array(lens), num_q_heads,
                                                     _ptr(q), _ptr(gate), scale, _ptr(out)), "tt_hip_attn_decode")

    def encode_swa(self, kv: KVCacheManager, layer: int, q: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                   seq_len, window: int, scale: float, slot=0, gate: Optional[torch.Tensor] = None) -> None:
        """``Attention.encodeSWA`` (Attention.swift:229-266): keys ``[max(0, seq_len - window), seq_len)``."""
        slots = list(slot) if isinstance(slot, (list, tuple)) else [slot]
        lens = list(seq_len) if isinstance(seq_len, (list, tuple)) else [seq_len]
        if len(slots) != len(lens):
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "Attention.encode_swa")
        self.ctx._check(self._lib.tt_hip_attn_decode_swa(self.ctx.handle, kv.handle, layer, len(slots),
                                                         capi.int_array(slots), capi.int_array(lens), window, num_q_heads,
                                                         _ptr(q), _ptr(gate), scale, _ptr(out)), "tt_hip_attn_decode_swa")

    def encode_full_keep(self, kv: KVCacheManager, layer: int, q: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                         seq_len, keep_mask: torch.Tensor, scale: float, slot=0, gate: Optional[torch.Tensor] = None,
                         keep_stride: Optional[int] = None) -> None:
        """``Attention.encodeFull(..., keepMask:)``: ``keep_mask`` is a uint8 device tensor, one byte per key
        position (0 drops the key); for several sequences their masks are ``keep_stride`` bytes apart."""
        slots = list(slot) if isinstance(slot, (list, tuple)) else [slot]
        lens = list(seq_len) if isinstance(seq_len, (list, tuple)) else [seq_len]
        if len(slots) != len(lens) or keep_mask.dtype != torch.uint8:
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "Attention.encode_full_keep")
        self.ctx._check(self._lib.tt_hip_attn_decode_keep(self.ctx.handle, kv.handle, layer, len(slots),
                                                          capi.int_array(slots), capi.int_array(lens), _ptr_raw(keep_mask),
                                                          keep_stride if keep_stride is not None else max(lens),
                                                          num_q_heads, _ptr(q), _ptr(gate), scale, _ptr(out)),
                        "tt_hip_attn_decode_keep")

    def encode_full_keep_indices(self, kv: KVCacheManager, layer: int, q: torch.Tensor, out: torch.Tensor, num_q_heads: int,
                                 seq_len, keep_indices: torch.Tensor, keep_counts: torch.Tensor, scale: float, slot=0,
                                 gate: Optional[torch.Tensor] = None, keep_index_stride: Optional[int] = None) -> None:
        """The same selection compacted (``DecodeKeySelection.indices`` / ``.count``): int32 device tensors, per
        sequence a list of key ids ``keep_index_stride`` entries apart and how many of them count."""
        slots = list(slot) if isinstance(slot, (list, tuple)) else [slot]
        lens = list(seq_len) if isinstance(seq_len, (list, tuple)) else [seq_len]
        if len(slots) != len(lens) or keep_indices.dtype != torch.int32 or keep_counts.dtype != torch.int32:
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "Attention.encode_full_keep_indices")
        self.ctx._check(self._lib.tt_hip_attn_decode_keep_indices(
            self.ctx.handle, kv.handle, layer, len(slots), capi.int_array(slots), capi.int_array(lens), _ptr_raw(keep_indices),
            keep_index_stride if keep_index_stride is not None else keep_indices.shape[-1], _ptr_raw(keep_counts), num_q_heads,
            _ptr(q), _ptr(gate), scale, _ptr(out)), "tt_hip_attn_decode_keep_indices")

    def encode_verify_rows(self, kv: KVCacheManager, layer: int, q: torch.Tensor, out: torch.Tensor,
                           num_q_heads: int, start_positions: Sequence[int], rows: int, scale: float,
                           slots: Sequence[int], gate: Optional[torch.Tensor] = None, window: int = 0) -> None:
        """Row r of sequence i attends like a decode at ``start_positions[i] + r`` (over its last ``window`` keys)."""
        self.ctx._check(self._lib.tt_hip_attn_verify_swa(self.ctx.handle, kv.handle, layer, len(slots),
                                                         capi.int_array(slots), capi.int_array(start_positions), rows,
                                                         window, num_q_heads, _ptr(q), _ptr(gate), scale, _ptr(out)),
                        "tt_hip_attn_verify_swa")


@dataclass
class PrefillAttentionParams:
    """``PrefillAttentionParams`` (PrefillAttention.swift:5-55); strides in elements."""
    start_position: int
    query_count: int
    kv_valid_count: int
    num_q_heads: int
    scale: float
    q_stride: int
    o_stride: int
    gate_stride: int = 0
    sliding_window: int = 0  # 0: every key up to the row's own


class PrefillAttention:
    def __init__(self, ctx: HIPContext):
        self.ctx = ctx
        self._lib = ctx._lib

    def encode_causal(self, kv: KVCacheManager, layer: int, slot: int, q: torch.Tensor, out: torch.Tensor,
                      params: PrefillAttentionParams, gate: Optional[torch.Tensor] = None,
                      keep_mask: Optional[torch.Tensor] = None, keep_stride: int = 0,
                      keep_indices: Optional[torch.Tensor] = None, keep_index_stride: int = 0,
                      keep_counts: Optional[torch.Tensor] = None) -> None:
        """``keep_mask`` / ``keep_stride``: a QSA chunk's per-query selection in its mask form (one row of
        ``keep_stride`` bytes per query, a zero byte drops that key for that query).  ``keep_indices`` /
        ``keep_index_stride`` / ``keep_counts``: the same selection compacted (int32 key ids per query and how
        many of them), as ``encodeCausal`` takes it for the tiled kernel."""
        p = params
        if keep_indices is not None:
            if (keep_counts is None or keep_mask is not None or p.sliding_window or keep_indices.dtype != torch.int32
                    or keep_counts.dtype != torch.int32):
                raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "PrefillAttention.encode_causal")
            self.ctx._check(self._lib.tt_hip_attn_prefill_keep_indices(
                self.ctx.handle, kv.handle, layer, slot, p.start_position, p.query_count, p.kv_valid_count,
                _ptr_raw(keep_indices), keep_index_stride or keep_indices.shape[-1], _ptr_raw(keep_counts), p.num_q_heads,
                _ptr(q), p.q_stride, _ptr(gate), p.gate_stride or p.q_stride, p.scale, _ptr(out), p.o_stride),
                "tt_hip_attn_prefill_keep_indices")
            return
        if keep_mask is not None:
            if keep_mask.dtype != torch.uint8 or p.sliding_window:
                raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "PrefillAttention.encode_causal")
            self.ctx._check(self._lib.tt_hip_attn_prefill_keep(
                self.ctx.handle, kv.handle, layer, slot, p.start_position, p.query_count, p.kv_valid_count,
                _ptr_raw(keep_mask), keep_stride or keep_mask.shape[-1], p.num_q_heads, _ptr(q), p.q_stride, _ptr(gate),
                p.gate_stride or p.q_stride, p.scale, _ptr(out), p.o_stride), "tt_hip_attn_prefill_keep")
            return
        if p.sliding_window:
            self.ctx._check(self._lib.tt_hip_attn_prefill_swa(self.ctx.handle, kv.handle, layer, slot, p.start_position,
                                                              p.query_count, p.kv_valid_count, p.sliding_window,
                                                              p.num_q_heads, _ptr(q), p.q_stride, _ptr(gate),
                                                              p.gate_stride or p.q_stride, p.scale, _ptr(out), p.o_stride),
                            "tt_hip_attn_prefill_swa")
            return
        self.ctx._check(self._lib.tt_hip_attn_prefill(self.ctx.handle, kv.handle, layer, slot, p.start_position,
                                                      p.query_count, p.kv_valid_count, p.num_q_heads, _ptr(q),
                                                      p.q_stride, _ptr(gate), p.gate_stride or p.q_stride, p.scale,
                                                      _ptr(out), p.o_stride), "tt_hip_attn_prefill")


class QKVEpilogue:
    """Split [query ; gate], per-head q/k RMS norms, NeoX sub-dim RoPE and the K/V cache write in one
    launch: ``encodeGatedFullPostProjection`` (RealForwardRunner+DecodeFullAttention.swift:123-185)
    for decode / verify rows, ``PrefillQKVEpilogue.encodeNeoxSubdimNoVNorm`` + ``copyPrefillKVToCache``
    for a chunk.  Norm weights are bfloat16 bit patterns (``torch.bfloat16`` or ``int16``/``uint16``)."""

    def __init__(self, ctx: HIPContext):
        self.ctx = ctx
        self._lib = ctx._lib

    def encode(self, kv: KVCacheManager, layer: int, q_packed: torch.Tensor, k_proj: torch.Tensor,
               v_proj: torch.Tensor, q_norm_weight: torch.Tensor, k_norm_weight: torch.Tensor, q_out: torch.Tensor,
               gate_out: torch.Tensor, num_q_heads: int, positions, rows: int, eps: float, rotary_dim: int,
               theta: float, slots=0, q_packed_stride: Optional[int] = None, kv_stride: Optional[int] = None,
               q_stride: Optional[int] = None, gate_stride: Optional[int] = None) -> None:
        """Token ``i * rows + r`` of sequence ``i`` sits at ``positions[i] + r`` of ``slots[i]``."""
        slot_list = list(slots) if isinstance(slots, (list, tuple)) else [slots]
        pos_list = list(positions) if isinstance(positions, (list, tuple)) else [positions]
        if len(slot_list) != len(pos_list):
            raise TinyTitanHIPError(capi.ERR_INVALID_ARGUMENT, "QKVEpilogue.encode")
        width = num_q_heads * kv.head_dim
        self.ctx._check(self._lib.tt_hip_qkv_epilogue_append(
            self.ctx.handle, kv.handle, layer, len(slot_list), capi.int_array(slot_list), capi.int_array(pos_list), rows,
            num_q_heads, _ptr(q_packed), q_packed_stride or 2 * width, _ptr(k_proj), _ptr(v_proj),
            kv_stride or kv.kv_heads * kv.head_dim, _ptr16(q_norm_weight), _ptr16(k_norm_weight), eps, rotary_dim, theta,
            _ptr(q_out), q_stride or width, _ptr(gate_out), gate_stride or width), "tt_hip_qkv_epilogue_append")


class AffineProjection:
    """``y[t] = W x[t]`` over affine-quantised weights (4 or 8 bits, bfloat16 scale and bias per group of
    64 columns): ``RealForwardRunner.encodeAffineProjection`` for o_proj
    (RealForwardRunner+PrefillProjection.swift:53-66) and the decode GEMVs behind the gate
    (``DequantInt4GEMV.encode`` / ``encodeTwoRows``, DequantInt4GEMV.swift:72-143).
    ``weights`` is a uint8 device tensor ``[rows][columns * bits / 8]``; ``scales`` / ``biases`` hold
    bfloat16 bit patterns ``[rows][columns / 64]``."""

    def __init__(self, ctx: HIPContext):
        self.ctx = ctx
        self._lib = ctx._lib

    def encode(self, weight_bits: int, weights: torch.Tensor, scales: torch.Tensor, biases: torch.Tensor,
               x: torch.Tensor, y: torch.Tensor, rows: int, columns: int, token_count: int,
               x_stride: Optional[int] = None, y_stride: Optional[int] = None, weights_offset: int = 0) -> None:
        """``weights_offset`` is a byte offset into ``weights`` (the reference binds tensors at offsets
        into one buffer)."""
        self.ctx._check(self._lib.tt_hip_affine_projection(
            self.ctx.handle, weight_bits, _ptr_raw(weights) + weights_offset, _ptr16(scales), _ptr16(biases), _ptr(x),
            _ptr(y), rows, columns, token_count, x_stride or columns, y_stride or rows), "tt_hip_affine_projection")


@dataclass(frozen=True)
class QSAExactness:
    """When dense attention equals the sparse selection (QSAExactness.swift:22-65): the indexer keeps
    ``budget / compress_ratio`` complete blocks and always the incomplete tail block."""
    budget: int
    compress_ratio: int

    def __post_init__(self):
        if self.budget <= 0 or self.compress_ratio <= 0:
            raise ValueError("budget and compress_ratio must be positive")

    @property
    def kept_blocks(self) -> int:
        return self.budget // self.compress_ratio

    @property
    def maximum_exact_visible_keys(self) -> int:
        return self.kept_blocks * self.compress_ratio + (self.compress_ratio - 1)

    def is_dense_exact(self, visible_keys: int) -> bool:
        if visible_keys < 0:
            raise ValueError("visible_keys must not be negative")
        return visible_keys // self.compress_ratio <= self.kept_blocks

    def is_dense_exact_for_context(self, tokens: int) -> bool:
        return tokens <= 0 or self.is_dense_exact(tokens)

    @property
    def indexer_required_from_context(self) -> int:
        return self.maximum_exact_visible_keys + 1


class QSAIndexerRequired(RuntimeError):
    """A context outgrew the dense-exact window and no indexer was built (QSAExactness.swift:73-92)."""

    def __init__(self, visible_keys: int, exact_window: int):
        self.visible_keys, self.exact_window = visible_keys, exact_window
        super().__init__(
            f"context reaches {visible_keys} tokens, past the {exact_window} where dense attention matches this "
            "model's sparse selection exactly. This model's QSA indexer was not built, and running dense here would "
            "attend to keys the model would have dropped -- silently, and with plausible output. Check the load "
            "diagnostics for the indexer, or shorten the prompt or lower --max-new so prompt + generation stays "
            f"within {exact_window}.")


@dataclass
class QSASelection:
    """What ``select_keys_prefill`` hands the attention (QSASelection in QSAIndexer.swift:493-497): the byte mask,
    one row of ``mask_stride`` per query, and the ascending index list with its counts."""
    mask: Optional[torch.Tensor]
    mask_stride: int
    indices: torch.Tensor
    index_stride: int
    counts: torch.Tensor


class QSAIndexer:
    """The sparse attention's block indexer (QSAIndexer.swift:24-110): per layer a cache of raw indexer keys
    ``[capacity][head_dim]`` (before norm and rotation) and of pooled blocks
    ``[capacity / compress_ratio + 1][head_dim]`` (after them); scores of pooled blocks against the indexer's
    query heads; the selection.  The projections that produce raw keys and query rows are the caller's
    (``AffineProjection`` serves them); rows arrive here as fp16 tensors."""

    def __init__(self, ctx: HIPContext, heads: int, head_dim: int, compress_ratio: int, budget: int, rope_theta: float,
                 capacity: int):
        if capacity <= 0:
            raise ValueError("capacity must be positive")
        self.ctx, self._lib = ctx, ctx._lib
        self.heads, self.head_dim, self.compress_ratio, self.budget = heads, head_dim, compress_ratio, budget
        self.rope_theta, self.capacity = rope_theta, capacity
        self.exactness = QSAExactness(budget, compress_ratio)
        self.device = torch.device("cuda", ctx.device)
        self.raw_keys: dict = {}
        self.pooled: dict = {}
        self.scores_buf = torch.zeros(max(1, capacity // compress_ratio + 1), dtype=torch.float32, device=self.device)
        self.keep_buf = torch.zeros(capacity, dtype=torch.uint8, device=self.device)
        self.keep_index_buf: Optional[torch.Tensor] = None
        self.keep_count_buf: Optional[torch.Tensor] = None
        self.scored_blocks_per_row = 0

    @property
    def selection_width(self) -> int:
        """Cells a query keeps: the budget plus the tail block's extra members (QSAIndexer.swift:91)."""
        return self.budget + self.compress_ratio - 1

    def reset(self) -> None:
        self.raw_keys.clear()
        self.pooled.clear()

    def layer_buffers(self, layer: int):
        if layer not in self.raw_keys:
            self.raw_keys[layer] = torch.zeros(self.capacity, self.head_dim, dtype=torch.float16, device=self.device)
            self.pooled[layer] = torch.zeros(self.capacity // self.compress_ratio + 1, self.head_dim,
                                             dtype=torch.float16, device=self.device)
        return self.raw_keys[layer], self.pooled[layer]

    def raw_key_destination(self, layer: int, start_position: int, tokens: int) -> torch.Tensor:
        """The raw-key cache rows a chunk's key projection writes into (QSAIndexer.swift:236-245)."""
        if start_position + tokens > self.capacity:
            raise ValueError(f"QSA indexer capacity {self.capacity} exceeded at {start_position + tokens}")
        return self.layer_buffers(layer)[0][start_position:start_position + tokens]

    def encode_pool_prefill(self, layer: int, start_position: int, tokens: int, key_norm: torch.Tensor,
                            eps: float) -> None:
        """Repools every block a chunk touched, then norm and rotation at ``block * compress_ratio``
        (QSAIndexer.swift:196-233).  One token is ``encodeAppendKey``'s repooling (QSAIndexer+Scratch.swift:88-110)."""
        end = start_position + tokens
        if end > self.capacity:
            raise ValueError(f"QSA indexer capacity {self.capacity} exceeded at {end}")
        raw, pooled = self.layer_buffers(layer)
        first_block = start_position // self.compress_ratio
        block_count = (end - 1) // self.compress_ratio - first_block + 1
        self.ctx._check(self._lib.tt_hip_qsa_pool_blocks(
            self.ctx.handle, _ptr(raw), _ptr(pooled), self.head_dim, first_block, block_count, self.compress_ratio, end,
            _ptr16(key_norm), eps, self.rope_theta), "tt_hip_qsa_pool_blocks")

    def encode_scores(self, layer: int, query_rows: torch.Tensor, query_norm: torch.Tensor, start_position: int,
                      tokens: int, eps: float) -> torch.Tensor:
        """Norm and rotation of the projected query rows ``[tokens][heads][head_dim]`` (in place), then the
        scores of every block up to the last query's (``encodeScores``, QSAIndexer.swift:271-330, for one token;
        ``encodeScoresPrefill``, :332-403, for a chunk).  Returns the scores ``[tokens][blocks]``."""
        _, pooled = self.layer_buffers(layer)
        self.ctx._check(self._lib.tt_hip_qsa_norm_rope_rows(
            self.ctx.handle, _ptr(query_rows), tokens, self.heads, self.head_dim, _ptr16(query_norm), eps,
            self.rope_theta, start_position, 1), "tt_hip_qsa_norm_rope_rows")
        blocks = (start_position + tokens - 1) // self.compress_ratio + 1
        if self.scores_buf.numel() < blocks * tokens:
            self.scores_buf = torch.zeros(blocks * tokens, dtype=torch.float32, device=self.device)
        self.ctx._check(self._lib.tt_hip_qsa_block_scores(
            self.ctx.handle, _ptr(query_rows), _ptr(pooled), self.scores_buf.data_ptr(), blocks, self.head_dim,
            self.heads, blocks, tokens), "tt_hip_qsa_block_scores")
        self.scored_blocks_per_row = blocks
        return self.scores_buf[:blocks * tokens].view(tokens, blocks)

    def encode_decode_step(self, layer: int, position: int, query_rows: torch.Tensor, key_norm: torch.Tensor,
                           query_norm: torch.Tensor, eps: float) -> torch.Tensor:
        """One decode step's repooling, query norm and rotation, and block scores in a single launch: the token at
        ``position`` (its raw key already in the cache) -- ``encodeAppendKey``'s repooling
        (QSAIndexer+Scratch.swift:88-110) and ``encodeScores`` (QSAIndexer.swift:271-330).  ``query_rows``
        ``[heads][head_dim]`` is read only.  Returns the scores ``[1][blocks]``, bit for bit those of
        ``encode_pool_prefill(layer, position, 1, ...)`` + ``encode_scores(layer, ..., position, 1, ...)``."""
        if position + 1 > self.capacity:
            raise ValueError(f"QSA indexer capacity {self.capacity} exceeded at {position + 1}")
        raw, pooled = self.layer_buffers(layer)
        blocks = position // self.compress_ratio + 1
        if self.scores_buf.numel() < blocks:
            self.scores_buf = torch.zeros(blocks, dtype=torch.float32, device=self.device)
        self.ctx._check(self._lib.tt_hip_qsa_decode_scores(
            self.ctx.handle, _ptr(raw), _ptr(pooled), self.head_dim, self.compress_ratio, position + 1, _ptr16(key_norm),
            _ptr(query_rows), self.heads, _ptr16(query_norm), position, eps, self.rope_theta, self.scores_buf.data_ptr()),
            "tt_hip_qsa_decode_scores")
        self.scored_blocks_per_row = blocks
        return self.scores_buf[:blocks].view(1, blocks)

    def _select(self, rows: int, first_visible: int, score_stride: int, keep_stride: int, compact: bool,
                mask: bool = True) -> None:
        width = self.selection_width
        if not mask and not compact:
            raise ValueError("a selection is a mask, an index list or both")
        if mask and self.keep_buf.numel() < keep_stride * rows:
            self.keep_buf = torch.zeros(keep_stride * rows, dtype=torch.uint8, device=self.device)
        if compact and (self.keep_index_buf is None or self.keep_index_buf.numel() < rows * width):
            self.keep_index_buf = torch.zeros(rows * width, dtype=torch.int32, device=self.device)
        if compact and (self.keep_count_buf is None or self.keep_count_buf.numel() < rows):
            self.keep_count_buf = torch.zeros(rows, dtype=torch.int32, device=self.device)
        self.ctx._check(self._lib.tt_hip_qsa_select(
            self.ctx.handle, self.scores_buf.data_ptr(), score_stride, rows, first_visible, self.compress_ratio, width,
            self.keep_buf.data_ptr() if mask else None, keep_stride, self.keep_index_buf.data_ptr() if compact else None, width,
            self.keep_count_buf.data_ptr() if compact else None), "tt_hip_qsa_select")

    def select_keys(self, visible_keys: int) -> Optional[torch.Tensor]:
        """The decode step's byte mask over ``visible_keys`` cells, or None when everything visible is kept
        (``selectKeys`` / ``encodeSelectKeys``, QSAIndexer+Scratch.swift:228-284)."""
        if visible_keys <= self.selection_width:
            return None
        self._select(1, visible_keys, self.scores_buf.numel(), (visible_keys + 3) // 4 * 4, False)
        return self.keep_buf

    def select_keys_compact(self, visible_keys: int):
        """``(mask, indices, count)``: the mask and the ascending index list of one decode step; inside the dense
        window ``(None, None, visible_keys)`` (``selectKeysCompact``, QSAIndexer+Scratch.swift:191-217)."""
        if visible_keys <= self.selection_width:
            return None, None, visible_keys
        self._select(1, visible_keys, self.scores_buf.numel(), (visible_keys + 3) // 4 * 4, True)
        return self.keep_buf, self.keep_index_buf, int(self.keep_count_buf[0].item())

    def select_keys_prefill(self, start_position: int, tokens: int, mask: bool = True) -> Optional[QSASelection]:
        """The chunk's selection -- one mask row and one index row per query -- or None when every query of the
        chunk is inside the dense-exact window (``selectKeysPrefill``, QSAIndexer.swift:414-497).  ``mask=False``
        leaves the mask rows out (``QSASelection.mask`` is None): the attention's index-list form needs none, and
        they are ``tokens x context`` bytes where the lists are ``tokens x width`` words."""
        last_visible = start_position + tokens
        if last_visible <= self.selection_width:
            return None
        stride = (last_visible + 3) // 4 * 4  # the attention reads a row's mask four bytes at a time
        self._select(tokens, start_position + 1, self.scored_blocks_per_row, stride, True, mask=mask)
        return QSASelection(self.keep_buf if mask else None, stride, self.keep_index_buf, self.selection_width,
                            self.keep_count_buf)

    # --- auxiliary state of a restored prefix (QSAIndexer+State.swift:11-113) ----------------------------

    def append_snapshot_payload(self, payload: bytearray, position: int) -> None:
        """Appends what a restored prefix of ``position`` tokens needs, in the reference's wire format: u32 layer
        count; per layer (ascending) u32 layer, u32 blocks, u32 tail, the pooled blocks ``[blocks][head_dim]`` fp16,
        then the raw keys of the last, possibly partial, block ``[tail][head_dim]`` fp16 (all little endian).  Raw
        keys of earlier blocks are not needed: a block is pooled when its last member arrives and never read raw again."""
        if position <= 0 or position > self.capacity:
            raise ValueError(f"QSA position {position} outside 1...{self.capacity}")
        layers = sorted(self.pooled.keys())
        payload += int(len(layers)).to_bytes(4, "little")
        blocks = (position + self.compress_ratio - 1) // self.compress_ratio
        tail = position - (blocks - 1) * self.compress_ratio
        self.ctx.synchronize()
        for layer in layers:
            raw, pooled = self.raw_keys[layer], self.pooled[layer]
            for value in (layer, blocks, tail):
                payload += int(value).to_bytes(4, "little")
            payload += pooled[:blocks].cpu().numpy().tobytes()
            first = (blocks - 1) * self.compress_ratio
            payload += raw[first:first + tail].cpu().numpy().tobytes()

    def restore_snapshot_payload(self, data: bytes, offset: int, position: int) -> int:
        """Restores what ``append_snapshot_payload`` wrote; returns the offset behind it.  Raises ``ValueError`` on a
        truncated payload or one that covers other blocks than ``position`` implies (the reference's ``malformed``)."""
        if position <= 0:
            raise ValueError("QSA restore needs a positive position")
        import numpy as np

        def u32() -> int:
            nonlocal offset
            if offset + 4 > len(data):
                raise ValueError(f"QSA payload truncated at {offset}")
            value = int.from_bytes(data[offset:offset + 4], "little")
            offset += 4
            return value

        expected_blocks = (position + self.compress_ratio - 1) // self.compress_ratio
        expected_tail = position - (expected_blocks - 1) * self.compress_ratio
        row = self.head_dim * 2
        for _ in range(u32()):
            layer, blocks, tail = u32(), u32(), u32()
            if blocks != expected_blocks or tail != expected_tail:
                raise ValueError(f"QSA layer {layer} covers {blocks}/{tail} blocks/tail, expected "
                                 f"{expected_blocks}/{expected_tail}")
            pooled_bytes, raw_bytes = blocks * row, tail * row
            if offset + pooled_bytes + raw_bytes > len(data):
                raise ValueError(f"QSA layer {layer} payload truncated")
            if position > self.capacity:
                raise ValueError(f"QSA layer {layer} live buffers are too small")
            raw, pooled = self.layer_buffers(layer)
            rows = np.frombuffer(data, dtype=np.float16, count=blocks * self.head_dim, offset=offset)
            pooled[:blocks].copy_(torch.from_numpy(rows.reshape(blocks, self.head_dim).copy()))
            offset += pooled_bytes
            rows = np.frombuffer(data, dtype=np.float16, count=tail * self.head_dim, offset=offset)
            first = (blocks - 1) * self.compress_ratio
            raw[first:first + tail].copy_(torch.from_numpy(rows.reshape(tail, self.head_dim).copy()))
            offset += raw_bytes
        torch.cuda.synchronize(self.device)
        return offset
