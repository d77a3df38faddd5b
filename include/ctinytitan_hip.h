/*
 * CTinyTitanHIP -- C ABI of the MI355X (gfx950) KV-cache attention path.
 *
 * What TinyTitan's Swift runner calls in place of its Metal attention
 * encoders: an fp16 KV cache resident in HBM, GQA decode attention over it,
 * causal chunked prefill attention, and multi-row (MTP / wide) verify, each
 * with the Qwen sigmoid output gate fused into the epilogue.
 *
 * Conventions follow the reference's existing Swift->C module TinyTitanKernelsC
 * (sources/TinyTitanKernelsC/include/tinytitan_kernels.h,
 * tinytitan_expert_io.h:42-58): plain C99 prototypes, caller-owned pointers and
 * explicit sizes, outputs written (never accumulated), opaque handles made by
 * create(..., int *out_err) / destroy, int status returns with 0 = success.
 * Shape violations that the Swift side traps on (precondition) are returned as
 * status codes here; nothing in this library aborts the process.
 *
 * Memory: q / gate / out / k / v pointers are DEVICE pointers (HBM) of IEEE
 * binary16 elements (tt_half = raw bits).  slots / seq_lens / start_positions
 * are HOST arrays, read before the call returns.  Work is enqueued on the
 * context's HIP stream and completes asynchronously; tt_hip_sync blocks.
 * One call at a time per context (the runner holds its forwardStepGate,
 * sources/TinyTitan/Runtime/Inference/RealForwardRunner+Decode.swift:28-45);
 * a second thread entering gets TT_HIP_ERR_BUSY, mirroring the re-entrancy
 * guard of sources/TinyTitan/Kernels/Attention/Attention.swift:346-359.
 */
#ifndef CTINYTITAN_HIP_H
#define CTINYTITAN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TT_HIP_API __attribute__((visibility("default")))

typedef uint16_t tt_half; /* IEEE binary16 bit pattern */
typedef struct tt_hip_ctx tt_hip_ctx;
typedef struct tt_hip_kv tt_hip_kv;

enum tt_hip_status {
    TT_HIP_OK = 0,
    TT_HIP_ERR_INVALID_ARGUMENT = 1, /* null handle/pointer, negative count, slot or layer out of range */
    TT_HIP_ERR_SHAPE = 2,            /* head counts / head_dim / strides the kernels do not serve */
    TT_HIP_ERR_CURSOR = 3,           /* position does not match the slot's cursor, or rewind past it */
    TT_HIP_ERR_CAPACITY = 4,         /* rows beyond capacity / max context */
    TT_HIP_ERR_BUSY = 5,             /* context re-entered while a call is being enqueued */
    TT_HIP_ERR_OUT_OF_MEMORY = 6,    /* HBM allocation failed */
    TT_HIP_ERR_HIP = 7,              /* a HIP runtime call failed; see tt_hip_last_hip_error */
    TT_HIP_ERR_NO_DEVICE = 8,        /* no gfx950 device at that index */
    TT_HIP_ERR_STALE = 9,            /* graph replay after a buffer its kernels address was reallocated or freed */
    TT_HIP_ERR_SCRATCH = 10          /* tt_hip_attn_decode_noalloc: the call needs more scratch than its fixed array holds */
};

/* Limits (the reference allows at most 256 slots,
 * sources/TinyTitan/Runtime/KVCache/KVCacheManager.swift:91). */
#define TT_HIP_MAX_SLOTS 256
#define TT_HIP_KV_BLOCK_TOKENS 32 /* capacity granularity: tokens per swizzled K/V block */

/* ---- context ------------------------------------------------------------ */

/* Replaces MetalContext + the per-Attention split scratch
 * (sources/TinyTitan/Kernels/Attention/Attention.swift:59-71,140-156): owns a
 * HIP stream, the split-K partial buffers and timing events. */
TT_HIP_API tt_hip_ctx *tt_hip_ctx_create(int device, int *out_err);
TT_HIP_API void tt_hip_ctx_destroy(tt_hip_ctx *ctx);

/* Enqueue on a caller-owned hipStream_t instead of the context's own
 * (NULL restores the context's stream).  The reference's equivalent is the
 * MTLCommandBuffer argument of every encode call (Attention.swift:270-284). */
TT_HIP_API int tt_hip_ctx_set_stream(tt_hip_ctx *ctx, void *hip_stream);
/* Enqueue on HIP's legacy default (null) stream, whose handle is NULL and therefore cannot be
 * passed to tt_hip_ctx_set_stream.  A caller whose other work runs there (a framework's default
 * stream) gets the usual stream order between its kernels and these calls.  The context's own
 * stream is created non-blocking: it has NO order with the null stream, so a caller that stays on
 * it must synchronise (tt_hip_sync, or its own events) around buffers that other streams write or
 * free.  The null stream cannot be captured into a graph. */
TT_HIP_API int tt_hip_ctx_set_default_stream(tt_hip_ctx *ctx);
TT_HIP_API void *tt_hip_ctx_stream(tt_hip_ctx *ctx);

/* Blocks until everything enqueued on the context's stream has finished
 * (the runner's waitForCompletion on the last command buffer). */
TT_HIP_API int tt_hip_sync(tt_hip_ctx *ctx);

/* Timing, the counterpart of recordKernelGPU(role:)
 * (sources/TinyTitan/Runtime/Inference/RealForwardRunner+Diagnostics.swift:43).
 * timer_begin/timer_end bracket a region of enqueued work with HIP events on
 * the context's stream; timer_end blocks and returns the elapsed nanoseconds. */
TT_HIP_API int tt_hip_timer_begin(tt_hip_ctx *ctx);
TT_HIP_API int tt_hip_timer_end(tt_hip_ctx *ctx, uint64_t *out_ns);

/* Per-kernel timing of the dominant attention kernel (the pass over K/V), the
 * counterpart of the reference's per-kernel split TINYTITAN_KERNEL_SPLIT
 * (RealForwardRunner+DecodeFullAttention.swift:83).  While enabled, every
 * launch of that kernel carries its own pair of HIP events (up to max_launches
 * pairs; later launches go untimed), bound to the dispatch itself: a pair reads
 * the dispatch's begin-to-end time, as a kernel trace would.  (The same holds
 * for the epilogue, projection and read-control kernels; the indexer's entry
 * points, which span several launches, record a pair around them instead.)
 * profile_read blocks until the stream is idle, returns how many launches were
 * timed and their summed duration, and clears the record. */
TT_HIP_API int tt_hip_profile_enable(tt_hip_ctx *ctx, int max_launches);
TT_HIP_API int tt_hip_profile_disable(tt_hip_ctx *ctx);
TT_HIP_API int tt_hip_profile_read(tt_hip_ctx *ctx, int *out_launches, uint64_t *out_total_ns);
/* What a pair of events RECORDED on this stream with nothing between them reads (measured when profiling
 * was enabled, minimum of 16 pairs): the part of a duration bracketed that way -- the indexer's entry points --
 * that is not the kernels.  Pairs bound to a dispatch carry no such part. */
TT_HIP_API int tt_hip_profile_event_overhead_ns(tt_hip_ctx *ctx, uint64_t *out_ns);

/* Measurement control (no counterpart in the reference): a plain streaming read of `bytes` of device
 * memory at `src` (16-byte aligned), one workgroup per CU over contiguous shares, rounded down to
 * a whole number of 64 KiB turns per workgroup (*out_bytes_read says how much was read; less than
 * one turn is TT_HIP_ERR_SHAPE).  Timed by tt_hip_profile_* like the attention pass, it gives the
 * time a launch that only reads the same bytes takes on this device -- what a decode pass over a
 * cache of that size is compared with.  `sink` may be NULL. */
TT_HIP_API int tt_hip_calibrate_read(tt_hip_ctx *ctx, const void *src, size_t bytes, uint32_t *sink,
                                     size_t *out_bytes_read);

/* HIP-graph capture of a sequence of calls on the context's stream, so that a
 * launch-bound inner loop (one attention call per layer of a decode step)
 * replays with a single host call.  Everything enqueued between graph_begin
 * and graph_end is recorded, not run.  Calls that would have to allocate while
 * capturing (first use of a larger split scratch, tt_hip_kv_reserve growth,
 * tt_hip_kv_create*) return TT_HIP_ERR_BUSY and leave the capture intact: run
 * the same sequence once eagerly first.
 * A graph is a recording of ONE step: sequence lengths, positions, slots and
 * every pointer are frozen at capture, so a replay repeats exactly that step
 * (a decode step at another length is another graph).  Its kernels address the
 * context's scratch and the caches' stores directly; once any of them has been
 * reallocated or freed since the capture (a later eager call that grew the
 * split scratch, the staging pages or the selection workspace,
 * tt_hip_kv_reserve growth, tt_hip_kv_destroy), tt_hip_graph_launch returns
 * TT_HIP_ERR_STALE instead of replaying: capture again.  The
 * reference's analogue is encoding a whole layer into one MTLCommandBuffer
 * (RealForwardRunner+DecodeLayers.swift:76-82). */
typedef struct tt_hip_graph tt_hip_graph;
TT_HIP_API int tt_hip_graph_begin(tt_hip_ctx *ctx);
TT_HIP_API int tt_hip_graph_end(tt_hip_ctx *ctx, tt_hip_graph **out_graph);
TT_HIP_API int tt_hip_graph_launch(tt_hip_ctx *ctx, tt_hip_graph *graph);
TT_HIP_API void tt_hip_graph_destroy(tt_hip_graph *graph);

/* Split-K geometry report, the counterpart of Attention.splitGeometry
 * (Attention.swift:202-227): for a decode/verify of `rows` query tokens per
 * sequence over `seq_len` keys, how many key splits and workgroups one call
 * launches over an fp16 cache (over quantised pages a few verify rows stay in
 * tiles of 16 up to twice the keys).  Pure host arithmetic. */
TT_HIP_API int tt_hip_split_geometry(tt_hip_ctx *ctx, int n_seq, int n_q_heads, int n_kv_heads, int head_dim,
                                     int rows, int seq_len, int *out_split_tokens, int *out_splits,
                                     int *out_workgroups);

/* Optional overrides (0 = automatic).  Mirrors the reference's env switches
 * for attention variants (Attention.swift:186-188). */
TT_HIP_API int tt_hip_set_split_tokens(tt_hip_ctx *ctx, int split_tokens);

/* Switches between variants of the kernels, for measurement (A/B on one box) and as a way back should a
 * variant misbehave on some machine; the defaults are the measured-best ones.  The counterpart of the
 * reference's TINYTITAN_ATTN_* environment switches (Attention.swift:186-188), as explicit calls: the library
 * reads no environment variable.  Takes effect from the next call on the context; TT_HIP_ERR_BUSY inside a
 * graph capture, TT_HIP_ERR_INVALID_ARGUMENT for an unknown option or value. */
enum tt_hip_option {
    /* -1 (default): K/V loads of launches that read every page once are marked non-temporal from 16 MiB of
     * pages per launch on; 0 / 1: never / always. */
    TT_HIP_OPT_KV_STREAM = 1,
    /* 1 (default): a chunk that goes through the split-K tiles over several key ranges is launched XCD-major
     * (the workgroups one XCD runs side by side are token tiles of one KV head over one key range); 0: split-major. */
    TT_HIP_OPT_XCD_GRID = 2,
    /* Measurement control, 0 (default) / 1: attention calls that split their keys launch the pass over K/V WITHOUT
     * the combine pass behind it -- their outputs are NOT written.  For timing a run of nothing but that kernel
     * (say, captured in one graph) with one event pair around the whole run: the kernel's sustained launch
     * duration with nothing subtracted or assumed.  No counterpart in the reference. */
    TT_HIP_OPT_MEASURE_PASS_ONLY = 3
};
TT_HIP_API int tt_hip_set_option(tt_hip_ctx *ctx, int option, int value);

TT_HIP_API const char *tt_hip_strerror(int status);
TT_HIP_API const char *tt_hip_last_hip_error(tt_hip_ctx *ctx);

/* ---- KV cache ------------------------------------------------------------ */

/* Replaces KVCacheManager (sources/TinyTitan/Runtime/KVCache/KVCacheManager.swift:62-333):
 * one K and one V store per layer, a region per slot, a cursor per slot.
 * Storage is fp16 in HBM as [layer][slot][kv_head] pages; inside a page rows
 * are grouped into blocks of 32 tokens swizzled for the MFMA operand layout
 * (see tt_hip_kv_k_offset / tt_hip_kv_v_offset), so callers never address
 * rows directly: they append and read token-major rows through this ABI.
 * initial_capacity_tokens is rounded up to a multiple of 32; the reference
 * starts at min(maxContext, 8192) and doubles (KVCacheManager.swift:270-285).
 * A page (one slot's rows of one KV head) is addressed with 32 bits: max_context_tokens
 * beyond 0x7ff00000 bytes of page (4.19 M tokens at fp16, head_dim 256) is TT_HIP_ERR_CAPACITY. */
TT_HIP_API tt_hip_kv *tt_hip_kv_create(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim, int n_slots,
                                       int initial_capacity_tokens, int max_context_tokens, int *out_err);
TT_HIP_API void tt_hip_kv_destroy(tt_hip_kv *kv);

/* The same cache at KVCachePrecision int8 / int4 (sources/TinyTitanCore/Engine/SessionBuildOptions.swift:6-13;
 * KVCacheManager(..., precision:), KVCacheManager+Storage.swift:21, :65): bits = 8 or 4 stores every
 * token's row as affine levels with one fp16 scale and one fp16 bias per group of 64 consecutive
 * elements (quantizationGroupSize); bits = 16 is tt_hip_kv_create.  On such a cache
 *   tt_hip_kv_append     quantises while it writes -- it replaces KVCacheQuantizer.encode
 *                        (sources/TinyTitan/Kernels/Quant/KVCacheQuantizer.swift:14-66; kernel
 *                        kv_cache_quantize_affine, sources/TinyTitanCore/Metal/Quant/kv_cache_quantize.metal:7-73):
 *                        bias = group minimum, scale = (maximum - minimum) / (2^bits - 1),
 *                        level = round(clamp((x - bias) / scale)) in fp32;
 *   tt_hip_kv_read       gives level * scale + bias rounded to fp16;
 *   tt_hip_attn_*        read the levels and dequantise in registers, the way attn_load_kv does
 *                        (sources/TinyTitanCore/Metal/Attention/attention.metal:89-117), the
 *                        kvFormat argument of Attention.encodeFull (Attention.swift:270-284) and
 *                        PrefillAttentionParams.kvBits (PrefillAttention.swift:5-55);
 *   snapshots            carry the stored rows (levels, scales, biases), as the reference's do;
 *   tt_hip_qkv_epilogue_append   quantises the K (normed, rotated, rounded to fp16) and V rows it
 *                        writes, with the same arithmetic.
 * HBM per token and layer side: 544 bytes (8 bits) or 288 (4 bits) against 1024 for 2 x 256. */
TT_HIP_API tt_hip_kv *tt_hip_kv_create_quantized(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim,
                                                 int n_slots, int initial_capacity_tokens, int max_context_tokens,
                                                 int bits, int *out_err);
TT_HIP_API int tt_hip_kv_precision_bits(const tt_hip_kv *kv); /* 16, 8 or 4; -1 for NULL */

/* A cache for sliding-window layers, stored as a ring: the row of position p lives at
 * p % capacity, capacity = ring_capacity_tokens rounded up to 32 and fixed (tt_hip_kv_reserve is a
 * no-op), while cursors and positions run up to max_context_tokens.  The reference keeps the
 * sliding-window layers of a model this way (KVCacheManager.ringCapacity(layer:),
 * physicalSlot(layer:position:) = position % capacity, KVCacheManager+Validation.swift:47-59;
 * attn_ring_slot, sources/TinyTitanCore/Metal/Attention/attention.metal:81-86); a caller makes one
 * handle for those layers and one for the full-attention layers.
 *   rows      tt_hip_kv_append / _read / _export_rows / _import_rows / tt_hip_qkv_epilogue_append take
 *             ranges that do not wrap (position % capacity + n_tokens <= capacity, the
 *             reference's validateContiguousPhysicalRange), else TT_HIP_ERR_CAPACITY;
 *   keys      an attention call may only read rows the ring still holds: with a window,
 *             window + rows + 30 <= capacity serves every position; without one, while the
 *             sequence fits the capacity; else TT_HIP_ERR_CAPACITY;
 *   snapshot  slot 0's first min(position, capacity) stored rows, as the reference's.
 * bits as in tt_hip_kv_create_quantized. */
TT_HIP_API tt_hip_kv *tt_hip_kv_create_ring(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim, int n_slots,
                                            int ring_capacity_tokens, int max_context_tokens, int bits, int *out_err);

/* KVCacheManager.rowLayout (KVCacheManager+Validation.swift:30-41): bytes per stored token row and
 * bytes of its packed levels (rounded up to 2), for a row of `elements` values.  Pure host
 * arithmetic; 512 elements -> 1024 / 544 / 288 bytes at 16 / 8 / 4 bits. */
TT_HIP_API int tt_hip_kv_row_layout(int elements, int bits, size_t *stride_bytes, size_t *value_bytes);

/* Rows [position, position + n_tokens) in the reference's stored row format -- fp16 values, or
 * [packed levels][fp16 scale per group][fp16 bias per group] with the groups numbered across
 * the whole n_kv_heads * head_dim row and, at 4 bits, even elements in the low nibble -- to
 * (export) or from (import) DEVICE memory, row_stride_bytes apart (even, >= tt_hip_kv_token_stride_bytes).
 * Export takes a NULL k_rows or v_rows to skip that side.  Import writes the rows as they are
 * (no re-quantisation): export -> import reproduces the cache bit for bit.  What KVView hands
 * to byte-level readers in the reference (KVCacheManager+Views.swift:19-71). */
TT_HIP_API int tt_hip_kv_export_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, void *k_rows,
                                     void *v_rows, size_t row_stride_bytes);
TT_HIP_API int tt_hip_kv_import_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens,
                                     const void *k_rows, const void *v_rows, size_t row_stride_bytes);

TT_HIP_API int tt_hip_kv_capacity(const tt_hip_kv *kv);            /* tokens per slot, or -1 */
TT_HIP_API int tt_hip_kv_max_context(const tt_hip_kv *kv);
TT_HIP_API int tt_hip_kv_position(const tt_hip_kv *kv, int slot);  /* cursor (KVCacheManager+Storage.swift:281-285), or -1 */
TT_HIP_API size_t tt_hip_kv_token_stride_bytes(const tt_hip_kv *kv); /* stored row: 1024 / 544 / 288 for 2 x 256 at 16 / 8 / 4 bits */
TT_HIP_API size_t tt_hip_kv_bytes(const tt_hip_kv *kv);             /* HBM held by all layers, K and V */

/* Write rows [position, position + n_tokens) of `slot` in `layer` from
 * token-major fp16 rows k[t * src_token_stride + kv_head * head_dim + d]
 * (elements).  Replaces the decode GEMV writing into kSlot/vSlot in place
 * (RealForwardRunner+DecodeFullAttention.swift:28-38), the prefill blit
 * copyPrefillKVToCache (RealForwardRunner+PrefillKV.swift:99-145) and the
 * verify row copy (RealForwardRunner+VerifyDecodeOrderAttention.swift:86-92).
 * Does not move the cursor (every layer writes the same position before one
 * advance).  TT_HIP_ERR_CAPACITY when position + n_tokens exceeds capacity:
 * call tt_hip_kv_reserve first, as the runner does (RealForwardRunner+Decode.swift:277). */
TT_HIP_API int tt_hip_kv_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k,
                                const tt_half *v, size_t src_token_stride);

/* Gather rows back to token-major fp16 (inverse of append).  Serves snapshot /
 * prompt-cache readers (KVCacheManager+Snapshot.swift) and tests. */
TT_HIP_API int tt_hip_kv_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k_out,
                              tt_half *v_out, size_t dst_token_stride);

/* Rows by a list of positions: row t of the output is the row of positions[t] (token-major fp16,
 * level * scale + bias on a quantised cache), for the compacted form of a sparse selection --
 * DecodeKeySelection.indices / count (sources/TinyTitan/Kernels/Attention/QSASelection.swift:22-32), the
 * list the reference's window path gathers before its kernel iterates it
 * (KVCacheManager.prepareDecodeWindow, sources/TinyTitan/Runtime/KVCache/KVCacheManager+HostStreaming.swift:304-340;
 * RealForwardRunner+DecodeFullAttention.swift:9-24).  With 32-token swizzled blocks the way to read
 * only what is selected is to gather it: tt_hip_kv_gather, tt_hip_kv_append into a scratch cache
 * handle at positions 0 .. n-1, then tt_hip_attn_decode over n keys there -- O(selection) instead of
 * O(context), the same result as tt_hip_attn_decode_keep over the equivalent mask.
 * positions is a DEVICE array of n_tokens ints (logical positions; a ring maps them itself); it
 * cannot be checked on the host: a position outside [0, capacity) (a ring: [0, max_context)) gives
 * a row of zeros. */
TT_HIP_API int tt_hip_kv_gather(tt_hip_kv *kv, int layer, int slot, const int *positions, int n_tokens, tt_half *k_out,
                                tt_half *v_out, size_t dst_token_stride);

/* Cursor bookkeeping: advance (KVCacheManager+Storage.swift:266-278), rewind --
 * cursor only, no copy, 0 <= position <= cursor else TT_HIP_ERR_CURSOR
 * (:299-309) --, reset of one slot or of all with slot = -1, and reserve,
 * which doubles capacity until `tokens` fit, clamps at max_context without
 * failing, preserves every slot's live rows and is a no-op below capacity
 * (:99-139). */
TT_HIP_API int tt_hip_kv_advance(tt_hip_kv *kv, int slot, int n_tokens);
TT_HIP_API int tt_hip_kv_rewind(tt_hip_kv *kv, int slot, int position);
TT_HIP_API int tt_hip_kv_reset(tt_hip_kv *kv, int slot);
TT_HIP_API int tt_hip_kv_reserve(tt_hip_kv *kv, int tokens);
/* TT_HIP_ERR_CURSOR unless the slot's cursor equals `position`: the check
 * produceToken makes before a step (RealForwardRunner+Decode.swift:222-226). */
TT_HIP_API int tt_hip_kv_expect_position(const tt_hip_kv *kv, int slot, int position);

/* Element offsets (in halves, within one [slot][kv_head] page) of key/value
 * element (position, d).  Pure host arithmetic, the same functions the kernels
 * use; exported so that the layout is testable and documented in one place. */
TT_HIP_API size_t tt_hip_kv_k_offset(int head_dim, int position, int d);
TT_HIP_API size_t tt_hip_kv_v_offset(int head_dim, int position, int d);

/* ---- attention ----------------------------------------------------------- */

/* GQA decode, one query token per sequence: replaces Attention.encodeFull +
 * encodeSigmoidGateMul (Attention.swift:270-307; RealForwardRunner+
 * DecodeFullAttention.swift:43-90) and, with n_seq > 1, the per-row loop
 * encodeBatchRowAttention (RealForwardRunner+BatchAttention.swift:147-219).
 *   slots[i], seq_lens[i]  host arrays; seq_lens[i] is the EXCLUSIVE key count
 *                          (position + 1, i.e. including the row just appended)
 *   q     [n_seq][n_q_heads][head_dim]   gate likewise, or NULL for no gate
 *   out   [n_seq][n_q_heads][head_dim]
 * q head h reads KV head h / (n_q_heads / n_kv_heads).  seq_len 0 writes zeros.
 * The gate multiplies in fp32 after normalisation, then one fp16 round. */
TT_HIP_API int tt_hip_attn_decode(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                  const int *seq_lens, int n_q_heads, const tt_half *q, const tt_half *gate,
                                  float scale, tt_half *out);

/* tt_hip_attn_decode for callers that cannot allocate: code under HIP graph capture, tight serving
 * loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments,
 * kernels and results as tt_hip_attn_decode (bit for bit), but the split-K partial results go to a
 * fixed array inside the library's device image (33 MiB per GPU, held until the process ends) and
 * the per-sequence tables stay on the stack: the call makes no hipMalloc / hipFree and no host
 * allocation, on its first use as on any other.
 * Limits, beyond which it returns TT_HIP_ERR_SCRATCH and launches nothing: n_seq <= 64, and
 * 32768 partial rows = (key splits summed over the sequences) x KV heads x 16 query rows (32 from
 * 17 q heads per KV head on).  Every sequence takes the splits its own keys need; with the
 * planner's own split length a call of up to 64 sequences stays below 20000 rows (C2 uses 4096),
 * and only a split override (tt_hip_set_split_tokens) can exceed the array.
 * Every call on a GPU shares that GPU's array, from whichever context: calls that overlap on one
 * GPU (two streams, two contexts, two threads) race on it.  Nothing in it has to start at zero --
 * a call writes every partial its combine pass reads -- so it is never cleared. */
TT_HIP_API int tt_hip_attn_decode_noalloc(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                          const int *seq_lens, int n_q_heads, const tt_half *q,
                                          const tt_half *gate, float scale, tt_half *out);

/* Causal chunk attention: replaces PrefillAttention.encodeCausal with
 * PrefillAttentionParams{startPosition, queryCount, kvValidCount, strides}
 * (sources/TinyTitan/Kernels/Attention/PrefillAttention.swift:5-55,165-258) and
 * the gate pass over t*qDim (RealForwardRunner+PrefillAttention.swift:417-423).
 * Query row t (absolute start_pos + t) attends keys [0, min(kv_valid,
 * start_pos + t + 1)); the chunk's own K/V rows must already be appended.
 *   q[t * q_stride + h * head_dim + d], gate likewise with gate_stride,
 *   out[t * o_stride + h * head_dim + d]      (strides in elements, >= n_q_heads*head_dim)
 * Requires start_pos + q_len <= kv_valid <= capacity (validate, :334-363). */
TT_HIP_API int tt_hip_attn_prefill(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len,
                                   int kv_valid, int n_q_heads, const tt_half *q, size_t q_stride,
                                   const tt_half *gate, size_t gate_stride, float scale, tt_half *out,
                                   size_t o_stride);

/* Sliding-window forms.  A row at absolute position p attends keys
 * [max(0, p + 1 - window), p + 1) instead of [0, p + 1); window 0 means no window.
 *   decode_swa   replaces Attention.encodeSWA (Attention.swift:229-266; kvStart = seqLen > window ?
 *                seqLen - window : 0), on a cache that keeps every row or on a ring
 *                (tt_hip_kv_create_ring, the reference's ringCapacity argument); the kernel walks
 *                only the blocks the window touches;
 *   prefill_swa  replaces PrefillAttentionParams.slidingWindow (PrefillAttention.swift:12;
 *                first = abs_q + 1 > slidingWindow ? abs_q + 1 - slidingWindow : 0,
 *                prefill.metal:1200-1202).
 *   verify_swa   the rows of a wide verify over a sliding-window layer: row r of sequence i is a
 *                decode_swa at position start_positions[i] + r (the reference runs such layers
 *                row by row through encodeSWA and checks its rings with
 *                WideVerifyRollbackPlan.checkRings, WideVerifyGDNRollback.swift:394-410).
 * Everything else as in tt_hip_attn_decode / tt_hip_attn_prefill / tt_hip_attn_verify. */
TT_HIP_API int tt_hip_attn_decode_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                      const int *seq_lens, int window, int n_q_heads, const tt_half *q,
                                      const tt_half *gate, float scale, tt_half *out);

/* Decode over a sparse key selection: keep_mask holds one byte per key position of each sequence
 * (sequence i's mask starts at keep_mask + i * keep_stride and covers seq_lens[i] positions); a
 * zero byte drops that key entirely, so that the result equals attention over the kept keys alone.
 * Replaces the keepMask argument of Attention.encodeFull (sources/TinyTitan/Kernels/Attention/Attention.swift:270-284,
 * bound at :436-437; kernels attention_decode_partial / _partial_simd, keep[p] at
 * sources/TinyTitanCore/Metal/Attention/attention.metal:182-188, :229, :526), which the runner passes
 * for a QSA layer's DecodeKeySelection.mask (RealForwardRunner+DecodeFullAttention.swift:68-82).
 * Positions are logical (before the ring mapping), as there.  A sequence whose every key is
 * dropped gives zeros.  Blocks of 32 keys without a kept key are not read, and at long contexts
 * not worked on (masks that start on 4-byte boundaries): a selection costs the blocks it touches,
 * not the context.
 * keep_mask is a device pointer. */
TT_HIP_API int tt_hip_attn_decode_keep(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                       const int *seq_lens, const uint8_t *keep_mask, size_t keep_stride,
                                       int n_q_heads, const tt_half *q, const tt_half *gate, float scale, tt_half *out);

/* The same decode with the selection compacted: sequence i keeps the keys keep_indices[i * keep_index_stride + j],
 * j < keep_counts[i] (at most keep_index_stride of them; unsorted and repeated entries are fine, entries at or
 * past seq_lens[i] are ignored) -- DecodeKeySelection.indices / .count of the reference
 * (sources/TinyTitan/Kernels/Attention/QSAIndexer.swift:414-497), which its runner hands to the host-streaming
 * window (KVCacheManager+HostStreaming.swift:304-340).  The lists are written out as one row of selection bytes per
 * sequence in a store the context owns (grown on demand: TT_HIP_ERR_BUSY inside a graph capture if it has to grow)
 * and served as tt_hip_attn_decode_keep serves them: one small launch (about 3 us) more than the mask form, and
 * up to a context of 256k keys less than gathering the listed rows (tt_hip_kv_gather) and decoding over the copy.
 * keep_indices and keep_counts are device pointers. */
TT_HIP_API int tt_hip_attn_decode_keep_indices(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                               const int *seq_lens, const uint32_t *keep_indices, size_t keep_index_stride,
                                               const uint32_t *keep_counts, int n_q_heads, const tt_half *q,
                                               const tt_half *gate, float scale, tt_half *out);

/* A prefill chunk over per-query selections: row t of the chunk (position start_pos + t) sees key p
 * iff p <= start_pos + t and keep_mask[t * keep_stride + p] != 0 -- the mask form of the keepMask /
 * keepStride arguments of PrefillAttention.encodeCausal for a QSA layer
 * (RealForwardRunner+PrefillAttention.swift:395-410; kernels keep[t * keepStride + key],
 * sources/TinyTitanCore/Metal/Prefill/prefill.metal:1063-1068, :1129, :1002).  A row with no
 * kept key gives zeros.  Served by the GQA-packed split-K tiles (the MFMA chunk kernel takes no
 * selection, as in the reference only its tiled kernel does).  keep_mask is a device pointer, 4-byte aligned; keep_stride >= start_pos + q_len
 * and a multiple of 4, else TT_HIP_ERR_SHAPE.  A tile's workgroup lists the key blocks its rows keep a key of
 * and walks only those: a sparse chunk costs its selection, not its context. */
TT_HIP_API int tt_hip_attn_prefill_keep(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len,
                                        int kv_valid, const uint8_t *keep_mask, size_t keep_stride, int n_q_heads,
                                        const tt_half *q, size_t q_stride, const tt_half *gate, size_t gate_stride,
                                        float scale, tt_half *out, size_t o_stride);
/* The same chunk with the selection compacted: row t keeps the keys keep_indices[t * keep_index_stride + i],
 * i < keep_counts[t] (at most keep_index_stride of them), of which it sees those below
 * min(kv_valid, start_pos + t + 1) -- the keepIndices / keepIndexStride / keepCounts arguments of
 * PrefillAttention.encodeCausal (RealForwardRunner+PrefillAttention.swift:389-391, :404-406; the tiled kernel's
 * `useKeep == 2` walk, keepIdx[t * keepIdxStride + step] for step < keepCount[t],
 * sources/TinyTitanCore/Metal/Prefill/prefill.metal:1069-1077, :1110-1117).  The reference's lists are ascending
 * and free of repeats; here entries may come in any order, and a key listed twice is kept ONCE (the reference's walk
 * would add it twice) -- callers that keep to the reference's contract see no difference.
 * The lists are served as lists: one launch turns them into a plan per tile of tokens -- the ascending list of the
 * 32-key blocks that hold a listed key, and per block and token the listed keys as 32 bits -- which the attention
 * kernel walks in place of rows of selection bytes.  Work and memory are of the order of the selection (a tile's plan
 * is at most min(blocks of the context, tokens x keep_index_stride) x (1 + tokens) words), never rows x context, and
 * there is no limit on q_len x context; long chunks go in pieces of rows so that a piece's plan stays below 128 MiB.
 * The plan lives in a store the context owns (grown on demand: TT_HIP_ERR_BUSY inside a graph capture if it has to
 * grow).  Same result as the mask form up to the order of the additions.  keep_indices and keep_counts are device
 * pointers. */
TT_HIP_API int tt_hip_attn_prefill_keep_indices(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len,
                                                int kv_valid, const uint32_t *keep_indices, size_t keep_index_stride,
                                                const uint32_t *keep_counts, int n_q_heads, const tt_half *q,
                                                size_t q_stride, const tt_half *gate, size_t gate_stride, float scale,
                                                tt_half *out, size_t o_stride);
TT_HIP_API int tt_hip_attn_prefill_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len,
                                       int kv_valid, int sliding_window, int n_q_heads, const tt_half *q,
                                       size_t q_stride, const tt_half *gate, size_t gate_stride, float scale,
                                       tt_half *out, size_t o_stride);
TT_HIP_API int tt_hip_attn_verify_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                      const int *start_positions, int rows, int window, int n_q_heads,
                                      const tt_half *q, const tt_half *gate, float scale, tt_half *out);

/* Multi-row verify (MTP pair / wide verify): replaces
 * encodeFullAttentionDecodeOrderRows (RealForwardRunner+VerifyDecodeOrderAttention.swift:52-110)
 * and verifyGreedyPair's 2-token prefill (RealForwardRunner+MTPVerify.swift:57-103).
 * Row r of sequence i attends keys [0, start_positions[i] + r + 1), i.e. it
 * equals a decode at position start + r; the `rows` draft K/V rows must
 * already be appended at [start, start + rows).  The cache is read once per
 * sequence for all rows.
 *   q / gate / out  [n_seq][rows][n_q_heads][head_dim] */
TT_HIP_API int tt_hip_attn_verify(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                  const int *start_positions, int rows, int n_q_heads, const tt_half *q,
                                  const tt_half *gate, float scale, tt_half *out);

/* Inference-state snapshots of the KV cache, in the reference's wire format
 * (KVCacheManager+Snapshot.swift:12-118): for every layer, slot 0's first
 * min(position, capacity) rows of K as token-major fp16 rows (n_kv_heads *
 * head_dim * 2 bytes per token), then the same rows of V -- i.e. what the
 * reference appends from its own token-major buffers, so that prompt-cache and
 * checkpoint files are interchangeable although the HBM pages here are swizzled.
 *   segment_count    2 * n_layers (snapshotSegmentLengths :12-37)
 *   segment_lengths  TT_HIP_ERR_CURSOR unless 0 < position <= max_context
 *                    (invalidPosition); n_lengths must be segment_count
 *   export           slot 0 at its cursor; `lengths` must be what
 *                    segment_lengths gives there (else TT_HIP_ERR_SHAPE, the
 *                    reference's invalidLayout); writes at host_dst + *offset and
 *                    advances *offset (appendSnapshotPayload :39-66)
 *   restore          grows to `position` first, THEN compares lengths
 *                    (:71-83), resets every cursor, fills slot 0 and sets its
 *                    cursor to `position`; reads at host_src + *offset and
 *                    advances *offset (restoreSnapshot :68-118).  A payload too
 *                    short for the lengths is TT_HIP_ERR_SHAPE (after the growth).
 * Host pointers; both calls block until the copy is done. */
TT_HIP_API int tt_hip_kv_snapshot_segment_count(const tt_hip_kv *kv);
TT_HIP_API int tt_hip_kv_snapshot_segment_lengths(const tt_hip_kv *kv, int position, size_t *lengths, int n_lengths);
TT_HIP_API int tt_hip_kv_snapshot_export(tt_hip_kv *kv, const size_t *lengths, int n_lengths, void *host_dst,
                                         size_t dst_bytes, size_t *offset);
TT_HIP_API int tt_hip_kv_snapshot_restore(tt_hip_kv *kv, int position, const size_t *lengths, int n_lengths,
                                          const void *host_src, size_t src_bytes, size_t *offset);

/* Pre-attention epilogue fused with the KV append: from the raw QKV projections
 * of n_seq * rows tokens (token i * rows + r of sequence i sits at
 * positions[i] + r) to the attention kernels' inputs, in one launch.
 *   q_packed  [token][n_q_heads][2 * head_dim]  per head [query ; gate]
 *             (token stride q_packed_stride elements)
 *   k_proj, v_proj  [token][n_kv_heads * head_dim]  (token stride kv_stride)
 *   q_norm_weight_bf16, k_norm_weight_bf16  [head_dim] bfloat16, shared by all heads
 *   q_out, gate_out  [token][n_q_heads * head_dim] fp16 (strides q_stride, gate_stride)
 * query and key: per-head RMS norm 1/sqrt(mean(x^2) + eps) * weight, then NeoX
 * sub-dim RoPE over the first rotary_dim dims (pairs (i, i + rotary_dim/2),
 * frequency rope_theta^(-2i/rotary_dim), angle = position * frequency); the gate
 * is copied out; K (normed, rotated) and V rows are written into the cache at
 * [positions[i], positions[i] + rows) of slots[i] -- no separate tt_hip_kv_append.
 * Arithmetic is fp32 with one fp16 rounding, as the CPU engine does it
 * (CPUQwen35.swift:266-300, CPUTensorOps.swift:70-84, :120-139).
 * Replaces Elementwise.encodeSplitQGate + RMSNorm.encodeBF16WPerHead x2 +
 * RoPE.encodeNeoxSubdim x2 + the K/V slot writes of a decode row
 * (RealForwardRunner+DecodeFullAttention.swift:123-185) and, for a chunk,
 * PrefillQKVEpilogue.encodeNeoxSubdimNoVNorm (PrefillQKVEpilogue.swift:18-110)
 * + copyPrefillKVToCache (RealForwardRunner+PrefillKV.swift:99-145).
 * Does not move the cursors.  TT_HIP_ERR_SHAPE: strides below the packed
 * widths, rotary_dim above head_dim or not a multiple of 16. */
TT_HIP_API int tt_hip_qkv_epilogue_append(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                          const int *positions, int rows, int n_q_heads, const tt_half *q_packed,
                                          size_t q_packed_stride, const tt_half *k_proj, const tt_half *v_proj,
                                          size_t kv_stride, const uint16_t *q_norm_weight_bf16,
                                          const uint16_t *k_norm_weight_bf16, float eps, int rotary_dim,
                                          float rope_theta, tt_half *q_out, size_t q_stride, tt_half *gate_out,
                                          size_t gate_stride);

/* The projection behind the gate (o_proj): y[t] = W x[t] for token_count rows of x, W a
 * rows x columns matrix of affine levels -- weight_bits = 4 (two per byte, column 2 k in the low
 * nibble of byte k) or 8 -- with one bfloat16 scale and one bfloat16 bias per row and group of 64
 * columns (scales, biases: [rows][columns / 64], row-major), the reference's packed MLX-affine
 * layout.  x: fp16 [token][columns], token stride x_stride elements; y: fp16 [token][rows], token
 * stride y_stride elements, written, not accumulated.
 * Replaces RealForwardRunner.encodeAffineProjection for family .o
 * (sources/TinyTitan/Runtime/Inference/RealForwardRunner+PrefillProjection.swift:53-66, called at
 * +PrefillAttention.swift:424-436) and the GEMVs the decode paths run on the attention output:
 * DequantInt4GEMV.encode / encodeTwoRows (sources/TinyTitan/Kernels/Quant/DequantInt4GEMV.swift:72-143;
 * kernels dequant_int4_gemv_simd / dequant_int4_gemv2_simd,
 * sources/TinyTitanCore/Metal/Quant/dequant_int4.metal:101-280), the 8-bit kernels
 * (dequant_int8.metal) and encodeBatchOProj (+BatchAttention.swift:221-240).  It is the device
 * form of the reference's C entry points tinytitan_int4_affine_gemv / tinytitan_int8_affine_gemv
 * (sources/TinyTitanKernelsC/include/tinytitan_kernels.h:9-53) with fp16 activations.
 * Arithmetic: below 513 tokens as the GEMV kernels and the C entry points do it -- per row and
 * group scale * sum(level * x) + bias * sum(x), all in fp32, one rounding to fp16 at the store.
 * From 513 tokens on (prefill chunks) as the reference's tensor-operation path does it
 * (MPPPrefillInt4QMM, taken there from 32 tokens on;
 * sources/TinyTitanCore/Metal/TensorCore/tensorops.metal:80-125): each weight becomes the fp16 number
 * level * scale + bias (scale and bias must then lie within fp16's range) and x . w accumulates in
 * fp32.  Three kernels: up to 9 tokens a dot-product GEMV over all CUs, up to 512 tokens MFMA
 * tiles of 32 tokens x 32 rows with the factored arithmetic, beyond that a GEMM in tiles of 128 tokens x
 * 128 or 256 rows.
 * The two larger ones need more than 64 KiB of LDS; tt_hip_ctx_create raises their limits, so
 * every call may be captured.
 * TT_HIP_ERR_SHAPE: weight_bits other than 4 or 8, columns not a multiple of 64 (the reference's
 * precondition), strides below the row widths, x not 16-byte aligned or x_stride not a multiple
 * of 8, an odd weights / scales / biases / y address (the reference's files keep tensors 2-byte
 * aligned, DequantInt4GEMV.swift:87-92; a 16-byte aligned weights pointer takes the fast loads). */
TT_HIP_API int tt_hip_affine_projection(tt_hip_ctx *ctx, int weight_bits, const void *weights,
                                        const uint16_t *scales_bf16, const uint16_t *biases_bf16, const tt_half *x,
                                        tt_half *y, int rows, int columns, int token_count, size_t x_stride,
                                        size_t y_stride);

/* ---- The sparse-attention block indexer: what produces the selections that
 * tt_hip_attn_decode_keep / tt_hip_attn_prefill_keep / tt_hip_kv_gather take.  Buffers are the
 * caller's (the reference's QSAIndexer owns them per layer: raw keys [cells][head_dim] before norm
 * and rotation, pooled blocks [cells / ratio + 1][head_dim] after them; QSAIndexer.swift:62-70).
 * head_dim is 128 (the reference's indexer) or 256. */

/* pooled[b] = mean of the raw keys present in block b (cells [b * ratio, min((b + 1) * ratio,
 * n_kv))) for block_count blocks from first_block; blocks that start at or past n_kv are left
 * alone.  fp32 sum in member order, divided by the members present, one rounding to fp16.
 * With key_norm_bf16 (bf16 [head_dim]) the pooled row then takes the indexer's RMS norm, a rounding
 * to fp16, and a NeoX rotation over the whole row at the position of the block's first member
 * (b * ratio, frequency rope_theta^(-2i / head_dim)), as the reference's three kernels in a row
 * do; NULL leaves the plain mean.
 * Replaces qsa_pool_block / qsa_pool_blocks (sources/TinyTitanCore/Metal/Attention/qsa.metal:20-66)
 * and, with the norm weight, QSAIndexer.encodePoolPrefill (QSAIndexer.swift:196-233) and the
 * repooling half of encodeAppendKey (QSAIndexer+Scratch.swift:88-110). */
TT_HIP_API int tt_hip_qsa_pool_blocks(tt_hip_ctx *ctx, const tt_half *raw_keys, tt_half *pooled, int head_dim,
                                      int first_block, int block_count, int ratio, int n_kv,
                                      const uint16_t *key_norm_bf16, float eps, float rope_theta);

/* RMS norm (bf16 weight shared by every head), a rounding to fp16, NeoX rotation over the whole
 * head, a rounding to fp16 -- in place on rows [token][heads][head_dim]; token t sits at
 * position + t * position_stride.  The indexer's query rows take it with stride 1
 * (RMSNorm.encodeBF16WPerHead + RoPE.encodeNeoxSubdim(Strided), QSAIndexer.swift:296-309 for a
 * decode row, :343-357 for a chunk; kernels rope_neox_subdim / rope_neox_subdim_strided,
 * sources/TinyTitanCore/Metal/Primitives/rope.metal:80-134). */
TT_HIP_API int tt_hip_qsa_norm_rope_rows(tt_hip_ctx *ctx, tt_half *rows, int token_count, int heads, int head_dim,
                                         const uint16_t *norm_bf16, float eps, float rope_theta, int position,
                                         int position_stride);

/* scores[t][b] = sum over heads of max(0, query[t][h] . pooled[b]), fp32, rectified per head
 * before the sum; query [token_count][heads][head_dim] normed and rotated, pooled
 * [blocks][head_dim], scores [token_count][score_stride].  heads is 1, 2, 4 (the reference's) or 8.
 * Products accumulate in fp32 on the matrix cores, in another order than the reference's chain
 * of fused multiply-adds: scores agree to fp32 rounding, not bit for bit.
 * Replaces qsa_block_scores / qsa_block_scores_rows (qsa.metal:76-130; QSAIndexer.encodeScores,
 * QSAIndexer.swift:311-330, and encodeScoresPrefill, :359-384). */
TT_HIP_API int tt_hip_qsa_block_scores(tt_hip_ctx *ctx, const tt_half *query, const tt_half *pooled, float *scores,
                                       size_t score_stride, int head_dim, int heads, int blocks, int token_count);

/* A decode step's indexer work before the selection in ONE launch: the block the newest key falls into is
 * pooled again from raw_keys (its members up to n_kv - 1, normed, rotated at the block's first position, stored in
 * pooled), the query token's head rows query[heads][head_dim] are normed and rotated at `position`, and
 * scores[b] = sum over heads of max(0, query[h] . pooled[b]) for every block b < (n_kv - 1) / ratio + 1.  The
 * same arithmetic element by element as tt_hip_qsa_pool_blocks (one block) + tt_hip_qsa_norm_rope_rows +
 * tt_hip_qsa_block_scores in a row: the scores and the pooled block are theirs bit for bit.  `query` is read only
 * (the separate path norms it in place).  Replaces the three encodes of a decode step, QSAIndexer.encodeAppendKey's
 * repooling (QSAIndexer+Scratch.swift:88-110) and QSAIndexer.encodeScores (QSAIndexer.swift:271-330). */
TT_HIP_API int tt_hip_qsa_decode_scores(tt_hip_ctx *ctx, const tt_half *raw_keys, tt_half *pooled, int head_dim, int ratio, int n_kv,
                                        const uint16_t *key_norm_bf16, const tt_half *query, int heads,
                                        const uint16_t *query_norm_bf16, int position, float eps, float rope_theta, float *scores);

/* The selection of `rows` queries, row r seeing first_visible + r keys and scored in
 * scores[r * score_stride ...] (a decode step: rows 1, first_visible = its visible keys; a chunk:
 * first_visible = start_position + 1).  Per row: the ragged tail of the query's own block is kept;
 * complete blocks go in by score descending, the lower index first on ties (-0.0 ties +0.0), whole
 * until `width` cells (the reference's selectionWidth = budget + ratio - 1) are spent, the next
 * block giving its first cells for what remains.  A row that sees at most `width` keys keeps them
 * all.  keep[r * keep_stride + c] = 1 / 0 for c < visible and 0 from there to keep_stride;
 * indices (may be NULL): the kept cells ascending, counts (may be NULL) how many.  keep may be NULL
 * when indices and counts are given: the lists alone, as selectKeysCompact returns them -- a chunk's
 * mask rows are rows x context bytes, its lists rows x width words.  The outputs are
 * what the attention calls with a selection and tt_hip_kv_gather take.
 * Replaces qsa_select_decode (qsa.metal:156-226), QSAIndexer.selectKeys / selectKeysCompact /
 * encodeSelectKeys (QSAIndexer+Scratch.swift:191-284) and the host loop of selectKeysPrefill
 * (QSAIndexer.swift:414-497).  Scores must not be NaN (the reference's comparison has no order for
 * them either).  Up to 7 rows of more than 16,384 blocks each, or 8 of more than 32,768 (a decode or verify step at a long
 * context) are spread over many workgroups through a workspace the context allocates on first use:
 * that first call is refused with TT_HIP_ERR_BUSY while a graph is being captured.
 * TT_HIP_ERR_SHAPE: keep_stride below the last row's visible keys, score_stride below its complete
 * blocks, index_stride below width. */
TT_HIP_API int tt_hip_qsa_select(tt_hip_ctx *ctx, const float *scores, size_t score_stride, int rows, int first_visible,
                                 int ratio, int width, uint8_t *keep, size_t keep_stride, uint32_t *indices,
                                 size_t index_stride, uint32_t *counts);

#ifdef __cplusplus
}
#endif
#endif /* CTINYTITAN_HIP_H */
