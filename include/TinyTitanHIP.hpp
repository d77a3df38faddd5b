// Host-side mirror, in C++, of the Swift types whose attention work the C ABI takes over.
// Header-only; every method forwards to ctinytitan_hip.h.  Names, argument meaning and failure
// behaviour follow the reference:
//
//   KVCacheManager    sources/TinyTitan/Runtime/KVCache/KVCacheManager.swift:62-333,
//                     KVCacheManager+Storage.swift:99-139,266-309
//   Attention         sources/TinyTitan/Kernels/Attention/Attention.swift:270-307
//   PrefillAttention  sources/TinyTitan/Kernels/Attention/PrefillAttention.swift:5-55,165-258
//
// Swift `throws` and `precondition` failures both surface as tinytitan::Error carrying the ABI
// status; nothing aborts.  Pointers are device pointers to IEEE binary16 elements.
#pragma once

#include <stdexcept>
#include <string>
#include <utility>
#include <vector>

#include "ctinytitan_hip.h"

namespace tinytitan {

class Error : public std::runtime_error {
public:
    Error(int status, const char *where)
        : std::runtime_error(std::string(where) + ": " + tt_hip_strerror(status)), status_(status) {}
    int status() const { return status_; }

private:
    int status_;
};

inline void check(int status, const char *where) {
    if (status != TT_HIP_OK) throw Error(status, where);
}

// MetalContext's role for this path: the stream the work is enqueued on, plus scratch and timers.
class Context {
public:
    explicit Context(int device = 0) {
        int err = 0;
        handle_ = tt_hip_ctx_create(device, &err);
        if (!handle_) throw Error(err, "tt_hip_ctx_create");
    }
    ~Context() { tt_hip_ctx_destroy(handle_); }
    Context(const Context &) = delete;
    Context &operator=(const Context &) = delete;
    tt_hip_ctx *handle() const { return handle_; }
    void waitForCompletion() { check(tt_hip_sync(handle_), "tt_hip_sync"); }
    void setStream(void *hipStream) { check(tt_hip_ctx_set_stream(handle_, hipStream), "tt_hip_ctx_set_stream"); }
    void setDefaultStream() { check(tt_hip_ctx_set_default_stream(handle_), "tt_hip_ctx_set_default_stream"); }
    // Kernel-variant switches (the reference's TINYTITAN_ATTN_* environment switches, Attention.swift:186-188).
    void setOption(tt_hip_option option, int value) { check(tt_hip_set_option(handle_, option, value), "tt_hip_set_option"); }

private:
    tt_hip_ctx *handle_ = nullptr;
};

// KVCachePrecision (sources/TinyTitanCore/Engine/SessionBuildOptions.swift:6-13): raw value = bits per value.
enum class KVCachePrecision : int { int4 = 4, int8 = 8, fp16 = 16 };

class KVCacheManager {
public:
    static constexpr int quantizationGroupSize = 64;
    // KVCacheManager.rowLayout (KVCacheManager+Validation.swift:30-41): {stride, valueBytes} in bytes.
    static std::pair<size_t, size_t> rowLayout(int elements, KVCachePrecision precision) {
        size_t stride = 0, values = 0;
        const int st = tt_hip_kv_row_layout(elements, (int)precision, &stride, &values);
        if (st != TT_HIP_OK) throw Error(st, "KVCacheManager.rowLayout");
        return {stride, values};
    }

    // initialCapacity defaults to min(maxContext, 8192) (KVCacheManager.swift:270-285).
    KVCacheManager(Context &context, int layers, int kvHeads, int headDim, int slots, int maxContext,
                   int initialCapacity = 0, KVCachePrecision precision = KVCachePrecision::fp16)
        : context_(context) {
        int err = 0;
        if (initialCapacity <= 0) initialCapacity = maxContext < 8192 ? maxContext : 8192;
        handle_ = tt_hip_kv_create_quantized(context.handle(), layers, kvHeads, headDim, slots, initialCapacity, maxContext,
                                             (int)precision, &err);
        if (!handle_) throw Error(err, "tt_hip_kv_create_quantized");
    }
    // A ring for sliding-window layers: the row of position p lives at p % ringCapacity (KVCacheManager.ringCapacity).
    struct Ring {
        int capacity;
    };
    KVCacheManager(Context &context, int layers, int kvHeads, int headDim, int slots, int maxContext, Ring ring,
                   KVCachePrecision precision = KVCachePrecision::fp16)
        : context_(context) {
        int err = 0;
        handle_ = tt_hip_kv_create_ring(context.handle(), layers, kvHeads, headDim, slots, ring.capacity, maxContext,
                                        (int)precision, &err);
        if (!handle_) throw Error(err, "tt_hip_kv_create_ring");
    }
    KVCachePrecision precision() const { return (KVCachePrecision)tt_hip_kv_precision_bits(handle_); }
    // Rows in the stored row format (device memory, rowStrideBytes apart); null skips a side on export.
    void exportRows(int layer, int slot, int position, int tokens, void *kRows, void *vRows, size_t rowStrideBytes) {
        check(tt_hip_kv_export_rows(handle_, layer, slot, position, tokens, kRows, vRows, rowStrideBytes), "KVCacheManager.exportRows");
    }
    void importRows(int layer, int slot, int position, int tokens, const void *kRows, const void *vRows, size_t rowStrideBytes) {
        check(tt_hip_kv_import_rows(handle_, layer, slot, position, tokens, kRows, vRows, rowStrideBytes), "KVCacheManager.importRows");
    }
    ~KVCacheManager() { tt_hip_kv_destroy(handle_); }
    KVCacheManager(const KVCacheManager &) = delete;
    KVCacheManager &operator=(const KVCacheManager &) = delete;
    tt_hip_kv *handle() const { return handle_; }

    int capacityTokens() const { return tt_hip_kv_capacity(handle_); }
    int maxContext() const { return tt_hip_kv_max_context(handle_); }
    size_t strideBytes() const { return tt_hip_kv_token_stride_bytes(handle_); }
    int position(int slot = 0) const {
        const int p = tt_hip_kv_position(handle_, slot);
        if (p < 0) throw Error(TT_HIP_ERR_INVALID_ARGUMENT, "KVCacheManager.position");
        return p;
    }
    void advance(int slot = 0, int by = 1) { check(tt_hip_kv_advance(handle_, slot, by), "KVCacheManager.advance"); }
    void rewind(int slot, int to) { check(tt_hip_kv_rewind(handle_, slot, to), "KVCacheManager.rewind"); }
    void reset(int slot = -1) { check(tt_hip_kv_reset(handle_, slot), "KVCacheManager.reset"); }
    void reserve(int tokens) { check(tt_hip_kv_reserve(handle_, tokens), "KVCacheManager.reserve"); }
    // Inference-state snapshots (KVCacheManager+Snapshot.swift:12-118), reference wire format.
    std::vector<size_t> snapshotSegmentLengths(int position) const {
        std::vector<size_t> lengths((size_t)tt_hip_kv_snapshot_segment_count(handle_));
        check(tt_hip_kv_snapshot_segment_lengths(handle_, position, lengths.data(), (int)lengths.size()),
              "KVCacheManager.snapshotSegmentLengths");
        return lengths;
    }
    void appendSnapshotPayload(std::vector<unsigned char> &payload, const std::vector<size_t> &segmentLengths) {
        size_t total = 0;
        for (size_t n : segmentLengths) total += n;
        size_t offset = payload.size();
        payload.resize(offset + total);
        check(tt_hip_kv_snapshot_export(handle_, segmentLengths.data(), (int)segmentLengths.size(), payload.data(),
                                        payload.size(), &offset),
              "KVCacheManager.appendSnapshotPayload");
    }
    void restoreSnapshot(int position, const std::vector<size_t> &segmentLengths, const void *bytes, size_t count,
                         size_t &offset) {
        check(tt_hip_kv_snapshot_restore(handle_, position, segmentLengths.data(), (int)segmentLengths.size(), bytes, count,
                                         &offset),
              "KVCacheManager.restoreSnapshot");
    }
    void expectPosition(int slot, int position) const {
        check(tt_hip_kv_expect_position(handle_, slot, position), "KVCacheManager.expectPosition");
    }
    // The reference hands out write targets (kSlot / vSlot / kRange / vRange) into token-major rows;
    // here the rows are written through the cache, which owns their layout.
    void write(int layer, int slot, int position, int count, const tt_half *k, const tt_half *v, size_t tokenStride) {
        check(tt_hip_kv_append(handle_, layer, slot, position, count, k, v, tokenStride), "KVCacheManager.write");
    }
    void read(int layer, int slot, int position, int count, tt_half *k, tt_half *v, size_t tokenStride) {
        check(tt_hip_kv_read(handle_, layer, slot, position, count, k, v, tokenStride), "KVCacheManager.read");
    }
    // Rows of the listed positions (a device array): the compacted form of a sparse selection, for a scratch cache.
    void gather(int layer, int slot, const int *devicePositions, int count, tt_half *k, tt_half *v, size_t tokenStride) {
        check(tt_hip_kv_gather(handle_, layer, slot, devicePositions, count, k, v, tokenStride), "KVCacheManager.gather");
    }

private:
    Context &context_;
    tt_hip_kv *handle_ = nullptr;
};

class Attention {
public:
    explicit Attention(Context &context) : context_(context) {}

    // Attention.encodeFull + Elementwise.encodeSigmoidGateMul: seqLen is the exclusive key count.
    void encodeFull(KVCacheManager &kv, int layer, const tt_half *q, tt_half *out, int numQHeads, int seqLen,
                    float scale, int slot = 0, const tt_half *gate = nullptr) {
        check(tt_hip_attn_decode(context_.handle(), kv.handle(), layer, 1, &slot, &seqLen, numQHeads, q, gate, scale, out),
              "Attention.encodeFull");
    }
    // The same decode for callers that cannot allocate (no counterpart in the reference): split partials in the
    // library's fixed per-GPU array; TT_HIP_ERR_SCRATCH beyond 64 sequences or 32768 partial rows.
    void encodeFullNoAlloc(KVCacheManager &kv, int layer, const tt_half *q, tt_half *out, int numQHeads, int seqLen,
                           float scale, int slot = 0, const tt_half *gate = nullptr) {
        check(tt_hip_attn_decode_noalloc(context_.handle(), kv.handle(), layer, 1, &slot, &seqLen, numQHeads, q, gate,
                                         scale, out),
              "Attention.encodeFullNoAlloc");
    }
    // Attention.encodeSWA (Attention.swift:229-266): keys [max(0, seqLen - window), seqLen); no ring storage.
    void encodeSWA(KVCacheManager &kv, int layer, const tt_half *q, tt_half *out, int numQHeads, int seqLen, int window,
                   float scale, int slot = 0, const tt_half *gate = nullptr) {
        check(tt_hip_attn_decode_swa(context_.handle(), kv.handle(), layer, 1, &slot, &seqLen, window, numQHeads, q, gate,
                                     scale, out),
              "Attention.encodeSWA");
    }
    // Attention.encodeFull(..., keepMask:): one byte per key position, 0 drops the key (a QSA layer's selection).
    void encodeFullKeep(KVCacheManager &kv, int layer, const tt_half *q, tt_half *out, int numQHeads, int seqLen,
                        const uint8_t *keepMask, float scale, int slot = 0, const tt_half *gate = nullptr) {
        check(tt_hip_attn_decode_keep(context_.handle(), kv.handle(), layer, 1, &slot, &seqLen, keepMask, (size_t)seqLen,
                                      numQHeads, q, gate, scale, out),
              "Attention.encodeFullKeep");
    }
    // The same selection compacted (DecodeKeySelection.indices / .count): keepCount key ids at keepIndices.
    void encodeFullKeepIndices(KVCacheManager &kv, int layer, const tt_half *q, tt_half *out, int numQHeads, int seqLen,
                               const uint32_t *keepIndices, const uint32_t *keepCount, size_t keepIndexStride, float scale,
                               int slot = 0, const tt_half *gate = nullptr) {
        check(tt_hip_attn_decode_keep_indices(context_.handle(), kv.handle(), layer, 1, &slot, &seqLen, keepIndices,
                                              keepIndexStride, keepCount, numQHeads, q, gate, scale, out),
              "Attention.encodeFullKeepIndices");
    }
    // One query token for each of several slots (encodeBatchRowAttention's loop as one call).
    void encodeBatch(KVCacheManager &kv, int layer, const std::vector<int> &slots, const std::vector<int> &seqLens,
                     const tt_half *q, tt_half *out, int numQHeads, float scale, const tt_half *gate = nullptr) {
        if (slots.size() != seqLens.size()) throw Error(TT_HIP_ERR_INVALID_ARGUMENT, "Attention.encodeBatch");
        check(tt_hip_attn_decode(context_.handle(), kv.handle(), layer, (int)slots.size(), slots.data(), seqLens.data(),
                                 numQHeads, q, gate, scale, out),
              "Attention.encodeBatch");
    }
    // encodeFullAttentionDecodeOrderRows: row r attends start + r + 1 keys.
    void encodeVerifyRows(KVCacheManager &kv, int layer, const std::vector<int> &slots,
                          const std::vector<int> &startPositions, int rows, const tt_half *q, tt_half *out,
                          int numQHeads, float scale, const tt_half *gate = nullptr, int window = 0) {
        if (slots.size() != startPositions.size()) throw Error(TT_HIP_ERR_INVALID_ARGUMENT, "Attention.encodeVerifyRows");
        check(tt_hip_attn_verify_swa(context_.handle(), kv.handle(), layer, (int)slots.size(), slots.data(),
                                     startPositions.data(), rows, window, numQHeads, q, gate, scale, out),
              "Attention.encodeVerifyRows");
    }

private:
    Context &context_;
};

// PrefillAttentionParams (PrefillAttention.swift:5-55); strides in elements.
struct PrefillAttentionParams {
    int startPosition = 0;
    int queryCount = 0;
    int kvValidCount = 0;
    int numQHeads = 0;
    float scale = 1.0f;
    size_t qStride = 0;
    size_t oStride = 0;
    size_t gateStride = 0;
    int slidingWindow = 0;  // 0: every key up to the row's own
};

class PrefillAttention {
public:
    explicit PrefillAttention(Context &context) : context_(context) {}
    void encodeCausal(KVCacheManager &kv, int layer, int slot, const tt_half *q, tt_half *out,
                      const PrefillAttentionParams &p, const tt_half *gate = nullptr) {
        check(tt_hip_attn_prefill_swa(context_.handle(), kv.handle(), layer, slot, p.startPosition, p.queryCount,
                                      p.kvValidCount, p.slidingWindow, p.numQHeads, q, p.qStride, gate,
                                      p.gateStride ? p.gateStride : p.qStride, p.scale, out, p.oStride),
              "PrefillAttention.encodeCausal");
    }
    // encodeCausal(..., keepMask:, keepStride:) of a QSA chunk, mask form: a row of keepStride bytes per query.
    void encodeCausalKeep(KVCacheManager &kv, int layer, int slot, const tt_half *q, tt_half *out,
                          const PrefillAttentionParams &p, const uint8_t *keepMask, size_t keepStride,
                          const tt_half *gate = nullptr) {
        check(tt_hip_attn_prefill_keep(context_.handle(), kv.handle(), layer, slot, p.startPosition, p.queryCount,
                                       p.kvValidCount, keepMask, keepStride, p.numQHeads, q, p.qStride, gate,
                                       p.gateStride ? p.gateStride : p.qStride, p.scale, out, p.oStride),
              "PrefillAttention.encodeCausalKeep");
    }
    // encodeCausal(..., keepIndices:, keepIndexStride:, keepCounts:): the same selection compacted, keepCounts[t] key ids
    // per query at keepIndices[t * keepIndexStride ...].
    void encodeCausalKeepIndices(KVCacheManager &kv, int layer, int slot, const tt_half *q, tt_half *out,
                                 const PrefillAttentionParams &p, const uint32_t *keepIndices, size_t keepIndexStride,
                                 const uint32_t *keepCounts, const tt_half *gate = nullptr) {
        check(tt_hip_attn_prefill_keep_indices(context_.handle(), kv.handle(), layer, slot, p.startPosition, p.queryCount,
                                               p.kvValidCount, keepIndices, keepIndexStride, keepCounts, p.numQHeads, q,
                                               p.qStride, gate, p.gateStride ? p.gateStride : p.qStride, p.scale, out,
                                               p.oStride),
              "PrefillAttention.encodeCausalKeepIndices");
    }

private:
    Context &context_;
};

/// Split [query ; gate], per-head q/k RMS norms, NeoX sub-dim RoPE and the K/V cache write in one
/// launch: encodeGatedFullPostProjection (RealForwardRunner+DecodeFullAttention.swift:123-185) for
/// decode rows, PrefillQKVEpilogue.encodeNeoxSubdimNoVNorm (PrefillQKVEpilogue.swift:18-110) +
/// copyPrefillKVToCache for a chunk.
struct QKVEpilogueParams {
    int numQHeads = 0;
    int headDim = 0;
    int rows = 1;  // tokens per sequence
    float eps = 1e-6f;
    int rotaryDim = 0;
    float theta = 1e7f;
    size_t qPackedStride = 0, kvStride = 0, qStride = 0, gateStride = 0;  // elements; 0: packed
};

class QKVEpilogue {
public:
    explicit QKVEpilogue(Context &context) : context_(context) {}
    void encode(KVCacheManager &kv, int layer, const std::vector<int> &slots, const std::vector<int> &positions,
                const tt_half *qPacked, const tt_half *kProj, const tt_half *vProj, const uint16_t *qNormWeightBF16,
                const uint16_t *kNormWeightBF16, tt_half *qOut, tt_half *gateOut, const QKVEpilogueParams &p) {
        if (slots.size() != positions.size()) throw Error(TT_HIP_ERR_INVALID_ARGUMENT, "QKVEpilogue.encode");
        const size_t width = (size_t)p.numQHeads * (size_t)p.headDim;
        const size_t kvWidth = kv.strideBytes() / 2;
        check(tt_hip_qkv_epilogue_append(context_.handle(), kv.handle(), layer, (int)slots.size(), slots.data(),
                                         positions.data(), p.rows, p.numQHeads, qPacked,
                                         p.qPackedStride ? p.qPackedStride : 2 * width, kProj, vProj,
                                         p.kvStride ? p.kvStride : kvWidth, qNormWeightBF16, kNormWeightBF16, p.eps,
                                         p.rotaryDim, p.theta, qOut, p.qStride ? p.qStride : width, gateOut,
                                         p.gateStride ? p.gateStride : width),
              "QKVEpilogue.encode");
    }

private:
    Context &context_;
};

// encodeAffineProjection for o_proj (RealForwardRunner+PrefillProjection.swift:53-66) and the decode
// GEMVs behind the gate (DequantInt4GEMV.swift:72-143): strides in elements, 0 = packed.
class AffineProjection {
public:
    explicit AffineProjection(Context &context) : context_(context) {}
    void encode(int weightBits, const void *weights, const uint16_t *scalesBF16, const uint16_t *biasesBF16,
                const tt_half *x, tt_half *y, int rows, int columns, int tokenCount, size_t xStrideElements = 0,
                size_t yStrideElements = 0) {
        check(tt_hip_affine_projection(context_.handle(), weightBits, weights, scalesBF16, biasesBF16, x, y, rows,
                                       columns, tokenCount, xStrideElements ? xStrideElements : (size_t)columns,
                                       yStrideElements ? yStrideElements : (size_t)rows),
              "AffineProjection.encode");
    }

private:
    Context &context_;
};

// When dense attention equals the sparse selection (QSAExactness.swift:22-65): the indexer keeps
// budget / compressRatio complete blocks and always the incomplete tail block.
struct QSAExactness {
    int budget, compressRatio;
    QSAExactness(int budget_, int compressRatio_) : budget(budget_), compressRatio(compressRatio_) {
        if (budget <= 0 || compressRatio <= 0) throw std::invalid_argument("QSAExactness: budget and compressRatio must be positive");
    }
    int keptBlocks() const { return budget / compressRatio; }
    int maximumExactVisibleKeys() const { return keptBlocks() * compressRatio + (compressRatio - 1); }
    bool isDenseExact(int visibleKeys) const { return visibleKeys / compressRatio <= keptBlocks(); }
    bool isDenseExactForContext(int tokens) const { return tokens <= 0 || isDenseExact(tokens); }
    int indexerRequiredFromContext() const { return maximumExactVisibleKeys() + 1; }
};

// The kernels of the sparse attention's block indexer over buffers the caller owns (the reference's
// QSAIndexer keeps them per layer: raw keys [cells][headDim], pooled blocks [cells / ratio + 1][headDim],
// scores, the byte mask and the index list; QSAIndexer.swift:62-90).  Method names follow the encoders they
// replace; the projections in front (indexer q / k) are AffineProjection's.
class QSAIndexer {
public:
    QSAIndexer(Context &context, int heads, int headDim, int compressRatio, int budget, float ropeTheta)
        : context_(context), heads_(heads), headDim_(headDim), ratio_(compressRatio), budget_(budget), theta_(ropeTheta) {}
    int selectionWidth() const { return budget_ + ratio_ - 1; }  // QSAIndexer.swift:91
    QSAExactness exactness() const { return QSAExactness(budget_, ratio_); }

    // encodePoolPrefill (QSAIndexer.swift:196-233); with tokens = 1 the repooling of encodeAppendKey
    // (QSAIndexer+Scratch.swift:88-110).
    void encodePoolPrefill(const tt_half *rawKeys, tt_half *pooled, int startPosition, int tokens,
                           const uint16_t *keyNormBF16, float eps) {
        const int end = startPosition + tokens, firstBlock = startPosition / ratio_;
        const int blockCount = (end - 1) / ratio_ - firstBlock + 1;
        check(tt_hip_qsa_pool_blocks(context_.handle(), rawKeys, pooled, headDim_, firstBlock, blockCount, ratio_, end,
                                     keyNormBF16, eps, theta_),
              "QSAIndexer.encodePoolPrefill");
    }
    // encodeScores / encodeScoresPrefill behind the query projection (QSAIndexer.swift:296-330, :343-403):
    // queryRows [tokens][heads][headDim] are normed and rotated in place, then scored against every block up
    // to the last query's; scores [tokens][blocks].  Returns the blocks scored per row.
    int encodeScores(tt_half *queryRows, const uint16_t *queryNormBF16, const tt_half *pooled, float *scores,
                     int startPosition, int tokens, float eps) {
        check(tt_hip_qsa_norm_rope_rows(context_.handle(), queryRows, tokens, heads_, headDim_, queryNormBF16, eps, theta_,
                                        startPosition, 1),
              "QSAIndexer.encodeScores(norm, rope)");
        const int blocks = (startPosition + tokens - 1) / ratio_ + 1;
        check(tt_hip_qsa_block_scores(context_.handle(), queryRows, pooled, scores, (size_t)blocks, headDim_, heads_, blocks,
                                      tokens),
              "QSAIndexer.encodeScores");
        return blocks;
    }
    // A decode step in one launch: encodeAppendKey's repooling of the newest key's block and encodeScores for the
    // token at `position` (QSAIndexer+Scratch.swift:88-110, QSAIndexer.swift:271-330).  queryRows [heads][headDim]
    // is read only; scores [blocks].  Returns the blocks scored.
    int encodeDecodeStep(const tt_half *rawKeys, tt_half *pooled, const uint16_t *keyNormBF16, const tt_half *queryRows,
                         const uint16_t *queryNormBF16, float *scores, int position, float eps) {
        check(tt_hip_qsa_decode_scores(context_.handle(), rawKeys, pooled, headDim_, ratio_, position + 1, keyNormBF16,
                                       queryRows, heads_, queryNormBF16, position, eps, theta_, scores),
              "QSAIndexer.encodeDecodeStep");
        return position / ratio_ + 1;
    }
    // selectKeys / selectKeysCompact / encodeSelectKeys (QSAIndexer+Scratch.swift:191-284) with rows = 1 and
    // firstVisible = the visible keys; selectKeysPrefill (QSAIndexer.swift:414-497) with rows = the chunk's
    // tokens and firstVisible = startPosition + 1.  false: every row is inside the dense-exact window and
    // nothing was written (the reference returns nil there).
    bool encodeSelectKeys(const float *scores, size_t scoreStride, int rows, int firstVisible, uint8_t *keep,
                          size_t keepStride, uint32_t *indices = nullptr, uint32_t *counts = nullptr) {
        if (firstVisible + rows - 1 <= selectionWidth()) return false;
        check(tt_hip_qsa_select(context_.handle(), scores, scoreStride, rows, firstVisible, ratio_, selectionWidth(), keep,
                                keepStride, indices, (size_t)selectionWidth(), counts),
              "QSAIndexer.encodeSelectKeys");
        return true;
    }

private:
    Context &context_;
    int heads_, headDim_, ratio_, budget_;
    float theta_;
};

}  // namespace tinytitan
