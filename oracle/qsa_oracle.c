/*
 * CPU oracle for the sparse-attention block indexer (the code that chooses the
 * keys a query may attend to) -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, the smoke check
 * and the benchmark's cpu_baseline leg may build, load or call it.  The
 * library under tinytitan_amd/ must never link or import anything from here.
 *
 * Every function restates one piece of the reference in plain C99 and cites
 * the lines it follows.  Paths are relative to the reference checkout.  The
 * reference has this path as Metal kernels plus host Swift only (no C or CPU
 * engine form), so none of it can be compiled here.
 *
 * Pinning status (what checks each function besides this text):
 *   tt_oracle_qsa_pool_blocks
 *       closed forms (a block of equal rows pools to that row; a ragged last
 *       block of m members divides by m, not by the ratio, which a
 *       wrong-count version fails), float64 means in numpy            (pinned)
 *   tt_oracle_qsa_block_scores
 *       closed forms (one-hot queries read single pooled elements; two heads
 *       with opposite signs give the positive one alone, which a
 *       sum-then-rectify version fails), float64 numpy                (pinned)
 *   tt_oracle_qsa_select_keys
 *       the four cases of the reference's own tests with their expected cells
 *       (tests/TinyTitan/Kernels/Attention/QSAIndexerTests.swift:42-106), an
 *       independent numpy restatement over cells (stable argsort of per-cell
 *       scores), counts and the dense window of
 *       tests/TinyTitan/Runtime/QSAExactnessTests.swift                (pinned)
 *   The norm and the rotation between pooling and scoring are the oracle's
 *   tt_oracle_rms_norm_per_slice and tt_oracle_rope_neox (attn_oracle.c), with
 *   a rounding to fp16 after each stage as the Metal chain stores it; how
 *   Metal's division, rsqrt, pow, cos and sin round is not visible in the
 *   source: PARITY UNPINNED at that level (tests hold the chain to a
 *   tolerance).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define TT_ORACLE_API __attribute__((visibility("default")))

uint16_t tt_oracle_f32_to_f16(float value); /* attn_oracle.c */
float tt_oracle_f16_to_f32(uint16_t bits);

/* qsa_pool_blocks (sources/TinyTitanCore/Metal/Attention/qsa.metal:44-66; the one-block
 * form :20-36 is the same with block_count 1): pooled[b] = mean of the raw keys present
 * in block b, summed in fp32 in member order, one rounding to fp16. */
TT_ORACLE_API int tt_oracle_qsa_pool_blocks(const uint16_t *raw_f16, uint16_t *pooled_f16, int dim, int first_block,
                                            int block_count, int ratio, int n_kv) {
    if (!raw_f16 || !pooled_f16 || dim <= 0 || first_block < 0 || block_count < 0 || ratio <= 0 || n_kv < 0) return -1;
    for (int local = 0; local < block_count; ++local) {
        const long block = (long)first_block + local;
        const long first = block * ratio;
        if (first >= n_kv) continue;
        const int count = (int)((n_kv - first) < ratio ? (n_kv - first) : ratio);
        for (int d = 0; d < dim; ++d) {
            float acc = 0.0f;
            for (int i = 0; i < count; ++i) acc += tt_oracle_f16_to_f32(raw_f16[(first + i) * dim + d]);
            pooled_f16[block * dim + d] = tt_oracle_f32_to_f16(acc / (float)count);
        }
    }
    return 0;
}

/* qsa_block_scores_rows (qsa.metal:106-130; one query row is qsa_block_scores, :76-96):
 * score[t][b] = sum over heads of max(0, dot(q[t][h], pooled[b])), the dot product a chain
 * of fp32 fused multiply-adds in element order, rectified per head before the sum. */
TT_ORACLE_API int tt_oracle_qsa_block_scores(const uint16_t *query_f16, const uint16_t *pooled_f16, float *scores, int dim,
                                             int heads, int blocks, int tokens) {
    if (!query_f16 || !pooled_f16 || !scores || dim <= 0 || heads <= 0 || blocks < 0 || tokens < 0) return -1;
#pragma omp parallel for schedule(static)
    for (long cell = 0; cell < (long)tokens * blocks; ++cell) {
        const long t = cell / blocks, b = cell - t * blocks;
        const uint16_t *row = pooled_f16 + b * dim;
        float total = 0.0f;
        for (int h = 0; h < heads; ++h) {
            const uint16_t *q = query_f16 + (t * heads + h) * dim;
            float dot = 0.0f;
            for (int d = 0; d < dim; ++d) dot = fmaf(tt_oracle_f16_to_f32(q[d]), tt_oracle_f16_to_f32(row[d]), dot);
            total += dot > 0.0f ? dot : 0.0f;
        }
        scores[cell] = total;
    }
    return 0;
}

static const float *g_rank_scores; /* qsort has no context argument; calls are serialised by the binding */

static int rank_before(const void *pa, const void *pb) {
    const int a = *(const int *)pa, b = *(const int *)pb;
    const float sa = g_rank_scores[a], sb = g_rank_scores[b];
    if (sa == sb) return a < b ? -1 : (a > b ? 1 : 0);
    return sa > sb ? -1 : 1;
}

/* QSAIndexer.selectKeys (sources/TinyTitan/Kernels/Attention/QSAIndexer+Scratch.swift:228-262)
 * and one row of selectKeysPrefill (QSAIndexer.swift:455-493): the ragged tail of the query's
 * own block is always kept; complete blocks go in by score descending, lower index first on
 * ties, whole until the cell budget `width` runs out, the next one cut to what remains.
 * With visible <= width every visible key is kept (the prefill form writes that row; the decode
 * form returns no mask): the return value is 0 then, 1 for a real selection, -1 for bad arguments.
 * keep: [visible] bytes.  indices (may be NULL): the kept cells ascending, at most `width`
 * (QSAIndexer.swift:484-492); *count (may be NULL) how many. */
TT_ORACLE_API int tt_oracle_qsa_select_keys(const float *scores, int visible, int ratio, int width, uint8_t *keep,
                                            uint32_t *indices, uint32_t *count) {
    if (!keep || visible < 0 || ratio <= 0 || width < 0) return -1;
    int selected = 0;
    if (visible <= width) {
        memset(keep, 1, (size_t)visible);
    } else {
        selected = 1;
        memset(keep, 0, (size_t)visible);
        const int complete = (visible / ratio) * ratio;
        for (int cell = complete; cell < visible; ++cell) keep[cell] = 1;
        int remaining = width - (visible - complete);
        if (remaining > 0) {
            if (!scores) return -1;
            const int blocks = complete / ratio;
            int *ranked = (int *)malloc(sizeof(int) * (size_t)(blocks > 0 ? blocks : 1));
            if (!ranked) return -1;
            for (int b = 0; b < blocks; ++b) ranked[b] = b;
            g_rank_scores = scores;
            qsort(ranked, (size_t)blocks, sizeof(int), rank_before);
            for (int r = 0; r < blocks && remaining > 0; ++r) {
                const int take = ratio < remaining ? ratio : remaining;
                for (int offset = 0; offset < take; ++offset) keep[ranked[r] * ratio + offset] = 1;
                remaining -= take;
            }
            free(ranked);
        }
    }
    uint32_t written = 0;
    for (int key = 0; key < visible; ++key) {
        if (!keep[key]) continue;
        if ((int)written == width && selected) break;
        if (indices) indices[written] = (uint32_t)key;
        ++written;
    }
    if (count) *count = written;
    return selected;
}
