/*
 * CPU oracle for the KV-cache attention path -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, the smoke check
 * and the benchmark's cpu_baseline leg may build, load or call it.  The
 * library under tinytitan_amd/ must never link or import anything from here.
 *
 * Every function restates, in plain C99, one piece of the reference's own CPU
 * attention (Swift, not buildable off macOS) and cites the lines it follows.
 * Paths below are relative to the reference checkout.
 *
 * Pinning status (what checks each function besides this text):
 *   tt_oracle_splitmix64_next / tt_oracle_seedtree_key
 *       published SplitMix64 and FNV-1a known answers            (pinned)
 *   tt_oracle_f32_to_f16 / tt_oracle_f16_to_f32
 *       exhaustive round trip over all 65536 halves + numpy      (pinned)
 *   tt_oracle_softmax_inplace, tt_oracle_sigmoid, tt_oracle_rope_neox
 *       the reference's own closed-form unit checks
 *       (tests/TinyTitan/CPUEngine/CPUEngineTests.swift:909-956) (pinned)
 *   tt_oracle_decode            vs tt_oracle_attention_ref (independent
 *       formulation), an independent numpy restatement, closed forms
 *       (single key, uniform scores, GQA duplicate-head equivalence) (pinned)
 *   tt_oracle_attention_batch   row r == tt_oracle_decode at base+r, vs
 *       tt_oracle_prefill_ref, brute force on tiny shapes.  The reference
 *       holds no test of this function itself and its two contractions run
 *       in Apple Accelerate cblas_sgemm (closed source, macOS SDK, no pinned
 *       version); bit-level agreement with Accelerate's summation order is
 *       PARITY UNPINNED.  Value-level agreement is pinned by the checks above.
 *   tt_oracle_rms_norm_per_slice
 *       the reference's unit checks (CPUEngineTests.swift:886-901), closed
 *       forms (constant slice -> gamma, scale invariance), numpy     (pinned)
 *   tt_oracle_qkv_epilogue      composition of the two pinned pieces above in
 *       the order of CPUQwen35.attention (:266-300); pinned against an
 *       independent numpy statement and by: position 0 == norm only, gate ==
 *       the packed rows' second halves bit for bit, per-token == batch (pinned)
 *   tt_oracle_attention_ref, tt_oracle_prefill_ref
 *       each other, numpy, closed forms (pinned at value level; vDSP/vForce
 *       summation order is PARITY UNPINNED for the same reason).
 *   tt_oracle_kv_row_layout     the reference's own known answers: 1024 / 544 /
 *       288 bytes per 512-element row
 *       (tests/TinyTitan/Kernels/Attention/KVCacheQuantizedAttentionTests.swift:96-98) (pinned)
 *   tt_oracle_kv_quantize_rows, tt_oracle_kv_dequantize_rows
 *       closed forms (constant group -> scale 0 and exact values; group minimum
 *       -> 0 and maximum -> top level; an exactly representable ramp -> its own
 *       indices and an exact round trip; round half away from zero at x.5;
 *       hand-packed nibble order), the error bound scale/2, an independent
 *       numpy statement, and the reference test's own bar on its own seeded
 *       inputs (attention over the quantised rows within 0.02 / 0.20 of the
 *       fp16 result, KVCacheQuantizedAttentionTests.swift:9-83)      (pinned)
 *       Metal compiles with fast math: whether its division is a reciprocal
 *       multiply and its dequantisation a fused multiply-add is not visible in
 *       the source; this file divides and multiplies-then-adds in IEEE fp32.
 *       A value that lands within one fp32 ulp of a rounding boundary could
 *       quantise one level apart there: PARITY UNPINNED at that level.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

#define TT_ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* PRNG: sources/TinyTitanValidation/Support/PRNG/SplitMix64.swift:11-23     */
/* ------------------------------------------------------------------------ */

TT_ORACLE_API uint64_t tt_oracle_splitmix64_next(uint64_t *state) {
    *state += 0x9E3779B97F4A7C15ULL;
    uint64_t z = *state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ULL;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBULL;
    return z ^ (z >> 31);
}

/* Uniform float in [lo, hi), 24-bit mantissa (SplitMix64.swift:26-29). */
TT_ORACLE_API float tt_oracle_splitmix64_uniform(uint64_t *state, float lo, float hi) {
    float u = (float)(tt_oracle_splitmix64_next(state) >> 40) / (float)(1 << 24);
    return lo + (hi - lo) * u;
}

/* Child stream seed = root ^ FNV-1a64(label)
 * (sources/TinyTitanValidation/Support/PRNG/SeedTree.swift:12-19). */
TT_ORACLE_API uint64_t tt_oracle_seedtree_key(uint64_t root, const char *label) {
    uint64_t h = 0xCBF29CE484222325ULL;
    for (const unsigned char *p = (const unsigned char *)label; *p; ++p) {
        h ^= (uint64_t)*p;
        h *= 0x100000001B3ULL;
    }
    return root ^ h;
}

TT_ORACLE_API void tt_oracle_fill_uniform(uint64_t root, const char *label, float lo, float hi,
                                          float *out, size_t count) {
    uint64_t state = tt_oracle_seedtree_key(root, label);
    for (size_t i = 0; i < count; ++i) out[i] = tt_oracle_splitmix64_uniform(&state, lo, hi);
}

/* ------------------------------------------------------------------------ */
/* fp16 storage rounding.  The reference's kernel tests round inputs to       */
/* Float16 and widen them again before the fp32 reference sees them           */
/* (tests/TinyTitan/Kernels/Attention/AttentionTests.swift:200-202).          */
/* IEEE binary16, round-to-nearest-even, written out bit by bit so that it    */
/* shares no code with the compiler's or numpy's conversion.                  */
/* ------------------------------------------------------------------------ */

TT_ORACLE_API uint16_t tt_oracle_f32_to_f16(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    uint32_t sign = (bits >> 16) & 0x8000u;
    uint32_t exponent = (bits >> 23) & 0xFFu;
    uint32_t mantissa = bits & 0x7FFFFFu;
    if (exponent == 0xFFu) { /* inf / nan */
        return (uint16_t)(sign | 0x7C00u | (mantissa ? (0x200u | (mantissa >> 13)) : 0u));
    }
    int32_t e = (int32_t)exponent - 127 + 15;
    if (e >= 31) return (uint16_t)(sign | 0x7C00u); /* overflow -> inf */
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign; /* below half the smallest subnormal */
        mantissa |= 0x800000u;              /* make the leading one explicit */
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half = mantissa >> shift;
        uint32_t rest = mantissa & ((1u << shift) - 1u);
        uint32_t midpoint = 1u << (shift - 1u);
        if (rest > midpoint || (rest == midpoint && (half & 1u))) half += 1u;
        return (uint16_t)(sign | half);
    }
    uint32_t half = ((uint32_t)e << 10) | (mantissa >> 13);
    uint32_t rest = mantissa & 0x1FFFu;
    if (rest > 0x1000u || (rest == 0x1000u && (half & 1u))) half += 1u; /* may carry into inf */
    return (uint16_t)(sign | half);
}

TT_ORACLE_API float tt_oracle_f16_to_f32(uint16_t half) {
    uint32_t sign = ((uint32_t)half & 0x8000u) << 16;
    uint32_t exponent = (half >> 10) & 0x1Fu;
    uint32_t mantissa = half & 0x3FFu;
    uint32_t bits;
    if (exponent == 0) {
        if (mantissa == 0) {
            bits = sign;
        } else { /* subnormal: normalise */
            int shift = 0;
            while (!(mantissa & 0x400u)) { mantissa <<= 1; ++shift; }
            mantissa &= 0x3FFu;
            bits = sign | ((uint32_t)(127 - 15 - shift + 1) << 23) | (mantissa << 13);
        }
    } else if (exponent == 31) {
        bits = sign | 0x7F800000u | (mantissa << 13);
    } else {
        bits = sign | ((exponent - 15 + 127) << 23) | (mantissa << 13);
    }
    float out;
    memcpy(&out, &bits, 4);
    return out;
}

TT_ORACLE_API void tt_oracle_round_through_f16(float *values, size_t count) {
    for (size_t i = 0; i < count; ++i) values[i] = tt_oracle_f16_to_f32(tt_oracle_f32_to_f16(values[i]));
}

TT_ORACLE_API void tt_oracle_f32_to_f16_array(const float *in, uint16_t *out, size_t count) {
    for (size_t i = 0; i < count; ++i) out[i] = tt_oracle_f32_to_f16(in[i]);
}

TT_ORACLE_API void tt_oracle_f16_to_f32_array(const uint16_t *in, float *out, size_t count) {
    for (size_t i = 0; i < count; ++i) out[i] = tt_oracle_f16_to_f32(in[i]);
}

/* ------------------------------------------------------------------------ */
/* CPUOps: sources/TinyTitan/CPUEngine/CPUTensorOps.swift                     */
/* ------------------------------------------------------------------------ */

/* CPUTensorOps.swift:43-46 */
TT_ORACLE_API float tt_oracle_sigmoid(float x) { return 1.0f / (1.0f + expf(-x)); }

/* CPUTensorOps.swift:103-113: peak, expf(x - peak), running total, multiply by 1/total. */
TT_ORACLE_API void tt_oracle_softmax_inplace(float *values, int count) {
    if (count <= 0) return;
    float peak = values[0];
    for (int i = 1; i < count; ++i)
        if (values[i] > peak) peak = values[i];
    float total = 0.0f;
    for (int i = 0; i < count; ++i) {
        float value = expf(values[i] - peak);
        values[i] = value;
        total += value;
    }
    float inverse = 1.0f / total;
    for (int i = 0; i < count; ++i) values[i] *= inverse;
}

/* CPUTensorOps.swift:120-139: NeoX rotation over the first rotary_dim dims of
 * every head; pairs (i, i + rotary_dim/2); frequency theta^(-2i/rotary_dim);
 * angle = position * frequency, all in fp32.  values holds count/head_dim heads. */
TT_ORACLE_API void tt_oracle_rope_neox(float *values, int count, int head_dim, int rotary_dim,
                                       int position, float theta) {
    int half = rotary_dim / 2;
    int heads = count / head_dim;
    for (int head = 0; head < heads; ++head) {
        int base = head * head_dim;
        for (int index = 0; index < half; ++index) {
            float frequency = powf(theta, -(float)index * 2.0f / (float)rotary_dim);
            float angle = (float)position * frequency;
            float cosine = cosf(angle);
            float sine = sinf(angle);
            float a = values[base + index];
            float b = values[base + half + index];
            values[base + index] = a * cosine - b * sine;
            values[base + half + index] = a * sine + b * cosine;
        }
    }
}

/* CPUTensorOps.swift:70-84: RMS norm of each width-long slice with its own
 * statistics, sequential fp32 sum, scale = 1 / sqrt(sum / width + epsilon),
 * out = value * scale * gamma[index]. */
TT_ORACLE_API void tt_oracle_rms_norm_per_slice(float *values, int count, int width, const float *gamma,
                                                float epsilon) {
    int slices = count / width;
    for (int slice = 0; slice < slices; ++slice) {
        int base = slice * width;
        float sum = 0.0f;
        for (int index = 0; index < width; ++index) sum += values[base + index] * values[base + index];
        float scale = 1.0f / sqrtf(sum / (float)width + epsilon);
        for (int index = 0; index < width; ++index) values[base + index] = values[base + index] * scale * gamma[index];
    }
}

/* The arithmetic between the QKV projections and the attention block:
 * CPUQwen35.attention (CPUQwen35.swift:266-300) for one token,
 * CPUQwen35.attentionBatch (CPUQwen35+BatchAttention.swift:49-86) for a chunk
 * whose row r sits at base_position + r.
 *
 *   packed   [tokens][heads][2*dim]   per head [query ; gate]
 *   k_rows   [tokens][kv_heads*dim]
 *   q_out, gate_out [tokens][heads*dim];  k_out [tokens][kv_heads*dim]
 *
 * query and key: per-head RMS norm (gamma shared by all heads), then NeoX
 * sub-dim RoPE; gate is copied; V is not touched by this stage. */
TT_ORACLE_API int tt_oracle_qkv_epilogue(const float *packed, const float *k_rows, int tokens, int heads, int kv_heads,
                                         int dim, const float *q_gamma, const float *k_gamma, float epsilon,
                                         int rotary_dim, float theta, int base_position, float *q_out,
                                         float *gate_out, float *k_out) {
    if (tokens < 0 || heads <= 0 || kv_heads <= 0 || dim <= 0 || rotary_dim < 0 || rotary_dim > dim || rotary_dim % 2)
        return 1;
    int q_width = heads * dim, k_width = kv_heads * dim;
    for (int row = 0; row < tokens; ++row) {
        const float *src = packed + (size_t)row * heads * 2 * dim;
        float *q = q_out + (size_t)row * q_width;
        float *g = gate_out + (size_t)row * q_width;
        float *k = k_out + (size_t)row * k_width;
        for (int head = 0; head < heads; ++head)
            for (int index = 0; index < dim; ++index) {
                q[head * dim + index] = src[head * 2 * dim + index];
                g[head * dim + index] = src[head * 2 * dim + dim + index];
            }
        memcpy(k, k_rows + (size_t)row * k_width, (size_t)k_width * sizeof(float));
        tt_oracle_rms_norm_per_slice(q, q_width, dim, q_gamma, epsilon);
        tt_oracle_rms_norm_per_slice(k, k_width, dim, k_gamma, epsilon);
        tt_oracle_rope_neox(q, q_width, dim, rotary_dim, base_position + row, theta);
        tt_oracle_rope_neox(k, k_width, dim, rotary_dim, base_position + row, theta);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Decode oracle: the attention block of CPUQwen35.attention                  */
/* (sources/TinyTitan/CPUEngine/CPUQwen35.swift:307-351).                     */
/*                                                                            */
/*   query  [heads][dim]                                                      */
/*   gate   [heads][dim] or NULL (no gate)                                    */
/*   keys   [cached][kv_heads*dim]   values likewise (token-major, :85-86)    */
/*   out    [heads][dim]                                                      */
/*                                                                            */
/* kvHead = head / (heads / kv_heads) (:316,325); score = dot * scale with    */
/* the dot accumulated over dim in index order (:329-333); softmaxInPlace     */
/* (:335); weighted V sum skipping weight == 0 (:336-343); out *= sigmoid     */
/* (gate) in fp32 (:351).  The reference derives scale = 1/sqrt(dim) (:317);  */
/* it is an argument here because the GPU dispatch takes it as one            */
/* (sources/TinyTitan/Kernels/Attention/Attention.swift:270-284).             */
/* ------------------------------------------------------------------------ */
TT_ORACLE_API int tt_oracle_decode(const float *query, const float *gate, const float *keys,
                                   const float *values, int cached, int heads, int kv_heads, int dim,
                                   float scale, float *out) {
    if (heads <= 0 || kv_heads <= 0 || dim <= 0 || heads % kv_heads != 0 || cached < 0) return 1;
    int group = heads / kv_heads;
    size_t width = (size_t)kv_heads * (size_t)dim;
    memset(out, 0, sizeof(float) * (size_t)heads * (size_t)dim);
    if (cached == 0) return 0; /* nothing to attend to: zeros, as AttentionRef (Attention.swift:72) */
    float *scores = (float *)malloc(sizeof(float) * (size_t)cached);
    if (!scores) return 2;
    for (int head = 0; head < heads; ++head) {
        int kv_head = head / group;
        size_t query_base = (size_t)head * dim;
        for (int step = 0; step < cached; ++step) {
            size_t base = (size_t)step * width + (size_t)kv_head * dim;
            float total = 0.0f;
            for (int index = 0; index < dim; ++index) total += keys[base + index] * query[query_base + index];
            scores[step] = total * scale;
        }
        tt_oracle_softmax_inplace(scores, cached);
        for (int step = 0; step < cached; ++step) {
            float weight = scores[step];
            if (weight == 0.0f) continue;
            size_t base = (size_t)step * width + (size_t)kv_head * dim;
            for (int index = 0; index < dim; ++index) out[query_base + index] += weight * values[base + index];
        }
    }
    free(scores);
    if (gate) {
        size_t total = (size_t)heads * dim;
        for (size_t index = 0; index < total; ++index) out[index] *= tt_oracle_sigmoid(gate[index]);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Row-major fp32 GEMM standing in for tinytitan_sgemm_rowmajor               */
/* (sources/TinyTitanKernelsC/dequant_affine.c:139-160, which forwards to     */
/* Accelerate cblas_sgemm and is an empty stub off Apple, :151-158).          */
/*   transposed != 0: out[rows, columns] = a[rows, inner] * b[columns, inner]^T */
/*   transposed == 0: out[rows, columns] = a[rows, inner] * b[inner, columns]   */
/* ------------------------------------------------------------------------ */
static int oracle_sgemm_rowmajor(int transposed, int rows, int columns, int inner, const float *a,
                                 const float *b, float *out) {
    /* Every out[r][c] is accumulated over the inner index in ascending order,
     * one multiply and one add per term.  For b^T the operand is first copied
     * to [inner][columns] so that the same loop nest serves both cases and the
     * compiler can vectorise across columns without reordering any sum. */
    float *b_copy = NULL;
    if (transposed) {
        b_copy = (float *)malloc(sizeof(float) * (size_t)inner * (size_t)columns);
        if (!b_copy) return 2;
        for (int c = 0; c < columns; ++c)
            for (int k = 0; k < inner; ++k) b_copy[(size_t)k * columns + c] = b[(size_t)c * inner + k];
        b = b_copy;
    }
    for (int r = 0; r < rows; ++r) {
        float *restrict out_row = out + (size_t)r * columns;
        for (int c = 0; c < columns; ++c) out_row[c] = 0.0f;
        const float *a_row = a + (size_t)r * inner;
        for (int k = 0; k < inner; ++k) {
            float weight = a_row[k];
            const float *restrict b_row = b + (size_t)k * columns;
            for (int c = 0; c < columns; ++c) out_row[c] += weight * b_row[c];
        }
    }
    free(b_copy);
    return 0;
}

/* One head over the whole chunk: CPUQwen35.attentionHead
 * (sources/TinyTitan/CPUEngine/CPUQwen35+BatchAttention.swift:119-178).
 * Gather the head's Q rows and the KV head's K/V rows (:125-139), scores =
 * Q_h * K_h^T (:141-145), per row: limit = base_position + row (:148), scale
 * and peak over columns 0...limit (:157-160), expf and total (:161-166),
 * multiply by 1/total (:167-168), zero the columns past the limit (:169),
 * result = scores * V_h (:172-176).  Returns 3 when a row's limit is past the
 * cache (the reference throws internalInconsistency, :149-152). */
static int oracle_attention_head(const float *query, int tokens, int heads, int head, int dim,
                                 const float *keys, const float *values, int positions, int kv_heads,
                                 int kv_head, int base_position, float scale, float *result) {
    size_t key_width = (size_t)kv_heads * dim;
    float *query_head = (float *)malloc(sizeof(float) * (size_t)tokens * dim);
    float *key_head = (float *)malloc(sizeof(float) * (size_t)positions * dim);
    float *value_head = (float *)malloc(sizeof(float) * (size_t)positions * dim);
    float *scores = (float *)malloc(sizeof(float) * (size_t)tokens * positions);
    int status = 0;
    if (!query_head || !key_head || !value_head || !scores) {
        status = 2;
        goto done;
    }
    for (int row = 0; row < tokens; ++row)
        memcpy(query_head + (size_t)row * dim, query + (size_t)row * heads * dim + (size_t)head * dim,
               sizeof(float) * dim);
    for (int position = 0; position < positions; ++position) {
        size_t from = (size_t)position * key_width + (size_t)kv_head * dim;
        memcpy(key_head + (size_t)position * dim, keys + from, sizeof(float) * dim);
        memcpy(value_head + (size_t)position * dim, values + from, sizeof(float) * dim);
    }
    status = oracle_sgemm_rowmajor(1, tokens, positions, dim, query_head, key_head, scores);
    if (status) goto done;
    for (int row = 0; row < tokens; ++row) {
        int limit = base_position + row;
        if (limit >= positions) {
            status = 3;
            goto done;
        }
        float *score_row = scores + (size_t)row * positions;
        float peak = -INFINITY;
        for (int column = 0; column <= limit; ++column) {
            score_row[column] *= scale;
            if (score_row[column] > peak) peak = score_row[column];
        }
        float total = 0.0f;
        for (int column = 0; column <= limit; ++column) {
            float value = expf(score_row[column] - peak);
            score_row[column] = value;
            total += value;
        }
        float normalization = 1.0f / total;
        for (int column = 0; column <= limit; ++column) score_row[column] *= normalization;
        for (int column = limit + 1; column < positions; ++column) score_row[column] = 0.0f;
    }
    status = oracle_sgemm_rowmajor(0, tokens, dim, positions, scores, value_head, result);
done:
    free(query_head);
    free(key_head);
    free(value_head);
    free(scores);
    return status;
}

/* ------------------------------------------------------------------------ */
/* Prefill / verify oracle: the attention part of CPUQwen35.attentionBatch    */
/* (CPUQwen35+BatchAttention.swift:88-112).                                   */
/*                                                                            */
/*   query  [tokens][heads*dim]     gate likewise or NULL                     */
/*   keys   [positions][kv_heads*dim], ALREADY holding the chunk's own rows   */
/*          at [base_position, base_position+tokens) (:88-92)                 */
/*   out    [tokens][heads*dim]                                               */
/*                                                                            */
/* Per head: attentionHead, scatter back (:97-107); gate in fp32 after the    */
/* value product (:112).  threads > 1 runs heads in parallel -- the           */
/* reference's head loop is serial, so threads == 1 is the faithful setting.  */
/* ------------------------------------------------------------------------ */
TT_ORACLE_API int tt_oracle_attention_batch(const float *query, const float *gate, const float *keys,
                                            const float *values, int tokens, int positions,
                                            int base_position, int heads, int kv_heads, int dim,
                                            float scale, int threads, float *out) {
    if (heads <= 0 || kv_heads <= 0 || dim <= 0 || heads % kv_heads != 0) return 1;
    if (tokens <= 0 || positions <= 0 || base_position < 0) return 1;
    int group = heads / kv_heads;
    size_t query_width = (size_t)heads * dim;
    int status = 0;
#if defined(_OPENMP)
#pragma omp parallel for schedule(dynamic, 1) num_threads(threads > 0 ? threads : 1)
#endif
    for (int head = 0; head < heads; ++head) {
        float *head_out = (float *)malloc(sizeof(float) * (size_t)tokens * dim);
        int local = head_out ? oracle_attention_head(query, tokens, heads, head, dim, keys, values,
                                                     positions, kv_heads, head / group, base_position,
                                                     scale, head_out)
                             : 2;
        if (local == 0) {
            for (int row = 0; row < tokens; ++row)
                memcpy(out + (size_t)row * query_width + (size_t)head * dim, head_out + (size_t)row * dim,
                       sizeof(float) * dim);
        } else {
#if defined(_OPENMP)
#pragma omp critical
#endif
            status = local;
        }
        free(head_out);
    }
    (void)threads;
    if (status) return status;
    if (gate) {
        size_t total = (size_t)tokens * query_width;
        for (size_t index = 0; index < total; ++index) out[index] *= tt_oracle_sigmoid(gate[index]);
    }
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Second, differently ordered decode reference: AttentionRef.apply           */
/* (sources/TinyTitanValidation/Support/Reference/Attention/Attention.swift:  */
/* 14-114).  Full score row per q head, optional sliding window (window <= 0  */
/* means none; kvStart = seq_len - window when seq_len > window, :33-38),     */
/* max-shifted exp, sum, multiply by 1/sum, then one dot per output column    */
/* against V's strided column (:93-110).  scale < 0 selects 1/sqrt(head_dim)  */
/* (:31).  Empty range leaves zeros (:72).  vDSP/vForce are replaced by       */
/* index-order loops.                                                         */
/* ------------------------------------------------------------------------ */
TT_ORACLE_API int tt_oracle_attention_ref(const float *q, const float *k, const float *v, int head_dim,
                                          int num_q_heads, int num_kv_heads, int seq_len, int window,
                                          float scale, float *out) {
    if (num_kv_heads <= 0 || num_q_heads % num_kv_heads != 0 || head_dim <= 0 || seq_len < 0) return 1;
    int group_size = num_q_heads / num_kv_heads;
    if (scale < 0.0f) scale = 1.0f / sqrtf((float)head_dim);
    int kv_start = (window > 0 && seq_len > window) ? seq_len - window : 0;
    int count = seq_len - kv_start;
    memset(out, 0, sizeof(float) * (size_t)num_q_heads * head_dim);
    if (count <= 0) return 0;
    float *scores = (float *)malloc(sizeof(float) * (size_t)count);
    if (!scores) return 2;
    size_t stride = (size_t)num_kv_heads * head_dim;
    for (int qh = 0; qh < num_q_heads; ++qh) {
        int kv_head = qh / group_size;
        const float *q_row = q + (size_t)qh * head_dim;
        for (int p = kv_start; p < seq_len; ++p) {
            const float *k_row = k + ((size_t)p * num_kv_heads + kv_head) * head_dim;
            float dot = 0.0f;
            for (int d = 0; d < head_dim; ++d) dot += q_row[d] * k_row[d];
            scores[p - kv_start] = dot * scale;
        }
        float mx = scores[0];
        for (int i = 1; i < count; ++i)
            if (scores[i] > mx) mx = scores[i];
        float sum = 0.0f;
        for (int i = 0; i < count; ++i) {
            scores[i] = expf(scores[i] - mx);
            sum += scores[i];
        }
        float inv_sum = 1.0f / sum;
        for (int i = 0; i < count; ++i) scores[i] *= inv_sum;
        for (int d = 0; d < head_dim; ++d) {
            const float *column = v + ((size_t)kv_start * num_kv_heads + kv_head) * head_dim + d;
            float acc = 0.0f;
            for (int i = 0; i < count; ++i) acc += scores[i] * column[(size_t)i * stride];
            out[(size_t)qh * head_dim + d] = acc;
        }
    }
    free(scores);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Causal chunk reference with explicit strides: PrefillAttentionRef.apply    */
/* (sources/TinyTitanValidation/Support/Reference/Attention/                  */
/* PrefillAttentionRef.swift:59-101).  Row t (absolute start+t) attends keys  */
/* [first, min(kv_valid, start+t+1)), first = max(0, abs+1-window) when       */
/* window != 0 (:64-71); un-normalised exp weights accumulated per output     */
/* dim, divided by denom when denom > 0 else 0 (:95-96).                      */
/*   q[t*q_stride + h*D + d], k/v[key*kv_stride + kvh*D + d],                 */
/*   out[(t*q_heads + h)*D + d]  (packed, :61)                                */
/* ------------------------------------------------------------------------ */
TT_ORACLE_API int tt_oracle_prefill_ref(const float *q, const float *k, const float *v, int q_stride,
                                        int kv_stride, int head_dim, int q_heads, int kv_heads, int start,
                                        int chunk, int kv_valid, int window, float scale, float *out) {
    if (kv_heads <= 0 || q_heads % kv_heads != 0 || head_dim <= 0 || chunk < 0) return 1;
    int q_per_kv = q_heads / kv_heads;
    memset(out, 0, sizeof(float) * (size_t)chunk * q_heads * head_dim);
    int capacity = start + chunk + 1;
    float *scores = (float *)malloc(sizeof(float) * (size_t)(capacity > 0 ? capacity : 1));
    if (!scores) return 2;
    for (int t = 0; t < chunk; ++t) {
        int abs_q = start + t;
        int first = 0;
        if (window != 0) first = abs_q + 1 - window > 0 ? abs_q + 1 - window : 0;
        int last = kv_valid < abs_q + 1 ? kv_valid : abs_q + 1;
        for (int qh = 0; qh < q_heads; ++qh) {
            int kvh = qh / q_per_kv;
            int count = last - first;
            float max_score = -INFINITY;
            for (int key = first; key < last; ++key) {
                float score = 0.0f;
                for (int d = 0; d < head_dim; ++d)
                    score += q[(size_t)t * q_stride + (size_t)qh * head_dim + d] *
                             k[(size_t)key * kv_stride + (size_t)kvh * head_dim + d];
                score *= scale;
                scores[key - first] = score;
                if (score > max_score) max_score = score;
            }
            float denom = 0.0f;
            for (int i = 0; i < count; ++i) {
                /* the reference recomputes exp(score - max) per output dim (:90-93);
                 * expf is a pure function, so computing it once gives the same bits */
                scores[i] = expf(scores[i] - max_score);
                denom += scores[i];
            }
            for (int d = 0; d < head_dim; ++d) {
                float acc = 0.0f;
                for (int i = 0; i < count; ++i)
                    acc += scores[i] * v[(size_t)(first + i) * kv_stride + (size_t)kvh * head_dim + d];
                out[((size_t)t * q_heads + qh) * head_dim + d] = denom > 0.0f ? acc / denom : 0.0f;
            }
        }
    }
    free(scores);
    return 0;
}

/* ------------------------------------------------------------------------ */
/* Quantised KV rows (affine, one scale and bias per group of consecutive     */
/* elements of a token's row).                                                */
/* ------------------------------------------------------------------------ */

/* KVCacheManager.rowLayout
 * (sources/TinyTitan/Runtime/KVCache/KVCacheManager+Validation.swift:30-41):
 * packed values rounded up to 2 bytes, then one fp16 scale per group, then one
 * fp16 bias per group.  bits = 16 is the plain fp16 row. */
TT_ORACLE_API int tt_oracle_kv_row_layout(int elements, int bits, int group_size, int *stride, int *value_bytes) {
    if (elements <= 0 || group_size <= 0 || (bits != 16 && bits != 8 && bits != 4)) return 1;
    if (bits == 16) {
        *stride = elements * 2;
        *value_bytes = elements * 2;
        return 0;
    }
    int packed = (elements * bits + 7) / 8;
    int aligned_packed = (packed + 1) & ~1;
    int groups = (elements + group_size - 1) / group_size;
    *stride = aligned_packed + groups * 2 * 2;
    *value_bytes = aligned_packed;
    return 0;
}

static float kv_quantize_level(float value, float bias, float scale, float levels) {
    /* kv_cache_quantize.metal:57-60: round(clamp((value - bias) / scale, 0, levels)), 0 when scale == 0;
     * Metal's round() rounds halves away from zero, as roundf does. */
    if (!(scale > 0.0f)) return 0.0f;
    float x = (value - bias) / scale;
    if (x < 0.0f) x = 0.0f;
    if (x > levels) x = levels;
    return roundf(x);
}

/* kv_cache_quantize_affine (sources/TinyTitanCore/Metal/Quant/kv_cache_quantize.metal:7-73).
 * `source` holds fp16-representable values, `source_stride` floats per token;
 * `dest` receives rows of `dest_stride` bytes: packed values, scales, biases.
 * Bytes of the row that the kernel does not write (alignment padding) are left
 * as they are. */
TT_ORACLE_API int tt_oracle_kv_quantize_rows(const float *source, size_t source_stride, int tokens, int elements,
                                             int bits, int group_size, uint8_t *dest, size_t dest_stride) {
    int stride, value_bytes;
    if ((bits != 8 && bits != 4) || tt_oracle_kv_row_layout(elements, bits, group_size, &stride, &value_bytes)) return 1;
    if (dest_stride < (size_t)stride || source_stride < (size_t)elements) return 1;
    if (bits == 4 && (group_size & 1)) return 1; /* a byte's two nibbles share a group (:63-72) */
    const int groups = (elements + group_size - 1) / group_size;
    const float levels = bits == 4 ? 15.0f : 255.0f;
    for (int token = 0; token < tokens; ++token) {
        const float *row_in = source + (size_t)token * source_stride;
        uint8_t *row = dest + (size_t)token * dest_stride;
        for (int group = 0; group < groups; ++group) {
            const int first = group * group_size;
            const int last = first + group_size < elements ? first + group_size : elements;
            float minimum = INFINITY, maximum = -INFINITY; /* :31-32, over the active lanes */
            for (int flat = first; flat < last; ++flat) {
                if (row_in[flat] < minimum) minimum = row_in[flat];
                if (row_in[flat] > maximum) maximum = row_in[flat];
            }
            const float bias = minimum;                                                   /* :42 */
            const float scale = maximum > minimum ? (maximum - minimum) / levels : 0.0f;  /* :43 */
            uint16_t scale_bits = tt_oracle_f32_to_f16(scale), bias_bits = tt_oracle_f32_to_f16(bias);
            memcpy(row + value_bytes + 2 * (size_t)group, &scale_bits, 2);                /* :47-50 */
            memcpy(row + value_bytes + 2 * (size_t)(groups + group), &bias_bits, 2);
            /* the levels come from the fp32 scale and bias, not from their stored halves (:57-60) */
            if (bits == 8) {
                for (int flat = first; flat < last; ++flat)
                    row[flat] = (uint8_t)kv_quantize_level(row_in[flat], bias, scale, levels);
            } else {
                for (int flat = first; flat < last; flat += 2) { /* even lanes write low | high << 4 (:63-72) */
                    uint8_t low = (uint8_t)kv_quantize_level(row_in[flat], bias, scale, levels);
                    uint8_t high = 0;
                    if (flat + 1 < elements) high = (uint8_t)kv_quantize_level(row_in[flat + 1], bias, scale, levels);
                    row[flat / 2] = (uint8_t)(low | (high << 4));
                }
            }
        }
    }
    return 0;
}

/* attn_load_kv (sources/TinyTitanCore/Metal/Attention/attention.metal:89-117):
 * float(level) * float(scale) + float(bias) with the row's stored halves. */
TT_ORACLE_API int tt_oracle_kv_dequantize_rows(const uint8_t *rows, size_t row_stride, int tokens, int elements, int bits,
                                               int group_size, float *out) {
    int stride, value_bytes;
    if ((bits != 8 && bits != 4) || tt_oracle_kv_row_layout(elements, bits, group_size, &stride, &value_bytes)) return 1;
    if (row_stride < (size_t)stride) return 1;
    const int groups = (elements + group_size - 1) / group_size;
    for (int token = 0; token < tokens; ++token) {
        const uint8_t *row = rows + (size_t)token * row_stride;
        for (int flat = 0; flat < elements; ++flat) {
            unsigned level;
            if (bits == 8) {
                level = row[flat];
            } else {
                uint8_t packed = row[flat / 2];
                level = (flat & 1) == 0 ? (unsigned)(packed & 0x0Fu) : (unsigned)(packed >> 4);
            }
            const int group = flat / group_size;
            uint16_t scale_bits, bias_bits;
            memcpy(&scale_bits, row + value_bytes + 2 * (size_t)group, 2);
            memcpy(&bias_bits, row + value_bytes + 2 * (size_t)(groups + group), 2);
            out[(size_t)token * elements + flat] =
                (float)level * tt_oracle_f16_to_f32(scale_bits) + tt_oracle_f16_to_f32(bias_bits);
        }
    }
    return 0;
}

/* Number of worker threads the head-parallel variant can use. */
TT_ORACLE_API int tt_oracle_max_threads(void) {
#if defined(_OPENMP)
    return omp_get_max_threads();
#else
    return 1;
#endif
}
