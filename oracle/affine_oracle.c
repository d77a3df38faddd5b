/*
 * CPU oracle for the affine-quantised output projection (o_proj) that follows
 * the gated attention -- TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker, never the product: only tests/, the smoke check
 * and the benchmark's cpu_baseline leg may build, load or call it.  The
 * library under tinytitan_amd/ must never link or import anything from here.
 *
 * Every function restates one piece of the reference in plain C99 and cites
 * the lines it follows.  Paths are relative to the reference checkout.
 *
 * Pinning status (what checks each function besides this text):
 *   tt_oracle_bf16_bits / tt_oracle_bf16_to_f32
 *       known bit patterns (1.0 -> 0x3F80, the tie cases of round-to-nearest-
 *       even), exact round trip of every bf16 value                  (pinned)
 *   tt_oracle_affine_quantize_rows / tt_oracle_affine_dequantize_rows
 *       the reference's own bounds (|recovered - raw| <= scale + 1e-4,
 *       tests/TinyTitan/Validation/Reference/DequantInt4GEMVReferenceTests.swift:62-80),
 *       closed forms (constant group -> scale 1, bias = value; group minimum
 *       -> level 0, maximum -> top level), hand-packed nibble order  (pinned)
 *   tt_oracle_affine_gemv
 *       bit for bit against the reference's own C kernels
 *       (sources/TinyTitanKernelsC/int4_affine_gemv.c, int8_affine_gemv.c),
 *       compiled from where they lie into oracle/_ref/ by this folder's
 *       Makefile; the reference's closed form (constant row -> value * sum(x),
 *       tests/TinyTitan/Kernels/CPU/Int8AffineGEMVTests.swift:104-110) and its
 *       recorded value 955.4322 / 955.43225 for the two widths (:181-186);
 *       float64 dequantise-then-dot in numpy                         (pinned)
 *   tt_oracle_affine_projection
 *       per token == tt_oracle_affine_gemv followed by one fp16 rounding (the
 *       Metal kernels' `y[row] = half(acc)`,
 *       sources/TinyTitanCore/Metal/Quant/dequant_int4.metal:176-179)  (pinned)
 *       The Metal kernels sum a row in lane order and reduce with simd_sum;
 *       agreement with that summation order is PARITY UNPINNED (the
 *       reference's own bar between its kernel and its fp32 reference is
 *       5e-3 relative, Tolerances.swift:10).
 *   tt_oracle_affine_projection_half_weights
 *       the reference's tensor-operation path for chunks (weight tile rounded to
 *       half, sources/TinyTitanCore/Metal/TensorCore/tensorops.metal:80-125):
 *       float64 product of explicitly fp16-rounded dequantised weights in numpy;
 *       weights exactly representable in fp16 (power-of-two scale) -> equal to
 *       tt_oracle_affine_projection up to fp32 summation order         (pinned)
 *       The order in which Apple's matmul2d sums a 64-column group is not
 *       visible in the source: PARITY UNPINNED at that level.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define TT_ORACLE_API __attribute__((visibility("default")))
#define TT_AFFINE_GROUP 64

uint16_t tt_oracle_f32_to_f16(float value);  /* attn_oracle.c */
float tt_oracle_f16_to_f32(uint16_t bits);

/* sources/TinyTitan/Infrastructure/ModelIO/Quantization.swift:17-28 */
TT_ORACLE_API uint16_t tt_oracle_bf16_bits(float value) {
    uint32_t bits;
    memcpy(&bits, &value, 4);
    const uint32_t lsb = (bits >> 16) & 1u;
    return (uint16_t)((bits + 0x7FFFu + lsb) >> 16);
}

TT_ORACLE_API float tt_oracle_bf16_to_f32(uint16_t bits) {
    const uint32_t wide = (uint32_t)bits << 16;
    float value;
    memcpy(&value, &wide, 4);
    return value;
}

static int affine_shape_ok(int bits, size_t n) {
    return (bits == 4 || bits == 8) && n > 0 && n % TT_AFFINE_GROUP == 0;
}

/*
 * Quantization.quantizeInt4Affine (Quantization.swift:60-113) and
 * quantizeInt8Affine (:158-199): per group of 64, bias = min, scale =
 * (max - min) / top level, both rounded through bf16 before the levels are
 * taken against the rounded values; a constant group stores scale 1.
 * packed: rows * n * bits / 8 bytes, element 2k in the low nibble of byte k.
 */
TT_ORACLE_API int tt_oracle_affine_quantize_rows(int bits, const float *w, size_t rows, size_t n,
                                                 uint8_t *packed, uint16_t *scales, uint16_t *biases) {
    if (!affine_shape_ok(bits, n)) return 1;
    const size_t groups = n / TT_AFFINE_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    const int top = (1 << bits) - 1;
    memset(packed, 0, rows * row_bytes);
    for (size_t r = 0; r < rows; ++r) {
        for (size_t g = 0; g < groups; ++g) {
            const float *wg = w + r * n + g * TT_AFFINE_GROUP;
            float lo = INFINITY, hi = -INFINITY;
            for (int k = 0; k < TT_AFFINE_GROUP; ++k) {
                if (wg[k] < lo) lo = wg[k];
                if (wg[k] > hi) hi = wg[k];
            }
            const float scale_f = hi == lo ? 1.0f : (hi - lo) / (float)top;
            const uint16_t s_bits = tt_oracle_bf16_bits(scale_f), b_bits = tt_oracle_bf16_bits(lo);
            scales[r * groups + g] = s_bits;
            biases[r * groups + g] = b_bits;
            const float scale = tt_oracle_bf16_to_f32(s_bits), bias = tt_oracle_bf16_to_f32(b_bits);
            const float inverse = scale == 0.0f ? 0.0f : 1.0f / scale;
            for (int k = 0; k < TT_AFFINE_GROUP; ++k) {
                long q = lroundf(roundf((wg[k] - bias) * inverse)); /* Swift .rounded(): half away from zero */
                if (q < 0) q = 0;
                if (q > top) q = top;
                if (bits == 8) {
                    packed[r * row_bytes + g * TT_AFFINE_GROUP + k] = (uint8_t)q;
                } else {
                    uint8_t *byte = packed + r * row_bytes + g * (TT_AFFINE_GROUP / 2) + k / 2;
                    *byte = (k & 1) ? (uint8_t)((*byte & 0x0F) | (q << 4)) : (uint8_t)((*byte & 0xF0) | q);
                }
            }
        }
    }
    return 0;
}

/* Quantization.dequantizeInt4Affine (:119-136) / dequantizeInt8Affine (:205-220): level * scale + bias. */
TT_ORACLE_API int tt_oracle_affine_dequantize_rows(int bits, const uint8_t *packed, const uint16_t *scales,
                                                   const uint16_t *biases, size_t rows, size_t n, float *out) {
    if (!affine_shape_ok(bits, n)) return 1;
    const size_t groups = n / TT_AFFINE_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t i = 0; i < n; ++i) {
            const size_t g = i / TT_AFFINE_GROUP;
            const uint8_t byte = packed[r * row_bytes + (bits == 8 ? i : i / 2)];
            const int level = bits == 8 ? byte : ((i & 1) ? byte >> 4 : byte & 0x0F);
            const float scaled = (float)level * tt_oracle_bf16_to_f32(scales[r * groups + g]);
            out[r * n + i] = scaled + tt_oracle_bf16_to_f32(biases[r * groups + g]);
        }
    }
    return 0;
}

/*
 * The reference's C kernels, portable branch: int4_affine_gemv.c:114-134 and
 * int8_affine_gemv.c:123-142.  Per group one running dot and one running
 * sum(x) in element order, then acc += scale * dot + bias * sum(x).
 * x: n floats; out: rows floats, written.
 */
TT_ORACLE_API int tt_oracle_affine_gemv(int bits, const uint8_t *weights, const uint16_t *scales,
                                        const uint16_t *biases, const float *x, size_t rows, size_t n,
                                        float *out) {
    if (!affine_shape_ok(bits, n)) return 1;
    const size_t groups = n / TT_AFFINE_GROUP;
    const size_t row_bytes = n * (size_t)bits / 8;
    for (size_t r = 0; r < rows; ++r) {
        const uint8_t *w_row = weights + r * row_bytes;
        float acc = 0.0f;
        for (size_t g = 0; g < groups; ++g) {
            const float *xg = x + g * TT_AFFINE_GROUP;
            float dot = 0.0f, xsum = 0.0f;
            if (bits == 8) {
                const uint8_t *wg = w_row + g * TT_AFFINE_GROUP;
                for (int k = 0; k < TT_AFFINE_GROUP; ++k) {
                    dot += (float)wg[k] * xg[k];
                    xsum += xg[k];
                }
            } else {
                const uint8_t *wg = w_row + g * (TT_AFFINE_GROUP / 2);
                for (int k = 0; k < TT_AFFINE_GROUP / 2; ++k) {
                    const float x0 = xg[k * 2], x1 = xg[k * 2 + 1];
                    dot += (float)(wg[k] & 0x0F) * x0 + (float)(wg[k] >> 4) * x1;
                    xsum += x0 + x1;
                }
            }
            acc += tt_oracle_bf16_to_f32(scales[r * groups + g]) * dot
                 + tt_oracle_bf16_to_f32(biases[r * groups + g]) * xsum;
        }
        out[r] = acc;
    }
    return 0;
}

/*
 * RealForwardRunner.encodeAffineProjection
 * (sources/TinyTitan/Runtime/Inference/RealForwardRunner+PrefillProjection.swift:53-66)
 * in the shape the runner uses for o_proj (+PrefillAttention.swift:424-436,
 * +BatchAttention.swift:221-240): token t's row x[t * x_stride ..] of
 * `columns` fp16 values times the rows x columns matrix, result rounded to
 * fp16 into y[t * y_stride ..] (dequant_int4.metal:101-180).  x holds
 * fp16-representable floats; y receives the fp16-rounded values as floats.
 */
TT_ORACLE_API int tt_oracle_affine_projection(int bits, const uint8_t *weights, const uint16_t *scales,
                                              const uint16_t *biases, const float *x, size_t rows,
                                              size_t columns, size_t tokens, size_t x_stride, size_t y_stride,
                                              float *y) {
    if (!affine_shape_ok(bits, columns) || x_stride < columns || y_stride < rows) return 1;
    float *lines = (float *)malloc(tokens * rows * sizeof(float));
    if (!lines) return 2;
    /* tokens are independent: the split over threads changes no result */
#pragma omp parallel for schedule(static)
    for (long t = 0; t < (long)tokens; ++t) {
        float *line = lines + (size_t)t * rows;
        tt_oracle_affine_gemv(bits, weights, scales, biases, x + (size_t)t * x_stride, rows, columns, line);
        for (size_t r = 0; r < rows; ++r)
            y[(size_t)t * y_stride + r] = tt_oracle_f16_to_f32(tt_oracle_f32_to_f16(line[r]));
    }
    free(lines);
    return 0;
}

/*
 * The tensor-operation path the runner takes for chunks of 32 tokens and more
 * (MPPPrefillInt4QMM.minimumTokenCount, sources/TinyTitan/Kernels/TensorCore/MPPPrefillInt4QMM.swift:61-64;
 * kernel sources/TinyTitanCore/Metal/TensorCore/tensorops.metal:60-125): per group of 64 columns
 * the weight tile is dequantised to half -- weightTile = half(fma(float(q), scale, bias)) (:93-97) --
 * the group's product of the half activations and the half tile is taken into an fp32
 * groupProduct and added to the fp32 accumulator (:110-113); the result is rounded to half (:124).
 * Same arguments as tt_oracle_affine_projection.
 */
TT_ORACLE_API int tt_oracle_affine_projection_half_weights(int bits, const uint8_t *weights, const uint16_t *scales,
                                                           const uint16_t *biases, const float *x, size_t rows,
                                                           size_t columns, size_t tokens, size_t x_stride,
                                                           size_t y_stride, float *y) {
    if (!affine_shape_ok(bits, columns) || x_stride < columns || y_stride < rows) return 1;
    const size_t groups = columns / TT_AFFINE_GROUP;
    const size_t row_bytes = columns * (size_t)bits / 8;
    float *dense = (float *)malloc(rows * columns * sizeof(float));
    if (!dense) return 2;
    for (size_t r = 0; r < rows; ++r) {
        for (size_t i = 0; i < columns; ++i) {
            const size_t g = i / TT_AFFINE_GROUP;
            const uint8_t byte = weights[r * row_bytes + (bits == 8 ? i : i / 2)];
            const int level = bits == 8 ? byte : ((i & 1) ? byte >> 4 : byte & 0x0F);
            const float w = fmaf((float)level, tt_oracle_bf16_to_f32(scales[r * groups + g]),
                                 tt_oracle_bf16_to_f32(biases[r * groups + g]));
            dense[r * columns + i] = tt_oracle_f16_to_f32(tt_oracle_f32_to_f16(w));
        }
    }
#pragma omp parallel for schedule(static)
    for (long t = 0; t < (long)tokens; ++t) {
        const float *xt = x + (size_t)t * x_stride;
        for (size_t r = 0; r < rows; ++r) {
            const float *wr = dense + r * columns;
            float acc = 0.0f;
            for (size_t g = 0; g < groups; ++g) {
                float product = 0.0f;
                for (int k = 0; k < TT_AFFINE_GROUP; ++k) product += xt[g * TT_AFFINE_GROUP + k] * wr[g * TT_AFFINE_GROUP + k];
                acc += product;
            }
            y[(size_t)t * y_stride + r] = tt_oracle_f16_to_f32(tt_oracle_f32_to_f16(acc));
        }
    }
    free(dense);
    return 0;
}
