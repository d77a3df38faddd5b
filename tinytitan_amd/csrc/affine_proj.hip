// The projection behind the gate: y[t] = W x[t] with W stored as affine levels (4 or 8 bits, one
// bf16 scale and one bf16 bias per group of 64 columns), the runner's o_proj.
//
// Reference: RealForwardRunner.encodeAffineProjection
// (sources/TinyTitan/Runtime/Inference/RealForwardRunner+PrefillProjection.swift:53-66) as called for
// family .o (+PrefillAttention.swift:424-436) and the decode / batched-decode GEMVs behind it
// (DequantInt4GEMV.encode / encodeTwoRows, sources/TinyTitan/Kernels/Quant/DequantInt4GEMV.swift:72-143;
// kernels dequant_int4_gemv_simd / dequant_int4_gemv2_simd, sources/TinyTitanCore/Metal/Quant/dequant_int4.metal:101-280;
// CPU form tinytitan_int4_affine_gemv / tinytitan_int8_affine_gemv, sources/TinyTitanKernelsC).
// Arithmetic, as there: per row and group  scale * sum(level * x) + bias * sum(x)  in fp32, the row
// summed over its groups in fp32 and rounded to fp16 once.
//
// Mapping.  A wavefront owns 32 weight rows x a range of groups for a slab of 32 tokens.  One
// v_mfma_f32_32x32x16_f16 contracts 16 columns: A = 32 tokens x 16 columns of x, B = 16 columns x 32
// weight rows of levels (exact small integers in fp16), so a lane's 16 accumulators are 16 tokens
// of ONE weight row and the group's scale and bias are one value per lane.  A second MFMA per step
// against an all-ones B gives sum(x) of the same tokens in the same accumulator layout.  After the
// four steps of a group: acc += scale * dot + bias * sum(x), 32 fp32 FMAs.  Products of an fp16 x and
// an integer level are exact in the fp32 accumulator; only the order of the sums differs from the
// reference's.
// A lane reads one contiguous 16 bytes (4-bit) or 32 bytes (8-bit) of its weight row per group --
// columns 32 h .. 32 h + 31 of the group for lane half h -- and the x fragments follow that order,
// so weights go HBM -> registers -> MFMA operand with no shuffle and no LDS.
// The waves of a workgroup split the row's groups between them and add their partial rows through
// LDS in a fixed order (no atomics: the result does not depend on timing).
#include <cstdint>

#include "internal.h"

namespace tt {

namespace {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));

constexpr int kProjGroup = 64;      // Quantization.groupSize
constexpr int kProjWaves = 8;       // wavefronts per workgroup, splitting the groups of a row
constexpr int kProjHeld = 8;        // groups of x a wavefront keeps in registers
constexpr int kProjTileRows = 32;   // weight rows per tile = MFMA N
constexpr int kProjSlab = 32;       // tokens per slab = MFMA M

struct ProjArgs {
    const uint8_t *weights;
    const uint16_t *scales, *biases;
    const _Float16 *x;
    _Float16 *y;
    long long x_stride, y_stride;
    int rows, columns, tokens;
    int tiles_per_wg;  // consecutive 32-row tiles one workgroup walks with its x fragments kept
};

// Eight bytes -> eight halves holding 0..255 exactly: byte b under exponent byte 0x64 is 1024 + b.
__device__ __forceinline__ h8 levels_of_bytes(unsigned w0, unsigned w1) {
    const unsigned e = 0x64646464u;
    const u4v v = {__builtin_amdgcn_perm(e, w0, 0x04010400u), __builtin_amdgcn_perm(e, w0, 0x04030402u),
                   __builtin_amdgcn_perm(e, w1, 0x04010400u), __builtin_amdgcn_perm(e, w1, 0x04030402u)};
    return __builtin_bit_cast(h8, v) - (h8)(_Float16)1024;
}
// Eight nibbles of one dword in element order (element 2 k in the low nibble of byte k).
__device__ __forceinline__ h8 levels_of_nibbles(unsigned w) {
    const unsigned lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu, e = 0x64006400u;
    const u4v v = {__builtin_amdgcn_perm(hi, lo, 0x0c040c00u) | e, __builtin_amdgcn_perm(hi, lo, 0x0c050c01u) | e,
                   __builtin_amdgcn_perm(hi, lo, 0x0c060c02u) | e, __builtin_amdgcn_perm(hi, lo, 0x0c070c03u) | e};
    return __builtin_bit_cast(h8, v) - (h8)(_Float16)1024;
}

__device__ __forceinline__ float bf16_value(uint16_t bits) { return __builtin_bit_cast(float, (unsigned)bits << 16); }

// A lane's half group of levels: BITS * 4 bytes.  The reference only promises 2-byte alignment of a
// weight tensor inside its file (DequantInt4GEMV.swift:87-92); ALIGNED = false reads it that way.
template <int BITS, bool ALIGNED>
__device__ __forceinline__ void load_levels(unsigned (&w)[BITS], const uint8_t *src) {
    if constexpr (ALIGNED) {
#pragma unroll
        for (int i = 0; i < BITS / 4; ++i) {
            const u4v v = reinterpret_cast<const u4v *>(src)[i];
            w[4 * i] = v[0];
            w[4 * i + 1] = v[1];
            w[4 * i + 2] = v[2];
            w[4 * i + 3] = v[3];
        }
    } else {
        const uint16_t *p = reinterpret_cast<const uint16_t *>(src);
#pragma unroll
        for (int i = 0; i < BITS; ++i) w[i] = (unsigned)p[2 * i] | ((unsigned)p[2 * i + 1] << 16);
    }
}

template <int BITS, bool ALIGNED>
__global__ __launch_bounds__(kProjWaves * 64) void affine_proj_kernel(const ProjArgs a) {
    extern __shared__ float partial[];  // [wave][accumulator][lane]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int groups = a.columns / kProjGroup;
    const int per_wave = (groups + kProjWaves - 1) / kProjWaves;
    const int g_begin = min(groups, wave * per_wave), g_end = min(groups, g_begin + per_wave);
    constexpr int kHalfGroupBytes = BITS * 4;
    constexpr int kChunk = BITS == 4 ? 8 : 4;  // groups whose levels are in flight together
    const size_t row_bytes = (size_t)a.columns * BITS / 8;

    // x fragments: lane (token c of the slab, half h) holds columns 64 g + 32 h + 8 t .. + 7 for step t.
    const int token = blockIdx.y * kProjSlab + c;
    const bool live = token < a.tokens;
    const _Float16 *x_row = a.x + (long long)min(token, a.tokens - 1) * a.x_stride + 32 * h;
    h8 xa[kProjHeld][4];
    auto load_x = [&](int g0) {
#pragma unroll
        for (int gi = 0; gi < kProjHeld; ++gi) {
            const int g = min(g0 + gi, groups - 1);  // a valid address always
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const h8 v = *reinterpret_cast<const h8 *>(x_row + kProjGroup * g + 8 * t);
                xa[gi][t] = live ? v : (h8)(_Float16)0;
            }
        }
    };
    const bool x_held = g_end - g_begin <= kProjHeld;
    if (x_held) load_x(g_begin);
    const h8 ones = (h8)(_Float16)1;
    const f16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};

    for (int i = 0; i < a.tiles_per_wg; ++i) {
        const int tile = blockIdx.x * a.tiles_per_wg + i;
        if (tile * kProjTileRows >= a.rows) break;  // the whole workgroup
        const int row = min(tile * kProjTileRows + c, a.rows - 1);
        const uint8_t *w_row = a.weights + (size_t)row * row_bytes + h * kHalfGroupBytes;
        const uint16_t *s_row = a.scales + (size_t)row * groups, *b_row = a.biases + (size_t)row * groups;
        f16v acc = zero;
        for (int g0 = g_begin; g0 < g_end; g0 += kProjHeld) {
            if (!x_held) load_x(g0);
#pragma unroll
            for (int sub = 0; sub < kProjHeld; sub += kChunk) {
                if (g0 + sub >= g_end) break;  // the whole wavefront
                unsigned w[kChunk][BITS];
                float scale[kChunk], bias[kChunk];
#pragma unroll
                for (int gi = 0; gi < kChunk; ++gi) {
                    const int g = min(g0 + sub + gi, groups - 1);  // a valid address always
                    load_levels<BITS, ALIGNED>(w[gi], w_row + (size_t)g * (2 * kHalfGroupBytes));
                    scale[gi] = bf16_value(s_row[g]);
                    bias[gi] = bf16_value(b_row[g]);
                }
#pragma unroll
                for (int gi = 0; gi < kChunk; ++gi) {
                    if (g0 + sub + gi >= g_end) break;  // the whole wavefront
                    f16v dot = zero, xsum = zero;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        h8 levels;
                        if constexpr (BITS == 4) levels = levels_of_nibbles(w[gi][t]);
                        else levels = levels_of_bytes(w[gi][2 * t], w[gi][2 * t + 1]);
                        dot = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa[sub + gi][t], levels, dot, 0, 0, 0);
                        xsum = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa[sub + gi][t], ones, xsum, 0, 0, 0);
                    }
#pragma unroll
                    for (int j = 0; j < 16; ++j) acc[j] = fmaf(bias[gi], xsum[j], fmaf(scale[gi], dot[j], acc[j]));
                }
            }
        }
        // Add the waves' partial rows in wave order and write y: accumulator j of lane (c, h) is token
        // 8 (j / 4) + 4 h + j % 4 of the slab, weight row c of the tile.
        if (i > 0) __syncthreads();  // the previous tile's sums have been read
#pragma unroll
        for (int j = 0; j < 16; ++j) partial[(wave * 16 + j) * 64 + lane] = acc[j];
        __syncthreads();
#pragma unroll
        for (int j = wave; j < 16; j += kProjWaves) {
            float sum = 0.0f;
#pragma unroll
            for (int w2 = 0; w2 < kProjWaves; ++w2) sum += partial[(w2 * 16 + j) * 64 + lane];
            const int out_token = blockIdx.y * kProjSlab + 8 * (j / 4) + 4 * h + (j % 4);
            const int out_row = tile * kProjTileRows + c;
            if (out_token < a.tokens && out_row < a.rows) a.y[(long long)out_token * a.y_stride + out_row] = (_Float16)sum;
        }
    }
}

}  // namespace

}  // namespace tt

using namespace tt;

extern "C" int tt_hip_affine_projection(tt_hip_ctx *ctx, int weight_bits, const void *weights, const uint16_t *scales_bf16,
                                        const uint16_t *biases_bf16, const tt_half *x, tt_half *y, int rows, int columns,
                                        int token_count, size_t x_stride_, size_t y_stride_) {
    if (!ctx || !weights || !scales_bf16 || !biases_bf16 || !x || !y) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (rows <= 0 || columns <= 0 || token_count < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (weight_bits != 4 && weight_bits != 8) return TT_HIP_ERR_SHAPE;
    // Quantization.groupSize: the reference's precondition (DequantInt4GEMV.swift:84-86).
    if (columns % kProjGroup != 0) return TT_HIP_ERR_SHAPE;
    const long long x_stride = (long long)x_stride_, y_stride = (long long)y_stride_;
    if (x_stride < columns || y_stride < rows) return TT_HIP_ERR_SHAPE;
    // x rows are read 16 bytes at a time; weights at least 2-byte aligned, scales and biases are 16-bit values.
    if ((uintptr_t)x % 16 != 0 || x_stride % 8 != 0 || (uintptr_t)weights % 2 != 0 || (uintptr_t)y % 2 != 0 ||
        (uintptr_t)scales_bf16 % 2 != 0 || (uintptr_t)biases_bf16 % 2 != 0)
        return TT_HIP_ERR_SHAPE;
    if (token_count == 0) return TT_HIP_OK;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    ProjArgs a{};
    a.weights = static_cast<const uint8_t *>(weights);
    a.scales = scales_bf16;
    a.biases = biases_bf16;
    a.x = reinterpret_cast<const _Float16 *>(x);
    a.y = reinterpret_cast<_Float16 *>(y);
    a.x_stride = x_stride;
    a.y_stride = y_stride;
    a.rows = rows;
    a.columns = columns;
    a.tokens = token_count;
    const int tiles = (rows + kProjTileRows - 1) / kProjTileRows;
    const int slabs = (token_count + kProjSlab - 1) / kProjSlab;
    // One tile per workgroup while that does not yet fill the chip twice; beyond that a workgroup
    // keeps its x fragments and walks several tiles, which divides the reads of x.
    a.tiles_per_wg = 1;
    while (a.tiles_per_wg < 8 && (long long)((tiles + 2 * a.tiles_per_wg - 1) / (2 * a.tiles_per_wg)) * slabs >= 2LL * ctx->n_cus)
        a.tiles_per_wg *= 2;
    const dim3 grid((unsigned)((tiles + a.tiles_per_wg - 1) / a.tiles_per_wg), (unsigned)slabs);
    if (slabs > 65535) return TT_HIP_ERR_SHAPE;
    const size_t lds = (size_t)kProjWaves * 16 * 64 * sizeof(float);
    const bool aligned = (uintptr_t)weights % 16 == 0;
    const bool timed = ctx->profiling && !ctx->capturing && ctx->prof_used + 2 <= ctx->prof_events.size();
    if (timed) (void)hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream);
    if (weight_bits == 4) {
        if (aligned) hipLaunchKernelGGL((affine_proj_kernel<4, true>), grid, dim3(kProjWaves * 64), lds, ctx->stream, a);
        else hipLaunchKernelGGL((affine_proj_kernel<4, false>), grid, dim3(kProjWaves * 64), lds, ctx->stream, a);
    } else {
        if (aligned) hipLaunchKernelGGL((affine_proj_kernel<8, true>), grid, dim3(kProjWaves * 64), lds, ctx->stream, a);
        else hipLaunchKernelGGL((affine_proj_kernel<8, false>), grid, dim3(kProjWaves * 64), lds, ctx->stream, a);
    }
    const hipError_t e = hipGetLastError();
    if (timed) {
        (void)hipEventRecord(ctx->prof_events[ctx->prof_used + 1], ctx->stream);
        ctx->prof_used += 2;
    }
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "affine_proj_kernel launch");
}
