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
#include "wave_ops.h"

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
constexpr int kStagePitch = 2 * kProjGroup + 8;  // halves per token of a wavefront's x patch in LDS: two groups + 16 B
constexpr int kProjLdsBytes = kProjWaves * 16 * 64 * 4 + kProjWaves * kProjSlab * kStagePitch * 2;

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

// N consecutive bf16 values of a row, two to a register (the even group in the low half); past the row's
// end the last value again.
template <int N>
__device__ __forceinline__ void load_params(unsigned (&dst)[N / 2], const uint16_t *row, int first, int groups, bool vector) {
    if (vector) {
        if constexpr (N == 8) {
            const u4v v = *reinterpret_cast<const u4v *>(row + first);
            dst[0] = v[0];
            dst[1] = v[1];
            dst[2] = v[2];
            dst[3] = v[3];
        } else if constexpr (N == 4) {
            typedef unsigned u2v __attribute__((ext_vector_type(2)));
            const u2v v = *reinterpret_cast<const u2v *>(row + first);
            dst[0] = v[0];
            dst[1] = v[1];
        } else {
            static_assert(N == 2, "8, 4 or 2 values");
            dst[0] = *reinterpret_cast<const unsigned *>(row + first);
        }
    } else {
#pragma unroll
        for (int i = 0; i < N / 2; ++i)
            dst[i] = (unsigned)row[min(first + 2 * i, groups - 1)] | ((unsigned)row[min(first + 2 * i + 1, groups - 1)] << 16);
    }
}

template <int BITS, bool ALIGNED>
__global__ __launch_bounds__(kProjWaves * 64) void affine_proj_kernel(const ProjArgs a) {
    extern __shared__ float partial[];  // [wave][accumulator][lane], then each wavefront's x patch
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int c = lane & 31, h = lane >> 5;
    const int groups = a.columns / kProjGroup;
    const int per_wave = (groups + kProjWaves - 1) / kProjWaves;
    const int g_begin = min(groups, wave * per_wave), g_end = min(groups, g_begin + per_wave);
    constexpr int kHalfGroupBytes = BITS * 4;
    constexpr int kChunk = BITS == 4 ? 4 : 2;  // groups whose levels are in flight together
    const size_t row_bytes = (size_t)a.columns * BITS / 8;

    // x fragments: lane (token c of the slab, half h) holds columns 64 g + 32 h + 8 t .. + 7 for step t.
    const bool live = (int)blockIdx.y * kProjSlab + c < a.tokens;
    // They come through LDS: straight from global memory a lane would read 16 bytes of its own token's row per
    // instruction -- 32 cache lines touched for 1 KiB, each line touched again by three later instructions and by
    // then evicted by the other wavefronts' rows.  Instead the wavefront reads two groups of all 32 tokens with
    // whole lines (16 lanes = 256 contiguous bytes of a token), writes them to its own patch of LDS (rows padded
    // by 16 B) and reads the fragments back; LDS serves a wavefront's accesses in order, so no barrier is needed.
    h8 xa[kProjHeld][4];
    _Float16 *const stage = reinterpret_cast<_Float16 *>(partial + kProjWaves * 16 * 64) + wave * (kProjSlab * kStagePitch);
    auto load_x = [&](int g0) {
        h8 raw[2][8];
        auto fetch = [&](h8 (&dst)[8], int pair) {
            const int g = min(g0 + 2 * pair + ((lane >> 3) & 1), groups - 1);  // a valid address always
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int t = min((int)blockIdx.y * kProjSlab + 4 * i + (lane >> 4), a.tokens - 1);
                dst[i] = *reinterpret_cast<const h8 *>(a.x + (long long)t * a.x_stride + kProjGroup * g + 8 * (lane & 7));
            }
        };
        fetch(raw[0], 0);
#pragma unroll
        for (int pair = 0; pair < kProjHeld / 2; ++pair) {
            if (pair + 1 < kProjHeld / 2) fetch(raw[(pair + 1) & 1], pair + 1);
#pragma unroll
            for (int i = 0; i < 8; ++i)
                *reinterpret_cast<h8 *>(stage + (4 * i + (lane >> 4)) * kStagePitch + 8 * (lane & 15)) = raw[pair & 1][i];
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int gi = 0; gi < 2; ++gi)
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const h8 v = *reinterpret_cast<const h8 *>(stage + c * kStagePitch + kProjGroup * gi + 32 * h + 8 * t);
                    xa[2 * pair + gi][t] = live ? v : (h8)(_Float16)0;
                }
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        }
    };
    const bool x_held = g_end - g_begin <= kProjHeld;  // then loaded once, with the first tile
    // a row's N scales (N * 2 bytes) in one load where every such run is aligned
    const bool params_vector = groups % kChunk == 0 && per_wave % kChunk == 0 && (uintptr_t)a.scales % (2 * kChunk) == 0 &&
                               (uintptr_t)a.biases % (2 * kChunk) == 0;
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
#pragma unroll
            for (int sub = 0; sub < kProjHeld; sub += kChunk) {
                if (g0 + sub >= g_end) break;  // the whole wavefront
                unsigned w[kChunk][BITS];
                unsigned scale_pairs[kChunk / 2], bias_pairs[kChunk / 2];
#pragma unroll
                for (int gi = 0; gi < kChunk; ++gi) {
                    const int g = min(g0 + sub + gi, groups - 1);  // a valid address always
                    load_levels<BITS, ALIGNED>(w[gi], w_row + (size_t)g * (2 * kHalfGroupBytes));
                }
                load_params<kChunk>(scale_pairs, s_row, g0 + sub, groups, params_vector);
                load_params<kChunk>(bias_pairs, b_row, g0 + sub, groups, params_vector);
                // x (re)loaded while the levels are on their way
                if (sub == 0 && (!x_held || i == 0)) load_x(g0);
                // Every load of the chunk is issued before its first use: left to itself the scheduler
                // sinks each group's loads to its MFMAs and the wavefront waits for memory once per group.
                __builtin_amdgcn_sched_barrier(0);
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
                    // a bf16 is the upper half of the float
                    const unsigned sp = scale_pairs[gi / 2], bp = bias_pairs[gi / 2];
                    const float scale = __builtin_bit_cast(float, (gi & 1) ? (sp & 0xffff0000u) : (sp << 16));
                    const float bias = __builtin_bit_cast(float, (gi & 1) ? (bp & 0xffff0000u) : (bp << 16));
#pragma unroll
                    for (int j = 0; j < 16; ++j) acc[j] = fmaf(bias, xsum[j], fmaf(scale, dot[j], acc[j]));
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

// ---------------------------------------------------------------------------
// Up to nine tokens (a decode row, the two-row and four-row verify passes, a small decode batch): the matrix cores
// have little to amortise, and 32-row tiles would leave three quarters of the chip idle at 2048 rows.
// Here a workgroup owns 8 weight rows and its eight wavefronts take the columns 512 at a time in
// turn: a lane takes 8 consecutive columns of each row (one dword of nibbles or two of bytes,
// coalesced; they lie in one group), widens them to fp16 levels and contracts them with its 8 x
// values by v_dot2_f32_f16 (products exact, fp32 accumulation), then
// acc += scale * dot + bias * sum(x) as above.  All of a wavefront's loads for a 512-column chunk
// are independent, so they are in flight together; lanes are added by DPP moves (six vector instructions a
// sum; as six shuffles through LDS each, the 8 x TOK sums were most of the kernel: one token 5.5 -> 4.2 us a step,
// four tokens 11.0 -> 6.3, which moved the hand-over to the MFMA kernel's flat 10.6 us from 5 tokens to 10),
// wavefronts through LDS in a fixed order.  256 workgroups at 2048 rows.
// ---------------------------------------------------------------------------
constexpr int kGemvWaves = 8, kGemvRows = 8, kGemvMaxTokens = 9;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ float dot8(h8 a, h8 b) {
    float d = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const h2 ai = {a[2 * i], a[2 * i + 1]}, bi = {b[2 * i], b[2 * i + 1]};
        d = __builtin_amdgcn_fdot2(ai, bi, d, false);
    }
    return d;
}

template <int BITS, int TOK, bool ALIGNED>
__global__ __launch_bounds__(kGemvWaves * 64) void affine_gemv_kernel(const ProjArgs a) {
    __shared__ float partial[kGemvWaves][kGemvRows * TOK];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int row0 = blockIdx.x * kGemvRows;
    const int groups = a.columns / kProjGroup;
    const int chunks = (a.columns + 511) / 512;
    const size_t row_bytes = (size_t)a.columns * BITS / 8;
    const h8 ones = (h8)(_Float16)1;
    float acc[kGemvRows][TOK];
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
        for (int t = 0; t < TOK; ++t) acc[r][t] = 0.0f;
#pragma unroll 1  // one straight-line body: every load of a chunk is issued before the first use
    for (int chunk = wave; chunk < chunks; chunk += kGemvWaves) {
        const int wanted = 512 * chunk + 8 * lane;
        const bool inside = wanted < a.columns;
        const int column = inside ? wanted : 0;  // a valid address always
        h8 xv[TOK];
        float xsum[TOK];
#pragma unroll
        for (int t = 0; t < TOK; ++t) {  // loaded from a valid address; zeroed below where the lane is past the row
            xv[t] = *reinterpret_cast<const h8 *>(a.x + (long long)t * a.x_stride + column);
        }
        const int g = column / kProjGroup;
        unsigned w[kGemvRows][BITS / 4];
        uint16_t scale_bits[kGemvRows], bias_bits[kGemvRows];
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) {
            const int row = min(row0 + r, a.rows - 1);
            const uint8_t *src = a.weights + (size_t)row * row_bytes + (size_t)column * BITS / 8;
#pragma unroll
            for (int i = 0; i < BITS / 4; ++i) {
                if constexpr (ALIGNED) w[r][i] = reinterpret_cast<const unsigned *>(src)[i];
                else w[r][i] = (unsigned)reinterpret_cast<const uint16_t *>(src)[2 * i] |
                               ((unsigned)reinterpret_cast<const uint16_t *>(src)[2 * i + 1] << 16);
            }
            scale_bits[r] = a.scales[(size_t)row * groups + g];
            bias_bits[r] = a.biases[(size_t)row * groups + g];
        }
        // Every load above is issued before anything below: left to itself the scheduler sinks each
        // load to its use to save registers and the wavefront then waits for them one by one.
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
            xv[t] = inside ? xv[t] : (h8)(_Float16)0;
            xsum[t] = dot8(xv[t], ones);
        }
#pragma unroll
        for (int r = 0; r < kGemvRows; ++r) {
            h8 levels;
            if constexpr (BITS == 4) levels = levels_of_nibbles(w[r][0]);
            else levels = levels_of_bytes(w[r][0], w[r][1]);
            const float scale = bf16_value(scale_bits[r]), bias = bf16_value(bias_bits[r]);
#pragma unroll
            for (int t = 0; t < TOK; ++t) acc[r][t] = fmaf(bias, xsum[t], fmaf(scale, dot8(xv[t], levels), acc[r][t]));
        }
    }
#pragma unroll
    for (int r = 0; r < kGemvRows; ++r)
#pragma unroll
        for (int t = 0; t < TOK; ++t) {
            const float v = wave_sum_in_lane63(acc[r][t]);
            if (lane == 63) partial[wave][r * TOK + t] = v;
        }
    __syncthreads();
    if (threadIdx.x < kGemvRows * TOK) {
        const int r = threadIdx.x / TOK, t = threadIdx.x % TOK;
        float v = 0.0f;
#pragma unroll
        for (int w2 = 0; w2 < kGemvWaves; ++w2) v += partial[w2][threadIdx.x];
        if (row0 + r < a.rows) a.y[(long long)t * a.y_stride + row0 + r] = (_Float16)v;
    }
}

template <int BITS, bool ALIGNED>
void launch_gemv(tt_hip_ctx *ctx, const ProjArgs &a) {
    const dim3 grid((unsigned)((a.rows + kGemvRows - 1) / kGemvRows));
    const dim3 block(kGemvWaves * 64);
    switch (a.tokens) {
        case 1: launch_profiled(ctx, affine_gemv_kernel<BITS, 1, ALIGNED>, grid, block, 0u, a); break;
        case 2: launch_profiled(ctx, affine_gemv_kernel<BITS, 2, ALIGNED>, grid, block, 0u, a); break;
        case 3: launch_profiled(ctx, affine_gemv_kernel<BITS, 3, ALIGNED>, grid, block, 0u, a); break;
        case 4: launch_profiled(ctx, affine_gemv_kernel<BITS, 4, ALIGNED>, grid, block, 0u, a); break;
        case 5: launch_profiled(ctx, affine_gemv_kernel<BITS, 5, ALIGNED>, grid, block, 0u, a); break;
        case 6: launch_profiled(ctx, affine_gemv_kernel<BITS, 6, ALIGNED>, grid, block, 0u, a); break;
        case 7: launch_profiled(ctx, affine_gemv_kernel<BITS, 7, ALIGNED>, grid, block, 0u, a); break;
        case 8: launch_profiled(ctx, affine_gemv_kernel<BITS, 8, ALIGNED>, grid, block, 0u, a); break;
        default: launch_profiled(ctx, affine_gemv_kernel<BITS, 9, ALIGNED>, grid, block, 0u, a); break;
    }
}

// ---------------------------------------------------------------------------
// A prefill chunk (513 tokens and more): a GEMM.  The reference's tensor-operation path for these
// (MPPPrefillInt4QMM, kernel sources/TinyTitanCore/Metal/TensorCore/tensorops.metal:60-125, taken from 32
// tokens on) dequantises a weight tile to HALF -- weightTile = half(fma(float(q), scale, bias)) --
// and multiplies half tiles into an fp32 accumulator; this kernel does the same: a level becomes
// the fp16 number level * scale + bias (one fused fp16 multiply-add: the exact value rounded once,
// where the reference rounds through fp32 first; scale and bias are bf16 values, exact in fp16
// within its range), and x . w accumulates in fp32 on the matrix cores.
//
// A workgroup of 4 wavefronts owns 128 tokens x 128 weight rows; a wavefront 32 of the rows against all
// 128 tokens, four 32x32 accumulators (no row's levels are widened twice).  Per group of 64 columns:
// the x tile (128 x 64) goes global -> registers -> LDS (one copy per workgroup, double buffered, rows
// padded to 144 B so that the fragment reads are conflict-free) and is read as A fragments; a lane
// reads its own 16 / 32 bytes of levels of its weight row straight from global memory, widens and
// scales them in registers into the B fragments of a group (no LDS, no shuffle), and 16 MFMAs per
// group follow (4 contraction steps x 4 token tiles), each step's A fragments read while the step before it
// multiplies; the rows' scales and biases come from a block in LDS, converted to fp16 once.  One barrier per
// group, in its middle.  The output tile leaves through LDS, [token][row], as 16-byte stores.
// ---------------------------------------------------------------------------
constexpr int kGemmTokens = 128, kGemmWaves = 4, kGemmRows = 32 * kGemmWaves;
// From here on the GEMM is the faster of the two MFMA kernels at 2048 x 4096: 39-40 us up to 1024 tokens and 48 us
// at 2048, where its grid fills the chip, against 33 us at 512 tokens and 45 us and more from 513 on for the factored
// kernel, whose workgroups then come in a third round.
constexpr int kGemmMinTokens = 513;
constexpr int kGemmThreads = kGemmWaves * 64;
constexpr int kGemmPitch = kProjGroup + 8;                           // halves per token row of the x tile in LDS
constexpr int kGemmParamGroups = 64;                                 // groups whose scales and biases sit in LDS at a time
constexpr int kGemmTileHalves = kGemmTokens * kGemmPitch;
constexpr int kGemmOutPitch = kGemmRows + 8;                         // halves per token of the output tile in LDS
static_assert(kGemmTokens * kGemmOutPitch <= 2 * kGemmTileHalves, "the output tile takes the x tiles' space");
// KS = parts the columns are split into inside a workgroup (1 or 2): KS x 4 wavefronts, part p's four take the
// groups [p x part_groups, (p + 1) x part_groups) with x tiles and a block of scales and biases of their own, and
// the parts' accumulators are added through LDS at the end, in a fixed order.  For chunks whose tiles number no
// more than the CUs: a workgroup's time is that of ONE wavefront's walk over the columns (44 us at 4096 columns,
// whatever the number of tiles); in two parts it is 39-40 us, and 48-51 us instead of 56-57 at 2048 tokens, where
// every CU has a workgroup.
constexpr int gemm_lds_bytes(int ks) { return ks * 2 * kGemmTileHalves * (int)sizeof(_Float16) + kGemmParamGroups * kGemmRows * 4; }
constexpr int gemm_rs_lds_bytes() { return 2 * kGemmTileHalves * (int)sizeof(_Float16) + kGemmParamGroups * 2 * kGemmRows * 4; }

template <int BITS, bool ALIGNED, int KS, bool RS = false>
__global__ __launch_bounds__(kGemmThreads * KS, 2) void affine_gemm_kernel(const ProjArgs a) {
    // RS (with KS = 2): the two parts split the ROWS instead of the columns -- a tile of 128 tokens x 256 rows, one x
    // tile for all eight wavefronts.
    constexpr int kThreads = kGemmThreads * KS, kPartParamGroups = RS ? kGemmParamGroups : kGemmParamGroups / KS;
    constexpr int kRows = RS ? kGemmRows * KS : kGemmRows;
    constexpr int kStageThreads = RS ? kThreads : kGemmThreads, kStagePasses = kGemmTokens * 8 / kStageThreads;
    static_assert(kGemmWaves * 64 * 64 * (int)sizeof(float) <= gemm_lds_bytes(2), "the parts' accumulators meet in the store");
    // per part two x tiles of kGemmTokens x kGemmPitch halves, then per part [kPartParamGroups][kGemmRows] (scale, bias) pairs as fp16
    extern __shared__ __attribute__((aligned(16))) _Float16 lds_store[];
    const int part = __builtin_amdgcn_readfirstlane((int)threadIdx.x / kGemmThreads);
    const int tid = threadIdx.x % kGemmThreads, lane = tid & 63, wave = tid >> 6;  // tid, wave: inside the part
    const int stage_tid = RS ? (int)threadIdx.x : tid;
    auto tile = [&](int which) { return lds_store + ((RS ? 0 : 2 * part) + which) * kGemmTileHalves; };
    unsigned *const params = reinterpret_cast<unsigned *>(lds_store + (RS ? 1 : KS) * 2 * kGemmTileHalves) + (RS ? 0 : part * kPartParamGroups * kRows);
    const int c = lane & 31, h = lane >> 5;
    // A wavefront owns 32 weight rows against all 128 tokens: every row's levels are widened by exactly one wavefront.
    // Workgroups are dealt to the 8 XCDs in turn, each with its own L2: the workgroups that share a token block
    // (its x rows are what they all read) get ids congruent modulo 8, i.e. one XCD.
    const int row_blocks = (a.rows + kRows - 1) / kRows;
    const int id = blockIdx.x;
    const int token_block = (id & 7) + 8 * (id / (8 * row_blocks));
    if (token_block * kGemmTokens >= a.tokens) return;  // the whole workgroup, before any barrier: padding of the grid
    const int token0 = token_block * kGemmTokens, row0 = ((id >> 3) % row_blocks) * kRows;
    const int groups = a.columns / kProjGroup;
    constexpr int kHalfGroupBytes = BITS * 4;
    // Levels are read kSpan groups at a time: a lane's 64 contiguous bytes of its row, so that a 128-byte line
    // is fetched once and used whole (16 bytes per group would touch the line again for each of its groups).
    constexpr int kSpan = BITS == 4 ? 4 : 2;
    // This part's groups: [first_group, first_group + part_groups), whole spans; below, g counts from first_group.
    constexpr int kColumnParts = RS ? 1 : KS;
    const int part_groups = (groups + kColumnParts * kSpan - 1) / (kColumnParts * kSpan) * kSpan, first_group = RS ? 0 : part * part_groups;
    const size_t row_bytes = (size_t)a.columns * BITS / 8;

    // x staging: thread -> 16 bytes (8 columns) of token tid / 8 (+ 32 per further pass): 8 threads read a row's 128 B
    const _Float16 *x_src[kStagePasses];
    int x_dst[kStagePasses];
#pragma unroll
    for (int p = 0; p < kStagePasses; ++p) {
        const int local = (stage_tid >> 3) + (kStageThreads / 8) * p;
        x_src[p] = a.x + (long long)min(token0 + local, a.tokens - 1) * a.x_stride + 8 * (stage_tid & 7);
        x_dst[p] = local * kGemmPitch + 8 * (stage_tid & 7);
    }
    const int param_at = (RS ? kGemmRows * part : 0) + 32 * wave + c;  // this lane's weight row inside the workgroup's tile
    const uint8_t *const w_src = a.weights + (size_t)min(row0 + param_at, a.rows - 1) * row_bytes;
    // Scales and biases of this workgroup's rows for groups [first, first + kGemmParamGroups): a thread takes eight
    // consecutive groups of a row, 16 bytes of scales and 16 of biases, and eight threads a row's 128 bytes, so the
    // rows are read as whole lines (one value per thread and load made 64 loads of 2 bytes per thread, every lane on
    // a line of its own: 16 us of a 107 us launch at 4096 tokens).  Converted to fp16 and stored [group][row], so that
    // the lanes of a wavefront -- consecutive rows -- read consecutive words.
    constexpr int kRowThreads = kPartParamGroups / 8, kPassRows = kStageThreads / kRowThreads;
    static_assert(kGemmParamGroups == 64 && kGemmThreads == 256 && kRows % kPassRows == 0, "eight groups a thread");
    const bool params_vector = (uintptr_t)a.scales % 16 == 0 && (uintptr_t)a.biases % 16 == 0 && groups % 8 == 0;
    auto stage_params = [&](int first) {
        const int k = 8 * (stage_tid % kRowThreads), g = first_group + first + k;
        const bool vector = params_vector && g + 8 <= groups;
#pragma unroll
        for (int i = 0; i < kRows / kPassRows; ++i) {
            const int local = stage_tid / kRowThreads + kPassRows * i;
            const size_t at = (size_t)min(row0 + local, a.rows - 1) * groups;
            unsigned scale_bits[4], bias_bits[4];
            load_params<8>(scale_bits, a.scales + at, g, groups, vector);
            load_params<8>(bias_bits, a.biases + at, g, groups, vector);
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const _Float16 scale = (_Float16)bf16_value((uint16_t)(scale_bits[j / 2] >> (16 * (j & 1))));
                const _Float16 bias = (_Float16)bf16_value((uint16_t)(bias_bits[j / 2] >> (16 * (j & 1))));
                params[(k + j) * kRows + local] = (unsigned)__builtin_bit_cast(uint16_t, scale) |
                                                      ((unsigned)__builtin_bit_cast(uint16_t, bias) << 16);
            }
        }
    };
    const f16v zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    f16v acc[4] = {zero, zero, zero, zero};  // one per 32-token tile

    // x rows are loaded two groups ahead of their use: slot g % 2 of x_ring holds group g's rows until they go
    // to LDS at the start of group g - 1 (the loop over a span is unrolled and spans are even, so the slot is a
    // constant).
    h8 x_ring[2][kStagePasses];
    auto load_x = [&](h8 (&dst)[kStagePasses], int g) {
        const int gc = min(first_group + g, groups - 1);  // past the end: the last group again, a valid address, unused
#pragma unroll
        for (int p = 0; p < kStagePasses; ++p) dst[p] = *reinterpret_cast<const h8 *>(x_src[p] + kProjGroup * gc);
    };
    auto store_x = [&](const h8 (&src)[kStagePasses], int g) {
#pragma unroll
        for (int p = 0; p < kStagePasses; ++p) *reinterpret_cast<h8 *>(tile(g & 1) + x_dst[p]) = src[p];
    };
    unsigned w_now[kSpan][BITS], w_next[kSpan][BITS];
    auto load_span = [&](unsigned (&w)[kSpan][BITS], int first) {
#pragma unroll
        for (int k = 0; k < kSpan; ++k) {
            const int g = min(first_group + first + k, groups - 1);  // past the end: the last group again, a valid address, unused
            load_levels<BITS, ALIGNED>(w[k], w_src + (size_t)g * (2 * kHalfGroupBytes) + h * kHalfGroupBytes);
        }
    };
    load_x(x_ring[0], 0);
    load_x(x_ring[1], 1);
    load_span(w_next, 0);
    stage_params(0);
    store_x(x_ring[0], 0);
    load_x(x_ring[0], 2);
    __syncthreads();

    // B fragments of a group: its levels widened and scaled, bw[g % 2].  They are made one group ahead, in the
    // shadow of the previous group's MFMAs: the matrix pipe takes 32 cycles per MFMA and the wavefront issues the
    // next group's VALU work meanwhile, instead of widening first and multiplying after.
    h8 bw[2][4];
    auto widen_scale = [&](h8 &dst, const unsigned (&w)[BITS], int t, h8 scale, h8 bias) {
        h8 levels;
        if constexpr (BITS == 4) levels = levels_of_nibbles(w[t]);
        else levels = levels_of_bytes(w[2 * t], w[2 * t + 1]);
        dst = __builtin_elementwise_fma(levels, scale, bias);
    };
    // Past the matrix's last group the scale and the bias are zero: such a group's products add nothing, and the
    // loop over a span needs no exit in its middle.
    auto pair_of = [&](int g) { return first_group + g < groups ? params[(g % kPartParamGroups) * kRows + param_at] : 0u; };
    auto scale_of = [&](unsigned pair) { return (h8)__builtin_bit_cast(_Float16, (uint16_t)(pair & 0xffffu)); };
    auto bias_of = [&](unsigned pair) { return (h8)__builtin_bit_cast(_Float16, (uint16_t)(pair >> 16)); };
    {
        const unsigned pair = pair_of(0);
#pragma unroll
        for (int t = 0; t < 4; ++t) widen_scale(bw[0][t], w_next[0], t, scale_of(pair), bias_of(pair));
    }
    // A fragments of contraction step t of a group: 32 tokens x 16 columns per token tile, af[t % 2]; a step's
    // fragments are read from LDS while the step before it multiplies.
    h8 af[2][4];
    auto read_fragments = [&](h8 (&dst)[4], int g, int t) {
        const _Float16 *xt = tile(g & 1);
#pragma unroll
        for (int tt = 0; tt < 4; ++tt) dst[tt] = *reinterpret_cast<const h8 *>(xt + (32 * tt + c) * kGemmPitch + 32 * h + 8 * t);
    };
    read_fragments(af[0], 0, 0);

    for (int g0 = 0; g0 < part_groups; g0 += kSpan) {
#pragma unroll
        for (int k = 0; k < kSpan; ++k)
#pragma unroll
            for (int i = 0; i < BITS; ++i) w_now[k][i] = w_next[k][i];
        load_span(w_next, g0 + kSpan);  // the next span's levels are in flight for the whole of this one
#pragma unroll
        for (int k = 0; k < kSpan; ++k) {
            const int g = g0 + k;
            static_assert(kSpan % 2 == 0, "the ring slots of a group must not depend on the span");
            // Group g + 1's rows go to the tile that group g - 1 was read from (every wavefront is past that
            // group's barrier, behind which nobody reads it), and their registers take group g + 3's.
            store_x(x_ring[(k + 1) & 1], g + 1);
            load_x(x_ring[(k + 1) & 1], g + 3);
            const unsigned pair_next = pair_of(g + 1);
            const h8 scale_next = scale_of(pair_next), bias_next = bias_of(pair_next);
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                __builtin_amdgcn_sched_barrier(0);
                if (t == 3) {
                    // Everybody's rows of group g + 1 are in LDS from here on, and nobody reads group g's any more.
                    __syncthreads();
                    read_fragments(af[0], g + 1, 0);
                } else {
                    read_fragments(af[(t + 1) & 1], g, t + 1);
                }
#pragma unroll
                for (int tt = 0; tt < 4; ++tt)
                    acc[tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[t & 1][tt], bw[k & 1][t], acc[tt], 0, 0, 0);
                // a quarter of the next group's fragments per MFMA step (after the last group: made and not used).
                // The empty statements tie the quarter to this step: without them all four are made in one run
                // before the group's first MFMA, and the matrix pipe idles meanwhile.
                unsigned(&w_of_next)[BITS] = k + 1 < kSpan ? w_now[(k + 1) % kSpan] : w_next[0];
#pragma unroll
                for (int i = 0; i < BITS / 4; ++i) asm volatile("" : "+v"(w_of_next[(BITS / 4) * t + i]));
                widen_scale(bw[(k + 1) & 1][t], w_of_next, t, scale_next, bias_next);
                asm volatile("" : "+v"(bw[(k + 1) & 1][t]));
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
                    __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one fragment read
                    __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);  // a share of the widening
                }
            }
            // The next block of scales and biases is first read one step before its first group is multiplied.
            if ((g + 2) % kPartParamGroups == 0 && g + 2 < part_groups) {  // the whole workgroup
                __syncthreads();                                       // everyone has read this block
                stage_params(g + 2);
                __syncthreads();
            }
        }
    }
    // The tile leaves through LDS: a lane holds 16 tokens of ONE row, 2 bytes of a token's output each; laid out
    // [token][row] in the space of the x tiles, a thread then writes 16 bytes -- eight rows of a token -- and 16
    // threads a token's 256 bytes (64 stores of 2 bytes per lane took 8 us of the launch at 4096 tokens).
    __syncthreads();  // nobody reads an x tile any more
    if constexpr (KS == 2 && !RS) {
        // part 1's accumulators join part 0's: [wavefront][value][lane] floats, every lane its own words
        float *const sums = reinterpret_cast<float *>(lds_store) + wave * 64 * 64 + lane;
        if (part == 1) {
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int j = 0; j < 16; ++j) sums[(16 * tt + j) * 64] = acc[tt][j];
        }
        __syncthreads();
        if (part == 0) {
#pragma unroll
            for (int tt = 0; tt < 4; ++tt)
#pragma unroll
                for (int j = 0; j < 16; ++j) acc[tt][j] += sums[(16 * tt + j) * 64];
        }
        __syncthreads();  // the sums are read: the output tile may take their place
    }
    _Float16 *const out_tile = lds_store;
    constexpr int kOutPitch = kRows + 8;
    if (part == 0 || RS) {
#pragma unroll
        for (int tt = 0; tt < 4; ++tt)
#pragma unroll
            for (int j = 0; j < 16; ++j)
                out_tile[(32 * tt + 8 * (j / 4) + 4 * h + (j % 4)) * kOutPitch + param_at] = (_Float16)acc[tt][j];
    }
    __syncthreads();
    const bool y_vector = (uintptr_t)a.y % 16 == 0 && a.y_stride % 8 == 0;
    const int thread = threadIdx.x;
    constexpr int kPieces = kRows / 8;
#pragma unroll
    for (int i = 0; i < kGemmTokens * kPieces / kThreads; ++i) {
        const int at = thread + kThreads * i, local = at / kPieces, piece = at % kPieces;
        const int token = token0 + local, row = row0 + 8 * piece;
        if (token >= a.tokens || row >= a.rows) continue;
        const h8 v = *reinterpret_cast<const h8 *>(out_tile + local * kOutPitch + 8 * piece);
        _Float16 *dst = a.y + (long long)token * a.y_stride + row;
        if (y_vector && row + 8 <= a.rows) {
            *reinterpret_cast<h8 *>(dst) = v;
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e)
                if (row + e < a.rows) dst[e] = v[e];
        }
    }
}

// 68 KiB of LDS (104 KiB with two parts): above the 64 KiB a kernel gets without asking.
template <int BITS, bool ALIGNED, int KS, bool RS = false>
int launch_gemm(tt_hip_ctx *ctx, const ProjArgs &a, dim3 grid) {
    auto kernel = affine_gemm_kernel<BITS, ALIGNED, KS, RS>;  // its LDS limit was raised when the context was created
    launch_profiled(ctx, kernel, grid, dim3(kGemmThreads * KS), (unsigned)(RS ? gemm_rs_lds_bytes() : gemm_lds_bytes(KS)), a);
    return TT_HIP_OK;
}

// 100 KiB of LDS: above the 64 KiB a kernel gets without asking.
template <int BITS, bool ALIGNED>
int launch_proj(tt_hip_ctx *ctx, const ProjArgs &a, dim3 grid) {
    auto kernel = affine_proj_kernel<BITS, ALIGNED>;  // its LDS limit was raised when the context was created
    launch_profiled(ctx, kernel, grid, dim3(kProjWaves * 64), (unsigned)kProjLdsBytes, a);
    return TT_HIP_OK;
}

}  // namespace

// The two MFMA kernels' dynamic LDS limits, set once per device when a context is created on it.
int configure_affine_kernels(tt_hip_ctx *ctx) {
    hipError_t e = hipSuccess;
#define TT_CFG(KERNEL, BYTES) \
    if (e == hipSuccess) e = hipFuncSetAttribute(reinterpret_cast<const void *>(KERNEL), hipFuncAttributeMaxDynamicSharedMemorySize, BYTES);
    TT_CFG((affine_gemm_kernel<4, true, 1>), gemm_lds_bytes(1))
    TT_CFG((affine_gemm_kernel<4, false, 1>), gemm_lds_bytes(1))
    TT_CFG((affine_gemm_kernel<8, true, 1>), gemm_lds_bytes(1))
    TT_CFG((affine_gemm_kernel<8, false, 1>), gemm_lds_bytes(1))
    TT_CFG((affine_gemm_kernel<4, true, 2>), gemm_lds_bytes(2))
    TT_CFG((affine_gemm_kernel<4, false, 2>), gemm_lds_bytes(2))
    TT_CFG((affine_gemm_kernel<8, true, 2>), gemm_lds_bytes(2))
    TT_CFG((affine_gemm_kernel<8, false, 2>), gemm_lds_bytes(2))
    TT_CFG((affine_gemm_kernel<4, true, 2, true>), gemm_rs_lds_bytes())
    TT_CFG((affine_gemm_kernel<4, false, 2, true>), gemm_rs_lds_bytes())
    TT_CFG((affine_gemm_kernel<8, true, 2, true>), gemm_rs_lds_bytes())
    TT_CFG((affine_gemm_kernel<8, false, 2, true>), gemm_rs_lds_bytes())
    TT_CFG((affine_proj_kernel<4, true>), kProjLdsBytes)
    TT_CFG((affine_proj_kernel<4, false>), kProjLdsBytes)
    TT_CFG((affine_proj_kernel<8, true>), kProjLdsBytes)
    TT_CFG((affine_proj_kernel<8, false>), kProjLdsBytes)
#undef TT_CFG
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "hipFuncSetAttribute(o_proj max dynamic LDS)");
}

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
    const bool aligned = (uintptr_t)weights % 16 == 0;
    if (token_count >= kGemmMinTokens) {
        const long long row_blocks = (rows + kGemmRows - 1) / kGemmRows, token_blocks = (token_count + kGemmTokens - 1) / kGemmTokens;
        const long long padded = (token_blocks + 7) / 8 * 8 * row_blocks;  // token blocks in eights: see the kernel's id mapping
        if (padded > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
        const dim3 tiles_grid((unsigned)padded);
        // Three forms of the kernel.  Tiles of 128 rows for no more than the CUs: the columns in two parts inside a
        // workgroup.  More than that: tiles of 256 rows, eight wavefronts, one workgroup per CU -- the x tile is then
        // fetched once for twice the rows, and what the card's power limit charges for is traffic (4096 tokens 94.5 ->
        // 87.7 us on one box, 92.7 -> 92.0 on another; 3072 tokens 82.1 -> 75.7; 8192 tokens 176 -> 167) -- unless their
        // last round of several would leave most of the chip idle (5120 tokens, 320 such tiles: 134.8 us against 125.4 with tiles
        // of 128 rows, two workgroups per CU).
        const long long wide_blocks = (rows + 2 * kGemmRows - 1) / (2 * kGemmRows), wide_tiles = token_blocks * wide_blocks;
        const long long last_round = wide_tiles % ctx->n_cus;
        int status;
        if (token_blocks * row_blocks <= ctx->n_cus && columns / kProjGroup >= 16) {
            if (weight_bits == 4) status = aligned ? launch_gemm<4, true, 2>(ctx, a, tiles_grid) : launch_gemm<4, false, 2>(ctx, a, tiles_grid);
            else status = aligned ? launch_gemm<8, true, 2>(ctx, a, tiles_grid) : launch_gemm<8, false, 2>(ctx, a, tiles_grid);
        } else if (wide_tiles <= ctx->n_cus || last_round == 0 || 10 * last_round > 6 * ctx->n_cus) {
            const dim3 wide_grid((unsigned)((token_blocks + 7) / 8 * 8 * wide_blocks));  // (padded <= 0x7fffffff holds for these too)
            if (weight_bits == 4) status = aligned ? launch_gemm<4, true, 2, true>(ctx, a, wide_grid) : launch_gemm<4, false, 2, true>(ctx, a, wide_grid);
            else status = aligned ? launch_gemm<8, true, 2, true>(ctx, a, wide_grid) : launch_gemm<8, false, 2, true>(ctx, a, wide_grid);
        } else {
            if (weight_bits == 4) status = aligned ? launch_gemm<4, true, 1>(ctx, a, tiles_grid) : launch_gemm<4, false, 1>(ctx, a, tiles_grid);
            else status = aligned ? launch_gemm<8, true, 1>(ctx, a, tiles_grid) : launch_gemm<8, false, 1>(ctx, a, tiles_grid);
        }
        if (status != TT_HIP_OK) return status;
    } else if (token_count <= kGemvMaxTokens) {
        // unaligned weights: a lane's dword sits at a 2-byte boundary
        const bool words = (uintptr_t)weights % 4 == 0;
        if (weight_bits == 4) {
            if (words) launch_gemv<4, true>(ctx, a);
            else launch_gemv<4, false>(ctx, a);
        } else {
            if (words) launch_gemv<8, true>(ctx, a);
            else launch_gemv<8, false>(ctx, a);
        }
    } else {
        int status;
        if (weight_bits == 4) status = aligned ? launch_proj<4, true>(ctx, a, grid) : launch_proj<4, false>(ctx, a, grid);
        else status = aligned ? launch_proj<8, true>(ctx, a, grid) : launch_proj<8, false>(ctx, a, grid);
        if (status != TT_HIP_OK) return status;
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "affine_proj_kernel launch");
}
