// The sparse-attention block indexer: what chooses the keys a query may attend to, in front of
// the attention calls that take a selection.
//
//   pool    pooled[b] = mean of the raw indexer keys of block b (then, optionally, RMS norm and a
//           NeoX rotation at the block's first position)              qsa_pool_block(s)
//   rows    RMS norm and rotation of indexer query rows, in place     RMSNorm + RoPE encoders
//   score   score[t][b] = sum over heads of max(0, q[t][h] . pooled[b])   qsa_block_scores(_rows)
//   select  per query the kept cells: the ragged tail of its own block, complete blocks by score
//           (lower index first on ties) until the budget is spent, the next block cut short;
//           as a byte mask and as an ascending index list              qsa_select_decode /
//                                                                      QSAIndexer.selectKeysPrefill
// (sources/TinyTitanCore/Metal/Attention/qsa.metal; sources/TinyTitan/Kernels/Attention/QSAIndexer.swift,
// QSAIndexer+Scratch.swift.)  The reference selects a prefill chunk's rows on the host; here every
// row is a workgroup of the same kernel that serves a decode step.
//
// Pooling and the row kernel are HBM-bound element-wise work (a wavefront per row, lane l holding
// elements l, l + 64, ...).  Scoring is a small GEMM: 32 query rows x 32 blocks per MFMA tile, the
// heads of a token being consecutive accumulator rows of one lane, so the rectified sum over
// heads needs at most one cross-lane exchange; a chunk's query row tiles reach the wavefronts through
// a ring in LDS.  Selection is a radix select over the 64-bit key (orderable score, inverted index)
// in LDS histograms -- the key's upper 16 bits in one pass, the few blocks that share them ranked by
// one wavefront, eight-bit passes where that does not settle it: one workgroup per query row with
// the row's scores in registers, or, for a few rows of very many blocks, many workgroups per row in
// two launches.
#include <cmath>
#include <cstdint>

#include "internal.h"
#include "wave_ops.h"

namespace tt {
namespace {

constexpr int kQsaMaxHalfDim = 128;  // head_dim up to 256
constexpr int kSelectThreads = 1024;

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef float f16v __attribute__((ext_vector_type(16)));

struct RowsArgs {
    const _Float16 *raw;   // pooling: [n_kv][D]
    _Float16 *data;        // pooling: pooled [blocks][D]; rows: [tokens][heads][D], in place
    const unsigned short *weight;  // bf16 [D]; nullptr: pooling only
    int first_block, block_count, ratio, n_kv;  // pooling
    int heads;                                  // rows
    long long n_rows;                           // rows: tokens * heads
    int position, position_stride;              // rows: token t sits at position + t * position_stride
    float eps;
    float freq[kQsaMaxHalfDim];  // theta^(-2i / D), computed on the host with the C library's powf
};

__device__ __forceinline__ float bf16_to_float(unsigned short w) { return __builtin_bit_cast(float, (unsigned)w << 16); }

// The 64 lanes' sum, to every lane: gathered in lane 63 by DPP moves and read from there (no trip through LDS).
__device__ __forceinline__ float wave_sum(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, wave_sum_in_lane63(x)), 63));
}

// RMS norm with a bf16 weight, a rounding to fp16, a NeoX rotation over the whole row (pairs
// (i, i + D / 2), frequency divisor D), a rounding to fp16: the order and the roundings of the
// reference's separate kernels (RMSNorm.encodeBF16WPerHead, then RoPE.encodeNeoxSubdim with
// rotaryDim = headDim; sources/TinyTitanCore/Metal/Primitives/rope.metal:32-50).  A lane holds
// elements lane + 64 e: both elements of a pair sit in the same lane, E / 2 apart.
// (the rotation's cosines and sines of a position, lane l's pairs: the heads of a token share them)
template <int D>
__device__ __forceinline__ void rope_angles(float (&c)[D / 128], float (&s)[D / 128], const RowsArgs &a, int lane, float position) {
#pragma unroll
    for (int e = 0; e < D / 128; ++e) {
        const float angle = position * a.freq[lane + 64 * e];
        c[e] = cosf(angle);
        s[e] = sinf(angle);
    }
}
template <int D>
__device__ __forceinline__ void norm_rope_row(_Float16 (&h)[D / 64], const RowsArgs &a, int lane, const float (&c)[D / 128],
                                              const float (&s)[D / 128], const unsigned short *weight) {
    constexpr int E = D / 64;
    float x[E], ss = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        x[e] = (float)h[e];
        ss += x[e] * x[e];
    }
    ss = wave_sum(ss);
    const float scale = 1.0f / sqrtf(ss / (float)D + a.eps);
#pragma unroll
    for (int e = 0; e < E; ++e) x[e] = (float)(_Float16)(x[e] * scale * bf16_to_float(weight[lane + 64 * e]));
#pragma unroll
    for (int e = 0; e < E / 2; ++e) {
        const float x0 = x[e], x1 = x[e + E / 2];
        h[e] = (_Float16)(x0 * c[e] - x1 * s[e]);
        h[e + E / 2] = (_Float16)(x0 * s[e] + x1 * c[e]);
    }
}
template <int D>
__device__ __forceinline__ void norm_rope_row(_Float16 (&h)[D / 64], const RowsArgs &a, int lane, float position,
                                              const unsigned short *weight) {
    float c[D / 128], s[D / 128];
    rope_angles<D>(c, s, a, lane, position);
    norm_rope_row<D>(h, a, lane, c, s, weight);
}
template <int D>
__device__ __forceinline__ void norm_rope_row(_Float16 (&h)[D / 64], const RowsArgs &a, int lane, float position) {
    norm_rope_row<D>(h, a, lane, position, a.weight);
}

// One wavefront per block.  The sum runs in member order in fp32 and is divided by the members
// present (a ragged last block is not diluted), as qsa_pool_blocks does (qsa.metal:44-66).
template <int D, bool NORM>
__global__ __launch_bounds__(256) void qsa_pool_kernel(const RowsArgs a) {
    constexpr int E = D / 64;
    const int lane = threadIdx.x & 63;
    const long long local = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
    if (local >= a.block_count) return;
    const long long block = a.first_block + local;
    const long long first = block * a.ratio;
    if (first >= a.n_kv) return;
    const int count = (int)min((long long)a.ratio, a.n_kv - first);
    float acc[E] = {};
    for (int i = 0; i < count; ++i) {
        const _Float16 *row = a.raw + (first + i) * D;
#pragma unroll
        for (int e = 0; e < E; ++e) acc[e] += (float)row[lane + 64 * e];
    }
    _Float16 h[E];
#pragma unroll
    for (int e = 0; e < E; ++e) h[e] = (_Float16)(acc[e] / (float)count);
    if constexpr (NORM) norm_rope_row<D>(h, a, lane, (float)(unsigned)first);
    _Float16 *out = a.data + block * D;
#pragma unroll
    for (int e = 0; e < E; ++e) out[lane + 64 * e] = h[e];
}

// One wavefront per R consecutive (token, head) rows, in place.  A row is 256 or 512 bytes and a wavefront's time is
// the trip to memory and back: with the rows of a chunk a wavefront takes four, all requested before the first is
// worked on, and the rotation's cosines and sines -- the accurate ones, a few hundred instructions each at these
// angles -- are computed once for the heads of a token.
template <int D, int R>
__global__ __launch_bounds__(256) void qsa_rows_kernel(const RowsArgs a) {
    constexpr int E = D / 64;
    const int lane = threadIdx.x & 63;
    const long long row0 = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * R;
    if (row0 >= a.n_rows) return;
    _Float16 h[R][E];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const _Float16 *p = a.data + min(row0 + r, a.n_rows - 1) * D;  // past the end the last row again, not stored
#pragma unroll
        for (int e = 0; e < E; ++e) h[r][e] = p[lane + 64 * e];
    }
    float c[D / 128], s[D / 128];
    unsigned angles_of = ~0u;  // the token whose cosines and sines are in hand: its heads' rows follow one another
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (row0 + r >= a.n_rows) break;  // the whole wavefront
        const unsigned token = (unsigned)((row0 + r) / a.heads);
        if (token != angles_of) {
            rope_angles<D>(c, s, a, lane, (float)((unsigned)a.position + token * (unsigned)a.position_stride));
            angles_of = token;
        }
        norm_rope_row<D>(h[r], a, lane, c, s, a.weight);
        _Float16 *p = a.data + (row0 + r) * D;
#pragma unroll
        for (int e = 0; e < E; ++e) p[lane + 64 * e] = h[r][e];
    }
}

struct ScoreArgs {
    const _Float16 *query;   // [tokens][H][D]
    const _Float16 *pooled;  // [blocks][D]
    float *scores;           // [tokens][score_stride]
    long long score_stride;
    long long q_rows;        // tokens * H
    int blocks, tokens;
    int row_tiles, row_tiles_per_wg;
};

// Fragment of a 32-row x D operand for v_mfma_f32_32x32x16_f16: lane l holds row l % 32, elements
// 16 s + 8 (l / 32) .. + 7 of step s.  Rows past the end repeat the last one (their results are not stored).
template <int D>
__device__ __forceinline__ void load_fragments(h8 (&f)[D / 16], const _Float16 *base, long long row, long long last_row, int lane) {
    const _Float16 *p = base + min(row, last_row) * D + 8 * (lane >> 5);
#pragma unroll
    for (int s = 0; s < D / 16; ++s) f[s] = *reinterpret_cast<const h8 *>(p + 16 * s);
}

// A wavefront owns NB x 32 blocks (their pooled fragments stay in registers) and walks query-row
// tiles of 32 rows = 32 / H tokens.  Accumulator layout: lane l holds block l % 32 and rows
// 8 (j / 4) + 4 (l / 32) + j % 4, j = 0..15 -- four consecutive rows per register quad.
// NB = 2 for chunks: a row tile's fragments (8 KiB at D = 128, from L1 / L2) then feed twice the
// MFMAs, which is what the kernel waits for otherwise.
template <int H>
__device__ __forceinline__ void store_scores(const ScoreArgs &a, f16v c, long long t0, long long b, int half) {
#pragma unroll
    for (int j = 0; j < 16; ++j) c[j] = fmaxf(c[j], 0.0f);
    if constexpr (H <= 4) {
        // a token's heads are H consecutive registers of one quad
        if (b >= a.blocks) return;
        float *const column = a.scores + t0 * a.score_stride + b;
        const bool whole = t0 + 32 / H <= a.tokens;  // the tile's tokens all exist: the same for every lane
#pragma unroll
        for (int g = 0; g < 4; ++g) {
#pragma unroll
            for (int u = 0; u < 4 / H; ++u) {
                float total = c[4 * g + u * H];
#pragma unroll
                for (int h = 1; h < H; ++h) total += c[4 * g + u * H + h];
                const int t = (8 * g + 4 * half + u * H) / H;
                if (whole || t0 + t < a.tokens) column[t * a.score_stride] = total;
            }
        }
    } else {
        // H = 8: rows 8 g .. 8 g + 7 are this lane's quad g and the other half's
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const float mine = ((c[4 * g] + c[4 * g + 1]) + c[4 * g + 2]) + c[4 * g + 3];
            float lo, hi;
            halves_of(mine, lo, hi);
            const long long t = t0 + g;
            if (half == 0 && t < a.tokens && b < a.blocks) a.scores[t * a.score_stride + b] = lo + hi;
        }
    }
}

template <int D, int H, int NB>
__global__ __launch_bounds__(256) void qsa_scores_kernel(const ScoreArgs a) {
    constexpr int S = D / 16;
    const int lane = threadIdx.x & 63;
    const long long block_tile = ((long long)blockIdx.x * 4 + (threadIdx.x >> 6)) * NB;
    const long long b0 = block_tile * 32;
    if (b0 >= a.blocks) return;
    h8 pooled[NB][S];
#pragma unroll
    for (int n = 0; n < NB; ++n) load_fragments<D>(pooled[n], a.pooled, b0 + 32 * n + (lane & 31), a.blocks - 1, lane);
    const int tile_begin = blockIdx.y * a.row_tiles_per_wg;
    const int tile_end = min(a.row_tiles, tile_begin + a.row_tiles_per_wg);
    if (tile_begin >= tile_end) return;
    const long long b = b0 + (lane & 31);
    const int half = lane >> 5;
    // Two sets of query fragments taken in turn (no copies from one to the other), the NB accumulator chains of a
    // row tile interleaved (an MFMA waits for the one before it in its chain), and a lane's stores of a tile under
    // one test of its block instead of one branch each.
    h8 q0[S], q1[S];
    load_fragments<D>(q0, a.query, (long long)tile_begin * 32 + (lane & 31), a.q_rows - 1, lane);
    auto row_tile = [&](const h8 (&q)[S], h8 (&q_next)[S], int tile) {
        if (tile + 1 < tile_end) load_fragments<D>(q_next, a.query, (long long)(tile + 1) * 32 + (lane & 31), a.q_rows - 1, lane);
        const long long t0 = (long long)tile * (32 / H);
        f16v c[NB];
#pragma unroll
        for (int n = 0; n < NB; ++n) c[n] = f16v{};
#pragma unroll
        for (int s = 0; s < S; ++s)
#pragma unroll
            for (int n = 0; n < NB; ++n) c[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(q[s], pooled[n][s], c[n], 0, 0, 0);
#pragma unroll
        for (int n = 0; n < NB; ++n) store_scores<H>(a, c[n], t0, b + 32 * n, half);
    };
    for (int tile = tile_begin; tile < tile_end; tile += 2) {
        row_tile(q0, q1, tile);
        if (tile + 1 < tile_end) row_tile(q1, q0, tile + 1);
    }
}

// The same for a launch of two row tiles or more (a chunk): the row tile's fragments come through LDS.
// Every wavefront above fetches the tile's 32 rows for itself, 16 bytes of a row per lane and one tile ahead -- four
// fetches of the same 8 KiB per workgroup, 32 cache lines touched per instruction, and one tile's arithmetic is less
// than the fetch takes.  Here the workgroup's 256 threads fetch a tile once, whole lines, TWO tiles ahead, into a ring
// of three tiles in LDS (rows padded by 16 bytes), and a wavefront reads its fragments from there; one barrier a tile.
// A wavefront past the last block still fetches.  Same MFMAs in the same order: the scores are the other kernel's bit
// for bit.
constexpr int kScoreRing = 3;
template <int D, int H, int NB>
__global__ __launch_bounds__(256) void qsa_scores_staged_kernel(const ScoreArgs a) {
    constexpr int S = D / 16, kPitch = D + 8, kRowPieces = D / 8, kPieces = 32 * kRowPieces / 256;
    __shared__ __attribute__((aligned(16))) _Float16 ring[kScoreRing][32 * kPitch];
    const int tid = threadIdx.x, lane = tid & 63;
    const long long b0 = ((long long)blockIdx.x * 4 + (tid >> 6)) * NB * 32;
    const bool active = b0 < a.blocks;
    const int tile_begin = blockIdx.y * a.row_tiles_per_wg;
    const int tile_end = min(a.row_tiles, tile_begin + a.row_tiles_per_wg);
    if (tile_begin >= tile_end) return;  // the whole workgroup
    h8 pooled[NB][S];
    if (active) {
#pragma unroll
        for (int n = 0; n < NB; ++n) load_fragments<D>(pooled[n], a.pooled, b0 + 32 * n + (lane & 31), a.blocks - 1, lane);
    }
    h8 piece[kPieces];
    auto fetch = [&](int tile) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int p = tid + 256 * i;
            const long long row = min((long long)tile * 32 + p / kRowPieces, a.q_rows - 1);  // past the end the last row again
            piece[i] = *reinterpret_cast<const h8 *>(a.query + row * D + 8 * (p % kRowPieces));
        }
    };
    auto stash = [&](int slot) {
#pragma unroll
        for (int i = 0; i < kPieces; ++i) {
            const int p = tid + 256 * i;
            *reinterpret_cast<h8 *>(&ring[slot][(p / kRowPieces) * kPitch + 8 * (p % kRowPieces)]) = piece[i];
        }
    };
    fetch(tile_begin);
    stash(0);
    if (tile_begin + 1 < tile_end) {
        fetch(tile_begin + 1);
        stash(1);
    }
    __syncthreads();
    const long long b = b0 + (lane & 31);
    const int half = lane >> 5;
    int slot = 0;
    for (int tile = tile_begin; tile < tile_end; ++tile) {
        const bool more = tile + 2 < tile_end;
        if (more) fetch(tile + 2);
        if (active) {
            const _Float16 *src = &ring[slot][(lane & 31) * kPitch + 8 * half];
            h8 q[S];
#pragma unroll
            for (int s = 0; s < S; ++s) q[s] = *reinterpret_cast<const h8 *>(src + 16 * s);
            const long long t0 = (long long)tile * (32 / H);
            f16v c[NB];
#pragma unroll
            for (int n = 0; n < NB; ++n) c[n] = f16v{};
#pragma unroll
            for (int s = 0; s < S; ++s)
#pragma unroll
                for (int n = 0; n < NB; ++n) c[n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(q[s], pooled[n][s], c[n], 0, 0, 0);
#pragma unroll
            for (int n = 0; n < NB; ++n) store_scores<H>(a, c[n], t0, b + 32 * n, half);
        }
        // the slot two ahead is the one read a tile ago: every wavefront has passed that tile's barrier
        if (more) stash(slot == 0 ? 2 : slot - 1);
        __syncthreads();
        slot = slot == kScoreRing - 1 ? 0 : slot + 1;
    }
}

// A decode step's three launches in one: the new key's block re-pooled (normed, rotated, stored), the query token's
// head rows normed and rotated, and the rectified scores of every block against them.  A workgroup owns 128 blocks
// (a wavefront 32, as above).  Every workgroup norms and rotates the query rows for itself into LDS -- H rows of D, a
// wavefront per row: less work than waiting for another launch to do it once -- and the one workgroup that owns the
// block the newest key falls into pools it first (a wavefront, members in order, like qsa_pool_kernel), stores it,
// and hands it to the lane that needs it through LDS.  The same functions as the separate kernels element by
// element, so the scores are theirs bit for bit.  The query rows are read only (the separate path norms in place).
struct DecodeArgs {
    RowsArgs key;               // raw, data = pooled, weight = key norm, ratio, n_kv, eps, freq
    const _Float16 *query;      // [H][D] as projected
    const unsigned short *query_weight;
    float *scores;              // [blocks]
    int blocks, position;
};

template <int D, int H>
__global__ __launch_bounds__(256) void qsa_decode_scores_kernel(const DecodeArgs a) {
    constexpr int S = D / 16, E = D / 64;
    __shared__ __attribute__((aligned(16))) _Float16 q_rows[H][D];
    __shared__ __attribute__((aligned(16))) _Float16 last_pooled[D];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const long long wg_first = (long long)blockIdx.x * 128;
    const long long last_block = ((long long)a.key.n_kv - 1) / a.key.ratio;
    const bool owns_last = last_block >= wg_first && last_block < wg_first + 128;
    for (int row = wave; row < H; row += 4) {
        _Float16 h[E];
#pragma unroll
        for (int e = 0; e < E; ++e) h[e] = a.query[row * D + lane + 64 * e];
        norm_rope_row<D>(h, a.key, lane, (float)(unsigned)a.position, a.query_weight);  // (frequencies and eps are the key's)
#pragma unroll
        for (int e = 0; e < E; ++e) q_rows[row][lane + 64 * e] = h[e];
    }
    if (owns_last && wave == 3) {  // (the wavefront with the fewest query rows to do)
        const long long first = last_block * a.key.ratio;
        const int count = (int)min((long long)a.key.ratio, (long long)a.key.n_kv - first);
        float acc[E] = {};
        for (int i = 0; i < count; ++i) {
            const _Float16 *row = a.key.raw + (first + i) * D;
#pragma unroll
            for (int e = 0; e < E; ++e) acc[e] += (float)row[lane + 64 * e];
        }
        _Float16 h[E];
#pragma unroll
        for (int e = 0; e < E; ++e) h[e] = (_Float16)(acc[e] / (float)count);
        norm_rope_row<D>(h, a.key, lane, (float)(unsigned)first);
        _Float16 *out = a.key.data + last_block * D;
#pragma unroll
        for (int e = 0; e < E; ++e) {
            out[lane + 64 * e] = h[e];
            last_pooled[lane + 64 * e] = h[e];
        }
    }
    const long long b0 = wg_first + 32 * wave;
    h8 pooled[S];
    if (b0 < a.blocks) load_fragments<D>(pooled, a.key.data, b0 + (lane & 31), a.blocks - 1, lane);  // (in flight across the barrier)
    __syncthreads();
    if (b0 >= a.blocks) return;
    const long long b = b0 + (lane & 31);
    const int half = lane >> 5;
    if (owns_last && min(b, (long long)a.blocks - 1) == last_block) {
#pragma unroll
        for (int s = 0; s < S; ++s) pooled[s] = *reinterpret_cast<const h8 *>(&last_pooled[8 * half + 16 * s]);
    }
    h8 q[S];
    {
        const int row = min(lane & 31, H - 1);  // rows past the end repeat the last one, as load_fragments does
#pragma unroll
        for (int s = 0; s < S; ++s) q[s] = *reinterpret_cast<const h8 *>(&q_rows[row][8 * half + 16 * s]);
    }
    f16v c = {};
#pragma unroll
    for (int s = 0; s < S; ++s) c = __builtin_amdgcn_mfma_f32_32x32x16_f16(q[s], pooled[s], c, 0, 0, 0);
    ScoreArgs sa{};
    sa.scores = a.scores;
    sa.score_stride = a.blocks;
    sa.blocks = a.blocks;
    sa.tokens = 1;
    store_scores<H>(sa, c, 0, b, half);
}

struct SelectArgs {
    const float *scores;
    long long score_stride;
    uint8_t *keep;
    long long keep_stride;
    unsigned *indices;  // may be nullptr
    long long index_stride;
    unsigned *counts;   // may be nullptr
    int first_visible, ratio, width;
};

// Scores as unsigned integers that order the same way; -0.0 ties +0.0 (qsa.metal:146-150).
__device__ __forceinline__ unsigned orderable(float s) {
    if (s == 0.0f) s = 0.0f;
    const unsigned f = __builtin_bit_cast(unsigned, s);
    return (f & 0x80000000u) ? ~f : (f | 0x80000000u);
}
__device__ __forceinline__ unsigned long long select_key(const float *scores, unsigned i) {
    return ((unsigned long long)orderable(scores[i]) << 32) | (unsigned long long)(0xFFFFFFFFu - i);
}

// The value, with its origin hidden from the optimiser: what is derived from it is computed where
// it is used instead of once and kept in registers across loops.
__device__ __forceinline__ unsigned opaque(unsigned x) {
    asm volatile("" : "+v"(x));
    return x;
}

// Exclusive prefix sum of one value per thread over a workgroup of THREADS threads; `total`
// receives the sum.  Two barriers.
// The largest value of the 64 lanes, in every lane: the same moves as the sum below, then lane 63's.
__device__ __forceinline__ unsigned wave_max(unsigned x, unsigned lane) {
    const unsigned in_row = lane & 15u;
    unsigned t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false);
    if (in_row >= 1u) x = max(x, t);
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false);
    if (in_row >= 2u) x = max(x, t);
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, false);
    if (in_row >= 4u) x = max(x, t);
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, false);
    if (in_row >= 8u) x = max(x, t);
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xf, 0xf, false);
    if ((lane & 31u) >= 16u) x = max(x, t);
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xf, 0xf, false);
    if (lane >= 32u) x = max(x, t);
    return (unsigned)__builtin_amdgcn_readlane((int)x, 63);
}

// Inclusive sum over the 64 lanes by data-parallel-primitive moves (no trip through LDS): within a row of 16 lanes by
// row_shr 1, 2, 4, 8, then lane 15 of every row into the row after it (row_bcast15) and lane 31 into the upper half
// (row_bcast31); a lane takes a step's value only where the move had a source.
__device__ __forceinline__ unsigned wave_inclusive_sum(unsigned x, unsigned lane) {
    const unsigned in_row = lane & 15u;
    unsigned t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x111, 0xf, 0xf, false);  // row_shr:1
    if (in_row >= 1u) x += t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x112, 0xf, 0xf, false);  // row_shr:2
    if (in_row >= 2u) x += t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x114, 0xf, 0xf, false);  // row_shr:4
    if (in_row >= 4u) x += t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x118, 0xf, 0xf, false);  // row_shr:8
    if (in_row >= 8u) x += t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x142, 0xf, 0xf, false);  // row_bcast:15
    if ((lane & 31u) >= 16u) x += t;
    t = (unsigned)__builtin_amdgcn_update_dpp(0, (int)x, 0x143, 0xf, 0xf, false);  // row_bcast:31
    if (lane >= 32u) x += t;
    return x;
}

template <int THREADS = kSelectThreads>
__device__ __forceinline__ unsigned workgroup_exclusive_sum(unsigned value, unsigned *wave_totals, unsigned &total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const unsigned incl = wave_inclusive_sum(value, (unsigned)lane);
    __syncthreads();  // wave_totals may still be read from an earlier call
    if (lane == 63) wave_totals[wave] = incl;
    __syncthreads();
    unsigned before = 0, all = 0;
#pragma unroll
    for (int w = 0; w < THREADS / 64; ++w) {
        const unsigned t = wave_totals[w];
        if (w < wave) before += t;
        all += t;
    }
    total = all;
    return before + incl - value;
}

// hist[digit] += 1 for every lane with `match`.  The upper bits of a score (sign, exponent) are the
// same for most blocks, and 64 lanes adding to one LDS counter go one after the other: when at
// least a quarter of the lanes share the first lane's digit, those add their count once.
__device__ __forceinline__ void histogram_add(unsigned *hist, unsigned digit, bool match, unsigned lane) {
    const unsigned long long todo = __ballot(match);
    if (todo == 0ull) return;
    const int lead = __ffsll((long long)todo) - 1;
    const unsigned d = (unsigned)__builtin_amdgcn_readlane((int)digit, lead);
    const unsigned long long same = __ballot(match && digit == d);
    if (4 * __popcll(same) >= __popcll(todo)) {
        if (lane == (unsigned)lead) atomicAdd(&hist[d], (unsigned)__popcll(same));
        if (digit == d) match = false;
    }
    if (match) atomicAdd(&hist[digit], 1u);
}

// The digit whose candidates straddle `rank` (digits descending), by the 64 lanes of one
// wavefront: lane l owns digits 255 - 4 l ... 252 - 4 l.  True in the one lane that finds it, with
// the digit, the rank among that digit's candidates and their count.
__device__ __forceinline__ bool choose_digit(const unsigned *hist, unsigned rank, unsigned lane, unsigned &digit,
                                             unsigned &rank_within, unsigned &count) {
    unsigned own[4], sum = 0;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
        own[u] = hist[255 - (4 * (int)lane + u)];
        sum += own[u];
    }
    const unsigned incl = wave_inclusive_sum(sum, lane);
    unsigned above = incl - sum;
    bool found = false;
    if (above <= rank && rank < above + sum) {
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            if (!found && rank < above + own[u]) {
                found = true;
                digit = 255u - (4u * lane + (unsigned)u);
                rank_within = rank - above;
                count = own[u];
            }
            above += own[u];
        }
    }
    return found;
}

// The key's two upper bytes in one pass: a histogram over the 2,048 values of its upper 16 bits at and below the
// row's largest (bin r = distance from the largest; scores further down are not counted: the rank sits among the
// best sixteenth of a row, a few hundred bins from the top).  Bin r lives at word (r % 32) * 64 + r / 32, so that
// lane l of the wavefront that picks the bin reads its 32 bins 32 l ... 32 l + 31 without bank conflicts.
constexpr unsigned kWideBins = 2048;
constexpr unsigned kListWords = kWideBins + 64;  // the same words hold a row's index list on its way out: the usual width is 2,051
__device__ __forceinline__ unsigned wide_slot(unsigned r) { return (r & 31u) * 64u + (r >> 5); }

// The bin whose candidates straddle `rank` (from the top), by the 64 lanes of one wavefront.  True in the one lane
// that finds it; false everywhere when the rank lies below the window.
__device__ __forceinline__ bool choose_wide(const unsigned *wide, unsigned rank, unsigned lane, unsigned &bin, unsigned &rank_within,
                                            unsigned &count) {
    unsigned sum = 0;
#pragma unroll 8
    for (unsigned u = 0; u < 32; ++u) sum += wide[u * 64u + lane];
    const unsigned incl = wave_inclusive_sum(sum, lane);
    unsigned above = incl - sum;
    bool found = false;
    if (above <= rank && rank < above + sum) {
        for (unsigned u = 0; u < 32; ++u) {
            const unsigned own = wide[u * 64u + lane];
            if (!found && rank < above + own) {
                found = true;
                bin = 32u * lane + u;
                rank_within = rank - above;
                count = own;
            }
            above += own;
        }
    }
    return found;
}

// One workgroup per query row; row r sees first_visible + r keys.  The block at rank
// B = remaining / ratio (score descending, lower index first) is found by a radix select in eight
// 8-bit passes over the 64-bit key; blocks with a larger key are kept whole, that block gives its
// first `remaining % ratio` cells, the rest go (qsa_select_decode, qsa.metal:156-226).  The passes
// stop early once a single candidate is left, which with distinct scores is after the score's
// four.  Inside the dense window (visible <= width) everything visible is kept
// (QSAIndexer.selectKeysPrefill, QSAIndexer.swift:455-462).  The mask row is zero from `visible`
// to keep_stride.
// This form re-reads the scores from memory in every pass: it serves rows with more blocks than
// the register form below holds.
__global__ __launch_bounds__(kSelectThreads) void qsa_select_stream_kernel(const SelectArgs a) {
    __shared__ unsigned hist[256];
    __shared__ unsigned wave_totals[kSelectThreads / 64];
    __shared__ unsigned long long prefix_sh;
    __shared__ unsigned rank_sh, candidates_sh;
    const unsigned tid = threadIdx.x;
    const long long row = blockIdx.x;
    const unsigned visible = (unsigned)a.first_visible + (unsigned)row;
    const unsigned ratio = (unsigned)a.ratio, width = (unsigned)a.width;
    const float *scores = a.scores + row * a.score_stride;
    uint8_t *keep = a.keep ? a.keep + row * a.keep_stride : nullptr;  // no mask asked for: the list alone
    unsigned *indices = a.indices ? a.indices + row * a.index_stride : nullptr;

    if (keep)
        for (long long c = visible + tid; c < a.keep_stride; c += kSelectThreads) keep[c] = 0;
    if (visible <= width) {
        for (unsigned c = tid; c < visible; c += kSelectThreads) {
            if (keep) keep[c] = 1;
            if (indices) indices[c] = c;
        }
        if (a.counts && tid == 0) a.counts[row] = visible;
        return;
    }
    const unsigned complete = (visible / ratio) * ratio;
    const unsigned tail = visible - complete;
    if (keep)
        for (unsigned c = complete + tid; c < visible; c += kSelectThreads) keep[c] = 1;
    const unsigned blocks = complete / ratio;
    const unsigned remaining = width > tail ? width - tail : 0;
    unsigned B = remaining / ratio;
    unsigned partial = remaining - B * ratio;
    // keyB: blocks with a larger key are whole, the one with this key gives `partial` cells
    unsigned long long keyB;
    if (remaining == 0) {
        keyB = ~0ull;  // nothing is larger, nothing is equal
    } else if (B >= blocks) {
        keyB = 0ull;   // every key is larger (a key is never 0: bit 63 or the inverted sign is set for finite scores)
        partial = 0;
    } else {
        if (tid == 0) {
            prefix_sh = 0ull;
            rank_sh = B;
            candidates_sh = blocks;
        }
        int pass = 7;
        for (; pass >= 0; --pass) {
            const unsigned shift = (unsigned)pass * 8u;
            if (tid < 256) hist[tid] = 0;
            __syncthreads();
            const unsigned long long prefix = prefix_sh;
            const unsigned rank = rank_sh;
            if (candidates_sh == 1) break;  // uniform: read after the barrier
            const unsigned long long mask = pass == 7 ? 0ull : (~0ull << (shift + 8u));
            for (unsigned i = tid; i < blocks; i += kSelectThreads) {
                const unsigned long long k = select_key(scores, i);
                if ((k & mask) == prefix) atomicAdd(&hist[(unsigned)(k >> shift) & 0xFFu], 1u);
            }
            __syncthreads();
            // digit d is the one whose candidates straddle the rank: above(d) <= rank < above(d) + hist[d],
            // above(d) = candidates with a larger digit.  Thread t looks at digit 255 - t, so an exclusive
            // prefix sum over threads is the count above.
            const unsigned mine = tid < 256 ? hist[255 - tid] : 0;
            unsigned total;
            const unsigned above = workgroup_exclusive_sum(mine, wave_totals, total);
            if (tid < 256 && above <= rank && rank < above + mine) {
                rank_sh = rank - above;
                prefix_sh = prefix | ((unsigned long long)(255 - tid) << shift);
                candidates_sh = mine;
            }
            __syncthreads();
        }
        if (pass >= 0) {
            // one candidate left below the digits fixed so far: its key is the answer
            const unsigned long long prefix = prefix_sh;
            const unsigned long long mask = pass == 7 ? 0ull : (~0ull << ((unsigned)pass * 8u + 8u));
            __syncthreads();
            for (unsigned i = tid; i < blocks; i += kSelectThreads) {
                const unsigned long long k = select_key(scores, i);
                if ((k & mask) == prefix) prefix_sh = k;
            }
            __syncthreads();
        }
        keyB = prefix_sh;
    }
    if (keep)
        for (unsigned c = tid; c < complete; c += kSelectThreads) {
            const unsigned block = c / ratio;
            const unsigned long long k = select_key(scores, block);
            keep[c] = (k > keyB || (k == keyB && c - block * ratio < partial)) ? 1 : 0;
        }
    if (!indices && !a.counts) return;
    // The kept cells ascending: every thread takes a contiguous run of blocks, counts its cells,
    // and writes them behind those of the threads before it; the tail cells come last.
    const unsigned per_thread = (blocks + kSelectThreads - 1) / kSelectThreads;
    const unsigned first = min(blocks, tid * per_thread), last = min(blocks, first + per_thread);
    unsigned cells = 0;
    for (unsigned i = first; i < last; ++i) {
        const unsigned long long k = select_key(scores, i);
        cells += k > keyB ? ratio : (k == keyB ? partial : 0u);
    }
    unsigned total;
    unsigned at = workgroup_exclusive_sum(cells, wave_totals, total);
    if (indices) {
        for (unsigned i = first; i < last; ++i) {
            const unsigned long long k = select_key(scores, i);
            const unsigned take = k > keyB ? ratio : (k == keyB ? partial : 0u);
            for (unsigned o = 0; o < take; ++o) indices[at + o] = i * ratio + o;
            at += take;
        }
        // the list holds at most `width` cells (QSAIndexer.swift:484-492); only a width below the tail reaches that
        for (unsigned c = tid; c < tail; c += kSelectThreads)
            if (total + c < width) indices[total + c] = complete + c;
    }
    if (a.counts && tid == 0) a.counts[row] = min(total + tail, width);
}

// The same selection with a row's scores held in registers: thread t keeps the orderable scores
// of blocks t, t + THREADS, ... (KPT of them), read once; the passes, the mask and the index list
// all work from there.  A row's passes are otherwise a chain of dependent trips to memory, which
// is what a decode step's single workgroup would spend its time on.
//   Index list: position of a kept block = cells kept before it.  Lanes of a wavefront hold
// consecutive blocks, so a ballot is 64 blocks' worth of a bitmap; the words, in block order, get
// one thread each: an exclusive sum of their bit counts over the workgroup, then the set bits.
// At most one block (the one at the rank) gives `partial` cells; whole blocks behind it shift by that.
template <int KPT, int THREADS>
__global__ __launch_bounds__(THREADS) void qsa_select_kernel(const SelectArgs a) {
    __shared__ unsigned hist[256];
    __shared__ unsigned wave_totals[THREADS / 64];
    __shared__ unsigned long long bitmap_sh[KPT * (THREADS / 64)];  // bit l of word (j, wavefront): that lane's block j is kept whole
    __shared__ unsigned offsets_sh[KPT * (THREADS / 64)];           // whole blocks before each word
    __shared__ unsigned prefix_hi_sh, prefix_lo_sh, rank_sh, candidates_sh, partial_block_sh, wide_found_sh;
    __shared__ unsigned wide[kListWords];
    __shared__ unsigned listed_hi[64], listed_lo[64], n_listed_sh;
    const unsigned tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const long long row = blockIdx.x;
    const unsigned visible = (unsigned)a.first_visible + (unsigned)row;
    const unsigned ratio = (unsigned)a.ratio, width = (unsigned)a.width;
    const float *scores = a.scores + row * a.score_stride;
    uint8_t *keep = a.keep ? a.keep + row * a.keep_stride : nullptr;  // no mask asked for: the list alone
    unsigned *indices = a.indices ? a.indices + row * a.index_stride : nullptr;

    if (keep)
        for (long long c = visible + tid; c < a.keep_stride; c += THREADS) keep[c] = 0;
    if (visible <= width) {
        for (unsigned c = tid; c < visible; c += THREADS) {
            if (keep) keep[c] = 1;
            if (indices) indices[c] = c;
        }
        if (a.counts && tid == 0) a.counts[row] = visible;
        return;
    }
    const unsigned complete = (visible / ratio) * ratio;
    const unsigned tail = visible - complete;
    const unsigned blocks = complete / ratio;
    unsigned ok[KPT];
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const unsigned i = (unsigned)j * THREADS + tid;
        ok[j] = i < blocks ? orderable(scores[i]) : 0u;
    }
    if (keep)
        for (unsigned c = complete + tid; c < visible; c += THREADS) keep[c] = 1;
    const unsigned remaining = width > tail ? width - tail : 0;
    const unsigned B = remaining / ratio;
    unsigned partial = remaining - B * ratio;
    // (key_hi, key_lo): the key of the block at rank B; larger keys are whole blocks.  rank_block: that block, or none
    unsigned key_hi, key_lo, rank_block = ~0u;
    if (remaining == 0) {
        key_hi = key_lo = ~0u;
    } else if (B >= blocks) {
        key_hi = key_lo = 0u;  // every key is larger: its low word, the inverted index, is never 0
        partial = 0;
    } else {
        if (tid == 0) {
            prefix_hi_sh = 0u;
            prefix_lo_sh = 0u;
            rank_sh = B;
            candidates_sh = blocks;
            wide_found_sh = 0u;
            n_listed_sh = 0u;
        }
        // The score's two upper bytes at once (see choose_wide); the 8-bit passes go on from the third byte, or from
        // the first when the rank lies below the window.
        unsigned top16 = 0u;
#pragma unroll
        for (int j = 0; j < KPT; ++j)
            if ((unsigned)j * THREADS + tid < blocks) top16 = max(top16, ok[j] >> 16);
        top16 = wave_max(top16, lane);
        if (lane == 0) wave_totals[wave] = top16;
        for (unsigned b = tid; b < kWideBins; b += THREADS) wide[b] = 0u;
        __syncthreads();
#pragma unroll
        for (int w = 0; w < THREADS / 64; ++w) top16 = max(top16, wave_totals[w]);
        {
            const unsigned tid = opaque(threadIdx.x);
#pragma unroll
            for (int j = 0; j < KPT; ++j) {
                const unsigned r = top16 - (ok[j] >> 16);
                if ((unsigned)j * THREADS + tid < blocks && r < kWideBins) atomicAdd(&wide[wide_slot(r)], 1u);
            }
        }
        __syncthreads();
        if (wave == 0) {
            unsigned bin, rank_within, count;
            if (choose_wide(wide, B, lane, bin, rank_within, count)) {
                prefix_hi_sh = (top16 - bin) << 16;
                rank_sh = rank_within;
                candidates_sh = count;
                wide_found_sh = 1u;
            }
        }
        __syncthreads();
        const bool few = wide_found_sh != 0u && candidates_sh <= 64u;
        if (few) {
            // At most a wavefront's worth of blocks share the rank's 16 bits (the usual case: a bin holds a few dozen of a
            // row's blocks): they are listed in LDS -- in any order --, one wavefront takes a key per lane and counts the
            // larger ones, and the lane that counts `rank` of them holds the answer.  Keys are distinct (their low word
            // is the block's index), so there is exactly one.
            const unsigned prefix16 = prefix_hi_sh >> 16;
            const unsigned tid = opaque(threadIdx.x);
#pragma unroll
            for (int j = 0; j < KPT; ++j) {
                const unsigned i = (unsigned)j * THREADS + tid;
                const bool match = i < blocks && (ok[j] >> 16) == prefix16;
                const unsigned long long m = __ballot(match);
                if (m != 0ull) {
                    const int lead = __ffsll((long long)m) - 1;
                    unsigned at = 0u;
                    if (lane == (unsigned)lead) at = atomicAdd(&n_listed_sh, (unsigned)__popcll(m));
                    at = (unsigned)__builtin_amdgcn_readlane((int)at, lead) + (unsigned)__popcll(m & ((1ull << lane) - 1ull));
                    if (match) {
                        listed_hi[at] = ok[j];
                        listed_lo[at] = ~i;
                    }
                }
            }
            __syncthreads();
            if (wave == 0) {
                const unsigned n = candidates_sh, rank = rank_sh;
                const unsigned my_hi = lane < n ? listed_hi[lane] : 0u, my_lo = lane < n ? listed_lo[lane] : 0u;
                unsigned larger = 0u;
                for (unsigned m = 0; m < n; ++m) {
                    const unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)my_hi, (int)m);
                    const unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)my_lo, (int)m);
                    larger += (hi > my_hi || (hi == my_hi && lo > my_lo)) ? 1u : 0u;
                }
                if (lane < n && larger == rank) {
                    prefix_hi_sh = my_hi;
                    prefix_lo_sh = my_lo;
                }
            }
            __syncthreads();
        }
        int pass = few ? -1 : (wide_found_sh ? 5 : 7);
        for (; pass >= 0; --pass) {
            if (tid < 256) hist[tid] = 0;
            __syncthreads();
            const unsigned prefix_hi = prefix_hi_sh, prefix_lo = prefix_lo_sh, rank = rank_sh;
            if (candidates_sh == 1) break;
            const unsigned tid = opaque(threadIdx.x);  // nothing per block is carried from pass to pass
            const bool high = pass >= 4;
            const unsigned shift = (unsigned)(pass & 3) * 8u;
            const unsigned fixed = (pass & 3) == 3 ? 0u : (~0u << (shift + 8u));  // digits of this word already chosen
#pragma unroll
            for (int j = 0; j < KPT; ++j) {
                const unsigned i = (unsigned)j * THREADS + tid;
                const unsigned word = high ? ok[j] : ~i;
                const bool match = i < blocks && (high ? (word & fixed) == prefix_hi : (ok[j] == prefix_hi && (word & fixed) == prefix_lo));
                histogram_add(hist, (word >> shift) & 0xFFu, match, lane);
            }
            __syncthreads();
            if (wave == 0) {
                unsigned digit, rank_within, count;
                if (choose_digit(hist, rank, lane, digit, rank_within, count)) {
                    rank_sh = rank_within;
                    if (high) prefix_hi_sh = prefix_hi | (digit << shift);
                    else prefix_lo_sh = prefix_lo | (digit << shift);
                    candidates_sh = count;
                }
            }
            __syncthreads();
        }
        if (pass >= 0) {
            // one candidate left below the digits chosen so far: its key is the answer
            const unsigned prefix_hi = prefix_hi_sh, prefix_lo = prefix_lo_sh;
            const unsigned fixed_hi = pass == 7 ? 0u : (pass >= 4 ? (~0u << ((unsigned)(pass & 3) * 8u + 8u)) : ~0u);
            const unsigned fixed_lo = pass >= 3 ? 0u : (~0u << ((unsigned)pass * 8u + 8u));
            __syncthreads();
            const unsigned tid = opaque(threadIdx.x);
#pragma unroll
            for (int j = 0; j < KPT; ++j) {
                const unsigned i = (unsigned)j * THREADS + tid;
                if (i < blocks && (ok[j] & fixed_hi) == prefix_hi && (~i & fixed_lo) == prefix_lo) {
                    prefix_hi_sh = ok[j];
                    prefix_lo_sh = ~i;
                }
            }
            __syncthreads();
        }
        key_hi = prefix_hi_sh;
        key_lo = prefix_lo_sh;
        rank_block = ~key_lo;  // the key is a block's: its low word is that block's inverted index
    }
    // The mask: `ratio` bytes per block, as one word where they are four and the row is word aligned.
    // With a list to write, the wavefront's whole blocks of every j also go into the bitmap: a wavefront's ballots are
    // gathered in two registers, ballot j in lane j, and leave for LDS in one store.
    const bool words = ratio == 4 && ((uintptr_t)keep & 3) == 0;
    const bool listing = indices || a.counts;
    if (tid == 0) partial_block_sh = rank_block;
    __syncthreads();
    const unsigned tid_mask = opaque(threadIdx.x);
    unsigned ballots_lo = 0u, ballots_hi = 0u;
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const unsigned i = (unsigned)j * THREADS + tid_mask;
        const bool valid = i < blocks;
        const bool whole = valid && (ok[j] > key_hi || (ok[j] == key_hi && ~i > key_lo));
        const bool at_rank = i == rank_block;
        if (valid && keep) {
            if (words) {
                const unsigned cells = whole ? 0x01010101u : (at_rank ? (0x01010101u & ((1u << (8u * partial)) - 1u)) : 0u);
                *reinterpret_cast<unsigned *>(keep + 4ull * i) = cells;
            } else {
                for (unsigned c = 0; c < ratio; ++c) keep[(unsigned long long)i * ratio + c] = (whole || (at_rank && c < partial)) ? 1 : 0;
            }
        }
        if (listing) {
            const unsigned long long m = __ballot(whole);
            ballots_lo = lane == (unsigned)j ? (unsigned)m : ballots_lo;
            ballots_hi = lane == (unsigned)j ? (unsigned)(m >> 32) : ballots_hi;
        }
    }
    if (!listing) return;
    if (lane < (unsigned)KPT) bitmap_sh[lane * (THREADS / 64) + wave] = ((unsigned long long)ballots_hi << 32) | ballots_lo;
    __syncthreads();
    // The kept cells ascending: word (j, wavefront) covers blocks j THREADS + 64 wavefront ..., so the words
    // in storage order are the blocks in order.  One word per thread: count, exclusive sum, then the set bits.
    constexpr unsigned kWords = KPT * (THREADS / 64);
    static_assert(kWords <= THREADS, "one bitmap word per thread");
    // (half a word per thread where the threads are twice the words: half the blocks to walk for the busiest one)
    constexpr bool kHalves = 2 * kWords <= THREADS;
    constexpr unsigned kPieces = kHalves ? 2 * kWords : kWords, kPieceBlocks = kHalves ? 32u : 64u;
    unsigned long long word = 0ull;
    if (tid < kPieces) {
        if constexpr (kHalves) word = reinterpret_cast<const unsigned *>(bitmap_sh)[tid];  // little endian: the low half first
        else word = bitmap_sh[tid];
    }
    unsigned whole_blocks;
    unsigned before = workgroup_exclusive_sum<THREADS>((unsigned)__popcll(word), wave_totals, whole_blocks);
    const unsigned partial_block = partial_block_sh;
    const unsigned total = whole_blocks * ratio + (partial_block != ~0u ? partial : 0u);
    // The list is put together in LDS (the histogram's words, free by now) where it fits -- a thread's blocks land at
    // places of their own, 16 bytes here and 16 bytes there -- and leaves in whole lines.
    const bool staged = indices && width <= kListWords;
    unsigned *const list = staged ? wide : indices;
    if (indices && 2 * whole_blocks <= kWords * KPT) {
        // few kept blocks per word against the KPT rounds of the other way (a long context against the
        // budget): the word's thread writes them
        const unsigned w = kHalves ? tid / 2 : tid;
        const unsigned first_block = (w / (THREADS / 64)) * THREADS + (w % (THREADS / 64)) * 64 + (kHalves ? (tid & 1u) * 32u : 0u);
        if (tid < kPieces && partial_block != ~0u && partial_block - first_block < kPieceBlocks) {
            // the cut block sits behind the whole blocks before it
            const unsigned rank = before + (unsigned)__popcll(word & ((1ull << (partial_block - first_block)) - 1ull));
            for (unsigned c = 0; c < partial; ++c) list[rank * ratio + c] = partial_block * ratio + c;
        }
        unsigned long long m = word;
        while (m) {
            const unsigned i = first_block + (unsigned)__ffsll((long long)m) - 1u;
            m &= m - 1;
            const unsigned at = before * ratio + ((partial_block != ~0u && i > partial_block) ? partial : 0u);
            for (unsigned c = 0; c < ratio; ++c) list[at + c] = i * ratio + c;
            ++before;
        }
    } else if (indices) {
        // many kept blocks per word: every lane writes its own blocks, behind the word's offset and the
        // lanes before it
        if constexpr (kHalves) {
            if (tid < kPieces && (tid & 1u) == 0u) offsets_sh[tid / 2] = before;
        } else {
            if (tid < kWords) offsets_sh[tid] = before;
        }
        __syncthreads();
#pragma unroll 1  // reads the bitmap, not the register-held scores: a rolled loop keeps the kernel's registers down
        for (int j = 0; j < KPT; ++j) {
            const unsigned i = (unsigned)j * THREADS + tid;
            const unsigned long long m = bitmap_sh[j * (THREADS / 64) + wave];
            const unsigned rank = offsets_sh[j * (THREADS / 64) + wave] + (unsigned)__popcll(m & ((1ull << lane) - 1ull));
            if ((m >> lane) & 1ull) {
                const unsigned at = rank * ratio + ((partial_block != ~0u && i > partial_block) ? partial : 0u);
                for (unsigned c = 0; c < ratio; ++c) list[at + c] = i * ratio + c;
            } else if (i == partial_block) {
                for (unsigned c = 0; c < partial; ++c) list[rank * ratio + c] = i * ratio + c;
            }
        }
    }
    if (indices) {
        // the list holds at most `width` cells (QSAIndexer.swift:484-492); only a width below the tail reaches that
        for (unsigned c = tid; c < tail; c += THREADS)
            if (total + c < width) list[total + c] = complete + c;
    }
    if (staged) {
        __syncthreads();
        const unsigned cells = min(total + tail, width);
        for (unsigned c = tid; c < cells; c += THREADS) indices[c] = wide[c];
    }
    if (a.counts && tid == 0) a.counts[row] = min(total + tail, width);
}

// ---- One query row over many workgroups: a decode step at a long context.
// A single workgroup is one CU's arithmetic, and at 64 Ki blocks the passes above are some
// hundred microseconds of it.  Here a row is cut into chunks of kChunkBlocks blocks, one
// workgroup each, in two launches:
//   1. every chunk adds its blocks to a histogram over the upper 12 bits of the orderable score;
//   2. every chunk finds, from that histogram, the bin the block at rank B falls into (each for
//      itself: 4096 counters), then settles its own blocks: a higher bin is a whole block, a
//      lower one is dropped (mask bytes written, one bit per whole block into a bitmap), blocks
//      of that bin go to a candidate list.  The chunk that finishes last (a counter; nobody
//      waits) copies the bitmap to LDS, resolves the candidates with the radix select over their
//      remaining bits -- they are the few blocks that share 12 bits with the answer, unless many
//      scores tie -- writes their mask bytes, sets their bits, and reads the index list off the copy.
// The workspace (histogram, counters) is zero between calls: the last chunk leaves it so.
constexpr int kChunkThreads = 256;
constexpr int kChunkKeys = 8;                                // per thread
constexpr int kChunkBlocks = kChunkThreads * kChunkKeys;     // 2048
constexpr int kBinBits = 12, kBins = 1 << kBinBits;
constexpr int kMultiRows = 8;                                // rows a call may spread this way
constexpr int kMaxSpreadBlocks = 262144;                     // blocks of a row whose bitmap the last chunk holds in LDS (32 KiB)

struct MultiArgs {
    SelectArgs s;
    unsigned *hist;                 // [rows][kBins]
    unsigned long long *counters;   // [rows][2]: one word, candidates appended (low half) and chunks done (high half)
    unsigned long long *bitmap;     // [rows][bitmap_words]: bit b of word w = block 64 w + b is kept whole
    unsigned long long *candidates; // [rows][cand_stride] keys
    long long bitmap_words, cand_stride;
};

__device__ __forceinline__ void chunk_keys(unsigned (&ok)[kChunkKeys], const float *scores, unsigned base, unsigned blocks, unsigned tid) {
#pragma unroll
    for (int j = 0; j < kChunkKeys; ++j) {
        const unsigned i = base + (unsigned)j * kChunkThreads + tid;
        ok[j] = i < blocks ? orderable(scores[i]) : 0u;
    }
}

__global__ __launch_bounds__(kChunkThreads) void qsa_select_histogram_kernel(const MultiArgs a) {
    __shared__ unsigned hist[kBins];
    const unsigned tid = threadIdx.x, lane = tid & 63;
    const long long row = blockIdx.y;
    const unsigned visible = (unsigned)a.s.first_visible + (unsigned)row;
    const unsigned blocks = visible / (unsigned)a.s.ratio;
    const unsigned base = blockIdx.x * kChunkBlocks;
    if (base >= blocks) return;
    unsigned ok[kChunkKeys];
    chunk_keys(ok, a.s.scores + row * a.s.score_stride, base, blocks, tid);
    for (unsigned b = tid; b < kBins; b += kChunkThreads) hist[b] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < kChunkKeys; ++j)
        histogram_add(hist, ok[j] >> (32 - kBinBits), base + (unsigned)j * kChunkThreads + tid < blocks, lane);
    __syncthreads();
    unsigned *out = a.hist + row * kBins;
    for (unsigned b = tid; b < kBins; b += kChunkThreads) {
        const unsigned n = hist[b];
        if (n) atomicAdd(&out[b], n);
    }
}

__global__ __launch_bounds__(kChunkThreads) void qsa_select_settle_kernel(const MultiArgs a) {
    __shared__ unsigned hist[256];
    __shared__ unsigned wave_totals[kChunkThreads / 64];
    __shared__ unsigned bin_sh, rank_sh, ticket_sh, n_cand_sh, candidates_sh, partial_block_sh;
    __shared__ unsigned long long prefix_sh;
    __shared__ unsigned long long bitmap_sh[kMaxSpreadBlocks / 64];  // the last chunk's copy of the row's bitmap
    const unsigned tid = threadIdx.x, lane = tid & 63;
    const long long row = blockIdx.y;
    const unsigned ratio = (unsigned)a.s.ratio, width = (unsigned)a.s.width;
    const unsigned visible = (unsigned)a.s.first_visible + (unsigned)row;
    const unsigned complete = (visible / ratio) * ratio, tail = visible - complete, blocks = complete / ratio;
    // the host sends a row here only with visible > width, width > tail and B < blocks
    const unsigned remaining = width - tail, B = remaining / ratio, partial = remaining - B * ratio;
    const float *scores = a.s.scores + row * a.s.score_stride;
    uint8_t *keep = a.s.keep ? a.s.keep + row * a.s.keep_stride : nullptr;  // no mask asked for: the list alone
    unsigned *g_hist = a.hist + row * kBins;
    unsigned long long *counter = a.counters + row * 2;
    unsigned long long *bitmap = a.bitmap + row * a.bitmap_words;
    unsigned long long *cand = a.candidates + row * a.cand_stride;
    const unsigned base = blockIdx.x * kChunkBlocks;
    const unsigned n_chunks = (blocks + kChunkBlocks - 1) / kChunkBlocks;
    if (blockIdx.x >= n_chunks) return;

    unsigned ok[kChunkKeys];
    chunk_keys(ok, scores, base, blocks, tid);  // in flight while the histogram is read
    // The bin of the block at rank B: thread t owns the 16 bins below 4096 - 16 t, highest first.
    constexpr int kOwn = kBins / kChunkThreads;
    unsigned own[kOwn], own_sum = 0;
#pragma unroll
    for (int u = 0; u < kOwn; ++u) {
        own[u] = g_hist[kBins - 1 - ((int)tid * kOwn + u)];
        own_sum += own[u];
    }
    unsigned all;
    unsigned above = workgroup_exclusive_sum<kChunkThreads>(own_sum, wave_totals, all);
    if (above <= B && B < above + own_sum) {
#pragma unroll
        for (int u = 0; u < kOwn; ++u) {
            if (above <= B && B < above + own[u]) {
                bin_sh = kBins - 1 - ((int)tid * kOwn + u);
                rank_sh = B - above;
            }
            above += own[u];
        }
    }
    __syncthreads();
    const unsigned bin = bin_sh;

    const bool words = ratio == 4 && ((uintptr_t)keep & 3) == 0;
    // a wavefront's candidates take one update of the list's counter (a trip to memory and back)
    unsigned wave_candidates = 0;
#pragma unroll
    for (int j = 0; j < kChunkKeys; ++j) {
        const unsigned i = base + (unsigned)j * kChunkThreads + tid;
        wave_candidates += (unsigned)__popcll(__ballot(i < blocks && (ok[j] >> (32 - kBinBits)) == bin));
    }
    unsigned at = 0;
    if (wave_candidates) {
        if (lane == 0) at = (unsigned)atomicAdd(counter, (unsigned long long)wave_candidates);
        at = (unsigned)__builtin_amdgcn_readfirstlane((int)at);
    }
#pragma unroll
    for (int j = 0; j < kChunkKeys; ++j) {
        const unsigned i = base + (unsigned)j * kChunkThreads + tid;
        const bool valid = i < blocks;
        const unsigned key_bin = ok[j] >> (32 - kBinBits);
        const bool whole = valid && key_bin > bin, candidate = valid && key_bin == bin;
        const unsigned long long whole_mask = __ballot(whole), cand_mask = __ballot(candidate);
        if (lane == 0 && (i >> 6) < a.bitmap_words) bitmap[i >> 6] = whole_mask;  // i is a multiple of 64 here
        if (candidate) cand[at + (unsigned)__popcll(cand_mask & ((1ull << lane) - 1ull))] = ((unsigned long long)ok[j] << 32) | (unsigned long long)~i;
        at += (unsigned)__popcll(cand_mask);
        if (valid && !candidate && keep) {
            if (words) *reinterpret_cast<unsigned *>(keep + 4ull * i) = whole ? 0x01010101u : 0u;
            else for (unsigned c = 0; c < ratio; ++c) keep[(unsigned long long)i * ratio + c] = whole ? 1 : 0;
        }
    }
    if (blockIdx.x == 0 && keep) {
        for (unsigned c = complete + tid; c < visible; c += kChunkThreads) keep[c] = 1;
        for (long long c = visible + tid; c < a.s.keep_stride; c += kChunkThreads) keep[c] = 0;
    }
    // Who finishes last goes on; everything written above is visible to it.  The counter's high half
    // counts the chunks done; what its low half holds when the last chunk draws its number is the
    // final count of candidates (every other chunk appended before it drew).
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned long long drawn = atomicAdd(counter, 1ull << 32);
        ticket_sh = (unsigned)(drawn >> 32);
        n_cand_sh = (unsigned)drawn;
    }
    __syncthreads();
    if (ticket_sh != n_chunks - 1) return;
    __threadfence();

    // The whole-block bits of every chunk, into LDS: the candidates kept whole join them there, and
    // the index list is read off it.
    const unsigned n_words = (blocks + 63) / 64;
    for (unsigned w = tid; w < n_words; w += kChunkThreads)
        bitmap_sh[w] = __hip_atomic_load(&bitmap[w], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    // Radix select of the candidate at rank_sh over the bits below the bin: 4 bits, then 8 at a time.
    const unsigned n_cand = n_cand_sh;
    // Up to kChunkBlocks candidates are read once and stay in registers; more (many scores tie) are
    // re-read in every pass.
    const bool held = n_cand <= kChunkBlocks;
    unsigned long long held_keys[kChunkKeys];
    if (held) {
#pragma unroll
        for (int j = 0; j < kChunkKeys; ++j) {
            const unsigned n = (unsigned)j * kChunkThreads + tid;
            held_keys[j] = n < n_cand ? cand[n] : 0ull;
        }
    }
    auto for_each_candidate = [&](auto &&visit) {
        if (held) {
#pragma unroll
            for (int j = 0; j < kChunkKeys; ++j)
                if ((unsigned)j * kChunkThreads + tid < n_cand) visit(held_keys[j]);
        } else {
            for (unsigned n = tid; n < n_cand; n += kChunkThreads) visit(cand[n]);
        }
    };
    if (tid == 0) {
        prefix_sh = (unsigned long long)bin << (64 - kBinBits);
        candidates_sh = n_cand;
        partial_block_sh = ~0u;
    }
    int pass = 6;
    for (; pass >= 0; --pass) {
        hist[tid] = 0;
        __syncthreads();
        const unsigned long long prefix = prefix_sh;
        const unsigned rank = rank_sh;
        if (candidates_sh == 1) break;
        const unsigned shift = pass == 6 ? 48u : (unsigned)pass * 8u;
        const unsigned digits = pass == 6 ? 0xFu : 0xFFu;
        const unsigned long long fixed = pass == 6 ? (~0ull << (64 - kBinBits)) : (~0ull << (shift + 8u));
        for_each_candidate([&](unsigned long long k) {
            if ((k & fixed) == prefix) atomicAdd(&hist[(unsigned)(k >> shift) & digits], 1u);
        });
        __syncthreads();
        if (tid < 64) {
            unsigned digit, rank_within, count;
            if (choose_digit(hist, rank, lane, digit, rank_within, count)) {
                rank_sh = rank_within;
                prefix_sh = prefix | ((unsigned long long)digit << shift);
                candidates_sh = count;
            }
        }
        __syncthreads();
    }
    if (pass >= 0) {
        const unsigned long long prefix = prefix_sh;
        const unsigned long long fixed = pass == 6 ? (~0ull << (64 - kBinBits)) : (~0ull << ((unsigned)pass * 8u + 8u));
        __syncthreads();
        for_each_candidate([&](unsigned long long k) {
            if ((k & fixed) == prefix) prefix_sh = k;
        });
        __syncthreads();
    }
    const unsigned long long key = prefix_sh;
    for_each_candidate([&](unsigned long long k) {
        const unsigned i = ~(unsigned)k;
        const bool whole = k > key, at_rank = k == key;
        if (whole) atomicOr(reinterpret_cast<unsigned *>(bitmap_sh) + (i >> 5), 1u << (i & 31));  // little endian: bit i of the 64-bit words
        if (at_rank) partial_block_sh = i;
        if (!keep) return;
        if (words) *reinterpret_cast<unsigned *>(keep + 4ull * i) = whole ? 0x01010101u : (at_rank ? (0x01010101u & ((1u << (8u * partial)) - 1u)) : 0u);
        else for (unsigned c = 0; c < ratio; ++c) keep[(unsigned long long)i * ratio + c] = (whole || (at_rank && c < partial)) ? 1 : 0;
    });
    // leave the workspace zero for the next call
    for (unsigned b = tid; b < kBins; b += kChunkThreads) g_hist[b] = 0;
    if (tid == 0) *counter = 0ull;
    unsigned *indices = a.s.indices ? a.s.indices + row * a.s.index_stride : nullptr;
    if (!indices && !a.s.counts) return;
    __syncthreads();
    // The index list off the bitmap: a thread takes a run of words, counts its bits, and writes
    // its blocks' cells behind those of the threads before it.
    const unsigned per_thread = (n_words + kChunkThreads - 1) / kChunkThreads;
    const unsigned first = min(n_words, tid * per_thread), last = min(n_words, first + per_thread);
    unsigned bits = 0;
    for (unsigned w = first; w < last; ++w) bits += (unsigned)__popcll(bitmap_sh[w]);
    unsigned whole_blocks;
    unsigned before = workgroup_exclusive_sum<kChunkThreads>(bits, wave_totals, whole_blocks);
    const unsigned partial_block = partial_block_sh;
    const unsigned total = whole_blocks * ratio + (partial_block != ~0u ? partial : 0u);
    if (indices) {
        for (unsigned w = first; w < last; ++w) {
            unsigned long long m = bitmap_sh[w];
            if (partial_block != ~0u && (partial_block >> 6) == w) {
                // the cut block sits behind the whole blocks before it: those of earlier words, and the lower bits of this one
                const unsigned rank = before + (unsigned)__popcll(m & ((1ull << (partial_block & 63)) - 1ull));
                for (unsigned c = 0; c < partial; ++c) indices[rank * ratio + c] = partial_block * ratio + c;
            }
            while (m) {
                const unsigned i = w * 64 + (unsigned)__ffsll((long long)m) - 1u;
                m &= m - 1;
                const unsigned at = before * ratio + ((partial_block != ~0u && i > partial_block) ? partial : 0u);
                for (unsigned c = 0; c < ratio; ++c) indices[at + c] = i * ratio + c;
                ++before;
            }
        }
        for (unsigned c = tid; c < tail; c += kChunkThreads)
            if (total + c < width) indices[total + c] = complete + c;
    }
    if (a.s.counts && tid == 0) a.s.counts[row] = min(total + tail, width);
}

void fill_frequencies(RowsArgs &a, int head_dim, float theta) {
    for (int i = 0; i < head_dim / 2; ++i) a.freq[i] = powf(theta, -(float)(2 * i) / (float)head_dim);
}

struct Timed {
    tt_hip_ctx *ctx;
    bool on;
    explicit Timed(tt_hip_ctx *c) : ctx(c), on(c->profiling && !c->capturing && c->prof_used + 2 <= c->prof_events.size()) {
        if (on) (void)hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream);
    }
    int finish(const char *what) {
        const hipError_t e = hipGetLastError();
        if (on) {
            (void)hipEventRecord(ctx->prof_events[ctx->prof_used + 1], ctx->stream);
            ctx->prof_used += 2;
        }
        return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, what);
    }
};

}  // namespace
}  // namespace tt

using namespace tt;

extern "C" int tt_hip_qsa_pool_blocks(tt_hip_ctx *ctx, const tt_half *raw_keys, tt_half *pooled, int head_dim, int first_block,
                                      int block_count, int ratio, int n_kv, const uint16_t *key_norm_bf16, float eps,
                                      float rope_theta) {
    if (!ctx || !raw_keys || !pooled) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (first_block < 0 || block_count < 0 || ratio <= 0 || n_kv < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (head_dim != 128 && head_dim != 256) return TT_HIP_ERR_SHAPE;
    if ((uintptr_t)raw_keys % 2 != 0 || (uintptr_t)pooled % 2 != 0 || (uintptr_t)key_norm_bf16 % 2 != 0) return TT_HIP_ERR_SHAPE;
    if ((long long)first_block + block_count > 0x7fffffffLL / ratio) return TT_HIP_ERR_SHAPE;
    if (key_norm_bf16 && !(rope_theta > 0.0f)) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (block_count == 0) return TT_HIP_OK;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    RowsArgs a{};
    a.raw = reinterpret_cast<const _Float16 *>(raw_keys);
    a.data = reinterpret_cast<_Float16 *>(pooled);
    a.weight = key_norm_bf16;
    a.first_block = first_block;
    a.block_count = block_count;
    a.ratio = ratio;
    a.n_kv = n_kv;
    a.eps = eps;
    if (key_norm_bf16) fill_frequencies(a, head_dim, rope_theta);
    const dim3 grid((unsigned)((block_count + 3) / 4));
    if (head_dim == 128) {
        if (key_norm_bf16) hipLaunchKernelGGL((qsa_pool_kernel<128, true>), grid, dim3(256), 0, ctx->stream, a);
        else hipLaunchKernelGGL((qsa_pool_kernel<128, false>), grid, dim3(256), 0, ctx->stream, a);
    } else {
        if (key_norm_bf16) hipLaunchKernelGGL((qsa_pool_kernel<256, true>), grid, dim3(256), 0, ctx->stream, a);
        else hipLaunchKernelGGL((qsa_pool_kernel<256, false>), grid, dim3(256), 0, ctx->stream, a);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "qsa_pool_kernel launch");
}

extern "C" int tt_hip_qsa_norm_rope_rows(tt_hip_ctx *ctx, tt_half *rows, int token_count, int heads, int head_dim,
                                         const uint16_t *norm_bf16, float eps, float rope_theta, int position,
                                         int position_stride) {
    if (!ctx || !rows || !norm_bf16) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (token_count < 0 || heads <= 0 || position < 0 || position_stride < 0 || !(rope_theta > 0.0f)) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (head_dim != 128 && head_dim != 256) return TT_HIP_ERR_SHAPE;
    if ((uintptr_t)rows % 2 != 0 || (uintptr_t)norm_bf16 % 2 != 0) return TT_HIP_ERR_SHAPE;
    if ((long long)position + (long long)token_count * position_stride > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
    const long long n_rows = (long long)token_count * heads;
    if (n_rows > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
    if (n_rows == 0) return TT_HIP_OK;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    RowsArgs a{};
    a.data = reinterpret_cast<_Float16 *>(rows);
    a.weight = norm_bf16;
    a.heads = heads;
    a.n_rows = n_rows;
    a.position = position;
    a.position_stride = position_stride;
    a.eps = eps;
    fill_frequencies(a, head_dim, rope_theta);
    if (n_rows >= 4096) {  // a chunk's rows: four to a wavefront
        const dim3 grid((unsigned)((n_rows + 15) / 16));
        if (head_dim == 128) hipLaunchKernelGGL((qsa_rows_kernel<128, 4>), grid, dim3(256), 0, ctx->stream, a);
        else hipLaunchKernelGGL((qsa_rows_kernel<256, 4>), grid, dim3(256), 0, ctx->stream, a);
    } else {
        const dim3 grid((unsigned)((n_rows + 3) / 4));
        if (head_dim == 128) hipLaunchKernelGGL((qsa_rows_kernel<128, 1>), grid, dim3(256), 0, ctx->stream, a);
        else hipLaunchKernelGGL((qsa_rows_kernel<256, 1>), grid, dim3(256), 0, ctx->stream, a);
    }
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "qsa_rows_kernel launch");
}

template <int D>
static void launch_decode_scores(tt_hip_ctx *ctx, int heads, dim3 grid, const DecodeArgs &a) {
    switch (heads) {
        case 1: hipLaunchKernelGGL((qsa_decode_scores_kernel<D, 1>), grid, dim3(256), 0, ctx->stream, a); break;
        case 2: hipLaunchKernelGGL((qsa_decode_scores_kernel<D, 2>), grid, dim3(256), 0, ctx->stream, a); break;
        case 4: hipLaunchKernelGGL((qsa_decode_scores_kernel<D, 4>), grid, dim3(256), 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL((qsa_decode_scores_kernel<D, 8>), grid, dim3(256), 0, ctx->stream, a); break;
    }
}

extern "C" int tt_hip_qsa_decode_scores(tt_hip_ctx *ctx, const tt_half *raw_keys, tt_half *pooled, int head_dim, int ratio, int n_kv,
                                        const uint16_t *key_norm_bf16, const tt_half *query, int heads,
                                        const uint16_t *query_norm_bf16, int position, float eps, float rope_theta, float *scores) {
    if (!ctx || !raw_keys || !pooled || !key_norm_bf16 || !query || !query_norm_bf16 || !scores) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (ratio <= 0 || n_kv <= 0 || position < 0 || !(rope_theta > 0.0f)) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (head_dim != 128 && head_dim != 256) return TT_HIP_ERR_SHAPE;
    if (heads != 1 && heads != 2 && heads != 4 && heads != 8) return TT_HIP_ERR_SHAPE;
    // pooled rows are read 16 bytes at a time; everything else as 16-bit (32-bit) values
    if ((uintptr_t)pooled % 16 != 0 || (uintptr_t)raw_keys % 2 != 0 || (uintptr_t)query % 2 != 0 || (uintptr_t)scores % 4 != 0 ||
        (uintptr_t)key_norm_bf16 % 2 != 0 || (uintptr_t)query_norm_bf16 % 2 != 0)
        return TT_HIP_ERR_SHAPE;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    DecodeArgs a{};
    a.key.raw = reinterpret_cast<const _Float16 *>(raw_keys);
    a.key.data = reinterpret_cast<_Float16 *>(pooled);
    a.key.weight = key_norm_bf16;
    a.key.ratio = ratio;
    a.key.n_kv = n_kv;
    a.key.eps = eps;
    fill_frequencies(a.key, head_dim, rope_theta);
    a.query = reinterpret_cast<const _Float16 *>(query);
    a.query_weight = query_norm_bf16;
    a.scores = scores;
    a.blocks = (n_kv - 1) / ratio + 1;
    a.position = position;
    const dim3 grid((unsigned)((a.blocks + 127) / 128));
    Timed timed(ctx);
    if (head_dim == 128) launch_decode_scores<128>(ctx, heads, grid, a);
    else launch_decode_scores<256>(ctx, heads, grid, a);
    return timed.finish("qsa_decode_scores_kernel launch");
}

template <int D, int NB>
static void launch_scores(tt_hip_ctx *ctx, int heads, dim3 grid, const ScoreArgs &a) {
    if (a.row_tiles >= 2) {  // a chunk: the query rows staged through LDS (one fetch for the workgroup's four wavefronts even with a tile each)
        switch (heads) {
            case 1: hipLaunchKernelGGL((qsa_scores_staged_kernel<D, 1, NB>), grid, dim3(256), 0, ctx->stream, a); break;
            case 2: hipLaunchKernelGGL((qsa_scores_staged_kernel<D, 2, NB>), grid, dim3(256), 0, ctx->stream, a); break;
            case 4: hipLaunchKernelGGL((qsa_scores_staged_kernel<D, 4, NB>), grid, dim3(256), 0, ctx->stream, a); break;
            default: hipLaunchKernelGGL((qsa_scores_staged_kernel<D, 8, NB>), grid, dim3(256), 0, ctx->stream, a); break;
        }
        return;
    }
    switch (heads) {
        case 1: hipLaunchKernelGGL((qsa_scores_kernel<D, 1, NB>), grid, dim3(256), 0, ctx->stream, a); break;
        case 2: hipLaunchKernelGGL((qsa_scores_kernel<D, 2, NB>), grid, dim3(256), 0, ctx->stream, a); break;
        case 4: hipLaunchKernelGGL((qsa_scores_kernel<D, 4, NB>), grid, dim3(256), 0, ctx->stream, a); break;
        default: hipLaunchKernelGGL((qsa_scores_kernel<D, 8, NB>), grid, dim3(256), 0, ctx->stream, a); break;
    }
}

extern "C" int tt_hip_qsa_block_scores(tt_hip_ctx *ctx, const tt_half *query, const tt_half *pooled, float *scores,
                                       size_t score_stride, int head_dim, int heads, int blocks, int token_count) {
    if (!ctx || !query || !pooled || !scores) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (blocks < 0 || token_count < 0 || heads <= 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (head_dim != 128 && head_dim != 256) return TT_HIP_ERR_SHAPE;
    if (heads != 1 && heads != 2 && heads != 4 && heads != 8) return TT_HIP_ERR_SHAPE;
    if (score_stride < (size_t)blocks) return TT_HIP_ERR_SHAPE;
    // rows are read 16 bytes at a time
    if ((uintptr_t)query % 16 != 0 || (uintptr_t)pooled % 16 != 0 || (uintptr_t)scores % 4 != 0) return TT_HIP_ERR_SHAPE;
    if (blocks == 0 || token_count == 0) return TT_HIP_OK;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    ScoreArgs a{};
    a.query = reinterpret_cast<const _Float16 *>(query);
    a.pooled = reinterpret_cast<const _Float16 *>(pooled);
    a.scores = scores;
    a.score_stride = (long long)score_stride;
    a.q_rows = (long long)token_count * heads;
    a.blocks = blocks;
    a.tokens = token_count;
    a.row_tiles = (int)((a.q_rows + 31) / 32);
    // Two block tiles per wavefront where the launch stays wide without them: a chunk over a long context.
    const bool wide = head_dim == 128 && a.row_tiles >= 8 && blocks >= 4096;
    const long long tiles_per_wg = wide ? 8 : 4;
    const long long block_wgs = ((long long)(blocks + 31) / 32 + tiles_per_wg - 1) / tiles_per_wg;
    // Split the query rows over grid.y until the launch holds about two workgroups per CU; a
    // workgroup then re-reads its pooled fragments once per split, which is small against the rows it walks.
    // (Four per CU, the rule before the row tiles went through LDS: 128 rows behind 131k keys 22.8 against 17.4 us, 256
    // rows 24.9 against 22.6, 256 rows behind 16k keys 10.0 against 9.4; 4,096-token chunks the same either way.)
    long long splits = (2LL * ctx->n_cus + block_wgs - 1) / block_wgs;
    if (splits > a.row_tiles) splits = a.row_tiles;
    if (splits > 65535) splits = 65535;
    if (splits < 1) splits = 1;
    a.row_tiles_per_wg = (int)((a.row_tiles + splits - 1) / splits);
    const dim3 grid((unsigned)block_wgs, (unsigned)((a.row_tiles + a.row_tiles_per_wg - 1) / a.row_tiles_per_wg));
    Timed timed(ctx);
    if (wide) launch_scores<128, 2>(ctx, heads, grid, a);
    else if (head_dim == 128) launch_scores<128, 1>(ctx, heads, grid, a);
    else launch_scores<256, 1>(ctx, heads, grid, a);
    return timed.finish("qsa_scores_kernel launch");
}

// Workspace of the multi-workgroup selection, zeroed when allocated and left zero by every call.
static int ensure_select_workspace(tt_hip_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->select_ws_bytes) return TT_HIP_OK;
    if (ctx->capturing) return TT_HIP_ERR_BUSY;  // allocating would synchronise inside a capture
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    if (ctx->select_ws) (void)hipFree(ctx->select_ws);
    ctx->select_ws = nullptr;
    ctx->select_ws_bytes = 0;
    ++ctx->generation;
    e = hipMalloc(&ctx->select_ws, bytes);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMalloc(selection workspace)");
    // on the stream the selection kernels run on (created non-blocking: the null stream orders nothing with it)
    e = hipMemsetAsync(ctx->select_ws, 0, bytes, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMemsetAsync(selection workspace)");
    ctx->select_ws_bytes = bytes;
    return TT_HIP_OK;
}

extern "C" int tt_hip_qsa_select(tt_hip_ctx *ctx, const float *scores, size_t score_stride, int rows, int first_visible,
                                 int ratio, int width, uint8_t *keep, size_t keep_stride, uint32_t *indices,
                                 size_t index_stride, uint32_t *counts) {
    if (!ctx || !scores) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (!keep && (!indices || !counts)) return TT_HIP_ERR_INVALID_ARGUMENT;  // a mask, a list with its counts, or both
    if (rows < 0 || first_visible < 0 || ratio <= 0 || width < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    const long long last_visible = (long long)first_visible + rows - 1;
    if (last_visible > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
    if (keep && rows > 0 && (long long)keep_stride < last_visible) return TT_HIP_ERR_SHAPE;
    if (rows > 1 && (long long)score_stride < last_visible / ratio) return TT_HIP_ERR_SHAPE;
    // a row lists at most `width` cells: the selection's size, or inside the dense window what it sees
    if (indices && (long long)index_stride < (long long)width) return TT_HIP_ERR_SHAPE;
    if ((uintptr_t)scores % 4 != 0 || (uintptr_t)indices % 4 != 0 || (uintptr_t)counts % 4 != 0) return TT_HIP_ERR_SHAPE;
    if (rows == 0) return TT_HIP_OK;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    SelectArgs a{};
    a.scores = scores;
    a.score_stride = (long long)score_stride;
    a.keep = keep;
    a.keep_stride = (long long)keep_stride;
    a.indices = indices;
    a.index_stride = (long long)index_stride;
    a.counts = counts;
    a.first_visible = first_visible;
    a.ratio = ratio;
    a.width = width;
    // blocks of the row that sees most; a thread of the register form holds 1, 4, 16, 32 or 64 of them
    const long long max_blocks = last_visible / ratio;
    const dim3 grid((unsigned)rows), wg(kSelectThreads);
    // A few rows with many blocks each (a decode or verify step at a long context) spread over many
    // workgroups, provided every row has a real selection to make (B < blocks, see the kernel).  The
    // two launches and their trips through memory cost about what one workgroup needs for 16 Ki blocks.
    // (more rows run side by side as workgroups of their own: 8 rows of 32,768 blocks 43.3 us that way, 47.1 us spread;
    // 4 rows of 17,500 blocks the same either way)
    bool spread = rows <= kMultiRows && max_blocks > 16LL * kSelectThreads * (rows >= 8 ? 2 : 1) && max_blocks <= kMaxSpreadBlocks;
    for (int r = 0; r < rows && spread; ++r) {
        const long long visible = (long long)first_visible + r, complete = visible / ratio * ratio, tail = visible - complete;
        spread = visible > width && width > tail && (width - tail) / ratio < complete / ratio;
    }
    if (spread) {
        const long long chunks = (max_blocks + kChunkBlocks - 1) / kChunkBlocks;
        MultiArgs m{};
        m.s = a;
        m.bitmap_words = chunks * (kChunkBlocks / 64);
        m.cand_stride = chunks * kChunkBlocks;
        const size_t hist_bytes = (size_t)kMultiRows * kBins * 4, counter_bytes = (size_t)kMultiRows * 16;
        const size_t bitmap_bytes = (size_t)rows * m.bitmap_words * 8, cand_bytes = (size_t)rows * m.cand_stride * 8;
        const int st = ensure_select_workspace(ctx, hist_bytes + counter_bytes + bitmap_bytes + cand_bytes);
        if (st != TT_HIP_OK) return st;
        // The histograms and counters must be zero when a call starts, so they sit first, at offsets that
        // do not depend on the call; bitmap and candidates behind them are written before they are read.
        uint8_t *ws = static_cast<uint8_t *>(ctx->select_ws);
        m.hist = reinterpret_cast<unsigned *>(ws);
        m.counters = reinterpret_cast<unsigned long long *>(ws + hist_bytes);
        m.bitmap = reinterpret_cast<unsigned long long *>(ws + hist_bytes + counter_bytes);
        m.candidates = reinterpret_cast<unsigned long long *>(ws + hist_bytes + counter_bytes + bitmap_bytes);
        const dim3 chunk_grid((unsigned)chunks, (unsigned)rows), chunk_wg(kChunkThreads);
        Timed timed(ctx);
        hipLaunchKernelGGL(qsa_select_histogram_kernel, chunk_grid, chunk_wg, 0, ctx->stream, m);
        hipLaunchKernelGGL(qsa_select_settle_kernel, chunk_grid, chunk_wg, 0, ctx->stream, m);
        return timed.finish("qsa_select_settle_kernel launch");
    }
    Timed timed(ctx);
    // Many rows (a long chunk) fill the chip by themselves: workgroups of 256 threads spend less of their time in
    // barriers and more of them fit a CU.  Fewer rows want their latency short: 1024 threads each.
    constexpr int kSmall = 256;
    const dim3 small_wg(kSmall);
    // (from 1024 rows on: 128 rows behind 32k keys take 53.0 us a step with the small workgroups and 35.8 us with the
    // large ones, 256 rows behind 16k keys 47.7 / 35.4, 512 rows behind 2k keys 28.3 / 26.4, 1024 rows behind 8k keys
    // 58.4 / 57.6, 2048 rows behind 16k keys 116.6 / 121.3, 4096 rows from position 0 64.2 / 78.7)
    constexpr int small_from = 1024;
    // scores per thread: the smallest of 1, 2, 4, 8, 16, 32, 64 that holds the row (every unused one is a turn of
    // each unrolled loop all the same)
    if (rows >= small_from && max_blocks <= 4LL * kSmall) hipLaunchKernelGGL((qsa_select_kernel<4, kSmall>), grid, small_wg, 0, ctx->stream, a);
    else if (rows >= small_from && max_blocks <= 8LL * kSmall) hipLaunchKernelGGL((qsa_select_kernel<8, kSmall>), grid, small_wg, 0, ctx->stream, a);
    else if (rows >= small_from && max_blocks <= 16LL * kSmall) hipLaunchKernelGGL((qsa_select_kernel<16, kSmall>), grid, small_wg, 0, ctx->stream, a);
    else if (rows >= small_from && max_blocks <= 32LL * kSmall) hipLaunchKernelGGL((qsa_select_kernel<32, kSmall>), grid, small_wg, 0, ctx->stream, a);
    else if (rows >= small_from && max_blocks <= 64LL * kSmall) hipLaunchKernelGGL((qsa_select_kernel<64, kSmall>), grid, small_wg, 0, ctx->stream, a);
    else if (max_blocks <= 1LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<1, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 2LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<2, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 4LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<4, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 8LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<8, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 16LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<16, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 32LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<32, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else if (max_blocks <= 64LL * kSelectThreads) hipLaunchKernelGGL((qsa_select_kernel<64, kSelectThreads>), grid, wg, 0, ctx->stream, a);
    else hipLaunchKernelGGL(qsa_select_stream_kernel, grid, wg, 0, ctx->stream, a);
    return timed.finish("qsa_select_kernel launch");
}
