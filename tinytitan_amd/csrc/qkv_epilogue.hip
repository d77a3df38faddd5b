// Pre-attention epilogue fused with the KV append: what sits between the QKV projections and
// the attention kernels.
//
//   q_proj output, per token and head [query(D) ; gate(D)]  ->  query: per-head RMS norm (bf16
//       weight shared by all heads), NeoX sub-dim RoPE, fp16   |  gate: copied out, contiguous
//   k_proj output  ->  per-head RMS norm, RoPE, written straight into the swizzled KV page
//   v_proj output  ->  written straight into the swizzled KV page
//
// One launch replaces, for a decode row, Elementwise.encodeSplitQGate + two
// RMSNorm.encodeBF16WPerHead + two RoPE.encodeNeoxSubdim and the K/V slot writes
// (sources/TinyTitan/Runtime/Inference/RealForwardRunner+DecodeFullAttention.swift:123-185),
// and for a prefill chunk PrefillQKVEpilogue.encodeNeoxSubdimNoVNorm
// (sources/TinyTitan/Kernels/Prefill/Epilogues/PrefillQKVEpilogue.swift:18-110) plus the
// copyPrefillKVToCache blit (RealForwardRunner+PrefillKV.swift:99-145).  Arithmetic follows the
// CPU engine (sources/TinyTitan/CPUEngine/CPUQwen35.swift:266-300; CPUTensorOps.swift:70-84,
// :120-139): everything in fp32 from the fp16 projections to ONE fp16 rounding at the end (the
// Metal chain rounds to fp16 after the norm and again after the rotation).
//
// HBM-bound element-wise work.  A wavefront owns one (token, head) slice: D/64 consecutive dims
// per lane, the sum of squares by a butterfly, the rotation partner by one cross-lane read.  K and
// V of whole 32-token blocks go through LDS and leave as full swizzled lines, like the plain
// block append; ragged edges and decode rows scatter.
#include <cmath>
#include <cstdint>

#include "internal.h"
#include "kv_layout.h"

namespace tt {

constexpr int kMaxEpilogueSeq = 64;
constexpr int kMaxRotaryHalf = 128;
constexpr int kEpiloguePad = 8;  // halves of padding per LDS row

struct EpilogueArgs {
    const _Float16 *q_packed, *k_proj, *v_proj;
    _Float16 *q_out, *gate_out;
    _Float16 *k_layer, *v_layer;
    const unsigned short *q_weight, *k_weight;  // bf16
    long long qp_stride, kv_stride, q_stride, g_stride, page_elems;
    int n_tokens, rows, n_q_heads, n_kv_heads;
    int rotary_half;
    float eps;
    // Workgroup ranges: [0, block_wgs) whole K/V blocks, then row_wgs of ragged K/V rows, then
    // the query slices (hpw q heads per wavefront).
    int block_wgs, row_wgs, hpw;
    int first_block, n_blocks;  // whole blocks (single-sequence calls only)
    int head_rows, tail_rows;   // ragged rows before / after the whole blocks (per sequence: rows when no blocks)
    int slot[kMaxEpilogueSeq], position[kMaxEpilogueSeq];
    float freq[kMaxRotaryHalf];  // theta^(-2i / rotary_dim), computed on the host with the C library's powf
};

namespace {

__device__ __forceinline__ float bf16_to_float(unsigned short w) { return __builtin_bit_cast(float, (unsigned)w << 16); }

// A head slice is held across a wavefront: lane l holds dims [l * E, l * E + E), E = D / 64.
// Rotation pairs are (i, i + rotary_half): the partner lane is rotary_half / E lanes away.
template <int E>
struct Rotation {
    float c[E], s[E];  // cos / sin of this lane's dims (1 / 0 where the dim is not rotated)
    int partner;       // lane holding the other element of each pair
    bool low, rotated;
};

// Every head of a token turns by the same angles: computed once per (wavefront, token).
template <int E>
__device__ __forceinline__ Rotation<E> rotation_for(int rotary_half, const float *freq, int position, int lane) {
    Rotation<E> r;
    const int d0 = lane * E;
    const int shift = rotary_half / E;
    r.low = d0 < rotary_half;
    r.rotated = d0 < 2 * rotary_half;
    r.partner = (r.low ? lane + shift : lane - shift) & 63;
#pragma unroll
    for (int e = 0; e < E; ++e) {
        r.c[e] = 1.0f;
        r.s[e] = 0.0f;
        if (r.rotated) {
            const int i = (r.low ? d0 : d0 - rotary_half) + e;
            const float angle = (float)position * freq[i];
            r.c[e] = cosf(angle);
            r.s[e] = sinf(angle);
        }
    }
    return r;
}

// Per-head RMS norm (weight shared by all heads) and NeoX sub-dim rotation of one head slice.
template <int D>
__device__ __forceinline__ void norm_rope(float (&x)[D / 64], const float (&w)[D / 64], float eps, const Rotation<D / 64> &rot) {
    constexpr int E = D / 64;
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) ss += x[e] * x[e];
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
    const float scale = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < E; ++e) x[e] = x[e] * scale * w[e];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const float other = __shfl(x[e], rot.partner);
        if (rot.rotated) x[e] = rot.low ? x[e] * rot.c[e] - other * rot.s[e] : other * rot.s[e] + x[e] * rot.c[e];
    }
}

template <int E>
__device__ __forceinline__ void load_weight(float (&w)[E], const unsigned short *weight, int d0) {
#pragma unroll
    for (int e = 0; e < E; ++e) w[e] = bf16_to_float(weight[d0 + e]);
}

// E consecutive halves <-> fp32.  VEC: the address is a multiple of 2 E bytes (one load/store).
template <int E>
struct HalfVec {
    typedef _Float16 type __attribute__((ext_vector_type(E)));
};
template <>
struct HalfVec<1> {
    typedef _Float16 type;
};
template <int E, bool VEC>
__device__ __forceinline__ void load_halves(float (&x)[E], const _Float16 *p) {
    if constexpr (VEC && E > 1) {
        const typename HalfVec<E>::type v = *reinterpret_cast<const typename HalfVec<E>::type *>(p);
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = (float)v[e];
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = (float)p[e];
    }
}
template <int E, bool VEC>
__device__ __forceinline__ void store_halves(_Float16 *p, const float (&x)[E]) {
    if constexpr (VEC && E > 1) {
        typename HalfVec<E>::type v;
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] = (_Float16)x[e];
        *reinterpret_cast<typename HalfVec<E>::type *>(p) = v;
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) p[e] = (_Float16)x[e];
    }
}

}  // namespace

// ALIGNED: every caller pointer and stride is a multiple of D/64 halves.
template <int D, bool ALIGNED>
__global__ __launch_bounds__(256) void qkv_epilogue_kernel(const EpilogueArgs a) {
    constexpr int E = D / 64;
    extern __shared__ __attribute__((aligned(16))) _Float16 tile[];
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int d0 = lane * E;
    const int wg = blockIdx.x;

    if (wg < a.block_wgs) {
        // ---- whole 32-token K/V blocks of a single sequence: one workgroup per (block, kv head).
        // These come first in the grid: they are the longest-running workgroups.
        const int blk = wg / a.n_kv_heads, kvh = wg - blk * a.n_kv_heads;
        constexpr int ROW = D + kEpiloguePad;
        constexpr int RPW = kBlockTokens / 4;  // rows per wavefront
        _Float16 *kt = tile, *vt = tile + kBlockTokens * ROW;
        const int token0 = a.head_rows + blk * kBlockTokens;
        const int position0 = a.position[0] + token0;
        float k[RPW][E], v[RPW][E], w[E];
#pragma unroll
        for (int r = 0; r < RPW; ++r) {  // all of the wavefront's rows in flight at once
            const long long off = (long long)(token0 + wave * RPW + r) * a.kv_stride + (long long)kvh * D + d0;
            load_halves<E, ALIGNED>(k[r], a.k_proj + off);
            load_halves<E, ALIGNED>(v[r], a.v_proj + off);
        }
        load_weight<E>(w, a.k_weight, d0);
#pragma unroll
        for (int r = 0; r < RPW; ++r) {
            const int row = wave * RPW + r;
            const Rotation<E> rot = rotation_for<E>(a.rotary_half, a.freq, position0 + row, lane);
            norm_rope<D>(k[r], w, a.eps, rot);
            store_halves<E, true>(kt + row * ROW + d0, k[r]);
            store_halves<E, true>(vt + row * ROW + d0, v[r]);
        }
        __syncthreads();
        const size_t dst0 = ((size_t)a.slot[0] * a.n_kv_heads + kvh) * (size_t)a.page_elems +
                            (size_t)(a.first_block + blk) * (size_t)(kBlockTokens * D);
        constexpr int PIECES = kBlockTokens * D / 8;
        for (int p = threadIdx.x; p < PIECES; p += 256) {
            const int d8 = p >> 5, key = p & 31;  // K piece (d / 8, key)
            *reinterpret_cast<h8 *>(a.k_layer + dst0 + (size_t)p * 8) = *reinterpret_cast<const h8 *>(kt + key * ROW + d8 * 8);
            const int d = p >> 2, c = p & 3;  // V piece (d, chunk)
            h8 x;
#pragma unroll
            for (int i = 0; i < 8; ++i) x[i] = vt[v_key_at(c, i) * ROW + d];
            *reinterpret_cast<h8 *>(a.v_layer + dst0 + (size_t)p * 8) = x;
        }
        return;
    }

    if (wg < a.block_wgs + a.row_wgs) {
        // ---- ragged K/V rows: one wavefront per (row, kv head); rows are the head_rows before the
        // whole blocks and the tail_rows after them (every row of every sequence when there are none)
        const long long item = (long long)(wg - a.block_wgs) * 4 + wave;
        const int per_seq = a.head_rows + a.tail_rows;
        const int n_seq = a.n_tokens / a.rows;
        if (item >= (long long)n_seq * per_seq * a.n_kv_heads) return;
        const int rk = (int)(item / a.n_kv_heads), kvh = (int)(item - (long long)rk * a.n_kv_heads);
        const int seq = rk / per_seq;
        int row = rk - seq * per_seq;
        if (row >= a.head_rows) row += a.n_blocks * kBlockTokens;  // skip what the block workgroups cover
        const int token = seq * a.rows + row;
        const int position = a.position[seq] + row;
        const long long off = (long long)token * a.kv_stride + (long long)kvh * D + d0;
        float k[E], v[E], w[E];
        load_halves<E, ALIGNED>(k, a.k_proj + off);
        load_halves<E, ALIGNED>(v, a.v_proj + off);
        load_weight<E>(w, a.k_weight, d0);
        const Rotation<E> rot = rotation_for<E>(a.rotary_half, a.freq, position, lane);
        norm_rope<D>(k, w, a.eps, rot);
        const size_t page = ((size_t)a.slot[seq] * a.n_kv_heads + kvh) * (size_t)a.page_elems;
        store_halves<E, true>(a.k_layer + page + k_offset(D, position, d0), k);  // E dims inside one 8-dim group
#pragma unroll
        for (int e = 0; e < E; ++e) a.v_layer[page + v_offset(D, position, d0 + e)] = (_Float16)v[e];
        return;
    }

    // ---- query slices: one wavefront per (token, group of hpw <= 4 q heads); the heads' loads are
    // all in flight before the first is used and they share the token's rotation
    {
        const int groups = a.n_q_heads / a.hpw;
        const long long item = (long long)(wg - a.block_wgs - a.row_wgs) * 4 + wave;
        if (item >= (long long)a.n_tokens * groups) return;
        const int token = (int)(item / groups), head0 = (int)(item - (long long)token * groups) * a.hpw;
        const int seq = token / a.rows;
        const int position = a.position[seq] + (token - seq * a.rows);
        const _Float16 *src = a.q_packed + token * a.qp_stride + (long long)head0 * 2 * D + d0;
        float q[4][E], g[4][E], w[E];
#pragma unroll
        for (int h = 0; h < 4; ++h)
            if (h < a.hpw) {
                load_halves<E, ALIGNED>(q[h], src + h * 2 * D);
                load_halves<E, ALIGNED>(g[h], src + h * 2 * D + D);
            }
        load_weight<E>(w, a.q_weight, d0);
        const Rotation<E> rot = rotation_for<E>(a.rotary_half, a.freq, position, lane);
        _Float16 *qo = a.q_out + token * a.q_stride + (long long)head0 * D + d0;
        _Float16 *go = a.gate_out + token * a.g_stride + (long long)head0 * D + d0;
#pragma unroll
        for (int h = 0; h < 4; ++h)
            if (h < a.hpw) {
                norm_rope<D>(q[h], w, a.eps, rot);
                store_halves<E, ALIGNED>(qo + h * D, q[h]);
                store_halves<E, ALIGNED>(go + h * D, g[h]);
            }
    }
}

template <int D>
static int launch_epilogue_d(tt_hip_ctx *ctx, const EpilogueArgs &args, unsigned grid, bool aligned) {
    const size_t lds = args.block_wgs > 0 ? (size_t)2 * kBlockTokens * (D + kEpiloguePad) * sizeof(_Float16) : 0;
    const bool timed = ctx->profiling && !ctx->capturing && ctx->prof_used + 2 <= ctx->prof_events.size();
    if (timed) (void)hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream);
    if (aligned) hipLaunchKernelGGL((qkv_epilogue_kernel<D, true>), dim3(grid), dim3(256), lds, ctx->stream, args);
    else hipLaunchKernelGGL((qkv_epilogue_kernel<D, false>), dim3(grid), dim3(256), lds, ctx->stream, args);
    hipError_t e = hipGetLastError();
    if (timed) {
        (void)hipEventRecord(ctx->prof_events[ctx->prof_used + 1], ctx->stream);
        ctx->prof_used += 2;
    }
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "qkv_epilogue_kernel launch");
}

}  // namespace tt

using namespace tt;

extern "C" int tt_hip_qkv_epilogue_append(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                                          const int *positions, int rows, int n_q_heads, const tt_half *q_packed,
                                          size_t q_packed_stride_, const tt_half *k_proj, const tt_half *v_proj,
                                          size_t kv_stride_, const uint16_t *q_norm_weight_bf16,
                                          const uint16_t *k_norm_weight_bf16, float eps, int rotary_dim, float rope_theta,
                                          tt_half *q_out, size_t q_stride_, tt_half *gate_out, size_t gate_stride_) {
    const long long q_packed_stride = (long long)q_packed_stride_, kv_stride = (long long)kv_stride_;
    const long long q_stride = (long long)q_stride_, gate_stride = (long long)gate_stride_;
    if (!ctx || !kv || kv->ctx != ctx || !slots || !positions) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (!q_packed || !k_proj || !v_proj || !q_norm_weight_bf16 || !k_norm_weight_bf16 || !q_out || !gate_out)
        return TT_HIP_ERR_INVALID_ARGUMENT;
    if (layer < 0 || layer >= kv->n_layers || n_seq <= 0 || n_seq > kMaxEpilogueSeq || rows <= 0)
        return TT_HIP_ERR_INVALID_ARGUMENT;
    const int D = kv->head_dim, KH = kv->n_kv_heads;
    if (n_q_heads <= 0 || n_q_heads % KH != 0) return TT_HIP_ERR_SHAPE;
    // The reference's preconditions (PrefillQKVEpilogue.swift:40-55), plus this kernel's lane
    // mapping: a lane's D/64 dims and their rotation partners must not straddle lanes.
    if (rotary_dim < 0 || rotary_dim % 2 != 0 || rotary_dim > D || (rotary_dim / 2) % (D / 64) != 0 ||
        rotary_dim / 2 > kMaxRotaryHalf)
        return TT_HIP_ERR_SHAPE;
    if (q_packed_stride < (long long)n_q_heads * 2 * D || q_stride < (long long)n_q_heads * D ||
        gate_stride < (long long)n_q_heads * D || kv_stride < (long long)KH * D)
        return TT_HIP_ERR_SHAPE;
    if (!(eps >= 0.0f) || !(rope_theta > 0.0f)) return TT_HIP_ERR_INVALID_ARGUMENT;
    EpilogueArgs a{};
    for (int s = 0; s < n_seq; ++s) {
        if (slots[s] < 0 || slots[s] >= kv->n_slots || positions[s] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        if ((long long)positions[s] + rows > kv->capacity) return TT_HIP_ERR_CAPACITY;
        a.slot[s] = slots[s];
        a.position[s] = positions[s];
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    a.q_packed = reinterpret_cast<const _Float16 *>(q_packed);
    a.k_proj = reinterpret_cast<const _Float16 *>(k_proj);
    a.v_proj = reinterpret_cast<const _Float16 *>(v_proj);
    a.q_out = reinterpret_cast<_Float16 *>(q_out);
    a.gate_out = reinterpret_cast<_Float16 *>(gate_out);
    a.k_layer = kv->k[layer];
    a.v_layer = kv->v[layer];
    a.q_weight = q_norm_weight_bf16;
    a.k_weight = k_norm_weight_bf16;
    a.qp_stride = q_packed_stride;
    a.kv_stride = kv_stride;
    a.q_stride = q_stride;
    a.g_stride = gate_stride;
    a.page_elems = (long long)kv->page_elems();
    a.n_tokens = n_seq * rows;
    a.rows = rows;
    a.n_q_heads = n_q_heads;
    a.n_kv_heads = KH;
    a.rotary_half = rotary_dim / 2;
    a.eps = eps;
    // theta^(-2i / rotary_dim) exactly as the CPU engine computes it (CPUTensorOps.swift:129).
    for (int i = 0; i < a.rotary_half; ++i) a.freq[i] = powf(rope_theta, -(float)i * 2.0f / (float)rotary_dim);
    a.hpw = n_q_heads % 4 == 0 ? 4 : (n_q_heads % 2 == 0 ? 2 : 1);
    // Whole blocks only for one sequence (a prefill chunk); decode and verify rows are few.
    int first_full = 0, last_full_end = 0;
    if (n_seq == 1) {
        first_full = ((positions[0] + kBlockTokens - 1) / kBlockTokens) * kBlockTokens;
        last_full_end = ((positions[0] + rows) / kBlockTokens) * kBlockTokens;
    }
    if (n_seq == 1 && last_full_end > first_full) {
        a.first_block = first_full / kBlockTokens;
        a.n_blocks = (last_full_end - first_full) / kBlockTokens;
        a.head_rows = first_full - positions[0];
        a.tail_rows = positions[0] + rows - last_full_end;
    } else {
        a.first_block = 0;
        a.n_blocks = 0;
        a.head_rows = rows;
        a.tail_rows = 0;
    }
    a.block_wgs = a.n_blocks * KH;
    const long long ragged = (long long)n_seq * (a.head_rows + a.tail_rows) * KH;
    a.row_wgs = (int)((ragged + 3) / 4);
    const long long q_wgs = ((long long)a.n_tokens * (n_q_heads / a.hpw) + 3) / 4;
    const long long grid = (long long)a.block_wgs + a.row_wgs + q_wgs;
    if (grid > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
    const uintptr_t e_bytes = (uintptr_t)(D / 64) * 2;
    const bool aligned = (((uintptr_t)q_packed | (uintptr_t)k_proj | (uintptr_t)v_proj | (uintptr_t)q_out | (uintptr_t)gate_out) % e_bytes) == 0 &&
                         (q_packed_stride | kv_stride | q_stride | gate_stride) % (D / 64) == 0;
    switch (D) {
        case 256: return launch_epilogue_d<256>(ctx, a, (unsigned)grid, aligned);
        case 128: return launch_epilogue_d<128>(ctx, a, (unsigned)grid, aligned);
        case 64: return launch_epilogue_d<64>(ctx, a, (unsigned)grid, aligned);
        default: return TT_HIP_ERR_SHAPE;
    }
}
