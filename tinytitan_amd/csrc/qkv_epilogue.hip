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
// HBM-bound element-wise work.  A (token, head) slice is held by D/8 consecutive lanes, 8 dims
// (one 16-byte access) each: the sum of squares by a butterfly, the rotation partner by one cross-lane read.  K and
// V of whole 32-token blocks go through LDS and leave as full swizzled lines, like the plain
// block append; ragged edges and decode rows scatter.
#include <cmath>
#include <cstdint>

#include "internal.h"
#include "wave_ops.h"
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
    int kv_bits;  // 16: fp16 pages; 8 / 4: quantised pages (every K/V row then takes the row path)
    int rotary_half;
    float eps;
    // Workgroup ranges: [0, block_wgs) whole K/V blocks, then row_wgs of ragged K/V rows, then
    // the query slices (hpw q heads per wavefront).
    int block_wgs, row_wgs;
    int first_block, n_blocks;  // whole blocks (single-sequence calls only)
    int head_rows, tail_rows;   // ragged rows before / after the whole blocks (per sequence: rows when no blocks)
    int slot[kMaxEpilogueSeq], position[kMaxEpilogueSeq];
    int row0[kMaxEpilogueSeq];  // where position[s] is stored: the same, or position % capacity on a ring
    float freq[kMaxRotaryHalf];  // theta^(-2i / rotary_dim), computed on the host with the C library's powf
};

namespace {

constexpr int E = 8;  // dims per lane: one 16-byte access

__device__ __forceinline__ float bf16_to_float(unsigned short w) { return __builtin_bit_cast(float, (unsigned)w << 16); }

// A head slice (D dims) is held by D / 8 consecutive lanes, 8 dims each, so a wavefront works on
// 64 / (D / 8) slices at once.  Rotation pairs are (i, i + rotary_half): the partner lane is
// rotary_half / 8 lanes away inside the slice's lane group.
struct Rotation {
    float c[E], s[E];  // cos / sin of this lane's dims
    int partner;       // lane holding the other element of each pair
    bool low, rotated;
};

// Every head of a token turns by the same angles.  The accurate cosf / sinf are the expensive part
// of this kernel, and only the lanes that hold rotated dims would evaluate them (8 each, the
// others idling), so the work is spread instead: lane j of a slice's group of LPS lanes
// evaluates angle indices j, j + LPS, ... (at most 4), and every lane then collects the 8 it
// needs with cross-lane reads.
template <int LPS>
__device__ __forceinline__ Rotation rotation_for(int rotary_half, const float *freq, int position, int lane, int d0) {
    Rotation r;
    const int shift = rotary_half / E;
    r.low = d0 < rotary_half;
    r.rotated = d0 < 2 * rotary_half;
    r.partner = (r.low ? lane + shift : lane - shift) & 63;
    const int j = lane % LPS, group = lane - j;
    const int first = r.rotated ? (r.low ? d0 : d0 - rotary_half) : 0;  // first angle index this lane needs
    const int my_slot = first / LPS, my_lane = group + first % LPS;     // 8 | LPS: the 8 sit in one slot
#pragma unroll
    for (int e = 0; e < E; ++e) {
        r.c[e] = 1.0f;
        r.s[e] = 0.0f;
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        if (t * LPS < rotary_half) {  // wave-uniform
            const int i = t * LPS + j;
            const float angle = (float)position * freq[min(i, rotary_half - 1)];
            const float ct = cosf(angle), st = sinf(angle);
#pragma unroll
            for (int e = 0; e < E; ++e) {
                const float cc = __shfl(ct, my_lane + e), ss = __shfl(st, my_lane + e);
                if (r.rotated && my_slot == t) {
                    r.c[e] = cc;
                    r.s[e] = ss;
                }
            }
        }
    }
    return r;
}

// Per-head RMS norm (weight shared by all heads) and NeoX sub-dim rotation of the slices a
// wavefront holds (one per group of D / 8 lanes).
template <int D>
__device__ __forceinline__ void norm_rope(float (&x)[E], const float (&w)[E], float eps, const Rotation &rot) {
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < E; ++e) ss += x[e] * x[e];
    ss = group_sum<D / 8>(ss);  // the slice's lanes: DPP moves, no trip through LDS
    const float scale = 1.0f / sqrtf(ss / (float)D + eps);
#pragma unroll
    for (int e = 0; e < E; ++e) x[e] = x[e] * scale * w[e];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const float other = __shfl(x[e], rot.partner);
        if (rot.rotated) x[e] = rot.low ? x[e] * rot.c[e] - other * rot.s[e] : other * rot.s[e] + x[e] * rot.c[e];
    }
}

__device__ __forceinline__ void load_weight(float (&w)[E], const unsigned short *weight, int d0) {
#pragma unroll
    for (int e = 0; e < E; ++e) w[e] = bf16_to_float(weight[d0 + e]);
}

// 8 consecutive halves <-> fp32.  VEC: the address is a multiple of 16 bytes (one load/store).
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
template <bool VEC>
__device__ __forceinline__ void load_halves(float (&x)[E], const _Float16 *p) {
    if constexpr (VEC) {
        const h8 v = *reinterpret_cast<const h8 *>(p);
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = (float)v[e];
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) x[e] = (float)p[e];
    }
}
template <bool VEC>
__device__ __forceinline__ void store_halves(_Float16 *p, const float (&x)[E]) {
    if constexpr (VEC) {
        h8 v;
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] = (_Float16)x[e];
        *reinterpret_cast<h8 *>(p) = v;
    } else {
#pragma unroll
        for (int e = 0; e < E; ++e) p[e] = (_Float16)x[e];
    }
}

// Quantised pages: this lane's 8 consecutive dims of one K or V row, quantised the way
// kv_cache_quantize_affine does it (sources/TinyTitanCore/Metal/Quant/kv_cache_quantize.metal:7-73;
// the same arithmetic as kvq_append_kernel) and stored in the page's block layout.  The 8 lanes that
// hold a group of 64 dims find its minimum and maximum with three exchanges.  `x` holds the fp16
// values the quantiser's source row would hold.  Every lane runs the exchanges; `active` gates
// the stores.
__device__ __forceinline__ void store_quantised(const EpilogueArgs &a, uint8_t *block, bool is_v, int head_dim, int key,
                                                int d0, const float (&x)[E], int lane, bool active) {
    const int bits = a.kv_bits;
    float lo = x[0], hi = x[0];
#pragma unroll
    for (int e = 1; e < E; ++e) {
        lo = fminf(lo, x[e]);
        hi = fmaxf(hi, x[e]);
    }
    lo = group_min<8>(lo);  // a group of 64 dims is 8 lanes
    hi = group_max<8>(hi);
    const float levels = bits == 4 ? 15.0f : 255.0f;
    const float scale = hi > lo ? __fdiv_rn(hi - lo, levels) : 0.0f;
    unsigned q[E], upper[E];
#pragma unroll
    for (int e = 0; e < E; ++e) {
        q[e] = scale > 0.0f ? (unsigned)roundf(fminf(fmaxf(__fdiv_rn(x[e] - lo, scale), 0.0f), levels)) : 0u;
        upper[e] = __shfl_down(q[e], 4);  // the lane 32 dims up: the high nibbles of a 4-bit V byte
    }
    if (!active) return;
    if (!is_v) {
        if (bits == 8) {
            typedef unsigned u2 __attribute__((ext_vector_type(2)));
            const u2 w = {q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24), q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24)};
            *reinterpret_cast<u2 *>(block + kq_level_byte(8, key, d0)) = w;
        } else {
            unsigned w = 0;
#pragma unroll
            for (int e = 0; e < E; ++e) w |= q[e] << (4 * e);
            *reinterpret_cast<unsigned *>(block + kq_level_byte(4, key, d0)) = w;
        }
    } else if (bits == 8) {
#pragma unroll
        for (int e = 0; e < E; ++e) block[vq_level_byte(8, key, d0 + e)] = (uint8_t)q[e];
    } else if ((d0 & 32) == 0) {
#pragma unroll
        for (int e = 0; e < E; ++e) block[vq_level_byte(4, key, d0 + e)] = (uint8_t)(q[e] | (upper[e] << 4));
    }
    if ((lane & 7) == 0) {
        const int group = d0 / kQuantGroup;
        *reinterpret_cast<_Float16 *>(block + (is_v ? vq_scale_byte(head_dim, bits, key, group) : kq_scale_byte(head_dim, bits, key, group))) = (_Float16)scale;
        *reinterpret_cast<_Float16 *>(block + (is_v ? vq_bias_byte(head_dim, bits, key, group) : kq_bias_byte(head_dim, bits, key, group))) = (_Float16)lo;
    }
}

}  // namespace

// ALIGNED: every caller pointer is a multiple of 16 bytes and every stride a multiple of 8 halves.
template <int D, bool ALIGNED>
__global__ __launch_bounds__(256) void qkv_epilogue_kernel(const EpilogueArgs a) {
    constexpr int LPS = D / E;     // lanes per slice
    constexpr int SPW = 64 / LPS;  // slices a wavefront holds per access: 2, 4, 8 at D = 256, 128, 64
    extern __shared__ __attribute__((aligned(16))) _Float16 tile[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int sub = lane / LPS;          // which of the wavefront's slices
    const int d0 = (lane % LPS) * E;     // this lane's first dim
    const int wg = blockIdx.x;

    if (wg < a.block_wgs) {
        // ---- whole 32-token K/V blocks of a single sequence: one workgroup per (block, kv head).
        // These come first in the grid: they are the longest-running workgroups.
        const int blk = wg / a.n_kv_heads, kvh = wg - blk * a.n_kv_heads;
        constexpr int ROW = D + kEpiloguePad;
        constexpr int RPW = kBlockTokens / 4;  // rows per wavefront
        constexpr int NI = RPW / SPW;          // accesses per wavefront, SPW rows each
        _Float16 *kt = tile, *vt = tile + kBlockTokens * ROW;
        const int token0 = a.head_rows + blk * kBlockTokens;
        const int position0 = a.position[0] + token0;
        float k[NI][E], v[NI][E], w[E];
#pragma unroll
        for (int i = 0; i < NI; ++i) {  // all of the wavefront's rows in flight at once
            const int row = wave * RPW + i * SPW + sub;
            const long long off = (long long)(token0 + row) * a.kv_stride + (long long)kvh * D + d0;
            load_halves<ALIGNED>(k[i], a.k_proj + off);
            load_halves<ALIGNED>(v[i], a.v_proj + off);
        }
        load_weight(w, a.k_weight, d0);
#pragma unroll
        for (int i = 0; i < NI; ++i) {
            const int row = wave * RPW + i * SPW + sub;
            const Rotation rot = rotation_for<LPS>(a.rotary_half, a.freq, position0 + row, lane, d0);
            norm_rope<D>(k[i], w, a.eps, rot);
            store_halves<true>(kt + row * ROW + d0, k[i]);
            store_halves<true>(vt + row * ROW + d0, v[i]);
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
        // ---- ragged K/V rows: a lane group per (row, kv head); rows are the head_rows before the
        // whole blocks and the tail_rows after them (every row of every sequence when there are none)
        const long long item = ((long long)(wg - a.block_wgs) * 4 + wave) * SPW + sub;
        const int per_seq = a.head_rows + a.tail_rows;
        const int n_seq = a.n_tokens / a.rows;
        const bool active = item < (long long)n_seq * per_seq * a.n_kv_heads;
        const long long it = active ? item : 0;  // idle lane groups shadow item 0 (no stores)
        const int rk = (int)(it / a.n_kv_heads), kvh = (int)(it - (long long)rk * a.n_kv_heads);
        const int seq = rk / per_seq;
        int row = rk - seq * per_seq;
        if (row >= a.head_rows) row += a.n_blocks * kBlockTokens;  // skip what the block workgroups cover
        const int token = seq * a.rows + row;
        const int position = a.position[seq] + row;  // for the rotation
        const int stored = a.row0[seq] + row;        // for the page
        const long long off = (long long)token * a.kv_stride + (long long)kvh * D + d0;
        float k[E], v[E], w[E];
        load_halves<ALIGNED>(k, a.k_proj + off);
        load_halves<ALIGNED>(v, a.v_proj + off);
        load_weight(w, a.k_weight, d0);
        const Rotation rot = rotation_for<LPS>(a.rotary_half, a.freq, position, lane, d0);
        norm_rope<D>(k, w, a.eps, rot);
        if (a.kv_bits != 16) {  // wave-uniform
            const size_t at = ((size_t)a.slot[seq] * a.n_kv_heads + kvh) * (size_t)a.page_elems * 2 +
                              (size_t)(stored >> 5) * block_bytes(D, a.kv_bits);
#pragma unroll
            for (int e = 0; e < E; ++e) k[e] = (float)(_Float16)k[e];  // what the K row holds as fp16
            store_quantised(a, reinterpret_cast<uint8_t *>(a.k_layer) + at, false, D, stored & 31, d0, k, lane, active);
            store_quantised(a, reinterpret_cast<uint8_t *>(a.v_layer) + at, true, D, stored & 31, d0, v, lane, active);
            return;
        }
        if (active) {
            const size_t page = ((size_t)a.slot[seq] * a.n_kv_heads + kvh) * (size_t)a.page_elems;
            store_halves<true>(a.k_layer + page + k_offset(D, stored, d0), k);  // one whole 8-dim group
#pragma unroll
            for (int e = 0; e < E; ++e) a.v_layer[page + v_offset(D, stored, d0 + e)] = (_Float16)v[e];
        }
        return;
    }

    // ---- query slices: one wavefront per (token, run of QI * SPW q heads); all of the run's loads
    // are in flight before the first is used, and every head shares the token's rotation
    {
        constexpr int QI = 4;  // accesses per wavefront: 8 / 16 / 32 heads at D = 256 / 128 / 64
        const int runs = (a.n_q_heads + QI * SPW - 1) / (QI * SPW);
        const long long item = (long long)(wg - a.block_wgs - a.row_wgs) * 4 + wave;
        if (item >= (long long)a.n_tokens * runs) return;
        const int token = (int)(item / runs);
        const int head_first = (int)(item - (long long)token * runs) * (QI * SPW);
        const int seq = token / a.rows;
        const int position = a.position[seq] + (token - seq * a.rows);
        float q[QI][E], g[QI][E], w[E];
#pragma unroll
        for (int i = 0; i < QI; ++i) {
            const int head = min(head_first + i * SPW + sub, a.n_q_heads - 1);  // past the last head: shadow it
            const _Float16 *src = a.q_packed + token * a.qp_stride + (long long)head * 2 * D + d0;
            load_halves<ALIGNED>(q[i], src);
            load_halves<ALIGNED>(g[i], src + D);
        }
        load_weight(w, a.q_weight, d0);
        const Rotation rot = rotation_for<LPS>(a.rotary_half, a.freq, position, lane, d0);
#pragma unroll
        for (int i = 0; i < QI; ++i) {
            const int head = head_first + i * SPW + sub;
            norm_rope<D>(q[i], w, a.eps, rot);
            if (head < a.n_q_heads) {
                store_halves<ALIGNED>(a.q_out + token * a.q_stride + (long long)head * D + d0, q[i]);
                store_halves<ALIGNED>(a.gate_out + token * a.g_stride + (long long)head * D + d0, g[i]);
            }
        }
    }
}

template <int D>
static int launch_epilogue_d(tt_hip_ctx *ctx, const EpilogueArgs &args, unsigned grid, bool aligned) {
    const size_t lds = args.block_wgs > 0 ? (size_t)2 * kBlockTokens * (D + kEpiloguePad) * sizeof(_Float16) : 0;
    if (aligned) launch_profiled(ctx, qkv_epilogue_kernel<D, true>, dim3(grid), dim3(256), (unsigned)lds, args);
    else launch_profiled(ctx, qkv_epilogue_kernel<D, false>, dim3(grid), dim3(256), (unsigned)lds, args);
    hipError_t e = hipGetLastError();
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
    // mapping: a lane's 8 dims and their rotation partners must not straddle lanes.
    if (rotary_dim < 0 || rotary_dim % 2 != 0 || rotary_dim > D || (rotary_dim / 2) % 8 != 0 ||
        rotary_dim / 2 > kMaxRotaryHalf)
        return TT_HIP_ERR_SHAPE;
    if (q_packed_stride < (long long)n_q_heads * 2 * D || q_stride < (long long)n_q_heads * D ||
        gate_stride < (long long)n_q_heads * D || kv_stride < (long long)KH * D)
        return TT_HIP_ERR_SHAPE;
    if (!(eps >= 0.0f) || !(rope_theta > 0.0f)) return TT_HIP_ERR_INVALID_ARGUMENT;
    EpilogueArgs a{};
    for (int s = 0; s < n_seq; ++s) {
        if (slots[s] < 0 || slots[s] >= kv->n_slots || positions[s] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        if (!kv->holds_rows(positions[s], rows)) return TT_HIP_ERR_CAPACITY;
        a.slot[s] = slots[s];
        a.position[s] = positions[s];
        a.row0[s] = kv->physical(positions[s]);
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
    a.kv_bits = kv->bits;
    a.rotary_half = rotary_dim / 2;
    a.eps = eps;
    // theta^(-2i / rotary_dim) exactly as the CPU engine computes it (CPUTensorOps.swift:129).
    for (int i = 0; i < a.rotary_half; ++i) a.freq[i] = powf(rope_theta, -(float)i * 2.0f / (float)rotary_dim);
    // Whole blocks only for one sequence (a prefill chunk); decode and verify rows are few.
    int first_full = 0, last_full_end = 0;
    const int row0 = a.row0[0];  // whole blocks are blocks of the page: counted from where the rows are stored
    // (quantised pages: every row through the row path, which quantises.  Short chunks too: a block's workgroup writes
    // its 32 tokens one after the other, and with a handful of blocks those few workgroups are the whole launch's time
    // -- 128 tokens 6.6 us by blocks, 5.0 us by rows; 256 tokens 7.0 / 5.6; 512 tokens 7.9 / 8.2.)
    if (n_seq == 1 && kv->bits == 16 && rows >= 384) {
        first_full = ((row0 + kBlockTokens - 1) / kBlockTokens) * kBlockTokens;
        last_full_end = ((row0 + rows) / kBlockTokens) * kBlockTokens;
    }
    if (n_seq == 1 && last_full_end > first_full) {
        a.first_block = first_full / kBlockTokens;
        a.n_blocks = (last_full_end - first_full) / kBlockTokens;
        a.head_rows = first_full - row0;
        a.tail_rows = row0 + rows - last_full_end;
    } else {
        a.first_block = 0;
        a.n_blocks = 0;
        a.head_rows = rows;
        a.tail_rows = 0;
    }
    a.block_wgs = a.n_blocks * KH;
    const int spw = 64 / (D / 8);  // slices per wavefront access
    const long long ragged = (long long)n_seq * (a.head_rows + a.tail_rows) * KH;
    a.row_wgs = (int)((ragged + 4 * spw - 1) / (4 * spw));
    const long long runs = (n_q_heads + 4 * spw - 1) / (4 * spw);
    const long long q_wgs = ((long long)a.n_tokens * runs + 3) / 4;
    const long long grid = (long long)a.block_wgs + a.row_wgs + q_wgs;
    if (grid > 0x7fffffffLL) return TT_HIP_ERR_SHAPE;
    const bool aligned = (((uintptr_t)q_packed | (uintptr_t)k_proj | (uintptr_t)v_proj | (uintptr_t)q_out | (uintptr_t)gate_out) % 16) == 0 &&
                         (q_packed_stride | kv_stride | q_stride | gate_stride) % 8 == 0;
    switch (D) {
        case 256: return launch_epilogue_d<256>(ctx, a, (unsigned)grid, aligned);
        case 128: return launch_epilogue_d<128>(ctx, a, (unsigned)grid, aligned);
        case 64: return launch_epilogue_d<64>(ctx, a, (unsigned)grid, aligned);
        default: return TT_HIP_ERR_SHAPE;
    }
}
