// Split-K flash attention over the swizzled KV pages (fp16 values, or 8 / 4-bit levels
// dequantised in registers; linear pages or a ring): GQA decode, multi-row verify and causal
// prefill for the shapes the chunk kernel does not take, each with an optional sliding
// window, on gfx950 MFMA.
//
// Formulation (everything transposed so that per-query-row state is per-lane):
//   S^T[key][row]  = K[key][:] . Q[row][:]        A = K fragment,  B = Q^T fragment
//   O^T[d][row]   += V^T[d][key] * P^T[key][row]  A = V^T fragment, B = P^T fragment
// A lane owns one query row (column of S^T / O^T): the running max, the running
// sum and the rescale factor are plain per-lane scalars, the key reduction is
// in-register plus one or two cross-lane steps, and P goes from the first
// contraction's result registers straight into the second one's B operand
// because the V page stores keys in exactly that order.
//
// Replaces attention_decode_partial / attention_decode_combine
// (sources/TinyTitanCore/Metal/Attention/attention.metal:162-269, :395-437) and,
// for multi-row tiles, attention_prefill_causal_q8
// (sources/TinyTitanCore/Metal/Prefill/prefill.metal:1172-1313).
#include <type_traits>

#include "internal.h"
#include "wave_ops.h"

namespace tt {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr float kNegBig = -1.0e30f;  // finite stand-in for "no key seen yet"
// A row's reference maximum only moves when a block's maximum exceeds it by more than this (log2
// units): probabilities stay below 2^4, and the accumulators -- 144 registers that the 32-row
// variant keeps in AGPRs, so a rescale is three instructions each -- are rescaled a handful of
// times per row instead of in almost every block (with 32 rows per wave SOME row sees a new
// maximum in nearly every block).  Any reference works for the merges: m, l and O move together.
// Over fp16 pages the threshold is 8 (probabilities below 2^8, well inside fp16): a wavefront that walks only a few
// dozen blocks, as in a sparse chunk, spends a visible share of them rescaling.  Over quantised pages it stays 4: there
// a probability is multiplied by a group's scale (up to 514) and a boost of 4 before it becomes an fp16 operand.
constexpr float kLazyRescale = 4.0f, kLazyRescaleHalfPages = 8.0f;
constexpr int kLdsPad = 4;           // floats of padding per staged O row

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

// Eight halves from a row that is only guaranteed 2-byte alignment, as ONE load and without a
// branch (global loads take any alignment here; a branch on the alignment would make the
// compiler wait for every outstanding load where the two paths join).
typedef h8 h8_unaligned __attribute__((aligned(2)));
// (A pointer rebuilt from scalar registers has lost its address space; the query pointer is device memory, and
// saying so keeps its loads global ones, counted apart from LDS traffic.)
typedef const __attribute__((address_space(1))) _Float16 *global_halves;
__device__ __forceinline__ h8 load_h8(global_halves p) {
    return *reinterpret_cast<const __attribute__((address_space(1))) h8_unaligned *>(p);
}

// Tile decoding shared by both kernels.
struct TileInfo {
    int kvh, hsub, tok_tile, t0, tile_rows, tile_end, start, total;
    int k0;  // first key of split 0: 0, or the block that holds the first key the tile's first row sees through its window
};

__device__ __forceinline__ TileInfo tile_info(const SplitKHot &a, const SplitKSeq &sq, int tile) {
    TileInfo t;
    if (a.tok_tiles == 1 && a.hsubs == 1) {  // a decode step, a verify pass of a few rows: a tile is a KV head
        t.tok_tile = 0;
        t.hsub = 0;
        t.kvh = tile;
    } else {
        t.tok_tile = tile % a.tok_tiles;
        t.hsub = (tile / a.tok_tiles) % a.hsubs;
        t.kvh = tile / (a.tok_tiles * a.hsubs);
    }
    t.start = sq.start;
    t.total = sq.total;
    t.t0 = t.tok_tile * a.tt;
    t.tile_rows = min(a.tt, a.rows - t.t0);
    t.tile_end = max(0, min(t.total, t.start + t.t0 + t.tile_rows));  // keys visible to the tile's last row
    const int first_lim = min(t.total, t.start + t.t0 + 1);
    t.k0 = (a.window > 0 && first_lim > a.window) ? ((first_lim - a.window) & ~31) : 0;
    return t;
}

// The gate's four values of one output item, asked for ahead of the arithmetic they end up multiplying (a combine pass
// that fetches them only when its sums are done waits for memory once more with nothing else to do).
__device__ __forceinline__ void load_gate4(const SplitKArgs &a, int seq, int tok, int head, int d, int D, bool aligned, float (&g)[4]) {
    g[0] = g[1] = g[2] = g[3] = 0.0f;
    if (!a.gate) return;
    const _Float16 *gp = a.gate + seq * a.g_seq_stride + tok * a.g_tok_stride + (long long)head * D + d;
    if (aligned) {
        const h4 gv = *reinterpret_cast<const h4 *>(gp);
#pragma unroll
        for (int i = 0; i < 4; ++i) g[i] = (float)gv[i];
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) g[i] = (float)gp[i];
    }
}
// Final value of one output element with the gate's values in hand: normalise, gate in fp32, round once.
__device__ __forceinline__ void store_out4_gated(const SplitKArgs &a, int seq, int tok, int head, int d, int D, f4 o, float inv_l,
                                                 bool aligned, const float (&g)[4]) {
    f4 r = o * inv_l;
    if (a.gate) {
#pragma unroll
        for (int i = 0; i < 4; ++i) r[i] *= 1.0f / (1.0f + __expf(-g[i]));
    }
    _Float16 *op = a.out + seq * a.o_seq_stride + tok * a.o_tok_stride + (long long)head * D + d;
    if (aligned) {
        *reinterpret_cast<h4 *>(op) = h4{(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) op[i] = (_Float16)r[i];
    }
}

// Final value of one output element: normalise, gate in fp32, round once.
__device__ __forceinline__ void store_out4(const SplitKArgs &a, int seq, int tok, int head, int d, int D, f4 o,
                                           float inv_l, bool aligned) {
    f4 r = o * inv_l;
    if (a.gate) {
        const _Float16 *gp = a.gate + seq * a.g_seq_stride + tok * a.g_tok_stride + (long long)head * D + d;
        float g0, g1, g2, g3;
        if (aligned) {
            h4 gv = *reinterpret_cast<const h4 *>(gp);
            g0 = (float)gv[0]; g1 = (float)gv[1]; g2 = (float)gv[2]; g3 = (float)gv[3];
        } else {
            g0 = (float)gp[0]; g1 = (float)gp[1]; g2 = (float)gp[2]; g3 = (float)gp[3];
        }
        r[0] *= 1.0f / (1.0f + __expf(-g0));
        r[1] *= 1.0f / (1.0f + __expf(-g1));
        r[2] *= 1.0f / (1.0f + __expf(-g2));
        r[3] *= 1.0f / (1.0f + __expf(-g3));
    }
    _Float16 *op = a.out + seq * a.o_seq_stride + tok * a.o_tok_stride + (long long)head * D + d;
    if (aligned) {
        h4 hv = {(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
        *reinterpret_cast<h4 *>(op) = hv;
    } else {
        op[0] = (_Float16)r[0]; op[1] = (_Float16)r[1]; op[2] = (_Float16)r[2]; op[3] = (_Float16)r[3];
    }
}

// ---------------------------------------------------------------------------
// Register tiles of one 32-key block and the per-row online-softmax state.
// NT = 32 uses v_mfma_f32_32x32x16_f16 (32 query rows per wave), NT = 16 uses
// v_mfma_f32_16x16x32_f16 (16 query rows, half the accumulator registers).
// ---------------------------------------------------------------------------
template <int D, int NT>
struct KTile;
template <int D, int NT>
struct VTile;
template <int D>
struct KTile<D, 32> {
    h8 f[D / 16];
};
template <int D>
struct VTile<D, 32> {
    h8 f[D / 32][2];
};
template <int D>
struct KTile<D, 16> {
    h8 a[D / 32], b[D / 32];  // S^T tile a: keys {0-7, 16-23}; tile b: keys {8-15, 24-31}
};
template <int D>
struct VTile<D, 16> {
    h8 f[D / 16];
};

template <int D, int NT>
struct Lane {
    static constexpr int LN = NT;
    int li, g;       // position inside the lane group, lane group
    int koff, voff;  // this lane's element offset inside a K / V block
    __device__ __forceinline__ explicit Lane(int lane) {
        li = lane & (LN - 1);
        g = lane / LN;
        if constexpr (NT == 32) {
            koff = (g * 32 + li) * 8;
            voff = (li * 4 + g) * 8;
        } else {
            const int ka = li < 8 ? li : li + 8;
            koff = (g * 32 + ka) * 8;
            voff = (li * 4 + g) * 8;
        }
    }
};

// K/V pages are read through buffer resources: the lane's byte offset inside a
// block is one VGPR for the whole kernel, the block/step offset rides in an SGPR
// and the immediate, so the loads need no per-load address registers, and reads
// past the page would return zeros instead of faulting.
typedef int i4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void *base, unsigned bytes) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, bytes, 0x00020000);
}

// AUX is the load's cache policy: 0, or kStreamed for pages that a launch reads exactly once (a decode step, a
// verify pass of a few rows).  Those loads are marked non-temporal: the data is not kept in L2 or in the
// memory-side cache ahead of lines that will be used again (the split partials, the next layer's weights), and
// a pass over 64 MiB of pages runs 7 % faster for it (13.5 -> 12.5 us), the step behind it 10 %.
constexpr int kStreamed = 2;  // the nt bit of a gfx950 buffer load
template <int AUX>
__device__ __forceinline__ h8 buf_load_h8(__amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes, unsigned wave_bytes) {
    i4 r = __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, wave_bytes, AUX);
    return __builtin_bit_cast(h8, r);
}

// `block_bytes` is the block's byte offset inside the page (wave-uniform, always that of a block
// the page holds).  `void_bytes` is added to every lane's offset: 0 for a real load; kVoidLoad
// makes every lane's offset exceed the resource's size, so the load returns zeros without going
// to memory -- the lane offset is what the hardware's range check is defined on.
constexpr unsigned kVoidLoad = 0x7ff00000u;

template <int AUX, int D, int NT>
__device__ __forceinline__ void load_k(KTile<D, NT> &t, __amdgpu_buffer_rsrc_t rk, unsigned block_bytes,
                                       const Lane<D, NT> &ln, unsigned void_bytes = 0) {
    const unsigned lane_bytes = (unsigned)ln.koff * 2u + void_bytes;
    if constexpr (NT == 32) {
#pragma unroll
        for (int s = 0; s < D / 16; ++s) t.f[s] = buf_load_h8<AUX>(rk, lane_bytes, block_bytes + s * (2 * 32 * 16));
    } else {
#pragma unroll
        for (int s = 0; s < D / 32; ++s) {
            t.a[s] = buf_load_h8<AUX>(rk, lane_bytes, block_bytes + s * (4 * 32 * 16));
            t.b[s] = buf_load_h8<AUX>(rk, lane_bytes, block_bytes + s * (4 * 32 * 16) + 128);
        }
    }
}

template <int AUX, int D, int NT>
__device__ __forceinline__ void load_v(VTile<D, NT> &t, __amdgpu_buffer_rsrc_t rv, unsigned block_bytes,
                                       const Lane<D, NT> &ln, unsigned void_bytes = 0) {
    const unsigned lane_bytes = (unsigned)ln.voff * 2u + void_bytes;
    if constexpr (NT == 32) {
#pragma unroll
        for (int mt = 0; mt < D / 32; ++mt)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) t.f[mt][tt] = buf_load_h8<AUX>(rv, lane_bytes, block_bytes + mt * (32 * 4 * 16) + tt * 32);
    } else {
#pragma unroll
        for (int mt = 0; mt < D / 16; ++mt) t.f[mt] = buf_load_h8<AUX>(rv, lane_bytes, block_bytes + mt * (16 * 4 * 16));
    }
}

template <int D, int NT>
struct RowState {
    static constexpr int MT = (NT == 32) ? D / 32 : D / 16;
    typedef typename std::conditional<NT == 32, f16v, f4>::type acc_t;
    float m, l;
    acc_t o[MT];
    __device__ __forceinline__ void init() {
        m = kNegBig;
        l = 0.0f;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) o[mt] = (acc_t)0.0f;
    }
};

// One 32-key block, phase 1: S^T = K Q^T (log2 domain, scaled).  For NT = 16 the
// query fragments come from LDS (`qlds`, one h8 per lane per step) so that the
// wave stays within 256 registers; for NT = 32 they live in registers (`qf`).
template <int D, int NT>
struct Scores;
template <int D>
struct Scores<D, 32> {
    f16v s;
};
template <int D>
struct Scores<D, 16> {
    f4 sa, sb;
};

template <int D, int NT>
__device__ __forceinline__ void block_scores(Scores<D, NT> &sc, const KTile<D, NT> &kt, const h8 *qf, const h8 *qlds,
                                             int lane) {
    if constexpr (NT == 32) {
        (void)qlds;
        (void)lane;
        sc.s = (f16v)0.0f;
#pragma unroll
        for (int t = 0; t < D / 16; ++t) sc.s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kt.f[t], qf[t], sc.s, 0, 0, 0);
    } else {
        (void)qf;
        sc.sa = (f4)0.0f;
        sc.sb = (f4)0.0f;
#pragma unroll
        for (int t = 0; t < D / 32; ++t) {
            const h8 q = qlds[t * 64 + lane];
            sc.sa = __builtin_amdgcn_mfma_f32_16x16x32_f16(kt.a[t], q, sc.sa, 0, 0, 0);
            sc.sb = __builtin_amdgcn_mfma_f32_16x16x32_f16(kt.b[t], q, sc.sb, 0, 0, 0);
        }
    }
}

// Rescaling the 32-row variant's accumulators.  They live in AGPRs, which only the matrix instructions, loads and the
// accvgpr moves can name.  Written as `o *= alpha` the compiler copies all of them to VGPRs at the top of EVERY block
// -- 128 to 144 instructions -- whether the block's rows move their reference or not, and only the multiplies and the
// copies back sit behind the branch.  Here four accumulator registers at a time are operands of an assembly block
// that wants them in AGPRs and multiplies them where they are, so a block that moves no row touches no accumulator.
// Wait states the hardware leaves to software: a vector instruction must not read or overwrite a matrix instruction's
// result for up to 18 cycles after that issued (`rescale_settle` waits 19 ahead of the first block: in the loop sixteen
// score MFMAs and the softmax separate them from the last P.V MFMA anyway), and a matrix instruction must not read a
// register within 2 cycles of a vector instruction writing it (every block ends on a wait of 5).
__device__ __forceinline__ void rescale_settle() { asm volatile("s_nop 15\n\ts_nop 2"); }
__device__ __forceinline__ void rescale4(float &a0, float &a1, float &a2, float &a3, float alpha) {
    float t0, t1, t2, t3;
    asm volatile(
        "v_accvgpr_read_b32 %4, %0\n\tv_accvgpr_read_b32 %5, %1\n\tv_accvgpr_read_b32 %6, %2\n\tv_accvgpr_read_b32 %7, %3\n\t"
        "v_mul_f32 %4, %8, %4\n\tv_mul_f32 %5, %8, %5\n\tv_mul_f32 %6, %8, %6\n\tv_mul_f32 %7, %8, %7\n\t"
        "v_accvgpr_write_b32 %0, %4\n\tv_accvgpr_write_b32 %1, %5\n\tv_accvgpr_write_b32 %2, %6\n\tv_accvgpr_write_b32 %3, %7\n\t"
        "s_nop 4"
        : "+a"(a0), "+a"(a1), "+a"(a2), "+a"(a3), "=&v"(t0), "=&v"(t1), "=&v"(t2), "=&v"(t3)
        : "v"(alpha));
}
__device__ __forceinline__ void rescale_tile(f16v &o, float alpha) {
#pragma unroll
    for (int j = 0; j < 16; j += 4) {
        float a0 = o[j], a1 = o[j + 1], a2 = o[j + 2], a3 = o[j + 3];
        rescale4(a0, a1, a2, a3, alpha);
        o[j] = a0;
        o[j + 1] = a1;
        o[j + 2] = a2;
        o[j + 3] = a3;
    }
}

// Phase 2a: mask and online softmax of one block.  This lane's row sees keys [lo, lim); kbase is
// the block's first key.  Leaves the block's probabilities in `pf` as fp16 B
// operands of the P.V MFMAs and rescales the row's accumulators (`extra` is a further one that
// follows the same running max, or null).
template <int D, int NT>
struct Probs;
template <int D>
struct Probs<D, 32> {
    h8 pf[2];
};
template <int D>
struct Probs<D, 16> {
    h8 pf;
};

template <int D, int NT>
__device__ __forceinline__ void block_softmax(RowState<D, NT> &st, Scores<D, NT> &sc, Probs<D, NT> &pr,
                                              const Lane<D, NT> &ln, int kbase, int lo, int lim, float scale_log2e,
                                              typename RowState<D, NT>::acc_t *extra = nullptr, unsigned kept = ~0u,
                                              const unsigned *row_keep = nullptr, unsigned row_bits = ~0u) {
    // kept: bit i set = key kbase + i takes part (a sparse selection shared by the tile's rows; all ones without one).
    // row_keep: this lane's own row's 32 selection bytes of the block, as 8 words (a per-query selection).
    // row_bits: the same as one bit per key (a per-query selection that came as index lists); all ones without one.
    const bool any_row_bits = __any(row_bits != ~0u);
    const bool need_mask = __any(kbase + 32 > lim || kbase < lo) || kept != ~0u || row_keep != nullptr || any_row_bits;
    unsigned rk[4] = {~0u, ~0u, ~0u, ~0u};  // the words that hold this lane's keys, picked by the lane's place in the tile
    if (row_keep) {
        if constexpr (NT == 32) {  // key offsets 8 a + 4 g + (v & 3): word 2 a + g
#pragma unroll
            for (int i = 0; i < 4; ++i) rk[i] = ln.g ? row_keep[2 * i + 1] : row_keep[2 * i];
        } else {  // tile a: offsets 4 (g & 1) + 16 (g >> 1) + v, tile b: 8 more
            const unsigned lo_a = (ln.g & 1) ? row_keep[1] : row_keep[0], hi_a = (ln.g & 1) ? row_keep[5] : row_keep[4];
            const unsigned lo_b = (ln.g & 1) ? row_keep[3] : row_keep[2], hi_b = (ln.g & 1) ? row_keep[7] : row_keep[6];
            rk[0] = (ln.g >> 1) ? hi_a : lo_a;
            rk[1] = (ln.g >> 1) ? hi_b : lo_b;
        }
    }
    if constexpr (NT == 32) {
        f16v &s = sc.s;
        // The three reasons to drop a key, each behind its own wave-uniform test and over all 16 values at once: a
        // selected block far behind the chunk's rows needs no range test, a dense block at the diagonal no selection.
        const bool need_range = __any(kbase + 32 > lim || kbase < lo);
#pragma unroll
        for (int v = 0; v < 16; ++v) s[v] *= scale_log2e;
        if (need_range) {
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const int key = kbase + 8 * (v >> 2) + 4 * ln.g + (v & 3);
                if (key >= lim || key < lo) s[v] = -INFINITY;
            }
        }
        if (kept != ~0u) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (!((kept >> (8 * (v >> 2) + 4 * ln.g + (v & 3))) & 1u)) s[v] = -INFINITY;
        }
        if (row_keep) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (!((rk[v >> 2] >> (8 * (v & 3))) & 0xffu)) s[v] = -INFINITY;
        }
        if (any_row_bits) {
#pragma unroll
            for (int v = 0; v < 16; ++v)
                if (!((row_bits >> (8 * (v >> 2) + 4 * ln.g + (v & 3))) & 1u)) s[v] = -INFINITY;
        }
        float mx = kNegBig;
#pragma unroll
        for (int v = 0; v < 16; ++v) mx = fmaxf(mx, s[v]);
        mx = max_across_halves(mx);
        const float m_new = mx > st.m + (extra ? kLazyRescale : kLazyRescaleHalfPages) ? mx : st.m;
        const float alpha = fast_exp2(st.m - m_new);
        float psum = 0.0f;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const float p = fast_exp2(s[v] - m_new);
            psum += p;
            pr.pf[v >> 3][v & 7] = (_Float16)p;
        }
        st.l = st.l * alpha + psum;
        st.m = m_new;
        if (!__all(alpha == 1.0f)) {
            rescale_settle();
#pragma unroll
            for (int mt = 0; mt < D / 32; ++mt) rescale_tile(st.o[mt], alpha);
            if (extra) rescale_tile(*extra, alpha);
        }
    } else {
        f4 &sa = sc.sa, &sb = sc.sb;
        const int key0 = kbase + (ln.g & 1) * 4 + (ln.g >> 1) * 16;  // first key of this lane's tile-a results
        float mx = kNegBig;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            float xa = sa[v] * scale_log2e, xb = sb[v] * scale_log2e;
            if (need_mask) {
                if (key0 + v >= lim || key0 + v < lo || !((kept & row_bits) >> (key0 + v - kbase) & 1u) || !((rk[0] >> (8 * v)) & 0xffu))
                    xa = -INFINITY;
                if (key0 + 8 + v >= lim || key0 + 8 + v < lo || !((kept & row_bits) >> (key0 + 8 + v - kbase) & 1u) ||
                    !((rk[1] >> (8 * v)) & 0xffu))
                    xb = -INFINITY;
            }
            sa[v] = xa;
            sb[v] = xb;
            mx = fmaxf(mx, fmaxf(xa, xb));
        }
        mx = max_across_quarters(mx);
        const float m_new = mx > st.m + (extra ? kLazyRescale : kLazyRescaleHalfPages) ? mx : st.m;
        const float alpha = fast_exp2(st.m - m_new);
        float psum = 0.0f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const float pa = fast_exp2(sa[v] - m_new), pb = fast_exp2(sb[v] - m_new);
            psum += pa + pb;
            pr.pf[v] = (_Float16)pa;
            pr.pf[4 + v] = (_Float16)pb;
        }
        st.l = st.l * alpha + psum;
        st.m = m_new;
        if (!__all(alpha == 1.0f)) {
#pragma unroll
            for (int mt = 0; mt < D / 16; ++mt) st.o[mt] *= alpha;
            if (extra) *extra *= alpha;
        }
    }
}

// Phase 2b: O^T += V^T P^T.
template <int D, int NT>
__device__ __forceinline__ void block_softmax_pv(RowState<D, NT> &st, Scores<D, NT> &sc, const VTile<D, NT> &vt,
                                                 const Lane<D, NT> &ln, int kbase, int lo, int lim, float scale_log2e,
                                                 unsigned kept = ~0u, const unsigned *row_keep = nullptr, unsigned row_bits = ~0u) {
    Probs<D, NT> pr;
    block_softmax<D, NT>(st, sc, pr, ln, kbase, lo, lim, scale_log2e, nullptr, kept, row_keep, row_bits);
    if constexpr (NT == 32) {
#pragma unroll
        for (int mt = 0; mt < D / 32; ++mt)
#pragma unroll
            for (int t = 0; t < 2; ++t)
                st.o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt.f[mt][t], pr.pf[t], st.o[mt], 0, 0, 0);
    } else {
#pragma unroll
        for (int mt = 0; mt < D / 16; ++mt) st.o[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vt.f[mt], pr.pf, st.o[mt], 0, 0, 0);
    }
}

// The two phases of a 32-row fp16 tile with the NEXT block's loads between their MFMAs: a fragment's load follows the
// MFMA that read it, into the same registers, one scheduling region per pair.  Where the block's loads stand apart
// from the MFMAs in the source, the compiler is free to move them ahead of the MFMAs -- into 64 other registers,
// which the per-query selection's variant does not have: it then parks the tile in AGPRs at the end of the block,
// behind a wait for every load, and nothing of the next block is in flight under the arithmetic of this one.
template <int AUX, int D>
__device__ __forceinline__ void block_scores_refill(Scores<D, 32> &sc, KTile<D, 32> &kt, const h8 *qf, __amdgpu_buffer_rsrc_t rk,
                                                    unsigned next_bytes, const Lane<D, 32> &ln, unsigned void_bytes) {
    const unsigned lane_bytes = (unsigned)ln.koff * 2u + void_bytes;
    sc.s = (f16v)0.0f;
#pragma unroll
    for (int t = 0; t < D / 16; ++t) {
        sc.s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kt.f[t], qf[t], sc.s, 0, 0, 0);
        asm volatile("" : "+a"(sc.s));  // (an MFMA is no memory operation: only its result's use here keeps it ahead of the load)
        kt.f[t] = buf_load_h8<AUX>(rk, lane_bytes, next_bytes + t * (2 * 32 * 16));
        __builtin_amdgcn_sched_barrier(0);
    }
}
template <int AUX, int D>
__device__ __forceinline__ void block_softmax_pv_refill(RowState<D, 32> &st, Scores<D, 32> &sc, VTile<D, 32> &vt,
                                                        const Lane<D, 32> &ln, int kbase, int lo, int lim, float scale_log2e,
                                                        __amdgpu_buffer_rsrc_t rv, unsigned next_bytes, unsigned void_bytes,
                                                        unsigned kept, const unsigned *row_keep, unsigned row_bits) {
    Probs<D, 32> pr;
    block_softmax<D, 32>(st, sc, pr, ln, kbase, lo, lim, scale_log2e, nullptr, kept, row_keep, row_bits);
    const unsigned lane_bytes = (unsigned)ln.voff * 2u + void_bytes;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int mt = 0; mt < D / 32; ++mt) {
#pragma unroll
        for (int t = 0; t < 2; ++t) st.o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vt.f[mt][t], pr.pf[t], st.o[mt], 0, 0, 0);
        asm volatile("" : "+a"(st.o[mt]));
#pragma unroll
        for (int t = 0; t < 2; ++t) vt.f[mt][t] = buf_load_h8<AUX>(rv, lane_bytes, next_bytes + mt * (32 * 4 * 16) + t * 32);
        __builtin_amdgcn_sched_barrier(0);
    }
}

// ---------------------------------------------------------------------------
// Quantised pages (8 or 4 bits per value; layout in kv_layout.h).  A block's tiles hold the
// levels as loaded plus this lane's scales and biases; levels become fp16 MFMA operands in
// registers, right before the instruction that uses them:
//   K  operand = level * scale + bias per (key, group of 64 dims), one packed fp16 FMA per two
//      elements -- the loader of sources/TinyTitanCore/Metal/Attention/attention.metal:89-117
//      with one fp16 rounding of the product-sum instead of none.
//   V  O^T[d][row] = sum_key (level * scale + bias) P = sum_key level * (scale * P)
//                                                     + sum_key bias * P:
//      the scale goes into P (one B operand per group), the levels are the A operand as they
//      are, and the bias term is ONE more MFMA per key step whose A rows are the groups' biases;
//      its accumulator (row = group) is added to the group's dims once, at the end.  scale * P
//      carries a factor 4 (the level accumulators are divided by 4 at the end), which keeps
//      small probabilities times small scales out of fp16's subnormal range; fp16 values bound
//      scale to 514 and P stays below 16, so 4 * scale * P stays below 32896.
// Levels are widened with v_perm_b32: byte b under exponent byte 0x64 is the fp16 number
// 1024 + b, and subtracting 1024 is exact.
// ---------------------------------------------------------------------------
typedef unsigned u2v __attribute__((ext_vector_type(2)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
constexpr float kProbBoost = 4.0f;

template <int AUX, int N>
__device__ __forceinline__ void buf_load_words(unsigned (&dst)[N], __amdgpu_buffer_rsrc_t rsrc, unsigned lane_bytes,
                                               unsigned wave_bytes) {
    static_assert(N == 1 || N == 2 || N == 4, "one load instruction");
    if constexpr (N == 1) {
        dst[0] = __builtin_amdgcn_raw_buffer_load_b32(rsrc, lane_bytes, wave_bytes, AUX);
    } else if constexpr (N == 2) {
        const u2v r = __builtin_amdgcn_raw_buffer_load_b64(rsrc, lane_bytes, wave_bytes, AUX);
        dst[0] = r[0];
        dst[1] = r[1];
    } else {
        const u4v r = __builtin_bit_cast(u4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, lane_bytes, wave_bytes, AUX));
        dst[0] = r[0];
        dst[1] = r[1];
        dst[2] = r[2];
        dst[3] = r[3];
    }
}

// Eight bytes -> eight halves holding 0..255 exactly.
__device__ __forceinline__ h8 widen_bytes(unsigned w0, unsigned w1) {
    const unsigned e = 0x64646464u;
    const u4v x = {__builtin_amdgcn_perm(e, w0, 0x04010400u), __builtin_amdgcn_perm(e, w0, 0x04030402u),
                   __builtin_amdgcn_perm(e, w1, 0x04010400u), __builtin_amdgcn_perm(e, w1, 0x04030402u)};
    return __builtin_bit_cast(h8, x) - (h8)(_Float16)1024;
}
// Eight nibbles of one dword, element 2 i in the low nibble of byte i, in element order.
__device__ __forceinline__ h8 widen_nibbles(unsigned w) {
    const unsigned lo = w & 0x0f0f0f0fu, hi = (w >> 4) & 0x0f0f0f0fu, e = 0x64006400u;
    const u4v x = {__builtin_amdgcn_perm(hi, lo, 0x0c040c00u) | e, __builtin_amdgcn_perm(hi, lo, 0x0c050c01u) | e,
                   __builtin_amdgcn_perm(hi, lo, 0x0c060c02u) | e, __builtin_amdgcn_perm(hi, lo, 0x0c070c03u) | e};
    return __builtin_bit_cast(h8, x) - (h8)(_Float16)1024;
}

template <int BITS>
__device__ __forceinline__ h8 k_operand(const unsigned (&w)[BITS / 4], unsigned scale_bias) {
    const h2 sb = __builtin_bit_cast(h2, scale_bias);
    h8 levels;
    if constexpr (BITS == 8) levels = widen_bytes(w[0], w[1]);
    else levels = widen_nibbles(w[0]);
    return levels * (h8)sb[0] + (h8)sb[1];
}

template <int D, int NT, int BITS>
struct KTileQ;
template <int D, int NT, int BITS>
struct VTileQ;
// K levels: one load per lane holds the 16 dims of a key's unit -- 16 bytes at 8 bits, 8 at 4 --
// and feeds two contraction steps (dims 0-7, then 8-15).  The lane's unit of step pair p is
// 2 p + g (32-row tiles: dims 32 p + 16 g ..) or 4 p + g (16-row tiles: dims 64 p + 16 g ..); the
// query fragments in LDS are laid out in the same order (q_dim_of_step).
template <int D, int BITS>
struct KTileQ<D, 32, BITS> {
    unsigned f[D / 32][BITS / 2];
    unsigned sb[D / 64];  // {scale, bias} of this lane's key, per group
};
template <int D, int BITS>
struct KTileQ<D, 16, BITS> {
    unsigned a[D / 64][BITS / 2], b[D / 64][BITS / 2];
    unsigned sba[D / 64], sbb[D / 64];
};
// V levels: one load per lane holds its chunk's eight keys for the dims d and d + 32 -- two runs
// of 8 bytes at 8 bits, the low and high nibbles of one run at 4 bits.
template <int D, int BITS>
struct VTileQ<D, 32, BITS> {
    unsigned f[D / 64][2][BITS / 2];  // [pair of dim tiles 2 j, 2 j + 1][key step][dword]
    unsigned sc[D / 64][2][4];        // 8 scales per group and key step
    unsigned bias[2][4];              // rows = groups: this lane's group's 8 biases per key step, or zeros
};
template <int D, int BITS>
struct VTileQ<D, 16, BITS> {
    unsigned f[D / 32][BITS / 2];  // load i = 2 j + rr: dim tiles 4 j + rr and 4 j + 2 + rr
    unsigned sc[D / 64][4];
    unsigned bias[4];
};

// First dim of the 8 that lane group g contracts in step t of a quantised tile.
template <int NT>
__device__ __forceinline__ int q_dim_of_step(int t, int g) {
    return (NT == 32 ? 32 : 64) * (t >> 1) + 16 * g + 8 * (t & 1);
}

// The operand of contraction step `half` (0 / 1) of a loaded K unit.
template <int BITS>
__device__ __forceinline__ h8 k_unit_operand(const unsigned (&w)[BITS / 2], int half, unsigned scale_bias) {
    if constexpr (BITS == 8) {
        const unsigned pair[2] = {w[2 * half], w[2 * half + 1]};
        return k_operand<8>(pair, scale_bias);
    } else {
        const unsigned one[1] = {w[half]};
        return k_operand<4>(one, scale_bias);
    }
}
// The two V operands of a loaded run: dims d (lo) and d + 32 (hi).
template <int BITS>
__device__ __forceinline__ void v_run_operands(const unsigned (&w)[BITS / 2], h8 &lo, h8 &hi) {
    if constexpr (BITS == 8) {
        lo = widen_bytes(w[0], w[1]);
        hi = widen_bytes(w[2], w[3]);
    } else {
        lo = widen_bytes(w[0] & 0x0f0f0f0fu, w[1] & 0x0f0f0f0fu);
        hi = widen_bytes((w[0] >> 4) & 0x0f0f0f0fu, (w[1] >> 4) & 0x0f0f0f0fu);
    }
}

// Byte offsets of this lane inside a block's K / V levels, and of the tile's loads.
template <int D, int NT, int BITS>
struct QuantOffsets {
    static constexpr unsigned LEVELS = 32u * D * BITS / 8, GPH = D / 64;
    static constexpr unsigned K_UNIT = 16u * BITS / 8;                 // bytes of one key's unit
    static constexpr unsigned K_PAIR = (NT == 32 ? 2u : 4u) * 32u * K_UNIT;  // bytes between step pairs
    static constexpr unsigned V_RUN = 8u * BITS / 4;                   // bytes of one (dim pair, chunk) run
    __device__ __forceinline__ static unsigned k_lane(const Lane<D, NT> &ln) { return (unsigned)ln.koff / 8u * K_UNIT; }
    __device__ __forceinline__ static unsigned v_lane(const Lane<D, NT> &ln) { return (unsigned)ln.voff / 8u * V_RUN; }
};

template <int AUX, int D, int NT, int BITS>
__device__ __forceinline__ void load_k(KTileQ<D, NT, BITS> &t, __amdgpu_buffer_rsrc_t rk, unsigned block_bytes,
                                       const Lane<D, NT> &ln, unsigned void_bytes = 0) {
    typedef QuantOffsets<D, NT, BITS> O;
    const unsigned lane_bytes = O::k_lane(ln) + void_bytes;
    if constexpr (NT == 32) {
#pragma unroll
        for (int p = 0; p < D / 32; ++p) buf_load_words<AUX>(t.f[p], rk, lane_bytes, block_bytes + p * O::K_PAIR);
        buf_load_words<AUX>(t.sb, rk, (unsigned)ln.li * O::GPH * 4 + void_bytes, block_bytes + O::LEVELS);
    } else {
#pragma unroll
        for (int p = 0; p < D / 64; ++p) {
            buf_load_words<AUX>(t.a[p], rk, lane_bytes, block_bytes + p * O::K_PAIR);
            buf_load_words<AUX>(t.b[p], rk, lane_bytes, block_bytes + p * O::K_PAIR + 8 * O::K_UNIT);
        }
        const unsigned ka = ln.li < 8 ? ln.li : ln.li + 8;
        buf_load_words<AUX>(t.sba, rk, ka * O::GPH * 4 + void_bytes, block_bytes + O::LEVELS);
        buf_load_words<AUX>(t.sbb, rk, ka * O::GPH * 4 + void_bytes, block_bytes + O::LEVELS + 8 * O::GPH * 4);
    }
}

template <int AUX, int D, int NT, int BITS>
__device__ __forceinline__ void load_v(VTileQ<D, NT, BITS> &t, __amdgpu_buffer_rsrc_t rv, unsigned block_bytes,
                                       const Lane<D, NT> &ln, unsigned void_bytes = 0) {
    typedef QuantOffsets<D, NT, BITS> O;
    const unsigned lane_bytes = O::v_lane(ln) + void_bytes;  // (row * 4 + chunk) runs
    const unsigned param_lane = (unsigned)ln.g * 16 + void_bytes;
    // Bias rows: lane rows 0 .. GPH-1 carry a group's biases, the others read zeros (void load).
    const unsigned bias_lane = (unsigned)ln.li * 64 + (unsigned)ln.g * 16 + ((unsigned)ln.li < O::GPH ? void_bytes : kVoidLoad);
    if constexpr (NT == 32) {
#pragma unroll
        for (int j = 0; j < D / 64; ++j)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) buf_load_words<AUX>(t.f[j][tt], rv, lane_bytes, block_bytes + (j * 32 * 4 + tt * 2) * O::V_RUN);
#pragma unroll
        for (int grp = 0; grp < (int)O::GPH; ++grp)
#pragma unroll
            for (int tt = 0; tt < 2; ++tt) buf_load_words<AUX>(t.sc[grp][tt], rv, param_lane, block_bytes + O::LEVELS + grp * 64 + tt * 32);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) buf_load_words<AUX>(t.bias[tt], rv, bias_lane, block_bytes + O::LEVELS + O::GPH * 64 + tt * 32);
    } else {
#pragma unroll
        for (int i = 0; i < D / 32; ++i) buf_load_words<AUX>(t.f[i], rv, lane_bytes, block_bytes + i * 16 * 4 * O::V_RUN);
#pragma unroll
        for (int grp = 0; grp < (int)O::GPH; ++grp) buf_load_words<AUX>(t.sc[grp], rv, param_lane, block_bytes + O::LEVELS + grp * 64);
        buf_load_words<AUX>(t.bias, rv, bias_lane, block_bytes + O::LEVELS + O::GPH * 64);
    }
}

// The two phases over quantised tiles also REFILL the tiles for the wave's next block: a
// load's registers are free as soon as its levels have been widened, so the load for the next
// block is issued right there, before the MFMAs that use the widened copies.  Every load thus
// has a whole block of work between issue and use -- a tile that was refilled in one piece
// after the phase had only the other phase (levels are half the bytes of fp16 values, so half
// as much was in flight), and the wave stood waiting for memory twice per block.  `next_bytes` /
// `void_bytes` address the next block as in load_k; the scale/bias words of K are fetched into
// spare registers first and swapped in at the end.
template <int AUX, int D, int NT, int BITS>
__device__ __forceinline__ void block_scores(Scores<D, NT> &sc, KTileQ<D, NT, BITS> &kt, const h8 *qf, const h8 *qlds, int lane,
                                             __amdgpu_buffer_rsrc_t rk, unsigned next_bytes, const Lane<D, NT> &ln,
                                             unsigned void_bytes) {
    typedef QuantOffsets<D, NT, BITS> O;
    constexpr int GPH = D / 64;
    const unsigned lane_bytes = O::k_lane(ln) + void_bytes;
    (void)qf;
    if constexpr (NT == 32) {
        unsigned sb_next[GPH];
        buf_load_words<AUX>(sb_next, rk, (unsigned)ln.li * GPH * 4 + void_bytes, next_bytes + O::LEVELS);
        sc.s = (f16v)0.0f;
        h8 q = qlds[lane];
#pragma unroll
        for (int p = 0; p < D / 32; ++p) {
            const h8 q1 = qlds[(2 * p + 1) * 64 + lane];
            const h8 q_next = qlds[(p + 1 < D / 32 ? 2 * p + 2 : 2 * p) * 64 + lane];  // read ahead of their use
            // widening the second half fills the time the first MFMA runs (they chain on one accumulator)
            const h8 k0 = k_unit_operand<BITS>(kt.f[p], 0, kt.sb[p / 2]);
            sc.s = __builtin_amdgcn_mfma_f32_32x32x16_f16(k0, q, sc.s, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const h8 k1 = k_unit_operand<BITS>(kt.f[p], 1, kt.sb[p / 2]);
            buf_load_words<AUX>(kt.f[p], rk, lane_bytes, next_bytes + p * O::K_PAIR);
            sc.s = __builtin_amdgcn_mfma_f32_32x32x16_f16(k1, q1, sc.s, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            q = q_next;
        }
#pragma unroll
        for (int grp = 0; grp < GPH; ++grp) kt.sb[grp] = sb_next[grp];
    } else {
        unsigned sba_next[GPH], sbb_next[GPH];
        const unsigned ka = ln.li < 8 ? ln.li : ln.li + 8;
        buf_load_words<AUX>(sba_next, rk, ka * GPH * 4 + void_bytes, next_bytes + O::LEVELS);
        buf_load_words<AUX>(sbb_next, rk, ka * GPH * 4 + void_bytes, next_bytes + O::LEVELS + 8 * GPH * 4);
        sc.sa = (f4)0.0f;
        sc.sb = (f4)0.0f;
        h8 q = qlds[lane];
#pragma unroll
        for (int p = 0; p < D / 64; ++p) {
            const h8 q1 = qlds[(2 * p + 1) * 64 + lane];
            const h8 q_next = qlds[(p + 1 < D / 64 ? 2 * p + 2 : 2 * p) * 64 + lane];
            const h8 a0 = k_unit_operand<BITS>(kt.a[p], 0, kt.sba[p]);
            sc.sa = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, q, sc.sa, 0, 0, 0);
            const h8 b0 = k_unit_operand<BITS>(kt.b[p], 0, kt.sbb[p]);
            sc.sb = __builtin_amdgcn_mfma_f32_16x16x32_f16(b0, q, sc.sb, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            const h8 a1 = k_unit_operand<BITS>(kt.a[p], 1, kt.sba[p]);
            buf_load_words<AUX>(kt.a[p], rk, lane_bytes, next_bytes + p * O::K_PAIR);
            sc.sa = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, q1, sc.sa, 0, 0, 0);
            const h8 b1 = k_unit_operand<BITS>(kt.b[p], 1, kt.sbb[p]);
            buf_load_words<AUX>(kt.b[p], rk, lane_bytes, next_bytes + p * O::K_PAIR + 8 * O::K_UNIT);
            sc.sb = __builtin_amdgcn_mfma_f32_16x16x32_f16(b1, q1, sc.sb, 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
            q = q_next;
        }
#pragma unroll
        for (int grp = 0; grp < GPH; ++grp) {
            kt.sba[grp] = sba_next[grp];
            kt.sbb[grp] = sbb_next[grp];
        }
    }
}

__device__ __forceinline__ h8 words_as_h8(const unsigned (&w)[4]) {
    const u4v x = {w[0], w[1], w[2], w[3]};
    return __builtin_bit_cast(h8, x);
}

// `bias_acc` accumulates sum_key bias[group][key] * P[key][row] in its row `group`.
template <int AUX, int D, int NT, int BITS>
__device__ __forceinline__ void block_softmax_pv(RowState<D, NT> &st, Scores<D, NT> &sc, VTileQ<D, NT, BITS> &vt,
                                                 const Lane<D, NT> &ln, int kbase, int lo, int lim, float scale_log2e,
                                                 typename RowState<D, NT>::acc_t &bias_acc, __amdgpu_buffer_rsrc_t rv,
                                                 unsigned next_bytes, unsigned void_bytes, unsigned kept = ~0u,
                                                 const unsigned *row_keep = nullptr, unsigned row_bits = ~0u) {
    typedef QuantOffsets<D, NT, BITS> O;
    constexpr int GPH = D / 64;
    const unsigned lane_bytes = O::v_lane(ln) + void_bytes;
    const unsigned param_lane = (unsigned)ln.g * 16 + void_bytes;
    const unsigned bias_lane = (unsigned)ln.li * 64 + (unsigned)ln.g * 16 + ((unsigned)ln.li < (unsigned)GPH ? void_bytes : kVoidLoad);
    Probs<D, NT> pr;
    block_softmax<D, NT>(st, sc, pr, ln, kbase, lo, lim, scale_log2e, &bias_acc, kept, row_keep, row_bits);
    if constexpr (NT == 32) {
        h8 ps[GPH][2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
            const h8 boosted = pr.pf[t] * (h8)(_Float16)kProbBoost;
#pragma unroll
            for (int grp = 0; grp < GPH; ++grp) {
                ps[grp][t] = boosted * words_as_h8(vt.sc[grp][t]);
                buf_load_words<AUX>(vt.sc[grp][t], rv, param_lane, next_bytes + O::LEVELS + grp * 64 + t * 32);
            }
            bias_acc = __builtin_amdgcn_mfma_f32_32x32x16_f16(words_as_h8(vt.bias[t]), pr.pf[t], bias_acc, 0, 0, 0);
            buf_load_words<AUX>(vt.bias[t], rv, bias_lane, next_bytes + O::LEVELS + GPH * 64 + t * 32);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
            for (int j = 0; j < D / 64; ++j) {  // dim tiles 2 j (dims 64 j + row) and 2 j + 1 (32 above), both of group j
                h8 lo_op, hi_op;
                v_run_operands<BITS>(vt.f[j][t], lo_op, hi_op);
                buf_load_words<AUX>(vt.f[j][t], rv, lane_bytes, next_bytes + (j * 32 * 4 + t * 2) * O::V_RUN);
                st.o[2 * j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(lo_op, ps[j][t], st.o[2 * j], 0, 0, 0);
                st.o[2 * j + 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(hi_op, ps[j][t], st.o[2 * j + 1], 0, 0, 0);
                __builtin_amdgcn_sched_barrier(0);
            }
    } else {
        h8 ps[GPH];
        const h8 boosted = pr.pf * (h8)(_Float16)kProbBoost;
#pragma unroll
        for (int grp = 0; grp < GPH; ++grp) {
            ps[grp] = boosted * words_as_h8(vt.sc[grp]);
            buf_load_words<AUX>(vt.sc[grp], rv, param_lane, next_bytes + O::LEVELS + grp * 64);
        }
        bias_acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(words_as_h8(vt.bias), pr.pf, bias_acc, 0, 0, 0);
        buf_load_words<AUX>(vt.bias, rv, bias_lane, next_bytes + O::LEVELS + GPH * 64);
        __builtin_amdgcn_sched_barrier(0);
        // load i = 2 j + rr covers rows 16 rr + lane row of 64-dim group j: dims 64 j + 16 rr + row
        // (tile 4 j + rr) and 32 above (tile 4 j + 2 + rr)
#pragma unroll
        for (int i = 0; i < D / 32; ++i) {
            const int j = i >> 1, rr = i & 1;
            h8 lo_op, hi_op;
            v_run_operands<BITS>(vt.f[i], lo_op, hi_op);
            buf_load_words<AUX>(vt.f[i], rv, lane_bytes, next_bytes + i * 16 * 4 * O::V_RUN);
            st.o[4 * j + rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(lo_op, ps[j], st.o[4 * j + rr], 0, 0, 0);
            st.o[4 * j + 2 + rr] = __builtin_amdgcn_mfma_f32_16x16x32_f16(hi_op, ps[j], st.o[4 * j + 2 + rr], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

// ---------------------------------------------------------------------------
// Pass 1.  grid = (split, tile, sequence); WAVES wavefronts per workgroup, wave
// w takes key blocks w, w + WAVES, ... of the split (split 0 starts at key 0, or
// at the block of the first key the tile's window reaches).  A block's K and V
// tiles live in registers; the next block's K loads are issued as soon as the
// score MFMAs have consumed the current ones and its V loads right after the P.V
// MFMAs, so a wave always has 16-32 KiB in flight (BITS = 16; the quantised tiles
// are refilled fragment by fragment inside the phases).  The NT = 16 variant fits
// 256 registers, so two workgroups share a CU and their phases overlap.  The
// workgroup merges its waves through LDS and writes one partial, or the final
// rows when the launch has a single split.  BITS: 16, 8 or 4 per cached value.
// ---------------------------------------------------------------------------
// KEEP = 1: a sparse key selection, one byte per key position (0 drops the key), as the reference's decode kernels take it
// (keep[p], sources/TinyTitanCore/Metal/Attention/attention.metal:182-188, :229): a dropped key is as if it were absent.
// KEEP = 2: one such row of bytes per query row, keep[t * stride + key], as its chunk kernels take it
// (sources/TinyTitanCore/Metal/Prefill/prefill.metal:1063-1068, :1129).
// KEEP = 3: the same selection as per-query index lists (keepIdx / keepCount, prefill.metal:1069-1117), served from the
// plan keep_plan_kernel makes of them: per token tile the ascending list of key blocks its tokens keep a key of, and per
// entry and token the kept keys as 32 bits -- the walk costs the selection, never the context.
// The hot arguments and this workgroup's sequence entry, by three scalar loads issued together (the compiler
// would fetch each field where it is first used: five or six dependent trips to the kernarg segment before
// the first K/V load can go out, about 0.15 us each).
typedef int i16v __attribute__((ext_vector_type(16)));
struct HotWords {
    i16v lo, hi;
};
__device__ __forceinline__ void load_hot(SplitKHot &hot, SplitKSeq &sq, int seq) {
    const unsigned long long base = (unsigned long long)__builtin_amdgcn_kernarg_segment_ptr();  // a scalar pair
    const unsigned long long entry = base + (unsigned)seq * (unsigned)sizeof(SplitKSeq);
    HotWords w;
    i4 e;
    asm volatile("s_load_dwordx16 %0, %3, 0x0\n\ts_load_dwordx16 %1, %3, 0x40\n\ts_load_dwordx4 %2, %4, 0x80\n\ts_waitcnt lgkmcnt(0)"
                 : "=&s"(w.lo), "=&s"(w.hi), "=&s"(e)
                 : "s"(base), "s"(entry)
                 : "memory");
    hot = __builtin_bit_cast(SplitKHot, w);
    sq = __builtin_bit_cast(SplitKSeq, e);
}
static_assert(offsetof(SplitKArgs, hot) == 0 && offsetof(SplitKArgs, seq) == 0x80, "load_hot's offsets");

// STREAM: the launch reads every K/V byte once (see kStreamed).
// A row's 32 selection bytes of one key block, as 8 words in two loads (the row stride is a multiple of 4 bytes, which is
// all a buffer load of four dwords asks for; dwords past the buffer's range read as zero one by one).
__device__ __forceinline__ void load_row_words(unsigned (&dst)[8], __amdgpu_buffer_rsrc_t rsrc, unsigned bytes) {
    const u4v lo = __builtin_bit_cast(u4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, bytes, 0, 0));
    const u4v hi = __builtin_bit_cast(u4v, __builtin_amdgcn_raw_buffer_load_b128(rsrc, bytes + 16u, 0, 0));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        dst[i] = lo[i];
        dst[4 + i] = hi[i];
    }
}

template <int D, int NT, int WAVES, int BITS, int KEEP = 0, int STREAM = 0>
__global__ __launch_bounds__(WAVES * 64, (NT == 16 && KEEP < 2 ? 2 : 1)) void attn_splitk_kernel(const SplitKArgs args) {
    constexpr int AUX = STREAM ? kStreamed : 0;
    extern __shared__ float lds[];
    constexpr int ROW = D + kLdsPad;  // staged O row stride in floats
    constexpr int REGION = NT * ROW + NT * 2;
    constexpr int KS = (NT == 32) ? D / 16 : D / 32;
    constexpr unsigned BLK_BYTES = BITS == 16 ? 32 * D * 2 : 32 * D * BITS / 8 + 32 * (D / 64) * 4;  // bytes per block
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // scalar: block pointers stay in SGPRs
    const Lane<D, NT> ln(lane);
    const int li = ln.li, g = ln.g;
    const int seq = blockIdx.z;
    SplitKHot a;
    SplitKSeq sq;
    load_hot(a, sq, seq);
    int split = blockIdx.x, tile = blockIdx.y;
    if (a.flags & kHotXcdGrid) {  // many token tiles: the (split, tile) pairs are dealt out XCD by XCD, tile fastest
        const unsigned pairs = (unsigned)a.n_tiles * (unsigned)a.n_splits_max, per_xcd = (pairs + 7u) >> 3;
        const unsigned pair = (blockIdx.x & 7u) * per_xcd + (blockIdx.x >> 3);
        if (pair >= pairs) return;  // the grid is rounded up to a multiple of eight
        split = (int)(pair / (unsigned)a.n_tiles);
        tile = (int)(pair - (unsigned)split * (unsigned)a.n_tiles);
    }
    const TileInfo ti = tile_info(a, sq, tile);
    const int k_begin = ti.k0 + split * a.split_len;
    if (k_begin >= ti.tile_end && split != 0) return;  // split 0 always runs so that an empty range yields zeros
    const int k_end = min(k_begin + a.split_len, ti.tile_end);
    const int b_end = (k_end + 31) >> 5;

    const size_t page = ((size_t)sq.slot * a.n_kv_heads + ti.kvh) * (size_t)a.page_elems;
    const __amdgpu_buffer_rsrc_t rk = make_rsrc(a.k_layer + page, (unsigned)(a.page_elems * 2));
    const __amdgpu_buffer_rsrc_t rv = make_rsrc(a.v_layer + page, (unsigned)(a.page_elems * 2));

    // This lane's query row.
    const int t_local = (li * a.gh_inv) >> 16;  // li / gh
    const int hg = li - t_local * a.gh;
    const bool valid = t_local < ti.tile_rows;
    const int tok = ti.t0 + (valid ? t_local : 0);  // clamped so that the address is always in range
    const int head = ti.kvh * a.group + ti.hsub * a.gh + hg;
    const int lim = valid ? min(ti.total, ti.start + tok + 1) : 0;  // keys [lo, lim) are visible
    const int lo = (a.window > 0 && lim > a.window) ? lim - a.window : 0;  // sliding window: the last `window` keys
    const global_halves qp = (global_halves)(a.q + seq * a.q_seq_stride + tok * a.q_tok_stride + (long long)head * D);

    // Order of the first requests.  A wave's vector loads are issued in program order and an issue stalls while
    // the CU's memory pipeline is full, which it is as soon as every wave of the chip has asked for its first
    // block: a load behind 32 KiB of K/V requests only goes out when most of that data has arrived, microseconds
    // later.  So the query is requested first, then K of the first block; the wave then takes the query (short
    // wait: it was first in line), and V of the first block follows while the first scores are worked out.
    // The NT = 16 variant and every quantised variant keep the query fragments in LDS (the quantised 32-row
    // variant would otherwise need more than 512 registers), each wave its OWN copy, in the region it stages its
    // accumulators in at the end: no wave waits for another before its first block.  The fp16 32-row variant
    // keeps them in registers.
    constexpr bool Q_IN_LDS = NT == 16 || BITS != 16;
    constexpr int QSTEP = NT == 32 ? 16 : 32;  // dims per contraction step
    h8 qf[KS];
    h8 *qlds = reinterpret_cast<h8 *>(lds + wave * REGION);  // [step][lane] h8: KS KiB of the wave's REGION
    static_assert(!Q_IN_LDS || KS * 1024 <= REGION * 4, "the wave's query copy fits its merge region");
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        // quantised tiles contract the dims in their own order (two steps per loaded unit)
        const h8 x = load_h8(qp + (BITS == 16 ? QSTEP * s + 8 * g : q_dim_of_step<NT>(s, g)));
        qf[s] = x;
    }
    // Unconditional (straight-line code keeps the compiler's count of outstanding loads exact): a
    // wave whose first block lies past the split's end issues void loads.
    int b = (k_begin >> 5) + wave;
    typename std::conditional<BITS == 16, KTile<D, NT>, KTileQ<D, NT, BITS>>::type kt;
    typename std::conditional<BITS == 16, VTile<D, NT>, VTileQ<D, NT, BITS>>::type vt;
    // Selection bytes: lane i (and i + 32) holds the byte of key 32 b + i of the block in hand; the next block's
    // are loaded a block ahead.  Past the sequence's end the buffer load returns 0 (those keys are not visible anyway).
    // A block without a kept key is not read: its loads are void (no memory traffic), its turn works on zeros that
    // the selection masks anyway, so the HBM bytes of a selection are the blocks it touches, not the context.
    // (Skipping the turn's arithmetic too, with a branch around it, made the kernel slower: the compiler then
    // waits for every load in flight at the join.)  The first block of a wavefront is read before its bytes
    // are known -- waiting for them would put a round trip in front of it.
    // Where the mask starts on a word boundary the wavefront also learns up front which of its blocks hold a kept
    // key at all -- lane j reads the 32 bytes of its j-th block, one ballot makes a 64-bit word of them (the host
    // keeps a split to 64 blocks per wavefront) -- and then walks only those: their arithmetic goes as well.
    __amdgpu_buffer_rsrc_t rkeep;
    unsigned keep_cur = 1, keep_next = 1, keep_after = 1;
    const int b_first = b;
    unsigned long long todo = 0;  // bit j: block b_first + j * WAVES is still to be worked on
    unsigned block_words = 0;
    if constexpr (KEEP == 1) {
        rkeep = make_rsrc(args.keep + seq * args.keep_seq_stride, (unsigned)ti.total);
        keep_cur = __builtin_amdgcn_raw_buffer_load_b8(rkeep, (unsigned)b * 32u + (unsigned)(lane & 31), 0, 0);
        if (a.keep_words) {
#pragma unroll
            for (int i = 0; i < 8; ++i)
                block_words |= __builtin_amdgcn_raw_buffer_load_b32(rkeep, (unsigned)(b_first + lane * WAVES) * 32u + 4u * i, 0, 0);
        } else {
            // block by block: the next block is the wavefront's second, and its bytes are asked for ahead of the
            // first block's data
            keep_next = __builtin_amdgcn_raw_buffer_load_b8(rkeep, (unsigned)(b + WAVES) * 32u + (unsigned)(lane & 31), 0, 0);
        }
    }
    // Per-query selections: the lane's own row of bytes, 32 per block as 8 words, a block ahead.  The range of the
    // buffer is the rows' extent, so a read past it (void blocks, rows of padding lanes) returns 0.
    // Here too a block that no row of the tile keeps a key of is not read: the words of the next two blocks are in hand.
    unsigned row_cur[8], row_next[8], row_after[8];
    unsigned row_bytes0 = 0;
    unsigned window_words[kKeepWindows] = {};
    int *const listed = reinterpret_cast<int *>(lds + WAVES * REGION);  // the workgroup's touched blocks, then [wave][window] counts
    int n_listed = 0, list_at = 0, nxt = 0, aft = 0;
    auto listed_block = [&](int i) { return i < n_listed ? __builtin_amdgcn_readfirstlane(listed[i]) : b_end; };
    if constexpr (KEEP == 2) {
        rkeep = make_rsrc(args.keep + seq * args.keep_seq_stride, (unsigned)((long long)a.rows * args.keep_row_stride));
        row_bytes0 = (unsigned)((long long)tok * args.keep_row_stride);
        load_row_words(row_cur, rkeep, row_bytes0 + (unsigned)b * 32u);
        if (a.keep_words) {
            // Long splits: which of the split's blocks does ANY row of the tile keep a key of?  Wavefront w looks at
            // the split's blocks [512 w, 512 w + 512) -- lane j at blocks j, j + 64, ... of them, consecutive lanes
            // at consecutive 32 bytes, so that a load instruction reads a contiguous 2 KiB -- in every token's row of
            // bytes (a tile's rows are its tokens times the heads that share them); the touched blocks go into a
            // list in LDS and the loop walks only those, arithmetic included, so a sparse chunk costs its selection
            // and not its context -- and a split can be as long as kKeepWindows * 64 blocks a wavefront: few
            // workgroups, each with one prologue, one merge and one partial.
            // Two rows at a time, straight-line: their 4 kKeepWindows loads are all in flight together (a loop over
            // single rows waits for each row's loads before it asks for the next: ~3 us a row); a tile's odd last
            // row is paired with void loads.
            for (int r = 0; r < ti.tile_rows; r += 2) {
                u4v got[2][kKeepWindows][2];
#pragma unroll
                for (int rr = 0; rr < 2; ++rr) {
                    const unsigned row = r + rr < ti.tile_rows ? (unsigned)((long long)(ti.t0 + r + rr) * args.keep_row_stride) : kVoidLoad;
#pragma unroll
                    for (int w = 0; w < kKeepWindows; ++w) {
                        const unsigned at = row + (unsigned)((k_begin >> 5) + (wave * kKeepWindows + w) * 64 + lane) * 32u;
                        got[rr][w][0] = __builtin_bit_cast(u4v, __builtin_amdgcn_raw_buffer_load_b128(rkeep, at, 0, 0));
                        got[rr][w][1] = __builtin_bit_cast(u4v, __builtin_amdgcn_raw_buffer_load_b128(rkeep, at + 16u, 0, 0));
                    }
                }
#pragma unroll
                for (int w = 0; w < kKeepWindows; ++w) {
                    const u4v any = got[0][w][0] | got[0][w][1] | got[1][w][0] | got[1][w][1];
                    window_words[w] |= any[0] | any[1] | any[2] | any[3];
                }
            }
        } else {
            load_row_words(row_next, rkeep, row_bytes0 + (unsigned)(b + WAVES) * 32u);
        }
    }
    // Index lists: this wavefront takes entries e_at, e_at + WAVES, ... of the tile's list up to the split's end.  The block
    // of the entry after next and the row's bits of the next two entries are always on their way.
    const int *plan_blocks_tile = nullptr;
    const unsigned *plan_bits_tile = nullptr;
    int e_at = 0, e_hi = 0, walked = 0, after_block = 0;
    unsigned bits_cur = ~0u, bits_next = ~0u, bits_after = ~0u;
    const int bits_col = valid ? t_local : 0;
    auto plan_block = [&](int k) {  // block of the wavefront's k-th entry (a load; every lane the same word)
        const int e = e_at + k * WAVES;
        const int got = plan_blocks_tile[e < e_hi ? e : 0];
        return e < e_hi ? got : b_end;
    };
    auto plan_row_bits = [&](int k) {
        const int e = e_at + k * WAVES;
        const unsigned got = plan_bits_tile[(size_t)(e < e_hi ? e : 0) * a.tt + bits_col];
        return e < e_hi ? got : 0u;
    };
    if constexpr (KEEP == 3) {
        const int *ranges = args.plan_ranges + (size_t)ti.tok_tile * (a.n_splits_max + 1) + split;
        e_at = __builtin_amdgcn_readfirstlane(ranges[0]) + wave;
        e_hi = __builtin_amdgcn_readfirstlane(ranges[1]);
        plan_blocks_tile = args.plan_blocks + (size_t)ti.tok_tile * args.plan_cap;
        plan_bits_tile = args.plan_bits + (size_t)ti.tok_tile * args.plan_cap * a.tt;
        const int b0 = plan_block(0), b1 = plan_block(1);
        after_block = plan_block(2);
        bits_cur = plan_row_bits(0);
        bits_next = plan_row_bits(1);
        b = __builtin_amdgcn_readfirstlane(b0);
        nxt = __builtin_amdgcn_readfirstlane(b1);
    }
    const bool first_real = b < b_end;
    const unsigned first_bytes = first_real ? (unsigned)(a.ring_blocks ? b % a.ring_blocks : b) * BLK_BYTES : 0u;
    const unsigned first_void = first_real ? 0u : kVoidLoad;
    load_k<AUX>(kt, rk, first_bytes, ln, first_void);
    __builtin_amdgcn_sched_barrier(0);  // the first block's K loads are issued HERE, before the query is waited for
    if constexpr (KEEP == 1) {
        const int mine = b_first < b_end ? (b_end - b_first + WAVES - 1) / WAVES : 0;  // this wavefront's blocks, at most 64
        todo = mine >= 64 ? ~0ull : ((1ull << mine) - 1ull);
        if (a.keep_words) {
            unsigned long long touched = __ballot(block_words != 0);
            // A mask is exactly `total` bytes: when that is not a multiple of 4 its last word straddles the end of
            // the buffer's range and may read as zero whatever its bytes hold.  The block of the last key is
            // therefore always walked; its keys are still tested byte by byte.
            if (ti.total & 3) {
                const int last_block = (ti.total - 1) >> 5, j = (last_block - b_first) / WAVES;
                if (last_block >= b_first && (last_block - b_first) % WAVES == 0 && j < 64) touched |= 1ull << j;
            }
            todo &= touched;
        }
        todo &= ~1ull;  // the first block is in hand
        if (a.keep_words) {
            const int nb0 = todo ? b_first + (__ffsll((long long)todo) - 1) * WAVES : b_end;
            keep_next = __builtin_amdgcn_raw_buffer_load_b8(rkeep, (unsigned)nb0 * 32u + (unsigned)(lane & 31), 0, 0);
        }
    }
    if constexpr (KEEP == 2) {
        if (a.keep_words) {
            // One list for the workgroup, its entries dealt out to the wavefronts in turn: every wavefront then walks
            // a quarter of the split's touched blocks, however they fall among the blocks each one looked at.
            // (the split has at most WAVES * kKeepWindows * 64 blocks: the host sees to it)
            int *const counts = listed + WAVES * kKeepWindows * 64;  // [wave][window]
            unsigned long long words[kKeepWindows];
#pragma unroll
            for (int w = 0; w < kKeepWindows; ++w) {
                const int j = (wave * kKeepWindows + w) * 64 + lane;  // the block's place in the split
                // (the wavefronts' first blocks -- the split's first WAVES -- are in hand)
                words[w] = __ballot(window_words[w] != 0 && (k_begin >> 5) + j < b_end && j >= WAVES);
                if (lane == 0) counts[wave * kKeepWindows + w] = __popcll(words[w]);
            }
            __syncthreads();
            int at = 0;
#pragma unroll
            for (int v = 0; v < WAVES; ++v)  // entries in (wave, window, lane) order: ascending blocks
#pragma unroll
                for (int w = 0; w < kKeepWindows; ++w) {
                    if (v == wave && w == 0) at = n_listed;
                    n_listed += counts[v * kKeepWindows + w];
                }
#pragma unroll
            for (int w = 0; w < kKeepWindows; ++w) {
                if ((words[w] >> lane) & 1ull)
                    listed[at + (int)__builtin_amdgcn_mbcnt_hi((unsigned)(words[w] >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)words[w], 0u))] =
                        (k_begin >> 5) + (wave * kKeepWindows + w) * 64 + lane;
                at += __popcll(words[w]);
            }
            __syncthreads();
            nxt = listed_block(wave);
            aft = listed_block(wave + WAVES);
            load_row_words(row_next, rkeep, row_bytes0 + (unsigned)nxt * 32u);
        }
    }
#pragma unroll
    for (int s = 0; s < KS; ++s) {
        qf[s] = valid ? qf[s] : (h8)(_Float16)0;
        if constexpr (Q_IN_LDS) qlds[s * 64 + lane] = qf[s];  // read back by this wave only: no barrier
    }
    __builtin_amdgcn_sched_barrier(0);
    load_v<AUX>(vt, rv, first_bytes, ln, first_void);
    __builtin_amdgcn_sched_barrier(0);

    RowState<D, NT> st;
    st.init();
    typename RowState<D, NT>::acc_t bias_acc = (typename RowState<D, NT>::acc_t)0.0f;  // quantised pages only
    // The next block's loads are issued UNCONDITIONALLY (void loads past the split's end).  A branch
    // around them would leave the compiler unable to count the loads in flight, and it would then
    // make the P.V step wait for the next block's K tile as well as for its own V tile.
    while (b < b_end) {
        Scores<D, NT> sc;
        int nb = b + WAVES;
        unsigned kept = ~0u;
        bool next_kept = true;
        const unsigned *row_keep = nullptr;
        if constexpr (KEEP == 1) {
            // the next block and the one after it, off the word of blocks still to do
            nb = todo ? b_first + (__ffsll((long long)todo) - 1) * WAVES : b_end;
            todo &= todo - 1;
            const int after = todo ? b_first + (__ffsll((long long)todo) - 1) * WAVES : b_end;
            keep_after = __builtin_amdgcn_raw_buffer_load_b8(rkeep, (unsigned)after * 32u + (unsigned)(lane & 31), 0, 0);
            kept = (unsigned)__ballot(keep_cur != 0);  // lanes 32..63 repeat lanes 0..31
            next_kept = __ballot(keep_next != 0) != 0ull;
        }
        if constexpr (KEEP == 2) {
            if (a.keep_words) {
                // the next touched block and the one after it, off the list (the one after that is read here, a turn ahead)
                nb = nxt;
                nxt = aft;
                aft = listed_block(wave + (list_at + 2) * WAVES);
                ++list_at;
                load_row_words(row_after, rkeep, row_bytes0 + (unsigned)nxt * 32u);
            } else {
                unsigned any = 0;
                load_row_words(row_after, rkeep, row_bytes0 + (unsigned)(nb + WAVES) * 32u);
#pragma unroll
                for (int i = 0; i < 8; ++i) any |= row_next[i];
                next_kept = __ballot(any != 0) != 0ull;
            }
            row_keep = row_cur;
        }
        unsigned row_bits = ~0u;
        if constexpr (KEEP == 3) {
            nb = nxt;
            nxt = __builtin_amdgcn_readfirstlane(after_block);
            after_block = plan_block(walked + 3);
            bits_after = plan_row_bits(walked + 2);
            ++walked;
            row_bits = bits_cur;
        }
        const bool real = nb < b_end && next_kept;
        const unsigned next = real ? (unsigned)(a.ring_blocks ? nb % a.ring_blocks : nb) * BLK_BYTES : 0u;
        const unsigned void_bytes = real ? 0u : kVoidLoad;
        if constexpr (BITS == 16 && NT == 32) {
            block_scores_refill<AUX, D>(sc, kt, qf, rk, next, ln, void_bytes);
            block_softmax_pv_refill<AUX, D>(st, sc, vt, ln, b << 5, lo, lim, a.scale_log2e, rv, next, void_bytes, kept, row_keep, row_bits);
        } else if constexpr (BITS == 16) {
            block_scores(sc, kt, qf, qlds, lane);
            load_k<AUX>(kt, rk, next, ln, void_bytes);
            block_softmax_pv<D, NT>(st, sc, vt, ln, b << 5, lo, lim, a.scale_log2e, kept, row_keep, row_bits);
            load_v<AUX>(vt, rv, next, ln, void_bytes);
        } else {  // the phases refill their tiles as they go
            block_scores<AUX, D, NT, BITS>(sc, kt, qf, qlds, lane, rk, next, ln, void_bytes);
            block_softmax_pv<AUX, D, NT, BITS>(st, sc, vt, ln, b << 5, lo, lim, a.scale_log2e, bias_acc, rv, next, void_bytes, kept,
                                          row_keep, row_bits);
        }
        if constexpr (KEEP == 1) {
            keep_cur = keep_next;
            keep_next = keep_after;
        }
        if constexpr (KEEP == 2) {
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                row_cur[i] = row_next[i];
                row_next[i] = row_after[i];
            }
        }
        if constexpr (KEEP == 3) {
            bits_cur = bits_next;
            bits_next = bits_after;
        }
        b = nb;
    }
    if constexpr (BITS != 16) {
        // Level accumulators carry the probability boost; the bias sums sit in row `group` of
        // bias_acc, i.e. in register `group` of the lane group 0 lane that owns this lane's query row.
        constexpr int TILES_PER_GROUP = RowState<D, NT>::MT / (D / 64);
#pragma unroll
        for (int grp = 0; grp < D / 64; ++grp) {
            const float group_bias = __shfl(bias_acc[grp], li);
#pragma unroll
            for (int mt = grp * TILES_PER_GROUP; mt < (grp + 1) * TILES_PER_GROUP; ++mt)
                st.o[mt] = st.o[mt] * (1.0f / kProbBoost) + group_bias;
        }
    }

    // Stage this wave's state in LDS.
    float l = st.l;
    l = (NT == 32) ? sum_across_halves(l) : sum_across_quarters(l);
    float *region = lds + wave * REGION;
    if (!valid) {
        // padding row: nothing to merge
    } else if constexpr (NT == 32) {
#pragma unroll
        for (int mt = 0; mt < D / 32; ++mt)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                f4 x = {st.o[mt][4 * vq], st.o[mt][4 * vq + 1], st.o[mt][4 * vq + 2], st.o[mt][4 * vq + 3]};
                *reinterpret_cast<f4 *>(region + li * ROW + 32 * mt + 8 * vq + 4 * g) = x;
            }
    } else {
#pragma unroll
        for (int mt = 0; mt < D / 16; ++mt) *reinterpret_cast<f4 *>(region + li * ROW + 16 * mt + 4 * g) = st.o[mt];
    }
    if (g == 0 && valid) {
        region[NT * ROW + 2 * li] = st.m;
        region[NT * ROW + 2 * li + 1] = l;
    }
    __syncthreads();

    // Merge the waves' states; every thread takes (row, 4 dims) items.
    const int n_valid = ti.tile_rows * a.gh;
    constexpr int D4 = D / 4;
    const size_t pbase = (((size_t)sq.first_split + split) * a.n_tiles + tile) * NT;
    for (int item = threadIdx.x; item < n_valid * D4; item += WAVES * 64) {
        const int n = item / D4;
        const int d = (item - n * D4) * 4;
        float mw[WAVES];
        float ms = kNegBig;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            mw[w] = lds[w * REGION + NT * ROW + 2 * n];
            ms = fmaxf(ms, mw[w]);
        }
        f4 acc = (f4)0.0f;
        float lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < WAVES; ++w) {
            const float f = fast_exp2(mw[w] - ms);
            lsum += f * lds[w * REGION + NT * ROW + 2 * n + 1];
            acc += f * *reinterpret_cast<const f4 *>(lds + w * REGION + n * ROW + d);
        }
        if (a.n_splits_max == 1) {
            const int tl = n / a.gh;
            const int hh = ti.kvh * a.group + ti.hsub * a.gh + (n - tl * a.gh);
            store_out4(args, seq, ti.t0 + tl, hh, d, D, acc, lsum > 0.0f ? 1.0f / lsum : 0.0f, (a.flags & kHotAligned) != 0);
        } else {
            *reinterpret_cast<f4 *>(a.part_o + (pbase + n) * D + d) = acc;
            if (d == 0) {
                a.part_ml[(pbase + n) * 2] = ms;
                a.part_ml[(pbase + n) * 2 + 1] = lsum;
            }
        }
    }
}

// ---------------------------------------------------------------------------
// Pass 2: cross-split log-sum-exp combine, gate and fp16 store.
// grid = (row within tile * D/64 + dim chunk, tile, sequence), 256 threads.
// Every wave first finds the row's global max over all splits (a few scalars
// per lane), which makes the per-split terms independent: a thread owns 4
// output dims (lane % 16) of the workgroup's 64-dim chunk and the splits
// 4 * wave + lane / 16, + 16, ..., all loads in flight at once; the 16 split
// groups add up through two shuffles and LDS.  All-empty input yields zeros
// (sources/TinyTitanCore/Metal/Attention/attention.metal:418-427).
// ---------------------------------------------------------------------------
template <int D, int NT>
__global__ __launch_bounds__(256) void attn_combine_kernel(const SplitKArgs args) {
    constexpr int DCH = D / 64;
    __shared__ float sm[4][68];
    const int n = blockIdx.x / DCH, dchunk = blockIdx.x - n * DCH;
    const int tile = blockIdx.y, seq = blockIdx.z;
    SplitKHot a;
    SplitKSeq sq;
    load_hot(a, sq, seq);
    const TileInfo ti = tile_info(a, sq, tile);
    if (n >= ti.tile_rows * a.gh) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int n_splits = (ti.tile_end - ti.k0 + a.split_len - 1) / a.split_len;
    if (n_splits < 1) n_splits = 1;
    // partial rows of split s: ((first_split + s) * n_tiles + tile) * NT + n
    const size_t tfirst = (size_t)sq.first_split;
    const size_t tstride = (size_t)a.n_tiles * NT;
    const size_t toff = (size_t)tile * NT + n;
    const int d = dchunk * 64 + (lane & 15) * 4;
    // the gate's values of the item this thread stores at the end (threads 0-15), first of all requests
    const int tl = n / a.gh;
    const int hh = ti.kvh * a.group + ti.hsub * a.gh + (n - tl * a.gh);
    const bool aligned = (a.flags & kHotAligned) != 0;
    float gate4[4] = {0.0f, 0.0f, 0.0f, 0.0f};
    if (threadIdx.x < 16) load_gate4(args, seq, ti.t0 + tl, hh, d, D, aligned, gate4);
    // This thread's first kBatch splits are requested BEFORE the global max is known: their
    // addresses do not depend on it, so the max's loads and these share one trip to memory.
    constexpr int kBatch = 8;
    const int s0 = wave * 4 + (lane >> 4);
    f4 po[kBatch];
    float pm[kBatch], pl[kBatch];
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        const int s = s0 + 16 * i;
        const size_t row = (tfirst + (s < n_splits ? s : 0)) * tstride + toff;
        pm[i] = s < n_splits ? a.part_ml[row * 2] : kNegBig;
        pl[i] = a.part_ml[row * 2 + 1];
        po[i] = *reinterpret_cast<const f4 *>(a.part_o + row * D + d);
    }
    float mg = kNegBig;
    for (int s = lane; s < n_splits; s += 64) mg = fmaxf(mg, a.part_ml[((tfirst + s) * tstride + toff) * 2]);
    mg = wave_max_f32(mg, lane);
    f4 acc = (f4)0.0f;
    float l = 0.0f;
#pragma unroll
    for (int i = 0; i < kBatch; ++i) {
        const float f = s0 + 16 * i < n_splits ? fast_exp2(pm[i] - mg) : 0.0f;
        l += f * pl[i];
        acc += f * po[i];
    }
#pragma unroll 4
    for (int s = s0 + 16 * kBatch; s < n_splits; s += 16) {
        const size_t row = (tfirst + s) * tstride + toff;
        const float f = fast_exp2(a.part_ml[row * 2] - mg);
        l += f * a.part_ml[row * 2 + 1];
        acc += f * *reinterpret_cast<const f4 *>(a.part_o + row * D + d);
    }
    // (lanes l, l ^ 16, l ^ 32, l ^ 48, added in that order: v_permlane16_swap / v_permlane32_swap, no trip through LDS)
    l = sum_across_quarters(l);
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] = sum_across_quarters(acc[i]);
    if (lane < 16) *reinterpret_cast<f4 *>(&sm[wave][lane * 4]) = acc;
    if (lane == 0) sm[wave][64] = l;
    __syncthreads();
    if (threadIdx.x < 16) {
        f4 o = (f4)0.0f;
        float lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            lsum += sm[w][64];
            o += *reinterpret_cast<const f4 *>(&sm[w][lane * 4]);
        }
        store_out4_gated(args, seq, ti.t0 + tl, hh, d, D, o, lsum > 0.0f ? 1.0f / lsum : 0.0f, aligned, gate4);
    }
}

// Pass 2 for launches of many tiles with few splits each (a chunk through the split-K tiles, or through the chunk
// kernel over key ranges): one workgroup per four rows of a tile instead of one per (row, 64 dims) -- the many tiny
// workgroups of attn_combine_kernel cost more to dispatch than these take to run.  A thread owns one (row, 4 dims)
// item and all of its splits, kCombineRowsSplits at a time: their loads are requested together, so a thread makes
// one trip to memory per turn, not one per split (the host sends more than two turns' worth to the other kernel).
// grid = (NT / 4, tile, sequence), 256 threads.
constexpr int kCombineRowsSplits = 16;

template <int D, int NT>
__global__ __launch_bounds__(256) void attn_combine_rows_kernel(const SplitKArgs args) {
    constexpr int D4 = D / 4, ROWS = 4;
    const int tile = blockIdx.y, seq = blockIdx.z;
    SplitKHot a;
    SplitKSeq sq;
    load_hot(a, sq, seq);
    const TileInfo ti = tile_info(a, sq, tile);
    int n_splits = (ti.tile_end - ti.k0 + a.split_len - 1) / a.split_len;
    if (n_splits < 1) n_splits = 1;
    const size_t tfirst = (size_t)sq.first_split, tstride = (size_t)a.n_tiles * NT;
    const int n_valid = ti.tile_rows * a.gh;
    for (int item = threadIdx.x; item < ROWS * D4; item += 256) {
        const int n = blockIdx.x * ROWS + item / D4, d = (item % D4) * 4;
        if (n >= n_valid) break;
        const size_t toff = (size_t)tile * NT + n;
        float mg = kNegBig, l = 0.0f;
        f4 acc = (f4)0.0f;
        for (int first = 0; first < n_splits; first += kCombineRowsSplits) {  // (one turn up to kCombineRowsSplits splits)
            float pm[kCombineRowsSplits], pl[kCombineRowsSplits];
            f4 po[kCombineRowsSplits];
#pragma unroll
            for (int i = 0; i < kCombineRowsSplits; ++i) {
                const int s = first + i;
                const size_t row = (tfirst + (s < n_splits ? s : 0)) * tstride + toff;
                pm[i] = s < n_splits ? a.part_ml[row * 2] : kNegBig;
                pl[i] = a.part_ml[row * 2 + 1];
                po[i] = *reinterpret_cast<const f4 *>(a.part_o + row * D + d);
            }
            float m_new = mg;
#pragma unroll
            for (int i = 0; i < kCombineRowsSplits; ++i) m_new = fmaxf(m_new, pm[i]);
            const float keep = fast_exp2(mg - m_new);  // (first turn: what is kept is zero anyway)
            l *= keep;
            acc *= keep;
            mg = m_new;
#pragma unroll
            for (int i = 0; i < kCombineRowsSplits; ++i) {
                const float f = first + i < n_splits ? fast_exp2(pm[i] - mg) : 0.0f;
                l += f * pl[i];
                acc += f * po[i];
            }
        }
        const int tl = n / a.gh;
        const int hh = ti.kvh * a.group + ti.hsub * a.gh + (n - tl * a.gh);
        store_out4(args, seq, ti.t0 + tl, hh, d, D, acc, l > 0.0f ? 1.0f / l : 0.0f, (a.flags & kHotAligned) != 0);
    }
}

// ---------------------------------------------------------------------------
// Host side: planning and launch.
// ---------------------------------------------------------------------------

// Behind the merge regions: the lists of touched blocks of a per-query selection, one per wave.
static constexpr size_t keep_list_bytes(int keep, int waves) { return keep == 2 ? (size_t)waves * kKeepWindows * (64 + 1) * sizeof(int) : 0; }

static size_t lds_bytes_for(int D, int NT, int waves) {
    // one merge region per wave; a wave's copy of the query fragments lives in its own region until then
    return (size_t)waves * ((size_t)NT * (D + kLdsPad) + (size_t)NT * 2) * sizeof(float);
}

int plan_launch(const tt_hip_ctx *ctx, int kind, int n_seq, int n_q_heads, int n_kv_heads, int head_dim, int rows,
                long long total_keys, int min_keys, int max_keys, LaunchPlan *plan, int kv_bits, bool small_tiles_ok) {
    if (n_kv_heads <= 0 || n_q_heads <= 0 || n_q_heads % n_kv_heads != 0) return TT_HIP_ERR_SHAPE;
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return TT_HIP_ERR_SHAPE;
    if (rows <= 0 || n_seq <= 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    const int group = n_q_heads / n_kv_heads;
    LaunchPlan p{};
    if (kind == 1) {  // prefill: 32 tokens of one q head per tile
        p.nt = 32;
        p.gh = 1;
    } else {
        // GQA-packed rows: all q heads of a KV head (times the tile's tokens) share one pass over K/V.
        p.gh = group;
        while (p.gh > 32 || group % p.gh != 0) --p.gh;  // largest divisor of group that fits a tile
        p.nt = (rows * p.gh <= 16) ? 16 : 32;
        // Tiles of 16 rows although the rows would fill tiles of 32, while the launch reads little: the 32-row
        // kernel's fixed costs (one workgroup per CU, 32 rows x D floats per wavefront merged through LDS and left as
        // the partial result) then outweigh reading the cache once per tile of 16.  "Little" is counted in keys walked
        // by tiles of 16 over the whole launch, keys x tiles of 16 x KV heads (figures for 2 KV heads of 256, fp16):
        //  * A few verify rows (up to four tiles of 16 per KV head, whose reads all come from HBM): 4 rows at 8k keys
        //    17.8 -> 13.1 us, at 2k keys 14.4 -> 10.9, 4 sequences x 4 rows at 4k keys 22.6 -> 16.2, 8 rows at 8k keys
        //    18.3 -> 15.1; at 64k keys 36.3 against 37.2 the other way.  Over quantised pages the 32-row tile is dearer
        //    still (4 rows at 64k keys over 8 bits 29.2 -> 25.0 us).
        //  * A short chunk behind a short context (more tiles, which re-read the same keys from L2), as long as the
        //    tiles are one round of workgroups: 32 rows from position 0 11.0 -> 6.5 us, 128 rows behind 1024 keys
        //    20.9 -> 17.6, 256 rows behind 1024 keys 26.0 -> 20.7; 128 rows behind 3072 keys 28.2 against 29.6 and 512
        //    rows from position 0 17.0 against 19.7 the other way.
        // With 8 KV heads of 128 the same counts hold per KV head four times earlier (4 sequences x 16 rows at 4k keys:
        // 24.4 us in tiles of 32, 30.0 in tiles of 16; 8 rows at 8k keys 16.7 against 13.4), with 4 of 64 twice.
        if (small_tiles_ok && p.nt == 32 && p.gh <= 16) {
            const long long tiles16 = (rows + 16 / p.gh - 1) / (16 / p.gh);
            const long long launch_tiles16 = tiles16 * n_kv_heads * (group / p.gh);  // per sequence
            long long limit;  // of keys x tiles of 16 over the launch (the rows' own keys included)
            if (tiles16 <= 4) limit = kv_bits == 16 ? 144 * 1024 : 288 * 1024;
            else if (launch_tiles16 * n_seq <= ctx->n_cus) limit = kv_bits == 16 ? 320 * 1024 : 384 * 1024;
            else limit = 0;
            if (total_keys * launch_tiles16 <= limit) p.nt = 16;
        }
    }
    p.tt = p.nt / p.gh;
    p.hsubs = group / p.gh;
    p.tok_tiles = (rows + p.tt - 1) / p.tt;
    p.n_tiles = n_kv_heads * p.hsubs * p.tok_tiles;
    p.waves = 4;
    const int min_split = 32 * p.waves;  // one key block per wave
    // Workgroup slots of the chip: the 16-row kernel fits two workgroups per CU, the 32-row one.
    const long long slots = (long long)ctx->n_cus * (p.nt == 16 ? 2 : 1);
    int split_len;
    if (ctx->split_override > 0) {
        split_len = ((ctx->split_override + 31) / 32) * 32;
    } else if (kind == 1) {
        split_len = ((max_keys + 31) / 32) * 32;  // prefill tiles are plentiful: no split
    } else if (min_keys == max_keys) {
        // Equal lengths: give every (sequence, tile) the same whole number of splits so that the
        // launch is exactly one round of at most n_cus workgroups -- a 257th workgroup would wait
        // for a CU and double the kernel's time.
        const long long pairs = (long long)n_seq * p.n_tiles;
        long long per_pair = ctx->n_cus / pairs;
        if (per_pair < 1) per_pair = 1;
        split_len = (int)((max_keys + per_pair - 1) / per_pair);
        split_len = ((split_len + min_split - 1) / min_split) * min_split;
    } else {
        // Ragged lengths: about two workgroups per slot evens out the unequal last splits.
        const long long target_wgs = 2 * slots;
        const long long key_work = total_keys * p.n_tiles;
        long long per_wg = (key_work + target_wgs - 1) / target_wgs;
        // ... and at most 256 splits for the longest sequence: the grid is (splits of the longest, tiles,
        // sequences), and one long sequence beside many short ones would otherwise launch a grid of
        // workgroups that find nothing to do.
        if (per_wg < (max_keys + 255) / 256) per_wg = (max_keys + 255) / 256;
        split_len = (int)(((per_wg + min_split - 1) / min_split) * min_split);
    }
    // Up to 384 keys: one split, whose workgroup writes the final rows itself -- a wavefront's three blocks cost less
    // than the second launch (one decode row at 128 keys 8.6 -> 6.3 us a step, at 256 keys 8.7 -> 7.4; at 512 keys
    // 10.3 against 8.7 the other way).
    if (ctx->split_override <= 0 && kind == 0 && max_keys <= 384) split_len = ((max_keys + 31) / 32) * 32;
    if (split_len < 32) split_len = 32;
    p.split_len = split_len;
    p.n_splits_max = max_keys > 0 ? (max_keys + split_len - 1) / split_len : 1;
    if (p.n_splits_max < 1) p.n_splits_max = 1;
    p.workgroups = (long long)p.n_splits_max * p.n_tiles * n_seq;
    p.xcd_grid = false;
    p.lds_bytes = lds_bytes_for(head_dim, p.nt, p.waves);
    *plan = p;
    return TT_HIP_OK;
}

template <int D, int NT>
static int launch_combine_one(tt_hip_ctx *ctx, const LaunchPlan &plan, int n_seq, const SplitKArgs &args) {
    // Many tiles with few splits each: from 64 of its workgroups on (8 sequences' decode rows, 4 sequences' verify
    // rows; a verify pass of 8 x 4 rows at 65k keys 174.5 -> 170.1 us a step, 8 sequences x 8 rows at 4k keys 36.9 ->
    // 30.0 us; with 32 workgroups -- 4 sequences' decode rows -- the other kernel is ahead, 13.1 against 14.3 us).
    if (plan.n_splits_max <= 2 * kCombineRowsSplits && (long long)plan.n_tiles * n_seq * (NT / 4) >= 64) {
        dim3 cgrid((unsigned)(NT / 4), (unsigned)plan.n_tiles, (unsigned)n_seq);
        hipLaunchKernelGGL((attn_combine_rows_kernel<D, NT>), cgrid, dim3(256), 0, ctx->stream, args);
    } else {
        // (a workgroup per row that a tile can have and 64 dims of it: tiles of 16 with 8 rows in use launch no idle half)
        const int tile_rows = args.hot.rows < plan.tt ? args.hot.rows : plan.tt;
        dim3 cgrid((unsigned)(tile_rows * plan.gh * (D / 64)), (unsigned)plan.n_tiles, (unsigned)n_seq);
        hipLaunchKernelGGL((attn_combine_kernel<D, NT>), cgrid, dim3(256), 0, ctx->stream, args);
    }
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "attn_combine_kernel launch");
}

template <int D, int NT, int WAVES, int BITS, int KEEP = 0, int STREAM = 0>
static int launch_one(tt_hip_ctx *ctx, const LaunchPlan &plan, int n_seq, const SplitKArgs &args) {
    auto kernel = attn_splitk_kernel<D, NT, WAVES, BITS, KEEP, STREAM>;  // its LDS limit was raised when the context was created
    dim3 grid((unsigned)plan.n_splits_max, (unsigned)plan.n_tiles, (unsigned)n_seq);
    if (plan.xcd_grid) grid = dim3((unsigned)(((long long)plan.n_splits_max * plan.n_tiles + 7) / 8 * 8), 1u, (unsigned)n_seq);
    launch_profiled(ctx, kernel, grid, dim3(WAVES * 64), (unsigned)(plan.lds_bytes + keep_list_bytes(KEEP, WAVES)), args);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(ctx, e, "attn_splitk_kernel launch");
    if (plan.n_splits_max > 1 && !ctx->pass_only) return launch_combine_one<D, NT>(ctx, plan, n_seq, args);
    return TT_HIP_OK;
}


// Every instantiation's dynamic LDS limit (a compile-time constant of the kernel), set once per device when a
// context is created on it: no launch has to configure anything, so none is refused inside a graph capture
// and nothing is remembered outside the context.
template <int D, int NT, int BITS, int KEEP>
static hipError_t configure_one() {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_splitk_kernel<D, NT, 4, BITS, KEEP, 0>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)(lds_bytes_for(D, NT, 4) + keep_list_bytes(KEEP, 4)));
    if constexpr (KEEP < 2) {  // (a chunk's per-query selections come with many token tiles: never streamed)
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_splitk_kernel<D, NT, 4, BITS, KEEP, 1>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds_bytes_for(D, NT, 4));
    }
    return e;
}
template <int D, int NT>
static hipError_t configure_tile() {
    hipError_t e = hipSuccess;
#define TT_CFG(BB, KK) \
    if (e == hipSuccess) e = configure_one<D, NT, BB, KK>();
    TT_CFG(16, 0) TT_CFG(8, 0) TT_CFG(4, 0)
    TT_CFG(16, 1) TT_CFG(8, 1) TT_CFG(4, 1)
    TT_CFG(16, 2) TT_CFG(8, 2) TT_CFG(4, 2)
    TT_CFG(16, 3) TT_CFG(8, 3) TT_CFG(4, 3)
#undef TT_CFG
    return e;
}
int configure_splitk_kernels(tt_hip_ctx *ctx) {
    hipError_t e = configure_tile<256, 16>();
    if (e == hipSuccess) e = configure_tile<256, 32>();
    if (e == hipSuccess) e = configure_tile<128, 16>();
    if (e == hipSuccess) e = configure_tile<128, 32>();
    if (e == hipSuccess) e = configure_tile<64, 16>();
    if (e == hipSuccess) e = configure_tile<64, 32>();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "hipFuncSetAttribute(split-K max dynamic LDS)");
}

// The combine pass on its own: for partials written by another kernel in this kernel's layout.
int launch_combine(tt_hip_ctx *ctx, const LaunchPlan &plan, int head_dim, int n_seq, const SplitKArgs &args) {
    if (plan.n_tiles > 65535 || n_seq > 65535) return TT_HIP_ERR_SHAPE;
#define TT_CASE(DD, NN) \
    if (head_dim == DD && plan.nt == NN) return launch_combine_one<DD, NN>(ctx, plan, n_seq, args);
    TT_CASE(256, 16)
    TT_CASE(256, 32)
    TT_CASE(128, 16)
    TT_CASE(128, 32)
    TT_CASE(64, 16)
    TT_CASE(64, 32)
#undef TT_CASE
    return TT_HIP_ERR_SHAPE;
}

int launch_splitk(tt_hip_ctx *ctx, const LaunchPlan &plan, int head_dim, int n_seq, const SplitKArgs &args, int kv_bits) {
    if (n_seq > kMaxSeqPerLaunch || plan.waves != 4) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (plan.n_tiles > 65535 || n_seq > 65535) return TT_HIP_ERR_SHAPE;
#define TT_CASE(DD, NN)                                                                              \
    if (head_dim == DD && plan.nt == NN) {                                                           \
        if (args.plan_blocks) {                                                                      \
            if (kv_bits == 16) return launch_one<DD, NN, 4, 16, 3>(ctx, plan, n_seq, args);          \
            if (kv_bits == 8) return launch_one<DD, NN, 4, 8, 3>(ctx, plan, n_seq, args);            \
            if (kv_bits == 4) return launch_one<DD, NN, 4, 4, 3>(ctx, plan, n_seq, args);            \
        }                                                                                            \
        if (args.keep && args.keep_row_stride > 0) {                                                 \
            if (kv_bits == 16) return launch_one<DD, NN, 4, 16, 2>(ctx, plan, n_seq, args);          \
            if (kv_bits == 8) return launch_one<DD, NN, 4, 8, 2>(ctx, plan, n_seq, args);            \
            if (kv_bits == 4) return launch_one<DD, NN, 4, 4, 2>(ctx, plan, n_seq, args);            \
        }                                                                                            \
        if (args.keep && plan.stream) {                                                              \
            if (kv_bits == 16) return launch_one<DD, NN, 4, 16, 1, 1>(ctx, plan, n_seq, args);       \
            if (kv_bits == 8) return launch_one<DD, NN, 4, 8, 1, 1>(ctx, plan, n_seq, args);         \
            if (kv_bits == 4) return launch_one<DD, NN, 4, 4, 1, 1>(ctx, plan, n_seq, args);         \
        }                                                                                            \
        if (args.keep) {                                                                             \
            if (kv_bits == 16) return launch_one<DD, NN, 4, 16, 1>(ctx, plan, n_seq, args);          \
            if (kv_bits == 8) return launch_one<DD, NN, 4, 8, 1>(ctx, plan, n_seq, args);            \
            if (kv_bits == 4) return launch_one<DD, NN, 4, 4, 1>(ctx, plan, n_seq, args);            \
        }                                                                                            \
        if (plan.stream) {                                                                           \
            if (kv_bits == 16) return launch_one<DD, NN, 4, 16, 0, 1>(ctx, plan, n_seq, args);       \
            if (kv_bits == 8) return launch_one<DD, NN, 4, 8, 0, 1>(ctx, plan, n_seq, args);         \
            if (kv_bits == 4) return launch_one<DD, NN, 4, 4, 0, 1>(ctx, plan, n_seq, args);         \
        }                                                                                            \
        if (kv_bits == 16) return launch_one<DD, NN, 4, 16>(ctx, plan, n_seq, args);                 \
        if (kv_bits == 8) return launch_one<DD, NN, 4, 8>(ctx, plan, n_seq, args);                   \
        if (kv_bits == 4) return launch_one<DD, NN, 4, 4>(ctx, plan, n_seq, args);                   \
    }
    TT_CASE(256, 16)
    TT_CASE(256, 32)
    TT_CASE(128, 16)
    TT_CASE(128, 32)
    TT_CASE(64, 16)
    TT_CASE(64, 32)
#undef TT_CASE
    return TT_HIP_ERR_SHAPE;
}

}  // namespace tt
