// Causal chunk (prefill) flash attention on gfx950 MFMA, K/V tiles staged in LDS.
//
// Same transposed formulation as the split-K kernel (a lane owns a query row):
//   S^T[key][row] = K . Q^T      A = K fragment from LDS,   B = Q^T fragment in registers
//   O^T[d][row]  += V^T . P^T    A = V^T fragment from LDS, B = P^T straight from S^T's registers
// with v_mfma_f32_32x32x16_f16.
//
// Work decomposition.  A wavefront owns 64 query rows of ONE q head as two
// 32-row tiles, processed one after the other: token tile i ("short") and token
// tile n_tiles-1-i ("long").  Tile i needs i+1 key blocks, its partner
// n_tiles-i, so every wavefront does the same number of MFMAs whatever i is --
// the causal triangle is balanced by construction instead of by a scheduler --
// and only 128 accumulator registers are live at a time.  A workgroup is 4 such
// wavefronts: the same tile pair for 4 q heads of one KV head, so they share
// every K/V block.  Blocks stream L2 -> LDS with direct-to-LDS 128-bit loads
// (no registers), four stages deep, one barrier per block; the K fragment
// layout in HBM is the MFMA operand layout, V is permuted into it by the copy.
//
// The online softmax rescales the accumulators lazily: the running reference
// max only moves when a row's block max exceeds it by more than 8 (log2 units),
// so probabilities stay below 2^8 (well inside fp16's range) and the
// accumulators are rescaled a handful of times per row instead of once per block.
//
// Replaces attention_prefill_causal_q8 / attention_prefill_causal_tiled
// (sources/TinyTitanCore/Metal/Prefill/prefill.metal:1056-1313) dispatched by
// PrefillAttention.encodeCausal (sources/TinyTitan/Kernels/Attention/PrefillAttention.swift:165-258).
#include "internal.h"
#include "wave_ops.h"

namespace tt {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

struct PrefillArgs {
    const _Float16 *k_slot;  // page of kv head 0 of this slot
    const _Float16 *v_slot;
    const _Float16 *q;
    const _Float16 *gate;
    _Float16 *out;
    long long page_elems;
    long long q_stride, g_stride, o_stride;
    int group;     // q heads per kv head
    int hsubs;     // group / 4
    int n_tiles;   // ceil(q_len / 32)
    int n_pairs;   // ceil(n_tiles / 2)
    int per_kvh;   // hsubs * n_pairs
    int xs;        // XCDs per kv head (8 / n_kv_heads), 0: plain mapping
    int n_kv_heads;
    int start, q_len, kv_valid;
    float scale_log2e;
};

namespace {

constexpr float kNegBig = -1.0e30f;
constexpr float kRescaleThreshold = 8.0f;
constexpr int kBuffers = 4;  // LDS stages (K block + V block each): 128 KiB at D = 256

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef const __attribute__((address_space(1))) void *gbl_ptr_t;

// 16 bytes per lane, global -> LDS without passing through registers: lane l's 16 bytes land at
// lds_addr + 16 l.  Issued as inline assembly on purpose: the compiler, when it sees an LDS DMA,
// guards every later LDS read with a full vmcnt(0) wait (it cannot tell the stages apart),
// which would turn a multi-stage prefetch into none.  Completion is tracked by hand instead:
// TT_WAIT_VMCNT before the barrier that publishes a stage.
__device__ __forceinline__ void copy16_global_to_lds(const void *base, unsigned lane_offset, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %1, %0" : : "s"(base), "v"(lane_offset), "s"(lds_addr) : "m0", "memory");
}

// vmcnt(n) only: leaves the LDS/scalar and export counters alone.
#define TT_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

struct TileState {
    float m, l;
};

typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// Softmax of one 32-row tile on one block's scores.
//
// Common path (softmax_slice): probabilities are taken against the row's current
// reference max without looking at the block's own max, so nothing in it waits on a reduction
// and nothing touches the accumulators; it also returns the largest exponent it used.  Only when
// some row's exponent exceeds the threshold (the first block of a row, and a handful of
// times after that) is the block redone by softmax_moving_reference, which moves the
// reference and rescales the accumulators.  A masked (diagonal) block always takes the second.

// Step v (0..15) of the common path, for score register v of the block: p = exp2(s * scale - m);
// every second step packs two probabilities into the B operand of the P.V MFMAs, adds them to
// the row sum -- taken over the ROUNDED probabilities (dot2 against ones), i.e. over exactly
// the weights the MFMAs see -- and folds the two exponents into `top`, the largest exponent used.
__device__ __forceinline__ void softmax_slice(int v, const f16v &s, float scale_log2e, float m, float &l, float &top,
                                              float &e_prev, float &t_prev, h8 (&pf)[2]) {
    const float t = __builtin_fmaf(s[v], scale_log2e, -m);
    const float e = fast_exp2(t);
    if (v & 1) {
        const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
        const h2 p = {(_Float16)e_prev, (_Float16)e};
        l = __builtin_amdgcn_fdot2(p, ones, l, false);
        pf[v >> 3][(v & 7) - 1] = p[0];
        pf[v >> 3][v & 7] = p[1];
        top = v == 1 ? fmaxf(t_prev, t) : fmaxf(fmaxf(t_prev, t), top);
    } else {
        e_prev = e;
        t_prev = t;
    }
}

// Full online-softmax step: mask, move the reference max up to the block max where it is
// exceeded, rescale the tile's state, and produce the probabilities.
template <int MT>
__device__ __forceinline__ void softmax_moving_reference(const f16v &s_raw, bool mask, int kbase, int lim, int g,
                                                         float scale_log2e, TileState &st, f16v (&o)[MT], h8 (&pf)[2]) {
    const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    float t[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) t[v] = s_raw[v] * scale_log2e;
    if (mask) {  // wave-uniform: only the blocks on or past the tile's diagonal
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = kbase + 8 * (v >> 2) + 4 * g + (v & 3);
            if (key >= lim) t[v] = -INFINITY;
        }
    }
    float mx = kNegBig;
#pragma unroll
    for (int v = 0; v < 16; ++v) mx = fmaxf(mx, t[v]);
    mx = max_across_halves(mx);
    const bool move = mx > st.m + kRescaleThreshold;  // per row (a row's first visible block always moves)
    const float m_new = move ? mx : st.m;
    if (__any(move)) {
        const float alpha = fast_exp2(st.m - m_new);  // 1 for the rows that stay
        st.l *= alpha;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
    }
    st.m = m_new;
#pragma unroll
    for (int v = 0; v < 16; v += 2) {
        const h2 p = {(_Float16)fast_exp2(t[v] - st.m), (_Float16)fast_exp2(t[v + 1] - st.m)};
        st.l = __builtin_amdgcn_fdot2(p, ones, st.l, false);
        pf[v >> 3][v & 7] = p[0];
        pf[v >> 3][(v & 7) + 1] = p[1];
    }
}

}  // namespace

template <int D>
__global__ __launch_bounds__(256, 1) __attribute__((amdgpu_waves_per_eu(1, 1))) void attn_prefill_kernel(const PrefillArgs a) {
    constexpr int KS = D / 16;  // k-steps of S^T
    constexpr int MT = D / 32;  // 32-dim tiles of O^T
    constexpr int BLOCK_BYTES = 32 * D * 2;
    constexpr int STAGE_BYTES = 2 * BLOCK_BYTES;  // K block then V block
    constexpr int CHUNKS = BLOCK_BYTES / 1024;    // 1 KiB chunks per block (= KS = 2 MT)
    constexpr int kCopiesPerBlock = 2 * (CHUNKS / 4);  // LDS-DMA instructions one wave issues per block
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int li = lane & 31, g = lane >> 5;

    // Workgroup -> (kv head, head sub-group, tile pair); kv heads are spread over XCDs so
    // that each XCD's L2 holds one kv head's K/V.
    int kvh, r;
    if (a.xs > 0) {
        const int x = blockIdx.x & 7, y = blockIdx.x >> 3;
        kvh = x / a.xs;
        r = y * a.xs + (x - kvh * a.xs);
    } else {
        kvh = blockIdx.x / a.per_kvh;
        r = blockIdx.x - kvh * a.per_kvh;
    }
    if (r >= a.per_kvh || kvh >= a.n_kv_heads) return;
    const int hsub = r / a.n_pairs;
    const int pair = r - hsub * a.n_pairs;
    const int head = kvh * a.group + hsub * 4 + wave;
    const _Float16 *kp = a.k_slot + (size_t)kvh * a.page_elems;
    const _Float16 *vp = a.v_slot + (size_t)kvh * a.page_elems;

    // Stage loader: this wave copies CHUNKS/4 K chunks and CHUNKS/4 V chunks of block j.
    const unsigned smem_base = (unsigned)(size_t)(lds_ptr_t)smem;
    const unsigned k_lane_offset = (unsigned)lane * 16u;
    const unsigned v_lane_offset = (unsigned)((li * 4 + g) * 16);  // this lane's 16 bytes inside a V chunk gather
    auto issue_block = [&](int j, int buffer) {
        const unsigned stage = smem_base + (unsigned)(buffer * STAGE_BYTES);
        const char *kb = reinterpret_cast<const char *>(kp + (size_t)j * (32 * D));
        const char *vb = reinterpret_cast<const char *>(vp + (size_t)j * (32 * D));
#pragma unroll
        for (int c = 0; c < CHUNKS / 4; ++c) {
            const int chunk = wave * (CHUNKS / 4) + c;
            // K: LDS layout == HBM layout (fragment s is chunk s).
            copy16_global_to_lds(kb + chunk * 1024, k_lane_offset, stage + chunk * 1024);
        }
#pragma unroll
        for (int c = 0; c < CHUNKS / 4; ++c) {
            const int chunk = wave * (CHUNKS / 4) + c;  // = 2 * mt + t
            const int mt = chunk >> 1, t = chunk & 1;
            // V: gather so that LDS holds fragment (mt, t) as [lane][8 halves].
            copy16_global_to_lds(vb + (32 * mt * 4 + 2 * t) * 16, v_lane_offset, stage + BLOCK_BYTES + chunk * 1024);
        }
    };

    // The same copies one at a time, for the interleaved loop: copy c (0 .. KS-1) of the pair of
    // blocks (ja, jb) -- K of ja, K of jb, V of ja, V of jb, CHUNKS/4 each.  A copy instruction
    // occupies the CU's vector memory path for ~16 cycles per wave and stalls the wave when that
    // path is backed up, so they are issued one by one between MFMAs, never in a burst.
    auto issue_copy = [&](int c, int ja, int jb, int stage_ja, int stage_jb) {
        constexpr int Q4 = CHUNKS / 4;
        const int which = c / Q4, i = c % Q4;  // compile-time after unrolling
        const int jx = (which & 1) ? jb : ja;
        const unsigned stage = smem_base + (unsigned)((((which & 1) ? stage_jb : stage_ja) & (kBuffers - 1)) * STAGE_BYTES);
        const int chunk = wave * Q4 + i;
        if (which < 2) {
            const char *kb = reinterpret_cast<const char *>(kp + (size_t)jx * (32 * D));
            copy16_global_to_lds(kb + chunk * 1024, k_lane_offset, stage + chunk * 1024);
        } else {
            const char *vb = reinterpret_cast<const char *>(vp + (size_t)jx * (32 * D));
            const int mt = chunk >> 1, t = chunk & 1;
            copy16_global_to_lds(vb + (32 * mt * 4 + 2 * t) * 16, v_lane_offset, stage + BLOCK_BYTES + chunk * 1024);
        }
    };

    const int n_passes = (pair == a.n_tiles - 1 - pair) ? 1 : 2;
    for (int pass = 0; pass < n_passes; ++pass) {
        // The long tile goes first: the short one then fills in behind it.
        const int tile = pass == 0 ? a.n_tiles - 1 - pair : pair;
        const int tok = tile * 32 + li;
        const bool valid = tok < a.q_len;
        const int lim = valid ? min(a.kv_valid, a.start + tok + 1) : 0;  // keys [0, lim) are visible
        const int end = min(a.kv_valid, a.start + min(a.q_len, tile * 32 + 32));
        const int nb = (end + 31) >> 5;                        // key blocks this tile needs
        const int mask_from = (a.start + tile * 32 + 1) >> 5;  // first block in which some row is masked

        if (pass > 0) __syncthreads();  // every wave is done reading the previous pass's stages
        for (int b0 = 0; b0 < 2 && b0 < nb; ++b0) issue_block(b0, b0);

        // Query fragments (B operand); rows of padding tokens are zero.
        h8 qf[KS];
        {
            const _Float16 *qp = a.q + (long long)(valid ? tok : 0) * a.q_stride + (long long)head * D + 8 * g;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const h8 x = *reinterpret_cast<const h8 *>(qp + 16 * s);
                qf[s] = valid ? x : (h8)(_Float16)0;
            }
            // The query fragments rest in accumulation registers: the VGPRs are needed for the
            // K/V fragments in flight, and an MFMA reads its B operand from either file.
#pragma unroll
            for (int s = 0; s < KS; ++s) asm volatile("" : "+a"(qf[s]));
        }
        f16v o[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) o[mt] = (f16v)0.0f;
        TileState st{kNegBig, 0.0f};
        TT_WAIT_VMCNT(0);  // stages 0/1 and the query rows; keeps the in-loop counting simple

        // Blocks [0, n_fast) are full and unmasked for every row of the tile; they go two at a
        // time through the interleaved body below, the rest (an odd one, the diagonal) singly.
        const int first_masked = min(mask_from, end >> 5);
        const int n_fast = first_masked & ~1;
        int issued = min(nb, 2);

        // Publish blocks [j, j + n) (their copies are the oldest outstanding ones) and refill the
        // stages that every wave has left: block b lives in stage b % kBuffers.
        auto acquire = [&](int j, int n, bool refill) {
            const int flying = issued - (j + n);  // newer blocks whose copies may stay in flight
            if (flying <= 0) TT_WAIT_VMCNT(0);
            else if (flying == 1) TT_WAIT_VMCNT(kCopiesPerBlock);
            else TT_WAIT_VMCNT(2 * kCopiesPerBlock);
            __syncthreads();
            while (refill && issued < nb && issued < j + kBuffers) {
                issue_block(issued, issued & (kBuffers - 1));
                ++issued;
            }
        };

        // The interleaved body never touches the accumulators with the VALU (they stay in
        // the accumulation registers).  When a row's exponent exceeds the threshold it leaves the
        // block(s) not yet accumulated to the one-block path below, which moves the reference
        // max and rescales, and the interleaved loop is re-entered behind them.
        int j = 0;
        while (j < nb) {
            int single_from = j, single_to = nb;
            bool resident = false;  // the single blocks were already acquired by the pair loop
#pragma nounroll
            for (; j < n_fast; j += 2) {
                acquire(j, 2, false);
                // Blocks j+2 and j+3 are copied during phases 1 and 2 (past the end of the tile
                // the last block is copied again, into a stage nobody reads: no branches here).
                const int ja = min(j + 2, nb - 1), jb = min(j + 3, nb - 1);
                const int stage_ja = j + 2, stage_jb = j + 3;
                issued = min(nb, j + 4);
#pragma unroll
                for (int s = 0; s < KS; ++s) asm volatile("" : "+a"(qf[s]));
                const char *stage_a = smem + (j & (kBuffers - 1)) * STAGE_BYTES + lane * 16;
                const char *stage_b = smem + ((j + 1) & (kBuffers - 1)) * STAGE_BYTES + lane * 16;
                h8 fa[KS], fb[KS], pa[2], pb[2];
                // The four phases below are written out in issue order, one MFMA + one LDS read +
                // one slice of softmax per step, with a scheduling fence after every step: a
                // wavefront issues in order, so the matrix pipe, the LDS and the VALU only overlap
                // if their instructions alternate in the stream.
                // Phase 1: scores of block a; K fragments of block b arrive behind them.
#pragma unroll
                for (int t = 0; t < KS; ++t) fa[t] = *reinterpret_cast<const h8 *>(stage_a + t * 1024);
                __builtin_amdgcn_sched_barrier(0);
                f16v sa = (f16v)0.0f, sb = (f16v)0.0f;
#pragma unroll
                for (int t = 0; t < KS; ++t) {
                    sa = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[t], qf[t], sa, 0, 0, 0);
                    fb[t] = *reinterpret_cast<const h8 *>(stage_b + t * 1024);
                    if ((t & 1) == 0) issue_copy(t / 2, ja, jb, stage_ja, stage_jb);
                    __builtin_amdgcn_sched_barrier(0);
                }
                // Phase 2: scores of block b on the MFMA pipe, softmax of block a on the VALU, V
                // fragments of block a from LDS into the registers its K fragments have left.
                float la = st.l, top_a, e_prev = 0.0f, t_prev = 0.0f;
#pragma unroll
                for (int t = 0; t < KS; ++t) {
                    sb = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[t], qf[t], sb, 0, 0, 0);
                    fa[t] = *reinterpret_cast<const h8 *>(stage_a + BLOCK_BYTES + t * 1024);
                    if (t < 16) softmax_slice(t, sa, a.scale_log2e, st.m, la, top_a, e_prev, t_prev, pa);
                    if ((t & 1) == 0) issue_copy(KS / 2 + t / 2, ja, jb, stage_ja, stage_jb);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (KS < 16) {
#pragma unroll
                    for (int t = KS; t < 16; ++t) softmax_slice(t, sa, a.scale_log2e, st.m, la, top_a, e_prev, t_prev, pa);
                }
                // (An empty asm that "uses" the probabilities: they are wanted HERE, computed
                // under the MFMAs, and would otherwise be sunk below the branch.)
                asm volatile("" : "+v"(pa[0]), "+v"(pa[1]), "+v"(la));
                if (__any(top_a > kRescaleThreshold)) {
                    single_from = j, single_to = j + 2, resident = true;
                    break;
                }
                st.l = la;
                // Phase 3: P.V of block a, softmax of block b, V fragments of block b.
                float lb = la, top_b;
#pragma unroll
                for (int t = 0; t < KS; ++t) {
                    const int mt = t % MT, ks = t / MT;
                    o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fa[2 * mt + ks], pa[ks], o[mt], 0, 0, 0);
                    fb[t] = *reinterpret_cast<const h8 *>(stage_b + BLOCK_BYTES + t * 1024);
                    if (t < 16) softmax_slice(t, sb, a.scale_log2e, st.m, lb, top_b, e_prev, t_prev, pb);
                    __builtin_amdgcn_sched_barrier(0);
                }
                if constexpr (KS < 16) {
#pragma unroll
                    for (int t = KS; t < 16; ++t) softmax_slice(t, sb, a.scale_log2e, st.m, lb, top_b, e_prev, t_prev, pb);
                }
                asm volatile("" : "+v"(pb[0]), "+v"(pb[1]), "+v"(lb));
                if (__any(top_b > kRescaleThreshold)) {
                    single_from = j + 1, single_to = j + 2, resident = true;
                    break;
                }
                st.l = lb;
                // Phase 4: P.V of block b.
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[2 * mt + t], pb[t], o[mt], 0, 0, 0);
            }
            if (!resident) single_from = j;  // the pair loop ran out: everything that is left
#pragma nounroll
            for (int jj = single_from; jj < single_to; ++jj) {
                if (!resident) acquire(jj, 1, true);
                const char *stage = smem + (jj & (kBuffers - 1)) * STAGE_BYTES + lane * 16;
                h8 kf[KS], vf[KS], pf[2];
#pragma unroll
                for (int t = 0; t < KS; ++t) kf[t] = *reinterpret_cast<const h8 *>(stage + t * 1024);
                __builtin_amdgcn_sched_barrier(0);
                f16v s = (f16v)0.0f;
#pragma unroll
                for (int t = 0; t < KS; ++t) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[t], qf[t], s, 0, 0, 0);
#pragma unroll
                for (int c = 0; c < KS; ++c) vf[c] = *reinterpret_cast<const h8 *>(stage + BLOCK_BYTES + c * 1024);
                __builtin_amdgcn_sched_barrier(0);
                softmax_moving_reference<MT>(s, jj >= first_masked, jj << 5, lim, g, a.scale_log2e, st, o, pf);
#pragma unroll
                for (int t = 0; t < 2; ++t)
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt)
                        o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[2 * mt + t], pf[t], o[mt], 0, 0, 0);
            }
            j = single_to;
        }

        // Epilogue: normalise, gate in fp32, one fp16 round, store.  Lane (li, g), register v of
        // tile mt holds dim 32 mt + 8 (v / 4) + 4 g + v % 4 of row li.
        const float l = sum_across_halves(st.l);
        if (valid) {
            const float inv = l > 0.0f ? 1.0f / l : 0.0f;
            _Float16 *op = a.out + (long long)tok * a.o_stride + (long long)head * D + 4 * g;
            const _Float16 *gp = a.gate ? a.gate + (long long)tok * a.g_stride + (long long)head * D + 4 * g : nullptr;
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int vq = 0; vq < 4; ++vq) {
                    const int d = 32 * mt + 8 * vq;
                    float r[4];
#pragma unroll
                    for (int i = 0; i < 4; ++i) r[i] = o[mt][4 * vq + i] * inv;
                    if (gp) {
                        const h4 gv = *reinterpret_cast<const h4 *>(gp + d);
#pragma unroll
                        for (int i = 0; i < 4; ++i) r[i] *= 1.0f / (1.0f + __expf(-(float)gv[i]));
                    }
                    const h4 hv = {(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
                    *reinterpret_cast<h4 *>(op + d) = hv;
                }
        }
    }
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------

// The kernel wants 4 q heads per KV head in a workgroup and 16-byte aligned rows; anything
// else is served by the split-K kernel.
bool prefill_kernel_serves(int n_q_heads, int n_kv_heads, int head_dim, bool aligned) {
    const int group = n_q_heads / n_kv_heads;
    return aligned && group % 4 == 0 && (head_dim == 256 || head_dim == 128 || head_dim == 64);
}

template <int D>
static int launch_prefill_d(tt_hip_ctx *ctx, const PrefillArgs &args, unsigned grid) {
    static bool attr_set[16] = {false};
    constexpr int lds = kBuffers * 2 * 32 * D * 2;  // four K+V stages: 128 KiB at D = 256
    auto kernel = attn_prefill_kernel<D>;
    if (ctx->device < 16 && !attr_set[ctx->device]) {
        if (ctx->capturing) return TT_HIP_ERR_BUSY;
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipFuncSetAttribute(max dynamic LDS)");
        attr_set[ctx->device] = true;
    }
    const bool timed = ctx->profiling && !ctx->capturing && ctx->prof_used + 2 <= ctx->prof_events.size();
    if (timed) (void)hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream);
    hipLaunchKernelGGL(kernel, dim3(grid), dim3(256), lds, ctx->stream, args);
    hipError_t e = hipGetLastError();
    if (timed) {
        (void)hipEventRecord(ctx->prof_events[ctx->prof_used + 1], ctx->stream);
        ctx->prof_used += 2;
    }
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "attn_prefill_kernel launch");
}

int launch_prefill(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start, int q_len, int kv_valid,
                   int n_q_heads, const tt_half *q, long long q_stride, const tt_half *gate, long long g_stride,
                   float scale, tt_half *out, long long o_stride) {
    PrefillArgs a{};
    const size_t slot_off = (size_t)slot * kv->n_kv_heads * kv->page_elems();
    a.k_slot = kv->k[layer] + slot_off;
    a.v_slot = kv->v[layer] + slot_off;
    a.q = reinterpret_cast<const _Float16 *>(q);
    a.gate = reinterpret_cast<const _Float16 *>(gate);
    a.out = reinterpret_cast<_Float16 *>(out);
    a.page_elems = (long long)kv->page_elems();
    a.q_stride = q_stride;
    a.g_stride = g_stride;
    a.o_stride = o_stride;
    a.group = n_q_heads / kv->n_kv_heads;
    a.hsubs = a.group / 4;
    a.n_tiles = (q_len + 31) / 32;
    a.n_pairs = (a.n_tiles + 1) / 2;
    a.per_kvh = a.hsubs * a.n_pairs;
    a.n_kv_heads = kv->n_kv_heads;
    a.xs = (kv->n_kv_heads <= 8 && 8 % kv->n_kv_heads == 0) ? 8 / kv->n_kv_heads : 0;
    a.start = start;
    a.q_len = q_len;
    a.kv_valid = kv_valid;
    a.scale_log2e = scale * 1.4426950408889634f;
    unsigned grid;
    if (a.xs > 0) grid = 8u * (unsigned)((a.per_kvh + a.xs - 1) / a.xs);
    else grid = (unsigned)(a.per_kvh * kv->n_kv_heads);
    switch (kv->head_dim) {
        case 256: return launch_prefill_d<256>(ctx, a, grid);
        case 128: return launch_prefill_d<128>(ctx, a, grid);
        case 64: return launch_prefill_d<64>(ctx, a, grid);
        default: return TT_HIP_ERR_SHAPE;
    }
}

}  // namespace tt
