// Causal chunk (prefill) flash attention on gfx950 MFMA, K/V tiles staged in LDS,
// score and value wavefronts specialised.
//
// Same transposed formulation as the split-K kernel (a lane owns a query row):
//   S^T[key][row] = K . Q^T      A = K fragment from LDS,   B = Q^T fragment in registers
//   O^T[d][row]  += V^T . P^T    A = V^T fragment from LDS, B = P^T as it left S^T's registers
// with v_mfma_f32_32x32x16_f16.
//
// Work decomposition.  A workgroup serves 4 q heads of one KV head over 64 query rows, as two
// 32-row tiles processed one after the other: token tile n_tiles-1-i ("long"), then tile i
// ("short").  Tile i needs i+1 key blocks, its partner n_tiles-i, so every workgroup does the
// same number of MFMAs whatever i is -- the causal triangle is balanced by construction.
//
// Each (head, tile) is served by TWO wavefronts on the same SIMD:
//   * the score wave holds Q (64 registers at D = 256), computes S^T for key block j, runs the
//     online softmax (reference max, row sum) and leaves P^T -- already in MFMA B-operand
//     order -- plus the per-row rescale factors in LDS;
//   * the value wave holds O^T (128 accumulation registers at D = 256) and, one step behind,
//     accumulates P^T(j-1) against V(j-1).
// Neither needs more than half of the register file, so two waves fit per SIMD, and the
// hardware overlaps one wave's MFMAs with the other's softmax VALU work and LDS reads; eight
// waves per CU also issue LDS reads about 1.6x faster than four can (the per-wave issue rate
// is what limits a 4-wave design).  One workgroup barrier per key block separates the steps.
//
// K/V blocks stream L2 -> LDS with direct-to-LDS 128-bit loads (no registers), four stages
// deep, issued two steps ahead of their first use; the K fragment layout in HBM is the MFMA
// operand layout, V is permuted into it by the copy.
//
// The online softmax rescales lazily: a row's reference max only moves when its block max
// exceeds it by more than 8 (log2 units), so probabilities stay below 2^8 (well inside fp16's
// range) and the value wave rescales its accumulators a handful of times per row.
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
    int n_pairs;   // ceil(n_tiles / 2); with single_tiles: n_tiles
    int single_tiles;  // 1: a workgroup takes ONE tile (tile = its pair index) instead of a long and a short one
    int per_kvh;   // hsubs * n_pairs
    int xs;        // XCDs per kv head (8 / n_kv_heads), 0: plain mapping
    int n_kv_heads;
    int start, q_len, kv_valid;
    int window;  // sliding window (0: none): the row at position p sees keys [max(0, p + 1 - window), p + 1)
    int ring_blocks;  // ring cache: key block b lives in block b % ring_blocks of the page; 0 = where it is
    float scale_log2e;
    // Key splits (n_splits > 1): workgroup (base, split) walks key blocks [split * split_blocks,
    // (split + 1) * split_blocks) of each of its tiles and leaves unnormalised partials
    // (reference max, sum, O) in the split-K kernel's layout for its combine pass.
    int n_splits, split_blocks, base_grid;
    int xcd_chunk;  // key ranges with xs > 0: (range, tile, head set) items one XCD takes, ceil(per_kvh * n_splits / xs)
    float *part_o;   // [split][head * n_tiles + tile][32 rows][D]
    float *part_ml;  // [split][head * n_tiles + tile][32 rows][2]
};

namespace {

constexpr float kNegBig = -1.0e30f;
constexpr float kRescaleThreshold = 8.0f;
constexpr int kBuffers = 4;  // LDS stages (K block + V block each): 128 KiB at D = 256

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

typedef __attribute__((address_space(3))) void *lds_ptr_t;
typedef _Float16 h2 __attribute__((ext_vector_type(2)));

// 16 bytes per lane, global -> LDS without passing through registers: lane l's 16 bytes land at
// lds_addr + 16 l.  Issued as inline assembly on purpose: the compiler, when it sees an LDS DMA,
// guards every later LDS read with a full vmcnt(0) wait (it cannot tell the stages apart),
// which would turn a multi-stage prefetch into none.  Completion is tracked by hand instead:
// TT_WAIT_VMCNT before the barrier that publishes a stage.
__device__ __forceinline__ void copy16_global_to_lds(const void *base, unsigned lane_offset, unsigned lds_addr) {
    // base and lds_addr are wave-uniform by construction; say so, in case the compiler lost track
    const unsigned long long b = (unsigned long long)base;
    const unsigned b_hi = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)(b >> 32));
    const unsigned b_lo = (unsigned)__builtin_amdgcn_readfirstlane((int)(unsigned)b);  // (the builtin returns a signed int)
    base = (const void *)(((unsigned long long)b_hi << 32) | (unsigned long long)b_lo);
    lds_addr = (unsigned)__builtin_amdgcn_readfirstlane((int)lds_addr);
    // m0 carries the LDS address of the copy.  The compiler owns m0 (it is a reserved register: naming it as a
    // clobber is not honoured), so the block saves it and puts it back; nothing else is touched.
    unsigned saved_m0;
    asm volatile("s_mov_b32 %0, m0\n\ts_mov_b32 m0, %3\n\tglobal_load_lds_dwordx4 %2, %1\n\ts_mov_b32 m0, %0"
                 : "=&s"(saved_m0)
                 : "s"(base), "v"(lane_offset), "s"(lds_addr)
                 : "memory");
}

// vmcnt(n) only: leaves the LDS/scalar and export counters alone.
#define TT_WAIT_VMCNT(n) __builtin_amdgcn_s_waitcnt(((n) & 0xF) | (((n) >> 4) << 14) | (0x7 << 4) | (0xF << 8))

// One online-softmax step of the score wave on a block's scores: mask, move the row's reference
// max where the block max exceeds it by more than the threshold, and produce the
// probabilities (B operand of the two P.V k-steps) against the reference.  The row sum is taken
// over the ROUNDED probabilities (dot2 against ones), i.e. over exactly the weights the P.V MFMAs
// see.  Returns the factor the row's accumulators must be scaled by before this block is added.
__device__ __forceinline__ float softmax_step(const f16v &s_raw, bool mask, int kbase, int lo, int lim, int g,
                                              float scale_log2e, float &m, float &l, h8 (&pf)[2]) {
    const h2 ones = {(_Float16)1.0f, (_Float16)1.0f};
    // The maximum is taken over the raw scores and scaled once (the host sends only chunks with scale > 0 here), and a
    // probability is one fused multiply-add and one exp2 off its raw score.
    float t[16];
#pragma unroll
    for (int v = 0; v < 16; ++v) t[v] = s_raw[v];
    if (mask) {  // wave-uniform: only the blocks on or past the tile's diagonal, or at its window's lower edge
#pragma unroll
        for (int v = 0; v < 16; ++v) {
            const int key = kbase + 8 * (v >> 2) + 4 * g + (v & 3);
            if (key >= lim || key < lo) t[v] = -INFINITY;
        }
    }
    float mx = fmaxf(t[0], t[1]);
#pragma unroll
    for (int v = 2; v < 16; v += 2) mx = fmaxf(fmaxf(t[v], t[v + 1]), mx);
    mx = max_across_halves(mx) * scale_log2e;
    const bool move = mx > m + kRescaleThreshold;  // a row's first visible block always moves
    const float m_new = move ? mx : m;
    const float alpha = move ? fast_exp2(m - m_new) : 1.0f;
    l *= alpha;
    m = m_new;
#pragma unroll
    for (int v = 0; v < 16; v += 2) {
        const h2 p = {(_Float16)fast_exp2(__builtin_fmaf(t[v], scale_log2e, -m)), (_Float16)fast_exp2(__builtin_fmaf(t[v + 1], scale_log2e, -m))};
        l = __builtin_amdgcn_fdot2(p, ones, l, false);
        pf[v >> 3][v & 7] = p[0];
        pf[v >> 3][(v & 7) + 1] = p[1];
    }
    return alpha;
}

}  // namespace

template <int D>
__global__ __launch_bounds__(512, 1) void attn_prefill_kernel(const PrefillArgs a) {
    constexpr int KS = D / 16;  // k-steps of S^T
    constexpr int MT = D / 32;  // 32-dim tiles of O^T
    constexpr int BLOCK_BYTES = 32 * D * 2;
    constexpr int CHUNKS = BLOCK_BYTES / 1024;    // 1 KiB chunks per block (= KS = 2 MT)
    constexpr int CPW = CHUNKS / 4;               // copies one wave issues per step (a K and a V block over 8 waves)
    constexpr int V_OFF = kBuffers * BLOCK_BYTES;    // K ring, then V ring, kBuffers blocks each
    constexpr int P_OFF = 2 * kBuffers * BLOCK_BYTES;  // P^T: [2 steps][4 heads][2 k-steps][64 lanes][16 B]
    constexpr int ALPHA_OFF = P_OFF + 2 * 4 * 2048;    // rescale factors: [2 steps][4 heads][32 rows] floats
    constexpr int LSUM_OFF = ALPHA_OFF + 2 * 4 * 128;  // row sums: [4 heads][32 rows] floats
    constexpr int STAGE_OFF = LSUM_OFF + 4 * 128;      // output rows on their way out: [4 heads][32 rows][32 dims + 16 B]
    constexpr int STAGE_PITCH = 64 + 16;
    extern __shared__ __attribute__((aligned(16))) char smem[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const bool value_wave = wave >= 4;
    const int w4 = wave & 3;
    const int li = lane & 31, g = lane >> 5;

    // Workgroup -> (kv head, head sub-group, tile pair); kv heads are spread over XCDs so
    // that each XCD's L2 holds one kv head's K/V.
    int split = blockIdx.x / a.base_grid;
    const int wg = blockIdx.x - split * a.base_grid;  // base_grid is a multiple of 8: wg & 7 is still the XCD
    int kvh, r;
    if (a.xcd_chunk > 0) {
        // Key ranges: the (range, tile, head set) items of a kv head, range-major, are cut into as many runs as the kv
        // head has XCDs (workgroup b runs on XCD b % 8).  Every XCD gets the same number of workgroups whatever the
        // number of tiles -- dealt out tile by tile, 3 or 5 tiles per head set leave some XCDs with twice the work of
        // others -- and a range's K/V blocks are fetched into one L2, or two, instead of all of the kv head's.
        const int x = blockIdx.x & 7, j = blockIdx.x >> 3;
        kvh = x / a.xs;
        const int w = (x - kvh * a.xs) * a.xcd_chunk + j;
        if (w >= a.per_kvh * a.n_splits) return;
        split = w / a.per_kvh;
        r = w - split * a.per_kvh;
    } else if (a.xs > 0) {
        const int x = wg & 7, y = wg >> 3;
        kvh = x / a.xs;
        r = y * a.xs + (x - kvh * a.xs);
    } else {
        kvh = wg / a.per_kvh;
        r = wg - kvh * a.per_kvh;
    }
    if (r >= a.per_kvh || kvh >= a.n_kv_heads) return;
    const int hsub = r / a.n_pairs;
    const int pair = r - hsub * a.n_pairs;
    const int head = kvh * a.group + hsub * 4 + w4;
    const _Float16 *kp = a.k_slot + (size_t)kvh * a.page_elems;
    const _Float16 *vp = a.v_slot + (size_t)kvh * a.page_elems;

    // Copies of step i: K block i + 4 and V block i + 2, 2 CHUNKS one-KiB chunks of which this wave
    // issues CPW.  Block b lives in slot b % kBuffers of its ring.  Past the end of the tile the
    // last block is copied again (into a slot nobody reads any more), so that every step puts
    // the same number of copies in flight and one constant vmcnt tracks them.
    const unsigned smem_base = (unsigned)(size_t)(lds_ptr_t)smem;
    const unsigned k_lane_offset = (unsigned)lane * 16u;
    const unsigned v_lane_offset = (unsigned)((li * 4 + g) * 16);  // this lane's 16 bytes inside a V chunk gather
    int jb = 0;  // first key block of this workgroup's range in the current tile
    // Block b of the tile in hand lives in slot (b + slot_off) % kBuffers.  When a second tile follows (carry_nb > 0:
    // it has that many blocks, from block 0), the copies past the end of the first fetch ITS first blocks -- K 0..3 and
    // V 0..3 are in LDS when the first tile's last step ends, in the slots that follow on, and the second tile starts
    // without waiting for memory.
    int slot_off = 0, carry_nb = 0;
    auto page_block = [&](int block) { return a.ring_blocks ? block % a.ring_blocks : block; };
    auto source_block = [&](int j, int nb) {  // the block that step-relative index j stands for
        if (j < nb || carry_nb == 0) return jb + max(min(j, nb - 1), 0);
        return min((j - nb) & (kBuffers - 1), carry_nb - 1);  // (a slot's block again once the four are in: the same bytes)
    };
    // A step's copies: this wave's CPW one-KiB chunks of ONE block -- K block i + 4 for the score waves (chunk
    // wave * CPW + c; the LDS layout is the HBM layout, fragment s is chunk s), V block i + 2 for the value waves
    // (gathered so that LDS holds fragment (mt, t) as [lane][8 halves]).  Where the block lies in the page and in the
    // ring is worked out ONCE per step (step_copies); a copy then costs two scalar adds on top of its load -- worked
    // out per copy it was 30 scalar instructions each, 120 to 145 a step in the instruction stream of a wave whose
    // matrix instructions wait behind them.
    struct StepCopies {
        const char *src;
        unsigned dst;
    };
    unsigned v_src_off[CPW];  // source offsets of this value wave's chunks inside a V block
#pragma unroll
    for (int c = 0; c < CPW; ++c) {
        const int chunk = w4 * CPW + c, mt = chunk >> 1, t = chunk & 1;
        v_src_off[c] = (unsigned)((32 * mt * 4 + 2 * t) * 16);
    }
    auto step_copies = [&](int i, int nb) {  // of step i; nb blocks in the range
        StepCopies sc;
        const int j = value_wave ? i + 2 : i + 4;
        const _Float16 *page = value_wave ? vp : kp;
        sc.src = reinterpret_cast<const char *>(page + (size_t)page_block(source_block(j, nb)) * (32 * D)) + (value_wave ? 0 : w4 * CPW * 1024);
        sc.dst = smem_base + (unsigned)((value_wave ? V_OFF : 0) + ((j + slot_off) & (kBuffers - 1)) * BLOCK_BYTES + w4 * CPW * 1024);
        return sc;
    };
    auto issue_copy = [&](const StepCopies &sc, int c) {  // copy c (0 .. CPW-1)
        if (!value_wave) copy16_global_to_lds(sc.src + c * 1024, k_lane_offset, sc.dst + c * 1024);
        else copy16_global_to_lds(sc.src + v_src_off[c], v_lane_offset, sc.dst + c * 1024);
    };
    auto issue_step = [&](int i, int nb) {
        const StepCopies sc = step_copies(i, nb);
#pragma unroll
        for (int c = 0; c < CPW; ++c) issue_copy(sc, c);
    };

    char *const p_mine = smem + P_OFF + w4 * 2048 + lane * 16;           // + step parity * 8192, + k-step * 1024
    float *const alpha_mine = reinterpret_cast<float *>(smem + ALPHA_OFF) + w4 * 32 + li;  // + step parity * 128
    float *const lsum_mine = reinterpret_cast<float *>(smem + LSUM_OFF) + w4 * 32 + li;

    // Tiles in pairs (tile i with tile n - 1 - i: every workgroup the same number of key blocks under a causal
    // mask from position 0) -- or, where the keys are cut into ranges, one tile each: deep in a context the tiles
    // are equally long anyway, and a workgroup with one tile leaves half the partial results of one with two.
    const int n_passes = (a.single_tiles || pair == a.n_tiles - 1 - pair) ? 1 : 2;
    for (int pass = 0; pass < n_passes; ++pass) {
        // The long tile goes first: the short one then fills in behind it.
        const int tile = a.single_tiles ? pair : (pass == 0 ? a.n_tiles - 1 - pair : pair);
        const int tok = tile * 32 + li;
        const bool valid = tok < a.q_len;
        const int lim = valid ? min(a.kv_valid, a.start + tok + 1) : 0;  // keys [lo, lim) are visible
        const int lo = (a.window > 0 && a.start + tok + 1 > a.window) ? a.start + tok + 1 - a.window : 0;
        // With a window the tile starts at the block of the first key its first row sees; the rows'
        // lower bounds differ, so the blocks up to the one of its last row's bound are masked too.
        const int tile_lo = (a.window > 0 && a.start + tile * 32 + 1 > a.window) ? a.start + tile * 32 + 1 - a.window : 0;
        const int window_block = tile_lo >> 5;
        const int last_lo_block = a.window > 0 ? (tile_lo + 31) >> 5 : -1;
        const int end = min(a.kv_valid, a.start + min(a.q_len, tile * 32 + 32));
        const int nb_tile = (end + 31) >> 5;                   // key blocks this tile needs
        const int mask_from = (a.start + tile * 32 + 1) >> 5;  // first block in which some row is masked by causality
        const int first_masked = min(mask_from, end >> 5);     // ... or cut by the valid length
        // This workgroup's share of them (all, without key splits); local step i is block jb + i.
        jb = a.n_splits > 1 ? split * a.split_blocks : window_block;  // (key splits and windows are not combined)
        const int nb = (a.n_splits > 1 ? min(nb_tile, jb + a.split_blocks) : nb_tile) - jb;
        if (nb <= 0) continue;  // nothing of this tile in the range (the same for every wave)

        if (pass > 0) __syncthreads();  // every wave is done with the previous pass's LDS
        const bool carried = carry_nb > 0;  // this tile's first blocks came in behind the previous tile's last
        carry_nb = 0;
        if (pass == 0 && n_passes == 2 && a.n_splits == 1 && a.window == 0) {
            // the second tile's blocks: keys [0, its last row's position], from block 0
            const int end2 = min(a.kv_valid, a.start + min(a.q_len, pair * 32 + 32));
            carry_nb = max((end2 + 31) >> 5, 0);
        }
        if (!carried) {
#pragma unroll
            for (int i = -4; i < 0; ++i) issue_step(i, nb);  // K blocks 0..3, V blocks 0..1
        }

        // End of step i.  K(i+2) and V(i+1) -- copies of step i-2 -- must have landed: the next
        // step reads them from LDS.  The copies of steps i-1 and i may still fly.  Then the
        // barrier that publishes them and this step's P^T.
        auto end_step = [&]() {
            TT_WAIT_VMCNT(2 * CPW);
            __syncthreads();
        };

        // Step i (0 .. nb + 1): the score waves run the MFMAs of block i, the value waves those of
        // block i - 2; both fetch the NEXT step's fragments from LDS into the registers the
        // MFMAs have just read, so that after the barrier the matrix pipe starts at once.
        // The two roles run separate loops (their register sets are disjoint that way) that
        // meet at the same barriers.
        if (!value_wave) {
            // Query fragments (B operand); rows of padding tokens are zero.
            h8 qf[KS];
            const _Float16 *qp = a.q + (long long)(valid ? tok : 0) * a.q_stride + (long long)head * D + 8 * g;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                const h8 x = *reinterpret_cast<const h8 *>(qp + 16 * s);
                qf[s] = valid ? x : (h8)(_Float16)0;
            }
            float m = kNegBig, l = 0.0f;
            TT_WAIT_VMCNT(0);  // the first stages and the query rows
            __syncthreads();
            h8 kf[KS];
#pragma unroll
            for (int t = 0; t < KS; ++t)
                kf[t] = *reinterpret_cast<const h8 *>(smem + (slot_off & (kBuffers - 1)) * BLOCK_BYTES + lane * 16 + t * 1024);
            __syncthreads();  // every score wave holds K block 0: step 0 may refill its slot
#pragma nounroll
            for (int i = 0; i < nb; ++i) {
                const char *next = smem + ((i + 1 + slot_off) & (kBuffers - 1)) * BLOCK_BYTES + lane * 16;
                const StepCopies sc = step_copies(i, nb);
                f16v s = (f16v)0.0f;
#pragma unroll
                for (int t = 0; t < KS; ++t) {
                    s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[t], qf[t], s, 0, 0, 0);
                    kf[t] = *reinterpret_cast<const h8 *>(next + t * 1024);
                    // this step's copies, one at a time between MFMAs: a burst would stall the wave
                    // on the CU's vector memory path (64 B/clk for all eight waves)
                    if (t % (KS / CPW) == 0) issue_copy(sc, t / (KS / CPW));
                    __builtin_amdgcn_sched_barrier(0);
                }
                h8 pf[2];
                const float alpha = softmax_step(s, jb + i >= first_masked || jb + i <= last_lo_block, (jb + i) << 5, lo, lim, g,
                                                 a.scale_log2e, m, l, pf);
                char *pdst = p_mine + (i & 1) * 8192;
                *reinterpret_cast<h8 *>(pdst) = pf[0];
                *reinterpret_cast<h8 *>(pdst + 1024) = pf[1];
                if (g == 0) alpha_mine[(i & 1) * 128] = alpha;
                end_step();
            }
            issue_step(nb, nb);
            end_step();  // the value waves' last two steps
            issue_step(nb + 1, nb);
            end_step();
            const float lt = sum_across_halves(l);
            if (g == 0) {
                if (a.n_splits > 1) {  // partial: the row's reference max (log2 domain) and sum over this key range
                    float *ml = a.part_ml + ((((size_t)split * a.group * a.n_kv_heads + head) * a.n_tiles + tile) * 32 + li) * 2;
                    ml[0] = m;
                    ml[1] = lt;
                } else {
                    *lsum_mine = lt;
                }
            }
            TT_WAIT_VMCNT(0);
            __syncthreads();
        } else {
            f16v o[MT];
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) o[mt] = (f16v)0.0f;
            TT_WAIT_VMCNT(0);
            __syncthreads();
            __syncthreads();  // (the score waves fetch K block 0 between these two)
            // Two steps behind the score wave: block j's P^T (written in step j) and V fragments are
            // fetched from LDS into registers during step j + 1 and consumed in step j + 2, so
            // that the MFMAs of a step start right after its barrier.
            issue_step(0, nb);
            end_step();  // step 0: the score waves' first
            issue_step(1, nb);
            h8 vf[2 * MT], pf[2];
#pragma unroll
            for (int c = 0; c < 2 * MT; ++c)
                vf[c] = *reinterpret_cast<const h8 *>(smem + V_OFF + (slot_off & (kBuffers - 1)) * BLOCK_BYTES + lane * 16 + c * 1024);
            pf[0] = *reinterpret_cast<const h8 *>(p_mine);
            pf[1] = *reinterpret_cast<const h8 *>(p_mine + 1024);
            float alpha = alpha_mine[0];
            end_step();  // step 1
#pragma nounroll
            for (int i = 2; i <= nb + 1; ++i) {
                const int jn = i - 1;  // the block fetched in this step (past the last one: stale but harmless data)
                const char *next = smem + V_OFF + ((jn + slot_off) & (kBuffers - 1)) * BLOCK_BYTES + lane * 16;
                const char *psrc = p_mine + (jn & 1) * 8192;
                const StepCopies sc = step_copies(i, nb);
                if (__any(alpha != 1.0f)) {
#pragma unroll
                    for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
                }
                h8 pn[2];
                pn[0] = *reinterpret_cast<const h8 *>(psrc);
                pn[1] = *reinterpret_cast<const h8 *>(psrc + 1024);
                alpha = alpha_mine[(jn & 1) * 128];
                // Both k-steps of a 32-dim tile back to back: consecutive MFMAs on one accumulator
                // forward it inside the matrix pipe instead of going through the register file.
#pragma unroll
                for (int c = 0; c < 2 * MT; ++c) {
                    o[c >> 1] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[c], pf[c & 1], o[c >> 1], 0, 0, 0);
                    vf[c] = *reinterpret_cast<const h8 *>(next + c * 1024);
                    if (c % (KS / CPW) == 0) issue_copy(sc, c / (KS / CPW));
                    __builtin_amdgcn_sched_barrier(0);
                }
                pf[0] = pn[0];
                pf[1] = pn[1];
                end_step();
            }
            TT_WAIT_VMCNT(0);
            __syncthreads();  // the row sums are in LDS
            // Lane (li, g), register v of tile mt holds dim 32 mt + 8 (v / 4) + 4 g + v % 4 of row li.
            if (a.n_splits > 1) {
                // Partial: the unnormalised accumulators, for the combine pass.
                float *po = a.part_o + ((((size_t)split * a.group * a.n_kv_heads + head) * a.n_tiles + tile) * 32 + li) * D + 4 * g;
#pragma unroll
                for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                    for (int vq = 0; vq < 4; ++vq) {
                        const f4 x = {o[mt][4 * vq], o[mt][4 * vq + 1], o[mt][4 * vq + 2], o[mt][4 * vq + 3]};
                        *reinterpret_cast<f4 *>(po + 32 * mt + 8 * vq) = x;
                    }
            } else {
                // Epilogue: normalise, gate in fp32, one fp16 round, store.  The rounded values go through LDS, one
                // 32-dim tile of the wave's 32 rows at a time (a region of their own: the rings may already hold the
                // next tile's blocks), so that a store instruction writes 64 contiguous bytes of 16 rows -- 8-byte
                // pieces straight from the accumulator layout took the value waves ~5 us per tile.
                char *const stage = smem + STAGE_OFF + w4 * (32 * STAGE_PITCH);
                const float lt = *lsum_mine;
                const float inv = lt > 0.0f ? 1.0f / lt : 0.0f;
                const _Float16 *gp = a.gate && valid ? a.gate + (long long)tok * a.g_stride + (long long)head * D + 4 * g : nullptr;
                const int out_row = lane >> 2, out_piece = lane & 3;  // a store: lane l writes piece l % 4 of row l / 4 (+ 16)
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
                    for (int vq = 0; vq < 4; ++vq) {
                        const int d = 32 * mt + 8 * vq;
                        float r4[4];
#pragma unroll
                        for (int i = 0; i < 4; ++i) r4[i] = o[mt][4 * vq + i] * inv;
                        if (gp) {
                            const h4 gv = *reinterpret_cast<const h4 *>(gp + d);
#pragma unroll
                            for (int i = 0; i < 4; ++i) r4[i] *= 1.0f / (1.0f + __expf(-(float)gv[i]));
                        }
                        const h4 hv = {(_Float16)r4[0], (_Float16)r4[1], (_Float16)r4[2], (_Float16)r4[3]};
                        *reinterpret_cast<h4 *>(stage + li * STAGE_PITCH + (8 * vq + 4 * g) * 2) = hv;
                    }
#pragma unroll
                    for (int half = 0; half < 2; ++half) {
                        const int row = 16 * half + out_row;
                        const h8 x = *reinterpret_cast<const h8 *>(stage + row * STAGE_PITCH + out_piece * 16);
                        const int t = tile * 32 + row;
                        if (t < a.q_len)
                            *reinterpret_cast<h8 *>(a.out + (long long)t * a.o_stride + (long long)head * D + 32 * mt + out_piece * 8) = x;
                    }
                }
            }
        }
        if (carry_nb > 0) slot_off = (slot_off + nb) & (kBuffers - 1);  // where the next tile's block 0 sits
    }
}


// The kernel wants 4 q heads per KV head in a workgroup and 16-byte aligned rows; anything
// else is served by the split-K kernel.
bool prefill_kernel_serves(int n_q_heads, int n_kv_heads, int head_dim, bool aligned) {
    const int group = n_q_heads / n_kv_heads;
    return aligned && group % 4 == 0 && (head_dim == 256 || head_dim == 128 || head_dim == 64);
}

// four K+V stages (128 KiB at D = 256) + P^T hand-over (16 KiB) + rescale factors and row sums + the output rows' staging (10 KiB)
static constexpr int prefill_lds_bytes(int D) { return kBuffers * 2 * 32 * D * 2 + 2 * 4 * 2048 + 2 * 4 * 128 + 4 * 128 + 4 * 32 * 80; }

int configure_prefill_kernels(tt_hip_ctx *ctx) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_kernel<256>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, prefill_lds_bytes(256));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_kernel<128>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, prefill_lds_bytes(128));
    if (e == hipSuccess)
        e = hipFuncSetAttribute(reinterpret_cast<const void *>(attn_prefill_kernel<64>),
                                hipFuncAttributeMaxDynamicSharedMemorySize, prefill_lds_bytes(64));
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "hipFuncSetAttribute(chunk kernel max dynamic LDS)");
}

template <int D>
static int launch_prefill_d(tt_hip_ctx *ctx, const PrefillArgs &args, unsigned grid) {
    constexpr int lds = prefill_lds_bytes(D);
    auto kernel = attn_prefill_kernel<D>;  // (its LDS limit was raised when the first context on this device was created)
    launch_profiled(ctx, kernel, dim3(grid), dim3(512), (unsigned)lds, args);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "attn_prefill_kernel launch");
}

int launch_prefill(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start, int q_len, int kv_valid,
                   int n_q_heads, const tt_half *q, long long q_stride, const tt_half *gate, long long g_stride,
                   float scale, tt_half *out, long long o_stride, int n_splits, int split_blocks, float *part_o,
                   float *part_ml, const PageSource *pages, int window) {
    PrefillArgs a{};
    if (window > 0 && n_splits > 1) return TT_HIP_ERR_INVALID_ARGUMENT;  // key ranges start at key 0
    a.window = window;
    if (!pages && kv->bits != 16) return TT_HIP_ERR_INVALID_ARGUMENT;  // this kernel reads fp16 pages only
    const size_t slot_off = (size_t)slot * kv->n_kv_heads * kv->page_elems();
    a.k_slot = pages ? pages->k : kv->k[layer] + slot_off;
    a.v_slot = pages ? pages->v : kv->v[layer] + slot_off;
    a.q = reinterpret_cast<const _Float16 *>(q);
    a.gate = reinterpret_cast<const _Float16 *>(gate);
    a.out = reinterpret_cast<_Float16 *>(out);
    a.page_elems = pages ? pages->page_elems : (long long)kv->page_elems();
    a.ring_blocks = pages ? pages->ring_blocks : kv->ring_blocks();
    a.q_stride = q_stride;
    a.g_stride = g_stride;
    a.o_stride = o_stride;
    a.group = n_q_heads / kv->n_kv_heads;
    a.hsubs = a.group / 4;
    a.n_tiles = (q_len + 31) / 32;
    a.single_tiles = n_splits > 1 ? 1 : 0;
    a.n_pairs = a.single_tiles ? a.n_tiles : (a.n_tiles + 1) / 2;
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
    a.base_grid = (int)grid;
    a.n_splits = n_splits > 1 ? n_splits : 1;
    a.split_blocks = split_blocks;
    a.part_o = part_o;
    a.part_ml = part_ml;
    if (a.n_splits > 1 && (!part_o || !part_ml || split_blocks <= 0)) return TT_HIP_ERR_INVALID_ARGUMENT;
    grid *= (unsigned)a.n_splits;
    a.xcd_chunk = 0;
    if (a.n_splits > 1 && a.xs > 0) {
        a.xcd_chunk = (a.per_kvh * a.n_splits + a.xs - 1) / a.xs;
        grid = 8u * (unsigned)a.xcd_chunk;
    }
    switch (kv->head_dim) {
        case 256: return launch_prefill_d<256>(ctx, a, grid);
        case 128: return launch_prefill_d<128>(ctx, a, grid);
        case 64: return launch_prefill_d<64>(ctx, a, grid);
        default: return TT_HIP_ERR_SHAPE;
    }
}

}  // namespace tt
