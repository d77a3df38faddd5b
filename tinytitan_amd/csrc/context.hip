// Context, error reporting, timing and the three attention entry points of the C ABI.
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <new>

#include "internal.h"

// Split-K partials of tt_hip_attn_decode_noalloc, the entry point for callers that cannot allocate: a fixed
// array in the library's own device image instead of the context's grown-on-demand buffers.  Every GPU the
// library runs on holds its own copy (33 MiB) at its own address until the process ends; host code reaches it
// only through the address hipGetSymbolAddress returns on that device (kept per context), never by this name.
// Layout: [kStaticPartialRows][256] floats of unnormalised O, then [kStaticPartialRows][2] floats of (max, sum).
static __device__ __align__(256) float scratch[tt::kStaticPartialRows * (256 + 2)];

namespace tt {

int hip_fail(tt_hip_ctx *ctx, hipError_t err, const char *what) {
    if (ctx) {
        ctx->last_hip_error = std::string(what) + ": " + hipGetErrorString(err);
    }
    (void)hipGetLastError();  // clear the sticky per-thread error
    return err == hipErrorOutOfMemory ? TT_HIP_ERR_OUT_OF_MEMORY : TT_HIP_ERR_HIP;
}

int ensure_partials(tt_hip_ctx *ctx, size_t rows, int head_dim) {
    // Sized for head_dim 256 so that a context serves every supported head_dim.
    (void)head_dim;
    if (rows <= ctx->part_rows) return TT_HIP_OK;
    if (ctx->capturing) return TT_HIP_ERR_BUSY;  // growing would synchronise and allocate inside a capture
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    if (ctx->part_o) (void)hipFree(ctx->part_o);
    if (ctx->part_ml) (void)hipFree(ctx->part_ml);
    ctx->part_o = nullptr;
    ctx->part_ml = nullptr;
    ctx->part_rows = 0;
    ++ctx->generation;
    size_t want = rows + rows / 4;
    e = hipMalloc(reinterpret_cast<void **>(&ctx->part_o), want * 256 * sizeof(float));
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMalloc(split partial O)");
    e = hipMalloc(reinterpret_cast<void **>(&ctx->part_ml), want * 2 * sizeof(float));
    if (e != hipSuccess) {
        (void)hipFree(ctx->part_o);
        ctx->part_o = nullptr;
        return hip_fail(ctx, e, "hipMalloc(split partial m/l)");
    }
    ctx->part_rows = want;
    return TT_HIP_OK;
}

int ensure_stage(tt_hip_ctx *ctx, size_t elems) {
    if (elems <= ctx->stage_elems) return TT_HIP_OK;
    if (ctx->capturing) return TT_HIP_ERR_BUSY;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    if (ctx->stage_k) (void)hipFree(ctx->stage_k);
    if (ctx->stage_v) (void)hipFree(ctx->stage_v);
    ctx->stage_k = ctx->stage_v = nullptr;
    ctx->stage_elems = 0;
    ++ctx->generation;
    const size_t want = elems + elems / 4;
    e = hipMalloc(reinterpret_cast<void **>(&ctx->stage_k), want * sizeof(_Float16));
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMalloc(dequantised K pages)");
    e = hipMalloc(reinterpret_cast<void **>(&ctx->stage_v), want * sizeof(_Float16));
    if (e != hipSuccess) {
        (void)hipFree(ctx->stage_k);
        ctx->stage_k = nullptr;
        return hip_fail(ctx, e, "hipMalloc(dequantised V pages)");
    }
    ctx->stage_elems = want;
    return TT_HIP_OK;
}

// Rows of selection bytes for a chunk whose selection arrives as index lists.
static int ensure_keep_rows(tt_hip_ctx *ctx, size_t bytes) {
    if (bytes <= ctx->keep_rows_bytes) return TT_HIP_OK;
    if (ctx->capturing) return TT_HIP_ERR_BUSY;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    if (ctx->keep_rows) (void)hipFree(ctx->keep_rows);
    ctx->keep_rows = nullptr;
    ctx->keep_rows_bytes = 0;
    ++ctx->generation;
    const size_t want = bytes + bytes / 4;
    e = hipMalloc(reinterpret_cast<void **>(&ctx->keep_rows), want);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipMalloc(selection rows)");
    ctx->keep_rows_bytes = want;
    return TT_HIP_OK;
}

// One workgroup per query row: clear the row's bytes, then set the byte of every listed key the row can see
// (key < min(kv_valid, start + row + 1), as the reference's kernel tests each list entry).  The row stride is a
// multiple of 16 bytes.
__global__ __launch_bounds__(256) void keep_rows_from_indices_kernel(uint8_t *rows, unsigned row_stride, const uint32_t *indices,
                                                                     unsigned index_stride, const uint32_t *counts, int start,
                                                                     int kv_valid) {
    const unsigned row = blockIdx.x;
    uint8_t *mine = rows + (size_t)row * row_stride;
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    for (unsigned at = threadIdx.x * 16u; at < row_stride; at += 256u * 16u) *reinterpret_cast<u4 *>(mine + at) = (u4)0u;
    __syncthreads();
    const unsigned limit = (unsigned)min(kv_valid, start + (int)row + 1);
    const unsigned count = min(counts[row], index_stride);
    const uint32_t *list = indices + (size_t)row * index_stride;
    for (unsigned i = threadIdx.x; i < count; i += 256u) {
        const unsigned key = list[i];
        if (key < limit) mine[key] = 1;
    }
}

// A chunk's per-query index lists (keepIdx[t * stride + i], i < keepCount[t]; the reference's tiled chunk kernel walks
// them entry by entry, sources/TinyTitanCore/Metal/Prefill/prefill.metal:1069-1117) turned into what a tile of `tt`
// tokens walks here: the ascending list of the 32-key blocks that hold a listed key some token of the tile can see
// (key < min(kv_valid, start + row + 1), the reference's test of each entry), where every key range of `split_blocks`
// blocks starts in that list, and per entry and token the listed keys of the block as 32 bits.  One workgroup per
// token tile; its work is the tile's list entries plus one pass over a bitmap of the context's blocks in LDS (a bit
// per block: 4 KiB per million keys) -- nothing of the order rows x context is written or read.  Entries may come in
// any order and repeat: a bit is set once.
// LDS: bitmap[W], prefix[W], partial[kPlanThreads + 1], chunk[chunk_entries * tt] words, W = ceil(ceil(kv_valid / 32) / 32).
constexpr int kPlanThreads = 1024;  // sixteen wavefronts: the walks are chains of dependent scalar work that only other wavefronts hide
__global__ __launch_bounds__(kPlanThreads) void keep_plan_kernel(const uint32_t *indices, unsigned index_stride, const uint32_t *counts,
                                                                 int start, int q_len, int kv_valid, int tt, int split_blocks,
                                                                 int n_splits, int cap, int chunk_entries, int *ranges, int *blocks,
                                                                 unsigned *bits) {
    constexpr int T = kPlanThreads;
    extern __shared__ unsigned plan_lds[];
    const int tile = blockIdx.x, tid = threadIdx.x;
    const int ctx_blocks = (kv_valid + 31) >> 5, W = (ctx_blocks + 31) >> 5;
    unsigned *bitmap = plan_lds, *prefix = plan_lds + W, *partial = plan_lds + 2 * W;
    const int rows = min(tt, q_len - tile * tt);
    // The tile's lists as one run of rows * index_stride places, every thread a run of `per` neighbouring ones (so
    // that the lanes of a wavefront work on entries far apart, which seldom meet in one word of LDS: the entries of a
    // sorted list that 64 neighbouring lanes hold fall into a handful of words, and their atomics queue up).  A
    // thread's first kHeld places are asked for at once, beside the rows' counts and ahead of everything else, and
    // stay in registers for both walks over the lists: one trip to memory for a tile of the usual size.  Places
    // beyond them are read again per walk, kBatch at a time.
    constexpr unsigned kHeld = 16, kBatch = 8;
    const uint32_t *lists = indices + (size_t)tile * tt * index_stride;
    const unsigned places = (unsigned)rows * index_stride, per = (places + T - 1u) / T, mine = (unsigned)tid * per;
    unsigned my_count = tid < rows ? min(counts[tile * tt + tid], index_stride) : 0u;
    unsigned held[kHeld];
#pragma unroll
    for (unsigned j = 0; j < kHeld; ++j) held[j] = lists[min(mine + j, places - 1u)];
    for (int w = tid; w < W; w += T) bitmap[w] = 0u;
    unsigned *row_counts = partial;  // (the scan's words: free until the bitmap is complete; tt <= 32)
    if (tid < rows) row_counts[tid] = my_count;
    __syncthreads();
    const unsigned row0 = min(mine, places - 1u) / index_stride;  // (the one division: a run's places are walked in order)
    auto for_listed_keys = [&](auto &&use) {  // use(key, row): every listed key that its row can see, in list order
        unsigned r = row0, i = mine - row0 * index_stride;  // the place in hand: entry i of the tile's row r
        unsigned count = row_counts[min(r, (unsigned)rows - 1u)], limit = (unsigned)min(kv_valid, start + tile * tt + (int)r + 1);
        auto place = [&](unsigned j, unsigned key) {
            if (j < per && r < (unsigned)rows && i < count && key < limit) use(key, r);
            if (++i == index_stride) {
                i = 0u;
                ++r;
                count = row_counts[min(r, (unsigned)rows - 1u)];
                limit = (unsigned)min(kv_valid, start + tile * tt + (int)r + 1);
            }
        };
#pragma unroll
        for (unsigned j = 0; j < kHeld; ++j) place(j, held[j]);
        for (unsigned base = kHeld; base < per; base += kBatch) {
            unsigned keys[kBatch];
#pragma unroll
            for (unsigned j = 0; j < kBatch; ++j) keys[j] = lists[min(mine + base + j, places - 1u)];
#pragma unroll
            for (unsigned j = 0; j < kBatch; ++j) place(base + j, keys[j]);
        }
    };
    for_listed_keys([&](unsigned key, unsigned) { atomicOr(&bitmap[key >> 10], 1u << ((key >> 5) & 31u)); });
    __syncthreads();  // (the scan takes the counts' words over: they are put back from my_count for the second walk)
    // exclusive prefix sums of the words' bit counts: a run of words per thread, a scan of the threads' runs inside
    // each wavefront by shuffles, the wavefronts' totals through LDS
    const int per_thread = (W + T - 1) / T, w_begin = tid * per_thread, w_end = min(W, w_begin + per_thread);
    unsigned run = 0;
    for (int w = w_begin; w < w_end; ++w) run += __popc(bitmap[w]);
    unsigned inclusive = run;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
        const unsigned below = __shfl_up(inclusive, off);
        if ((tid & 63) >= off) inclusive += below;
    }
    if ((tid & 63) == 63) partial[tid >> 6] = inclusive;
    __syncthreads();
    unsigned before = 0;
    for (int w = 0; w < (tid >> 6); ++w) before += partial[w];
    if (tid == T - 1) partial[T] = before + inclusive;
    run = before + inclusive - run;
    for (int w = w_begin; w < w_end; ++w) {
        prefix[w] = run;
        run += __popc(bitmap[w]);
    }
    __syncthreads();
    const int n_touched = (int)partial[T];  // at most min(ctx_blocks, listed entries) <= cap
    int *my_blocks = blocks + (size_t)tile * cap;
    for (int w = tid; w < W; w += T) {
        unsigned word = bitmap[w];
        int at = (int)prefix[w];
        while (word) {
            my_blocks[at++] = w * 32 + (__ffs((int)word) - 1);
            word &= word - 1u;
        }
    }
    for (int s = tid; s <= n_splits; s += T) {
        const long long first = (long long)s * split_blocks;
        int at = n_touched;
        if (first < ctx_blocks) at = (int)(prefix[first >> 5] + __popc(bitmap[first >> 5] & ((1u << (first & 31)) - 1u)));
        ranges[(size_t)tile * (n_splits + 1) + s] = at;
    }
    // The bits, a run of `chunk_entries` list entries at a time: gathered in LDS (atomics there cost a few cycles; in
    // global memory every listed key would be a request of its own to L2, ~8 cycles each and 32 us for a tile's 8,000
    // keys), then written out side by side.
    unsigned *my_bits = bits + (size_t)tile * cap * tt;
    unsigned *chunk = plan_lds + 2 * W + T + 1;  // chunk_entries * tt words
    if (tid < rows) row_counts[tid] = my_count;
    for (int first = 0; first < n_touched; first += chunk_entries) {
        const int here = min(chunk_entries, n_touched - first);
        __syncthreads();  // (the counts are back in their words; the previous run has been written out)
        for (int i = tid; i < here * tt; i += T) chunk[i] = 0u;
        __syncthreads();
        for_listed_keys([&](unsigned key, unsigned r) {
            const unsigned w = key >> 10, bit = (key >> 5) & 31u;
            const int rank = (int)(prefix[w] + __popc(bitmap[w] & ((1u << bit) - 1u))) - first;
            if (rank >= 0 && rank < here) atomicOr(&chunk[rank * tt + (int)r], 1u << (key & 31u));
        });
        __syncthreads();
        for (int i = tid; i < here * tt; i += T) my_bits[(size_t)first * tt + i] = chunk[i];
    }
}

// A plain streaming read, the control the decode pass is measured against: one workgroup per CU walks its own
// contiguous share, every thread keeping 16 loads of 16 bytes in flight (64 KiB per workgroup and turn), and
// folds what it read into one word that is stored only if it equals a value it cannot have.
typedef unsigned u4 __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(256) void calibrate_read_kernel(const u4 *src, unsigned turns, unsigned *sink) {
    const u4 *p = src + (size_t)blockIdx.x * turns * 4096 + threadIdx.x;
    u4 acc = {0u, 0u, 0u, 0u};
    for (unsigned t = 0; t < turns; ++t) {
        u4 x[16];
#pragma unroll
        for (int i = 0; i < 16; ++i) x[i] = __builtin_nontemporal_load(p + (size_t)t * 4096 + i * 256);
#pragma unroll
        for (int i = 0; i < 16; ++i) acc ^= x[i];
    }
    const unsigned folded = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
    if (folded == 0x9e3779b9u && sink) sink[0] = folded + threadIdx.x;  // practically never: keeps the loads alive
}

static bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

// A per-call table of one int per sequence: on the stack for the batch sizes a step has (the decode entry points
// are called once per layer and token and should not touch the heap), on the heap beyond that.
struct IntTable {
    explicit IntTable(int n) {
        if (n > kInline) {
            heap.resize((size_t)n);
            ints = heap.data();
        }
    }
    int *data() { return ints; }
    int &operator[](int i) { return ints[i]; }

private:
    static constexpr int kInline = 64;
    int inline_ints[kInline];
    std::vector<int> heap;
    int *ints = inline_ints;
};

// A chunk's selection as per-query index lists (one sequence): indices[row * stride + i], i < counts[row].
struct KeepLists {
    const uint32_t *indices;
    size_t stride;
    const uint32_t *counts;
};

// Shared body of decode / verify / prefill.
//   kind 0: rows query tokens per sequence, GQA-packed tiles, split-K.
//   kind 1: causal chunk of one sequence.
//   chunk_splits > 1 (kind 1, one sequence): the chunk kernel over chunk_splits key ranges of
//   chunk_split_blocks blocks, then the combine pass.
static int run_attention(tt_hip_ctx *ctx, tt_hip_kv *kv, int kind, int layer, int n_seq, const int *slots,
                         const int *starts, const int *totals, int rows, int n_q_heads, const tt_half *q,
                         long long q_seq_stride, long long q_tok_stride, const tt_half *gate, long long g_seq_stride,
                         long long g_tok_stride, float scale, tt_half *out, long long o_seq_stride,
                         long long o_tok_stride, int chunk_splits = 1, int chunk_split_blocks = 0,
                         const PageSource *pages = nullptr, int window = 0, const uint8_t *keep = nullptr,
                         long long keep_seq_stride = 0, long long keep_row_stride = 0, bool static_partials = false,
                         const KeepLists *lists = nullptr) {
    const int D = kv->head_dim;
    hipError_t e = hipSetDevice(ctx->device);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipSetDevice");
    for (int base = 0; base < n_seq; base += kMaxSeqPerLaunch) {
        const int n = n_seq - base < kMaxSeqPerLaunch ? n_seq - base : kMaxSeqPerLaunch;
        long long total_keys = 0;
        int max_keys = 0, min_keys = totals[base];
        // Keys a tile walks: all of them, or with a sliding window at most the window, the tile's
        // rows and the partial block in front.
        auto walked = [&](int i) {
            const long long reach = (long long)window + rows + 32;
            return window > 0 && totals[base + i] > reach ? (int)reach : totals[base + i];
        };
        min_keys = walked(0);
        for (int i = 0; i < n; ++i) {
            total_keys += walked(i);
            if (walked(i) > max_keys) max_keys = walked(i);
            if (walked(i) < min_keys) min_keys = walked(i);
        }
        LaunchPlan plan;
        const bool small_tiles_ok = kind == 0 && !keep && !lists && chunk_splits <= 1 && !pages;
        int st = plan_launch(ctx, kind, n, n_q_heads, kv->n_kv_heads, D, rows, total_keys, min_keys, max_keys, &plan, kv->bits,
                             small_tiles_ok);
        if (st != TT_HIP_OK) return st;
        if (chunk_splits > 1) {  // the chunk kernel's geometry: 32-row one-head tiles, its own key ranges
            plan.split_len = chunk_split_blocks * 32;
            plan.n_splits_max = chunk_splits;
        }
        // One selection per sequence: a wavefront keeps the blocks it still has to work on as one 64-bit word, at
        // most 64 per split.  One per query row: as a list, of at most kKeepWindows such words.
        const int keep_blocks = keep_row_stride > 0 ? 64 * kKeepWindows : 64;
        if (keep && plan.split_len > keep_blocks * plan.waves * 32) {
            plan.split_len = keep_blocks * plan.waves * 32;
            plan.n_splits_max = (max_keys + plan.split_len - 1) / plan.split_len;
            plan.workgroups = (long long)plan.n_splits_max * plan.n_tiles * n;
        }
        // A chunk's token tiles over several key ranges: workgroups that share an XCD share the K/V blocks of a range.
        plan.xcd_grid = ctx->xcd_grid && chunk_splits <= 1 && plan.tok_tiles > 1 && plan.n_splits_max > 1;
        // Pages that the launch reads once -- one tile per KV head, as in a decode step or a verify pass of a few
        // rows -- are loaded non-temporal once there are enough of them that they would not survive in the
        // 256 MiB memory-side cache until the same layer's next step anyway (16 MiB a launch: sixteen layers of it).
        {
            const long long kv_bytes = total_keys * (long long)kv->n_kv_heads * (long long)(kv->block_bytes() / kBlockTokens) * 2;
            plan.stream = plan.tok_tiles == 1 && plan.hsubs == 1 && chunk_splits <= 1 && keep_row_stride == 0 &&
                          (ctx->stream_override < 0 ? kv_bytes >= (16ll << 20) : ctx->stream_override != 0);
        }
        // A sequence's splits: what its own keys need (at least one), packed one sequence after the other.
        int first_split[kMaxSeqPerLaunch];
        size_t total_splits = 0;
        for (int i = 0; i < n; ++i) {
            first_split[i] = (int)total_splits;
            const int mine = chunk_splits > 1 ? chunk_splits : (walked(i) + plan.split_len - 1) / plan.split_len;
            total_splits += (size_t)(mine < 1 ? 1 : mine);
        }
        if (plan.n_splits_max > 1) {
            const size_t part_rows = total_splits * plan.n_tiles * plan.nt;
            if (static_partials) {
                if (part_rows > kStaticPartialRows) return TT_HIP_ERR_SCRATCH;
            } else {
                st = ensure_partials(ctx, part_rows, D);
                if (st != TT_HIP_OK) return st;
            }
        }
        SplitKArgs a;
        std::memset(&a, 0, sizeof(a));
        SplitKHot &h = a.hot;
        h.k_layer = kv->k[layer];
        h.v_layer = kv->v[layer];
        h.q = reinterpret_cast<const _Float16 *>(q) + base * q_seq_stride;
        a.gate = gate ? reinterpret_cast<const _Float16 *>(gate) + base * g_seq_stride : nullptr;
        a.out = reinterpret_cast<_Float16 *>(out) + base * o_seq_stride;
        h.part_o = static_partials ? ctx->static_scratch : ctx->part_o;
        h.part_ml = static_partials ? ctx->static_scratch + kStaticPartialRows * 256 : ctx->part_ml;
        h.page_elems = (long long)kv->page_elems();
        h.q_seq_stride = q_seq_stride;
        h.q_tok_stride = q_tok_stride;
        a.g_seq_stride = g_seq_stride;
        a.g_tok_stride = g_tok_stride;
        a.o_seq_stride = o_seq_stride;
        a.o_tok_stride = o_tok_stride;
        h.n_kv_heads = kv->n_kv_heads;
        h.group = n_q_heads / kv->n_kv_heads;
        h.rows = rows;
        h.gh = plan.gh;
        h.gh_inv = (65536 + plan.gh - 1) / plan.gh;
        h.tt = plan.tt;
        h.hsubs = plan.hsubs;
        h.tok_tiles = plan.tok_tiles;
        h.n_tiles = plan.n_tiles;
        h.split_len = plan.split_len;
        h.n_splits_max = plan.n_splits_max;
        const bool aligned = aligned16(h.q) && aligned16(a.out) && (!a.gate || aligned16(a.gate)) && q_seq_stride % 8 == 0 &&
                             q_tok_stride % 8 == 0 && g_seq_stride % 8 == 0 && g_tok_stride % 8 == 0 && o_seq_stride % 8 == 0 &&
                             o_tok_stride % 8 == 0;
        h.flags = (aligned ? kHotAligned : 0) | (plan.xcd_grid ? kHotXcdGrid : 0);
        h.scale_log2e = scale * 1.4426950408889634f;
        h.window = window;
        h.ring_blocks = kv->ring_blocks();
        a.keep = keep ? keep + base * keep_seq_stride : nullptr;
        a.keep_seq_stride = keep_seq_stride;
        a.keep_row_stride = keep_row_stride;
        // Finding a wavefront's touched blocks up front costs a round of loads in front of its first block: worth it
        // from about eight blocks a wavefront on (below that the block-by-block test with void loads is faster).
        // (Per-query rows are always word-aligned: the entry point requires it.)
        h.keep_words = a.keep && (uintptr_t)a.keep % 4 == 0 && keep_seq_stride % 4 == 0 && plan.split_len >= 8 * plan.waves * 32;
        for (int i = 0; i < n; ++i) {
            a.seq[i].slot = slots[base + i];
            a.seq[i].start = starts[base + i];
            a.seq[i].total = totals[base + i];
            a.seq[i].first_split = first_split[i];
        }
        if (lists) {
            // The lists' plan, in the context's selection store: [tile][n_splits + 1] range starts, [tile][cap] blocks,
            // [tile][cap][tt] bits; a tile's list cannot be longer than the context's blocks or its tokens' entries.
            const int ctx_blocks = (totals[base] + 31) / 32;
            const long long entries = (long long)plan.tt * (long long)lists->stride;
            const int cap = (int)(entries < ctx_blocks ? entries : ctx_blocks) > 0 ? (int)(entries < ctx_blocks ? entries : ctx_blocks) : 1;
            const size_t n_ranges = (size_t)plan.tok_tiles * (plan.n_splits_max + 1), n_blocks = (size_t)plan.tok_tiles * cap;
            st = ensure_keep_rows(ctx, (n_ranges + n_blocks + n_blocks * plan.tt) * sizeof(int));
            if (st != TT_HIP_OK) return st;
            int *ranges = reinterpret_cast<int *>(ctx->keep_rows);
            int *blocks = ranges + n_ranges;
            unsigned *bits = reinterpret_cast<unsigned *>(blocks + n_blocks);
            // LDS of the plan kernel: two words per 1,024 keys of context and the run of bits it gathers at a time, 32 KiB
            // of them or what the context's bitmap leaves of 64 KiB.
            const int words = (ctx_blocks + 31) / 32;
            int chunk_words = (65536 / 4) - (2 * words + kPlanThreads + 1);
            if (chunk_words > 8192) chunk_words = 8192;
            const int chunk_entries = chunk_words / plan.tt;
            if (chunk_entries < 1) return TT_HIP_ERR_CAPACITY;
            hipLaunchKernelGGL(keep_plan_kernel, dim3((unsigned)plan.tok_tiles), dim3(kPlanThreads),
                               (size_t)(2 * words + kPlanThreads + 1 + chunk_entries * plan.tt) * sizeof(unsigned), ctx->stream, lists->indices,
                               (unsigned)lists->stride, lists->counts, starts[base], rows, totals[base], plan.tt, plan.split_len / 32,
                               plan.n_splits_max, cap, chunk_entries, ranges, blocks, bits);
            e = hipGetLastError();
            if (e != hipSuccess) return hip_fail(ctx, e, "keep_plan_kernel launch");
            a.plan_ranges = ranges;
            a.plan_blocks = blocks;
            a.plan_bits = bits;
            a.plan_cap = cap;
        }
        if (chunk_splits > 1) {
            st = launch_prefill(ctx, kv, layer, slots[base], starts[base], rows, totals[base], n_q_heads, q, q_tok_stride, gate,
                                g_tok_stride, scale, out, o_tok_stride, chunk_splits, chunk_split_blocks, ctx->part_o,
                                ctx->part_ml, pages);
            if (st == TT_HIP_OK) st = launch_combine(ctx, plan, D, n, a);
        } else {
            st = launch_splitk(ctx, plan, D, n, a, kv->bits);
        }
        if (st != TT_HIP_OK) return st;
    }
    return TT_HIP_OK;
}

}  // namespace tt

using namespace tt;

extern "C" {

tt_hip_ctx *tt_hip_ctx_create(int device, int *out_err) {
    auto fail = [&](int code) -> tt_hip_ctx * {
        if (out_err) *out_err = code;
        return nullptr;
    };
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || device < 0 || device >= count) {
        (void)hipGetLastError();
        return fail(TT_HIP_ERR_NO_DEVICE);
    }
    hipDeviceProp_t prop;
    if (hipGetDeviceProperties(&prop, device) != hipSuccess) return fail(TT_HIP_ERR_HIP);
    if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0) return fail(TT_HIP_ERR_NO_DEVICE);
    if (hipSetDevice(device) != hipSuccess) return fail(TT_HIP_ERR_HIP);
    tt_hip_ctx *ctx = new (std::nothrow) tt_hip_ctx();
    if (!ctx) return fail(TT_HIP_ERR_OUT_OF_MEMORY);
    ctx->device = device;
    ctx->n_cus = prop.multiProcessorCount > 0 ? prop.multiProcessorCount : 256;
    if (hipStreamCreateWithFlags(&ctx->own_stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreate(&ctx->ev_begin) != hipSuccess || hipEventCreate(&ctx->ev_end) != hipSuccess) {
        tt_hip_ctx_destroy(ctx);
        return fail(TT_HIP_ERR_HIP);
    }
    ctx->stream = ctx->own_stream;
    // This device's copy of the static scratch array (the device is current).
    if (hipGetSymbolAddress(reinterpret_cast<void **>(&ctx->static_scratch), HIP_SYMBOL(scratch)) != hipSuccess ||
        !ctx->static_scratch) {
        (void)hipGetLastError();
        tt_hip_ctx_destroy(ctx);
        return fail(TT_HIP_ERR_HIP);
    }
    // The kernels' dynamic-LDS limits are properties of the device's copy of the code: set by the first context
    // on a device, found set by every later one.
    static std::mutex configured_lock;
    static bool configured[64] = {};
    {
        std::lock_guard<std::mutex> hold(configured_lock);
        if (device >= 64 || !configured[device]) {
            int st = configure_splitk_kernels(ctx);
            if (st == TT_HIP_OK) st = configure_prefill_kernels(ctx);
            if (st == TT_HIP_OK) st = configure_affine_kernels(ctx);
            if (st != TT_HIP_OK) {
                tt_hip_ctx_destroy(ctx);
                return fail(st);
            }
            if (device < 64) configured[device] = true;
        }
    }
    if (out_err) *out_err = TT_HIP_OK;
    return ctx;
}

void tt_hip_ctx_destroy(tt_hip_ctx *ctx) {
    if (!ctx) return;
    (void)hipSetDevice(ctx->device);
    (void)hipStreamSynchronize(ctx->stream);  // (null: the default stream)
    if (ctx->part_o) (void)hipFree(ctx->part_o);
    if (ctx->part_ml) (void)hipFree(ctx->part_ml);
    if (ctx->stage_k) (void)hipFree(ctx->stage_k);
    if (ctx->stage_v) (void)hipFree(ctx->stage_v);
    if (ctx->select_ws) (void)hipFree(ctx->select_ws);
    if (ctx->keep_rows) (void)hipFree(ctx->keep_rows);
    for (hipEvent_t ev : ctx->prof_events) (void)hipEventDestroy(ev);
    if (ctx->ev_begin) (void)hipEventDestroy(ctx->ev_begin);
    if (ctx->ev_end) (void)hipEventDestroy(ctx->ev_end);
    if (ctx->own_stream) (void)hipStreamDestroy(ctx->own_stream);
    delete ctx;
}

int tt_hip_ctx_set_stream(tt_hip_ctx *ctx, void *hip_stream) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    ctx->stream = hip_stream ? reinterpret_cast<hipStream_t>(hip_stream) : ctx->own_stream;
    return TT_HIP_OK;
}

int tt_hip_ctx_set_default_stream(tt_hip_ctx *ctx) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    ctx->stream = nullptr;  // the legacy default stream
    return TT_HIP_OK;
}

void *tt_hip_ctx_stream(tt_hip_ctx *ctx) { return ctx ? reinterpret_cast<void *>(ctx->stream) : nullptr; }

int tt_hip_sync(tt_hip_ctx *ctx) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "hipStreamSynchronize");
}

int tt_hip_timer_begin(tt_hip_ctx *ctx) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    hipError_t e = hipEventRecord(ctx->ev_begin, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventRecord");
    ctx->timer_open = true;
    return TT_HIP_OK;
}

int tt_hip_timer_end(tt_hip_ctx *ctx, uint64_t *out_ns) {
    if (!ctx || !out_ns || !ctx->timer_open) return TT_HIP_ERR_INVALID_ARGUMENT;
    ctx->timer_open = false;
    hipError_t e = hipEventRecord(ctx->ev_end, ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventRecord");
    e = hipEventSynchronize(ctx->ev_end);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventSynchronize");
    float ms = 0.0f;
    e = hipEventElapsedTime(&ms, ctx->ev_begin, ctx->ev_end);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipEventElapsedTime");
    *out_ns = (uint64_t)((double)ms * 1.0e6);
    return TT_HIP_OK;
}

int tt_hip_profile_enable(tt_hip_ctx *ctx, int max_launches) {
    if (!ctx || max_launches <= 0 || max_launches > (1 << 20)) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    while (ctx->prof_events.size() < (size_t)max_launches * 2) {
        hipEvent_t ev = nullptr;
        hipError_t e = hipEventCreate(&ev);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipEventCreate");
        ctx->prof_events.push_back(ev);
    }
    // Calibrate: an empty event pair on the idle stream.
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    float best = -1.0f;
    for (int i = 0; i < 16; ++i) {
        (void)hipEventRecord(ctx->prof_events[0], ctx->stream);
        (void)hipEventRecord(ctx->prof_events[1], ctx->stream);
        e = hipEventSynchronize(ctx->prof_events[1]);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipEventSynchronize");
        float ms = 0.0f;
        if (hipEventElapsedTime(&ms, ctx->prof_events[0], ctx->prof_events[1]) == hipSuccess && (best < 0.0f || ms < best))
            best = ms;
    }
    ctx->prof_overhead_ns = best > 0.0f ? (uint64_t)((double)best * 1.0e6) : 0;
    ctx->prof_used = 0;
    ctx->profiling = true;
    return TT_HIP_OK;
}

int tt_hip_profile_event_overhead_ns(tt_hip_ctx *ctx, uint64_t *out_ns) {
    if (!ctx || !out_ns) return TT_HIP_ERR_INVALID_ARGUMENT;
    *out_ns = ctx->prof_overhead_ns;
    return TT_HIP_OK;
}

int tt_hip_profile_disable(tt_hip_ctx *ctx) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    ctx->profiling = false;
    return TT_HIP_OK;
}

int tt_hip_profile_read(tt_hip_ctx *ctx, int *out_launches, uint64_t *out_total_ns) {
    if (!ctx || !out_launches || !out_total_ns) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    hipError_t e = hipStreamSynchronize(ctx->stream);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamSynchronize");
    double total_ms = 0.0;
    for (size_t i = 0; i + 1 < ctx->prof_used; i += 2) {
        float ms = 0.0f;
        e = hipEventElapsedTime(&ms, ctx->prof_events[i], ctx->prof_events[i + 1]);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipEventElapsedTime");
        total_ms += ms;
    }
    *out_launches = (int)(ctx->prof_used / 2);
    *out_total_ns = (uint64_t)(total_ms * 1.0e6);
    ctx->prof_used = 0;
    return TT_HIP_OK;
}

int tt_hip_graph_begin(tt_hip_ctx *ctx) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    hipError_t e = hipStreamBeginCapture(ctx->stream, hipStreamCaptureModeThreadLocal);
    if (e != hipSuccess) return hip_fail(ctx, e, "hipStreamBeginCapture");
    ctx->capturing = true;
    return TT_HIP_OK;
}

int tt_hip_graph_end(tt_hip_ctx *ctx, tt_hip_graph **out_graph) {
    if (!ctx || !out_graph || !ctx->capturing) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    ctx->capturing = false;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(ctx->stream, &graph);
    if (e != hipSuccess || !graph) return hip_fail(ctx, e, "hipStreamEndCapture");
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    if (e != hipSuccess) {
        (void)hipGraphDestroy(graph);
        return hip_fail(ctx, e, "hipGraphInstantiate");
    }
    tt_hip_graph *g = new (std::nothrow) tt_hip_graph();
    if (!g) {
        (void)hipGraphExecDestroy(exec);
        (void)hipGraphDestroy(graph);
        return TT_HIP_ERR_OUT_OF_MEMORY;
    }
    g->graph = graph;
    g->exec = exec;
    g->ctx = ctx;
    g->generation = ctx->generation;
    *out_graph = g;
    return TT_HIP_OK;
}

int tt_hip_graph_launch(tt_hip_ctx *ctx, tt_hip_graph *graph) {
    if (!ctx || !graph || !graph->exec) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    // Buffers whose addresses the graph's kernels carry have been released since the capture.
    if (graph->ctx != ctx || graph->generation != ctx->generation) return TT_HIP_ERR_STALE;
    hipError_t e = hipGraphLaunch(graph->exec, ctx->stream);
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "hipGraphLaunch");
}

void tt_hip_graph_destroy(tt_hip_graph *graph) {
    if (!graph) return;
    if (graph->exec) (void)hipGraphExecDestroy(graph->exec);
    if (graph->graph) (void)hipGraphDestroy(graph->graph);
    delete graph;
}

int tt_hip_split_geometry(tt_hip_ctx *ctx, int n_seq, int n_q_heads, int n_kv_heads, int head_dim, int rows,
                          int seq_len, int *out_split_tokens, int *out_splits, int *out_workgroups) {
    if (!ctx || seq_len < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    LaunchPlan plan;
    int st = plan_launch(ctx, 0, n_seq, n_q_heads, n_kv_heads, head_dim, rows, (long long)seq_len * n_seq, seq_len, seq_len, &plan, 16, true);
    if (st != TT_HIP_OK) return st;
    if (out_split_tokens) *out_split_tokens = plan.split_len;
    if (out_splits) *out_splits = plan.n_splits_max;
    if (out_workgroups) *out_workgroups = (int)plan.workgroups;
    return TT_HIP_OK;
}

int tt_hip_set_split_tokens(tt_hip_ctx *ctx, int split_tokens) {
    if (!ctx || split_tokens < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    ctx->split_override = split_tokens;
    return TT_HIP_OK;
}

int tt_hip_set_option(tt_hip_ctx *ctx, int option, int value) {
    if (!ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok || ctx->capturing) return TT_HIP_ERR_BUSY;
    switch (option) {
        case TT_HIP_OPT_KV_STREAM:
            if (value < -1 || value > 1) return TT_HIP_ERR_INVALID_ARGUMENT;
            ctx->stream_override = value;
            return TT_HIP_OK;
        case TT_HIP_OPT_XCD_GRID:
            if (value != 0 && value != 1) return TT_HIP_ERR_INVALID_ARGUMENT;
            ctx->xcd_grid = value != 0;
            return TT_HIP_OK;
        case TT_HIP_OPT_MEASURE_PASS_ONLY:
            if (value != 0 && value != 1) return TT_HIP_ERR_INVALID_ARGUMENT;
            ctx->pass_only = value != 0;
            return TT_HIP_OK;
        default: return TT_HIP_ERR_INVALID_ARGUMENT;
    }
}

int tt_hip_calibrate_read(tt_hip_ctx *ctx, const void *src, size_t bytes, uint32_t *sink, size_t *out_bytes_read) {
    if (!ctx || !src || (reinterpret_cast<uintptr_t>(src) & 15u) != 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const size_t per_turn = (size_t)ctx->n_cus * 65536;  // every workgroup reads 64 KiB per turn
    const size_t turns = bytes / per_turn;
    if (turns == 0 || turns > 0xffffffffull) return TT_HIP_ERR_SHAPE;
    if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    launch_profiled(ctx, calibrate_read_kernel, dim3((unsigned)ctx->n_cus), dim3(256), 0u, static_cast<const u4 *>(src),
                    (unsigned)turns, sink);
    const hipError_t e = hipGetLastError();
    if (out_bytes_read) *out_bytes_read = turns * per_turn;
    return e == hipSuccess ? TT_HIP_OK : hip_fail(ctx, e, "calibrate_read_kernel launch");
}

const char *tt_hip_strerror(int status) {
    switch (status) {
        case TT_HIP_OK: return "ok";
        case TT_HIP_ERR_INVALID_ARGUMENT: return "invalid argument";
        case TT_HIP_ERR_SHAPE: return "unsupported shape";
        case TT_HIP_ERR_CURSOR: return "KV cursor mismatch";
        case TT_HIP_ERR_CAPACITY: return "KV capacity exceeded";
        case TT_HIP_ERR_BUSY: return "context busy (re-entered)";
        case TT_HIP_ERR_OUT_OF_MEMORY: return "out of device memory";
        case TT_HIP_ERR_HIP: return "HIP runtime error";
        case TT_HIP_ERR_NO_DEVICE: return "no gfx950 device";
        case TT_HIP_ERR_STALE: return "graph captured before a buffer it uses was reallocated";
        case TT_HIP_ERR_SCRATCH: return "call needs more split scratch than the fixed array of the no-allocation entry point holds";
        default: return "unknown status";
    }
}

const char *tt_hip_last_hip_error(tt_hip_ctx *ctx) { return ctx ? ctx->last_hip_error.c_str() : ""; }

// ---- attention entry points ------------------------------------------------

static int check_common(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_q_heads, const void *q, const void *out) {
    if (!ctx || !kv || !q || !out) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (kv->ctx != ctx) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (layer < 0 || layer >= kv->n_layers) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (n_q_heads <= 0 || n_q_heads % kv->n_kv_heads != 0) return TT_HIP_ERR_SHAPE;
    return TT_HIP_OK;
}

int tt_hip_attn_decode(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots, const int *seq_lens,
                       int n_q_heads, const tt_half *q, const tt_half *gate, float scale, tt_half *out) {
    return tt_hip_attn_decode_swa(ctx, kv, layer, n_seq, slots, seq_lens, 0, n_q_heads, q, gate, scale, out);
}

int tt_hip_attn_decode_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots, const int *seq_lens,
                           int window, int n_q_heads, const tt_half *q, const tt_half *gate, float scale, tt_half *out) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (n_seq <= 0 || !slots || !seq_lens || window < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    IntTable starts(n_seq);
    for (int i = 0; i < n_seq; ++i) {
        if (slots[i] < 0 || slots[i] >= kv->n_slots || seq_lens[i] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        const long long first = window > 0 && seq_lens[i] > window ? seq_lens[i] - window : 0;
        if (!kv->holds_keys(first, seq_lens[i])) return TT_HIP_ERR_CAPACITY;
        starts[i] = seq_lens[i] - 1;
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const long long row = (long long)n_q_heads * kv->head_dim;
    return run_attention(ctx, kv, 0, layer, n_seq, slots, starts.data(), seq_lens, 1, n_q_heads, q, row, row, gate, row,
                         row, scale, out, row, row, 1, 0, nullptr, window);
}

// Same kernels and planner as tt_hip_attn_decode; the partials live in this device's copy of `scratch`
// (reached through the address taken at context creation) and the per-sequence tables on the stack, so the
// call allocates nothing on the device or the host.  Calls on one GPU share the array: they must not overlap.
int tt_hip_attn_decode_noalloc(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots, const int *seq_lens,
                               int n_q_heads, const tt_half *q, const tt_half *gate, float scale, tt_half *out) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (n_seq <= 0 || !slots || !seq_lens) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (n_seq > kMaxSeqPerLaunch) return TT_HIP_ERR_SCRATCH;  // one launch: its tables travel as kernel arguments
    int starts[kMaxSeqPerLaunch];
    for (int i = 0; i < n_seq; ++i) {
        if (slots[i] < 0 || slots[i] >= kv->n_slots || seq_lens[i] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        if (!kv->holds_keys(0, seq_lens[i])) return TT_HIP_ERR_CAPACITY;
        starts[i] = seq_lens[i] - 1;
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const long long row = (long long)n_q_heads * kv->head_dim;
    return run_attention(ctx, kv, 0, layer, n_seq, slots, starts, seq_lens, 1, n_q_heads, q, row, row, gate, row, row, scale,
                         out, row, row, 1, 0, nullptr, 0, nullptr, 0, 0, /*static_partials=*/true);
}

int tt_hip_attn_decode_keep(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots, const int *seq_lens,
                            const uint8_t *keep_mask, size_t keep_stride, int n_q_heads, const tt_half *q,
                            const tt_half *gate, float scale, tt_half *out) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (n_seq <= 0 || !slots || !seq_lens || !keep_mask) return TT_HIP_ERR_INVALID_ARGUMENT;
    IntTable starts(n_seq);
    for (int i = 0; i < n_seq; ++i) {
        if (slots[i] < 0 || slots[i] >= kv->n_slots || seq_lens[i] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        if (n_seq > 1 && keep_stride < (size_t)seq_lens[i]) return TT_HIP_ERR_SHAPE;  // masks would overlap
        if (!kv->holds_keys(0, seq_lens[i])) return TT_HIP_ERR_CAPACITY;
        starts[i] = seq_lens[i] - 1;
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const long long row = (long long)n_q_heads * kv->head_dim;
    return run_attention(ctx, kv, 0, layer, n_seq, slots, starts.data(), seq_lens, 1, n_q_heads, q, row, row, gate, row,
                         row, scale, out, row, row, 1, 0, nullptr, 0, keep_mask, (long long)keep_stride);
}

int tt_hip_attn_decode_keep_indices(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots, const int *seq_lens,
                                    const uint32_t *keep_indices, size_t keep_index_stride, const uint32_t *keep_counts,
                                    int n_q_heads, const tt_half *q, const tt_half *gate, float scale, tt_half *out) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (n_seq <= 0 || !slots || !seq_lens || !keep_indices || !keep_counts) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (keep_index_stride == 0 || keep_index_stride > 0x7fffffffULL) return TT_HIP_ERR_SHAPE;
    IntTable starts(n_seq);
    int longest = 0;
    for (int i = 0; i < n_seq; ++i) {
        if (slots[i] < 0 || slots[i] >= kv->n_slots || seq_lens[i] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        if (!kv->holds_keys(0, seq_lens[i])) return TT_HIP_ERR_CAPACITY;
        starts[i] = seq_lens[i] - 1;
        longest = std::max(longest, seq_lens[i]);
    }
    // One row of selection bytes per sequence in the context's store (a key at or past a sequence's length is
    // dropped by the kernel's own range test), then the mask form.
    const size_t row_stride = ((size_t)longest + 63) / 64 * 64 + 64;
    if ((unsigned long long)n_seq * row_stride > 0x7ff00000ULL) return TT_HIP_ERR_SHAPE;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    st = ensure_keep_rows(ctx, (size_t)n_seq * row_stride);
    if (st != TT_HIP_OK) return st;
    hipLaunchKernelGGL(keep_rows_from_indices_kernel, dim3((unsigned)n_seq), dim3(256), 0, ctx->stream, ctx->keep_rows,
                       (unsigned)row_stride, keep_indices, (unsigned)keep_index_stride, keep_counts, 0x3fffffff, (int)row_stride);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(ctx, e, "keep_rows_from_indices_kernel");
    const long long row = (long long)n_q_heads * kv->head_dim;
    return run_attention(ctx, kv, 0, layer, n_seq, slots, starts.data(), seq_lens, 1, n_q_heads, q, row, row, gate, row,
                         row, scale, out, row, row, 1, 0, nullptr, 0, ctx->keep_rows, (long long)row_stride);
}

int tt_hip_attn_prefill_keep(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len, int kv_valid,
                             const uint8_t *keep_mask, size_t keep_stride, int n_q_heads, const tt_half *q, size_t q_stride,
                             const tt_half *gate, size_t gate_stride, float scale, tt_half *out, size_t o_stride) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (slot < 0 || slot >= kv->n_slots || start_pos < 0 || q_len <= 0 || !keep_mask) return TT_HIP_ERR_INVALID_ARGUMENT;
    const size_t packed = (size_t)n_q_heads * kv->head_dim;
    if (q_stride < packed || o_stride < packed || (gate && gate_stride < packed)) return TT_HIP_ERR_SHAPE;
    if ((long long)start_pos + q_len > kv_valid) return TT_HIP_ERR_INVALID_ARGUMENT;
    // a row's bytes cover every position the chunk can see; rows are read a word at a time
    if (keep_stride < (size_t)start_pos + (size_t)q_len || keep_stride % 4 != 0 || (uintptr_t)keep_mask % 4 != 0)
        return TT_HIP_ERR_SHAPE;
    if ((unsigned long long)q_len * keep_stride > 0x7ff00000ULL) return TT_HIP_ERR_SHAPE;  // 32-bit addressing of the rows
    if (!kv->holds_keys(0, kv_valid)) return TT_HIP_ERR_CAPACITY;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    // The GQA-packed split-K tiles (the chunk kernel does not take a selection): every tile walks its rows' keys.
    return run_attention(ctx, kv, 0, layer, 1, &slot, &start_pos, &kv_valid, q_len, n_q_heads, q, 0, (long long)q_stride,
                         gate, 0, (long long)gate_stride, scale, out, 0, (long long)o_stride, 1, 0, nullptr, 0, keep_mask, 0,
                         (long long)keep_stride);
}

int tt_hip_attn_prefill_keep_indices(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len,
                                     int kv_valid, const uint32_t *keep_indices, size_t keep_index_stride,
                                     const uint32_t *keep_counts, int n_q_heads, const tt_half *q, size_t q_stride,
                                     const tt_half *gate, size_t gate_stride, float scale, tt_half *out, size_t o_stride) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (slot < 0 || slot >= kv->n_slots || start_pos < 0 || q_len <= 0 || !keep_indices || !keep_counts)
        return TT_HIP_ERR_INVALID_ARGUMENT;
    const size_t packed = (size_t)n_q_heads * kv->head_dim;
    if (q_stride < packed || o_stride < packed || (gate && gate_stride < packed)) return TT_HIP_ERR_SHAPE;
    if ((long long)start_pos + q_len > kv_valid) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (keep_index_stride == 0 || keep_index_stride > 0x7fffffffULL) return TT_HIP_ERR_SHAPE;
    if (!kv->holds_keys(0, kv_valid)) return TT_HIP_ERR_CAPACITY;
    // (the plan kernel's bitmap of the context's blocks lives in LDS, 8 bytes per 1,024 keys, beside a run of the bits
    // it gathers: 64 KiB hold 8 million keys less that run, beyond what a page can address)
    if (((long long)kv_valid + 1023) / 1024 * 8 + (kPlanThreads + 1 + 32) * 4 > 65536) return TT_HIP_ERR_CAPACITY;
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    // The lists are served as they are: a launch turns them into each token tile's list of touched key blocks and
    // per-token key bits (keep_plan_kernel), which the attention kernel then walks -- work and memory of the order of
    // the selection.  Long chunks go in pieces of rows, so that the plan of one piece stays below 128 MiB.
    const int group = n_q_heads / kv->n_kv_heads;
    int gh = group;
    while (gh > 32 || group % gh != 0) --gh;
    const int tt = 32 / gh;  // tokens per tile of the 32-row tiles (the planner's own rule)
    const long long ctx_blocks = ((long long)kv_valid + 31) / 32, entries = (long long)tt * (long long)keep_index_stride;
    const long long cap = entries < ctx_blocks ? entries : ctx_blocks;
    const long long per_tile = (cap * (1 + tt) + 260) * 4;
    long long tiles_per_call = (128ll << 20) / per_tile;
    if (tiles_per_call < 1) tiles_per_call = 1;
    const long long rows_per_call = tiles_per_call * tt;
    for (long long r0 = 0; r0 < q_len; r0 += rows_per_call) {
        const int rows = (int)(q_len - r0 < rows_per_call ? q_len - r0 : rows_per_call);
        const int start = start_pos + (int)r0;
        const KeepLists lists{keep_indices + (size_t)r0 * keep_index_stride, keep_index_stride, keep_counts + r0};
        st = run_attention(ctx, kv, 0, layer, 1, &slot, &start, &kv_valid, rows, n_q_heads,
                           q + (size_t)r0 * q_stride, 0, (long long)q_stride, gate ? gate + (size_t)r0 * gate_stride : nullptr, 0,
                           (long long)gate_stride, scale, out + (size_t)r0 * o_stride, 0, (long long)o_stride, 1, 0, nullptr, 0, nullptr,
                           0, 0, false, &lists);
        if (st != TT_HIP_OK) return st;
    }
    return TT_HIP_OK;
}

int tt_hip_attn_verify(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                       const int *start_positions, int rows, int n_q_heads, const tt_half *q, const tt_half *gate,
                       float scale, tt_half *out) {
    return tt_hip_attn_verify_swa(ctx, kv, layer, n_seq, slots, start_positions, rows, 0, n_q_heads, q, gate, scale, out);
}

int tt_hip_attn_verify_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int n_seq, const int *slots,
                           const int *start_positions, int rows, int window, int n_q_heads, const tt_half *q,
                           const tt_half *gate, float scale, tt_half *out) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (n_seq <= 0 || rows <= 0 || !slots || !start_positions || window < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    IntTable totals(n_seq);
    for (int i = 0; i < n_seq; ++i) {
        if (slots[i] < 0 || slots[i] >= kv->n_slots || start_positions[i] < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
        const long long first = window > 0 && start_positions[i] + 1 > window ? start_positions[i] + 1 - window : 0;
        if (!kv->holds_keys(first, (long long)start_positions[i] + rows)) return TT_HIP_ERR_CAPACITY;
        totals[i] = start_positions[i] + rows;
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const long long tok = (long long)n_q_heads * kv->head_dim;
    const long long seq = tok * rows;
    return run_attention(ctx, kv, 0, layer, n_seq, slots, start_positions, totals.data(), rows, n_q_heads, q, seq, tok,
                         gate, seq, tok, scale, out, seq, tok, 1, 0, nullptr, window);
}

int tt_hip_attn_prefill(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len, int kv_valid,
                        int n_q_heads, const tt_half *q, size_t q_stride, const tt_half *gate, size_t gate_stride,
                        float scale, tt_half *out, size_t o_stride) {
    return tt_hip_attn_prefill_swa(ctx, kv, layer, slot, start_pos, q_len, kv_valid, 0, n_q_heads, q, q_stride, gate,
                                   gate_stride, scale, out, o_stride);
}

int tt_hip_attn_prefill_swa(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start_pos, int q_len, int kv_valid,
                            int sliding_window, int n_q_heads, const tt_half *q, size_t q_stride, const tt_half *gate,
                            size_t gate_stride, float scale, tt_half *out, size_t o_stride) {
    int st = check_common(ctx, kv, layer, n_q_heads, q, out);
    if (st != TT_HIP_OK) return st;
    if (slot < 0 || slot >= kv->n_slots || start_pos < 0 || q_len <= 0 || sliding_window < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    const size_t packed = (size_t)n_q_heads * kv->head_dim;
    if (q_stride < packed || o_stride < packed || (gate && gate_stride < packed)) return TT_HIP_ERR_SHAPE;
    if ((long long)start_pos + q_len > kv_valid) return TT_HIP_ERR_INVALID_ARGUMENT;
    {
        const long long first = sliding_window > 0 && start_pos + 1 > sliding_window ? start_pos + 1 - sliding_window : 0;
        if (!kv->holds_keys(first, kv_valid)) return TT_HIP_ERR_CAPACITY;
    }
    BusyGuard guard(ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const bool aligned = aligned16(q) && aligned16(out) && (!gate || aligned16(gate)) && q_stride % 8 == 0 &&
                         o_stride % 8 == 0 && (!gate || gate_stride % 8 == 0);
    // A window that clips no row of the chunk is no window.
    const int window = sliding_window > 0 && (long long)start_pos + q_len > sliding_window ? sliding_window : 0;
    // (the chunk kernel takes a row's maximum over the raw scores: a scale that is not positive goes the split-K way)
    const bool serves = prefill_kernel_serves(n_q_heads, kv->n_kv_heads, kv->head_dim, aligned) && scale > 0.0f;
    const long long chunk_wgs = (long long)((q_len + 63) / 64) * (n_q_heads / 4);
    // The chunk kernel as it is -- a workgroup per pair of tiles and 4 heads, all their keys -- where its workgroups
    // fill half the chip, or a quarter of it with few key blocks each (a long first chunk of a prompt: 1024 rows from
    // position 0 take 39 us against 41 us through the split-K tiles, 1536 rows 51 against 66).  Fewer workgroups
    // walking more blocks lose to the other routes at any context: 128 rows behind 1920 keys took 100 us that way,
    // 25 us through the split-K tiles; behind a 1024-key window 62 us against 20 us.
    const long long pair_blocks = (2LL * start_pos + q_len) / 32 + 2;  // key blocks a workgroup's pair of tiles walks
    const bool filled = 2 * chunk_wgs >= ctx->n_cus || (window == 0 && 4 * chunk_wgs >= ctx->n_cus && pair_blocks <= 64);
    if (window > 0) {
        // The chunk kernel starts every tile at its window's first block; under-filled chunks over a
        // long window, quantised pages and head groups it does not serve go through the split-K
        // kernel (GQA-packed tiles, each walking only its rows' windows).
        if (serves && filled && kv->bits == 16) {
            if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
            return launch_prefill(ctx, kv, layer, slot, start_pos, q_len, kv_valid, n_q_heads, q, (long long)q_stride, gate,
                                  (long long)gate_stride, scale, out, (long long)o_stride, 1, 0, nullptr, nullptr, nullptr, window);
        }
        return run_attention(ctx, kv, 0, layer, 1, &slot, &start_pos, &kv_valid, q_len, n_q_heads, q, 0, (long long)q_stride,
                             gate, 0, (long long)gate_stride, scale, out, 0, (long long)o_stride, 1, 0, nullptr, window);
    }
    // Quantised pages: the split-K kernel reads them as they are (dequantising in registers, once
    // per 32-row tile -- 269 TFLOP/s on a 4096-row chunk).  A chunk that the MFMA chunk kernel
    // would take is instead served from fp16 pages of the slot's visible blocks, dequantised once
    // per call into the context's staging store (4096 rows: one 9 us pass, then the fp16 kernel).
    PageSource staged{};
    const PageSource *pages = nullptr;
    // From this many keys on a chunk that does not fill the chip goes through the chunk kernel over key ranges (below:
    // through the split-K tiles): 786,432 / rows, i.e. 12k keys at 64 rows, 6k at 128, and at least 4096 (2560 over
    // quantised pages, whose visible blocks are dequantised once per call first).  The split-K tiles read the keys once
    // per tile of rows and leave small partial results; the ranges read them once per range and leave rows x heads x D
    // floats per range.  One box, fp16, split-K / ranges: 64 rows at 8k keys 31.6 / 33.4 us, at 12k 37.2 / 35.3; 96
    // rows at 4k 28.4 / 32.4, at 12k 47.7 / 42.8; 128 rows at 4k 32.0 / 35.0, at 8k 44.3 / 39.1; 192 rows at 4k 41.8 /
    // 38.6.  Over 8 bits: 64 rows at 4k 24.4 / 35.4, at 16k 50.1 / 49.2, at 32k 80.7 / 71.9; 128 rows at 4k 34.6 /
    // 40.2, at 8k 48.9 / 45.0.
    const long long by_rows = 786432 / (q_len > 0 ? q_len : 1);
    const int floor_keys = kv->bits == 16 ? 4096 : 2560;
    const int ranges_from = by_rows > floor_keys ? (int)by_rows : floor_keys;
    // ... and from this many rows on: 64; at fp16 32 rows deep in a context (32 rows at 32k keys 50 us against 54 us,
    // 48 rows 62 against 73).  Over quantised pages fewer rows stay with the split-K tiles, which widen a block once per
    // tile of 16 rows: dequantising the whole context for them costs more than that at any length measured (32 rows
    // at 64k keys over 8 bits 82 us against 107 us, 12 rows at 32k keys 30 us against 62 us).
    const int rows_from = kv->bits == 16 ? (kv_valid >= 32768 ? 32 : 64) : 64;
    if (kv->bits != 16 && !kv->ring && serves && q_len >= rows_from && (filled || kv_valid >= ranges_from)) {
        const int n_blocks = (kv_valid + 31) / 32;
        const size_t page = (size_t)n_blocks * 32 * kv->head_dim;
        if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
        st = ensure_stage(ctx, page * kv->n_kv_heads);
        if (st != TT_HIP_OK) return st;
        st = launch_kvq_dequant_blocks(kv, layer, slot, n_blocks, ctx->stage_k, ctx->stage_v, page);
        if (st != TT_HIP_OK) return st;
        staged = PageSource{ctx->stage_k, ctx->stage_v, (long long)page, 0};
        pages = &staged;
    }
    if (serves && (kv->bits == 16 || pages)) {
        // The chunk kernel gives a workgroup 64 query rows of 4 heads and ALL their keys: one
        // workgroup per CU at 4096 rows x 16 heads, but a 128-row chunk (the reference's default
        // prefillChunkTokens) deep into a long context would be 8 workgroups walking 32k keys
        // each (1318 us at 16q/2kv/256).  Three routes, chosen from timings at that shape:
        //  * at least half a chip of workgroups, or a quarter with few blocks each: the chunk kernel as it is;
        //  * 64 rows or more over 4096 keys or more (2560 over quantised pages): the chunk kernel with the keys cut into
        //    ranges, a workgroup per (tile, 4 heads, range), and the combine pass over the partial
        //    results (128 rows at 32k keys 98-106 us, 1024 rows 507-538 us; 256 rows at 4k keys 39 us
        //    against 46 us the split-K way);
        //  * anything else: the split-K kernel, which packs a KV head's q heads into its tiles
        //    like a verify pass (64 rows at 16k keys 62 us against 89 us; 512 rows at 2k keys
        //    59 us against 104 us, where the partial results outweigh the keys).
        int n_splits = 1, split_blocks = 0;
        if (!filled && q_len >= rows_from && kv_valid >= ranges_from) {
            const int nb_total = (kv_valid + 31) / 32;
            // With ranges a workgroup takes one 32-row tile of 4 heads (not a pair of tiles) over one range of key
            // blocks.  The number of ranges by a small model of the two costs: rounds of workgroups on the chip x the
            // blocks of a range (0.8 us a block at D = 256), and the partial results -- rows x heads x D floats per range,
            // written by the kernel and read by the combine pass (~3 TB/s for the pair).  At least 8 blocks a range.
            const long long range_wgs = (long long)((q_len + 31) / 32) * (n_q_heads / 4);
            const double partial_us = (double)q_len * n_q_heads * kv->head_dim * 4.0 * 2.0 / 3.0e6;
            double best_us = 0.0;
            // (1, 2, 4 or 8 kv heads: a kv head's workgroups run on its 8 / n XCDs, an equal share each)
            const int xs = (kv->n_kv_heads <= 8 && 8 % kv->n_kv_heads == 0) ? 8 / kv->n_kv_heads : 0;
            const long long xcd_cus = ctx->n_cus / 8 > 0 ? ctx->n_cus / 8 : 1;
            for (int s = 2; s <= 32 && nb_total / s >= 8; ++s) {
                const int blocks = (nb_total + s - 1) / s;
                long long rounds = (range_wgs * s + ctx->n_cus - 1) / ctx->n_cus;
                if (xs > 0) rounds = ((range_wgs / kv->n_kv_heads * s + xs - 1) / xs + xcd_cus - 1) / xcd_cus;
                const double us = (double)rounds * blocks * 0.8 * kv->head_dim / 256.0 + s * partial_us;
                if (n_splits < 2 || us < best_us) {
                    best_us = us;
                    split_blocks = blocks;
                    n_splits = (nb_total + blocks - 1) / blocks;
                }
            }
        }
        if (filled || (pages && n_splits < 2)) {
            if (hipSetDevice(ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
            return launch_prefill(ctx, kv, layer, slot, start_pos, q_len, kv_valid, n_q_heads, q, (long long)q_stride, gate,
                                  (long long)gate_stride, scale, out, (long long)o_stride, 1, 0, nullptr, nullptr, pages);
        }
        if (n_splits >= 2)
            return run_attention(ctx, kv, 1, layer, 1, &slot, &start_pos, &kv_valid, q_len, n_q_heads, q, 0,
                                 (long long)q_stride, gate, 0, (long long)gate_stride, scale, out, 0, (long long)o_stride,
                                 n_splits, split_blocks, pages);
        return run_attention(ctx, kv, 0, layer, 1, &slot, &start_pos, &kv_valid, q_len, n_q_heads, q, 0,
                             (long long)q_stride, gate, 0, (long long)gate_stride, scale, out, 0, (long long)o_stride);
    }
    // What the chunk kernel does not serve (head groups that are no multiple of 4, unaligned rows, quantised pages
    // that are not staged, a non-positive scale): the split-K kernel.  Tiles of 32 rows of ONE head, each walking
    // all its keys, where they are plentiful and the context is short or they are very plentiful; otherwise --
    // a few rows deep in a context -- GQA-packed tiles over key ranges, like a verify pass (one row at 32k keys over
    // 8 bits took 460 us as 16 one-head tiles walking 32k keys each).
    const long long head_tiles = (long long)((q_len + 31) / 32) * n_q_heads;
    const int kind = 2 * head_tiles >= ctx->n_cus && (kv_valid <= 8192 || head_tiles >= 2LL * ctx->n_cus) ? 1 : 0;
    return run_attention(ctx, kv, kind, layer, 1, &slot, &start_pos, &kv_valid, q_len, n_q_heads, q, 0, (long long)q_stride,
                         gate, 0, (long long)gate_stride, scale, out, 0, (long long)o_stride);
}

}  // extern "C"
