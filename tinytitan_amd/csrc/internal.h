// Internal declarations shared by the translation units of libctinytitan_hip.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <atomic>
#include <string>
#include <vector>

#include "../../include/ctinytitan_hip.h"
#include "kv_layout.h"

namespace tt {

constexpr int kMaxSeqPerLaunch = 64;
// A wavefront of the split-K kernel lists the blocks that a per-query selection touches, over up to this many
// 64-block windows of its split: a split of such a launch is at most kKeepWindows * 64 blocks per wavefront.
constexpr int kKeepWindows = 8;
// Rows (sequence, tile, split, query row) of split-K partials the fixed scratch array of
// tt_hip_attn_decode_noalloc holds: 32 MiB of O rows + 256 KiB of (max, sum) pairs.
constexpr size_t kStaticPartialRows = 32768;

// Kernel arguments of the split-K attention kernel and its combine kernel.
// Passed by value (kernarg segment), so no per-call host->device copy is needed
// for the per-sequence tables.
//
// What every wave needs before it can issue its first K/V load sits in the first 128 bytes (`hot`) and in
// one 16-byte entry per sequence right behind them: the kernel fetches both with three scalar loads issued
// together, one trip to the kernarg segment instead of one per field as it is first used.
constexpr int kHotAligned = 1;  // q/gate/out rows are 16-byte aligned
// The grid is one-dimensional in x and XCD-major: consecutive workgroups go to consecutive XCDs, so the
// workgroups that one XCD runs side by side are given consecutive (split, tile) pairs, tile fastest -- token
// tiles of one KV head over one key range, whose K/V blocks they then share in that XCD's L2.
constexpr int kHotXcdGrid = 2;
struct SplitKHot {                         // dword
    const _Float16 *k_layer;               //  0
    const _Float16 *v_layer;               //  2
    const _Float16 *q;                     //  4
    long long page_elems;                  //  6  capacity * D: halves per (slot, kv_head) page
    long long q_seq_stride, q_tok_stride;  //  8, 10  elements; consecutive heads are D apart
    int n_kv_heads;                        // 12
    int group;                             // 13  q heads per kv head
    int rows;                              // 14  query tokens per sequence
    int gh;                                // 15  q heads per tile
    int tt;                                // 16  query tokens per tile (NT / gh)
    int hsubs;                             // 17  head sub-groups per kv head (group / gh)
    int tok_tiles;                         // 18  ceil(rows / tt)
    int split_len;                         // 19  keys per split, multiple of 32
    int window;       // 20  sliding window: a row at position p sees keys [max(0, p + 1 - window), p + 1); 0 = every key
    int ring_blocks;  // 21  ring cache: key block b lives in block b % ring_blocks of the page; 0 = where it is
    float scale_log2e;                     // 22
    int n_splits_max;                      // 23
    int n_tiles;                           // 24  n_kv_heads * hsubs * tok_tiles
    int flags;                             // 25  kHotAligned | kHotXcdGrid
    int keep_words;   // 26  per-sequence masks start on 4-byte boundaries: a wavefront may read its blocks' bytes as words
    int gh_inv;       // 27  ceil(65536 / gh): (i * gh_inv) >> 16 == i / gh for 0 <= i < 64, gh <= 32
    float *part_o;    // 28  [first_split(seq) + split][tile][NT][D]
    float *part_ml;   // 30  [first_split(seq) + split][tile][NT][2]  (max in log2 domain, sum)
};
static_assert(sizeof(SplitKHot) == 128, "the kernel loads the hot arguments as two 64-byte pieces");

struct SplitKSeq {
    int slot;
    int start;  // absolute position of query row 0
    int total;  // valid keys in the cache for this call
    int first_split;  // where this sequence's splits start in the partial buffers: a sequence takes as many
                      // splits as ITS keys need, so a short sequence beside a long one holds no empty partials
};

struct alignas(64) SplitKArgs {
    SplitKHot hot;
    SplitKSeq seq[kMaxSeqPerLaunch];
    const _Float16 *gate;  // nullptr: no gate
    _Float16 *out;
    long long g_seq_stride, g_tok_stride;
    long long o_seq_stride, o_tok_stride;
    const uint8_t *keep;          // sparse selection: one byte per key position, 0 drops the key; nullptr: every key
    long long keep_seq_stride;    // bytes between the masks of consecutive sequences
    long long keep_row_stride;    // > 0: one mask per query row, this many bytes apart (a multiple of 4); 0: one per sequence
    // A chunk's selection as per-query index lists, turned into a plan per token tile by keep_plan_kernel:
    const int *plan_ranges;       // [token tile][n_splits_max + 1]: where each split's entries start in the tile's list
    const int *plan_blocks;       // [token tile][plan_cap]: the key blocks the tile's tokens keep a key of, ascending
    const unsigned *plan_bits;    // [token tile][plan_cap][tt]: per entry and token, bit i = key 32 block + i is kept
    int plan_cap;                 // entries a tile's list has room for
};

struct LaunchPlan {
    int nt;  // 16 or 32 query rows per tile
    int gh, tt, hsubs, tok_tiles, n_tiles;
    int waves;
    int split_len, n_splits_max;
    long long workgroups;
    size_t lds_bytes;
    bool stream;  // every K/V byte is read once by the launch, and there are many of them: non-temporal loads
    bool xcd_grid;  // launch with kHotXcdGrid
};

}  // namespace tt

struct tt_hip_ctx {
    int device = 0;
    int n_cus = 256;
    hipStream_t own_stream = nullptr;
    hipStream_t stream = nullptr;
    hipEvent_t ev_begin = nullptr, ev_end = nullptr;
    bool timer_open = false;
    float *part_o = nullptr;
    float *part_ml = nullptr;
    float *static_scratch = nullptr;  // this device's address of the library's fixed scratch array
    size_t part_rows = 0;  // capacity in (seq, tile, split, n) rows
    _Float16 *stage_k = nullptr, *stage_v = nullptr;  // fp16 pages of one slot, dequantised for a prefill chunk
    size_t stage_elems = 0;                           // halves in each
    void *select_ws = nullptr;  // histograms, bitmaps and candidate lists of the multi-workgroup key selection; zero between calls
    size_t select_ws_bytes = 0;
    uint8_t *keep_rows = nullptr;  // selection bytes written out from a chunk's index lists (tt_hip_attn_prefill_keep_indices)
    size_t keep_rows_bytes = 0;
    int split_override = 0;
    bool xcd_grid = true;  // chunks through the split-K kernel launch XCD-major (TT_HIP_OPT_XCD_GRID)
    bool pass_only = false;  // measurement control (TT_HIP_OPT_MEASURE_PASS_ONLY): split-K launches go without their combine pass
    int stream_override = -1;  // -1: automatic; 0 / 1: never / always mark single-read K/V loads non-temporal
    bool capturing = false;
    // Bumped whenever device memory that a captured graph may have baked into its kernel arguments is released:
    // the split-K scratch, the staging pages, the selection workspace, a cache's stores (growth, destruction).
    // A graph remembers the value it was captured at and refuses to replay once it has moved.
    uint64_t generation = 0;
    // per-launch timing of the dominant kernel
    bool profiling = false;
    std::vector<hipEvent_t> prof_events;  // start/stop pairs
    size_t prof_used = 0;                 // events recorded so far
    uint64_t prof_overhead_ns = 0;        // elapsed time of an empty event pair (what a pair RECORDED around launches reads too much)
    std::atomic_flag busy = ATOMIC_FLAG_INIT;
    std::string last_hip_error;
};

// A kernel launch on the context's stream.  While the context profiles, the launch carries a start and a stop
// event bound to the dispatch itself: the pair then reads the kernel's own duration as the command processor stamps
// its begin and its end -- what a kernel trace reports -- and none of the cost of recording events around it.
template <typename F, typename... Args>
inline void launch_profiled(tt_hip_ctx *ctx, F kernel, dim3 grid, dim3 block, unsigned lds_bytes, Args... args) {
    if (ctx->profiling && !ctx->capturing && ctx->prof_used + 2 <= ctx->prof_events.size()) {
        hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, ctx->stream, ctx->prof_events[ctx->prof_used],
                              ctx->prof_events[ctx->prof_used + 1], 0u, args...);
        ctx->prof_used += 2;
    } else {
        hipLaunchKernelGGL(kernel, grid, block, lds_bytes, ctx->stream, args...);
    }
}

struct tt_hip_graph {
    hipGraph_t graph = nullptr;
    hipGraphExec_t exec = nullptr;
    tt_hip_ctx *ctx = nullptr;
    uint64_t generation = 0;  // the context's when the capture ended
};

struct tt_hip_kv {
    tt_hip_ctx *ctx = nullptr;
    int n_layers = 0, n_kv_heads = 0, head_dim = 0, n_slots = 0;
    int capacity = 0, max_context = 0;
    int bits = 16;                 // 16: fp16 values; 8 / 4: affine levels with per-group fp16 scale and bias
    bool ring = false;             // row of position p lives at p % capacity; capacity is fixed
    uint64_t generation = 0;       // bumped when the stores are reallocated
    std::vector<_Float16 *> k, v;  // one K and one V store per layer (bytes at 8 / 4 bits)
    std::vector<int> positions;
    size_t block_bytes() const { return tt::block_bytes(head_dim, bits); }
    size_t page_bytes() const { return (size_t)(capacity / tt::kBlockTokens) * block_bytes(); }
    size_t layer_bytes() const { return (size_t)n_slots * n_kv_heads * page_bytes(); }
    size_t page_elems() const { return page_bytes() / 2; }  // halves per (slot, kv head) page, whatever they hold
    int physical(int position) const { return ring ? position % capacity : position; }
    // Rows [position, position + n) must be storable in one piece: inside capacity, and on a ring
    // inside max_context without wrapping (KVCacheManager+Validation.swift:52-59).
    bool holds_rows(int position, int n) const {
        if (!ring) return (long long)position + n <= capacity;
        return (long long)position + n <= max_context && (long long)physical(position) + n <= capacity;
    }
    // Keys [first, last) readable by an attention call: on a ring only the last `capacity` rows exist.
    bool holds_keys(long long first, long long last) const {
        if (!ring) return last <= capacity;
        return last <= max_context && last - (first & ~31LL) <= capacity;
    }
    int ring_blocks() const { return ring ? capacity / tt::kBlockTokens : 0; }
};

namespace tt {

// Records a failed HIP call on the context and maps it to a status code.
int hip_fail(tt_hip_ctx *ctx, hipError_t err, const char *what);

// RAII guard of the one-call-at-a-time rule.
struct BusyGuard {
    tt_hip_ctx *ctx;
    bool ok;
    explicit BusyGuard(tt_hip_ctx *c) : ctx(c), ok(!c->busy.test_and_set(std::memory_order_acquire)) {}
    ~BusyGuard() {
        if (ok) ctx->busy.clear(std::memory_order_release);
    }
};

// Raise the dynamic LDS limits of the kernels that need more than the default (per device; the context's is current).
int configure_splitk_kernels(tt_hip_ctx *ctx);
int configure_prefill_kernels(tt_hip_ctx *ctx);
int configure_affine_kernels(tt_hip_ctx *ctx);

int ensure_partials(tt_hip_ctx *ctx, size_t rows, int head_dim);
int ensure_stage(tt_hip_ctx *ctx, size_t elems);

// K/V pages the chunk kernel reads instead of the cache's own (one slot's, kv head pages page_elems apart).
struct PageSource {
    const _Float16 *k, *v;
    long long page_elems;
    int ring_blocks;  // 0: linear pages
};

// Plans tile shape and split geometry.  kind: 0 decode/verify (GQA-packed rows), 1 prefill.  small_tiles_ok: the
// caller's kernels take tiles of 16 rows where the plan prefers them to one tile of 32 (no key selection, no ranges
// of the chunk kernel, whose callers fix the tile themselves).
int plan_launch(const tt_hip_ctx *ctx, int kind, int n_seq, int n_q_heads, int n_kv_heads, int head_dim, int rows,
                long long total_keys, int min_keys, int max_keys, LaunchPlan *plan, int kv_bits = 16, bool small_tiles_ok = false);

// kv_bits: 16 for fp16 pages, 8 / 4 for quantised ones.
int launch_splitk(tt_hip_ctx *ctx, const LaunchPlan &plan, int head_dim, int n_seq, const SplitKArgs &args, int kv_bits = 16);

bool prefill_kernel_serves(int n_q_heads, int n_kv_heads, int head_dim, bool aligned);
// n_splits > 1: every workgroup takes one of n_splits ranges of split_blocks key blocks and leaves
// unnormalised partials (layout of the split-K kernel at 32-row, one-head tiles) for launch_combine.
int launch_prefill(tt_hip_ctx *ctx, tt_hip_kv *kv, int layer, int slot, int start, int q_len, int kv_valid,
                   int n_q_heads, const tt_half *q, long long q_stride, const tt_half *gate, long long g_stride,
                   float scale, tt_half *out, long long o_stride, int n_splits = 1, int split_blocks = 0,
                   float *part_o = nullptr, float *part_ml = nullptr, const PageSource *pages = nullptr, int window = 0);
int launch_combine(tt_hip_ctx *ctx, const LaunchPlan &plan, int head_dim, int n_seq, const SplitKArgs &args);

int launch_kv_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k, const tt_half *v,
                     size_t stride);
int launch_kv_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k, tt_half *v, size_t stride);

// Quantised pages (kv_quant.hip): quantise-and-write, dequantised read, stored rows in and out.
int launch_kvq_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k, const tt_half *v,
                      size_t stride);
int launch_kvq_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k, tt_half *v, size_t stride,
                    const int *positions = nullptr, int limit = 0);
int launch_kvq_dequant_blocks(tt_hip_kv *kv, int layer, int slot, int n_blocks, _Float16 *k_dst, _Float16 *v_dst,
                              size_t dst_page_elems);
int launch_kvq_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, uint8_t *k_rows, uint8_t *v_rows,
                    size_t row_stride, bool to_rows);

}  // namespace tt
