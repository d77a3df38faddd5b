// HBM-resident KV cache (fp16, or 8 / 4-bit affine levels: kv_quant.hip): per-layer K and V
// stores of [slot][kv_head] pages, per-slot cursors, append / read-back kernels and capacity growth.
//
// Bookkeeping follows KVCacheManager (sources/TinyTitan/Runtime/KVCache/
// KVCacheManager.swift:62-333, KVCacheManager+Storage.swift:99-139, :266-309).
#include <cstdint>
#include <new>

#include "internal.h"

namespace tt {

// One thread per (token, kv_head, d): reads the caller's token-major row and
// scatters into the swizzled K and V blocks.  Eight consecutive threads fill
// one 16-byte K group; V elements land 16 bytes apart.
__global__ __launch_bounds__(256) void kv_append_kernel(_Float16 *__restrict__ k_layer, _Float16 *__restrict__ v_layer,
                                                        const _Float16 *__restrict__ k_src,
                                                        const _Float16 *__restrict__ v_src, long long src_stride,
                                                        long long page_elems, int slot, int n_kv_heads, int head_dim,
                                                        int position, int n_tokens) {
    const long long per_token = (long long)n_kv_heads * head_dim;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per_token * n_tokens) return;
    const int t = (int)(idx / per_token);
    const int rem = (int)(idx - (long long)t * per_token);
    const int kvh = rem / head_dim;
    const int d = rem - kvh * head_dim;
    const size_t page = ((size_t)slot * n_kv_heads + kvh) * (size_t)page_elems;
    const long long src = (long long)t * src_stride + rem;
    k_layer[page + k_offset(head_dim, position + t, d)] = k_src[src];
    v_layer[page + v_offset(head_dim, position + t, d)] = v_src[src];
}

__global__ __launch_bounds__(256) void kv_read_kernel(const _Float16 *__restrict__ k_layer,
                                                      const _Float16 *__restrict__ v_layer, _Float16 *__restrict__ k_dst,
                                                      _Float16 *__restrict__ v_dst, long long dst_stride,
                                                      long long page_elems, int slot, int n_kv_heads, int head_dim,
                                                      int position, int n_tokens, const int *__restrict__ positions,
                                                      int limit, int ring_capacity) {
    // positions: row t is the row of position positions[t] (a gather); a position outside [0, limit) gives zeros
    const long long per_token = (long long)n_kv_heads * head_dim;
    const long long idx = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= per_token * n_tokens) return;
    const int t = (int)(idx / per_token);
    const int rem = (int)(idx - (long long)t * per_token);
    const int kvh = rem / head_dim;
    const int d = rem - kvh * head_dim;
    const size_t page = ((size_t)slot * n_kv_heads + kvh) * (size_t)page_elems;
    const long long dst = (long long)t * dst_stride + rem;
    int pos = position + t;
    bool inside = true;
    if (positions) {
        pos = positions[t];
        inside = pos >= 0 && pos < limit;
        pos = inside ? (ring_capacity > 0 ? pos % ring_capacity : pos) : 0;
    }
    if (k_dst) k_dst[dst] = inside ? k_layer[page + k_offset(head_dim, pos, d)] : (_Float16)0;
    if (v_dst) v_dst[dst] = inside ? v_layer[page + v_offset(head_dim, pos, d)] : (_Float16)0;
}

// Whole 32-token blocks: one workgroup per (block, kv head).  The 32 source rows are read
// coalesced (16 bytes per thread along a row) into LDS, then written out in the swizzled order,
// 16 bytes per thread and contiguous across the workgroup: K as [d / 8][key][8], V as
// [d][chunk][8] with each chunk's eight keys gathered from LDS.  HBM sees each byte once, as
// full lines, in both directions.
constexpr int kAppendPad = 8;  // halves of padding per LDS row: rows 16 bytes off a bank-aligned stride

__global__ __launch_bounds__(256) void kv_append_blocks_kernel(_Float16 *__restrict__ k_layer, _Float16 *__restrict__ v_layer,
                                                               const _Float16 *__restrict__ k_src,
                                                               const _Float16 *__restrict__ v_src, long long src_stride,
                                                               long long page_elems, int slot, int n_kv_heads, int head_dim,
                                                               int first_block) {
    extern __shared__ __attribute__((aligned(16))) _Float16 tile[];  // K rows, then V rows: [32][head_dim + pad]
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const int row_halves = head_dim + kAppendPad;
    _Float16 *kt = tile, *vt = tile + kBlockTokens * row_halves;
    const int kvh = blockIdx.y;
    const int groups = head_dim >> 3;              // 16-byte groups per row
    const int pieces = kBlockTokens * groups;      // per tile
    const long long src0 = (long long)blockIdx.x * kBlockTokens * src_stride + (long long)kvh * head_dim;
    for (int p = threadIdx.x; p < pieces; p += 256) {
        const int row = p / groups, g8 = p - row * groups;
        const long long off = src0 + (long long)row * src_stride + g8 * 8;
        *reinterpret_cast<h8 *>(kt + row * row_halves + g8 * 8) = *reinterpret_cast<const h8 *>(k_src + off);
        *reinterpret_cast<h8 *>(vt + row * row_halves + g8 * 8) = *reinterpret_cast<const h8 *>(v_src + off);
    }
    __syncthreads();
    const size_t dst0 = ((size_t)slot * n_kv_heads + kvh) * (size_t)page_elems +
                        (size_t)(first_block + (int)blockIdx.x) * (size_t)(kBlockTokens * head_dim);
    for (int p = threadIdx.x; p < pieces; p += 256) {
        // K piece p = (d / 8, key)
        const int d8 = p >> 5, key = p & 31;
        *reinterpret_cast<h8 *>(k_layer + dst0 + (size_t)p * 8) = *reinterpret_cast<const h8 *>(kt + key * row_halves + d8 * 8);
        // V piece p = (d, chunk)
        const int d = p >> 2, c = p & 3;
        h8 x;
#pragma unroll
        for (int i = 0; i < 8; ++i) x[i] = vt[v_key_at(c, i) * row_halves + d];
        *reinterpret_cast<h8 *>(v_layer + dst0 + (size_t)p * 8) = x;
    }
}

static int launch_kv_append_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const _Float16 *k,
                                 const _Float16 *v, size_t stride) {
    const long long total = (long long)n_tokens * kv->n_kv_heads * kv->head_dim;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(kv_append_kernel, dim3(blocks), dim3(256), 0, kv->ctx->stream, kv->k[layer], kv->v[layer], k, v,
                       (long long)stride, (long long)kv->page_elems(), slot, kv->n_kv_heads, kv->head_dim, position, n_tokens);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(kv->ctx, e, "kv_append_kernel launch");
}

// Rows that cover whole 32-token blocks go through the block kernel (16-byte aligned sources
// only); the ragged head and tail of the range, and single decode rows, go element by element.
int launch_kv_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k, const tt_half *v,
                     size_t stride) {
    const _Float16 *ks = reinterpret_cast<const _Float16 *>(k), *vs = reinterpret_cast<const _Float16 *>(v);
    const int first_full = ((position + kBlockTokens - 1) / kBlockTokens) * kBlockTokens;
    const int last_full_end = ((position + n_tokens) / kBlockTokens) * kBlockTokens;
    const bool aligned = (((uintptr_t)ks | (uintptr_t)vs) & 15u) == 0 && (stride * 2) % 16 == 0;
    // Short chunks go by rows altogether: one small launch (128 tokens 2.9 us by blocks, 2.2 us by rows; 512 tokens
    // 3.0 / 3.7; 4096 tokens 4.1 / 15.8); with a ragged head or tail the blocks come with one or two more launches
    // (128 tokens at position 37 6.6 us, 1024 tokens 6.7 against 5.8 by rows).
    const bool ragged = first_full > position || last_full_end < position + n_tokens;
    const bool by_rows = n_tokens <= 256 || (ragged && n_tokens <= 1024);
    if (!aligned || last_full_end <= first_full || by_rows) return launch_kv_append_rows(kv, layer, slot, position, n_tokens, ks, vs, stride);
    if (first_full > position) {
        const int rc = launch_kv_append_rows(kv, layer, slot, position, first_full - position, ks, vs, stride);
        if (rc != TT_HIP_OK) return rc;
    }
    const size_t skip = (size_t)(first_full - position) * stride;
    const int n_blocks = (last_full_end - first_full) / kBlockTokens;
    const size_t lds = (size_t)2 * kBlockTokens * (kv->head_dim + kAppendPad) * sizeof(_Float16);
    hipLaunchKernelGGL(kv_append_blocks_kernel, dim3((unsigned)n_blocks, (unsigned)kv->n_kv_heads), dim3(256), lds,
                       kv->ctx->stream, kv->k[layer], kv->v[layer], ks + skip, vs + skip, (long long)stride,
                       (long long)kv->page_elems(), slot, kv->n_kv_heads, kv->head_dim, first_full / kBlockTokens);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(kv->ctx, e, "kv_append_blocks_kernel launch");
    const int tail = position + n_tokens - last_full_end;
    if (tail > 0) {
        const size_t tskip = (size_t)(last_full_end - position) * stride;
        return launch_kv_append_rows(kv, layer, slot, last_full_end, tail, ks + tskip, vs + tskip, stride);
    }
    return TT_HIP_OK;
}

// The inverse of kv_append_blocks_kernel: whole swizzled blocks are read as full lines, put
// back in token-major order in LDS, and leave as coalesced rows.
__global__ __launch_bounds__(256) void kv_read_blocks_kernel(const _Float16 *__restrict__ k_layer,
                                                             const _Float16 *__restrict__ v_layer,
                                                             _Float16 *__restrict__ k_dst, _Float16 *__restrict__ v_dst,
                                                             long long dst_stride, long long page_elems, int slot,
                                                             int n_kv_heads, int head_dim, int first_block) {
    extern __shared__ __attribute__((aligned(16))) _Float16 tile[];
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    const int row_halves = head_dim + kAppendPad;
    _Float16 *kt = tile, *vt = tile + kBlockTokens * row_halves;
    const int kvh = blockIdx.y;
    const int groups = head_dim >> 3;
    const int pieces = kBlockTokens * groups;
    const size_t src0 = ((size_t)slot * n_kv_heads + kvh) * (size_t)page_elems +
                        (size_t)(first_block + (int)blockIdx.x) * (size_t)(kBlockTokens * head_dim);
    for (int p = threadIdx.x; p < pieces; p += 256) {
        const int d8 = p >> 5, key = p & 31;  // K piece (d / 8, key)
        *reinterpret_cast<h8 *>(kt + key * row_halves + d8 * 8) = *reinterpret_cast<const h8 *>(k_layer + src0 + (size_t)p * 8);
        const int d = p >> 2, c = p & 3;  // V piece (d, chunk)
        const h8 x = *reinterpret_cast<const h8 *>(v_layer + src0 + (size_t)p * 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) vt[v_key_at(c, i) * row_halves + d] = x[i];
    }
    __syncthreads();
    const long long dst0 = (long long)blockIdx.x * kBlockTokens * dst_stride + (long long)kvh * head_dim;
    for (int p = threadIdx.x; p < pieces; p += 256) {
        const int row = p / groups, g8 = p - row * groups;
        const long long off = dst0 + (long long)row * dst_stride + g8 * 8;
        if (k_dst) *reinterpret_cast<h8 *>(k_dst + off) = *reinterpret_cast<const h8 *>(kt + row * row_halves + g8 * 8);
        if (v_dst) *reinterpret_cast<h8 *>(v_dst + off) = *reinterpret_cast<const h8 *>(vt + row * row_halves + g8 * 8);
    }
}

static int launch_kv_read_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, _Float16 *k, _Float16 *v,
                               size_t stride, const int *positions = nullptr, int limit = 0) {
    const long long total = (long long)n_tokens * kv->n_kv_heads * kv->head_dim;
    const unsigned blocks = (unsigned)((total + 255) / 256);
    hipLaunchKernelGGL(kv_read_kernel, dim3(blocks), dim3(256), 0, kv->ctx->stream, kv->k[layer], kv->v[layer], k, v,
                       (long long)stride, (long long)kv->page_elems(), slot, kv->n_kv_heads, kv->head_dim, position, n_tokens,
                       positions, limit, kv->ring ? kv->capacity : 0);
    hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(kv->ctx, e, "kv_read_kernel launch");
}

// Whole blocks through the block kernel (16-byte aligned destinations only), ragged edges row by row.
int launch_kv_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k, tt_half *v, size_t stride) {
    _Float16 *kd = reinterpret_cast<_Float16 *>(k), *vd = reinterpret_cast<_Float16 *>(v);
    const int first_full = ((position + kBlockTokens - 1) / kBlockTokens) * kBlockTokens;
    const int last_full_end = ((position + n_tokens) / kBlockTokens) * kBlockTokens;
    const bool aligned = (((uintptr_t)kd | (uintptr_t)vd) & 15u) == 0 && (stride * 2) % 16 == 0;
    if (!aligned || last_full_end <= first_full) return launch_kv_read_rows(kv, layer, slot, position, n_tokens, kd, vd, stride);
    auto at = [&](_Float16 *p, int token) { return p ? p + (size_t)(token - position) * stride : nullptr; };
    if (first_full > position) {
        const int rc = launch_kv_read_rows(kv, layer, slot, position, first_full - position, kd, vd, stride);
        if (rc != TT_HIP_OK) return rc;
    }
    const int n_blocks = (last_full_end - first_full) / kBlockTokens;
    const size_t lds = (size_t)2 * kBlockTokens * (kv->head_dim + kAppendPad) * sizeof(_Float16);
    hipLaunchKernelGGL(kv_read_blocks_kernel, dim3((unsigned)n_blocks, (unsigned)kv->n_kv_heads), dim3(256), lds,
                       kv->ctx->stream, kv->k[layer], kv->v[layer], at(kd, first_full), at(vd, first_full), (long long)stride,
                       (long long)kv->page_elems(), slot, kv->n_kv_heads, kv->head_dim, first_full / kBlockTokens);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return hip_fail(kv->ctx, e, "kv_read_blocks_kernel launch");
    const int tail = position + n_tokens - last_full_end;
    if (tail > 0) return launch_kv_read_rows(kv, layer, slot, last_full_end, tail, at(kd, last_full_end), at(vd, last_full_end), stride);
    return TT_HIP_OK;
}

static int round_up_block(long long tokens) {
    return (int)(((tokens + kBlockTokens - 1) / kBlockTokens) * kBlockTokens);
}

// Allocates zero-filled stores for every layer at `capacity` tokens per slot.
// Zero fill matters: rows past a sequence's end inside its last 32-token block
// are multiplied by probability 0 in the P.V contraction and must be finite.
static int alloc_layers(tt_hip_kv *kv, int capacity, std::vector<_Float16 *> *k_out, std::vector<_Float16 *> *v_out) {
    const size_t bytes = (size_t)kv->n_slots * kv->n_kv_heads * (size_t)(capacity / kBlockTokens) * kv->block_bytes();
    k_out->assign(kv->n_layers, nullptr);
    v_out->assign(kv->n_layers, nullptr);
    for (int layer = 0; layer < kv->n_layers; ++layer) {
        for (auto *store : {k_out, v_out}) {
            void *p = nullptr;
            hipError_t e = hipMalloc(&p, bytes);
            if (e == hipSuccess) e = hipMemsetAsync(p, 0, bytes, kv->ctx->stream);
            if (e != hipSuccess) {
                if (p) (void)hipFree(p);
                for (auto *q : *k_out)
                    if (q) (void)hipFree(q);
                for (auto *q : *v_out)
                    if (q) (void)hipFree(q);
                k_out->clear();
                v_out->clear();
                return hip_fail(kv->ctx, e, "hipMalloc(KV store)");
            }
            (*store)[layer] = reinterpret_cast<_Float16 *>(p);
        }
    }
    return TT_HIP_OK;
}

}  // namespace tt

using namespace tt;

extern "C" {

tt_hip_kv *tt_hip_kv_create(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim, int n_slots,
                            int initial_capacity_tokens, int max_context_tokens, int *out_err) {
    return tt_hip_kv_create_quantized(ctx, n_layers, n_kv_heads, head_dim, n_slots, initial_capacity_tokens,
                                      max_context_tokens, 16, out_err);
}

tt_hip_kv *tt_hip_kv_create_ring(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim, int n_slots,
                                 int ring_capacity_tokens, int max_context_tokens, int bits, int *out_err) {
    tt_hip_kv *kv = tt_hip_kv_create_quantized(ctx, n_layers, n_kv_heads, head_dim, n_slots, ring_capacity_tokens,
                                               max_context_tokens, bits, out_err);
    if (kv) kv->ring = true;  // capacity = min(ring capacity, max context), both rounded up to whole blocks, and fixed
    return kv;
}

tt_hip_kv *tt_hip_kv_create_quantized(tt_hip_ctx *ctx, int n_layers, int n_kv_heads, int head_dim, int n_slots,
                                      int initial_capacity_tokens, int max_context_tokens, int bits, int *out_err) {
    auto fail = [&](int code) -> tt_hip_kv * {
        if (out_err) *out_err = code;
        return nullptr;
    };
    if (!ctx || n_layers <= 0 || n_kv_heads <= 0 || n_slots <= 0 || n_slots > TT_HIP_MAX_SLOTS ||
        initial_capacity_tokens <= 0 || max_context_tokens <= 0)
        return fail(TT_HIP_ERR_INVALID_ARGUMENT);
    if (head_dim != 64 && head_dim != 128 && head_dim != 256) return fail(TT_HIP_ERR_SHAPE);
    if (bits != 16 && bits != 8 && bits != 4) return fail(TT_HIP_ERR_INVALID_ARGUMENT);
    // Allocating would put hipMalloc and a memset node on a capturing stream: create caches outside a capture.
    if (ctx->capturing) return fail(TT_HIP_ERR_BUSY);
    if (hipSetDevice(ctx->device) != hipSuccess) return fail(TT_HIP_ERR_HIP);
    tt_hip_kv *kv = new (std::nothrow) tt_hip_kv();
    if (!kv) return fail(TT_HIP_ERR_OUT_OF_MEMORY);
    kv->ctx = ctx;
    kv->bits = bits;
    kv->n_layers = n_layers;
    kv->n_kv_heads = n_kv_heads;
    kv->head_dim = head_dim;
    kv->n_slots = n_slots;
    kv->max_context = round_up_block(max_context_tokens);
    // The kernels address a page through a 32-bit buffer resource, and their void loads must land
    // past its end: a page may not exceed 0x7ff00000 bytes (4.19 M tokens at fp16, D = 256).
    if ((unsigned long long)(kv->max_context / kBlockTokens) * kv->block_bytes() > 0x7ff00000ull) {
        delete kv;
        return fail(TT_HIP_ERR_CAPACITY);
    }
    int capacity = round_up_block(initial_capacity_tokens);
    if (capacity > kv->max_context) capacity = kv->max_context;
    kv->capacity = capacity;
    kv->positions.assign(n_slots, 0);
    int st = alloc_layers(kv, capacity, &kv->k, &kv->v);
    if (st != TT_HIP_OK) {
        delete kv;
        return fail(st);
    }
    if (out_err) *out_err = TT_HIP_OK;
    return kv;
}

void tt_hip_kv_destroy(tt_hip_kv *kv) {
    if (!kv) return;
    (void)hipSetDevice(kv->ctx->device);
    (void)hipStreamSynchronize(kv->ctx->stream);
    ++kv->ctx->generation;  // a graph captured over this cache must not replay
    for (auto *p : kv->k)
        if (p) (void)hipFree(p);
    for (auto *p : kv->v)
        if (p) (void)hipFree(p);
    delete kv;
}

int tt_hip_kv_capacity(const tt_hip_kv *kv) { return kv ? kv->capacity : -1; }
int tt_hip_kv_max_context(const tt_hip_kv *kv) { return kv ? kv->max_context : -1; }
int tt_hip_kv_position(const tt_hip_kv *kv, int slot) {
    return (kv && slot >= 0 && slot < kv->n_slots) ? kv->positions[slot] : -1;
}
int tt_hip_kv_precision_bits(const tt_hip_kv *kv) { return kv ? kv->bits : -1; }

int tt_hip_kv_row_layout(int elements, int bits, size_t *stride_bytes, size_t *value_bytes) {
    if (elements <= 0 || (bits != 16 && bits != 8 && bits != 4)) return TT_HIP_ERR_INVALID_ARGUMENT;
    size_t values = (size_t)elements * 2, stride = values;
    if (bits != 16) {
        values = ((((size_t)elements * bits + 7) / 8) + 1) & ~(size_t)1;
        stride = values + (size_t)((elements + kQuantGroup - 1) / kQuantGroup) * 2 * 2;
    }
    if (stride_bytes) *stride_bytes = stride;
    if (value_bytes) *value_bytes = values;
    return TT_HIP_OK;
}

size_t tt_hip_kv_token_stride_bytes(const tt_hip_kv *kv) {
    size_t stride = 0;
    if (kv) (void)tt_hip_kv_row_layout(kv->n_kv_heads * kv->head_dim, kv->bits, &stride, nullptr);
    return stride;
}
size_t tt_hip_kv_bytes(const tt_hip_kv *kv) { return kv ? kv->layer_bytes() * 2 * kv->n_layers : 0; }

static int check_rows(const tt_hip_kv *kv, int layer, int slot, int position, int n_tokens) {
    if (!kv) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (layer < 0 || layer >= kv->n_layers || slot < 0 || slot >= kv->n_slots) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (position < 0 || n_tokens < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (!kv->holds_rows(position, n_tokens)) return TT_HIP_ERR_CAPACITY;
    return TT_HIP_OK;
}

int tt_hip_kv_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k, const tt_half *v,
                     size_t src_token_stride) {
    int st = check_rows(kv, layer, slot, position, n_tokens);
    if (st != TT_HIP_OK) return st;
    if (!k || !v) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (src_token_stride < (size_t)kv->n_kv_heads * kv->head_dim) return TT_HIP_ERR_SHAPE;
    if (n_tokens == 0) return TT_HIP_OK;
    BusyGuard guard(kv->ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    if (kv->bits != 16) return launch_kvq_append(kv, layer, slot, kv->physical(position), n_tokens, k, v, src_token_stride);
    return launch_kv_append(kv, layer, slot, kv->physical(position), n_tokens, k, v, src_token_stride);
}

int tt_hip_kv_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k_out, tt_half *v_out,
                   size_t dst_token_stride) {
    int st = check_rows(kv, layer, slot, position, n_tokens);
    if (st != TT_HIP_OK) return st;
    if (!k_out && !v_out) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (dst_token_stride < (size_t)kv->n_kv_heads * kv->head_dim) return TT_HIP_ERR_SHAPE;
    if (n_tokens == 0) return TT_HIP_OK;
    BusyGuard guard(kv->ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    if (kv->bits != 16) return launch_kvq_read(kv, layer, slot, kv->physical(position), n_tokens, k_out, v_out, dst_token_stride);
    return launch_kv_read(kv, layer, slot, kv->physical(position), n_tokens, k_out, v_out, dst_token_stride);
}

int tt_hip_kv_gather(tt_hip_kv *kv, int layer, int slot, const int *positions, int n_tokens, tt_half *k_out, tt_half *v_out,
                     size_t dst_token_stride) {
    if (!kv) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (layer < 0 || layer >= kv->n_layers || slot < 0 || slot >= kv->n_slots || n_tokens < 0 || !positions)
        return TT_HIP_ERR_INVALID_ARGUMENT;
    if (!k_out && !v_out) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (dst_token_stride < (size_t)kv->n_kv_heads * kv->head_dim) return TT_HIP_ERR_SHAPE;
    if ((long long)n_tokens * kv->n_kv_heads * kv->head_dim > 0x7fffffffLL * 256) return TT_HIP_ERR_SHAPE;
    if (n_tokens == 0) return TT_HIP_OK;
    BusyGuard guard(kv->ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    const int limit = kv->ring ? kv->max_context : kv->capacity;  // the kernel gives zeros for positions outside [0, limit)
    if (kv->bits != 16) return launch_kvq_read(kv, layer, slot, 0, n_tokens, k_out, v_out, dst_token_stride, positions, limit);
    return launch_kv_read_rows(kv, layer, slot, 0, n_tokens, reinterpret_cast<_Float16 *>(k_out),
                               reinterpret_cast<_Float16 *>(v_out), dst_token_stride, positions, limit);
}

// Rows in the stored format, to (to_rows) or from device memory at k_rows / v_rows; `position` is physical.
static int move_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, void *k_rows, void *v_rows,
                     size_t row_stride_bytes, bool to_rows) {
    if (kv->bits != 16)
        return launch_kvq_rows(kv, layer, slot, position, n_tokens, static_cast<uint8_t *>(k_rows),
                               static_cast<uint8_t *>(v_rows), row_stride_bytes, to_rows);
    if (to_rows)
        return launch_kv_read(kv, layer, slot, position, n_tokens, static_cast<tt_half *>(k_rows),
                              static_cast<tt_half *>(v_rows), row_stride_bytes / 2);
    return launch_kv_append(kv, layer, slot, position, n_tokens, static_cast<const tt_half *>(k_rows),
                            static_cast<const tt_half *>(v_rows), row_stride_bytes / 2);
}

static int check_stored_rows(const tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, size_t row_stride_bytes) {
    int st = check_rows(kv, layer, slot, position, n_tokens);
    if (st != TT_HIP_OK) return st;
    if (row_stride_bytes < tt_hip_kv_token_stride_bytes(kv) || row_stride_bytes % 2 != 0) return TT_HIP_ERR_SHAPE;
    return TT_HIP_OK;
}

int tt_hip_kv_export_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, void *k_rows, void *v_rows,
                          size_t row_stride_bytes) {
    int st = check_stored_rows(kv, layer, slot, position, n_tokens, row_stride_bytes);
    if (st != TT_HIP_OK) return st;
    if (!k_rows && !v_rows) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (n_tokens == 0) return TT_HIP_OK;
    BusyGuard guard(kv->ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    return move_rows(kv, layer, slot, kv->physical(position), n_tokens, k_rows, v_rows, row_stride_bytes, true);
}

int tt_hip_kv_import_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const void *k_rows,
                          const void *v_rows, size_t row_stride_bytes) {
    int st = check_stored_rows(kv, layer, slot, position, n_tokens, row_stride_bytes);
    if (st != TT_HIP_OK) return st;
    if (!k_rows || !v_rows) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (n_tokens == 0) return TT_HIP_OK;
    BusyGuard guard(kv->ctx);
    if (!guard.ok) return TT_HIP_ERR_BUSY;
    return move_rows(kv, layer, slot, kv->physical(position), n_tokens, const_cast<void *>(k_rows),
                     const_cast<void *>(v_rows), row_stride_bytes, false);
}

int tt_hip_kv_advance(tt_hip_kv *kv, int slot, int n_tokens) {
    if (!kv || slot < 0 || slot >= kv->n_slots || n_tokens < 0) return TT_HIP_ERR_INVALID_ARGUMENT;
    if ((long long)kv->positions[slot] + n_tokens > kv->max_context) return TT_HIP_ERR_CAPACITY;
    kv->positions[slot] += n_tokens;
    return TT_HIP_OK;
}

int tt_hip_kv_rewind(tt_hip_kv *kv, int slot, int position) {
    if (!kv || slot < 0 || slot >= kv->n_slots) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (position < 0 || position > kv->positions[slot]) return TT_HIP_ERR_CURSOR;
    kv->positions[slot] = position;
    return TT_HIP_OK;
}

int tt_hip_kv_reset(tt_hip_kv *kv, int slot) {
    if (!kv || slot < -1 || slot >= kv->n_slots) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (slot == -1) {
        for (auto &p : kv->positions) p = 0;
    } else {
        kv->positions[slot] = 0;
    }
    return TT_HIP_OK;
}

int tt_hip_kv_expect_position(const tt_hip_kv *kv, int slot, int position) {
    if (!kv || slot < 0 || slot >= kv->n_slots) return TT_HIP_ERR_INVALID_ARGUMENT;
    return kv->positions[slot] == position ? TT_HIP_OK : TT_HIP_ERR_CURSOR;
}

int tt_hip_kv_reserve(tt_hip_kv *kv, int tokens) {
    if (!kv) return TT_HIP_ERR_INVALID_ARGUMENT;
    long long needed = tokens < 1 ? 1 : tokens;
    if (needed > kv->max_context) needed = kv->max_context;  // clamp, never fail (KVCacheManager+Storage.swift:101)
    if (kv->capacity >= needed || kv->ring) return TT_HIP_OK;  // a ring keeps its capacity
    BusyGuard guard(kv->ctx);
    // Growth allocates, copies and synchronises: none of that may happen on a capturing stream.
    if (!guard.ok || kv->ctx->capturing) return TT_HIP_ERR_BUSY;
    long long target = kv->capacity;
    while (target < needed) target *= 2;
    if (target > kv->max_context) target = kv->max_context;
    if (hipSetDevice(kv->ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    std::vector<_Float16 *> nk, nv;
    int st = alloc_layers(kv, (int)target, &nk, &nv);
    if (st != TT_HIP_OK) return st;
    // Every slot's live rows move to its new region; whole 32-token blocks are
    // copied, so a block's swizzled interior needs no re-layout.
    const size_t block = kv->block_bytes();
    const size_t old_page = kv->page_bytes(), new_page = (size_t)(target / kBlockTokens) * block;
    for (int layer = 0; layer < kv->n_layers; ++layer) {
        char *ok = reinterpret_cast<char *>(kv->k[layer]), *ov = reinterpret_cast<char *>(kv->v[layer]);
        char *tk = reinterpret_cast<char *>(nk[layer]), *tv = reinterpret_cast<char *>(nv[layer]);
        for (int s = 0; s < kv->n_slots; ++s) {
            const int used = kv->positions[s] < kv->capacity ? kv->positions[s] : kv->capacity;
            const size_t bytes = (size_t)(round_up_block(used) / kBlockTokens) * block;
            if (bytes == 0) continue;
            for (int h = 0; h < kv->n_kv_heads; ++h) {
                const size_t page = (size_t)s * kv->n_kv_heads + h;
                const size_t from = page * old_page, to = page * new_page;
                hipError_t e = hipMemcpyAsync(tk + to, ok + from, bytes, hipMemcpyDeviceToDevice, kv->ctx->stream);
                if (e == hipSuccess) e = hipMemcpyAsync(tv + to, ov + from, bytes, hipMemcpyDeviceToDevice, kv->ctx->stream);
                if (e != hipSuccess) {
                    (void)hipStreamSynchronize(kv->ctx->stream);
                    for (auto *p : nk) (void)hipFree(p);
                    for (auto *p : nv) (void)hipFree(p);
                    return hip_fail(kv->ctx, e, "hipMemcpyAsync(KV growth)");
                }
            }
        }
    }
    hipError_t e = hipStreamSynchronize(kv->ctx->stream);
    if (e != hipSuccess) {
        for (auto *p : nk) (void)hipFree(p);
        for (auto *p : nv) (void)hipFree(p);
        return hip_fail(kv->ctx, e, "hipStreamSynchronize(KV growth)");
    }
    for (auto *p : kv->k) (void)hipFree(p);
    for (auto *p : kv->v) (void)hipFree(p);
    kv->k.swap(nk);
    kv->v.swap(nv);
    kv->capacity = (int)target;
    ++kv->generation;
    ++kv->ctx->generation;  // graphs captured over the old stores are stale
    return TT_HIP_OK;
}

// ---- snapshots -----------------------------------------------------------------------------
// Wire format of KVCacheManager+Snapshot.swift:12-118: for every layer, slot 0's first
// min(position, capacity) rows of K as stored token-major rows (token stride = the row layout's:
// n_kv_heads * head_dim * 2 bytes at fp16, levels + scales + biases when quantised), then the
// same rows of V; `lengths` lists the 2 * n_layers segment sizes.

int tt_hip_kv_snapshot_segment_count(const tt_hip_kv *kv) { return kv ? 2 * kv->n_layers : 0; }

int tt_hip_kv_snapshot_segment_lengths(const tt_hip_kv *kv, int position, size_t *lengths, int n_lengths) {
    if (!kv || !lengths) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (position <= 0 || position > kv->max_context) return TT_HIP_ERR_CURSOR;  // invalidPosition (:13-15)
    if (n_lengths != 2 * kv->n_layers) return TT_HIP_ERR_SHAPE;
    const size_t stored = (size_t)(position < kv->capacity ? position : kv->capacity);
    const size_t stride = tt_hip_kv_token_stride_bytes(kv);
    for (int i = 0; i < n_lengths; ++i) lengths[i] = stored * stride;
    return TT_HIP_OK;
}

// True when `lengths` is what this cache would produce at `position` (invalidLayout otherwise).
static bool snapshot_layout_matches(const tt_hip_kv *kv, int position, const size_t *lengths, int n_lengths) {
    if (n_lengths != 2 * kv->n_layers) return false;
    std::vector<size_t> expected((size_t)n_lengths);
    if (tt_hip_kv_snapshot_segment_lengths(kv, position, expected.data(), n_lengths) != TT_HIP_OK) return false;
    for (int i = 0; i < n_lengths; ++i)
        if (expected[(size_t)i] != lengths[i]) return false;
    return true;
}

int tt_hip_kv_snapshot_export(tt_hip_kv *kv, const size_t *lengths, int n_lengths, void *host_dst, size_t dst_bytes,
                              size_t *offset) {
    if (!kv || !lengths || !host_dst || !offset) return TT_HIP_ERR_INVALID_ARGUMENT;
    const int position = kv->positions[0];
    if (position <= 0 || position > kv->max_context) return TT_HIP_ERR_CURSOR;
    if (!snapshot_layout_matches(kv, position, lengths, n_lengths)) return TT_HIP_ERR_SHAPE;  // appendSnapshotPayload :42-45
    size_t total = 0;
    for (int i = 0; i < n_lengths; ++i) total += lengths[i];
    if (*offset > dst_bytes || total > dst_bytes - *offset) return TT_HIP_ERR_SHAPE;
    BusyGuard guard(kv->ctx);
    if (!guard.ok || kv->ctx->capturing) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(kv->ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    const size_t stride = tt_hip_kv_token_stride_bytes(kv);
    const int stored = position < kv->capacity ? position : kv->capacity;
    const size_t seg = (size_t)stored * stride;
    char *stage = nullptr;  // K rows then V rows of one layer
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&stage), 2 * seg);
    if (e != hipSuccess) return hip_fail(kv->ctx, e, "hipMalloc(snapshot staging)");
    int rc = TT_HIP_OK;
    char *dst = static_cast<char *>(host_dst) + *offset;
    for (int layer = 0; layer < kv->n_layers && rc == TT_HIP_OK; ++layer) {
        rc = move_rows(kv, layer, 0, 0, stored, stage, stage + seg, stride, true);
        if (rc != TT_HIP_OK) break;
        e = hipMemcpyAsync(dst, stage, 2 * seg, hipMemcpyDeviceToHost, kv->ctx->stream);
        if (e == hipSuccess) e = hipStreamSynchronize(kv->ctx->stream);  // the staging buffer is reused by the next layer
        if (e != hipSuccess) rc = hip_fail(kv->ctx, e, "snapshot copy to host");
        dst += 2 * seg;
    }
    (void)hipFree(stage);
    if (rc == TT_HIP_OK) *offset += total;
    return rc;
}

int tt_hip_kv_snapshot_restore(tt_hip_kv *kv, int position, const size_t *lengths, int n_lengths, const void *host_src,
                               size_t src_bytes, size_t *offset) {
    if (!kv || !lengths || !offset) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (position <= 0 || position > kv->max_context) return TT_HIP_ERR_CURSOR;
    // Grow to the snapshot's position BEFORE comparing lengths: they are a function of capacity,
    // and a fresh receiver starts below a long prefix (restoreSnapshot :71-83).
    int rc = tt_hip_kv_reserve(kv, position);
    if (rc != TT_HIP_OK) return rc;
    if (!snapshot_layout_matches(kv, position, lengths, n_lengths)) return TT_HIP_ERR_SHAPE;
    size_t total = 0;
    for (int i = 0; i < n_lengths; ++i) total += lengths[i];
    if (!host_src || *offset > src_bytes || total > src_bytes - *offset) return TT_HIP_ERR_SHAPE;  // copySnapshotSegment's guard
    BusyGuard guard(kv->ctx);
    if (!guard.ok || kv->ctx->capturing) return TT_HIP_ERR_BUSY;
    if (hipSetDevice(kv->ctx->device) != hipSuccess) return TT_HIP_ERR_HIP;
    for (auto &p : kv->positions) p = 0;  // reset() (:88)
    const size_t stride = tt_hip_kv_token_stride_bytes(kv);
    const int stored = position < kv->capacity ? position : kv->capacity;
    const size_t seg = (size_t)stored * stride;
    char *stage = nullptr;
    hipError_t e = hipMalloc(reinterpret_cast<void **>(&stage), 2 * seg);
    if (e != hipSuccess) return hip_fail(kv->ctx, e, "hipMalloc(snapshot staging)");
    const char *src = static_cast<const char *>(host_src) + *offset;
    for (int layer = 0; layer < kv->n_layers && rc == TT_HIP_OK; ++layer) {
        e = hipMemcpyAsync(stage, src, 2 * seg, hipMemcpyHostToDevice, kv->ctx->stream);
        if (e != hipSuccess) {
            rc = hip_fail(kv->ctx, e, "snapshot copy from host");
            break;
        }
        rc = move_rows(kv, layer, 0, 0, stored, stage, stage + seg, stride, false);
        e = hipStreamSynchronize(kv->ctx->stream);  // the staging buffer is reused by the next layer
        if (e != hipSuccess && rc == TT_HIP_OK) rc = hip_fail(kv->ctx, e, "hipStreamSynchronize(snapshot restore)");
        src += 2 * seg;
    }
    (void)hipFree(stage);
    if (rc != TT_HIP_OK) return rc;
    kv->positions[0] = position;
    *offset += total;
    return TT_HIP_OK;
}

size_t tt_hip_kv_k_offset(int head_dim, int position, int d) { return k_offset(head_dim, position, d); }
size_t tt_hip_kv_v_offset(int head_dim, int position, int d) { return v_offset(head_dim, position, d); }

}  // extern "C"
