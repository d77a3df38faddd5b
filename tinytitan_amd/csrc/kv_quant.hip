// Quantised KV pages: the affine group quantiser fused with the cache write, the readers that
// give rows back (dequantised fp16, or the reference's stored row format) and the writer that
// takes stored rows in.
//
// Quantiser: kv_cache_quantize_affine (sources/TinyTitanCore/Metal/Quant/kv_cache_quantize.metal:7-73)
// as encoded by KVCacheQuantizer (sources/TinyTitan/Kernels/Quant/KVCacheQuantizer.swift:14-66): per
// token and group of 64 consecutive elements of the row, bias = minimum, scale = (maximum -
// minimum) / (2^bits - 1), level = round(clamp((x - bias) / scale)), all in fp32; scale and bias
// are stored as fp16.  Loader: attn_load_kv (sources/TinyTitanCore/Metal/Attention/attention.metal:89-117).
// Stored row format: KVCacheManager.rowLayout (KVCacheManager+Validation.swift:30-41).
#include <cstdint>

#include "internal.h"
#include "wave_ops.h"

namespace tt {

namespace {

struct QuantArgs {
    uint8_t *k_layer, *v_layer;
    long long page_bytes;
    int slot, n_kv_heads, head_dim, position, n_tokens;
    const int *positions;  // the read kernel only: row t is the row of positions[t]; outside [0, limit) gives zeros
    int limit, ring_capacity;
};

__device__ __forceinline__ uint8_t *block_of(const QuantArgs &a, bool is_v, int kvh, int pos, int bits) {
    return (is_v ? a.v_layer : a.k_layer) + ((size_t)a.slot * a.n_kv_heads + kvh) * (size_t)a.page_bytes +
           (size_t)(pos >> 5) * block_bytes(a.head_dim, bits);
}

// One wavefront per (group of 64 elements, token, K or V), four to a workgroup: a lane owns one element.
template <int BITS>
__global__ __launch_bounds__(256) void kvq_append_kernel(const QuantArgs a, const _Float16 *__restrict__ k_src,
                                                         const _Float16 *__restrict__ v_src, long long src_stride) {
    const int lane = threadIdx.x & 63, token = blockIdx.y;
    const bool is_v = blockIdx.z != 0;
    const int group_of_row = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (group_of_row * kQuantGroup >= a.n_kv_heads * a.head_dim) return;  // the whole wavefront
    const int flat = group_of_row * kQuantGroup + lane;
    const int kvh = flat / a.head_dim, d = flat - kvh * a.head_dim, group = d / kQuantGroup;
    const float value = (float)(is_v ? v_src : k_src)[(long long)token * src_stride + flat];
    float lo = value, hi = value;
    lo = group_min<32>(lo);  // DPP and permlane moves inside each half of the wavefront, one exchange through LDS across
    hi = group_max<32>(hi);
    lo = fminf(lo, __shfl_xor(lo, 32));
    hi = fmaxf(hi, __shfl_xor(hi, 32));
    constexpr float kLevels = BITS == 4 ? 15.0f : 255.0f;
    const float scale = hi > lo ? __fdiv_rn(hi - lo, kLevels) : 0.0f;
    float level = 0.0f;
    if (scale > 0.0f) level = roundf(fminf(fmaxf(__fdiv_rn(value - lo, scale), 0.0f), kLevels));
    const unsigned q = (unsigned)level;
    const int pos = a.position + token, key = pos & 31;
    uint8_t *block = block_of(a, is_v, kvh, pos, BITS);
    if constexpr (BITS == 8) {
        block[is_v ? vq_level_byte(8, key, d) : kq_level_byte(8, key, d)] = (uint8_t)q;
    } else if (!is_v) {
        const unsigned odd = __shfl_down(q, 1);  // dims (d, d + 1) share a byte, even d low
        if (!(lane & 1)) block[kq_level_byte(4, key, d)] = (uint8_t)(q | (odd << 4));
    } else {
        const unsigned upper = __shfl_down(q, 32);  // dims (d, d + 32) of this key share a byte
        if (lane < 32) block[vq_level_byte(4, key, d)] = (uint8_t)(q | (upper << 4));
    }
    if (lane == 0) {
        const _Float16 s = (_Float16)scale, b = (_Float16)lo;
        *reinterpret_cast<_Float16 *>(block + (is_v ? vq_scale_byte(a.head_dim, BITS, key, group)
                                                    : kq_scale_byte(a.head_dim, BITS, key, group))) = s;
        *reinterpret_cast<_Float16 *>(block + (is_v ? vq_bias_byte(a.head_dim, BITS, key, group)
                                                    : kq_bias_byte(a.head_dim, BITS, key, group))) = b;
    }
}

// Whole 32-token blocks of a chunk: one workgroup per (block, kv head, K or V).  A thread takes 16 bytes -- eight
// consecutive elements -- of a source row at a time, so a row is read as whole lines and the eight lanes that hold a
// group of 64 find its minimum and maximum with three exchanges; levels, scales and biases are put together in LDS
// as the block is stored, and the block leaves as whole lines, 16 bytes per thread.  The same arithmetic, element
// by element, as kvq_append_kernel: the stored bytes are the same.
template <int BITS>
__global__ __launch_bounds__(256) void kvq_append_blocks_kernel(const QuantArgs a, const _Float16 *__restrict__ k_src,
                                                                const _Float16 *__restrict__ v_src, long long src_stride,
                                                                int first_block) {
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    extern __shared__ __attribute__((aligned(16))) uint8_t image[];  // the block as it is stored
    const bool is_v = blockIdx.z != 0;
    const int kvh = blockIdx.y, D = a.head_dim, pieces_per_row = D >> 3;
    const _Float16 *src = (is_v ? v_src : k_src) + (long long)blockIdx.x * kBlockTokens * src_stride + (long long)kvh * D;
    constexpr float kLevels = BITS == 4 ? 15.0f : 255.0f;
    // 32 x D / 8 pieces, a multiple of 256 (D is a multiple of 64): every thread takes every turn of the loop, and the
    // eight lanes of a group -- eight consecutive, aligned pieces of one row -- are always together.
    for (int p = threadIdx.x; p < kBlockTokens * pieces_per_row; p += 256) {
        const int key = p / pieces_per_row, d8 = p - key * pieces_per_row, d0 = d8 * 8, group = d0 / kQuantGroup;
        const h8 x = *reinterpret_cast<const h8 *>(src + (long long)key * src_stride + d0);
        float value[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) value[i] = (float)x[i];
        float lo = value[0], hi = value[0];
#pragma unroll
        for (int i = 1; i < 8; ++i) {
            lo = fminf(lo, value[i]);
            hi = fmaxf(hi, value[i]);
        }
        lo = group_min<8>(lo);  // DPP moves, no trip through LDS
        hi = group_max<8>(hi);
        const float scale = hi > lo ? __fdiv_rn(hi - lo, kLevels) : 0.0f;
        unsigned q[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            float level = 0.0f;
            if (scale > 0.0f) level = roundf(fminf(fmaxf(__fdiv_rn(value[i] - lo, scale), 0.0f), kLevels));
            q[i] = (unsigned)level;
        }
        unsigned nibbles = 0;  // (4 bits) the eight levels, element i in bits 4 i .. 4 i + 3
#pragma unroll
        for (int i = 0; i < 8; ++i) nibbles |= q[i] << (4 * i);
        if (!is_v) {
            if constexpr (BITS == 8) {
                u2 w = {q[0] | (q[1] << 8) | (q[2] << 16) | (q[3] << 24), q[4] | (q[5] << 8) | (q[6] << 16) | (q[7] << 24)};
                *reinterpret_cast<u2 *>(image + kq_level_byte(8, key, d0)) = w;
            } else {
                *reinterpret_cast<unsigned *>(image + kq_level_byte(4, key, d0)) = nibbles;
            }
        } else if constexpr (BITS == 8) {
#pragma unroll
            for (int i = 0; i < 8; ++i) image[vq_level_byte(8, key, d0 + i)] = (uint8_t)q[i];
        } else {
            // dims (d, d + 32) of a key share a byte, d in the low nibble: the lane four pieces on holds d + 32
            const unsigned upper = __shfl_down(nibbles, 4);
            if (!(d8 & 4)) {
#pragma unroll
                for (int i = 0; i < 8; ++i)
                    image[vq_level_byte(4, key, d0 + i)] = (uint8_t)(((nibbles >> (4 * i)) & 15u) | (((upper >> (4 * i)) & 15u) << 4));
            }
        }
        if (!(d8 & 7)) {
            const _Float16 s = (_Float16)scale, b = (_Float16)lo;
            *reinterpret_cast<_Float16 *>(image + (is_v ? vq_scale_byte(D, BITS, key, group) : kq_scale_byte(D, BITS, key, group))) = s;
            *reinterpret_cast<_Float16 *>(image + (is_v ? vq_bias_byte(D, BITS, key, group) : kq_bias_byte(D, BITS, key, group))) = b;
        }
    }
    __syncthreads();
    uint8_t *block = block_of(a, is_v, kvh, (first_block + (int)blockIdx.x) * kBlockTokens, BITS);
    const int lines = (int)(block_bytes(D, BITS) >> 4);  // a block is a multiple of 16 bytes and 16-byte aligned in its page
    for (int p = threadIdx.x; p < lines; p += 256)
        *reinterpret_cast<u4 *>(block + (size_t)p * 16) = *reinterpret_cast<const u4 *>(image + (size_t)p * 16);
}

__device__ __forceinline__ unsigned level_at(const uint8_t *block, bool is_v, int bits, int key, int d) {
    if (bits == 8) return block[is_v ? vq_level_byte(8, key, d) : kq_level_byte(8, key, d)];
    if (!is_v) return (block[kq_level_byte(4, key, d)] >> (4 * (d & 1))) & 15u;
    return (block[vq_level_byte(4, key, d)] >> (4 * ((d >> 5) & 1))) & 15u;
}

__device__ __forceinline__ float param_at(const uint8_t *block, size_t byte) {
    return (float)*reinterpret_cast<const _Float16 *>(block + byte);
}

// One thread per (token, element): level * scale + bias in fp32, one rounding to fp16.
template <int BITS>
__global__ __launch_bounds__(256) void kvq_read_kernel(const QuantArgs a, _Float16 *__restrict__ k_dst,
                                                       _Float16 *__restrict__ v_dst, long long dst_stride) {
    const int per_token = a.n_kv_heads * a.head_dim;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)per_token * a.n_tokens) return;
    const bool is_v = blockIdx.y != 0;
    _Float16 *dst = is_v ? v_dst : k_dst;
    if (!dst) return;
    const int token = (int)(idx / per_token), flat = (int)(idx - (long long)token * per_token);
    const int kvh = flat / a.head_dim, d = flat - kvh * a.head_dim, group = d / kQuantGroup;
    int pos = a.position + token;
    if (a.positions) {
        pos = a.positions[token];
        if (pos < 0 || pos >= a.limit) {
            dst[(long long)token * dst_stride + flat] = (_Float16)0;
            return;
        }
        if (a.ring_capacity > 0) pos %= a.ring_capacity;
    }
    const int key = pos & 31;
    const uint8_t *block = block_of(a, is_v, kvh, pos, BITS);
    const float scale = param_at(block, is_v ? vq_scale_byte(a.head_dim, BITS, key, group) : kq_scale_byte(a.head_dim, BITS, key, group));
    const float bias = param_at(block, is_v ? vq_bias_byte(a.head_dim, BITS, key, group) : kq_bias_byte(a.head_dim, BITS, key, group));
    dst[(long long)token * dst_stride + flat] = (_Float16)((float)level_at(block, is_v, BITS, key, d) * scale + bias);
}

// Stored rows: [levels of all elements][fp16 scale per group][fp16 bias per group].  One thread
// per (token, byte of the row).  TO_ROWS: pages -> rows; otherwise rows -> pages, where a thread
// owns one byte of the PAGE so that no two threads write the same byte.
template <int BITS, bool TO_ROWS>
__global__ __launch_bounds__(256) void kvq_rows_kernel(const QuantArgs a, uint8_t *__restrict__ k_rows,
                                                       uint8_t *__restrict__ v_rows, long long row_stride) {
    const int elements = a.n_kv_heads * a.head_dim, groups = elements / kQuantGroup, gph = a.head_dim / kQuantGroup;
    const int value_bytes = elements * BITS / 8, row_bytes = value_bytes + groups * 4;
    const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (long long)row_bytes * a.n_tokens) return;
    const bool is_v = blockIdx.y != 0;
    uint8_t *rows = is_v ? v_rows : k_rows;
    if (!rows) return;
    const int token = (int)(idx / row_bytes), j = (int)(idx - (long long)token * row_bytes);
    const int pos = a.position + token, key = pos & 31;
    uint8_t *row = rows + (long long)token * row_stride;
    if (j >= value_bytes) {  // a byte of a scale or a bias
        const int h = (j - value_bytes) >> 1, byte = (j - value_bytes) & 1;
        const bool is_bias = h >= groups;
        const int gflat = is_bias ? h - groups : h, kvh = gflat / gph, group = gflat - kvh * gph;
        uint8_t *block = block_of(a, is_v, kvh, pos, BITS);
        const size_t at = (is_v ? (is_bias ? vq_bias_byte(a.head_dim, BITS, key, group) : vq_scale_byte(a.head_dim, BITS, key, group))
                                : (is_bias ? kq_bias_byte(a.head_dim, BITS, key, group) : kq_scale_byte(a.head_dim, BITS, key, group))) + byte;
        if (TO_ROWS) row[j] = block[at];
        else block[at] = row[j];
        return;
    }
    if (BITS == 8 || !is_v) {  // the page byte holds the same elements as the row byte
        const int flat = BITS == 8 ? j : 2 * j, kvh = flat / a.head_dim, d = flat - kvh * a.head_dim;
        uint8_t *block = block_of(a, is_v, kvh, pos, BITS);
        const size_t at = is_v ? vq_level_byte(BITS, key, d) : kq_level_byte(BITS, key, d);
        if (TO_ROWS) row[j] = block[at];
        else block[at] = row[j];
    } else if (TO_ROWS) {  // 4-bit V: row byte = dims (d, d + 1), page bytes = dims (d, d + 32)
        const int flat = 2 * j, kvh = flat / a.head_dim, d = flat - kvh * a.head_dim;
        const uint8_t *block = block_of(a, true, kvh, pos, 4);
        row[j] = (uint8_t)(level_at(block, true, 4, key, d) | (level_at(block, true, 4, key, d + 1) << 4));
    } else {  // thread j owns the page byte of dims (d, d + 32), d = 64 (w / 32) + w % 32
        const int half = a.head_dim / 2, kvh = j / half, w = j - kvh * half, d = 64 * (w >> 5) + (w & 31);
        const int lo_flat = kvh * a.head_dim + d, hi_flat = lo_flat + 32;
        const unsigned lo = (row[lo_flat >> 1] >> (4 * (lo_flat & 1))) & 15u, hi = (row[hi_flat >> 1] >> (4 * (hi_flat & 1))) & 15u;
        block_of(a, true, kvh, pos, 4)[vq_level_byte(4, key, d)] = (uint8_t)(lo | (hi << 4));
    }
}

// Whole blocks of one slot as fp16 pages in the fp16 block order (kv_layout.h), for the MFMA chunk
// kernel: one workgroup per (block, kv head), a thread per 16-byte piece of the result, every
// access a full line.  Value = level * scale + bias in fp32, one rounding to fp16.
template <int BITS>
__global__ __launch_bounds__(256) void kvq_dequant_blocks_kernel(const QuantArgs a, _Float16 *__restrict__ k_dst,
                                                                 _Float16 *__restrict__ v_dst, long long dst_page_elems) {
    typedef _Float16 h8 __attribute__((ext_vector_type(8)));
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const int block = blockIdx.x, kvh = blockIdx.y, D = a.head_dim, gph = D / kQuantGroup;
    const size_t src = ((size_t)a.slot * a.n_kv_heads + kvh) * (size_t)a.page_bytes + (size_t)block * block_bytes(D, BITS);
    const uint8_t *kb = a.k_layer + src, *vb = a.v_layer + src;
    const size_t dst = (size_t)kvh * (size_t)dst_page_elems + (size_t)block * (size_t)(kBlockTokens * D);
    const size_t levels = block_level_bytes(D, BITS);
    for (int p = threadIdx.x; p < kBlockTokens * D / 8; p += 256) {
        {  // K piece (d / 8, key): eight dims of one key, one scale and bias
            const int d8 = p >> 5, key = p & 31;
            const uint8_t *src = kb + kq_level_byte(BITS, key, d8 * 8);  // 8 (or 4) consecutive bytes
            unsigned lv[8];
            if constexpr (BITS == 8) {
                const u2 w = *reinterpret_cast<const u2 *>(src);
#pragma unroll
                for (int i = 0; i < 8; ++i) lv[i] = (w[i >> 2] >> (8 * (i & 3))) & 255u;
            } else {
                const unsigned w = *reinterpret_cast<const unsigned *>(src);
#pragma unroll
                for (int i = 0; i < 8; ++i) lv[i] = (w >> (4 * i)) & 15u;
            }
            const _Float16 *sb = reinterpret_cast<const _Float16 *>(kb + levels + (size_t)(key * gph + (d8 >> 3)) * 4);
            const float scale = (float)sb[0], bias = (float)sb[1];
            h8 o;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (_Float16)((float)lv[i] * scale + bias);
            *reinterpret_cast<h8 *>(k_dst + dst + (size_t)p * 8) = o;
        }
        {  // V piece (d, chunk): one dim of eight keys, a scale and a bias per key
            const int d = p >> 2, chunk = p & 3;
            const u2 w = *reinterpret_cast<const u2 *>(vb + vq_level_byte(BITS, v_key_at(chunk, 0), d));  // the chunk's 8 keys
            const int shift = BITS == 8 ? 0 : 4 * ((d >> 5) & 1);
            unsigned lv[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) lv[i] = (w[i >> 2] >> (8 * (i & 3) + shift)) & (BITS == 8 ? 255u : 15u);
            const size_t params = levels + (size_t)((d >> 6) * kBlockTokens + chunk * 8) * 2;
            const h8 scale = *reinterpret_cast<const h8 *>(vb + params);
            const h8 bias = *reinterpret_cast<const h8 *>(vb + params + (size_t)gph * kBlockTokens * 2);
            h8 o;
#pragma unroll
            for (int i = 0; i < 8; ++i) o[i] = (_Float16)((float)lv[i] * (float)scale[i] + (float)bias[i]);
            *reinterpret_cast<h8 *>(v_dst + dst + (size_t)p * 8) = o;
        }
    }
}

QuantArgs quant_args(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens) {
    QuantArgs a;
    a.k_layer = reinterpret_cast<uint8_t *>(kv->k[layer]);
    a.v_layer = reinterpret_cast<uint8_t *>(kv->v[layer]);
    a.page_bytes = (long long)kv->page_bytes();
    a.slot = slot;
    a.n_kv_heads = kv->n_kv_heads;
    a.head_dim = kv->head_dim;
    a.position = position;
    a.n_tokens = n_tokens;
    a.positions = nullptr;
    a.limit = 0;
    a.ring_capacity = kv->ring ? kv->capacity : 0;
    return a;
}

int launched(tt_hip_kv *kv, const char *what) {
    const hipError_t e = hipGetLastError();
    return e == hipSuccess ? TT_HIP_OK : hip_fail(kv->ctx, e, what);
}

}  // namespace

static int launch_kvq_append_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const _Float16 *ks,
                                  const _Float16 *vs, size_t stride) {
    const QuantArgs a = quant_args(kv, layer, slot, position, n_tokens);
    const dim3 grid((unsigned)((kv->n_kv_heads * kv->head_dim / kQuantGroup + 3) / 4), (unsigned)n_tokens, 2);
    if (kv->bits == 8) hipLaunchKernelGGL(kvq_append_kernel<8>, grid, dim3(256), 0, kv->ctx->stream, a, ks, vs, (long long)stride);
    else hipLaunchKernelGGL(kvq_append_kernel<4>, grid, dim3(256), 0, kv->ctx->stream, a, ks, vs, (long long)stride);
    return launched(kv, "kvq_append_kernel launch");
}

// Rows that cover whole 32-token blocks go through the block kernel (16-byte aligned sources only); the ragged head
// and tail of the range, and single decode rows, go a wavefront per group.
int launch_kvq_append(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, const tt_half *k, const tt_half *v,
                      size_t stride) {
    const _Float16 *ks = reinterpret_cast<const _Float16 *>(k), *vs = reinterpret_cast<const _Float16 *>(v);
    const int first_full = ((position + kBlockTokens - 1) / kBlockTokens) * kBlockTokens;
    const int last_full_end = ((position + n_tokens) / kBlockTokens) * kBlockTokens;
    const bool aligned = (((uintptr_t)ks | (uintptr_t)vs) & 15u) == 0 && (stride * 2) % 16 == 0;
    // Short chunks go by rows altogether: a block's workgroup quantises its 32 tokens group by group, and with few
    // blocks that chain is the launch's time (32 tokens 6.1 us by blocks, 2.3 us by rows; 512 tokens 6.5 / 4.2; 1024
    // tokens 6.6 / 6.5; 4096 tokens 8.4 / 19.9); with a ragged head or tail the blocks come with one or two more
    // launches (1024 tokens 10.9 us against 6.5 by rows).
    const bool ragged = first_full > position || last_full_end < position + n_tokens;
    const bool by_rows = n_tokens <= 768 || (ragged && n_tokens <= 2048);
    if (!aligned || last_full_end <= first_full || by_rows) return launch_kvq_append_rows(kv, layer, slot, position, n_tokens, ks, vs, stride);
    if (first_full > position) {
        const int rc = launch_kvq_append_rows(kv, layer, slot, position, first_full - position, ks, vs, stride);
        if (rc != TT_HIP_OK) return rc;
    }
    const size_t skip = (size_t)(first_full - position) * stride;
    const int n_blocks = (last_full_end - first_full) / kBlockTokens;
    const QuantArgs a = quant_args(kv, layer, slot, first_full, n_blocks * kBlockTokens);
    const dim3 grid((unsigned)n_blocks, (unsigned)kv->n_kv_heads, 2);
    const size_t lds = block_bytes(kv->head_dim, kv->bits);
    if (kv->bits == 8)
        hipLaunchKernelGGL(kvq_append_blocks_kernel<8>, grid, dim3(256), lds, kv->ctx->stream, a, ks + skip, vs + skip, (long long)stride,
                           first_full / kBlockTokens);
    else
        hipLaunchKernelGGL(kvq_append_blocks_kernel<4>, grid, dim3(256), lds, kv->ctx->stream, a, ks + skip, vs + skip, (long long)stride,
                           first_full / kBlockTokens);
    const int rc = launched(kv, "kvq_append_blocks_kernel launch");
    if (rc != TT_HIP_OK) return rc;
    const int tail = position + n_tokens - last_full_end;
    if (tail > 0) {
        const size_t tskip = (size_t)(last_full_end - position) * stride;
        return launch_kvq_append_rows(kv, layer, slot, last_full_end, tail, ks + tskip, vs + tskip, stride);
    }
    return TT_HIP_OK;
}

int launch_kvq_read(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, tt_half *k, tt_half *v, size_t stride,
                    const int *positions, int limit) {
    QuantArgs a = quant_args(kv, layer, slot, position, n_tokens);
    a.positions = positions;
    a.limit = limit;
    const long long total = (long long)n_tokens * kv->n_kv_heads * kv->head_dim;
    const dim3 grid((unsigned)((total + 255) / 256), 2);
    _Float16 *kd = reinterpret_cast<_Float16 *>(k), *vd = reinterpret_cast<_Float16 *>(v);
    if (kv->bits == 8) hipLaunchKernelGGL(kvq_read_kernel<8>, grid, dim3(256), 0, kv->ctx->stream, a, kd, vd, (long long)stride);
    else hipLaunchKernelGGL(kvq_read_kernel<4>, grid, dim3(256), 0, kv->ctx->stream, a, kd, vd, (long long)stride);
    return launched(kv, "kvq_read_kernel launch");
}

// Blocks [0, n_blocks) of `slot`, every kv head, as fp16 pages of dst_page_elems halves each.
int launch_kvq_dequant_blocks(tt_hip_kv *kv, int layer, int slot, int n_blocks, _Float16 *k_dst, _Float16 *v_dst,
                              size_t dst_page_elems) {
    const QuantArgs a = quant_args(kv, layer, slot, 0, n_blocks * kBlockTokens);
    const dim3 grid((unsigned)n_blocks, (unsigned)kv->n_kv_heads);
    if (kv->bits == 8)
        hipLaunchKernelGGL(kvq_dequant_blocks_kernel<8>, grid, dim3(256), 0, kv->ctx->stream, a, k_dst, v_dst, (long long)dst_page_elems);
    else
        hipLaunchKernelGGL(kvq_dequant_blocks_kernel<4>, grid, dim3(256), 0, kv->ctx->stream, a, k_dst, v_dst, (long long)dst_page_elems);
    return launched(kv, "kvq_dequant_blocks_kernel launch");
}

// to_rows: pages -> stored rows at k_rows / v_rows (either may be null); otherwise the reverse.
int launch_kvq_rows(tt_hip_kv *kv, int layer, int slot, int position, int n_tokens, uint8_t *k_rows, uint8_t *v_rows,
                    size_t row_stride, bool to_rows) {
    const QuantArgs a = quant_args(kv, layer, slot, position, n_tokens);
    const long long row_bytes = (long long)kv->n_kv_heads * kv->head_dim * kv->bits / 8 + (long long)kv->n_kv_heads * kv->head_dim / kQuantGroup * 4;
    const dim3 grid((unsigned)((row_bytes * n_tokens + 255) / 256), 2);
    hipStream_t s = kv->ctx->stream;
    if (kv->bits == 8 && to_rows) hipLaunchKernelGGL((kvq_rows_kernel<8, true>), grid, dim3(256), 0, s, a, k_rows, v_rows, (long long)row_stride);
    else if (kv->bits == 8) hipLaunchKernelGGL((kvq_rows_kernel<8, false>), grid, dim3(256), 0, s, a, k_rows, v_rows, (long long)row_stride);
    else if (to_rows) hipLaunchKernelGGL((kvq_rows_kernel<4, true>), grid, dim3(256), 0, s, a, k_rows, v_rows, (long long)row_stride);
    else hipLaunchKernelGGL((kvq_rows_kernel<4, false>), grid, dim3(256), 0, s, a, k_rows, v_rows, (long long)row_stride);
    return launched(kv, "kvq_rows_kernel launch");
}

}  // namespace tt
