// Split-K flash attention over the swizzled KV pages: GQA decode, multi-row
// verify and (as a first path) causal prefill, on gfx950 MFMA.
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
#include "internal.h"

namespace tt {

typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

constexpr float kNegBig = -1.0e30f;  // finite stand-in for "no key seen yet"
constexpr int kLdsPad = 4;           // floats of padding per staged O row

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

__device__ __forceinline__ h8 load_h8(const _Float16 *p, bool aligned) {
    if (aligned) return *reinterpret_cast<const h8 *>(p);
    h8 r;
#pragma unroll
    for (int j = 0; j < 8; ++j) r[j] = p[j];
    return r;
}

// Tile decoding shared by both kernels.
struct TileInfo {
    int kvh, hsub, tok_tile, t0, tile_rows, tile_end, start, total;
};

__device__ __forceinline__ TileInfo tile_info(const SplitKArgs &a, int tile, int seq) {
    TileInfo t;
    t.tok_tile = tile % a.tok_tiles;
    t.hsub = (tile / a.tok_tiles) % a.hsubs;
    t.kvh = tile / (a.tok_tiles * a.hsubs);
    t.start = a.start[seq];
    t.total = a.total[seq];
    t.t0 = t.tok_tile * a.tt;
    t.tile_rows = min(a.tt, a.rows - t.t0);
    t.tile_end = max(0, min(t.total, t.start + t.t0 + t.tile_rows));  // keys visible to the tile's last row
    return t;
}

// Final value of one output element: normalise, gate in fp32, round once.
__device__ __forceinline__ void store_out4(const SplitKArgs &a, int seq, int tok, int head, int d, int D, f4 o,
                                           float inv_l) {
    f4 r = o * inv_l;
    if (a.gate) {
        const _Float16 *gp = a.gate + seq * a.g_seq_stride + tok * a.g_tok_stride + (long long)head * D + d;
        float g0, g1, g2, g3;
        if (a.aligned) {
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
    if (a.aligned) {
        h4 hv = {(_Float16)r[0], (_Float16)r[1], (_Float16)r[2], (_Float16)r[3]};
        *reinterpret_cast<h4 *>(op) = hv;
    } else {
        op[0] = (_Float16)r[0]; op[1] = (_Float16)r[1]; op[2] = (_Float16)r[2]; op[3] = (_Float16)r[3];
    }
}

// ---------------------------------------------------------------------------
// Pass 1.  grid = (split, tile, sequence); WAVES wavefronts per workgroup, wave
// w takes key blocks w, w + WAVES, ... of the split; the workgroup merges its
// waves through LDS and writes one partial (or the final rows when the launch
// has a single split).
// ---------------------------------------------------------------------------
template <int D, int NT, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void attn_splitk_kernel(const SplitKArgs a) {
    extern __shared__ float lds[];
    constexpr int LN = NT;             // lanes per lane group
    constexpr int ROW = D + kLdsPad;   // staged O row stride in floats
    constexpr int REGION = NT * ROW + NT * 2;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int li = lane & (LN - 1);
    const int g = lane / LN;
    const int split = blockIdx.x, tile = blockIdx.y, seq = blockIdx.z;
    const TileInfo ti = tile_info(a, tile, seq);
    const int k_begin = split * a.split_len;
    if (k_begin >= ti.tile_end && split != 0) return;  // split 0 always runs so that an empty range yields zeros
    const int k_end = min(k_begin + a.split_len, ti.tile_end);

    // This lane's query row.
    const int t_local = li / a.gh;
    const int hg = li - t_local * a.gh;
    const bool valid = t_local < ti.tile_rows;
    const int tok = ti.t0 + t_local;
    const int head = ti.kvh * a.group + ti.hsub * a.gh + hg;
    const int lim = valid ? min(ti.total, ti.start + tok + 1) : 0;  // keys [0, lim) are visible

    const size_t page = ((size_t)a.slot[seq] * a.n_kv_heads + ti.kvh) * (size_t)a.page_elems;
    const _Float16 *kp = a.k_layer + page;
    const _Float16 *vp = a.v_layer + page;
    const bool aligned = a.aligned != 0;

    float m = kNegBig, l = 0.0f;

    if constexpr (NT == 32) {
        constexpr int KS = D / 16, MT = D / 32;
        h8 qf[KS];
        {
            const _Float16 *qp = a.q + seq * a.q_seq_stride + tok * a.q_tok_stride + (long long)head * D;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                if (valid) qf[s] = load_h8(qp + 16 * s + 8 * g, aligned);
                else qf[s] = (h8)(_Float16)0;
            }
        }
        f16v o[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) o[mt] = (f16v)0.0f;

        for (int b = (k_begin >> 5) + wave; (b << 5) < k_end; b += WAVES) {
            const _Float16 *kb = kp + (size_t)b * (32 * D);
            const _Float16 *vb = vp + (size_t)b * (32 * D);
            h8 kf[KS];
            h8 vf[MT][2];
#pragma unroll
            for (int s = 0; s < KS; ++s) kf[s] = *reinterpret_cast<const h8 *>(kb + ((2 * s + g) * 32 + li) * 8);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 2; ++t)
                    vf[mt][t] = *reinterpret_cast<const h8 *>(vb + ((32 * mt + li) * 4 + 2 * t + g) * 8);
            f16v s = (f16v)0.0f;
#pragma unroll
            for (int st = 0; st < KS; ++st) s = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[st], qf[st], s, 0, 0, 0);
            const int kbase = b << 5;
            const bool need_mask = __any(kbase + 32 > lim);
            float mx = kNegBig;
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                float x = s[v] * a.scale_log2e;
                if (need_mask) {
                    const int key = kbase + 8 * (v >> 2) + 4 * g + (v & 3);
                    if (key >= lim) x = -INFINITY;
                }
                s[v] = x;
                mx = fmaxf(mx, x);
            }
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m, mx);
            const float alpha = fast_exp2(m - m_new);
            float psum = 0.0f;
            h8 pf[2];
#pragma unroll
            for (int v = 0; v < 16; ++v) {
                const float p = fast_exp2(s[v] - m_new);
                psum += p;
                pf[v >> 3][v & 7] = (_Float16)p;
            }
            l = l * alpha + psum;
            m = m_new;
            if (!__all(alpha == 1.0f)) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt)
#pragma unroll
                for (int t = 0; t < 2; ++t) o[mt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(vf[mt][t], pf[t], o[mt], 0, 0, 0);
        }
        l += __shfl_xor(l, 32);
        float *region = lds + wave * REGION;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int vq = 0; vq < 4; ++vq) {
                f4 x = {o[mt][4 * vq], o[mt][4 * vq + 1], o[mt][4 * vq + 2], o[mt][4 * vq + 3]};
                *reinterpret_cast<f4 *>(region + li * ROW + 32 * mt + 8 * vq + 4 * g) = x;
            }
        if (g == 0) {
            region[NT * ROW + 2 * li] = m;
            region[NT * ROW + 2 * li + 1] = l;
        }
    } else {
        constexpr int KS = D / 32, MT = D / 16;
        h8 qf[KS];
        {
            const _Float16 *qp = a.q + seq * a.q_seq_stride + tok * a.q_tok_stride + (long long)head * D;
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                if (valid) qf[s] = load_h8(qp + 32 * s + 8 * g, aligned);
                else qf[s] = (h8)(_Float16)0;
            }
        }
        f4 o[MT];
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) o[mt] = (f4)0.0f;
        const int ka = li < 8 ? li : li + 8;            // keys of S^T tile a: {0-7, 16-23}; tile b: +8
        const int kreg = (g & 1) * 4 + (g >> 1) * 16;   // first key of this lane's tile-a results

        for (int b = (k_begin >> 5) + wave; (b << 5) < k_end; b += WAVES) {
            const _Float16 *kb = kp + (size_t)b * (32 * D);
            const _Float16 *vb = vp + (size_t)b * (32 * D);
            h8 kfa[KS], kfb[KS], vf[MT];
#pragma unroll
            for (int s = 0; s < KS; ++s) {
                kfa[s] = *reinterpret_cast<const h8 *>(kb + ((4 * s + g) * 32 + ka) * 8);
                kfb[s] = *reinterpret_cast<const h8 *>(kb + ((4 * s + g) * 32 + ka + 8) * 8);
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) vf[mt] = *reinterpret_cast<const h8 *>(vb + ((16 * mt + li) * 4 + g) * 8);
            f4 sa = (f4)0.0f, sb = (f4)0.0f;
#pragma unroll
            for (int st = 0; st < KS; ++st) {
                sa = __builtin_amdgcn_mfma_f32_16x16x32_f16(kfa[st], qf[st], sa, 0, 0, 0);
                sb = __builtin_amdgcn_mfma_f32_16x16x32_f16(kfb[st], qf[st], sb, 0, 0, 0);
            }
            const int kbase = (b << 5) + kreg;
            const bool need_mask = __any((b << 5) + 32 > lim);
            float mx = kNegBig;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                float xa = sa[v] * a.scale_log2e, xb = sb[v] * a.scale_log2e;
                if (need_mask) {
                    if (kbase + v >= lim) xa = -INFINITY;
                    if (kbase + 8 + v >= lim) xb = -INFINITY;
                }
                sa[v] = xa;
                sb[v] = xb;
                mx = fmaxf(mx, fmaxf(xa, xb));
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16));
            mx = fmaxf(mx, __shfl_xor(mx, 32));
            const float m_new = fmaxf(m, mx);
            const float alpha = fast_exp2(m - m_new);
            float psum = 0.0f;
            h8 pf;
#pragma unroll
            for (int v = 0; v < 4; ++v) {
                const float pa = fast_exp2(sa[v] - m_new), pb = fast_exp2(sb[v] - m_new);
                psum += pa + pb;
                pf[v] = (_Float16)pa;
                pf[4 + v] = (_Float16)pb;
            }
            l = l * alpha + psum;
            m = m_new;
            if (!__all(alpha == 1.0f)) {
#pragma unroll
                for (int mt = 0; mt < MT; ++mt) o[mt] *= alpha;
            }
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) o[mt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(vf[mt], pf, o[mt], 0, 0, 0);
        }
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        float *region = lds + wave * REGION;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) *reinterpret_cast<f4 *>(region + li * ROW + 16 * mt + 4 * g) = o[mt];
        if (g == 0) {
            region[NT * ROW + 2 * li] = m;
            region[NT * ROW + 2 * li + 1] = l;
        }
    }
    __syncthreads();

    // Merge the waves' states; every thread takes (row, 4 dims) items.
    const int n_valid = ti.tile_rows * a.gh;
    constexpr int D4 = D / 4;
    const size_t pbase = (((size_t)seq * a.n_tiles + tile) * a.n_splits_max + split) * NT;
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
            store_out4(a, seq, ti.t0 + tl, hh, d, D, acc, lsum > 0.0f ? 1.0f / lsum : 0.0f);
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
// grid = (row within tile, tile, sequence), 256 threads: wave w folds splits
// w, w + 4, ... online, lanes hold 4 output dims each, then the four waves
// merge through LDS.  All-empty input yields zeros (attention.metal:418-427).
// ---------------------------------------------------------------------------
template <int D, int NT>
__global__ __launch_bounds__(256) void attn_combine_kernel(const SplitKArgs a) {
    constexpr int D4 = D / 4;
    __shared__ float sm[4][D + 2];
    const int n = blockIdx.x, tile = blockIdx.y, seq = blockIdx.z;
    const TileInfo ti = tile_info(a, tile, seq);
    if (n >= ti.tile_rows * a.gh) return;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    int n_splits = (ti.tile_end + a.split_len - 1) / a.split_len;
    if (n_splits < 1) n_splits = 1;
    const size_t tbase = ((size_t)seq * a.n_tiles + tile) * a.n_splits_max;
    float m = kNegBig, l = 0.0f;
    f4 acc = (f4)0.0f;
    const bool active = lane < D4;
    for (int s = wave; s < n_splits; s += 4) {
        const size_t row = (tbase + s) * NT + n;
        const float ms = a.part_ml[row * 2], ls = a.part_ml[row * 2 + 1];
        f4 os = (f4)0.0f;
        if (active) os = *reinterpret_cast<const f4 *>(a.part_o + row * D + lane * 4);
        const float m_new = fmaxf(m, ms);
        const float f_old = fast_exp2(m - m_new), f_new = fast_exp2(ms - m_new);
        acc = acc * f_old + os * f_new;
        l = l * f_old + ls * f_new;
        m = m_new;
    }
    if (active) *reinterpret_cast<f4 *>(&sm[wave][lane * 4]) = acc;
    if (lane == 0) {
        sm[wave][D] = m;
        sm[wave][D + 1] = l;
    }
    __syncthreads();
    if (wave == 0 && active) {
        float ms = kNegBig;
#pragma unroll
        for (int w = 0; w < 4; ++w) ms = fmaxf(ms, sm[w][D]);
        f4 o = (f4)0.0f;
        float lsum = 0.0f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const float f = fast_exp2(sm[w][D] - ms);
            lsum += f * sm[w][D + 1];
            o += f * *reinterpret_cast<const f4 *>(&sm[w][lane * 4]);
        }
        const int tl = n / a.gh;
        const int hh = ti.kvh * a.group + ti.hsub * a.gh + (n - tl * a.gh);
        store_out4(a, seq, ti.t0 + tl, hh, lane * 4, D, o, lsum > 0.0f ? 1.0f / lsum : 0.0f);
    }
}

// ---------------------------------------------------------------------------
// Host side: planning and launch.
// ---------------------------------------------------------------------------

static size_t lds_bytes_for(int D, int NT, int waves) {
    return (size_t)waves * ((size_t)NT * (D + kLdsPad) + (size_t)NT * 2) * sizeof(float);
}

int plan_launch(const tt_hip_ctx *ctx, int kind, int n_seq, int n_q_heads, int n_kv_heads, int head_dim, int rows,
                long long total_keys, int max_keys, LaunchPlan *plan) {
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
    }
    p.tt = p.nt / p.gh;
    p.hsubs = group / p.gh;
    p.tok_tiles = (rows + p.tt - 1) / p.tt;
    p.n_tiles = n_kv_heads * p.hsubs * p.tok_tiles;
    p.waves = 4;
    const int min_split = 32 * p.waves;
    int split_len;
    if (ctx->split_override > 0) {
        split_len = ((ctx->split_override + 31) / 32) * 32;
    } else if (kind == 1) {
        split_len = ((max_keys + 31) / 32) * 32;  // prefill tiles are plentiful: no split
    } else {
        // Aim at ~2 workgroups per CU; never less than one key block per wave.
        const long long target_wgs = 2LL * ctx->n_cus;
        const long long key_work = total_keys * p.n_tiles;
        long long per_wg = (key_work + target_wgs - 1) / target_wgs;
        split_len = (int)(((per_wg + min_split - 1) / min_split) * min_split);
    }
    if (split_len < 32) split_len = 32;
    p.split_len = split_len;
    p.n_splits_max = max_keys > 0 ? (max_keys + split_len - 1) / split_len : 1;
    if (p.n_splits_max < 1) p.n_splits_max = 1;
    p.workgroups = (long long)p.n_splits_max * p.n_tiles * n_seq;
    p.lds_bytes = lds_bytes_for(head_dim, p.nt, p.waves);
    *plan = p;
    return TT_HIP_OK;
}

template <int D, int NT, int WAVES>
static int launch_one(tt_hip_ctx *ctx, const LaunchPlan &plan, int n_seq, const SplitKArgs &args) {
    static bool attr_set[16] = {false};
    auto kernel = attn_splitk_kernel<D, NT, WAVES>;
    if (ctx->device < 16 && !attr_set[ctx->device]) {
        if (ctx->capturing) return TT_HIP_ERR_BUSY;  // first use configures the kernel: do it eagerly
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds_bytes);
        if (e != hipSuccess) return hip_fail(ctx, e, "hipFuncSetAttribute(max dynamic LDS)");
        attr_set[ctx->device] = true;
    }
    dim3 grid((unsigned)plan.n_splits_max, (unsigned)plan.n_tiles, (unsigned)n_seq);
    const bool timed = ctx->profiling && !ctx->capturing && ctx->prof_used + 2 <= ctx->prof_events.size();
    if (timed) (void)hipEventRecord(ctx->prof_events[ctx->prof_used], ctx->stream);
    hipLaunchKernelGGL(kernel, grid, dim3(WAVES * 64), plan.lds_bytes, ctx->stream, args);
    hipError_t e = hipGetLastError();
    if (timed) {
        (void)hipEventRecord(ctx->prof_events[ctx->prof_used + 1], ctx->stream);
        ctx->prof_used += 2;
    }
    if (e != hipSuccess) return hip_fail(ctx, e, "attn_splitk_kernel launch");
    if (plan.n_splits_max > 1) {
        dim3 cgrid((unsigned)NT, (unsigned)plan.n_tiles, (unsigned)n_seq);
        hipLaunchKernelGGL((attn_combine_kernel<D, NT>), cgrid, dim3(256), 0, ctx->stream, args);
        e = hipGetLastError();
        if (e != hipSuccess) return hip_fail(ctx, e, "attn_combine_kernel launch");
    }
    return TT_HIP_OK;
}

int launch_splitk(tt_hip_ctx *ctx, const LaunchPlan &plan, int head_dim, int n_seq, const SplitKArgs &args) {
    if (n_seq > kMaxSeqPerLaunch || plan.waves != 4) return TT_HIP_ERR_INVALID_ARGUMENT;
    if (plan.n_tiles > 65535 || n_seq > 65535) return TT_HIP_ERR_SHAPE;
#define TT_CASE(DD, NN) \
    if (head_dim == DD && plan.nt == NN) return launch_one<DD, NN, 4>(ctx, plan, n_seq, args);
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
