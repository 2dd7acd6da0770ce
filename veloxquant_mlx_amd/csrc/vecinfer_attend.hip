// Attention straight from VecInfer codebook indices (gfx950, wave64): neither keys nor values
// are ever materialised.
//
//   scores   q~ . k~^[t] = sum_j LUT[j][k_idx[t][j]],  LUT[j][c] = q~[j*sub .. ] . key_codebook[c]
//   output   sum_t P[t] v^[t] = sum_j sum_c W[j][c] value_codebook[c],  W[j][c] = sum of P[t] over
//            the tokens whose j-th value index is c
//
// so a token costs n_sub table look-ups and n_sub additions into a histogram per query row,
// whatever the head dimension; the histogram meets the value codebook once, at the end.  Both
// tables live in LDS.  One block of four waves per (kv head, tile of RB query rows, token
// split); a lane is a token.  The softmax reference is common to the block and moves lazily
// (only when a super-tile's maximum exceeds it by 2^8), in which case the histogram is
// rescaled.  Every block writes one (max, sum, accumulator) partial per row; the merge kernel
// of the packed-cache attention combines them.
#include "attend.hpp"
#include "vecinfer.hpp"

namespace vq {

constexpr int LA_THREADS = 256, LA_WAVES = 4;
constexpr int LA_TILES = 2;                       // 64-token tiles a wave holds scores of between the two phases
constexpr int LA_SUPER = LA_WAVES * LA_TILES * 64;   // tokens a block takes per step
constexpr float LA_SLACK = 8.0f;
constexpr float LA_LOG2E = 1.4426950408889634f, LA_LN2 = 0.6931471805599453f;
constexpr int LA_MAX_SUB = 32;                    // sub-vectors per head the kernel unrolls for

struct LutPlan {
    int rb;        // query rows per block (1, 2 or 4)
    int tiles;     // row tiles per (batch, kv head)
    int nsplit;    // token splits
    int64_t split_len;   // tokens per split, a multiple of LA_SUPER
    size_t lds;    // bytes of dynamic LDS
};

static LutPlan plan_lut(const vq_lut_attend_args &a) {
    LutPlan p;
    const int64_t nsk = a.D / a.k_sub_dim, nsv = a.D / a.v_sub_dim;
    const int64_t per_row = (nsk + nsv) * a.n_centroids * 4;
    const int64_t rows = (a.Hq / a.Hkv) * a.Sq;
    int rb = (int)(65536 / per_row);
    rb = rb >= 4 ? 4 : rb >= 2 ? 2 : 1;
    while (rb > 1 && rb / 2 >= rows) rb /= 2;
    p.rb = rb;
    p.tiles = (int)cdiv(rows, rb);
    p.lds = (size_t)(rb * per_row);
    const int64_t units = a.B * a.Hkv * p.tiles;
    int64_t ns = a.num_splits > 0 ? a.num_splits : cdiv(512, units > 0 ? units : 1);
    const int64_t max_splits = cdiv(a.n_tokens > 0 ? a.n_tokens : 1, LA_SUPER);
    if (ns > max_splits) ns = max_splits;
    if (ns > 256) ns = 256;
    if (ns < 1) ns = 1;
    p.split_len = cdiv(cdiv(a.n_tokens > 0 ? a.n_tokens : 1, ns), LA_SUPER) * LA_SUPER;
    p.nsplit = (int)cdiv(a.n_tokens > 0 ? a.n_tokens : 1, p.split_len);
    return p;
}

// indices of one token, n_sub of them, as bytes packed four to a word (IDX8) or as words
template <bool IDX8> struct TokIdx {
    uint32_t w[IDX8 ? LA_MAX_SUB / 4 : LA_MAX_SUB];
    // a token's indices fill nw words; whole 16-byte vectors when nw is a multiple of four
    __device__ __forceinline__ void load(const void *base, int64_t tok, int n_sub, bool valid) {
        constexpr int MAXW = IDX8 ? LA_MAX_SUB / 4 : LA_MAX_SUB;
        const int nw = IDX8 ? n_sub / 4 : n_sub;
        const uint32_t *p = (const uint32_t *)((const char *)base + tok * (int64_t)n_sub * (IDX8 ? 1 : 4));
        const bool vec = (nw & 3) == 0;   // uniform
#pragma unroll
        for (int i = 0; i < MAXW; i += 4) {
            if (i < nw) {   // uniform
                uint4 x = make_uint4(0, 0, 0, 0);
                if (valid) {
                    if (vec) x = *reinterpret_cast<const uint4 *>(p + i);
                    else {
                        x.x = p[i];
                        if (i + 1 < nw) x.y = p[i + 1];
                        if (i + 2 < nw) x.z = p[i + 2];
                        if (i + 3 < nw) x.w = p[i + 3];
                    }
                }
                w[i] = x.x; w[i + 1] = x.y; w[i + 2] = x.z; w[i + 3] = x.w;
            }
        }
    }
    // index j, never beyond the last centroid (a stray index must not leave the table)
    __device__ __forceinline__ uint32_t get(int j, uint32_t last) const {
        const uint32_t c = IDX8 ? (w[j >> 2] >> (8 * (j & 3))) & 0xffu : w[j];
        return c < last ? c : last;
    }
};

template <int RB, bool IDX8>
__global__ __launch_bounds__(LA_THREADS) void lut_attend_kernel(vq_lut_attend_args a, int tiles, int64_t split_len, int nparts,
                                                                float *__restrict__ ws) {
    extern __shared__ __align__(16) float s_tab[];
    __shared__ float s_max[LA_WAVES][4], s_sum[LA_WAVES][4];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int C = a.n_centroids;
    const int nsk = (int)(a.D / a.k_sub_dim), nsv = (int)(a.D / a.v_sub_dim);
    float *lut = s_tab;                       // [RB][nsk][C]
    float *hist = s_tab + RB * nsk * C;       // [RB][nsv][C]

    const int64_t bh = blockIdx.y / tiles;
    const int tile = (int)(blockIdx.y % tiles);
    const int64_t b = bh / a.Hkv, hkv = bh % a.Hkv;
    const int R = (int)(a.Hq / a.Hkv);
    const int n_rows = R * (int)a.Sq;
    // tile row r is head (r0 + r) % R of the group at query position (r0 + r) / R
    const int r0 = tile * RB;
    int64_t qrow[RB];      // flattened [B, Hq, Sq] row
    int64_t vis_hi[RB], vis_lo[RB];   // visible tokens [lo, hi)
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const int rr = r0 + r < n_rows ? r0 + r : n_rows - 1;
        const int64_t pos = rr / R;
        qrow[r] = (b * a.Hq + hkv * R + rr % R) * a.Sq + pos;
        const int64_t q_abs = a.n_tokens - a.Sq + pos;   // queries align to the end of the tokens
        vis_hi[r] = a.causal ? q_abs + 1 : a.n_tokens;
        vis_lo[r] = a.sliding_window > 0 && q_abs + 1 > a.sliding_window ? q_abs + 1 - a.sliding_window : 0;
    }

    // ---- tables: look-up table of the key side, zeroed histogram of the value side
    const float c2 = a.scale * LA_LOG2E;   // scores are kept in log2 units
    for (int e = tid; e < RB * nsk * C; e += LA_THREADS) {
        const int c = e % C, j = (e / C) % nsk, r = e / (C * nsk);
        float acc = 0.f;
        for (int i = 0; i < a.k_sub_dim; ++i)
            acc += ld_any(a.q, a.q_dtype, qrow[r] * a.D + j * a.k_sub_dim + i) *
                   ld_any(a.k_codebook, a.cb_dtype, (int64_t)c * a.k_sub_dim + i);
        lut[e] = acc * c2;
    }
    for (int e = tid; e < RB * nsv * C; e += LA_THREADS) hist[e] = 0.f;
    __syncthreads();

    // the block's share of the tokens, cut to what at least one of its rows can see
    int64_t t_begin = (int64_t)blockIdx.x * split_len;
    int64_t t_end = t_begin + split_len;
    if (t_end > a.n_tokens) t_end = a.n_tokens;
    {
        int64_t lo = vis_lo[0], hi = vis_hi[0];
#pragma unroll
        for (int r = 1; r < RB; ++r) { lo = vis_lo[r] < lo ? vis_lo[r] : lo; hi = vis_hi[r] > hi ? vis_hi[r] : hi; }
        if (t_begin < lo) t_begin = lo;
        if (t_end > hi) t_end = hi;
    }
    const char *kib = (const char *)a.k_idx + bh * a.cap_tokens * nsk * (IDX8 ? 1 : 4);
    const char *vib = (const char *)a.v_idx + bh * a.cap_tokens * nsv * (IDX8 ? 1 : 4);

    float m_row[RB], l_acc[RB];   // the block's softmax reference per row (log2 units), the lane's sum of probabilities
#pragma unroll
    for (int r = 0; r < RB; ++r) { m_row[r] = -INFINITY; l_acc[r] = 0.f; }

    for (int64_t base = t_begin; base < t_end; base += LA_SUPER) {
        // ---- phase 1: scores of the wave's tiles, and their maxima per row
        float s[LA_TILES][RB];
        TokIdx<IDX8> vi[LA_TILES];
        float wmax[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) wmax[r] = -INFINITY;
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const int64_t t = base + (wave * LA_TILES + T) * 64 + lane;
            const bool valid = t < t_end;
            TokIdx<IDX8> ki;
            ki.load(kib, t, nsk, valid);
            vi[T].load(vib, t, nsv, valid);
#pragma unroll
            for (int r = 0; r < RB; ++r) s[T][r] = 0.f;
#pragma unroll
            for (int j = 0; j < LA_MAX_SUB; ++j) {
                if (j < nsk) {   // uniform
                    const uint32_t c = ki.get(j, C - 1);
#pragma unroll
                    for (int r = 0; r < RB; ++r) s[T][r] += lut[(r * nsk + j) * C + c];
                }
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if (!(valid && t < vis_hi[r] && t >= vis_lo[r])) s[T][r] = -INFINITY;
                wmax[r] = fmaxf(wmax[r], s[T][r]);
            }
        }
#pragma unroll
        for (int r = 0; r < RB; ++r) {
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) wmax[r] = fmaxf(wmax[r], __shfl_xor(wmax[r], off));
            if (lane == 0) s_max[wave][r] = wmax[r];
        }
        __syncthreads();
        // ---- the block's reference moves only when the new maximum is far above it; then the
        // histogram and the running sums are rescaled (every thread sees the same decision)
        bool moved = false;
        float alpha[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const float bm = fmaxf(fmaxf(s_max[0][r], s_max[1][r]), fmaxf(s_max[2][r], s_max[3][r]));
            alpha[r] = 1.f;
            if (bm > m_row[r] + LA_SLACK) {
                alpha[r] = m_row[r] == -INFINITY ? 1.f : exp2f(m_row[r] - bm);   // nothing to rescale yet
                m_row[r] = bm;
                moved = true;
            }
        }
        if (moved) {
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                if (alpha[r] != 1.f) {
                    for (int e = tid; e < nsv * C; e += LA_THREADS) hist[r * nsv * C + e] *= alpha[r];
                    l_acc[r] *= alpha[r];
                }
            }
        }
        __syncthreads();   // s_max is free again; the rescaled histogram is in place
        // ---- phase 2: probabilities into the histogram
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            float p[RB];
            bool any = false;
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                p[r] = s[T][r] == -INFINITY ? 0.f : exp2f(s[T][r] - m_row[r]);
                l_acc[r] += p[r];
                any |= p[r] != 0.f;
            }
            if (any) {
#pragma unroll
                for (int j = 0; j < LA_MAX_SUB; ++j) {
                    if (j < nsv) {   // uniform
                        const uint32_t c = vi[T].get(j, C - 1);
#pragma unroll
                        for (int r = 0; r < RB; ++r)
                            if (p[r] != 0.f)
                                (void)__hip_atomic_fetch_add(&hist[(r * nsv + j) * C + c], p[r], __ATOMIC_RELAXED,
                                                             __HIP_MEMORY_SCOPE_WORKGROUP);
                    }
                }
            }
        }
    }

    // ---- sums of the block, histogram times value codebook, one partial per row
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        float l = l_acc[r];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) l += __shfl_xor(l, off);
        if (lane == 0) s_sum[wave][r] = l;
    }
    __syncthreads();
    for (int e = tid; e < RB * (int)a.D; e += LA_THREADS) {
        const int r = e / (int)a.D, d = e % (int)a.D;
        if (r0 + r >= n_rows) continue;
        const int j = d / a.v_sub_dim, i = d % a.v_sub_dim;
        const float *h = hist + (r * nsv + j) * C;
        float acc = 0.f;
        for (int c = 0; c < C; ++c) acc += h[c] * ld_any(a.v_codebook, a.cb_dtype, (int64_t)c * a.v_sub_dim + i);
        float *o = ws + (qrow[r] * nparts + blockIdx.x) * (a.D + 2);
        o[2 + d] = acc;
        if (d == 0) {
            o[0] = m_row[r] == -INFINITY ? -INFINITY : m_row[r] * LA_LN2;
            o[1] = s_sum[0][r] + s_sum[1][r] + s_sum[2][r] + s_sum[3][r];
        }
    }
}

static int validate_lut(const vq_lut_attend_args *a, const char *fn) {
    VQ_REQUIRE(a != nullptr, VQ_ERR_INVALID, "%s: null argument block", fn);
    VQ_REQUIRE(a->B >= 1 && a->Hq >= 1 && a->Hkv >= 1 && a->Sq >= 1 && a->D >= 1, VQ_ERR_INVALID,
               "%s: q must be 4D with positive sizes", fn);
    VQ_REQUIRE(a->Hq % a->Hkv == 0, VQ_ERR_INVALID, "%s: H_q=%lld must be a multiple of H_kv=%lld", fn, (long long)a->Hq,
               (long long)a->Hkv);
    VQ_REQUIRE(a->k_sub_dim >= 1 && a->v_sub_dim >= 1 && a->D % a->k_sub_dim == 0 && a->D % a->v_sub_dim == 0, VQ_ERR_INVALID,
               "%s: D=%lld must equal n_sub*sub_dim for keys (sub_dim %d) and values (sub_dim %d)", fn, (long long)a->D,
               a->k_sub_dim, a->v_sub_dim);
    VQ_REQUIRE(a->n_centroids >= 1, VQ_ERR_INVALID, "%s: n_centroids must be >= 1", fn);
    VQ_REQUIRE(a->n_tokens >= 1 && a->cap_tokens >= a->n_tokens, VQ_ERR_INVALID, "%s: need 1 <= n_tokens <= cap_tokens", fn);
    VQ_REQUIRE(!a->causal || a->Sq <= a->n_tokens, VQ_ERR_INVALID, "%s: S_q=%lld exceeds S_kv=%lld; queries align to the tail of the KV cache",
               fn, (long long)a->Sq, (long long)a->n_tokens);
    VQ_REQUIRE(a->sliding_window >= 0, VQ_ERR_INVALID, "%s: negative sliding window", fn);
    VQ_REQUIRE(is_float_tag(a->q_dtype) && is_float_tag(a->out_dtype) && is_float_tag(a->cb_dtype), VQ_ERR_INVALID,
               "%s: unsupported float dtype", fn);
    VQ_REQUIRE(a->idx_dtype == VQ_U8 || a->idx_dtype == VQ_I32 || a->idx_dtype == VQ_U32, VQ_ERR_INVALID,
               "%s: indices must be uint8, int32 or uint32", fn);
    // what the table kernel covers (the caps of the reference kernel, n_sub <= 16 and
    // n_centroids <= 256, veloxquant_mlx/metal/fused_sdpa.py:136-147, are inside these)
    VQ_REQUIRE(a->n_centroids <= 256, VQ_ERR_UNSUPPORTED, "%s: n_centroids=%d exceeds 256", fn, a->n_centroids);
    VQ_REQUIRE(a->D / a->k_sub_dim <= LA_MAX_SUB && a->D / a->v_sub_dim <= LA_MAX_SUB, VQ_ERR_UNSUPPORTED,
               "%s: more than %d sub-vectors per head", fn, LA_MAX_SUB);
    VQ_REQUIRE((a->D / a->k_sub_dim + a->D / a->v_sub_dim) * a->n_centroids * 4 <= 65536, VQ_ERR_UNSUPPORTED,
               "%s: look-up table and histogram of one query row exceed 64 KB of LDS", fn);
    if (a->idx_dtype == VQ_U8)
        VQ_REQUIRE((a->D / a->k_sub_dim) % 4 == 0 && (a->D / a->v_sub_dim) % 4 == 0, VQ_ERR_UNSUPPORTED,
                   "%s: uint8 indices need n_sub to be a multiple of 4", fn);
    return VQ_OK;
}

}  // namespace vq

using namespace vq;

extern "C" size_t vq_vecinfer_attend_workspace(const vq_lut_attend_args *a) {
    if (!a || validate_lut(a, "vq_vecinfer_attend_workspace") != VQ_OK) return 0;
    const LutPlan p = plan_lut(*a);
    return (size_t)(a->B * a->Hq * a->Sq) * (size_t)p.nsplit * (size_t)(a->D + 2) * sizeof(float);
}

extern "C" int vq_vecinfer_attend(const vq_lut_attend_args *a) {
    const char *fn = "vq_vecinfer_attend";
    int rc = validate_lut(a, fn);
    if (rc != VQ_OK) return rc;
    VQ_REQUIRE(a->q && a->out && a->k_idx && a->v_idx && a->k_codebook && a->v_codebook, VQ_ERR_INVALID, "%s: null pointer", fn);
    const LutPlan p = plan_lut(*a);
    const size_t need = (size_t)(a->B * a->Hq * a->Sq) * (size_t)p.nsplit * (size_t)(a->D + 2) * sizeof(float);
    VQ_REQUIRE(a->workspace && a->workspace_bytes >= need, VQ_ERR_INVALID, "%s: workspace of %zu bytes needed, %zu given", fn, need,
               a->workspace_bytes);
    VQ_REQUIRE((((uintptr_t)a->k_idx | (uintptr_t)a->v_idx) & 15u) == 0, VQ_ERR_UNSUPPORTED, "%s: index buffers must be 16-byte aligned", fn);
    VQ_REQUIRE(a->B * a->Hkv * p.tiles <= 65535, VQ_ERR_UNSUPPORTED, "%s: too many (batch, kv head, row tile) blocks", fn);
    hipStream_t st = (hipStream_t)a->stream;
    const dim3 grid((unsigned)p.nsplit, (unsigned)(a->B * a->Hkv * p.tiles));
    const bool idx8 = a->idx_dtype == VQ_U8;
#define VQ_LUT(RB, I8)                                                                                              \
    do {                                                                                                            \
        static bool allowed[64] = {};                                                                               \
        int dev = 0;                                                                                                \
        (void)hipGetDevice(&dev);                                                                                   \
        if (dev < 0 || dev >= 64 || !allowed[dev]) {                                                                \
            (void)hipFuncSetAttribute((const void *)lut_attend_kernel<RB, I8>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                      65536);                                                                       \
            if (dev >= 0 && dev < 64) allowed[dev] = true;                                                          \
        }                                                                                                           \
        hipLaunchKernelGGL((lut_attend_kernel<RB, I8>), grid, dim3(LA_THREADS), p.lds, st, *a, p.tiles, p.split_len, \
                           p.nsplit, (float *)a->workspace);                                                        \
    } while (0)
    if (idx8) { if (p.rb == 4) VQ_LUT(4, true); else if (p.rb == 2) VQ_LUT(2, true); else VQ_LUT(1, true); }
    else { if (p.rb == 4) VQ_LUT(4, false); else if (p.rb == 2) VQ_LUT(2, false); else VQ_LUT(1, false); }
#undef VQ_LUT
    VQ_HIP_CHECK_LAUNCH(fn);
    launch_merge_rows((const float *)a->workspace, a->B * a->Hq * a->Sq, p.nsplit, a->D, a->out, a->out_dtype, st);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}
