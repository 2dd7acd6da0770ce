// Attention straight from VecInfer codebook indices (gfx950, wave64): neither keys nor values
// are ever materialised.
//
//   scores   q~ . k~^[t] = sum_j LUT[j][k_idx[t][j]],  LUT[j][c] = q~[j*sub .. ] . key_codebook[c]
//   output   sum_t P[t] v^[t] = sum_j sum_c W[j][c] value_codebook[c],  W[j][c] = sum of P[t] over
//            the tokens whose j-th value index is c
//
// so a token costs n_sub table look-ups and n_sub additions into a histogram per query row,
// whatever the head dimension; the histogram meets the value codebook once, at the end.  Both
// tables live in LDS, and LDS traffic, not HBM, bounds the kernel.
//
// The histogram is an integer one.  A weight is exp2(score - reference) <= 1 with the reference
// at or above every score the block has seen, and it is added in units of 2^-F with an integer
// LDS atomic: on this chip a random-address ds_add_u32 costs what a ds_read_b32 does, a
// ds_add_f32 about 27 times that.  F is 20 for blocks of up to 2048 tokens, 19 up to 4096 and
// 18 up to 8192, so a cell cannot exceed 2^31.  The weight is rounded down after adding a
// per-token offset in [0, 1) from a low-discrepancy sequence (token number times the golden
// ratio), so that many weights below one unit still add up to their true total.  The sum of
// the weights is read back from the histogram itself, which makes the output an exact convex
// combination of centroids, and integer addition makes it independent of the order in which
// the waves arrive.  When a later tile of tokens raises the reference the histogram is rescaled
// in place.
//
// One block of four waves per (kv head, tile of RB query rows, token split); a lane is a token.
// Every block writes one (max, sum, accumulator) partial per row; the merge kernel of the
// packed-cache attention combines them.  Two kernels: lut_attend_u8_kernel for byte indices
// with the same, compile-time number of sub-vectors on both sides (tables laid out so that one
// LDS read returns the entries of all RB rows), and lut_attend_any_kernel for everything else.
#include <atomic>

#include "attend.hpp"
#include "vecinfer.hpp"

namespace vq {

constexpr int LA_THREADS = 256, LA_WAVES = 4;
constexpr int LA_TILES = 4;                           // 64-token tiles a wave holds scores of between the two phases
constexpr int LA_SUPER = LA_WAVES * LA_TILES * 64;    // tokens a block takes per step
constexpr int LA_MAX_SPLIT = 8192;                    // tokens per block
constexpr float LA_GOLDEN = 0.6180339887498949f;
constexpr float LA_HEADROOM = 1.0f;                   // a raised reference goes this far (log2) above the new maximum
constexpr float LA_LOG2E = 1.4426950408889634f, LA_LN2 = 0.6931471805599453f;
constexpr int LA_MAX_SUB = 32;                        // sub-vectors per head
constexpr int LA_ROW = 256;                           // centroids per table row of the byte-index kernel
constexpr size_t LA_MAX_LDS = 96 * 1024;

struct LutPlan {
    bool bytes;    // lut_attend_u8_kernel
    bool vt_apart; // lut_attend_u8_kernel: the transposed value codebook has LDS of its own
    int rb;        // query rows per block (1, 2 or 4)
    int tiles;     // row tiles per (batch, kv head)
    int nsplit;    // token splits
    int64_t split_len;   // tokens per split, a multiple of LA_SUPER, at most LA_MAX_SPLIT
    int fbits;     // weights are integers in units of 2^-fbits: split_len * 2^fbits <= 2^31
    size_t lds;    // bytes of dynamic LDS
};

static LutPlan plan_lut(const vq_lut_attend_args &a) {
    LutPlan p;
    const int64_t nsk = a.D / a.k_sub_dim, nsv = a.D / a.v_sub_dim;
    const int64_t rows = (a.Hq / a.Hkv) * a.Sq;
    p.bytes = a.idx_dtype == VQ_U8 && nsk == nsv && (nsk == 4 || nsk == 8 || nsk == 16 || nsk == 32) &&
              a.k_sub_dim % 4 == 0 && a.k_sub_dim <= 256 && a.n_centroids <= LA_ROW &&
              (((uintptr_t)a.q | (uintptr_t)a.k_codebook | (uintptr_t)a.v_codebook) & 15u) == 0;
    int rb;
    if (p.bytes) {
        rb = (int)(32 / nsk);   // table and histogram of a block: 2 * rb * nsk KB <= 64 KB, two blocks a CU
        rb = rb >= 4 ? 4 : rb >= 2 ? 2 : 1;
    } else {
        const int64_t per_row = (nsk + nsv) * a.n_centroids * 4;
        rb = (int)(65536 / per_row);
        rb = rb >= 4 ? 4 : rb >= 2 ? 2 : 1;
    }
    while (rb > 1 && rb / 2 >= rows) rb /= 2;
    p.rb = rb;
    p.tiles = (int)cdiv(rows, rb);
    p.vt_apart = false;
    if (p.bytes) {
        p.vt_apart = 2 * rb * nsk + a.k_sub_dim <= 78;   // 1 KB rows; two blocks of 78 fit the 160 KB of a CU
        const int64_t tab = p.vt_apart || rb * nsk > a.k_sub_dim ? rb * nsk : a.k_sub_dim;
        p.lds = (size_t)(tab + rb * nsk + (p.vt_apart ? a.k_sub_dim : 0)) * LA_ROW * 4;
    } else {
        p.lds = (size_t)(rb * (nsk + nsv) * a.n_centroids * 4);
    }
    const int64_t n = a.n_tokens > 0 ? a.n_tokens : 1;
    const int64_t units = a.B * a.Hkv * p.tiles;
    int64_t ns = a.num_splits > 0 ? a.num_splits : cdiv(1024, units > 0 ? units : 1);
    const int64_t max_splits = cdiv(n, LA_SUPER), min_splits = cdiv(n, LA_MAX_SPLIT);
    if (ns > max_splits) ns = max_splits;
    if (ns < min_splits) ns = min_splits;
    p.split_len = cdiv(cdiv(n, ns), LA_SUPER) * LA_SUPER;
    p.nsplit = (int)cdiv(n, p.split_len);
    p.fbits = p.split_len <= 2048 ? 20 : p.split_len <= 4096 ? 19 : 18;
    return p;
}

// ---- pieces both kernels share -----------------------------------------------------------

// Tile row r of a block is head (r0 + r) % R of the kv head's group at query position
// (r0 + r) / R; rows past the last one repeat it (their partials are not written).
struct RowGeom {
    int64_t b, hkv;
    int R, n_rows, r0;
    __device__ __forceinline__ int clamp(int r) const { return r0 + r < n_rows ? r0 + r : n_rows - 1; }
    __device__ __forceinline__ int64_t qrow(const vq_lut_attend_args &a, int r) const {   // row of the flattened [B, Hq, Sq]
        const int rr = clamp(r);
        return (b * a.Hq + hkv * R + rr % R) * a.Sq + rr / R;
    }
    // visible tokens [lo, hi): queries align to the end of the tokens
    __device__ __forceinline__ void visible(const vq_lut_attend_args &a, int r, int64_t &lo, int64_t &hi) const {
        const int64_t q_abs = a.n_tokens - a.Sq + clamp(r) / R;
        hi = a.causal ? q_abs + 1 : a.n_tokens;
        lo = a.sliding_window > 0 && q_abs + 1 > a.sliding_window ? q_abs + 1 - a.sliding_window : 0;
    }
};

// maximum over the wave, in every lane: four cross-lane moves inside the rows of 16, then one
// lane of each row
template <int CTRL> __device__ __forceinline__ float dpp_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x124>(v));   // row_ror 4
    v = fmaxf(v, dpp_move<0x128>(v));   // row_ror 8
    const int b = __builtin_bit_cast(int, v);
    return fmaxf(fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 0)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 16))),
                 fmaxf(__builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 32)), __builtin_bit_cast(float, __builtin_amdgcn_readlane(b, 48))));
}

// After the waves have published their tiles' maxima: raise the references that a maximum
// exceeds and rescale those rows of the histogram ([RB][row_words] integers).  Every thread
// takes the same decisions.  The caller synchronises afterwards.
template <int RB>
__device__ __forceinline__ void raise_references(const float (*s_max)[4], float (&m_row)[RB], uint32_t *hist, int row_words, int tid) {
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const float bm = fmaxf(fmaxf(s_max[0][r], s_max[1][r]), fmaxf(s_max[2][r], s_max[3][r]));
        if (bm > m_row[r]) {
            if (m_row[r] == -INFINITY) {
                m_row[r] = bm;   // nothing accumulated yet
            } else {
                const float m_new = bm + LA_HEADROOM;
                const float alpha = __builtin_amdgcn_exp2f(m_row[r] - m_new);
                m_row[r] = m_new;
                uint4 *h = reinterpret_cast<uint4 *>(hist + r * row_words);
                const int vec = (row_words & 3) == 0 && (reinterpret_cast<uintptr_t>(h) & 15u) == 0 ? row_words / 4 : 0;
                for (int e = tid; e < vec; e += LA_THREADS) {
                    uint4 x = h[e];
                    x.x = __float2uint_rn((float)x.x * alpha); x.y = __float2uint_rn((float)x.y * alpha);
                    x.z = __float2uint_rn((float)x.z * alpha); x.w = __float2uint_rn((float)x.w * alpha);
                    h[e] = x;
                }
                for (int e = 4 * vec + tid; e < row_words; e += LA_THREADS)
                    hist[r * row_words + e] = __float2uint_rn((float)hist[r * row_words + e] * alpha);
            }
        }
    }
}

// weight exp2(s - m) <= 1 in units of 1 / unit, rounded down after the token's offset
__device__ __forceinline__ uint32_t weight_units(float s, float m, float unit, float dither) {
    return s == -INFINITY ? 0u : __float2uint_rd(__builtin_amdgcn_exp2f(s - m) * unit + dither);
}
__device__ __forceinline__ float token_dither(int64_t t) {
    return __builtin_amdgcn_fractf((float)((uint32_t)t & 0xffffu) * LA_GOLDEN);
}

__device__ __forceinline__ void lds_add(uint32_t *p, uint32_t v) {
    (void)__hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// four consecutive elements from index i (a multiple of four) of a buffer whose base is 16-byte aligned
__device__ __forceinline__ float4 ld4_any(const void *p, int tag, int64_t i) {
    if (tag == VQ_F32) return *reinterpret_cast<const float4 *>((const float *)p + i);
    const uint2 raw = *reinterpret_cast<const uint2 *>((const u16 *)p + i);
    if (tag == VQ_F16) {
        const f16x2 lo = __builtin_bit_cast(f16x2, raw.x), hi = __builtin_bit_cast(f16x2, raw.y);
        return make_float4((float)lo[0], (float)lo[1], (float)hi[0], (float)hi[1]);
    }
    return make_float4(__builtin_bit_cast(float, raw.x << 16), __builtin_bit_cast(float, raw.x & 0xffff0000u),
                       __builtin_bit_cast(float, raw.y << 16), __builtin_bit_cast(float, raw.y & 0xffff0000u));
}

// a block none of whose rows sees a token of its split: empty partials
template <int RB>
__device__ __forceinline__ void write_empty(const vq_lut_attend_args &a, const RowGeom &g, int nparts, float *ws, int tid) {
    for (int e = tid; e < RB * ((int)a.D + 2); e += LA_THREADS) {
        const int r = e / ((int)a.D + 2), k = e % ((int)a.D + 2);
        if (g.r0 + r >= g.n_rows) continue;
        ws[(g.qrow(a, r) * nparts + blockIdx.x) * (a.D + 2) + k] = k == 0 ? -INFINITY : 0.f;
    }
}

// ---- byte indices, NS sub-vectors on both sides --------------------------------------------

template <int NW> struct ByteIdx {   // a token's NS = 4 * NW indices
    uint32_t w[NW];
    __device__ __forceinline__ void load(const uint8_t *row, bool valid) {
#pragma unroll
        for (int i = 0; i < NW; ++i) w[i] = 0;
        if (!valid) return;
        if constexpr (NW == 1) w[0] = *reinterpret_cast<const uint32_t *>(row);
        else if constexpr (NW == 2) { const uint2 x = *reinterpret_cast<const uint2 *>(row); w[0] = x.x; w[1] = x.y; }
        else {
#pragma unroll
            for (int i = 0; i < NW; i += 4) {
                const uint4 x = *reinterpret_cast<const uint4 *>(row + 4 * i);
                w[i] = x.x; w[i + 1] = x.y; w[i + 2] = x.z; w[i + 3] = x.w;
            }
        }
    }
    __device__ __forceinline__ uint32_t get(int j) const { return (w[j >> 2] >> (8 * (j & 3))) & 0xffu; }
};

// LDS: table [NS][256][RB] floats (later the value codebook transposed, [sub][256] floats),
// histogram [RB][NS][256] integers (first the staged query rows).
template <int RB, int NS>
__global__ __launch_bounds__(LA_THREADS) void lut_attend_u8_kernel(vq_lut_attend_args a, int tiles, int64_t split_len, int nparts,
                                                                   int vt_apart, int fbits, float *__restrict__ ws) {
    extern __shared__ __align__(16) float s_tab[];
    __shared__ float s_max[LA_WAVES][4], s_ref[4];
    __shared__ uint32_t s_sum[4];
    constexpr int NW = NS / 4;
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int C = a.n_centroids, SUB = a.k_sub_dim, D = (int)a.D;
    const float unit = (float)(1u << fbits), inv_unit = 1.0f / unit;
    float *lut = s_tab;
    // the transposed value codebook has rows of its own behind the histogram when two blocks
    // still fit a CU that way (vt_apart); otherwise it overwrites the table at the end
    const int tab_rows = vt_apart || RB * NS > SUB ? RB * NS : SUB;
    uint32_t *hist = reinterpret_cast<uint32_t *>(s_tab + tab_rows * LA_ROW);
    float *vt = vt_apart ? s_tab + (tab_rows + RB * NS) * LA_ROW : lut;

    RowGeom g;
    const int64_t bh = blockIdx.y / tiles;
    g.b = bh / a.Hkv; g.hkv = bh % a.Hkv;
    g.R = (int)(a.Hq / a.Hkv); g.n_rows = g.R * (int)a.Sq; g.r0 = (int)(blockIdx.y % tiles) * RB;
    int64_t vis_lo[RB], vis_hi[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) g.visible(a, r, vis_lo[r], vis_hi[r]);

    // the block's share of the tokens, cut to what at least one of its rows can see
    int64_t t_begin = (int64_t)blockIdx.x * split_len, t_end = t_begin + split_len;
    if (t_end > a.n_tokens) t_end = a.n_tokens;
    {
        int64_t lo = vis_lo[0], hi = vis_hi[0];
#pragma unroll
        for (int r = 1; r < RB; ++r) { lo = vis_lo[r] < lo ? vis_lo[r] : lo; hi = vis_hi[r] > hi ? vis_hi[r] : hi; }
        if (t_begin < lo) t_begin = lo;
        if (t_end > hi) t_end = hi;
    }
    if (t_begin >= t_end) { write_empty<RB>(a, g, nparts, ws, tid); return; }

    // ---- everything the block reads before its token loop is requested first: the first
    // step's indices, the query rows, the codebook rows of thread c = centroid c
    const uint8_t *kib = (const uint8_t *)a.k_idx + bh * a.cap_tokens * NS;
    const uint8_t *vib = (const uint8_t *)a.v_idx + bh * a.cap_tokens * NS;
    ByteIdx<NW> kn[LA_TILES], vn[LA_TILES];
    auto fetch = [&](int64_t base) {
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const int64_t t = base + (wave * LA_TILES + T) * 64 + lane;
            kn[T].load(kib + t * NS, t < t_end);
            vn[T].load(vib + t * NS, t < t_end);
        }
    };
    fetch(t_begin);
    float *sq = reinterpret_cast<float *>(hist);
    for (int e = tid; e < RB * D / 4; e += LA_THREADS) {
        const int r = 4 * e / D, d = 4 * e % D;
        *reinterpret_cast<float4 *>(sq + 4 * e) = ld4_any(a.q, a.q_dtype, g.qrow(a, r) * a.D + d);
    }
    if (vt_apart) {
        for (int i0 = 0; i0 < SUB; i0 += 4) {
            const float4 v = tid < C ? ld4_any(a.v_codebook, a.cb_dtype, (int64_t)tid * SUB + i0) : make_float4(0.f, 0.f, 0.f, 0.f);
            vt[(i0 + 0) * LA_ROW + tid] = v.x; vt[(i0 + 1) * LA_ROW + tid] = v.y;
            vt[(i0 + 2) * LA_ROW + tid] = v.z; vt[(i0 + 3) * LA_ROW + tid] = v.w;
        }
    }
    float4 kc_next = tid < C ? ld4_any(a.k_codebook, a.cb_dtype, (int64_t)tid * SUB) : make_float4(0.f, 0.f, 0.f, 0.f);
    __syncthreads();
    {
        const float c2 = a.scale * LA_LOG2E;   // scores are kept in log2 units
        float acc[RB][NS];
#pragma unroll
        for (int r = 0; r < RB; ++r)
#pragma unroll
            for (int j = 0; j < NS; ++j) acc[r][j] = 0.f;
        for (int i0 = 0; i0 < SUB; i0 += 4) {
            const float4 kc = kc_next;
            if (i0 + 4 < SUB && tid < C) kc_next = ld4_any(a.k_codebook, a.cb_dtype, (int64_t)tid * SUB + i0 + 4);
#pragma unroll
            for (int r = 0; r < RB; ++r)
#pragma unroll
                for (int j = 0; j < NS; ++j) {
                    const float4 qv = *reinterpret_cast<const float4 *>(sq + r * D + j * SUB + i0);
                    acc[r][j] += qv.x * kc.x + qv.y * kc.y + qv.z * kc.z + qv.w * kc.w;
                }
        }
#pragma unroll
        for (int j = 0; j < NS; ++j)
#pragma unroll
            for (int r = 0; r < RB; ++r) lut[(j * LA_ROW + tid) * RB + r] = acc[r][j] * c2;
    }
    __syncthreads();   // the staged query rows are dead
    for (int e = tid; e < RB * NS * LA_ROW / 4; e += LA_THREADS) reinterpret_cast<uint4 *>(hist)[e] = make_uint4(0, 0, 0, 0);
    __syncthreads();

    float m_row[RB];   // the block's softmax reference per row, log2 units
#pragma unroll
    for (int r = 0; r < RB; ++r) m_row[r] = -INFINITY;

    // the indices of a step are loaded one step ahead
    wait_global_accesses();
    for (int64_t base = t_begin; base < t_end; base += LA_SUPER) {
        // ---- phase 1: scores of the wave's tiles, and their maxima per row
        float s[LA_TILES][RB], wmax[RB];
        ByteIdx<NW> ki[LA_TILES], vi[LA_TILES];
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) { ki[T] = kn[T]; vi[T] = vn[T]; }
        fetch(base + LA_SUPER);
#pragma unroll
        for (int r = 0; r < RB; ++r) wmax[r] = -INFINITY;
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const int64_t t = base + (wave * LA_TILES + T) * 64 + lane;
            const bool valid = t < t_end;
#pragma unroll
            for (int r = 0; r < RB; ++r) s[T][r] = 0.f;
#pragma unroll
            for (int j = 0; j < NS; ++j) {
                const float *e = lut + (j * LA_ROW + ki[T].get(j)) * RB;
                if constexpr (RB == 4) { const float4 x = *reinterpret_cast<const float4 *>(e); s[T][0] += x.x; s[T][1] += x.y; s[T][2] += x.z; s[T][3] += x.w; }
                else if constexpr (RB == 2) { const float2 x = *reinterpret_cast<const float2 *>(e); s[T][0] += x.x; s[T][1] += x.y; }
                else s[T][0] += *e;
            }
#pragma unroll
            for (int r = 0; r < RB; ++r) {
                asm volatile("" : "+v"(s[T][r]));   // the look-ups stay whole reads, outside the masks' branches
                if (!(valid && t < vis_hi[r] && t >= vis_lo[r])) s[T][r] = -INFINITY;
                wmax[r] = fmaxf(wmax[r], s[T][r]);
            }
        }
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            wmax[r] = wave_max(wmax[r]);
            if (lane == 0) s_max[wave][r] = wmax[r];
        }
        lds_barrier();   // (LDS only: the indices requested above stay in flight)
        raise_references<RB>(s_max, m_row, hist, NS * LA_ROW, tid);
        lds_barrier();   // s_max is free again; a rescaled histogram is in place
        // ---- phase 2: weights into the histogram
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const float dither = token_dither(base + (wave * LA_TILES + T) * 64 + lane);
            uint32_t w[RB], any = 0;
#pragma unroll
            for (int r = 0; r < RB; ++r) { w[r] = weight_units(s[T][r], m_row[r], unit, dither); any |= w[r]; }
            if (__any(any != 0)) {
#pragma unroll
                for (int j = 0; j < NS; ++j) {
                    uint32_t *h = hist + j * LA_ROW + vi[T].get(j);
#pragma unroll
                    for (int r = 0; r < RB; ++r) lds_add(h + r * NS * LA_ROW, w[r]);
                }
            }
        }
    }
    __syncthreads();   // every weight has landed; the table is dead

    // ---- value codebook transposed over the table, the sums of the weights from sub-vector 0
    if (!vt_apart)
        for (int e = tid; e < SUB * LA_ROW; e += LA_THREADS)   // e % 256 == tid
            vt[e] = tid < C ? ld_any(a.v_codebook, a.cb_dtype, (int64_t)tid * SUB + e / LA_ROW) : 0.f;
    if (wave < RB) {
        const uint4 h = reinterpret_cast<const uint4 *>(hist + wave * NS * LA_ROW)[lane];
        uint32_t t = h.x + h.y + h.z + h.w;
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) t += __shfl_xor(t, off);
        if (lane == 0) s_sum[wave] = t;
    }
    if (tid == 0) {
#pragma unroll
        for (int r = 0; r < RB; ++r) s_ref[r] = m_row[r];
    }
    __syncthreads();
    // output (r, d): 256 centroids of histogram row (r, d / sub) against row d % sub of the
    // transposed codebook, four at a time; lanes start 16 bytes apart so a wave spreads over the banks
    for (int e = tid; e < RB * D; e += LA_THREADS) {
        const int r = e / D, d = e % D;
        if (g.r0 + r >= g.n_rows) continue;
        const uint32_t *h = hist + (r * NS + d / SUB) * LA_ROW;
        const float *v = vt + (d % SUB) * LA_ROW;
        float acc = 0.f;
        for (int it = 0; it < LA_ROW / 4; ++it) {
            const int c = 4 * ((it + lane) & (LA_ROW / 4 - 1));
            const uint4 hh = *reinterpret_cast<const uint4 *>(h + c);
            const float4 vv = *reinterpret_cast<const float4 *>(v + c);
            acc += (float)hh.x * vv.x + (float)hh.y * vv.y + (float)hh.z * vv.z + (float)hh.w * vv.w;
        }
        float *o = ws + (g.qrow(a, r) * nparts + blockIdx.x) * (a.D + 2);
        o[2 + d] = acc * inv_unit;
        if (d == 0) {
            o[0] = s_ref[r] == -INFINITY ? -INFINITY : s_ref[r] * LA_LN2;
            o[1] = (float)s_sum[r] * inv_unit;
        }
    }
}

// ---- any index type, any numbers of sub-vectors ---------------------------------------------

// LDS: table [RB][nsk][C] floats, histogram [RB][nsv][C] integers.  Indices are read from
// memory where they are used; a stray index is held to the last centroid.
template <int RB>
__global__ __launch_bounds__(LA_THREADS) void lut_attend_any_kernel(vq_lut_attend_args a, int tiles, int64_t split_len, int nparts,
                                                                    int fbits, float *__restrict__ ws) {
    extern __shared__ __align__(16) float s_tab[];
    __shared__ float s_max[LA_WAVES][4], s_ref[4];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int C = a.n_centroids, D = (int)a.D;
    const int nsk = D / a.k_sub_dim, nsv = D / a.v_sub_dim;
    const float unit = (float)(1u << fbits), inv_unit = 1.0f / unit;
    float *lut = s_tab;
    uint32_t *hist = reinterpret_cast<uint32_t *>(s_tab + RB * nsk * C);

    RowGeom g;
    const int64_t bh = blockIdx.y / tiles;
    g.b = bh / a.Hkv; g.hkv = bh % a.Hkv;
    g.R = (int)(a.Hq / a.Hkv); g.n_rows = g.R * (int)a.Sq; g.r0 = (int)(blockIdx.y % tiles) * RB;
    int64_t vis_lo[RB], vis_hi[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) g.visible(a, r, vis_lo[r], vis_hi[r]);
    int64_t t_begin = (int64_t)blockIdx.x * split_len, t_end = t_begin + split_len;
    if (t_end > a.n_tokens) t_end = a.n_tokens;
    {
        int64_t lo = vis_lo[0], hi = vis_hi[0];
#pragma unroll
        for (int r = 1; r < RB; ++r) { lo = vis_lo[r] < lo ? vis_lo[r] : lo; hi = vis_hi[r] > hi ? vis_hi[r] : hi; }
        if (t_begin < lo) t_begin = lo;
        if (t_end > hi) t_end = hi;
    }
    if (t_begin >= t_end) { write_empty<RB>(a, g, nparts, ws, tid); return; }

    const float c2 = a.scale * LA_LOG2E;
    for (int rj = 0; rj < RB * nsk; ++rj) {   // the query sub-vector is common to the block
        const int64_t qb = g.qrow(a, rj / nsk) * a.D + (rj % nsk) * a.k_sub_dim;
        for (int c = tid; c < C; c += LA_THREADS) {
            float acc = 0.f;
            for (int i = 0; i < a.k_sub_dim; ++i)
                acc += ld_any(a.q, a.q_dtype, qb + i) * ld_any(a.k_codebook, a.cb_dtype, (int64_t)c * a.k_sub_dim + i);
            lut[rj * C + c] = acc * c2;
        }
    }
    for (int e = tid; e < RB * nsv * C; e += LA_THREADS) hist[e] = 0u;
    __syncthreads();

    const int isz = a.idx_dtype == VQ_U8 ? 1 : 4;
    const char *kib = (const char *)a.k_idx + bh * a.cap_tokens * nsk * isz;
    const char *vib = (const char *)a.v_idx + bh * a.cap_tokens * nsv * isz;
    const uint32_t last = (uint32_t)(C - 1);
    float m_row[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) m_row[r] = -INFINITY;

    for (int64_t base = t_begin; base < t_end; base += LA_SUPER) {
        float s[LA_TILES][RB], wmax[RB];
#pragma unroll
        for (int r = 0; r < RB; ++r) wmax[r] = -INFINITY;
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const int64_t t = base + (wave * LA_TILES + T) * 64 + lane;
            const bool valid = t < t_end;
#pragma unroll
            for (int r = 0; r < RB; ++r) s[T][r] = 0.f;
            if (valid) {
                for (int j = 0; j < nsk; ++j) {
                    uint32_t c = ld_idx(kib, a.idx_dtype, t * nsk + j);
                    c = c < last ? c : last;
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
            wmax[r] = wave_max(wmax[r]);
            if (lane == 0) s_max[wave][r] = wmax[r];
        }
        __syncthreads();
        raise_references<RB>(s_max, m_row, hist, nsv * C, tid);
        __syncthreads();
#pragma unroll
        for (int T = 0; T < LA_TILES; ++T) {
            const int64_t t = base + (wave * LA_TILES + T) * 64 + lane;
            const float dither = token_dither(t);
            uint32_t w[RB], any = 0;
#pragma unroll
            for (int r = 0; r < RB; ++r) { w[r] = weight_units(s[T][r], m_row[r], unit, dither); any |= w[r]; }
            if (any != 0) {
                for (int j = 0; j < nsv; ++j) {
                    uint32_t c = ld_idx(vib, a.idx_dtype, t * nsv + j);
                    c = c < last ? c : last;
#pragma unroll
                    for (int r = 0; r < RB; ++r) lds_add(hist + (r * nsv + j) * C + c, w[r]);
                }
            }
        }
    }
    if (tid == 0) {
#pragma unroll
        for (int r = 0; r < RB; ++r) s_ref[r] = m_row[r];
    }
    __syncthreads();

    for (int e = tid; e < RB * D; e += LA_THREADS) {
        const int r = e / D, d = e % D;
        if (g.r0 + r >= g.n_rows) continue;
        const int j = d / a.v_sub_dim, i = d % a.v_sub_dim;
        const uint32_t *h = hist + (r * nsv + j) * C;
        float acc = 0.f;
        for (int c = 0; c < C; ++c) acc += (float)h[c] * ld_any(a.v_codebook, a.cb_dtype, (int64_t)c * a.v_sub_dim + i);
        float *o = ws + (g.qrow(a, r) * nparts + blockIdx.x) * (a.D + 2);
        o[2 + d] = acc * inv_unit;
        if (d == 0) {
            uint32_t sum = 0;   // the weights of sub-vector 0 add up to the sum over the tokens
            for (int c = 0; c < C; ++c) sum += hist[r * nsv * C + c];
            o[0] = s_ref[r] == -INFINITY ? -INFINITY : s_ref[r] * LA_LN2;
            o[1] = (float)sum * inv_unit;
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
    // what the table kernels cover (the caps of the reference kernel, n_sub <= 16 and
    // n_centroids <= 256, veloxquant_mlx/metal/fused_sdpa.py:136-147, are inside these)
    VQ_REQUIRE(a->n_centroids <= 256, VQ_ERR_UNSUPPORTED, "%s: n_centroids=%d exceeds 256", fn, a->n_centroids);
    VQ_REQUIRE(a->D / a->k_sub_dim <= LA_MAX_SUB && a->D / a->v_sub_dim <= LA_MAX_SUB, VQ_ERR_UNSUPPORTED,
               "%s: more than %d sub-vectors per head", fn, LA_MAX_SUB);
    VQ_REQUIRE(plan_lut(*a).lds <= LA_MAX_LDS, VQ_ERR_UNSUPPORTED, "%s: look-up table and histogram of one query row exceed %zu KB of LDS",
               fn, LA_MAX_LDS / 1024);
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
    // dynamic LDS above 64 KB has to be allowed once per kernel and device
#define VQ_LUT_LAUNCH(KERNEL, ...)                                                                                  \
    do {                                                                                                            \
        static std::atomic<bool> allowed[64] = {};   /* a second thread that gets here first repeats the same call */ \
        int dev = 0;                                                                                                \
        (void)hipGetDevice(&dev);                                                                                   \
        if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {                                \
            (void)hipFuncSetAttribute((const void *)KERNEL, hipFuncAttributeMaxDynamicSharedMemorySize, (int)LA_MAX_LDS); \
            if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);                          \
        }                                                                                                           \
        hipLaunchKernelGGL(KERNEL, grid, dim3(LA_THREADS), p.lds, st, *a, p.tiles, p.split_len, p.nsplit, __VA_ARGS__); \
    } while (0)
    float *ws = (float *)a->workspace;
    if (p.bytes) {
        const int ns = (int)(a->D / a->k_sub_dim);
#define VQ_LUT_U8(RB, NS) VQ_LUT_LAUNCH((lut_attend_u8_kernel<RB, NS>), (int)p.vt_apart, p.fbits, ws)
        if (ns == 4) { if (p.rb == 4) VQ_LUT_U8(4, 4); else if (p.rb == 2) VQ_LUT_U8(2, 4); else VQ_LUT_U8(1, 4); }
        else if (ns == 8) { if (p.rb == 4) VQ_LUT_U8(4, 8); else if (p.rb == 2) VQ_LUT_U8(2, 8); else VQ_LUT_U8(1, 8); }
        else if (ns == 16) { if (p.rb == 2) VQ_LUT_U8(2, 16); else VQ_LUT_U8(1, 16); }
        else VQ_LUT_U8(1, 32);
#undef VQ_LUT_U8
    } else {
        if (p.rb == 4) VQ_LUT_LAUNCH((lut_attend_any_kernel<4>), p.fbits, ws);
        else if (p.rb == 2) VQ_LUT_LAUNCH((lut_attend_any_kernel<2>), p.fbits, ws);
        else VQ_LUT_LAUNCH((lut_attend_any_kernel<1>), p.fbits, ws);
    }
#undef VQ_LUT_LAUNCH
    VQ_HIP_CHECK_LAUNCH(fn);
    launch_merge_rows(ws, a->B * a->Hq * a->Sq, p.nsplit, a->D, a->out, a->out_dtype, st);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}
