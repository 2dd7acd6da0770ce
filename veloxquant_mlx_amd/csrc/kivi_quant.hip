// KIVI asymmetric group quantisation, bit packing and reconstruction for gfx950.
//
// Math (float32, one rounding per operation, no contraction):
//   scale = max((gmax - gmin) / levels, eps)
//   code  = clamp(rint((x - gmin) / scale), 0, levels)      rint = half-to-even
//   xhat  = code * scale + gmin                              (two roundings)
// as in veloxquant_mlx/cache/kivi_cache.py:181-201 and
// veloxquant_mlx/metal/src/kivi_group_quant_{channel,token}.metal.
//
// Two kinds of kernels:
//   * tile kernels for head_dim 64/128/256 with 128-bit loads; key groups are
//     reduced with wavefront shuffles plus one LDS exchange between the four
//     waves of a block, value groups with shuffles only;
//   * generic kernels (any head_dim / group / bit width) in which every thread
//     rescans the group it needs -- slow but free of layout assumptions.
#include "common.hpp"

#include <type_traits>

namespace vq {

__device__ __forceinline__ float quant_code(float v, float mn, float sc, float levels) {
    float q = rintf(__fdiv_rn(__fsub_rn(v, mn), sc));
    return fminf(fmaxf(q, 0.0f), levels);
}
// Eight codes at once without eight IEEE divisions.  With rs ~ 1 / sc and nb = -mn * rs,
// q0 = fma(v, rs, nb) lies within 3e-7 * q + 6e-8 * |nb| of the correctly rounded quotient
// q = (v - mn) / sc, so rint(q0) == rint(q) unless q0 is that close to a tie k + 0.5:
// `tie_lo` = 0.5 - (5e-7 * (levels + 1) + 2e-7 * |nb|) is the distance from rint(q0) beyond
// which a lane counts as undecided.  A wave in which any lane is undecided about its code i (or `redo`:
// a scale too small for rcp) redoes code i with the true division -- with 16-bit inputs exact ties are
// common enough that one wave in eight has one among its 512 quotients.  Bit-identical to quant_code;
// the codes come back as floats.
__device__ __forceinline__ void quant_codes8(const float (&v)[8], const float (&mn)[8], const float (&sc)[8],
                                             const float (&rs)[8], const float (&nb)[8], const float (&tie_lo)[8],
                                             float levels, bool redo, float (&q)[8]) {
    bool close = redo, near[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float q0 = __builtin_fmaf(v[i], rs[i], nb[i]);
        const float r = rintf(q0);
        near[i] = fabsf(q0 - r) >= tie_lo[i];
        close |= near[i];
        q[i] = __builtin_amdgcn_fmed3f(r, 0.0f, levels);   // clamp; a NaN becomes 0 as with fmaxf / fminf
    }
    if (__any(close)) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (__any(redo | near[i])) q[i] = quant_code(v[i], mn[i], sc[i], levels);
    }
}
// The same with one limit for all eight codes: the largest distance from a whole number is compared once
// (a NaN quotient is neither close nor far, as above).
__device__ __forceinline__ void quant_codes8(const float (&v)[8], const float (&mn)[8], const float (&sc)[8],
                                             const float (&rs)[8], const float (&nb)[8], float tie, float levels,
                                             bool redo, float (&q)[8]) {
    float far = 0.f, dist[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float q0 = __builtin_fmaf(v[i], rs[i], nb[i]);
        const float r = rintf(q0);
        dist[i] = fabsf(q0 - r);
        far = fmaxf(far, dist[i]);
        q[i] = __builtin_amdgcn_fmed3f(r, 0.0f, levels);
    }
    if (__any(redo | (far >= tie))) {   // common with 16-bit inputs (exact ties): only the codes some lane is unsure of
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (__any(redo | (dist[i] >= tie))) q[i] = quant_code(v[i], mn[i], sc[i], levels);
    }
}
// The same when the parameters of the exact division are not at hand: `slow_params(mn, sc)` fetches them, and only
// a wave that redoes its codes calls it (every lane of the wave does: it may move data between lanes).
template <typename F>
__device__ __forceinline__ void quant_codes8_lazy(const float (&v)[8], const float (&rs)[8], const float (&nb)[8], float tie,
                                                  float levels, bool redo, float (&q)[8], F &&slow_params) {
    float far = 0.f, dist[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float q0 = __builtin_fmaf(v[i], rs[i], nb[i]);
        const float r = rintf(q0);
        dist[i] = fabsf(q0 - r);
        far = fmaxf(far, dist[i]);
        q[i] = __builtin_amdgcn_fmed3f(r, 0.0f, levels);
    }
    if (__any(redo | (far >= tie))) {
        float mn[8], sc[8];
        slow_params(mn, sc);
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (__any(redo | (dist[i] >= tie))) q[i] = quant_code(v[i], mn[i], sc[i], levels);
    }
}
// The same with a level count per code (channels of different bit widths in one row).
__device__ __forceinline__ void quant_codes8(const float (&v)[8], const float (&mn)[8], const float (&sc)[8],
                                             const float (&rs)[8], const float (&nb)[8], float tie,
                                             const float (&levels)[8], bool redo, float (&q)[8]) {
    float far = 0.f, dist[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const float q0 = __builtin_fmaf(v[i], rs[i], nb[i]);
        const float r = rintf(q0);
        dist[i] = fabsf(q0 - r);
        far = fmaxf(far, dist[i]);
        q[i] = __builtin_amdgcn_fmed3f(r, 0.0f, levels[i]);
    }
    if (__any(redo | (far >= tie))) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
            if (__any(redo | (dist[i] >= tie))) q[i] = quant_code(v[i], mn[i], sc[i], levels[i]);
    }
}
__device__ __forceinline__ float tie_limit(float levels, float nb) {
    return 0.5f - (5e-7f * (levels + 1.0f) + 2e-7f * fabsf(nb));
}
// Eight codes (exact small integers held as floats) as one bit field, code i at bit i * bits;
// bits * 8 <= 32.  Sums stay below 2^16 per half, so float arithmetic is exact.
__device__ __forceinline__ uint32_t field8(const float (&q)[8], int bits) {
    const float b = (float)(1 << bits);
    if (bits <= 2) {
        float f = q[7];
#pragma unroll
        for (int i = 6; i >= 0; --i) f = __builtin_fmaf(f, b, q[i]);
        return (uint32_t)f;
    }
    if (bits == 4) {
        const float lo = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(q[3], b, q[2]), b, q[1]), b, q[0]);
        const float hi = __builtin_fmaf(__builtin_fmaf(__builtin_fmaf(q[7], b, q[6]), b, q[5]), b, q[4]);
        return (uint32_t)lo | ((uint32_t)hi << 16);
    }
    return 0;   // 8 bits: two words, see bytes8
}
// eight codes as eight bytes
__device__ __forceinline__ uint2 bytes8(const float (&q)[8]) {
    const uint32_t a = (uint32_t)__builtin_fmaf(q[1], 256.0f, q[0]), b = (uint32_t)__builtin_fmaf(q[3], 256.0f, q[2]);
    const uint32_t c = (uint32_t)__builtin_fmaf(q[5], 256.0f, q[4]), d = (uint32_t)__builtin_fmaf(q[7], 256.0f, q[6]);
    return make_uint2(a | (b << 16), c | (d << 16));
}
__device__ __forceinline__ float fast_rcp(float x) { return __builtin_amdgcn_rcpf(x); }

__device__ __forceinline__ float recon(float q, float sc, float mn) {
    return __fadd_rn(__fmul_rn(q, sc), mn);
}
__device__ __forceinline__ float group_scale(float mn, float mx, float levels, float eps) {
    return fmaxf(__fdiv_rn(__fsub_rn(mx, mn), levels), eps);
}
// The same quotient in three operations where that is proved exact.  For levels = 2^b - 1, b = 1 .. 8, and
// r = 1 / levels rounded to float, q0 = x r, e = fma(-q0, levels, x), q = fma(e, r, q0) is the correctly
// rounded x / levels for every finite non-negative float x, subnormal quotients included: compared with the
// division over all 2 139 095 040 of them for each of the eight level counts on a CPU
// (tests/exact_level_division.c; the test suite runs a sample).  inf and NaN pass through as the division
// passes them.  `inv` is r, or 0 for any other level count (then the division is used).
struct LevelDiv { float levels, inv; };
__device__ __forceinline__ LevelDiv level_div(float levels) {
    const uint32_t n = (uint32_t)levels + 1u;
    const bool proved = (float)(n - 1u) == levels && n >= 2u && n <= 256u && (n & (n - 1u)) == 0u;
    return LevelDiv{levels, proved ? __fdiv_rn(1.0f, levels) : 0.0f};
}
__device__ __forceinline__ float group_scale(float mn, float mx, LevelDiv d, float eps) {
    const float x = __fsub_rn(mx, mn);
    float q;
    if (d.inv != 0.0f) {   // uniform
        const float q0 = __fmul_rn(x, d.inv);
        q = __builtin_fmaf(__builtin_fmaf(-q0, d.levels, x), d.inv, q0);
        q = x < INFINITY ? q : x;
    } else {
        q = __fdiv_rn(x, d.levels);
    }
    return fmaxf(q, eps);
}

template <typename T> __device__ __forceinline__ void load8(const T *p, float (&v)[8]);
template <> __device__ __forceinline__ void load8<f16>(const f16 *p, float (&v)[8]) {
    f16x8 h = *reinterpret_cast<const f16x8 *>(p);
#pragma unroll
    for (int i = 0; i < 8; ++i) v[i] = (float)h[i];
}
template <> __device__ __forceinline__ void load8<bf16_t>(const bf16_t *p, float (&v)[8]) {
    uint4 u = *reinterpret_cast<const uint4 *>(p);
    uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v[2 * i] = __uint_as_float(w[i] << 16);
        v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
}
template <> __device__ __forceinline__ void load8<float>(const float *p, float (&v)[8]) {
    float4 a = *reinterpret_cast<const float4 *>(p);
    float4 b = *reinterpret_cast<const float4 *>(p + 4);
    v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w;
    v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float (&v)[8]);
template <> __device__ __forceinline__ void store8<f16>(f16 *p, const float (&v)[8]) {
    f16x8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = (f16)v[i];
    *reinterpret_cast<f16x8 *>(p) = h;
}
template <> __device__ __forceinline__ void store8<bf16_t>(bf16_t *p, const float (&v)[8]) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) w[i] = (uint32_t)f32_to_bf16(v[2 * i]) | ((uint32_t)f32_to_bf16(v[2 * i + 1]) << 16);
    *reinterpret_cast<uint4 *>(p) = make_uint4(w[0], w[1], w[2], w[3]);
}
template <> __device__ __forceinline__ void store8<float>(float *p, const float (&v)[8]) {
    *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
    *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
}

template <typename M> __device__ __forceinline__ void store_meta(M *p, float v);
template <> __device__ __forceinline__ void store_meta<float>(float *p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_meta<f16>(f16 *p, float v) { *p = (f16)v; }
// eight consecutive scale / zero values, 16-byte aligned destination
template <typename M> __device__ __forceinline__ void store_meta8(M *p, const float (&v)[8]);
template <> __device__ __forceinline__ void store_meta8<float>(float *p, const float (&v)[8]) { store8<float>(p, v); }
template <> __device__ __forceinline__ void store_meta8<f16>(f16 *p, const float (&v)[8]) { store8<f16>(p, v); }
template <typename M> __device__ __forceinline__ float load_meta(const M *p);
template <> __device__ __forceinline__ float load_meta<float>(const float *p) { return *p; }
template <> __device__ __forceinline__ float load_meta<f16>(const f16 *p) { return (float)*p; }

// Write the eight codes one thread owns (channels 8*o .. 8*o+7 of one row) as
// part of a channel-packed row of words.  Every lane of the wave must call it.
template <int LPR>
__device__ __forceinline__ void store_codes_channel_packed(uint32_t *row_words, int o, const float (&q)[8],
                                                           int bits, bool valid) {
    if (bits == 8) {
        if (valid) *reinterpret_cast<uint2 *>(row_words + 2 * o) = bytes8(q);
    } else if (bits == 4) {
        const uint32_t w = field8(q, 4);
        if (valid) row_words[o] = w;
    } else if (bits == 2) {
        const uint32_t f = field8(q, 2);
        uint32_t hi = __shfl_down(f, 1);
        if (valid && (o & 1) == 0) row_words[o >> 1] = f | (hi << 16);
    } else {  // bits == 1
        const uint32_t f = field8(q, 1);
        uint32_t f1 = __shfl_down(f, 1), f2 = __shfl_down(f, 2), f3 = __shfl_down(f, 3);
        if (valid && (o & 3) == 0) row_words[o >> 2] = f | (f1 << 8) | (f2 << 16) | (f3 << 24);
    }
}

// Eight consecutive elements as loaded, with running per-element minima / maxima kept in the
// storage type where that is exact and cheaper (fp16: packed min / max, two elements per
// instruction).
template <typename T> struct Raw8 {
    float v[8];
    struct Acc { float mn[8], mx[8]; };
    __device__ __forceinline__ void load(const T *p) { load8<T>(p, v); }
    __device__ __forceinline__ void floats(float (&o)[8]) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = v[i];
    }
    static __device__ __forceinline__ void init(Acc &a) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { a.mn[i] = INFINITY; a.mx[i] = -INFINITY; }
    }
    __device__ __forceinline__ void fold(Acc &a) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) { a.mn[i] = fminf(a.mn[i], v[i]); a.mx[i] = fmaxf(a.mx[i], v[i]); }
    }
    static __device__ __forceinline__ void result(const Acc &a, float (&mn)[8], float (&mx)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { mn[i] = a.mn[i]; mx[i] = a.mx[i]; }
    }
    // minimum / maximum over the eight elements
    __device__ __forceinline__ void span(float &mn, float &mx) const {
        mn = INFINITY; mx = -INFINITY;
#pragma unroll
        for (int i = 0; i < 8; ++i) { mn = fminf(mn, v[i]); mx = fmaxf(mx, v[i]); }
    }
};
template <> struct Raw8<f16> {
    f16x8 h;
    struct Acc { f16x8 mn, mx; };
    __device__ __forceinline__ void load(const f16 *p) { h = *reinterpret_cast<const f16x8 *>(p); }
    __device__ __forceinline__ void floats(float (&o)[8]) const {
#pragma unroll
        for (int i = 0; i < 8; ++i) o[i] = (float)h[i];
    }
    static __device__ __forceinline__ void init(Acc &a) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { a.mn[i] = (f16)INFINITY; a.mx[i] = (f16)-INFINITY; }
    }
    // bare packed min / max: the compiler's own forms quiet signalling NaNs first, two more
    // instructions per pair, and inputs with NaNs are rejected before they get here
    static __device__ __forceinline__ uint32_t pk_min(uint32_t a, uint32_t b) {
        uint32_t d;
        asm("v_pk_min_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
        return d;
    }
    static __device__ __forceinline__ uint32_t pk_max(uint32_t a, uint32_t b) {
        uint32_t d;
        asm("v_pk_max_f16 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
        return d;
    }
    __device__ __forceinline__ void fold(Acc &a) const {
        typedef uint32_t w4 __attribute__((ext_vector_type(4)));
        w4 mn = __builtin_bit_cast(w4, a.mn), mx = __builtin_bit_cast(w4, a.mx);
        const w4 x = __builtin_bit_cast(w4, h);
#pragma unroll
        for (int i = 0; i < 4; ++i) { mn[i] = pk_min(mn[i], x[i]); mx[i] = pk_max(mx[i], x[i]); }
        a.mn = __builtin_bit_cast(f16x8, mn);
        a.mx = __builtin_bit_cast(f16x8, mx);
    }
    static __device__ __forceinline__ void result(const Acc &a, float (&mn)[8], float (&mx)[8]) {
#pragma unroll
        for (int i = 0; i < 8; ++i) { mn[i] = (float)a.mn[i]; mx[i] = (float)a.mx[i]; }
    }
    __device__ __forceinline__ void span(float &mn, float &mx) const {
        typedef uint32_t w4 __attribute__((ext_vector_type(4)));
        const w4 x = __builtin_bit_cast(w4, h);
        const uint32_t a = pk_min(pk_min(x[0], x[1]), pk_min(x[2], x[3])), b = pk_max(pk_max(x[0], x[1]), pk_max(x[2], x[3]));
        const f16x2 a2 = __builtin_bit_cast(f16x2, a), b2 = __builtin_bit_cast(f16x2, b);
        mn = fminf((float)a2[0], (float)a2[1]);
        mx = fmaxf((float)b2[0], (float)b2[1]);
    }
};

// ---------------------------------------------------------------------------
// Keys: groups along tokens.  One block per (group, bh); 256 threads = RPP rows
// of LPR threads, each thread owning 8 consecutive channels of its rows.
// MODE 0: write the reconstruction; MODE 1: write packed codes + scale/zero.
// ---------------------------------------------------------------------------
constexpr int KT_MAXP = 8;

template <typename T, typename M, int LPR, int MODE, int NP>
__device__ __forceinline__ void kivi_key_tile_body(int bx, int64_t bh,
    const T *__restrict__ x, T *__restrict__ out, int64_t S, int64_t x_stride_bh, int group, float levels,
    float eps, int bits, uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero,
    int64_t cap_tokens, int64_t dst_tok0, int W, const int32_t *__restrict__ rows = nullptr, int64_t rows_stride = 0) {
    constexpr int D = LPR * 8;
    constexpr int RPP = 256 / LPR;
    // `rows` (MODE 0 only): position s of the (b, h) slab stands for row rows[bh * rows_stride + s] of x and of
    // out -- groups are formed over the routed order, rows are read and written where they lie
    auto routed = [&](int64_t s) -> int64_t { return rows != nullptr ? (int64_t)rows[bh * rows_stride + s] : s; };
    // per-row-slot minima / maxima, then the group's (zero, scale, 1 / scale) per channel
    __shared__ __align__(16) float s_mn[RPP][D];
    __shared__ __align__(16) float s_mx[RPP][D];
    __shared__ __align__(16) float s_par[4][D];
    const int gk = bx;
    const int tid = threadIdx.x, r = tid / LPR, o = tid % LPR;
    const int64_t s0 = (int64_t)gk * group;
    const T *xb = x + bh * x_stride_bh;

    Raw8<T> v[NP];   // NP passes of RPP rows cover the group
    typename Raw8<T>::Acc acc;
    Raw8<T>::init(acc);
    // every row is requested before the first is used (and, under a routing, every row number before the first row)
    int64_t src[NP];
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        int rl = p * RPP + r;
        int64_t s = s0 + rl;
        src[p] = rl < group && s < S ? routed(s) : -1;
    }
#pragma unroll
    for (int p = 0; p < NP; ++p)
        if (src[p] >= 0) v[p].load(xb + src[p] * D + 8 * o);
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        int rl = p * RPP + r;
        if (rl < group && s0 + rl < S) v[p].fold(acc);
    }
    float mn[8], mx[8];
    Raw8<T>::result(acc, mn, mx);
    *reinterpret_cast<float4 *>(&s_mn[r][8 * o]) = make_float4(mn[0], mn[1], mn[2], mn[3]);
    *reinterpret_cast<float4 *>(&s_mn[r][8 * o + 4]) = make_float4(mn[4], mn[5], mn[6], mn[7]);
    *reinterpret_cast<float4 *>(&s_mx[r][8 * o]) = make_float4(mx[0], mx[1], mx[2], mx[3]);
    *reinterpret_cast<float4 *>(&s_mx[r][8 * o + 4]) = make_float4(mx[4], mx[5], mx[6], mx[7]);
    __syncthreads();
    // one thread per channel folds the row slots and does the one division of the group
    for (int ch = tid; ch < D; ch += 256) {
        float a = INFINITY, b = -INFINITY;
#pragma unroll
        for (int j = 0; j < RPP; ++j) { a = fminf(a, s_mn[j][ch]); b = fmaxf(b, s_mx[j][ch]); }
        const float scv = group_scale(a, b, level_div(levels), eps);
        const float rsv = fast_rcp(scv);
        s_par[0][ch] = a;
        s_par[1][ch] = scv;
        s_par[2][ch] = rsv;
        s_par[3][ch] = -a * rsv;
    }
    __syncthreads();
    float sc[8], rs[8], nb[8];
    auto row8 = [&](int k, float (&d)[8]) {
        const float4 lo = *reinterpret_cast<const float4 *>(&s_par[k][8 * o]), hi = *reinterpret_cast<const float4 *>(&s_par[k][8 * o + 4]);
        d[0] = lo.x; d[1] = lo.y; d[2] = lo.z; d[3] = lo.w; d[4] = hi.x; d[5] = hi.y; d[6] = hi.z; d[7] = hi.w;
    };
    row8(0, mn); row8(1, sc); row8(2, rs); row8(3, nb);
    bool redo = false;
    float tie_all = 0.5f;   // the tightest of the eight channels' limits
#pragma unroll
    for (int i = 0; i < 8; ++i) { tie_all = fminf(tie_all, tie_limit(levels, nb[i])); redo |= !(rs[i] < 1e30f); }
    if (MODE == 1 && r == 0) {
        int64_t gdst = dst_tok0 / group + gk;
        int64_t gcap = (cap_tokens + group - 1) / group;
        M *sp = scale + (bh * gcap + gdst) * D + 8 * o;
        M *zp = zero + (bh * gcap + gdst) * D + 8 * o;
        store_meta8<M>(sp, sc);
        store_meta8<M>(zp, mn);
    }
#pragma unroll
    for (int p = 0; p < NP; ++p) {
        int rl = p * RPP + r;
        int64_t s = s0 + rl;
        bool valid = rl < group && s < S;
        if (p * RPP >= group) break;  // uniform across the block
        float x8[8], q[8];
        if (valid) v[p].floats(x8);
        else {   // keep the arithmetic defined; the lane's results are not stored
#pragma unroll
            for (int i = 0; i < 8; ++i) x8[i] = mn[i];
        }
        quant_codes8(x8, mn, sc, rs, nb, tie_all, levels, redo, q);
        if (MODE == 0) {
            if (valid) {
                float y[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = recon(q[i], sc[i], mn[i]);
                store8<T>(rows != nullptr ? out + bh * x_stride_bh + src[p] * D + 8 * o : out + (bh * S + s) * D + 8 * o, y);
            }
        } else {
            uint32_t *row = packed + (bh * cap_tokens + dst_tok0 + (valid ? s : 0)) * W;
            store_codes_channel_packed<LPR>(row, o, q, bits, valid);
        }
    }
}

template <typename T, typename M, int LPR, int MODE, int NP>
__global__ __launch_bounds__(256) void kivi_key_tile_kernel(
    const T *__restrict__ x, T *__restrict__ out, int64_t S, int64_t x_stride_bh, int group, float levels,
    float eps, int bits, uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero,
    int64_t cap_tokens, int64_t dst_tok0, int W, const int32_t *__restrict__ rows, int64_t rows_stride) {
    kivi_key_tile_body<T, M, LPR, MODE, NP>((int)blockIdx.x, (int64_t)blockIdx.y, x, out, S, x_stride_bh, group, levels, eps,
                                            bits, packed, scale, zero, cap_tokens, dst_tok0, W, rows, rows_stride);
}

// ---------------------------------------------------------------------------
// Values: groups along channels.  One block per (row tile, bh); a group is
// reduced across g/8 neighbouring lanes.  MODE 0 reconstruction, MODE 1
// channel-packed codes, MODE 2 token-packed codes (transposed through LDS).
// ---------------------------------------------------------------------------
constexpr int VT_TILES = 4;   // row tiles of 256 / LPR rows one block of the value kernel takes

template <typename T, typename M, int LPR, int MODE>
__device__ __forceinline__ void kivi_value_tile_body(int bx, int64_t bh,
    const T *__restrict__ x, T *__restrict__ out, int64_t S, int64_t x_stride_bh, int group, float levels,
    float eps, int bits, uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero,
    int64_t cap_tokens, int64_t dst_tok0, int W) {
    constexpr int D = LPR * 8;
    constexpr int RPP = 256 / LPR;
    constexpr int ROWS = RPP * VT_TILES;
    constexpr int LDS_STRIDE = D + 8;
    __shared__ __align__(8) unsigned char s_codes[MODE == 2 ? ROWS * LDS_STRIDE : 4];
    // token-packed scale / zero rows of the tile, staged so that they leave as whole vectors
    constexpr int MAXGV = 4;
    __shared__ __align__(16) M s_meta[MODE == 2 ? 2 * MAXGV * ROWS : 1];
    const int tid = threadIdx.x, r = tid / LPR, o = tid % LPR;
    const int64_t tile_tok0 = (int64_t)bx * ROWS;
    const int GL = group / 8;  // lanes per group (power of two <= LPR)
    const int GV = D / group;

    // every load of the thread's VT_TILES rows goes out before the first is used
    Raw8<T> v[VT_TILES];
    bool valid[VT_TILES];
#pragma unroll
    for (int j = 0; j < VT_TILES; ++j) {
        const int64_t s = tile_tok0 + j * RPP + r;
        valid[j] = s < S;
        if (valid[j]) v[j].load(x + bh * x_stride_bh + s * D + 8 * o);
    }
#pragma unroll
    for (int j = 0; j < VT_TILES; ++j) {
        const int rl = j * RPP + r;
        const int64_t s = tile_tok0 + rl;
        float mn = INFINITY, mx = -INFINITY;
        if (valid[j]) v[j].span(mn, mx);
        for (int off = 1; off < GL; off <<= 1) {
            mn = fminf(mn, __shfl_xor(mn, off));
            mx = fmaxf(mx, __shfl_xor(mx, off));
        }
        const float sc = group_scale(mn, mx, level_div(levels), eps);
        if (MODE != 0 && valid[j] && (o % GL) == 0) {
            int gv = o / GL;
            if (MODE == 2 && GV <= MAXGV) {
                store_meta<M>(&s_meta[gv * ROWS + rl], sc);
                store_meta<M>(&s_meta[(MAXGV + gv) * ROWS + rl], mn);
            } else {
                int64_t mi = (MODE == 1) ? ((bh * cap_tokens + dst_tok0 + s) * GV + gv)
                                         : ((bh * GV + gv) * cap_tokens + dst_tok0 + s);
                store_meta<M>(scale + mi, sc);
                store_meta<M>(zero + mi, mn);
            }
        }
        float q[8];
        {
            const float rs = fast_rcp(sc), nb = -mn * rs, tl = tie_limit(levels, nb);
            float x8[8], mn8[8], sc8[8], rs8[8], nb8[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) { mn8[i] = mn; sc8[i] = sc; rs8[i] = rs; nb8[i] = nb; }
            if (valid[j]) v[j].floats(x8);
            else {   // keep the arithmetic defined; the lane's results are not stored
#pragma unroll
                for (int i = 0; i < 8; ++i) x8[i] = 0.0f;
            }
            quant_codes8(x8, mn8, sc8, rs8, nb8, tl, levels, !(rs < 1e30f), q);
            if (!valid[j]) {
#pragma unroll
                for (int i = 0; i < 8; ++i) q[i] = 0.0f;
            }
        }
        if (MODE == 0) {
            if (valid[j]) {
                float y[8];
#pragma unroll
                for (int i = 0; i < 8; ++i) y[i] = recon(q[i], sc, mn);
                store8<T>(out + (bh * S + s) * D + 8 * o, y);
            }
            continue;
        }
        if (MODE == 1) {
            uint32_t *row = packed + (bh * cap_tokens + dst_tok0 + (valid[j] ? s : 0)) * W;
            store_codes_channel_packed<LPR>(row, o, q, bits, valid[j]);
        } else {
            *reinterpret_cast<uint2 *>(&s_codes[rl * LDS_STRIDE + 8 * o]) = bytes8(q);
        }
    }
    if (MODE == 2) {
        __syncthreads();
        if (GV <= MAXGV) {
            constexpr int VEC = 16 / (int)sizeof(M);          // elements per 16-byte store
            const int nvec = 2 * GV * (ROWS / VEC);
            const int64_t tok = dst_tok0 + tile_tok0;
            const bool whole = tile_tok0 + ROWS <= S && (tok % VEC) == 0 && (cap_tokens % VEC) == 0;
            for (int idx = tid; idx < nvec; idx += 256) {
                const int which = idx / (GV * (ROWS / VEC)), rem = idx % (GV * (ROWS / VEC));
                const int gv = rem / (ROWS / VEC), t0 = (rem % (ROWS / VEC)) * VEC;
                M *dst = (which ? zero : scale) + (bh * GV + gv) * cap_tokens + tok + t0;
                const M *src = &s_meta[(which * MAXGV + gv) * ROWS + t0];
                if (whole) *reinterpret_cast<uint4 *>(dst) = *reinterpret_cast<const uint4 *>(src);
                else
                    for (int i = 0; i < VEC; ++i)
                        if (tile_tok0 + t0 + i < S) dst[i] = src[i];
            }
        }
        const int per = 32 / bits;
        const int nwords = (ROWS / per) * D;
        for (int idx = tid; idx < nwords; idx += 256) {
            int wl = idx / D, d = idx % D;
            if (tile_tok0 + (int64_t)wl * per >= S) continue;
            uint32_t w = 0;
            for (int i = 0; i < per; ++i) w |= (uint32_t)s_codes[(wl * per + i) * LDS_STRIDE + d] << (i * bits);
            int64_t wrow = (dst_tok0 + tile_tok0) / per + wl;
            packed[(bh * (cap_tokens / per) + wrow) * D + d] = w;
        }
    }
}

template <typename T, typename M, int LPR, int MODE>
__global__ __launch_bounds__(256) void kivi_value_tile_kernel(
    const T *__restrict__ x, T *__restrict__ out, int64_t S, int64_t x_stride_bh, int group, float levels,
    float eps, int bits, uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero,
    int64_t cap_tokens, int64_t dst_tok0, int W) {
    kivi_value_tile_body<T, M, LPR, MODE>((int)blockIdx.x, (int64_t)blockIdx.y, x, out, S, x_stride_bh, group, levels, eps,
                                          bits, packed, scale, zero, cap_tokens, dst_tok0, W);
}

// ---------------------------------------------------------------------------
// Values, token-packed, head_dim 128: a thread owns the PER = 32 / BITS tokens of one packed word for 8
// consecutive channels, so the eight words it writes (one per channel) are made of its own codes -- no
// transposition through LDS -- and leave as one 32-byte piece; the scale / zero of a (token, channel group) are
// reduced across the group's lanes with lane moves inside a row of 16 lanes, and a thread's PER values of a
// channel group leave as whole vectors of the token-major rows.  16 lanes cover the 128 channels of PER tokens,
// a wave four such stretches, a block sixteen.
// ---------------------------------------------------------------------------
template <int CTRL> __device__ __forceinline__ float lane_move(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
// lane k's value in every lane of its quad
template <int K> __device__ __forceinline__ float quad_bcast(float x) { return lane_move<K * 0x55>(x); }
__device__ __forceinline__ float pick4(int i, float a, float b, float c, float d) { return (i & 2) ? ((i & 1) ? d : c) : ((i & 1) ? b : a); }
template <typename M> __device__ __forceinline__ void store_meta2(M *p, float a, float b);
template <> __device__ __forceinline__ void store_meta2<float>(float *p, float a, float b) { *reinterpret_cast<float2 *>(p) = make_float2(a, b); }
template <> __device__ __forceinline__ void store_meta2<f16>(f16 *p, float a, float b) {
    *reinterpret_cast<uint32_t *>(p) = __builtin_bit_cast(uint32_t, f16x2{(f16)a, (f16)b});
}
__device__ __forceinline__ float bare_min(float a, float b) { float d; asm("v_min_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b)); return d; }
__device__ __forceinline__ float bare_max(float a, float b) { float d; asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b)); return d; }
// minimum and maximum over the GL lanes (4, 8 or 16, aligned) that hold a channel group
template <int GL> __device__ __forceinline__ void group_span(float &mn, float &mx) {
    mn = bare_min(mn, lane_move<0xB1>(mn)); mx = bare_max(mx, lane_move<0xB1>(mx));     // quad_perm [1,0,3,2]
    mn = bare_min(mn, lane_move<0x4E>(mn)); mx = bare_max(mx, lane_move<0x4E>(mx));     // quad_perm [2,3,0,1]
    if constexpr (GL >= 8) { mn = bare_min(mn, lane_move<0x141>(mn)); mx = bare_max(mx, lane_move<0x141>(mx)); }   // row_half_mirror
    if constexpr (GL >= 16) { mn = bare_min(mn, lane_move<0x140>(mn)); mx = bare_max(mx, lane_move<0x140>(mx)); }  // row_mirror
}
constexpr int VP_STRETCHES = 16;   // stretches of PER tokens per block of 256 threads

// The same walk writing the reconstruction instead (the round trip): stretches of 8 tokens, the last one of a
// sequence may be short.
template <typename T, int GL>
__global__ __launch_bounds__(256) void kivi_value_roundtrip_kernel(const T *__restrict__ x, T *__restrict__ out, int64_t S,
                                                                   int64_t x_stride_bh, float levels, float eps) {
    constexpr int D = 128, PER = 8;
    const int tid = threadIdx.x, o = tid & 15;
    const int64_t bh = blockIdx.y;
    const int64_t t0 = ((int64_t)blockIdx.x * VP_STRETCHES + (tid >> 4)) * PER;
    if (t0 >= S) return;
    const T *xb = x + bh * x_stride_bh + t0 * D + 8 * o;
    T *ob = out + (bh * S + t0) * D + 8 * o;
    const LevelDiv ld = level_div(levels);
    Raw8<T> v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) v[i].load(xb + (t0 + i < S ? (int64_t)i * D : 0));   // past the end: the first row again
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        float mn, mx;
        v[i].span(mn, mx);
        group_span<GL>(mn, mx);
        const float sc = group_scale(mn, mx, ld, eps), rs = fast_rcp(sc), nb = -mn * rs, tl = tie_limit(levels, nb);
        float x8[8], q[8], y[8], mn8[8], sc8[8], rs8[8], nb8[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) { mn8[c] = mn; sc8[c] = sc; rs8[c] = rs; nb8[c] = nb; }
        v[i].floats(x8);
        quant_codes8(x8, mn8, sc8, rs8, nb8, tl, levels, !(rs < 1e30f), q);
#pragma unroll
        for (int c = 0; c < 8; ++c) y[c] = recon(q[c], sc, mn);
        if (t0 + i < S) store8<T>(ob + (int64_t)i * D, y);
    }
}

// The GL lanes of a channel group hold the same (token, group) extrema after the fold: with GL = 4 or 8 each of them
// works out the scale, reciprocal and offset of 8 / GL of every eight tokens and the group passes them round.
// value of the lane four lanes up (lanes 0-3, 8-11 of a row of 16) or down (lanes 4-7, 12-15)
__device__ __forceinline__ float other_quad(float x) {
    int t = __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x104, 0xF, 0x5, false);   // row_shl:4 into quads 0, 2
    t = __builtin_amdgcn_update_dpp(t, __builtin_bit_cast(int, x), 0x114, 0xF, 0xA, false);       // row_shr:4 into quads 1, 3
    return __builtin_bit_cast(float, t);
}
// all[t], t = 0..7: element t % TP of lane t / TP of the group (TP = 8 / GL)
template <int GL> __device__ __forceinline__ void group_gather8(const float (&own)[8 / GL], bool upper_quad, float (&all)[8]) {
    if constexpr (GL == 4) {
        all[0] = quad_bcast<0>(own[0]); all[1] = quad_bcast<0>(own[1]); all[2] = quad_bcast<1>(own[0]); all[3] = quad_bcast<1>(own[1]);
        all[4] = quad_bcast<2>(own[0]); all[5] = quad_bcast<2>(own[1]); all[6] = quad_bcast<3>(own[0]); all[7] = quad_bcast<3>(own[1]);
    } else {
        const float other = other_quad(own[0]);
        const float lo = upper_quad ? other : own[0], hi = upper_quad ? own[0] : other;   // lanes 0-3 / 4-7 of the group
        all[0] = quad_bcast<0>(lo); all[1] = quad_bcast<1>(lo); all[2] = quad_bcast<2>(lo); all[3] = quad_bcast<3>(lo);
        all[4] = quad_bcast<0>(hi); all[5] = quad_bcast<1>(hi); all[6] = quad_bcast<2>(hi); all[7] = quad_bcast<3>(hi);
    }
}
// element TP * j + e of eight values, j the lane's place in its group
template <int GL> __device__ __forceinline__ float group_pick8(int j, int e, const float (&v)[8]) {
    if constexpr (GL == 4) return pick4(j, v[e], v[2 + e], v[4 + e], v[6 + e]);
    else return (j & 4) ? pick4(j, v[4], v[5], v[6], v[7]) : pick4(j, v[0], v[1], v[2], v[3]);
}

template <typename T, typename M, int BITS, int GL, bool TWO = false>
__device__ __forceinline__ void kivi_value_pack_body(int bx, int64_t bh, const T *__restrict__ x, int64_t S,
                                                     int64_t x_stride_bh, float levels, float eps,
                                                     uint32_t *__restrict__ packed, M *__restrict__ scale,
                                                     M *__restrict__ zero, int64_t cap_tokens, int64_t dst_tok0,
                                                     const T *__restrict__ alt = nullptr, int64_t alt_first = 0,
                                                     int64_t alt_rs = 128) {
    constexpr int D = 128, PER = 32 / BITS, HALF = PER / 2, GV = 16 / GL;
    constexpr bool SHARE = GL <= 8;
    constexpr int TP = SHARE ? 8 / GL : 1;
    const int tid = threadIdx.x, o = tid & 15;
    const int64_t t0 = ((int64_t)bx * VP_STRETCHES + (tid >> 4)) * PER;   // the stretch's first token
    if (t0 >= S) return;                                                  // S is a multiple of PER: whole rows of 16 lanes leave
    // TWO: tokens from alt_first (a multiple of PER) on are rows of a second tensor, as in the key body
    const bool from_alt = TWO && t0 >= alt_first;
    const int64_t rs = from_alt ? alt_rs : (int64_t)D;
    const T *xb = (from_alt ? alt + (t0 - alt_first) * rs : x + bh * x_stride_bh + t0 * D) + 8 * o;
    const LevelDiv ld = level_div(levels);
    Raw8<T> v[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) v[i].load(xb + (int64_t)i * rs);
    float lo[8], hi[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) { lo[c] = 0.f; hi[c] = 0.f; }
    const int64_t tok = dst_tok0 + t0;
    const int64_t mi = (bh * GV + o / GL) * cap_tokens + tok;
    auto code_fields = [&](int i, const float (&q)[8]) __attribute__((always_inline)) {
        // code of token i at bits [BITS * i, BITS * (i + 1)): two exact float sums of 16 bits each
        const float w = (float)(1u << (BITS * (i % HALF)));
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            if (i < HALF) lo[c] = __builtin_fmaf(q[c], w, lo[c]);
            else hi[c] = __builtin_fmaf(q[c], w, hi[c]);
        }
    };
    if constexpr (SHARE) {
        const int j = o & (GL - 1);
        const bool upper_quad = (o & 4) != 0;
#pragma unroll
        for (int i0 = 0; i0 < PER; i0 += 8) {
            float mnb[8], mxb[8];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v[i0 + i].span(mnb[i], mxb[i]);
                group_span<GL>(mnb[i], mxb[i]);
            }
            float own_sc[TP], own_rs[TP], own_nb[TP], own_mn[TP], tie = 0.5f;
            bool redo = false;   // the lane's own tokens: any lane's flag redoes the whole wave
#pragma unroll
            for (int e = 0; e < TP; ++e) {
                own_mn[e] = group_pick8<GL>(j, e, mnb);
                own_sc[e] = group_scale(own_mn[e], group_pick8<GL>(j, e, mxb), ld, eps);
                own_rs[e] = fast_rcp(own_sc[e]);
                own_nb[e] = -own_mn[e] * own_rs[e];
                tie = fminf(tie, tie_limit(levels, own_nb[e]));
                redo |= !(own_rs[e] < 1e30f);
            }
            // one limit for the eight tokens, the tightest: a few more rows take the division
            tie = fminf(tie, lane_move<0xB1>(tie));
            tie = fminf(tie, lane_move<0x4E>(tie));
            if constexpr (GL == 8) tie = fminf(tie, lane_move<0x141>(tie));
            float rsb[8], nbb[8];
            group_gather8<GL>(own_rs, upper_quad, rsb);
            group_gather8<GL>(own_nb, upper_quad, nbb);
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                float x8[8], q[8], rs8[8], nb8[8];
#pragma unroll
                for (int c = 0; c < 8; ++c) { rs8[c] = rsb[i]; nb8[c] = nbb[i]; }
                v[i0 + i].floats(x8);
                quant_codes8_lazy(x8, rs8, nb8, tie, levels, redo, q, [&](float (&m8)[8], float (&s8)[8]) {
                    float scb[8];
                    group_gather8<GL>(own_sc, upper_quad, scb);
#pragma unroll
                    for (int c = 0; c < 8; ++c) { m8[c] = mnb[i]; s8[c] = scb[i]; }
                });
                code_fields(i0 + i, q);
            }
            // every lane its own tokens' scale and zero
            if constexpr (TP == 2) {
                store_meta2<M>(scale + mi + i0 + 2 * j, own_sc[0], own_sc[1]);
                store_meta2<M>(zero + mi + i0 + 2 * j, own_mn[0], own_mn[1]);
            } else {
                store_meta<M>(scale + mi + i0 + j, own_sc[0]);
                store_meta<M>(zero + mi + i0 + j, own_mn[0]);
            }
        }
    } else {
        float scv[PER], mnv[PER];
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            float mn, mx;
            v[i].span(mn, mx);
            group_span<GL>(mn, mx);
            const float sc = group_scale(mn, mx, ld, eps), rs = fast_rcp(sc), nb = -mn * rs, tl = tie_limit(levels, nb);
            scv[i] = sc;
            mnv[i] = mn;
            float x8[8], q[8], mn8[8], sc8[8], rs8[8], nb8[8];
#pragma unroll
            for (int c = 0; c < 8; ++c) { mn8[c] = mn; sc8[c] = sc; rs8[c] = rs; nb8[c] = nb; }
            v[i].floats(x8);
            quant_codes8(x8, mn8, sc8, rs8, nb8, tl, levels, !(rs < 1e30f), q);
            code_fields(i, q);
        }
        if ((o & (GL - 1)) == 0) {   // the first lane of a channel group writes its PER scales and zeros
#pragma unroll
            for (int i = 0; i < PER; i += 8) {
                const float s8[8] = {scv[i], scv[i + 1], scv[i + 2], scv[i + 3], scv[i + 4], scv[i + 5], scv[i + 6], scv[i + 7]};
                const float z8[8] = {mnv[i], mnv[i + 1], mnv[i + 2], mnv[i + 3], mnv[i + 4], mnv[i + 5], mnv[i + 6], mnv[i + 7]};
                store_meta8<M>(scale + mi + i, s8);
                store_meta8<M>(zero + mi + i, z8);
            }
        }
    }
    uint32_t wd[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) wd[c] = (uint32_t)lo[c] | ((uint32_t)hi[c] << 16);
    uint4 *wp = reinterpret_cast<uint4 *>(packed + (bh * (cap_tokens / PER) + tok / PER) * D + 8 * o);
    wp[0] = make_uint4(wd[0], wd[1], wd[2], wd[3]);
    wp[1] = make_uint4(wd[4], wd[5], wd[6], wd[7]);
}

template <typename T, typename M, int BITS, int GL>
__global__ __launch_bounds__(256) void kivi_value_pack_kernel(const T *__restrict__ x, int64_t S, int64_t x_stride_bh,
                                                              float levels, float eps, uint32_t *__restrict__ packed,
                                                              M *__restrict__ scale, M *__restrict__ zero,
                                                              int64_t cap_tokens, int64_t dst_tok0) {
    kivi_value_pack_body<T, M, BITS, GL>((int)blockIdx.x, (int64_t)blockIdx.y, x, S, x_stride_bh, levels, eps, packed, scale,
                                         zero, cap_tokens, dst_tok0);
}

// ---------------------------------------------------------------------------
// Keys, head_dim 128, groups of 4 * TPL tokens (32 or 64): one wave per group.  Lane 4 * o + tq owns 8
// consecutive channels (chunk o of 16) of the TPL tokens tq * TPL .. of the group, so the per-channel minima and
// maxima are folded in the lane and then across the four lanes of a quad with lane moves -- no block-shared
// memory, no barrier -- and every lane ends up with the parameters of its 8 channels.  A row's 8 codes are one
// 4-bit word (two lanes' fields make a 2-bit word).  MODE 0 writes the reconstruction, MODE 1 codes + scale/zero.
// ---------------------------------------------------------------------------
template <typename T> struct QuadFold {   // fold a Raw8 accumulator across the quad
    static __device__ __forceinline__ void run(typename Raw8<T>::Acc &a) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            a.mn[i] = bare_min(a.mn[i], lane_move<0xB1>(a.mn[i])); a.mx[i] = bare_max(a.mx[i], lane_move<0xB1>(a.mx[i]));
            a.mn[i] = bare_min(a.mn[i], lane_move<0x4E>(a.mn[i])); a.mx[i] = bare_max(a.mx[i], lane_move<0x4E>(a.mx[i]));
        }
    }
};
template <> struct QuadFold<f16> {
    template <int CTRL> static __device__ __forceinline__ uint32_t mv(uint32_t x) {
        return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)x, CTRL, 0xF, 0xF, true);
    }
    static __device__ __forceinline__ void run(Raw8<f16>::Acc &a) {
        typedef uint32_t w4 __attribute__((ext_vector_type(4)));
        w4 mn = __builtin_bit_cast(w4, a.mn), mx = __builtin_bit_cast(w4, a.mx);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            mn[i] = Raw8<f16>::pk_min(mn[i], mv<0xB1>(mn[i])); mx[i] = Raw8<f16>::pk_max(mx[i], mv<0xB1>(mx[i]));
            mn[i] = Raw8<f16>::pk_min(mn[i], mv<0x4E>(mn[i])); mx[i] = Raw8<f16>::pk_max(mx[i], mv<0x4E>(mx[i]));
        }
        a.mn = __builtin_bit_cast(f16x8, mn);
        a.mx = __builtin_bit_cast(f16x8, mx);
    }
};
constexpr int KQ_WAVES = 4;   // groups per block

// MIXED (round trip only): channel c of (sequence, head) bh has `levels_hi` levels where hi_mask[bh * 128 + c] is
// set and `levels` otherwise (Kitty's channel-wise mixed precision, veloxquant_mlx/quantizers/kitty.py:138-169,
// which forms both reconstructions of the whole tensor and selects per channel).
// TWO (the cache's append): tokens from `alt_first` on are rows of a second tensor, `alt` being the row of token
// alt_first for this (sequence, head) and `alt_rs` its row stride in elements; alt_first is a multiple of the group
// (or lies at or past S), so a group reads one source.
template <typename T, typename M, int MODE, int TPL, bool MIXED = false, bool TWO = false>
__device__ __forceinline__ void kivi_key_quad_body(int gk, int64_t bh, const T *__restrict__ x, T *__restrict__ out, int64_t S,
                                                   int64_t x_stride_bh, float levels, float eps, int bits,
                                                   uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero,
                                                   int64_t cap_tokens, int64_t dst_tok0, int W,
                                                   const uint8_t *__restrict__ hi_mask = nullptr, float levels_hi = 0.f,
                                                   const float *__restrict__ group_levels = nullptr,
                                                   const T *__restrict__ alt = nullptr, int64_t alt_first = 0, int64_t alt_rs = 128) {
    constexpr int D = 128, G = 4 * TPL;
    const int lane = threadIdx.x & 63, o = lane >> 2, tq = lane & 3;
    const int64_t s0 = (int64_t)gk * G;
    if (s0 >= S) return;   // the whole wave
    const int64_t r0 = s0 + tq * TPL;   // the lane's first token
    const bool from_alt = TWO && s0 >= alt_first;   // the same for the wave
    const int64_t row_gap = from_alt ? alt_rs : (int64_t)D;   // elements between rows (a constant without TWO)
    const T *xg = (from_alt ? alt + (s0 - alt_first) * row_gap : x + bh * x_stride_bh + s0 * D) + 8 * o;   // the group's first row
    const T *xb = xg + (int64_t)(tq * TPL) * row_gap;
    if (group_levels != nullptr) {   // round trip only: a level count per token group, 0 = the group passes through
        levels = group_levels[gk];
        if (levels == 0.f) {
#pragma unroll
            for (int i = 0; i < TPL; ++i)
                if (r0 + i < S) *reinterpret_cast<uint4 *>(out + (bh * S + r0 + i) * D + 8 * o) = *reinterpret_cast<const uint4 *>(xb + (int64_t)i * row_gap);
            return;
        }
    }
    Raw8<T> v[TPL];
    typename Raw8<T>::Acc acc;
    Raw8<T>::init(acc);
    // a whole group (all but the last of a ragged sequence): every row is requested before the first is used
    const bool whole = s0 + G <= S;   // the same for the wave
    if (whole) {
#pragma unroll
        for (int i = 0; i < TPL; ++i) v[i].load(xb + (int64_t)i * row_gap);
#pragma unroll
        for (int i = 0; i < TPL; ++i) v[i].fold(acc);
    } else {   // a row past the end stands in as the group's first row, which changes no minimum or maximum
#pragma unroll
        for (int i = 0; i < TPL; ++i) v[i].load(r0 + i < S ? xb + (int64_t)i * row_gap : xg);
#pragma unroll
        for (int i = 0; i < TPL; ++i) v[i].fold(acc);
    }
    QuadFold<T>::run(acc);
    float mn[8], mx[8], sc[8], rs[8], nb[8];
    Raw8<T>::result(acc, mn, mx);
    const LevelDiv ld = level_div(levels);
    LevelDiv ldh = ld;
    uint2 hi8 = make_uint2(0u, 0u);   // MIXED: the lane's eight mask bytes
    if constexpr (MIXED) {
        ldh = level_div(levels_hi);
        hi8 = *reinterpret_cast<const uint2 *>(hi_mask + bh * D + 8 * o);
    }
    float lv[8];
    bool redo = false;
    float tie_all = 0.5f;   // one limit for the lane's 8 channels, the tightest: a few more rows take the division
    float own_sc[2] = {0.f, 0.f};
    if constexpr (MIXED) {
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            const bool hi = (((c < 4 ? hi8.x : hi8.y) >> (8 * (c & 3))) & 0xFFu) != 0u;
            const LevelDiv d = hi ? ldh : ld;
            lv[c] = d.levels;
            sc[c] = group_scale(mn[c], mx[c], d, eps);
            rs[c] = fast_rcp(sc[c]);
            nb[c] = -mn[c] * rs[c];
            tie_all = fminf(tie_all, tie_limit(lv[c], nb[c]));
            redo |= !(rs[c] < 1e30f);
        }
    } else {
        // The four lanes of a quad hold the same eight minima and maxima: lane tq works out the parameters of
        // channels 2 tq and 2 tq + 1 only and the quad passes them round (a quarter of the divisions; the same
        // values, so the same codes).  `redo` stays the lane's own: any lane's flag redoes the whole wave.
        float own_rs[2], own_nb[2];
#pragma unroll
        for (int e = 0; e < 2; ++e) {
            const float m = pick4(tq, mn[e], mn[2 + e], mn[4 + e], mn[6 + e]), x = pick4(tq, mx[e], mx[2 + e], mx[4 + e], mx[6 + e]);
            own_sc[e] = group_scale(m, x, ld, eps);
            own_rs[e] = fast_rcp(own_sc[e]);
            own_nb[e] = -m * own_rs[e];
            tie_all = fminf(tie_all, tie_limit(levels, own_nb[e]));
            redo |= !(own_rs[e] < 1e30f);
        }
        tie_all = fminf(tie_all, lane_move<0xB1>(tie_all));
        tie_all = fminf(tie_all, lane_move<0x4E>(tie_all));
#define VQ_QUAD_GATHER(DST, SRC) \
        DST[0] = quad_bcast<0>(SRC[0]); DST[1] = quad_bcast<0>(SRC[1]); DST[2] = quad_bcast<1>(SRC[0]); DST[3] = quad_bcast<1>(SRC[1]); \
        DST[4] = quad_bcast<2>(SRC[0]); DST[5] = quad_bcast<2>(SRC[1]); DST[6] = quad_bcast<3>(SRC[0]); DST[7] = quad_bcast<3>(SRC[1])
        VQ_QUAD_GATHER(rs, own_rs);
        VQ_QUAD_GATHER(nb, own_nb);
        if (MODE == 0) { VQ_QUAD_GATHER(sc, own_sc); }
    }
    if (MODE == 1) {
        const int64_t gdst = dst_tok0 / G + gk, gcap = (cap_tokens + G - 1) / G;
        if constexpr (MIXED) {
            if (tq == 0) {
                store_meta8<M>(scale + (bh * gcap + gdst) * D + 8 * o, sc);
                store_meta8<M>(zero + (bh * gcap + gdst) * D + 8 * o, mn);
            }
        } else {   // every lane its own two channels
            store_meta2<M>(scale + (bh * gcap + gdst) * D + 8 * o + 2 * tq, own_sc[0], own_sc[1]);
            store_meta2<M>(zero + (bh * gcap + gdst) * D + 8 * o + 2 * tq, pick4(tq, mn[0], mn[2], mn[4], mn[6]),
                           pick4(tq, mn[1], mn[3], mn[5], mn[7]));
        }
    }
    uint32_t *const words0 = MODE == 1 ? packed + (bh * cap_tokens + dst_tok0 + r0) * W : nullptr;   // the lane's first row of words
    auto rows = [&](auto whole_group) __attribute__((always_inline)) {
        constexpr bool WHOLE = decltype(whole_group)::value;
#pragma unroll
        for (int i = 0; i < TPL; ++i) {
            const int64_t srow = r0 + i;
            const bool valid = WHOLE || srow < S;
            float x8[8], q[8];
            v[i].floats(x8);   // a row past the end holds the group's first row; its results are not stored
            if constexpr (MIXED) quant_codes8(x8, mn, sc, rs, nb, tie_all, lv, redo, q);
            else if (MODE == 0) quant_codes8(x8, mn, sc, rs, nb, tie_all, levels, redo, q);
            else
                quant_codes8_lazy(x8, rs, nb, tie_all, levels, redo, q, [&](float (&m8)[8], float (&s8)[8]) {
#pragma unroll
                    for (int c = 0; c < 8; ++c) m8[c] = mn[c];
                    VQ_QUAD_GATHER(s8, own_sc);
                });
            if (MODE == 0) {
                if (valid) {
                    float y[8];
#pragma unroll
                    for (int c = 0; c < 8; ++c) y[c] = recon(q[c], sc[c], mn[c]);
                    store8<T>(out + (bh * S + srow) * D + 8 * o, y);
                }
            } else {
                // (a whole group: one base for the lane's rows, the rows a constant apart)
                uint32_t *row_words = WHOLE ? words0 + (int64_t)i * W : packed + (bh * cap_tokens + dst_tok0 + (valid ? srow : 0)) * W;
                if (bits == 8) {
                    if (valid) *reinterpret_cast<uint2 *>(row_words + 2 * o) = bytes8(q);
                } else if (bits == 4) {
                    const uint32_t w = field8(q, 4);
                    if (valid) row_words[o] = w;
                } else {   // 2 bits: chunk o + 1 sits four lanes up
                    const uint32_t f = field8(q, 2);
                    const uint32_t up = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)f, 0x104, 0xF, 0xF, true);   // row_shl:4
                    if (valid && (o & 1) == 0) row_words[o >> 1] = f | (up << 16);
                }
            }
        }
    };
    if (whole) rows(std::true_type{});
    else rows(std::false_type{});
}

#undef VQ_QUAD_GATHER

template <typename T, typename M, int MODE, int TPL>
__global__ __launch_bounds__(64 * KQ_WAVES) void kivi_key_quad_kernel(
    const T *__restrict__ x, T *__restrict__ out, int64_t S, int64_t x_stride_bh, float levels, float eps, int bits,
    uint32_t *__restrict__ packed, M *__restrict__ scale, M *__restrict__ zero, int64_t cap_tokens, int64_t dst_tok0, int W) {
    kivi_key_quad_body<T, M, MODE, TPL>((int)blockIdx.x * KQ_WAVES + (int)(threadIdx.x >> 6), (int64_t)blockIdx.y, x, out, S,
                                        x_stride_bh, levels, eps, bits, packed, scale, zero, cap_tokens, dst_tok0, W);
}

// Keys and values of one cache flush in a single launch: blocks [0, key_blocks) of a (b, h)
// take the key groups, the rest the value row tiles.  The two bodies are those of the kernels
// above; a chunked prefill flushes a few hundred tokens at a time, where a second launch costs
// as much as the work.
struct PackDst { uint32_t *packed; void *scale, *zero; };
// the same for head_dim 128, groups of 32 or 64, 2 or 4 bits, token-packed values: the quad-layout key body and the
// word-owning value body, neither of which uses block-shared memory
template <typename T, int TPL>
__global__ __launch_bounds__(64 * KQ_WAVES) void kivi_key_quad_mixed_kernel(const T *__restrict__ x, T *__restrict__ out, int64_t S,
                                                                           int64_t x_stride_bh, float levels_lo, float levels_hi,
                                                                           const uint8_t *__restrict__ hi_mask, float eps) {
    kivi_key_quad_body<T, float, 0, TPL, true>((int)blockIdx.x * KQ_WAVES + (int)(threadIdx.x >> 6), (int64_t)blockIdx.y, x, out, S,
                                               x_stride_bh, levels_lo, eps, 0, nullptr, nullptr, nullptr, 0, 0, 0, hi_mask, levels_hi);
}

// Round trip with a level count per token group (AgeTieredKV: windows of different ages at different bit widths,
// veloxquant_mlx/quantizers/age_tiered.py:117-174); fp16 / bf16 rows only (a passing group is copied as 16-byte pieces).
template <typename T, int TPL>
__global__ __launch_bounds__(64 * KQ_WAVES) void kivi_key_quad_grouplevels_kernel(const T *__restrict__ x, T *__restrict__ out, int64_t S,
                                                                                 int64_t x_stride_bh, const float *__restrict__ group_levels,
                                                                                 float eps) {
    kivi_key_quad_body<T, float, 0, TPL>((int)blockIdx.x * KQ_WAVES + (int)(threadIdx.x >> 6), (int64_t)blockIdx.y, x, out, S, x_stride_bh,
                                         1.f, eps, 0, nullptr, nullptr, nullptr, 0, 0, 0, nullptr, 0.f, group_levels);
}

// Sum and sum of squares over the tokens of every channel of x [N, S, D] in double precision: block (chunk, n)
// takes a stretch of tokens, a thread eight channels of every (256 / LPR)-th token of it, and writes
// partial[((n * chunks + chunk) * 2 + which) * D + channel]; the few partials of a channel are added by the caller
// (in a fixed order: the result does not depend on scheduling).
template <typename T, int LPR>
__global__ __launch_bounds__(256) void channel_moments_kernel(const T *__restrict__ x, int64_t S, int64_t x_stride_n,
                                                              double *__restrict__ partial, int64_t tokens_per_chunk) {
    constexpr int D = LPR * 8, RPP = 256 / LPR, RPW = 64 / LPR;   // rows per pass of the block / of a wave
    __shared__ double s_part[4][2][D];
    const int tid = threadIdx.x, o = tid % LPR, r = tid / LPR, wave = tid >> 6;
    const int64_t n = blockIdx.y, t_begin = (int64_t)blockIdx.x * tokens_per_chunk;
    const int64_t t_end = t_begin + tokens_per_chunk < S ? t_begin + tokens_per_chunk : S;
    double sum[8], sq[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) { sum[c] = 0.0; sq[c] = 0.0; }
    const T *xb = x + n * x_stride_n + 8 * o;
    // four rows are requested before the first is added (the sums keep their order: row by row)
    int64_t t = t_begin + r;
    for (; t + 3 * RPP < t_end; t += 4 * RPP) {
        float v[4][8];
#pragma unroll
        for (int i = 0; i < 4; ++i) load8<T>(xb + (t + i * RPP) * D, v[i]);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int c = 0; c < 8; ++c) { sum[c] += (double)v[i][c]; sq[c] += (double)v[i][c] * (double)v[i][c]; }
        }
    }
    for (; t < t_end; t += RPP) {
        float v[8];
        load8<T>(xb + t * D, v);
#pragma unroll
        for (int c = 0; c < 8; ++c) { sum[c] += (double)v[c]; sq[c] += (double)v[c] * (double)v[c]; }
    }
    // rows of a wave sit LPR lanes apart
#pragma unroll
    for (int c = 0; c < 8; ++c) {
#pragma unroll
        for (int off = LPR; off < 64; off <<= 1) { sum[c] += __shfl_xor(sum[c], off); sq[c] += __shfl_xor(sq[c], off); }
    }
    if ((tid & 63) < LPR) {
#pragma unroll
        for (int c = 0; c < 8; ++c) { s_part[wave][0][8 * o + c] = sum[c]; s_part[wave][1][8 * o + c] = sq[c]; }
    }
    __syncthreads();
    (void)RPW;
    for (int e = tid; e < 2 * D; e += 256) {
        const int which = e / D, ch = e % D;
        const double total = ((s_part[0][which][ch] + s_part[1][which][ch]) + s_part[2][which][ch]) + s_part[3][which][ch];
        partial[((n * gridDim.x + blockIdx.x) * 2 + which) * D + ch] = total;
    }
}

// variance[n][c] = max(sq / S - (sum / S)^2, 0) from the partial sums of channel_moments_kernel, the chunks added
// in order, double arithmetic with one rounding per operation, the result rounded to float32.
__global__ __launch_bounds__(256) void channel_variance_kernel(const double *__restrict__ partial, int64_t N, int chunks, int D,
                                                               double n_tokens, float *__restrict__ variance) {
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= N * D) return;
    const int64_t n = e / D;
    const int c = (int)(e - n * D);
    double sum = 0.0, sq = 0.0;
    for (int k = 0; k < chunks; ++k) {
        sum += partial[((n * chunks + k) * 2 + 0) * D + c];
        sq += partial[((n * chunks + k) * 2 + 1) * D + c];
    }
    const double mean = sum / n_tokens;
    const double var = sq / n_tokens - mean * mean;
    variance[e] = (float)(var > 0.0 ? var : (var == var ? 0.0 : var));   // clamp at zero; a NaN stays a NaN
}

// mask[n][c] = 1 where channel c is among the n_hi largest of variance[n][:]: the rank of a channel is the number
// of channels that come before it in a stable ascending sort of -variance (equal values: the lower channel first;
// a NaN after every number), one block of D threads per row.
__global__ void channel_hi_mask_kernel(const float *__restrict__ variance, int D, int n_hi, uint8_t *__restrict__ mask) {
    extern __shared__ uint32_t s_key[];
    const int c = threadIdx.x;
    const int64_t n = blockIdx.x;
    // -variance as an unsigned key that orders like the sort: -0 and +0 alike, NaN last
    const float t = -variance[n * D + c] + 0.0f;
    const uint32_t b = __float_as_uint(t);
    const uint32_t key = t != t ? 0xFFFFFFFFu : ((b & 0x80000000u) ? ~b : (b | 0x80000000u));
    s_key[c] = key;
    __syncthreads();
    int before = 0;
    for (int j = 0; j < D; ++j) {
        const uint32_t kj = s_key[j];
        before += (kj < key) || (kj == key && j < c);
    }
    mask[n * D + c] = before < n_hi ? 1 : 0;
}

template <typename T, typename M, int BITS, int TPL>
__global__ __launch_bounds__(256) void kivi_kv_pack_kernel(
    const T *__restrict__ k, const T *__restrict__ v, int64_t S, int64_t x_stride_bh, float levels, float eps, PackDst kd,
    PackDst vd, int64_t cap_tokens, int64_t dst_tok0, int key_blocks) {
    const int bx = (int)blockIdx.x;
    if (bx < key_blocks)
        kivi_key_quad_body<T, M, 1, TPL>(bx * KQ_WAVES + (int)(threadIdx.x >> 6), (int64_t)blockIdx.y, k, nullptr, S, x_stride_bh,
                                         levels, eps, BITS, kd.packed, (M *)kd.scale, (M *)kd.zero, cap_tokens, dst_tok0,
                                         128 / (32 / BITS));
    else
        kivi_value_pack_body<T, M, BITS, TPL / 2>(bx - key_blocks, (int64_t)blockIdx.y, v, S, x_stride_bh, levels, eps, vd.packed,
                                                  (M *)vd.scale, (M *)vd.zero, cap_tokens, dst_tok0);
}
// A whole append of the packed cache in one launch: the keys and values of tokens [0, n_flush) of [tail ; new rows]
// are quantised and packed straight from where they lie (new rows are not copied into the tail first), and the rows
// from n_flush on, old or new, go to the front of the spare tail.  Blocks [0, key_blocks) take key groups, the next
// value_blocks the value stretches, the rest the kept rows (one 16-byte piece a thread).
struct NewRows { const void *k, *v; int64_t k_sb, k_sh, k_ss, v_sb, v_sh, v_ss; };   // strides in elements
template <typename T, typename M, int BITS, int TPL>
__global__ __launch_bounds__(256) void kivi_kv_append_kernel(
    const T *__restrict__ k_tail, const T *__restrict__ v_tail, int64_t tail_cap, NewRows nw, int H, int64_t n_tail, int64_t n_flush,
    int64_t need, float levels, float eps, PackDst kd, PackDst vd, int64_t cap_tokens, int64_t dst_tok0, int key_blocks,
    int value_blocks, T *__restrict__ k_spare, T *__restrict__ v_spare, int64_t spare_cap) {
    constexpr int D = 128;
    const int bx = (int)blockIdx.x;
    const int64_t bh = blockIdx.y, b = bh / H, h = bh - b * H;
    const T *kn = (const T *)nw.k + b * nw.k_sb + h * nw.k_sh, *vn = (const T *)nw.v + b * nw.v_sb + h * nw.v_sh;
    if (bx < key_blocks) {
        kivi_key_quad_body<T, M, 1, TPL, false, true>(bx * KQ_WAVES + (int)(threadIdx.x >> 6), bh, k_tail, nullptr, n_flush, tail_cap * D,
                                                      levels, eps, BITS, kd.packed, (M *)kd.scale, (M *)kd.zero, cap_tokens, dst_tok0,
                                                      128 / (32 / BITS), nullptr, 0.f, nullptr, kn, n_tail, nw.k_ss);
    } else if (bx < key_blocks + value_blocks) {
        kivi_value_pack_body<T, M, BITS, TPL / 2, true>(bx - key_blocks, bh, v_tail, n_flush, tail_cap * D, levels, eps, vd.packed,
                                                        (M *)vd.scale, (M *)vd.zero, cap_tokens, dst_tok0, vn, n_tail, nw.v_ss);
    } else {
        constexpr int RV = D * (int)sizeof(T) / 16;   // 16-byte pieces of a row
        const int64_t keep = need - n_flush, i = (int64_t)(bx - key_blocks - value_blocks) * 256 + threadIdx.x;
        if (i >= 2 * keep * RV) return;
        const bool values = i >= keep * RV;
        const int64_t j = values ? i - keep * RV : i, r = n_flush + j / RV, c = j % RV;
        const T *tail = values ? v_tail : k_tail, *fresh = values ? vn : kn;
        const int64_t fs = values ? nw.v_ss : nw.k_ss;
        const uint4 x = r < n_tail ? reinterpret_cast<const uint4 *>(tail + (bh * tail_cap + r) * D)[c]
                                   : reinterpret_cast<const uint4 *>(fresh + (r - n_tail) * fs)[c];
        reinterpret_cast<uint4 *>((values ? v_spare : k_spare) + (bh * spare_cap + (r - n_flush)) * D)[c] = x;
    }
}

template <typename T, typename M, int LPR, int NP, int VMODE>
__global__ __launch_bounds__(256) void kivi_kv_tile_kernel(
    const T *__restrict__ k, const T *__restrict__ v, int64_t S, int64_t x_stride_bh, int group, float levels, float eps,
    int bits, PackDst kd, PackDst vd, int64_t cap_tokens, int64_t dst_tok0, int W, int key_blocks) {
    const int bx = (int)blockIdx.x;
    if (bx < key_blocks)
        kivi_key_tile_body<T, M, LPR, 1, NP>(bx, (int64_t)blockIdx.y, k, nullptr, S, x_stride_bh, group, levels, eps, bits,
                                             kd.packed, (M *)kd.scale, (M *)kd.zero, cap_tokens, dst_tok0, W);
    else
        kivi_value_tile_body<T, M, LPR, VMODE>(bx - key_blocks, (int64_t)blockIdx.y, v, nullptr, S, x_stride_bh, group, levels,
                                               eps, bits, vd.packed, (M *)vd.scale, (M *)vd.zero, cap_tokens, dst_tok0, W);
}

// ---------------------------------------------------------------------------
// Generic kernels: every thread rescans the group(s) it needs.
// ---------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void scan_group(const T *xb, int64_t S, int64_t D, int axis, int group, int64_t s,
                                           int64_t d, float &mn, float &mx) {
    mn = INFINITY; mx = -INFINITY;
    if (axis == VQ_AXIS_TOKEN) {
        int64_t a = (s / group) * group, b = a + group < S ? a + group : S;
        for (int64_t t = a; t < b; ++t) { float v = Elem<T>::ld(xb + t * D + d); mn = fminf(mn, v); mx = fmaxf(mx, v); }
    } else {
        int64_t a = (d / group) * group, b = a + group < D ? a + group : D;
        for (int64_t t = a; t < b; ++t) { float v = Elem<T>::ld(xb + s * D + t); mn = fminf(mn, v); mx = fmaxf(mx, v); }
    }
}

template <typename T>
__global__ void kivi_roundtrip_generic_kernel(const T *__restrict__ x, T *__restrict__ out, int64_t BH, int64_t S,
                                              int64_t D, int axis, int group, float levels, float eps) {
    int64_t n = BH * S * D;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t d = e % D, s = (e / D) % S, bh = e / (D * S);
        const T *xb = x + bh * S * D;
        float mn, mx;
        scan_group<T>(xb, S, D, axis, group, s, d, mn, mx);
        float sc = group_scale(mn, mx, levels, eps);
        float v = Elem<T>::ld(xb + s * D + d);
        Elem<T>::st(out + e, recon(quant_code(v, mn, sc, levels), sc, mn));
    }
}

// One thread per output word.  layout 0: word = `per` channels of one token
// (keys, or channel-packed values); layout 1: word = `per` tokens of one channel.
template <typename T, typename M>
__global__ void kivi_pack_generic_kernel(const T *__restrict__ x, int64_t BH, int64_t S, int64_t D,
                                         int64_t x_stride_bh, int axis, int group, float levels, float eps,
                                         int bits, int layout, uint32_t *__restrict__ packed,
                                         M *__restrict__ scale, M *__restrict__ zero, int64_t cap_tokens,
                                         int64_t dst_tok0) {
    const int per = 32 / bits;
    const int64_t W = (D + per - 1) / per;
    const int64_t GV = (D + group - 1) / group;
    const int64_t GKcap = (cap_tokens + group - 1) / group;
    const int64_t rows = layout == 0 ? S : (S + per - 1) / per;
    const int64_t cols = layout == 0 ? W : D;
    const int64_t n = BH * rows * cols;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t c = e % cols, rr = (e / cols) % rows, bh = e / (cols * rows);
        const T *xb = x + bh * x_stride_bh;
        uint32_t word = 0;
        for (int i = 0; i < per; ++i) {
            int64_t s = layout == 0 ? rr : rr * per + i;
            int64_t d = layout == 0 ? c * per + i : c;
            if (s >= S || d >= D) continue;
            float mn, mx;
            scan_group<T>(xb, S, D, axis, group, s, d, mn, mx);
            float sc = group_scale(mn, mx, levels, eps);
            float v = Elem<T>::ld(xb + s * D + d);
            word |= (uint32_t)quant_code(v, mn, sc, levels) << (i * bits);
            // the thread that meets the first element of a group records its parameters
            if (axis == VQ_AXIS_TOKEN) {
                if (s % group == 0) {
                    int64_t mi = (bh * GKcap + (dst_tok0 + s) / group) * D + d;
                    store_meta<M>(scale + mi, sc);
                    store_meta<M>(zero + mi, mn);
                }
            } else if (d % group == 0) {
                int64_t mi = layout == 0 ? ((bh * cap_tokens + dst_tok0 + s) * GV + d / group)
                                         : ((bh * GV + d / group) * cap_tokens + dst_tok0 + s);
                store_meta<M>(scale + mi, sc);
                store_meta<M>(zero + mi, mn);
            }
        }
        if (layout == 0)
            packed[(bh * cap_tokens + dst_tok0 + rr) * W + c] = word;
        else
            packed[(bh * (cap_tokens / per) + dst_tok0 / per + rr) * D + c] = word;
    }
}

// Reconstruction from packed codes: one thread per output element.
template <typename O, typename M>
__global__ void kivi_dequant_kernel(const uint32_t *__restrict__ packed, const M *__restrict__ scale,
                                    const M *__restrict__ zero, int64_t BH, int64_t S, int64_t D, int axis,
                                    int group, int bits, int layout, int64_t cap_tokens, int64_t src_tok0,
                                    O *__restrict__ out) {
    const int per = 32 / bits;
    const int64_t W = (D + per - 1) / per;
    const int64_t GV = (D + group - 1) / group;
    const int64_t GKcap = (cap_tokens + group - 1) / group;
    const uint32_t mask = bits == 32 ? 0xffffffffu : ((1u << bits) - 1u);
    const int64_t n = BH * S * D;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t d = e % D, s = (e / D) % S, bh = e / (D * S);
        int64_t t = src_tok0 + s;
        uint32_t word;
        int sh;
        if (layout == 0) {
            word = packed[(bh * cap_tokens + t) * W + d / per];
            sh = (int)(d % per) * bits;
        } else {
            word = packed[(bh * (cap_tokens / per) + t / per) * D + d];
            sh = (int)(t % per) * bits;
        }
        float c = (float)((word >> sh) & mask);
        int64_t mi;
        if (axis == VQ_AXIS_TOKEN) mi = (bh * GKcap + t / group) * D + d;
        else mi = layout == 0 ? ((bh * cap_tokens + t) * GV + d / group) : ((bh * GV + d / group) * cap_tokens + t);
        Elem<O>::st(out + e, recon(c, load_meta<M>(scale + mi), load_meta<M>(zero + mi)));
    }
}

// The same reconstruction, eight consecutive channels of a token per thread, for D % 8 == 0, group % 8 == 0 and
// 2, 4 or 8 bits: a thread's codes are one piece of one or two words (channel-packed) or the same field of eight
// consecutive words (token-packed), its scale / zero eight consecutive values (keys) or one (values), and the eight
// results leave as one store.  PB = log2(bits).
template <typename O, typename M, int PB>
__global__ __launch_bounds__(256) void kivi_dequant8_kernel(const uint32_t *__restrict__ packed, const M *__restrict__ scale,
                                                            const M *__restrict__ zero, int64_t n_rows, int64_t S, int D, int axis,
                                                            int group, int layout, int64_t cap_tokens, int64_t src_tok0,
                                                            O *__restrict__ out) {
    constexpr int BITS = 1 << PB, PER = 32 / BITS;
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    const int pieces = D / 8;
    const int64_t e = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (e >= n_rows * pieces) return;
    const int64_t row = e / pieces;                 // bh * S + s
    const int d0 = 8 * (int)(e - row * pieces);
    const int64_t bh = row / S, t = src_tok0 + (row - bh * S);
    float c[8];
    if (layout == 0) {
        const uint32_t *w = packed + (bh * cap_tokens + t) * ((D + PER - 1) / PER);
        if constexpr (PER >= 8) {
            const uint32_t x = w[d0 / PER] >> ((d0 % PER) * BITS);
#pragma unroll
            for (int i = 0; i < 8; ++i) c[i] = (float)((x >> (i * BITS)) & MASK);
        } else {   // 8 bits: two words
            const uint2 x = *reinterpret_cast<const uint2 *>(w + d0 / PER);
#pragma unroll
            for (int i = 0; i < 4; ++i) { c[i] = (float)((x.x >> (8 * i)) & 255u); c[4 + i] = (float)((x.y >> (8 * i)) & 255u); }
        }
    } else {
        const uint32_t *w = packed + (bh * (cap_tokens / PER) + t / PER) * D + d0;
        const uint4 a = *reinterpret_cast<const uint4 *>(w), b = *reinterpret_cast<const uint4 *>(w + 4);
        const int sh = (int)(t % PER) * BITS;
        const uint32_t x[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
        for (int i = 0; i < 8; ++i) c[i] = (float)((x[i] >> sh) & MASK);
    }
    float y[8];
    if (axis == VQ_AXIS_TOKEN) {
        const int64_t mi = (bh * ((cap_tokens + group - 1) / group) + t / group) * D + d0;
        float sc[8], zr[8];
        load8<M>(scale + mi, sc);
        load8<M>(zero + mi, zr);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = recon(c[i], sc[i], zr[i]);
    } else {
        const int64_t GV = D / group;
        const int64_t mi = layout == 0 ? (bh * cap_tokens + t) * GV + d0 / group : (bh * GV + d0 / group) * cap_tokens + t;
        const float sc = load_meta<M>(scale + mi), zr = load_meta<M>(zero + mi);
#pragma unroll
        for (int i = 0; i < 8; ++i) y[i] = recon(c[i], sc, zr);
    }
    store8<O>(out + row * D + d0, y);
}

__global__ void pack_words_kernel(const uint8_t *__restrict__ idx, int64_t rows, int64_t D, int bits,
                                  uint32_t *__restrict__ words) {
    const int per = 32 / bits;
    const int64_t W = (D + per - 1) / per, n = rows * W;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t w = e % W, r = e / W;
        uint32_t acc = 0;
        for (int i = 0; i < per; ++i) {
            int64_t d = w * per + i;
            if (d < D) acc |= ((uint32_t)idx[r * D + d]) << (i * bits);
        }
        words[e] = acc;
    }
}
__global__ void unpack_words_kernel(const uint32_t *__restrict__ words, int64_t rows, int64_t D, int bits,
                                    uint8_t *__restrict__ idx) {
    const int per = 32 / bits;
    const int64_t W = (D + per - 1) / per, n = rows * D;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t d = e % D, r = e / D;
        idx[e] = (uint8_t)((words[r * W + d / per] >> ((d % per) * bits)) & mask);
    }
}
__global__ void bit_pack_kernel(const uint8_t *__restrict__ idx, int64_t nbytes, int bits, uint8_t *__restrict__ packed) {
    const int per = 8 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < nbytes; e += (int64_t)gridDim.x * blockDim.x) {
        uint32_t acc = 0;
        for (int i = 0; i < per; ++i) acc |= ((uint32_t)idx[e * per + i] & mask) << (i * bits);
        packed[e] = (uint8_t)acc;
    }
}
__global__ void bit_unpack_kernel(const uint8_t *__restrict__ packed, int64_t n, int bits, uint8_t *__restrict__ idx) {
    const int per = 8 / bits;
    const uint32_t mask = (1u << bits) - 1u;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x)
        idx[e] = (uint8_t)((packed[e / per] >> ((e % per) * bits)) & mask);
}

static inline int grid_for(int64_t n, int block) {
    int64_t g = (n + block - 1) / block;
    if (g < 1) g = 1;
    if (g > 65536 * 16) g = 65536 * 16;
    return (int)g;
}
// L2 norm of every row of x [n_rows, D] in float32: LPR = D / 8 lanes per row, 16-byte loads, the squares
// summed per lane and then across the row's lanes.
template <typename T, int LPR>
__global__ __launch_bounds__(256) void row_norm_kernel(const T *__restrict__ x, int64_t n_rows, float *__restrict__ out) {
    constexpr int D = LPR * 8, RPB = 256 / LPR;
    const int tid = threadIdx.x, r = tid / LPR, o = tid % LPR;
    for (int64_t row = (int64_t)blockIdx.x * RPB + r; row < n_rows; row += (int64_t)gridDim.x * RPB) {
        float v[8];
        load8<T>(x + row * D + 8 * o, v);
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < 8; ++i) acc = __builtin_fmaf(v[i], v[i], acc);
#pragma unroll
        for (int off = 1; off < LPR; off <<= 1) acc += __shfl_xor(acc, off);
        if (o == 0) out[row] = sqrtf(acc);
    }
}

// Routing order of one salience block: for every row of norms [BH, S] (non-negative float32; their bit patterns
// order like the values), the positions of the S - n_hi rows outside the n_hi largest norms in ascending order,
// then the positions of the n_hi largest in ascending order; equal norms at the threshold go to the later
// positions first.  One block per row: a radix select over the norm bits (four passes of eight bits) finds the
// threshold and how many rows equal to it are taken, then every thread walks a contiguous stretch of positions
// twice (count, then write) around a block-wide scan, which keeps both parts in order.
constexpr int ZR_THREADS = 256;
__global__ __launch_bounds__(ZR_THREADS) void zip_route_kernel(const float *__restrict__ norms, int64_t S, int64_t n_hi,
                                                               int32_t *__restrict__ order) {
    __shared__ unsigned s_hist[256];
    __shared__ unsigned s_prefix, s_pmask;
    __shared__ long long s_want;
    __shared__ long long s_cnt[ZR_THREADS];
    const int tid = threadIdx.x;
    const uint32_t *key = reinterpret_cast<const uint32_t *>(norms) + (int64_t)blockIdx.x * S;
    int32_t *dst = order + (int64_t)blockIdx.x * S;
    if (tid == 0) { s_prefix = 0; s_pmask = 0; s_want = n_hi; }
    for (int shift = 24; shift >= 0; shift -= 8) {
        s_hist[tid] = 0;
        __syncthreads();
        const unsigned prefix = s_prefix, pmask = s_pmask;
        for (int64_t i = tid; i < S; i += ZR_THREADS) {
            const uint32_t k = key[i];
            if ((k & pmask) == prefix) atomicAdd(&s_hist[(k >> shift) & 255u], 1u);
        }
        __syncthreads();
        if (tid == 0) {   // the digit in which the s_want-th largest of the rows that match so far lies
            long long above = 0;
            int b = 255;
            for (; b > 0; --b) {
                if (above + s_hist[b] >= s_want) break;
                above += s_hist[b];
            }
            s_want -= above;
            s_prefix = prefix | ((unsigned)b << shift);
            s_pmask = pmask | (255u << shift);
        }
        __syncthreads();
    }
    const uint32_t v = s_prefix;          // the threshold norm
    const long long take_eq = s_want;     // rows equal to it that belong to the block, the latest ones
    const int64_t C = (S + ZR_THREADS - 1) / ZR_THREADS;
    const int64_t i0 = (int64_t)tid * C < S ? (int64_t)tid * C : S, i1 = i0 + C < S ? i0 + C : S;
    long long eq_here = 0;
    for (int64_t i = i0; i < i1; ++i) eq_here += key[i] == v;
    s_cnt[tid] = eq_here;
    __syncthreads();
    long long eq_after = 0;               // rows equal to the threshold in later stretches
    for (int t = tid + 1; t < ZR_THREADS; ++t) eq_after += s_cnt[t];
    __syncthreads();
    // a row equal to the threshold is taken when at most take_eq such rows lie at or after it
    long long seen = 0, sel_here = 0;
    for (int64_t i = i0; i < i1; ++i) {
        const uint32_t k = key[i];
        const bool eq = k == v;
        sel_here += k > v || (eq && eq_after + eq_here - seen <= take_eq);
        seen += eq;
    }
    s_cnt[tid] = sel_here;
    __syncthreads();
    long long sel_before = 0;
    for (int t = 0; t < tid; ++t) sel_before += s_cnt[t];
    int64_t out_sel = (S - n_hi) + sel_before, out_rest = i0 - sel_before;
    seen = 0;
    for (int64_t i = i0; i < i1; ++i) {
        const uint32_t k = key[i];
        const bool eq = k == v;
        const bool sel = k > v || (eq && eq_after + eq_here - seen <= take_eq);
        seen += eq;
        if (sel) dst[out_sel++] = (int32_t)i;
        else dst[out_rest++] = (int32_t)i;
    }
}

// The same order for rows of at most ZR_THREADS * KPT norms, with every norm of the row in a register (position
// j * ZR_THREADS + tid): one read of the norms, the histogram's digit found by all threads at once (a suffix sum over
// the 256 bins instead of one thread walking them), and the two ordered parts written from per-wave ballots -- chunk j
// of 256 positions, wave w, lane l is the order of the positions, so "rows before" and "equal rows at or after" are
// sums over whole (chunk, wave) cells plus bits of the lane's own ballot.
template <int KPT>
__global__ __launch_bounds__(ZR_THREADS) void zip_route_regs_kernel(const float *__restrict__ norms, int S, int n_hi,
                                                                    int32_t *__restrict__ order) {
    constexpr int NW = ZR_THREADS / 64, CELLS = KPT * NW;
    static_assert(CELLS <= ZR_THREADS, "one thread per (chunk, wave) cell");
    __shared__ unsigned s_hist[256];
    __shared__ unsigned s_wsum[NW];
    __shared__ unsigned s_prefix, s_pmask;
    __shared__ int s_want;
    __shared__ int s_cell[CELLS];
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const uint32_t *key = reinterpret_cast<const uint32_t *>(norms) + (int64_t)blockIdx.x * S;
    int32_t *dst = order + (int64_t)blockIdx.x * S;
    uint32_t k[KPT];
#pragma unroll
    for (int j = 0; j < KPT; ++j) k[j] = j * ZR_THREADS + tid < S ? key[j * ZR_THREADS + tid] : 0u;
    if (tid == 0) { s_prefix = 0; s_pmask = 0; s_want = n_hi; }
    for (int shift = 24; shift >= 0; shift -= 8) {
        s_hist[tid] = 0;
        __syncthreads();
        const unsigned prefix = s_prefix, pmask = s_pmask;
        const int want = s_want;
#pragma unroll
        for (int j = 0; j < KPT; ++j)
            if (j * ZR_THREADS + tid < S && (k[j] & pmask) == prefix) atomicAdd(&s_hist[(k[j] >> shift) & 255u], 1u);
        __syncthreads();
        // rows in bins above bin `tid`: a suffix sum over the 256 bins
        const unsigned h = s_hist[tid];
        unsigned suf = h;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const unsigned up = __shfl_down(suf, off);
            if (lane + off < 64) suf += up;
        }
        if (lane == 0) s_wsum[wave] = suf;
        __syncthreads();
        unsigned above = suf - h;
        for (int w = wave + 1; w < NW; ++w) above += s_wsum[w];
        // the digit in which the want-th largest of the rows that match so far lies (bin 0 if none above holds it)
        if ((int)above < want && (tid == 0 || (int)(above + h) >= want)) {
            s_want = want - (int)above;
            s_prefix = prefix | ((unsigned)tid << shift);
            s_pmask = pmask | (255u << shift);
        }
        __syncthreads();
    }
    const uint32_t v = s_prefix;     // the threshold norm
    const int take_eq = s_want;      // rows equal to it that belong to the block, the latest ones
    const unsigned long long lt = (1ull << lane) - 1ull;   // the lanes before this one
    // exclusive prefix sum of s_cell over the cells in (chunk, wave) order, in place; returns the total
    auto scan_cells = [&]() __attribute__((always_inline)) {
        int x = tid < CELLS ? s_cell[tid] : 0;
        const int own = x;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) {
            const int dn = __shfl_up(x, off);
            if (lane >= off) x += dn;
        }
        if (lane == 63) s_wsum[wave] = (unsigned)x;
        __syncthreads();
        int base = 0, total = 0;
        for (int w = 0; w < NW; ++w) { if (w < wave) base += (int)s_wsum[w]; total += (int)s_wsum[w]; }
        if (tid < CELLS) s_cell[tid] = base + x - own;
        __syncthreads();
        return total;
    };
    // rows equal to the threshold, per cell
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const unsigned long long b = __ballot(j * ZR_THREADS + tid < S && k[j] == v);
        if (lane == 0) s_cell[j * NW + wave] = __popcll(b);
    }
    __syncthreads();
    const int eq_total = scan_cells();
    // a row equal to the threshold is taken when at most take_eq such rows lie at or after it
    unsigned sel_bits = 0;   // bit j: the lane's row of chunk j belongs to the high block
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const bool in = j * ZR_THREADS + tid < S, eq = in && k[j] == v;
        const unsigned long long b = __ballot(eq);
        const int at_or_after = eq_total - s_cell[j * NW + wave] - __popcll(b & lt);
        if (in && (k[j] > v || (eq && at_or_after <= take_eq))) sel_bits |= 1u << j;
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const unsigned long long b = __ballot((sel_bits >> j) & 1u);
        if (lane == 0) s_cell[j * NW + wave] = __popcll(b);
    }
    __syncthreads();
    scan_cells();
#pragma unroll
    for (int j = 0; j < KPT; ++j) {
        const int i = j * ZR_THREADS + tid;
        const bool sel = (sel_bits >> j) & 1u;
        const unsigned long long b = __ballot(sel);
        const int before = s_cell[j * NW + wave] + __popcll(b & lt);   // rows of the high block at earlier positions
        if (i < S) dst[sel ? (S - n_hi) + before : i - before] = i;
    }
}

static inline bool pow2(int64_t v) { return v > 0 && (v & (v - 1)) == 0; }
static inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace vq

using namespace vq;

// ---- launchers ----------------------------------------------------------------

template <typename T, typename M, int LPR>
static void launch_key_tile(int mode, const void *x, void *out, int64_t BH, int64_t S, int64_t xs, int group,
                            int levels, float eps, int bits, void *packed, void *scale, void *zero, int64_t cap,
                            int64_t tok0, hipStream_t st, const int32_t *rows = nullptr, int64_t rows_stride = 0) {
    dim3 grid((unsigned)cdiv(S, group), (unsigned)BH);
    int W = (int)cdiv(LPR * 8, 32 / (bits > 0 ? bits : 8));
    // fewer passes held in registers let more blocks share a CU
    constexpr int RPP = 256 / LPR;
    const bool small = group <= (KT_MAXP / 2) * RPP;
#define VQ_LK(MODE, NP)                                                                                               \
    hipLaunchKernelGGL((kivi_key_tile_kernel<T, M, LPR, MODE, NP>), grid, dim3(256), 0, st, (const T *)x, (T *)out, S, \
                       xs, group, (float)levels, eps, bits, (uint32_t *)packed, (M *)scale, (M *)zero, cap, tok0, W, rows, rows_stride)
    if (mode == 0) { if (small) VQ_LK(0, KT_MAXP / 2); else VQ_LK(0, KT_MAXP); }
    else { if (small) VQ_LK(1, KT_MAXP / 2); else VQ_LK(1, KT_MAXP); }
#undef VQ_LK
}
template <typename T, typename M, int LPR>
static void launch_value_tile(int mode, const void *x, void *out, int64_t BH, int64_t S, int64_t xs, int group,
                              int levels, float eps, int bits, void *packed, void *scale, void *zero, int64_t cap,
                              int64_t tok0, hipStream_t st) {
    constexpr int ROWS = (256 / LPR) * VT_TILES;
    dim3 grid((unsigned)cdiv(S, ROWS), (unsigned)BH);
    int W = (int)cdiv(LPR * 8, 32 / (bits > 0 ? bits : 8));
#define VQ_LV(MODE)                                                                                                  \
    hipLaunchKernelGGL((kivi_value_tile_kernel<T, M, LPR, MODE>), grid, dim3(256), 0, st, (const T *)x, (T *)out, S, \
                       xs, group, (float)levels, eps, bits, (uint32_t *)packed, (M *)scale, (M *)zero, cap, tok0, W)
    if (mode == 0) VQ_LV(0);
    else if (mode == 1) VQ_LV(1);
    else VQ_LV(2);
#undef VQ_LV
}

// mode: 0 round trip, 1 channel-packed codes, 2 token-packed codes (values only)
template <typename T, typename M>
static bool try_tile_path(int mode, int axis, const void *x, void *out, int64_t BH, int64_t S, int64_t D, int64_t xs,
                          int group, int levels, float eps, int bits, void *packed, void *scale, void *zero,
                          int64_t cap, int64_t tok0, hipStream_t st) {
    if (!(D == 64 || D == 128 || D == 256)) return false;
    if (!aligned16(x) || (xs % 8) != 0 || BH > 65535) return false;
    if (mode == 0 && !aligned16(out)) return false;
    if (mode != 0 && !(bits == 1 || bits == 2 || bits == 4 || bits == 8)) return false;
    if (mode != 0 && !(aligned16(packed) && aligned16(scale) && aligned16(zero))) return false;
    const int LPR = (int)(D / 8), RPP = 256 / LPR;
    if (axis == VQ_AXIS_TOKEN) {
        if (D == 128 && (group == 32 || group == 64) && (mode == 0 || bits == 2 || bits == 4 || bits == 8)) {
            const dim3 grid((unsigned)cdiv(cdiv(S, group), KQ_WAVES), (unsigned)BH);
            const int W = (int)cdiv(D, 32 / (bits > 0 ? bits : 8));
#define VQ_KQ(MODE, TPL)                                                                                                  \
            hipLaunchKernelGGL((kivi_key_quad_kernel<T, M, MODE, TPL>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, \
                               S, xs, (float)levels, eps, bits, (uint32_t *)packed, (M *)scale, (M *)zero, cap, tok0, W)
            if (mode == 0) { if (group == 32) VQ_KQ(0, 8); else VQ_KQ(0, 16); }
            else { if (group == 32) VQ_KQ(1, 8); else VQ_KQ(1, 16); }
#undef VQ_KQ
            return true;
        }
        if (group > KT_MAXP * RPP) return false;
#define VQ_K(L) launch_key_tile<T, M, L>(mode, x, out, BH, S, xs, group, levels, eps, bits, packed, scale, zero, cap, tok0, st)
        if (LPR == 8) VQ_K(8); else if (LPR == 16) VQ_K(16); else VQ_K(32);
#undef VQ_K
        return true;
    }
    if (group % 8 != 0 || !pow2(group / 8) || group > D || D % group != 0) return false;
    if (mode == 0 && D == 128 && group >= 32) {
        const dim3 grid((unsigned)cdiv(S, VP_STRETCHES * 8), (unsigned)BH);
#define VQ_VR(GL) hipLaunchKernelGGL((kivi_value_roundtrip_kernel<T, GL>), grid, dim3(256), 0, st, (const T *)x, (T *)out, S, xs, (float)levels, eps)
        if (group == 32) VQ_VR(4); else if (group == 64) VQ_VR(8); else VQ_VR(16);
#undef VQ_VR
        return true;
    }
    if (mode == 2 && D == 128 && (bits == 2 || bits == 4) && group >= 32 && !std::is_same<T, float>::value &&
        S % (32 / bits) == 0 && tok0 % 8 == 0 && cap % 8 == 0) {
        const dim3 grid((unsigned)cdiv(S, VP_STRETCHES * (32 / bits)), (unsigned)BH);
#define VQ_VP(BITS, GL)                                                                                              \
        hipLaunchKernelGGL((kivi_value_pack_kernel<T, M, BITS, GL>), grid, dim3(256), 0, st, (const T *)x, S, xs,       \
                           (float)levels, eps, (uint32_t *)packed, (M *)scale, (M *)zero, cap, tok0)
        if (bits == 4) { if (group == 32) VQ_VP(4, 4); else if (group == 64) VQ_VP(4, 8); else VQ_VP(4, 16); }
        else { if (group == 32) VQ_VP(2, 4); else if (group == 64) VQ_VP(2, 8); else VQ_VP(2, 16); }
#undef VQ_VP
        return true;
    }
    if (mode == 2 && ((RPP * VT_TILES) % (32 / bits)) != 0) return false;   // a block's rows hold whole words
#define VQ_V(L) launch_value_tile<T, M, L>(mode, x, out, BH, S, xs, group, levels, eps, bits, packed, scale, zero, cap, tok0, st)
    if (LPR == 8) VQ_V(8); else if (LPR == 16) VQ_V(16); else VQ_V(32);
#undef VQ_V
    return true;
}

namespace vq {
// Keys (groups along tokens) and values (groups along channels, v_layout) of the same S tokens in
// one launch where the tile kernels take the shape, else as two single calls.
// The whole append as one launch where the fused key / value kernel takes the shape (head size 128, 16-bit rows,
// token-packed values, groups of 32 / 64, 2 or 4 bits) and no group of flushed tokens mixes old and new rows.
bool append_one_launch(const void *k_new, const void *v_new, const int64_t ks[3], const int64_t vs[3], const void *k_tail,
                       const void *v_tail, void *k_spare, void *v_spare, int dtype, int64_t B, int64_t H, int64_t D, int64_t tail_cap,
                       int64_t spare_cap, int64_t n_tail, int64_t n_flush, int64_t need, int group, int levels, float eps, int bits,
                       int v_layout, void *kp, void *ksc, void *kz, void *vp, void *vsc, void *vz, int meta_dtype, int64_t cap,
                       int64_t tok0, void *stream) {
    const int per = bits >= 1 && bits <= 8 ? 32 / bits : 1;
    const int64_t BH = B * H;
    const bool ok = D == 128 && (dtype == VQ_F16 || dtype == VQ_BF16) && (meta_dtype == VQ_F16 || meta_dtype == VQ_F32) && BH >= 1 &&
                    BH <= 65535 && H <= 0x7fffffff && n_flush >= 1 && v_layout == VQ_V_TOKEN_PACKED && (group == 32 || group == 64) &&
                    (bits == 2 || bits == 4) && levels >= 1 && levels <= (1 << bits) - 1 && tok0 >= 0 && tok0 + n_flush <= cap &&
                    tok0 % group == 0 && tok0 % per == 0 && n_flush % per == 0 && cap % per == 0 && tok0 % 8 == 0 && cap % 8 == 0 &&
                    (n_tail >= n_flush || n_tail % group == 0) && aligned16(k_tail) && aligned16(v_tail) && aligned16(k_new) &&
                    aligned16(v_new) && aligned16(k_spare) && aligned16(v_spare) && aligned16(kp) && aligned16(ksc) && aligned16(kz) &&
                    aligned16(vp) && aligned16(vsc) && aligned16(vz) && ks[0] % 8 == 0 && ks[1] % 8 == 0 && ks[2] % 8 == 0 &&
                    vs[0] % 8 == 0 && vs[1] % 8 == 0 && vs[2] % 8 == 0;
    if (!ok) return false;
    const int kb = (int)cdiv(cdiv(n_flush, group), KQ_WAVES), vb = (int)cdiv(n_flush, VP_STRETCHES * per);
    const int64_t keep = need - n_flush;
    const int rb = (int)cdiv(2 * keep * (D * 2 / 16), 256);
    const dim3 grid((unsigned)(kb + vb + rb), (unsigned)BH);
    const PackDst kd = {(uint32_t *)kp, ksc, kz}, vd = {(uint32_t *)vp, vsc, vz};
    const NewRows nw = {k_new, v_new, ks[0], ks[1], ks[2], vs[0], vs[1], vs[2]};
    hipStream_t st = (hipStream_t)stream;
#define VQ_AP(T, M, BITS, TPL)                                                                                                  \
    hipLaunchKernelGGL((kivi_kv_append_kernel<T, M, BITS, TPL>), grid, dim3(256), 0, st, (const T *)k_tail, (const T *)v_tail, tail_cap, \
                       nw, (int)H, n_tail, n_flush, need, (float)levels, eps, kd, vd, cap, tok0, kb, vb, (T *)k_spare, (T *)v_spare,    \
                       spare_cap)
#define VQ_AP_B(T, M)                                                                                  \
    do {                                                                                               \
        if (bits == 4) { if (group == 32) VQ_AP(T, M, 4, 8); else VQ_AP(T, M, 4, 16); }                \
        else { if (group == 32) VQ_AP(T, M, 2, 8); else VQ_AP(T, M, 2, 16); }                          \
    } while (0)
    if (dtype == VQ_F16) { if (meta_dtype == VQ_F16) VQ_AP_B(f16, f16); else VQ_AP_B(f16, float); }
    else { if (meta_dtype == VQ_F16) VQ_AP_B(bf16_t, f16); else VQ_AP_B(bf16_t, float); }
#undef VQ_AP_B
#undef VQ_AP
    return true;
}

int pack_kv_pair(const void *k, const void *v, int dtype, int64_t BH, int64_t S, int64_t D, int64_t xs, int group,
                 int levels, float eps, int bits, int v_layout, void *kp, void *ks, void *kz, void *vp, void *vs, void *vz,
                 int meta_dtype, int64_t cap, int64_t tok0, void *stream) {
    const int per = bits >= 1 && bits <= 8 ? 32 / bits : 1;
    constexpr int LPR = 16, RPP = 256 / LPR, ROWS = RPP * VT_TILES;
    const bool tokpacked = v_layout == VQ_V_TOKEN_PACKED;
    const bool fused = D == 128 && (dtype == VQ_F16 || dtype == VQ_BF16) && (meta_dtype == VQ_F16 || meta_dtype == VQ_F32) &&
                       BH >= 1 && BH <= 65535 && S >= 1 && xs % 8 == 0 && xs >= S * D && aligned16(k) && aligned16(v) &&
                       aligned16(kp) && aligned16(ks) && aligned16(kz) && aligned16(vp) && aligned16(vs) && aligned16(vz) &&
                       (bits == 2 || bits == 4 || bits == 8) && levels >= 1 && levels <= (1 << bits) - 1 &&
                       group >= 8 && group <= KT_MAXP * RPP && group % 8 == 0 && pow2(group / 8) && D % group == 0 &&
                       (v_layout == VQ_V_CHANNEL_PACKED || (tokpacked && RPP % per == 0)) && tok0 >= 0 && tok0 + S <= cap &&
                       tok0 % group == 0 && (!tokpacked || (tok0 % per == 0 && S % per == 0 && cap % per == 0));
    if (!fused) {
        const int rc = vq_kivi_quant_pack(k, dtype, BH, S, D, xs, VQ_AXIS_TOKEN, group, levels, eps, bits, VQ_V_CHANNEL_PACKED,
                                          kp, ks, kz, meta_dtype, cap, tok0, stream);
        if (rc != VQ_OK) return rc;
        return vq_kivi_quant_pack(v, dtype, BH, S, D, xs, VQ_AXIS_CHANNEL, group, levels, eps, bits, v_layout, vp, vs, vz,
                                  meta_dtype, cap, tok0, stream);
    }
    const PackDst kd = {(uint32_t *)kp, ks, kz}, vd = {(uint32_t *)vp, vs, vz};
    hipStream_t st = (hipStream_t)stream;
    if (tokpacked && (group == 32 || group == 64) && (bits == 2 || bits == 4) && tok0 % 8 == 0 && cap % 8 == 0) {
        // group = 4 * TPL tokens for the keys = 8 * GL channels for the values: GL = TPL / 2
        const int kb = (int)cdiv(cdiv(S, group), KQ_WAVES), vb = (int)cdiv(S, VP_STRETCHES * per);
        const dim3 g2((unsigned)(kb + vb), (unsigned)BH);
#define VQ_KV2(T, M, BITS, TPL)                                                                                          \
        hipLaunchKernelGGL((kivi_kv_pack_kernel<T, M, BITS, TPL>), g2, dim3(256), 0, st, (const T *)k, (const T *)v, S, xs,  \
                           (float)levels, eps, kd, vd, cap, tok0, kb)
#define VQ_KV2_B(T, M)                                                                                                    \
        do {                                                                                                             \
            if (bits == 4) { if (group == 32) VQ_KV2(T, M, 4, 8); else VQ_KV2(T, M, 4, 16); }                            \
            else { if (group == 32) VQ_KV2(T, M, 2, 8); else VQ_KV2(T, M, 2, 16); }                                      \
        } while (0)
        if (dtype == VQ_F16) { if (meta_dtype == VQ_F16) VQ_KV2_B(f16, f16); else VQ_KV2_B(f16, float); }
        else { if (meta_dtype == VQ_F16) VQ_KV2_B(bf16_t, f16); else VQ_KV2_B(bf16_t, float); }
#undef VQ_KV2_B
#undef VQ_KV2
        VQ_HIP_CHECK_LAUNCH("vq_kivi_cache_append");
        return VQ_OK;
    }
    const int key_blocks = (int)cdiv(S, group), value_blocks = (int)cdiv(S, ROWS);
    const dim3 grid((unsigned)(key_blocks + value_blocks), (unsigned)BH);
    const int W = (int)cdiv(LPR * 8, per);
#define VQ_KV(T, M, NP, VM)                                                                                              \
    hipLaunchKernelGGL((kivi_kv_tile_kernel<T, M, LPR, NP, VM>), grid, dim3(256), 0, st, (const T *)k, (const T *)v, S, xs, \
                       group, (float)levels, eps, bits, kd, vd, cap, tok0, W, key_blocks)
#define VQ_KV_NP(T, M, VM)                                                                \
    do {                                                                                  \
        if (group <= (KT_MAXP / 2) * RPP) VQ_KV(T, M, KT_MAXP / 2, VM); else VQ_KV(T, M, KT_MAXP, VM); \
    } while (0)
#define VQ_KV_M(T, VM)                                                                    \
    do {                                                                                  \
        if (meta_dtype == VQ_F16) VQ_KV_NP(T, f16, VM); else VQ_KV_NP(T, float, VM);      \
    } while (0)
    if (dtype == VQ_F16) { if (tokpacked) VQ_KV_M(f16, 2); else VQ_KV_M(f16, 1); }
    else { if (tokpacked) VQ_KV_M(bf16_t, 2); else VQ_KV_M(bf16_t, 1); }
#undef VQ_KV_M
#undef VQ_KV_NP
#undef VQ_KV
    VQ_HIP_CHECK_LAUNCH("vq_kivi_cache_append");
    return VQ_OK;
}
}  // namespace vq

extern "C" int vq_row_norms(const void *x, int dtype, int64_t n_rows, int64_t D, float *out, void *stream) {
    const char *fn = "vq_row_norms";
    VQ_REQUIRE(n_rows >= 0 && D >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    if (n_rows * D == 0) return VQ_OK;
    VQ_REQUIRE(x && out, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE((D == 64 || D == 128 || D == 256) && aligned16(x), VQ_ERR_UNSUPPORTED,
               "%s: needs head_dim 64/128/256 and 16-byte aligned rows", fn);
    hipStream_t st = (hipStream_t)stream;
    int64_t blocks = cdiv(n_rows, 256 / (D / 8));
    if (blocks > 65536) blocks = 65536;
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (D == 64) hipLaunchKernelGGL((row_norm_kernel<T, 8>), dim3((unsigned)blocks), dim3(256), 0, st, (const T *)x, n_rows, out);
        else if (D == 128) hipLaunchKernelGGL((row_norm_kernel<T, 16>), dim3((unsigned)blocks), dim3(256), 0, st, (const T *)x, n_rows, out);
        else hipLaunchKernelGGL((row_norm_kernel<T, 32>), dim3((unsigned)blocks), dim3(256), 0, st, (const T *)x, n_rows, out);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_zip_route(const float *norms, int64_t BH, int64_t S, int64_t n_hi, int32_t *order, void *stream) {
    const char *fn = "vq_zip_route";
    VQ_REQUIRE(BH >= 0 && S >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(n_hi >= 1 && n_hi < S, VQ_ERR_INVALID, "%s: n_hi=%lld must be in [1, S) (one block needs no routing)", fn,
               (long long)n_hi);
    VQ_REQUIRE(S < ((int64_t)1 << 31) && BH <= 0x7fffffff, VQ_ERR_INVALID, "%s: positions must fit 31 bits", fn);
    if (BH == 0) return VQ_OK;
    VQ_REQUIRE(norms && order, VQ_ERR_INVALID, "%s: null pointer", fn);
    if (S <= 8 * ZR_THREADS)
        hipLaunchKernelGGL(zip_route_regs_kernel<8>, dim3((unsigned)BH), dim3(ZR_THREADS), 0, (hipStream_t)stream, norms, (int)S,
                           (int)n_hi, order);
    else if (S <= 32 * ZR_THREADS)
        hipLaunchKernelGGL(zip_route_regs_kernel<32>, dim3((unsigned)BH), dim3(ZR_THREADS), 0, (hipStream_t)stream, norms, (int)S,
                           (int)n_hi, order);
    else
        hipLaunchKernelGGL(zip_route_kernel, dim3((unsigned)BH), dim3(ZR_THREADS), 0, (hipStream_t)stream, norms, S, n_hi, order);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_kivi_quant_dequant_rows(const void *x, void *out, int dtype, int64_t BH, int64_t n_rows, int64_t D,
                                          int64_t stride_bh, const int32_t *rows, int64_t rows_stride, int group, int levels,
                                          float eps, void *stream) {
    const char *fn = "vq_kivi_quant_dequant_rows";
    VQ_REQUIRE(group >= 1 && levels >= 1, VQ_ERR_INVALID, "%s: group_size and levels must be >= 1", fn);
    VQ_REQUIRE(BH >= 0 && n_rows >= 0 && D >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    if (BH * n_rows * D == 0) return VQ_OK;
    VQ_REQUIRE(x && out && rows, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(rows_stride >= n_rows, VQ_ERR_INVALID, "%s: rows_stride %lld below n_rows %lld", fn, (long long)rows_stride,
               (long long)n_rows);
    VQ_REQUIRE((D == 64 || D == 128 || D == 256) && aligned16(x) && aligned16(out) && stride_bh % 8 == 0 && BH <= 65535 &&
                   group <= KT_MAXP * (256 / (int)(D / 8)),
               VQ_ERR_UNSUPPORTED, "%s: needs head_dim 64/128/256, 16-byte aligned slabs and a group the tile kernel holds", fn);
    hipStream_t st = (hipStream_t)stream;
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (D == 64) launch_key_tile<T, float, 8>(0, x, out, BH, n_rows, stride_bh, group, levels, eps, 0, nullptr, nullptr, nullptr, 0, 0, st, rows, rows_stride);
        else if (D == 128) launch_key_tile<T, float, 16>(0, x, out, BH, n_rows, stride_bh, group, levels, eps, 0, nullptr, nullptr, nullptr, 0, 0, st, rows, rows_stride);
        else launch_key_tile<T, float, 32>(0, x, out, BH, n_rows, stride_bh, group, levels, eps, 0, nullptr, nullptr, nullptr, 0, 0, st, rows, rows_stride);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_kivi_quant_pack_kv(const void *k, const void *v, int dtype, int64_t BH, int64_t S, int64_t D,
                                     int64_t x_stride_bh, int group, int levels, float eps, int pack_bits, int v_layout,
                                     void *k_packed, void *k_scale, void *k_zero, void *v_packed, void *v_scale,
                                     void *v_zero, int meta_dtype, int64_t cap_tokens, int64_t dst_tok0, void *stream) {
    // argument checks are those of the single calls; an invalid pair fails there
    return pack_kv_pair(k, v, dtype, BH, S, D, x_stride_bh, group, levels, eps, pack_bits, v_layout, k_packed, k_scale, k_zero,
                        v_packed, v_scale, v_zero, meta_dtype, cap_tokens, dst_tok0, stream);
}

extern "C" int vq_kivi_quant_dequant(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D, int axis,
                                     int group, int levels, float eps, void *stream) {
    VQ_REQUIRE(axis == VQ_AXIS_TOKEN || axis == VQ_AXIS_CHANNEL, VQ_ERR_INVALID,
               "vq_kivi_quant_dequant: axis must be -1 or -2 (VQ_AXIS_CHANNEL / VQ_AXIS_TOKEN), got %d", axis);
    VQ_REQUIRE(group >= 1, VQ_ERR_INVALID, "vq_kivi_quant_dequant: group_size must be >= 1, got %d", group);
    VQ_REQUIRE(levels >= 1, VQ_ERR_INVALID, "vq_kivi_quant_dequant: levels must be >= 1, got %d", levels);
    VQ_REQUIRE(BH >= 0 && S >= 0 && D >= 0, VQ_ERR_INVALID, "vq_kivi_quant_dequant: negative dimension");
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "vq_kivi_quant_dequant: unsupported dtype tag %d", dtype);
    if (BH * S * D == 0) return VQ_OK;
    VQ_REQUIRE(x && out, VQ_ERR_INVALID, "vq_kivi_quant_dequant: null pointer");
    hipStream_t st = (hipStream_t)stream;
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (!try_tile_path<T, float>(0, axis, x, out, BH, S, D, S * D, group, levels, eps, 0, nullptr, nullptr, nullptr,
                                     0, 0, st))
            hipLaunchKernelGGL((kivi_roundtrip_generic_kernel<T>), dim3(grid_for(BH * S * D, 256)), dim3(256), 0, st,
                               (const T *)x, (T *)out, BH, S, D, axis, group, (float)levels, eps);
    });
    VQ_HIP_CHECK_LAUNCH("vq_kivi_quant_dequant");
    return VQ_OK;
}

extern "C" int vq_kivi_quant_dequant_mixed(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D, int group,
                                           int levels_lo, int levels_hi, const uint8_t *hi_mask, float eps, void *stream) {
    const char *fn = "vq_kivi_quant_dequant_mixed";
    VQ_REQUIRE(D == 128 && (group == 32 || group == 64), VQ_ERR_UNSUPPORTED,
               "%s: head_dim 128 and groups of 32 or 64 tokens only (got head_dim %lld, group %d)", fn, (long long)D, group);
    VQ_REQUIRE(levels_lo >= 1 && levels_hi >= 1, VQ_ERR_INVALID, "%s: level counts must be >= 1, got %d and %d", fn, levels_lo, levels_hi);
    VQ_REQUIRE(BH >= 0 && S >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    if (BH * S == 0) return VQ_OK;
    VQ_REQUIRE(x && out && hi_mask, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(aligned16(x) && aligned16(out) && ((uintptr_t)hi_mask % 8) == 0, VQ_ERR_UNSUPPORTED,
               "%s: x and out must be 16-byte aligned, hi_mask 8-byte aligned", fn);
    VQ_REQUIRE(BH <= 65535, VQ_ERR_UNSUPPORTED, "%s: at most 65535 (sequence, head) pairs, got %lld", fn, (long long)BH);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)cdiv(cdiv(S, group), KQ_WAVES), (unsigned)BH);
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (group == 32)
            hipLaunchKernelGGL((kivi_key_quad_mixed_kernel<T, 8>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D,
                               (float)levels_lo, (float)levels_hi, hi_mask, eps);
        else
            hipLaunchKernelGGL((kivi_key_quad_mixed_kernel<T, 16>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D,
                               (float)levels_lo, (float)levels_hi, hi_mask, eps);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_kivi_quant_dequant_grouplevels(const void *x, void *out, int dtype, int64_t BH, int64_t S, int64_t D, int group,
                                                 const float *group_levels, float eps, void *stream) {
    const char *fn = "vq_kivi_quant_dequant_grouplevels";
    VQ_REQUIRE(D == 128 && (group == 32 || group == 64), VQ_ERR_UNSUPPORTED,
               "%s: head_dim 128 and groups of 32 or 64 tokens only (got head_dim %lld, group %d)", fn, (long long)D, group);
    VQ_REQUIRE(dtype == VQ_F16 || dtype == VQ_BF16, VQ_ERR_UNSUPPORTED, "%s: fp16 or bf16 rows only, got dtype tag %d", fn, dtype);
    VQ_REQUIRE(BH >= 0 && S >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    if (BH * S == 0) return VQ_OK;
    VQ_REQUIRE(x && out && group_levels, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(aligned16(x) && aligned16(out), VQ_ERR_UNSUPPORTED, "%s: x and out must be 16-byte aligned", fn);
    VQ_REQUIRE(BH <= 65535, VQ_ERR_UNSUPPORTED, "%s: at most 65535 (sequence, head) pairs, got %lld", fn, (long long)BH);
    hipStream_t st = (hipStream_t)stream;
    const dim3 grid((unsigned)cdiv(cdiv(S, group), KQ_WAVES), (unsigned)BH);
    if (dtype == VQ_F16) {
        using T = vq::f16;
        if (group == 32) hipLaunchKernelGGL((kivi_key_quad_grouplevels_kernel<T, 8>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D, group_levels, eps);
        else hipLaunchKernelGGL((kivi_key_quad_grouplevels_kernel<T, 16>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D, group_levels, eps);
    } else {
        using T = vq::bf16_t;
        if (group == 32) hipLaunchKernelGGL((kivi_key_quad_grouplevels_kernel<T, 8>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D, group_levels, eps);
        else hipLaunchKernelGGL((kivi_key_quad_grouplevels_kernel<T, 16>), grid, dim3(64 * KQ_WAVES), 0, st, (const T *)x, (T *)out, S, S * D, group_levels, eps);
    }
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_channel_moments(const void *x, int dtype, int64_t N, int64_t S, int64_t D, int64_t x_stride_n, double *partial,
                                  int chunks, void *stream) {
    const char *fn = "vq_channel_moments";
    VQ_REQUIRE(D == 64 || D == 128 || D == 256, VQ_ERR_UNSUPPORTED, "%s: head_dim 64, 128 or 256, got %lld", fn, (long long)D);
    VQ_REQUIRE(N >= 0 && S >= 0 && chunks >= 1 && chunks <= 65535, VQ_ERR_INVALID, "%s: bad dimensions", fn);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    if (N == 0) return VQ_OK;
    VQ_REQUIRE(x && partial, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(aligned16(x) && x_stride_n % 8 == 0 && x_stride_n >= S * D, VQ_ERR_UNSUPPORTED,
               "%s: rows must be 16-byte aligned and x_stride_n >= S * D", fn);
    VQ_REQUIRE(N <= 65535, VQ_ERR_UNSUPPORTED, "%s: at most 65535 slabs, got %lld", fn, (long long)N);
    hipStream_t st = (hipStream_t)stream;
    const int64_t per = cdiv(S > 0 ? S : 1, chunks);
    const dim3 grid((unsigned)chunks, (unsigned)N);
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (D == 64) hipLaunchKernelGGL((channel_moments_kernel<T, 8>), grid, dim3(256), 0, st, (const T *)x, S, x_stride_n, partial, per);
        else if (D == 128) hipLaunchKernelGGL((channel_moments_kernel<T, 16>), grid, dim3(256), 0, st, (const T *)x, S, x_stride_n, partial, per);
        else hipLaunchKernelGGL((channel_moments_kernel<T, 32>), grid, dim3(256), 0, st, (const T *)x, S, x_stride_n, partial, per);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_channel_variance(const double *partial, int64_t N, int chunks, int64_t D, int64_t S, float *variance,
                                   void *stream) {
    const char *fn = "vq_channel_variance";
    VQ_REQUIRE(N >= 0 && D >= 1 && D <= 65536 && chunks >= 1 && S >= 1, VQ_ERR_INVALID, "%s: bad dimensions", fn);
    if (N == 0) return VQ_OK;
    VQ_REQUIRE(partial && variance, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipLaunchKernelGGL(channel_variance_kernel, dim3((unsigned)cdiv(N * D, 256)), dim3(256), 0, (hipStream_t)stream, partial, N, chunks,
                       (int)D, (double)S, variance);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_channel_hi_mask(const float *variance, int64_t N, int64_t D, int64_t n_hi, uint8_t *mask, void *stream) {
    const char *fn = "vq_channel_hi_mask";
    VQ_REQUIRE(N >= 0 && N <= 0x7fffffff && D >= 1, VQ_ERR_INVALID, "%s: bad dimensions", fn);
    VQ_REQUIRE(D <= 1024, VQ_ERR_UNSUPPORTED, "%s: at most 1024 channels, got %lld", fn, (long long)D);
    VQ_REQUIRE(n_hi >= 0 && n_hi <= D, VQ_ERR_INVALID, "%s: n_hi=%lld outside [0, %lld]", fn, (long long)n_hi, (long long)D);
    if (N == 0) return VQ_OK;
    VQ_REQUIRE(variance && mask, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipLaunchKernelGGL(channel_hi_mask_kernel, dim3((unsigned)N), dim3((unsigned)D), (size_t)D * sizeof(uint32_t), (hipStream_t)stream,
                       variance, (int)D, (int)n_hi, mask);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_kivi_quant_pack(const void *x, int dtype, int64_t BH, int64_t S, int64_t D, int64_t x_stride_bh,
                                  int axis, int group, int levels, float eps, int pack_bits, int v_layout,
                                  void *packed, void *scale, void *zero, int meta_dtype, int64_t cap_tokens,
                                  int64_t dst_tok0, void *stream) {
    const char *fn = "vq_kivi_quant_pack";
    VQ_REQUIRE(axis == VQ_AXIS_TOKEN || axis == VQ_AXIS_CHANNEL, VQ_ERR_INVALID, "%s: bad axis %d", fn, axis);
    VQ_REQUIRE(group >= 1, VQ_ERR_INVALID, "%s: group_size must be >= 1, got %d", fn, group);
    VQ_REQUIRE(pack_bits >= 1 && pack_bits <= 8, VQ_ERR_INVALID, "%s: pack_bits must be in 1..8, got %d", fn, pack_bits);
    VQ_REQUIRE(levels >= 1 && levels <= (1 << pack_bits) - 1, VQ_ERR_INVALID,
               "%s: levels=%d does not fit pack_bits=%d", fn, levels, pack_bits);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    VQ_REQUIRE(meta_dtype == VQ_F32 || meta_dtype == VQ_F16, VQ_ERR_INVALID, "%s: meta dtype must be f32 or f16", fn);
    VQ_REQUIRE(BH >= 0 && S >= 0 && D >= 1, VQ_ERR_INVALID, "%s: bad dimensions", fn);
    VQ_REQUIRE(dst_tok0 >= 0 && dst_tok0 + S <= cap_tokens, VQ_ERR_INVALID,
               "%s: tokens [%lld, %lld) exceed capacity %lld", fn, (long long)dst_tok0, (long long)(dst_tok0 + S),
               (long long)cap_tokens);
    VQ_REQUIRE(x_stride_bh >= S * D, VQ_ERR_INVALID, "%s: x_stride_bh too small", fn);
    const bool tokpacked = axis == VQ_AXIS_CHANNEL && v_layout == VQ_V_TOKEN_PACKED;
    VQ_REQUIRE(v_layout == VQ_V_CHANNEL_PACKED || v_layout == VQ_V_TOKEN_PACKED, VQ_ERR_INVALID, "%s: bad v_layout", fn);
    const int per = 32 / pack_bits;
    if (axis == VQ_AXIS_TOKEN)
        VQ_REQUIRE(dst_tok0 % group == 0, VQ_ERR_INVALID, "%s: key blocks must start on a group boundary", fn);
    if (tokpacked)
        VQ_REQUIRE(dst_tok0 % per == 0 && S % per == 0 && cap_tokens % per == 0, VQ_ERR_INVALID,
                   "%s: token-packed values need dst_tok0, S and cap_tokens to be multiples of %d", fn, per);
    if (BH * S == 0) return VQ_OK;
    VQ_REQUIRE(x && packed && scale && zero, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipStream_t st = (hipStream_t)stream;
    const int mode = tokpacked ? 2 : 1;
    const int64_t n_words = tokpacked ? BH * (S / per) * D : BH * S * cdiv(D, per);
#define VQ_PACK(T, M)                                                                                              \
    if (!try_tile_path<T, M>(mode, axis, x, nullptr, BH, S, D, x_stride_bh, group, levels, eps, pack_bits, packed,  \
                             scale, zero, cap_tokens, dst_tok0, st))                                              \
        hipLaunchKernelGGL((kivi_pack_generic_kernel<T, M>), dim3(grid_for(n_words, 128)), dim3(128), 0, st,      \
                           (const T *)x, BH, S, D, x_stride_bh, axis, group, (float)levels, eps, pack_bits,       \
                           tokpacked ? 1 : 0, (uint32_t *)packed, (M *)scale, (M *)zero, cap_tokens, dst_tok0)
    VQ_DISPATCH_FLOAT(dtype, T, {
        if (meta_dtype == VQ_F32) { VQ_PACK(T, float); } else { VQ_PACK(T, f16); }
    });
#undef VQ_PACK
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_kivi_dequant(const void *packed, const void *scale, const void *zero, int meta_dtype, int64_t BH,
                               int64_t S, int64_t D, int axis, int group, int pack_bits, int v_layout,
                               int64_t cap_tokens, int64_t src_tok0, void *out, int out_dtype, void *stream) {
    const char *fn = "vq_kivi_dequant";
    VQ_REQUIRE(axis == VQ_AXIS_TOKEN || axis == VQ_AXIS_CHANNEL, VQ_ERR_INVALID, "%s: bad axis %d", fn, axis);
    VQ_REQUIRE(group >= 1, VQ_ERR_INVALID, "%s: group_size must be >= 1", fn);
    VQ_REQUIRE(pack_bits >= 1 && pack_bits <= 8, VQ_ERR_INVALID, "%s: pack_bits must be in 1..8", fn);
    VQ_REQUIRE(meta_dtype == VQ_F32 || meta_dtype == VQ_F16, VQ_ERR_INVALID, "%s: meta dtype must be f32 or f16", fn);
    VQ_REQUIRE(is_float_tag(out_dtype), VQ_ERR_INVALID, "%s: unsupported out dtype", fn);
    VQ_REQUIRE(src_tok0 >= 0 && src_tok0 + S <= cap_tokens, VQ_ERR_INVALID, "%s: token range exceeds capacity", fn);
    const bool tokpacked = axis == VQ_AXIS_CHANNEL && v_layout == VQ_V_TOKEN_PACKED;
    if (tokpacked) VQ_REQUIRE(cap_tokens % (32 / pack_bits) == 0, VQ_ERR_INVALID, "%s: capacity not word aligned", fn);
    if (BH * S * D == 0) return VQ_OK;
    VQ_REQUIRE(packed && scale && zero && out, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipStream_t st = (hipStream_t)stream;
    const int pb = pack_bits == 2 ? 1 : pack_bits == 4 ? 2 : pack_bits == 8 ? 3 : -1;
    if (pb > 0 && D % 8 == 0 && D % group == 0 && group % 8 == 0 && D <= (1 << 20) && aligned16(packed) && aligned16(scale) &&
        aligned16(zero) && aligned16(out) && BH * S * (D / 8) < ((int64_t)1 << 40)) {
        // eight channels a thread (channel-packed words hold 4, 8 or 16 codes: D % 8 == 0 keeps a thread inside its words)
        const int64_t n_rows = BH * S;
        const dim3 g8((unsigned)cdiv(n_rows * (D / 8), 256));
#define VQ_DQ8(O, M, PB) hipLaunchKernelGGL((kivi_dequant8_kernel<O, M, PB>), g8, dim3(256), 0, st, (const uint32_t *)packed,        \
                                            (const M *)scale, (const M *)zero, n_rows, S, (int)D, axis, group, tokpacked ? 1 : 0,   \
                                            cap_tokens, src_tok0, (O *)out)
        VQ_DISPATCH_FLOAT(out_dtype, O, {
            if (meta_dtype == VQ_F32) { if (pb == 1) VQ_DQ8(O, float, 1); else if (pb == 2) VQ_DQ8(O, float, 2); else VQ_DQ8(O, float, 3); }
            else { if (pb == 1) VQ_DQ8(O, f16, 1); else if (pb == 2) VQ_DQ8(O, f16, 2); else VQ_DQ8(O, f16, 3); }
        });
#undef VQ_DQ8
        VQ_HIP_CHECK_LAUNCH(fn);
        return VQ_OK;
    }
    dim3 grid(grid_for(BH * S * D, 256));
    VQ_DISPATCH_FLOAT(out_dtype, O, {
        if (meta_dtype == VQ_F32)
            hipLaunchKernelGGL((kivi_dequant_kernel<O, float>), grid, dim3(256), 0, st, (const uint32_t *)packed,
                               (const float *)scale, (const float *)zero, BH, S, D, axis, group, pack_bits,
                               tokpacked ? 1 : 0, cap_tokens, src_tok0, (O *)out);
        else
            hipLaunchKernelGGL((kivi_dequant_kernel<O, f16>), grid, dim3(256), 0, st, (const uint32_t *)packed,
                               (const f16 *)scale, (const f16 *)zero, BH, S, D, axis, group, pack_bits,
                               tokpacked ? 1 : 0, cap_tokens, src_tok0, (O *)out);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_pack_words(const uint8_t *idx, int64_t rows, int64_t D, int bits, uint32_t *words, void *stream) {
    VQ_REQUIRE(bits >= 1 && bits <= 8, VQ_ERR_INVALID, "vq_pack_words: bits must be in 1..8, got %d", bits);
    VQ_REQUIRE(rows >= 0 && D >= 0, VQ_ERR_INVALID, "vq_pack_words: negative dimension");
    if (rows * D == 0) return VQ_OK;
    VQ_REQUIRE(idx && words, VQ_ERR_INVALID, "vq_pack_words: null pointer");
    hipLaunchKernelGGL(pack_words_kernel, dim3(grid_for(rows * cdiv(D, 32 / bits), 256)), dim3(256), 0,
                       (hipStream_t)stream, idx, rows, D, bits, words);
    VQ_HIP_CHECK_LAUNCH("vq_pack_words");
    return VQ_OK;
}
extern "C" int vq_unpack_words(const uint32_t *words, int64_t rows, int64_t D, int bits, uint8_t *idx, void *stream) {
    VQ_REQUIRE(bits >= 1 && bits <= 8, VQ_ERR_INVALID, "vq_unpack_words: bits must be in 1..8, got %d", bits);
    VQ_REQUIRE(rows >= 0 && D >= 0, VQ_ERR_INVALID, "vq_unpack_words: negative dimension");
    if (rows * D == 0) return VQ_OK;
    VQ_REQUIRE(idx && words, VQ_ERR_INVALID, "vq_unpack_words: null pointer");
    hipLaunchKernelGGL(unpack_words_kernel, dim3(grid_for(rows * D, 256)), dim3(256), 0, (hipStream_t)stream, words,
                       rows, D, bits, idx);
    VQ_HIP_CHECK_LAUNCH("vq_unpack_words");
    return VQ_OK;
}
extern "C" int vq_bit_pack(const uint8_t *idx, int64_t n, int bits, uint8_t *packed, void *stream) {
    VQ_REQUIRE(bits == 1 || bits == 2 || bits == 4, VQ_ERR_INVALID, "vq_bit_pack: bits must be 1, 2 or 4, got %d", bits);
    VQ_REQUIRE(n >= 0 && n % (8 / bits) == 0, VQ_ERR_INVALID,
               "vq_bit_pack: length %lld is not a multiple of %d", (long long)n, 8 / bits);
    if (n == 0) return VQ_OK;
    VQ_REQUIRE(idx && packed, VQ_ERR_INVALID, "vq_bit_pack: null pointer");
    hipLaunchKernelGGL(bit_pack_kernel, dim3(grid_for(n / (8 / bits), 256)), dim3(256), 0, (hipStream_t)stream, idx,
                       n / (8 / bits), bits, packed);
    VQ_HIP_CHECK_LAUNCH("vq_bit_pack");
    return VQ_OK;
}
extern "C" int vq_bit_unpack(const uint8_t *packed, int64_t n, int bits, uint8_t *idx, void *stream) {
    VQ_REQUIRE(bits == 1 || bits == 2 || bits == 4, VQ_ERR_INVALID, "vq_bit_unpack: bits must be 1, 2 or 4, got %d", bits);
    VQ_REQUIRE(n >= 0, VQ_ERR_INVALID, "vq_bit_unpack: negative length");
    if (n == 0) return VQ_OK;
    VQ_REQUIRE(idx && packed, VQ_ERR_INVALID, "vq_bit_unpack: null pointer");
    hipLaunchKernelGGL(bit_unpack_kernel, dim3(grid_for(n, 256)), dim3(256), 0, (hipStream_t)stream, packed, n, bits, idx);
    VQ_HIP_CHECK_LAUNCH("vq_bit_unpack");
    return VQ_OK;
}
