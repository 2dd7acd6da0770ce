// SKVQ clipped group quantisation round trip for gfx950.
//
// Per token row and per group of `group` consecutive (optionally permuted) channels
// (veloxquant_mlx/quantizers/skvq.py:105-183, float32, one rounding per operation):
//   mid = (gmax + gmin) * 0.5,  rng = gmax - gmin
//   for every clip factor a:  lo = mid - (a * rng) * 0.5,  scale = max((a * rng) / levels, 1e-8)
//                             code = clamp(rint((x - lo) / scale), 0, levels),  xhat = code * scale + lo
//                             err  = sum((xhat - x)^2) / group        (summed left to right)
//   the first a with the smallest err wins; out = cast(xhat of that a).
// A ragged last group is padded with the row's last (permuted) channel, as the reference pads.
// With a permutation, group j of a row of head h holds channels perm[h][j*group .. ], and the
// result goes back to the channels it came from (the inverse gather of
// veloxquant_mlx/cache/skvq_cache.py:236-251).
//
// One thread owns one group.  A block first stages its rows in LDS as float32 (stride group + 1
// words between groups, so the threads of a wave walk different banks), then every thread scans
// its group once per clip factor (held in registers for groups of 32 and 64, out of LDS otherwise),
// overwrites it with the winning reconstruction, and the block writes the rows back.  Staging completes before the first store, so out may alias x.
#include "common.hpp"

namespace vq {

constexpr int SK_THREADS = 256;
constexpr int SK_MAX_ALPHAS = 8;

struct SkAlphas { float a[SK_MAX_ALPHAS]; int n; };

// clamp(rint((x - lo) / sc), 0, levels) without an IEEE division on the common path.  t = x - lo is
// rounded once, as in the reference; q0 = t * rcp(sc) lies within 2.5 ulp (1.5e-7 relative) of the
// correctly rounded quotient, so rint(q0) is the reference's code unless q0 sits that close to a tie
// k + 0.5 -- a lane within 1e-6 * (|q0| + 1) of one takes the true division instead.
__device__ __forceinline__ float sk_code(float x, float lo, float sc, float rs, float levels) {
    const float t = __fsub_rn(x, lo);
    const float q0 = __fmul_rn(t, rs);
    float r = rintf(q0);
    if (fabsf(q0 - r) >= 0.5f - 1e-6f * (fabsf(q0) + 1.0f)) r = rintf(__fdiv_rn(t, sc));
    return fminf(fmaxf(r, 0.f), levels);
}

// Eight codes at a time with one tie limit for the whole call and one branch: when any lane of the wave
// has any of its eight q0 within `tie` of a half, all eight are formed again by true division (rare, and
// the same value wherever q0 was not close).  Outside |q0| <= levels + 1 the clamp decides whatever the
// rounding does; inside it q0 is within 1.5e-7 * (levels + 1) of the true quotient, less than the
// 1e-6 * (levels + 2) by which `tie` stays below one half.
__device__ __forceinline__ void sk_codes8(const float *x, float (&q)[8], float lo, float sc, float rs, float levels, float tie) {
    float far = 0.f, dist[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        const float q0 = __fmul_rn(__fsub_rn(x[j], lo), rs);
        q[j] = rintf(q0);
        dist[j] = fabsf(q0 - q[j]);
        far = fmaxf(far, dist[j]);
    }
    if (__builtin_amdgcn_ballot_w64(far >= tie) != 0) {   // exact ties are common with 16-bit inputs: only the codes some lane is unsure of
#pragma unroll
        for (int j = 0; j < 8; ++j)
            if (__builtin_amdgcn_ballot_w64(dist[j] >= tie) != 0) q[j] = rintf(__fdiv_rn(__fsub_rn(x[j], lo), sc));
    }
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = __builtin_amdgcn_fmed3f(q[j], 0.f, levels);   // a NaN becomes 0, as with fmaxf / fminf
}

// eight consecutive elements as one (16-bit types) or two (float32) 16-byte accesses
template <typename T> struct Vec8 {
    static __device__ __forceinline__ void ld(const T *p, float (&v)[8]) {
        if constexpr (sizeof(T) == 4) {
            const float4 a = *reinterpret_cast<const float4 *>(p), b = *reinterpret_cast<const float4 *>(p + 4);
            v[0] = a.x; v[1] = a.y; v[2] = a.z; v[3] = a.w; v[4] = b.x; v[5] = b.y; v[6] = b.z; v[7] = b.w;
        } else {
            union { uint4 u; T e[8]; } w;
            w.u = *reinterpret_cast<const uint4 *>(p);
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = Elem<T>::ld(&w.e[k]);
        }
    }
    static __device__ __forceinline__ void st(T *p, const float (&v)[8]) {
        if constexpr (sizeof(T) == 4) {
            *reinterpret_cast<float4 *>(p) = make_float4(v[0], v[1], v[2], v[3]);
            *reinterpret_cast<float4 *>(p + 4) = make_float4(v[4], v[5], v[6], v[7]);
        } else {
            union { uint4 u; T e[8]; } w;
#pragma unroll
            for (int k = 0; k < 8; ++k) Elem<T>::st(&w.e[k], v[k]);
            *reinterpret_cast<uint4 *>(p) = w.u;
        }
    }
};

template <typename T, int GROUP>   // GROUP > 0: the group size, known at compile time; 0: any
__global__ __launch_bounds__(SK_THREADS)
void skvq_roundtrip_kernel(const T *__restrict__ x, T *out, int64_t n_bh, int64_t H, int64_t r, int64_t D,
                           int64_t x_stride_bh, int64_t out_stride_bh, const int32_t *__restrict__ perm, const int32_t *__restrict__ inv,
                           int group, uint64_t group_magic, int G, int rows_pb, int tpr, bool vec, float levels, SkAlphas al) {
    extern __shared__ float s_x[];
    const int tid = threadIdx.x;
    const int gstride = group + 1, Dp = G * group;
    const int64_t row0 = (int64_t)blockIdx.x * rows_pb, n_rows = n_bh * r;   // n_rows < 2^31 (checked by the caller)

    // A thread moves pieces of eight consecutive channels: tpr threads side by side cover a row, the
    // block covers rpp rows per pass.  Rows that can move as 16-byte pieces (`vec`) do so; under a
    // channel order this needs the inverse order (channel -> place), which turns the gather into a
    // scatter inside LDS.  Without it, or with an odd head_dim, a piece is eight single-channel accesses
    // (gathers within the row's cache lines).
    // (Passing permuted rows through a second LDS image, to keep global accesses vectorised, measured
    // slower than these gathers: 0.92 ms against 0.79 ms on 16 x 8 x 8192 rows of 128 channels.)
    //
    // Where a row is one piece per thread (tpr * 8 >= Dp) a thread meets the same eight channels in every
    // row, so their LDS words -- a division by the group size and, under an order, a table look-up each --
    // are worked out once per head, not once per element; (sequence, head) and token of a row follow from
    // those of the block's first row by counting, not by dividing.
    const int lr_base = tid / tpr, cq = tid - lr_base * tpr, rpp = (int)blockDim.x / tpr;
    auto pos = [&](int j) {                        // LDS word of (permuted) channel j within a row
        if constexpr (GROUP > 0) return j + j / GROUP;
        const int gi = (int)(((uint64_t)(uint32_t)j * group_magic) >> 32);   // j / group
        return gi * gstride + (j - gi * group);
    };
    const bool scatter = vec && inv, one_piece = tpr * 8 >= Dp;
    const uint32_t bh_first = (uint32_t)row0 / (uint32_t)r, t_first = (uint32_t)row0 - bh_first * (uint32_t)r;
    const uint32_t head_first = bh_first % (uint32_t)H;
    struct Where { uint32_t bh, t, head; };
    auto where = [&](int lr) {                     // rows_pb rows span few (sequence, head) pairs
        Where w{bh_first, t_first + (uint32_t)lr, head_first};
        while (w.t >= (uint32_t)r) { w.t -= (uint32_t)r; ++w.bh; w.head = w.head + 1 == (uint32_t)H ? 0u : w.head + 1; }
        return w;
    };
    int off[8], fill_k = -1;
    uint32_t off_head = ~0u;
    auto place = [&](uint32_t head, int c0) {      // LDS words of channels (or places) c0 .. c0 + 7 of a row of `head`
        if (one_piece && head == off_head) return;
        off_head = head;
        fill_k = -1;
        const int32_t *iv = scatter ? inv + (int64_t)head * D : nullptr;
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const int c = c0 + k, j = (iv && c < (int)D) ? iv[c] : c;
            off[k] = pos(j);
            if (iv && j == (int)D - 1 && Dp > (int)D) fill_k = k;   // the order's last channel also fills a ragged last group
        }
    };
    for (int lr = lr_base; lr < rows_pb && lr_base < rpp; lr += rpp) {
        if (row0 + lr >= n_rows) continue;
        const Where w = where(lr);
        const T *src = x + (int64_t)w.bh * x_stride_bh + (int64_t)w.t * D;
        const int32_t *pm = perm ? perm + (int64_t)w.head * D : nullptr;
        float *dst = s_x + lr * G * gstride;
        for (int c0 = cq * 8; c0 < Dp; c0 += tpr * 8) {
            float v[8];
            place(w.head, c0);
            if (scatter) {      // stored-order piece, every channel dropped at its place in the head's order
                if (c0 < D) {
                    Vec8<T>::ld(src + c0, v);
#pragma unroll
                    for (int k = 0; k < 8; ++k) {
                        dst[off[k]] = v[k];
                        if (k == fill_k)
                            for (int jp = (int)D; jp < Dp; ++jp) dst[pos(jp)] = v[k];
                    }
                }
                continue;
            }
            if (vec && c0 < D) {
                Vec8<T>::ld(src + c0, v);
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int j = c0 + k, c = j < D ? j : (int)D - 1;
                    v[k] = Elem<T>::ld(src + (pm ? pm[c] : c));
                }
            }
#pragma unroll
            for (int k = 0; k < 8; ++k)
                if (c0 + k < Dp) dst[off[k]] = v[k];
        }
    }
    __syncthreads();

    if (tid < rows_pb * G && row0 + tid / G < n_rows) {
        float *p = s_x + tid * gstride;
        if constexpr (GROUP > 0) {
            // the group in registers: LDS is read once and written once, and the clip search runs
            // as straight-line code over GROUP values per factor
            float xv[GROUP];
#pragma unroll
            for (int j = 0; j < GROUP; ++j) xv[j] = p[j];
            float mn = xv[0], mx = xv[0];
#pragma unroll
            for (int j = 1; j < GROUP; ++j) { mn = fminf(mn, xv[j]); mx = fmaxf(mx, xv[j]); }
            const float mid = __fmul_rn(__fadd_rn(mx, mn), 0.5f), rng = __fsub_rn(mx, mn);
            const float tie = 0.5f - 1e-6f * (levels + 2.0f);
            float best_err = 0.f, best_lo = 0.f, best_sc = 1.f;
            for (int k = 0; k < al.n; ++k) {
                const float ar = __fmul_rn(al.a[k], rng);
                const float lo = __fsub_rn(mid, __fmul_rn(ar, 0.5f));
                const float sc = fmaxf(__fdiv_rn(ar, levels), 1e-8f);
                const float rs = __builtin_amdgcn_rcpf(sc);
                float sum = 0.f;
#pragma unroll
                for (int j0 = 0; j0 < GROUP; j0 += 8) {
                    float q[8];
                    sk_codes8(xv + j0, q, lo, sc, rs, levels, tie);
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const float d = __fsub_rn(__fadd_rn(__fmul_rn(q[j], sc), lo), xv[j0 + j]);
                        sum = __fadd_rn(sum, __fmul_rn(d, d));
                    }
                }
                const float err = __fdiv_rn(sum, (float)GROUP);
                if (k == 0 || err < best_err) { best_err = err; best_lo = lo; best_sc = sc; }
            }
            const float best_rs = __builtin_amdgcn_rcpf(best_sc);
#pragma unroll
            for (int j0 = 0; j0 < GROUP; j0 += 8) {
                float q[8];
                sk_codes8(xv + j0, q, best_lo, best_sc, best_rs, levels, tie);
#pragma unroll
                for (int j = 0; j < 8; ++j) p[j0 + j] = __fadd_rn(__fmul_rn(q[j], best_sc), best_lo);
            }
        } else {
        float mn = p[0], mx = p[0];
        for (int j = 1; j < group; ++j) { mn = fminf(mn, p[j]); mx = fmaxf(mx, p[j]); }
        const float mid = __fmul_rn(__fadd_rn(mx, mn), 0.5f), rng = __fsub_rn(mx, mn);
        float best_err = 0.f, best_lo = 0.f, best_sc = 1.f;
        for (int k = 0; k < al.n; ++k) {
            const float ar = __fmul_rn(al.a[k], rng);
            const float lo = __fsub_rn(mid, __fmul_rn(ar, 0.5f));
            const float sc = fmaxf(__fdiv_rn(ar, levels), 1e-8f);
            const float rs = __builtin_amdgcn_rcpf(sc);
            float sum = 0.f;
            for (int j = 0; j < group; ++j) {
                const float q = sk_code(p[j], lo, sc, rs, levels);
                const float d = __fsub_rn(__fadd_rn(__fmul_rn(q, sc), lo), p[j]);
                sum = __fadd_rn(sum, __fmul_rn(d, d));
            }
            const float err = __fdiv_rn(sum, (float)group);
            if (k == 0 || err < best_err) { best_err = err; best_lo = lo; best_sc = sc; }
        }
        const float best_rs = __builtin_amdgcn_rcpf(best_sc);
        for (int j = 0; j < group; ++j) {
            const float q = sk_code(p[j], best_lo, best_sc, best_rs, levels);
            p[j] = __fadd_rn(__fmul_rn(q, best_sc), best_lo);
        }
        }
    }
    __syncthreads();

    for (int lr = lr_base; lr < rows_pb && lr_base < rpp; lr += rpp) {
        if (row0 + lr >= n_rows) continue;
        const Where w = where(lr);
        T *dst = out + (int64_t)w.bh * out_stride_bh + (int64_t)w.t * D;
        const int32_t *pm = perm ? perm + (int64_t)w.head * D : nullptr;
        const float *srcl = s_x + lr * G * gstride;
        for (int c0 = cq * 8; c0 < (int)D; c0 += tpr * 8) {
            float v[8];
            place(w.head, c0);
#pragma unroll
            for (int k = 0; k < 8; ++k) v[k] = c0 + k < (int)D ? srcl[off[k]] : 0.f;
            if (vec) {
                Vec8<T>::st(dst + c0, v);
            } else {
#pragma unroll
                for (int k = 0; k < 8; ++k)
                    if (c0 + k < (int)D) Elem<T>::st(dst + (pm ? pm[c0 + k] : c0 + k), v[k]);
            }
        }
    }
}

}  // namespace vq

using namespace vq;

extern "C" int vq_skvq_clipped_roundtrip(const void *x, void *out, int dtype, int64_t B, int64_t H, int64_t r,
                                         int64_t D, int64_t x_stride_bh, int64_t out_stride_bh, const int32_t *perm,
                                         const int32_t *inv, int bits, int group, const float *alphas, int n_alphas, void *stream) {
    const char *fn = "vq_skvq_clipped_roundtrip";
    VQ_REQUIRE(bits >= 1 && bits <= 8, VQ_ERR_INVALID, "%s: bits must be in [1, 8], got %d", fn, bits);
    VQ_REQUIRE(group >= 1, VQ_ERR_INVALID, "%s: group_size must be >= 1, got %d", fn, group);
    VQ_REQUIRE(alphas && n_alphas >= 1 && n_alphas <= SK_MAX_ALPHAS, VQ_ERR_INVALID,
               "%s: between 1 and %d clip factors, got %d", fn, SK_MAX_ALPHAS, n_alphas);
    for (int k = 0; k < n_alphas; ++k)
        VQ_REQUIRE(alphas[k] > 0.f && alphas[k] <= 1.f, VQ_ERR_INVALID, "%s: alphas must lie in (0, 1], got %g", fn,
                   (double)alphas[k]);
    VQ_REQUIRE(B >= 0 && H >= 0 && r >= 0 && D >= 0, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(is_float_tag(dtype), VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn, dtype);
    if (B * H * r * D == 0) return VQ_OK;
    VQ_REQUIRE(x && out, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(x_stride_bh >= r * D && out_stride_bh >= r * D, VQ_ERR_INVALID, "%s: stride below r * D", fn);
    const int64_t G = (D + group - 1) / group;
    const int64_t row_words = G * (group + 1);
    VQ_REQUIRE(G <= SK_THREADS && row_words * 4 <= 48 * 1024 && group < 65536, VQ_ERR_UNSUPPORTED,
               "%s: head_dim %lld with group %d does not fit a block (at most %d groups, 48 KB per row)", fn,
               (long long)D, group, SK_THREADS);
    // one wave per block where a wave covers whole rows: blocks then interleave freely on a CU (the
    // phases of a block do not overlap each other, those of different blocks do)
    const int threads = (G <= 64 && (G * group + 7) / 8 <= 64) ? 64 : SK_THREADS;
    int64_t rows_pb = threads / G;
    if (rows_pb * row_words * 4 > 48 * 1024) rows_pb = 48 * 1024 / (row_words * 4);
    const int64_t n_rows = B * H * r, blocks = (n_rows + rows_pb - 1) / rows_pb;
    VQ_REQUIRE(n_rows <= 0x7fffffff, VQ_ERR_UNSUPPORTED, "%s: too many rows (%lld)", fn, (long long)n_rows);
    // floor(j / group) == (j * magic) >> 32 for j, group < 2^16 (a row holds at most 12288 words in LDS)
    const uint64_t group_magic = (1ull << 32) / (uint64_t)group + 1;
    // threads side by side on a row (eight channels each), and whether rows can move as 16-byte pieces
    const int64_t pieces = (G * group + 7) / 8;
    const int tpr = (int)(pieces < threads ? pieces : threads);
    VQ_REQUIRE(perm || !inv, VQ_ERR_INVALID, "%s: inv given without perm", fn);
    const bool vec = (perm == nullptr || inv != nullptr) && D % 8 == 0 && x_stride_bh % 8 == 0 && out_stride_bh % 8 == 0 &&
                     ((uintptr_t)x % 16 == 0) && ((uintptr_t)out % 16 == 0);
    SkAlphas al;
    al.n = n_alphas;
    for (int k = 0; k < SK_MAX_ALPHAS; ++k) al.a[k] = k < n_alphas ? alphas[k] : 1.f;
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = (size_t)(rows_pb * row_words * 4);
#define VQ_SK_LAUNCH(GROUP)                                                                                              \
    VQ_DISPATCH_FLOAT(dtype, T, {                                                                                      \
        hipLaunchKernelGGL((skvq_roundtrip_kernel<T, GROUP>), dim3((unsigned)blocks), dim3(threads), lds, st,          \
                           (const T *)x, (T *)out, B * H, H, r, D, x_stride_bh, out_stride_bh, perm, inv, group,       \
                           group_magic, (int)G, (int)rows_pb, tpr, vec, (float)((1 << bits) - 1), al);                 \
    })
    if (group == 32) { VQ_SK_LAUNCH(32); }
    else if (group == 64) { VQ_SK_LAUNCH(64); }
    else { VQ_SK_LAUNCH(0); }
#undef VQ_SK_LAUNCH
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}
