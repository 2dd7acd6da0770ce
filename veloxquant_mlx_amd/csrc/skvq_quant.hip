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
// its group once per clip factor, overwrites it with the winning reconstruction, and the block
// writes the rows back.  Staging completes before the first store, so out may alias x.
#include "common.hpp"

namespace vq {

constexpr int SK_THREADS = 256;
constexpr int SK_MAX_ALPHAS = 8;

struct SkAlphas { float a[SK_MAX_ALPHAS]; int n; };

template <typename T>
__global__ __launch_bounds__(SK_THREADS)
void skvq_roundtrip_kernel(const T *__restrict__ x, T *out, int64_t n_bh, int64_t H, int64_t r, int64_t D,
                           int64_t x_stride_bh, int64_t out_stride_bh, const int32_t *__restrict__ perm,
                           int group, int G, int rows_pb, float levels, SkAlphas al) {
    extern __shared__ float s_x[];
    const int tid = threadIdx.x;
    const int gstride = group + 1, Dp = G * group;
    const int64_t row0 = (int64_t)blockIdx.x * rows_pb, n_rows = n_bh * r;

    for (int e = tid; e < rows_pb * Dp; e += SK_THREADS) {
        const int lr = e / Dp, j = e % Dp;
        const int64_t row = row0 + lr;
        if (row >= n_rows) break;
        const int64_t bh = row / r, t = row % r;
        const int c = j < D ? j : (int)D - 1;
        const int src = perm ? perm[(bh % H) * D + c] : c;
        s_x[(lr * G + j / group) * gstride + j % group] = Elem<T>::ld(x + bh * x_stride_bh + t * D + src);
    }
    __syncthreads();

    if (tid < rows_pb * G && row0 + tid / G < n_rows) {
        float *p = s_x + tid * gstride;
        float mn = p[0], mx = p[0];
        for (int j = 1; j < group; ++j) { mn = fminf(mn, p[j]); mx = fmaxf(mx, p[j]); }
        const float mid = __fmul_rn(__fadd_rn(mx, mn), 0.5f), rng = __fsub_rn(mx, mn);
        float best_err = 0.f, best_lo = 0.f, best_sc = 1.f;
        for (int k = 0; k < al.n; ++k) {
            const float ar = __fmul_rn(al.a[k], rng);
            const float lo = __fsub_rn(mid, __fmul_rn(ar, 0.5f));
            const float sc = fmaxf(__fdiv_rn(ar, levels), 1e-8f);
            float sum = 0.f;
            for (int j = 0; j < group; ++j) {
                const float q = fminf(fmaxf(rintf(__fdiv_rn(__fsub_rn(p[j], lo), sc)), 0.f), levels);
                const float d = __fsub_rn(__fadd_rn(__fmul_rn(q, sc), lo), p[j]);
                sum = __fadd_rn(sum, __fmul_rn(d, d));
            }
            const float err = __fdiv_rn(sum, (float)group);
            if (k == 0 || err < best_err) { best_err = err; best_lo = lo; best_sc = sc; }
        }
        for (int j = 0; j < group; ++j) {
            const float q = fminf(fmaxf(rintf(__fdiv_rn(__fsub_rn(p[j], best_lo), best_sc)), 0.f), levels);
            p[j] = __fadd_rn(__fmul_rn(q, best_sc), best_lo);
        }
    }
    __syncthreads();

    for (int e = tid; e < rows_pb * (int)D; e += SK_THREADS) {
        const int lr = e / (int)D, j = e % (int)D;
        const int64_t row = row0 + lr;
        if (row >= n_rows) break;
        const int64_t bh = row / r, t = row % r;
        const int dst = perm ? perm[(bh % H) * D + j] : j;
        Elem<T>::st(out + bh * out_stride_bh + t * D + dst, s_x[(lr * G + j / group) * gstride + j % group]);
    }
}

}  // namespace vq

using namespace vq;

extern "C" int vq_skvq_clipped_roundtrip(const void *x, void *out, int dtype, int64_t B, int64_t H, int64_t r,
                                         int64_t D, int64_t x_stride_bh, int64_t out_stride_bh, const int32_t *perm,
                                         int bits, int group, const float *alphas, int n_alphas, void *stream) {
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
    VQ_REQUIRE(G <= SK_THREADS && row_words * 4 <= 48 * 1024, VQ_ERR_UNSUPPORTED,
               "%s: head_dim %lld with group %d does not fit a block (at most %d groups, 48 KB per row)", fn,
               (long long)D, group, SK_THREADS);
    int64_t rows_pb = SK_THREADS / G;
    if (rows_pb * row_words * 4 > 48 * 1024) rows_pb = 48 * 1024 / (row_words * 4);
    const int64_t n_rows = B * H * r, blocks = (n_rows + rows_pb - 1) / rows_pb;
    VQ_REQUIRE(blocks <= 0x7fffffff, VQ_ERR_UNSUPPORTED, "%s: too many rows (%lld)", fn, (long long)n_rows);
    SkAlphas al;
    al.n = n_alphas;
    for (int k = 0; k < SK_MAX_ALPHAS; ++k) al.a[k] = k < n_alphas ? alphas[k] : 1.f;
    hipStream_t st = (hipStream_t)stream;
    const size_t lds = (size_t)(rows_pb * row_words * 4);
    VQ_DISPATCH_FLOAT(dtype, T, {
        hipLaunchKernelGGL((skvq_roundtrip_kernel<T>), dim3((unsigned)blocks), dim3(SK_THREADS), lds, st, (const T *)x,
                           (T *)out, B * H, H, r, D, x_stride_bh, out_stride_bh, perm, group, (int)G, (int)rows_pb,
                           (float)((1 << bits) - 1), al);
    });
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}
