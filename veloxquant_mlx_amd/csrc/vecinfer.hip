// VecInfer product-VQ kernels for gfx950: nearest-centroid assignment and gather.
//
// Assignment follows veloxquant_mlx/metal/src/vecinfer_quantize.metal:8-28 and
// veloxquant_mlx/allocators/vecinfer.py:301-315 operation for operation:
// float32 differences, squares rounded separately, dimensions added left to
// right, strict '<' (the lowest index wins a tie).
//
// The codebook is staged once per block in LDS as float32; all lanes read the
// same centroid at the same time, which the LDS serves as a broadcast.
#include "vecinfer.hpp"

namespace vq {

constexpr int VQ_VPT = 4;  // sub-vectors per thread

// SUB: sub-vector length (0 = runtime), LDS_CB: codebook staged in LDS (else read from global memory).
template <int SUB, bool LDS_CB>
__global__ __launch_bounds__(256) void vq_assign_kernel(const void *__restrict__ x, int xt, int64_t N,
                                                        const void *__restrict__ cb, int ct, int nc, int sub_rt,
                                                        void *__restrict__ idx, int it) {
    extern __shared__ float s_cb[];
    const int sub = SUB ? SUB : sub_rt;
    if (LDS_CB) {
        for (int i = threadIdx.x; i < nc * sub; i += blockDim.x) s_cb[i] = ld_any(cb, ct, i);
        __syncthreads();
    }
    const int64_t tile = (int64_t)blockDim.x * VQ_VPT;
    for (int64_t base = (int64_t)blockIdx.x * tile; base < N; base += (int64_t)gridDim.x * tile) {
        if (SUB) {
            float xv[VQ_VPT][SUB ? SUB : 1];
            float best[VQ_VPT];
            int bi[VQ_VPT];
#pragma unroll
            for (int v = 0; v < VQ_VPT; ++v) {
                int64_t n = base + (int64_t)v * blockDim.x + threadIdx.x;
                best[v] = INFINITY;
                bi[v] = 0;
#pragma unroll
                for (int i = 0; i < SUB; ++i) xv[v][i] = n < N ? ld_any(x, xt, n * SUB + i) : 0.0f;
            }
            for (int c = 0; c < nc; ++c) {
                float cv[SUB ? SUB : 1];
#pragma unroll
                for (int i = 0; i < SUB; ++i) cv[i] = LDS_CB ? s_cb[c * SUB + i] : ld_any(cb, ct, c * SUB + i);
#pragma unroll
                for (int v = 0; v < VQ_VPT; ++v) {
                    float dist = 0.0f;
#pragma unroll
                    for (int i = 0; i < SUB; ++i) {
                        float d = __fsub_rn(xv[v][i], cv[i]);
                        dist = __fadd_rn(dist, __fmul_rn(d, d));
                    }
                    if (dist < best[v]) { best[v] = dist; bi[v] = c; }
                }
            }
#pragma unroll
            for (int v = 0; v < VQ_VPT; ++v) {
                int64_t n = base + (int64_t)v * blockDim.x + threadIdx.x;
                if (n < N) st_idx(idx, it, n, bi[v]);
            }
        } else {
            for (int v = 0; v < VQ_VPT; ++v) {
                int64_t n = base + (int64_t)v * blockDim.x + threadIdx.x;
                if (n >= N) continue;
                float best = INFINITY;
                int bi = 0;
                for (int c = 0; c < nc; ++c) {
                    float dist = 0.0f;
                    for (int i = 0; i < sub; ++i) {
                        float cvv = LDS_CB ? s_cb[c * sub + i] : ld_any(cb, ct, (int64_t)c * sub + i);
                        float d = __fsub_rn(ld_any(x, xt, n * sub + i), cvv);
                        dist = __fadd_rn(dist, __fmul_rn(d, d));
                    }
                    if (dist < best) { best = dist; bi = c; }
                }
                st_idx(idx, it, n, bi);
            }
        }
    }
}

__global__ void vq_dequant_kernel(const void *__restrict__ idx, int it, int64_t N, const void *__restrict__ cb,
                                  int ct, int nc, int sub, void *__restrict__ out, int ot) {
    const int64_t n = N * sub;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        int64_t v = e / sub;
        int i = (int)(e % sub);
        uint32_t c = ld_idx(idx, it, v);
        if (c >= (uint32_t)nc) c = (uint32_t)nc - 1u;  // clamp like vecinfer_dequant.metal
        st_any(out, ot, e, ld_any(cb, ct, (int64_t)c * sub + i));
    }
}

}  // namespace vq

using namespace vq;

static int launch_assign(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, int sub, void *idx, int it,
                         hipStream_t st) {
    const size_t lds = (size_t)nc * sub * sizeof(float);
    const bool use_lds = lds <= 64 * 1024;
    int64_t blocks = cdiv(N, 256 * VQ_VPT);
    if (blocks > 4096) blocks = 4096;
    if (blocks < 1) blocks = 1;
#define VQ_A(SUBV, L)                                                                                        \
    hipLaunchKernelGGL((vq_assign_kernel<SUBV, L>), dim3((unsigned)blocks), dim3(256), (L) ? lds : 0, st, x, xt, N, \
                       cb, ct, nc, sub, idx, it)
    if (!use_lds) { VQ_A(0, false); return VQ_OK; }
    switch (sub) {
        case 2: VQ_A(2, true); break;
        case 4: VQ_A(4, true); break;
        case 8: VQ_A(8, true); break;
        case 16: VQ_A(16, true); break;
        default: VQ_A(0, true); break;
    }
#undef VQ_A
    return VQ_OK;
}

extern "C" int vq_vecinfer_assign(const void *x, int x_dtype, int64_t N, const void *codebook, int cb_dtype,
                                  int n_centroids, int sub_dim, void *idx, int idx_dtype, void *stream) {
    const char *fn = "vq_vecinfer_assign";
    VQ_REQUIRE(is_float_tag(x_dtype) && is_float_tag(cb_dtype), VQ_ERR_INVALID, "%s: unsupported float dtype", fn);
    VQ_REQUIRE(idx_dtype == VQ_I32 || idx_dtype == VQ_U32 || idx_dtype == VQ_U8, VQ_ERR_INVALID,
               "%s: idx dtype must be int32, uint32 or uint8", fn);
    VQ_REQUIRE(n_centroids >= 1 && sub_dim >= 1, VQ_ERR_INVALID,
               "%s: codebook must be non-empty [n_centroids, sub_dim], got [%d, %d]", fn, n_centroids, sub_dim);
    VQ_REQUIRE(idx_dtype != VQ_U8 || n_centroids <= 256, VQ_ERR_INVALID,
               "%s: uint8 indices need n_centroids <= 256, got %d", fn, n_centroids);
    VQ_REQUIRE(N >= 0, VQ_ERR_INVALID, "%s: negative N", fn);
    if (N == 0) return VQ_OK;
    VQ_REQUIRE(x && codebook && idx, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipStream_t st = (hipStream_t)stream;
    if (!launch_assign_mfma(x, x_dtype, N, codebook, cb_dtype, n_centroids, sub_dim, idx, idx_dtype, st))
        launch_assign(x, x_dtype, N, codebook, cb_dtype, n_centroids, sub_dim, idx, idx_dtype, st);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_vecinfer_encode_keys(const void *keys, int k_dtype, int64_t B, int64_t H, int64_t S, int64_t D,
                                       const float *smooth, int smooth_rows, float hadamard_scale, const void *codebook,
                                       int cb_dtype, int n_centroids, int sub_dim, void *idx, int idx_dtype, void *k_hat,
                                       float *k_tilde, void *stream) {
    const char *fn = "vq_vecinfer_encode_keys";
    VQ_REQUIRE(is_float_tag(k_dtype) && is_float_tag(cb_dtype), VQ_ERR_INVALID, "%s: unsupported float dtype", fn);
    VQ_REQUIRE(idx_dtype == VQ_I32 || idx_dtype == VQ_U32 || idx_dtype == VQ_U8, VQ_ERR_INVALID,
               "%s: idx dtype must be int32, uint32 or uint8", fn);
    VQ_REQUIRE(B >= 0 && H >= 1 && S >= 0 && D >= 1, VQ_ERR_INVALID, "%s: keys must be 4D [B, H, S, D]", fn);
    VQ_REQUIRE(n_centroids >= 1 && sub_dim >= 1 && D % sub_dim == 0, VQ_ERR_INVALID,
               "%s: D=%lld not divisible by sub_dim=%d", fn, (long long)D, sub_dim);
    VQ_REQUIRE((D & (D - 1)) == 0, VQ_ERR_INVALID, "%s: D=%lld must be a power of 2 (Walsh-Hadamard transform)", fn, (long long)D);
    VQ_REQUIRE(idx_dtype != VQ_U8 || n_centroids <= 256, VQ_ERR_INVALID, "%s: uint8 indices need n_centroids <= 256, got %d", fn,
               n_centroids);
    VQ_REQUIRE(smooth == nullptr || smooth_rows == 1 || smooth_rows == H, VQ_ERR_INVALID,
               "%s: smooth must have 1 or H=%lld rows, got %d", fn, (long long)H, smooth_rows);
    if (B * S == 0) return VQ_OK;
    VQ_REQUIRE(keys && codebook && idx, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE(launch_encode_keys_mfma(keys, k_dtype, B, H, S, D, smooth, smooth_rows, hadamard_scale, codebook, cb_dtype,
                                       n_centroids, sub_dim, idx, idx_dtype, k_hat, k_tilde, (hipStream_t)stream),
               VQ_ERR_UNSUPPORTED,
               "%s: needs sub_dim 4 or 8, D / sub_dim in {8, 16, 32, 64}, n_centroids <= 256 and 16-byte aligned buffers", fn);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

extern "C" int vq_vecinfer_dequant(const void *idx, int idx_dtype, int64_t N, const void *codebook, int cb_dtype,
                                   int n_centroids, int sub_dim, void *out, int out_dtype, void *stream) {
    const char *fn = "vq_vecinfer_dequant";
    VQ_REQUIRE(is_float_tag(out_dtype) && is_float_tag(cb_dtype), VQ_ERR_INVALID, "%s: unsupported float dtype", fn);
    VQ_REQUIRE(idx_dtype == VQ_I32 || idx_dtype == VQ_U32 || idx_dtype == VQ_U8, VQ_ERR_INVALID,
               "%s: idx dtype must be int32, uint32 or uint8", fn);
    VQ_REQUIRE(n_centroids >= 1 && sub_dim >= 1, VQ_ERR_INVALID, "%s: codebook must be 2D and non-empty", fn);
    VQ_REQUIRE(N >= 0, VQ_ERR_INVALID, "%s: negative N", fn);
    if (N == 0) return VQ_OK;
    VQ_REQUIRE(idx && codebook && out, VQ_ERR_INVALID, "%s: null pointer", fn);
    hipStream_t st = (hipStream_t)stream;
    int64_t g = cdiv(N * sub_dim, 256);
    if (g > 1 << 20) g = 1 << 20;
    hipLaunchKernelGGL(vq_dequant_kernel, dim3((unsigned)g), dim3(256), 0, st, idx, idx_dtype, N, codebook, cb_dtype,
                       n_centroids, sub_dim, out, out_dtype);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}
