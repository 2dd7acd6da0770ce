// Appending new tokens to the un-quantised tail of a KIVI cache: keys and values in one launch.
#include "common.hpp"

namespace vq {

struct TailSrc { const uint4 *p; int64_t sb, sh, ss; };   // strides in 16-byte vectors

// One thread per 16 bytes of one tensor; blockIdx.y = 0 keys, 1 values.
__global__ __launch_bounds__(256) void kv_tail_append_kernel(TailSrc k, TailSrc v, uint4 *__restrict__ k_tail,
                                                             uint4 *__restrict__ v_tail, int64_t B, int64_t H, int64_t S,
                                                             int64_t row_vecs, int64_t tail_cap, int64_t pos) {
    const TailSrc src = blockIdx.y ? v : k;
    uint4 *dst = blockIdx.y ? v_tail : k_tail;
    const int64_t total = B * H * S * row_vecs;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t c = i % row_vecs, s = (i / row_vecs) % S, bh = i / (row_vecs * S);
        const int64_t b = bh / H, h = bh % H;
        dst[(bh * tail_cap + pos + s) * row_vecs + c] = src.p[b * src.sb + h * src.sh + s * src.ss + c];
    }
}

// A chunk with a flush: every row of [tail ; new] from min(n_tail, n_flush) on goes where it lives
// afterwards.  New rows below n_flush go into the tail (they are quantised from there by the
// launch that follows), rows from n_flush on, old or new, to the front of the spare tail.
__global__ __launch_bounds__(256) void kv_chunk_route_kernel(TailSrc k, TailSrc v, uint4 *__restrict__ k_tail,
                                                             uint4 *__restrict__ v_tail, uint4 *__restrict__ k_spare,
                                                             uint4 *__restrict__ v_spare, int64_t B, int64_t H, int64_t row_vecs,
                                                             int64_t tail_cap, int64_t spare_cap, int64_t n_tail, int64_t n_flush,
                                                             int64_t need) {
    const TailSrc src = blockIdx.y ? v : k;
    uint4 *tail = blockIdx.y ? v_tail : k_tail;
    uint4 *spare = blockIdx.y ? v_spare : k_spare;
    const int64_t r0 = n_tail < n_flush ? n_tail : n_flush, count = need - r0;
    const int64_t total = B * H * count * row_vecs;
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t c = i % row_vecs, r = r0 + (i / row_vecs) % count, bh = i / (row_vecs * count);
        const int64_t b = bh / H, h = bh % H;
        const uint4 x = r < n_tail ? tail[(bh * tail_cap + r) * row_vecs + c]
                                   : src.p[b * src.sb + h * src.sh + (r - n_tail) * src.ss + c];
        if (r < n_flush) tail[(bh * tail_cap + r) * row_vecs + c] = x;
        else spare[(bh * spare_cap + r - n_flush) * row_vecs + c] = x;
    }
}

int pack_kv_pair(const void *k, const void *v, int dtype, int64_t BH, int64_t S, int64_t D, int64_t xs, int group,
                 int levels, float eps, int bits, int v_layout, void *kp, void *ks, void *kz, void *vp, void *vs, void *vz,
                 int meta_dtype, int64_t cap, int64_t tok0, void *stream);
bool append_one_launch(const void *k_new, const void *v_new, const int64_t ks[3], const int64_t vs[3], const void *k_tail,
                       const void *v_tail, void *k_spare, void *v_spare, int dtype, int64_t B, int64_t H, int64_t D, int64_t tail_cap,
                       int64_t spare_cap, int64_t n_tail, int64_t n_flush, int64_t need, int group, int levels, float eps, int bits,
                       int v_layout, void *kp, void *ksc, void *kz, void *vp, void *vsc, void *vz, int meta_dtype, int64_t cap,
                       int64_t tok0, void *stream);

}  // namespace vq

using namespace vq;

extern "C" int vq_kv_tail_append(const void *k_new, const void *v_new, const int64_t k_strides[3],
                                 const int64_t v_strides[3], void *k_tail, void *v_tail, int elem_bytes, int64_t B,
                                 int64_t H, int64_t S, int64_t D, int64_t tail_cap, int64_t pos, void *stream) {
    const char *fn = "vq_kv_tail_append";
    VQ_REQUIRE(elem_bytes == 2 || elem_bytes == 4, VQ_ERR_INVALID, "%s: elem_bytes must be 2 or 4, got %d", fn, elem_bytes);
    VQ_REQUIRE(B >= 0 && H >= 0 && S >= 0 && D >= 1, VQ_ERR_INVALID, "%s: negative dimension", fn);
    VQ_REQUIRE(pos >= 0 && pos + S <= tail_cap, VQ_ERR_INVALID, "%s: tokens [%lld, %lld) exceed the tail capacity %lld", fn,
               (long long)pos, (long long)(pos + S), (long long)tail_cap);
    VQ_REQUIRE(k_strides && v_strides, VQ_ERR_INVALID, "%s: null strides", fn);
    VQ_REQUIRE((D * elem_bytes) % 16 == 0, VQ_ERR_UNSUPPORTED, "%s: D * elem_bytes must be a multiple of 16", fn);
    for (int i = 0; i < 3; ++i)
        VQ_REQUIRE(k_strides[i] >= 0 && v_strides[i] >= 0 && (k_strides[i] * elem_bytes) % 16 == 0 &&
                       (v_strides[i] * elem_bytes) % 16 == 0,
                   VQ_ERR_UNSUPPORTED, "%s: strides must be non-negative multiples of 16 bytes", fn);
    if (B * H * S == 0) return VQ_OK;
    VQ_REQUIRE(k_new && v_new && k_tail && v_tail, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE((((uintptr_t)k_new | (uintptr_t)v_new | (uintptr_t)k_tail | (uintptr_t)v_tail) & 15u) == 0, VQ_ERR_UNSUPPORTED,
               "%s: pointers must be 16-byte aligned", fn);
    const int64_t vec = 16 / elem_bytes, row_vecs = D / vec, total = B * H * S * row_vecs;
    int64_t blocks = (total + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    const TailSrc k = {(const uint4 *)k_new, k_strides[0] / vec, k_strides[1] / vec, k_strides[2] / vec};
    const TailSrc v = {(const uint4 *)v_new, v_strides[0] / vec, v_strides[1] / vec, v_strides[2] / vec};
    hipLaunchKernelGGL(kv_tail_append_kernel, dim3((unsigned)blocks, 2), dim3(256), 0, (hipStream_t)stream, k, v,
                       (uint4 *)k_tail, (uint4 *)v_tail, B, H, S, row_vecs, tail_cap, pos);
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

// One call for a whole chunk of a packed KIVI cache: append, quantise what aged out of the
// residual window, start the next tail.  The launches are those of the single-step entry points;
// what is saved is the host time between them, which dominates a chunked prefill whose
// attention launches are short.
extern "C" int vq_kivi_cache_append(const vq_kivi_append_args *pa, void *stream) {
    const char *fn = "vq_kivi_cache_append";
    VQ_REQUIRE(pa != nullptr, VQ_ERR_INVALID, "%s: null args", fn);
    const vq_kivi_append_args &a = *pa;
    VQ_REQUIRE(a.B >= 0 && a.H >= 0 && a.S >= 0 && a.D >= 1, VQ_ERR_INVALID, "%s: bad dimensions", fn);
    VQ_REQUIRE(a.dtype == VQ_F16 || a.dtype == VQ_BF16 || a.dtype == VQ_F32, VQ_ERR_INVALID, "%s: unsupported dtype tag %d", fn,
               a.dtype);
    VQ_REQUIRE(a.n_tail >= 0 && a.n_tail + a.S <= a.tail_cap, VQ_ERR_INVALID,
               "%s: %lld tail rows plus %lld new tokens exceed the tail capacity %lld", fn, (long long)a.n_tail,
               (long long)a.S, (long long)a.tail_cap);
    const int64_t need = a.n_tail + a.S, keep = need - a.n_flush;
    VQ_REQUIRE(a.n_flush >= 0 && a.n_flush <= need, VQ_ERR_INVALID, "%s: n_flush=%lld outside [0, %lld]", fn,
               (long long)a.n_flush, (long long)need);
    if (a.n_flush > 0) {
        VQ_REQUIRE(a.k_spare && a.v_spare && a.k_spare != a.k_tail && a.v_spare != a.v_tail, VQ_ERR_INVALID,
                   "%s: a flush needs spare tails distinct from the tails", fn);
        VQ_REQUIRE(keep <= a.spare_cap, VQ_ERR_INVALID, "%s: %lld kept rows exceed the spare capacity %lld", fn,
                   (long long)keep, (long long)a.spare_cap);
    }
    const int es = a.dtype == VQ_F32 ? 4 : 2;
    if (a.n_flush == 0)
        return vq_kv_tail_append(a.k_new, a.v_new, a.k_strides, a.v_strides, a.k_tail, a.v_tail, es, a.B, a.H, a.S, a.D,
                                 a.tail_cap, a.n_tail, stream);
    VQ_REQUIRE((a.D * es) % 16 == 0, VQ_ERR_UNSUPPORTED, "%s: D * element size must be a multiple of 16", fn);
    for (int i = 0; i < 3; ++i)
        VQ_REQUIRE(a.k_strides[i] >= 0 && a.v_strides[i] >= 0 && (a.k_strides[i] * es) % 16 == 0 &&
                       (a.v_strides[i] * es) % 16 == 0,
                   VQ_ERR_UNSUPPORTED, "%s: strides must be non-negative multiples of 16 bytes", fn);
    VQ_REQUIRE(a.B * a.H >= 1, VQ_ERR_INVALID, "%s: a flush of an empty batch", fn);
    VQ_REQUIRE((a.S == 0 || (a.k_new && a.v_new)) && a.k_tail && a.v_tail, VQ_ERR_INVALID, "%s: null pointer", fn);
    VQ_REQUIRE((((uintptr_t)a.k_new | (uintptr_t)a.v_new | (uintptr_t)a.k_tail | (uintptr_t)a.v_tail | (uintptr_t)a.k_spare |
                 (uintptr_t)a.v_spare) & 15u) == 0,
               VQ_ERR_UNSUPPORTED, "%s: pointers must be 16-byte aligned", fn);
    VQ_REQUIRE(a.k_packed && a.k_scale && a.k_zero && a.v_packed && a.v_scale && a.v_zero, VQ_ERR_INVALID,
               "%s: null packed store", fn);
    // one launch where the fused kernel takes the shape: new rows are quantised from where they lie
    if (a.S > 0 && append_one_launch(a.k_new, a.v_new, a.k_strides, a.v_strides, a.k_tail, a.v_tail, a.k_spare, a.v_spare, a.dtype,
                                     a.B, a.H, a.D, a.tail_cap, a.spare_cap, a.n_tail, a.n_flush, need, a.group, a.levels, a.eps,
                                     a.pack_bits, a.v_layout, a.k_packed, a.k_scale, a.k_zero, a.v_packed, a.v_scale, a.v_zero,
                                     a.meta_dtype, a.cap_tokens, a.dst_tok0, stream)) {
        VQ_HIP_CHECK_LAUNCH(fn);
        return VQ_OK;
    }
    const int64_t vec = 16 / es, row_vecs = a.D / vec;
    const int64_t r0 = a.n_tail < a.n_flush ? a.n_tail : a.n_flush, total = a.B * a.H * (need - r0) * row_vecs;
    if (total > 0) {
        int64_t blocks = (total + 255) / 256;
        if (blocks > 4096) blocks = 4096;
        const TailSrc k = {(const uint4 *)a.k_new, a.k_strides[0] / vec, a.k_strides[1] / vec, a.k_strides[2] / vec};
        const TailSrc v = {(const uint4 *)a.v_new, a.v_strides[0] / vec, a.v_strides[1] / vec, a.v_strides[2] / vec};
        hipLaunchKernelGGL(kv_chunk_route_kernel, dim3((unsigned)blocks, 2), dim3(256), 0, (hipStream_t)stream, k, v,
                           (uint4 *)a.k_tail, (uint4 *)a.v_tail, (uint4 *)a.k_spare, (uint4 *)a.v_spare, a.B, a.H, row_vecs,
                           a.tail_cap, a.spare_cap, a.n_tail, a.n_flush, need);
        VQ_HIP_CHECK_LAUNCH(fn);
    }
    return pack_kv_pair(a.k_tail, a.v_tail, a.dtype, a.B * a.H, a.n_flush, a.D, a.tail_cap * a.D, a.group, a.levels, a.eps,
                        a.pack_bits, a.v_layout, a.k_packed, a.k_scale, a.k_zero, a.v_packed, a.v_scale, a.v_zero, a.meta_dtype,
                        a.cap_tokens, a.dst_tok0, stream);
}
