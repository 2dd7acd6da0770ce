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
