// Shared pieces of the VecInfer kernels.
#pragma once
#include "common.hpp"

namespace vq {

// Element loads/stores typed at run time: they sit outside the distance loop,
// so one kernel per (SUB, codebook placement) serves every dtype combination.
__device__ __forceinline__ float ld_any(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}
__device__ __forceinline__ void st_any(void *p, int tag, int64_t i, float v) {
    if (tag == VQ_F16) ((f16 *)p)[i] = (f16)v;
    else if (tag == VQ_BF16) ((u16 *)p)[i] = f32_to_bf16(v);
    else ((float *)p)[i] = v;
}
__device__ __forceinline__ void st_idx(void *p, int tag, int64_t i, int v) {
    if (tag == VQ_U8) ((uint8_t *)p)[i] = (uint8_t)v;
    else ((int32_t *)p)[i] = v;
}
__device__ __forceinline__ uint32_t ld_idx(const void *p, int tag, int64_t i) {
    if (tag == VQ_U8) return ((const uint8_t *)p)[i];
    return (uint32_t)((const int32_t *)p)[i];
}

// MFMA assignment (vecinfer_mfma.hip).  Returns false, launching nothing, for shapes it does
// not cover (the exact vector kernel in vecinfer.hip takes those).
bool launch_assign_mfma(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, int sub, void *idx, int it,
                        hipStream_t st);

// Fused key encode (and optional decode) around the MFMA assignment: keys [B, heads, S, D] ->
// (keys / smooth) @ H -> indices [B * heads * S, D / sub], optionally k_hat (dtype of keys) and
// k_tilde (float32).  Returns false, launching nothing, for shapes it does not cover
// (sub_dim 4 or 8, D / sub_dim in {8, 16, 32, 64}, at most 256 centroids, 16-byte aligned buffers).
bool launch_encode_keys_mfma(const void *keys, int kt, int64_t B, int64_t heads, int64_t S, int64_t D, const float *smooth,
                             int smooth_rows, float h, const void *cb, int ct, int nc, int sub, void *idx, int it, void *k_hat,
                             float *k_tilde, hipStream_t st);

}  // namespace vq
