// VecInfer nearest-centroid assignment on the matrix unit (gfx950, wave64), with indices
// identical to the sequential float32 rule of veloxquant_mlx/metal/src/vecinfer_quantize.metal:8-28
// (squares rounded separately, dimensions added left to right, strict '<').
//
// The matrix unit cannot reproduce that rounding order, so it is used as a filter whose error
// is bounded, and every decision the bound cannot settle is re-taken with the exact rule:
//
//   t[c, v] = |c|^2 - 2 c.v     v_mfma_f32_16x16x32_f16: A = -2c (16 centroids), B = v (16
//                               sub-vectors), accumulator input = |c|^2 in float32.
//                               c and v travel as fp16 high part + fp16 remainder in separate
//                               k-slots (all four cross terms), so t is good to ~2^-20 for
//                               fp16, bf16 and float32 inputs alike.
//   per sub-vector the two smallest t are tracked (3 VALU ops per score: the centroid tile
//   number rides in the 4 low mantissa bits, then one min and one med3);
//   if second - first > eps (eps = 2^-14 (|v|^2 + max|c|^2), far above filter error plus the
//   rounding of the exact rule) the first is the answer;
//   otherwise, if the two leaders come from different trackers and no other tracked score
//   lies within eps, the exact rule decides between the two; in the remaining (very rare)
//   case the column's scores are recomputed and every centroid with t <= first + eps is
//   evaluated with the exact rule, lowest index winning ties.
//
// A wave keeps the whole codebook in registers as MFMA operands (n_centroids <= 256, sub_dim 4
// or 8) and walks 64 sub-vectors per step: one 16-byte load per lane, an LDS bounce to put
// the sub-vectors into B-operand order, 4 x 16 MFMAs.
#include "vecinfer.hpp"

namespace vq {

typedef uint32_t u32;
typedef uint32_t u32x4v __attribute__((ext_vector_type(4)));

constexpr int VM_MAXC = 256;
constexpr int VM_TILES = VM_MAXC / 16;

__device__ __forceinline__ float exact_dist(const float *x, const float *c, int sub) {
    float dist = 0.0f;
    for (int i = 0; i < sub; ++i) {
        const float d = __fsub_rn(x[i], c[i]);
        dist = __fadd_rn(dist, __fmul_rn(d, d));
    }
    return dist;
}

// Bare min / median-of-three: the scores are never NaN, so the canonicalising moves the
// compiler wraps around fminf would only cost issue slots in the hottest loop.
__device__ __forceinline__ float vmin(float a, float b) {
    float d;
    asm("v_min_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float vmed3(float a, float b, float c) {
    float d;
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

// two smallest of (a1 <= a2) and (b1 <= b2) with their indices
__device__ __forceinline__ void merge_top2(float &a1, float &a2, int &ia1, int &ia2, float b1, float b2, int ib1, int ib2) {
    const bool c = a1 <= b1;
    const float f = c ? a1 : b1;
    const int fi = c ? ia1 : ib1;
    const float sa = c ? a2 : b2, sb = c ? b1 : a1;
    const int sia = c ? ia2 : ib2, sib = c ? ib1 : ia1;
    const bool c2 = sa <= sb;
    a1 = f; ia1 = fi;
    a2 = c2 ? sa : sb;
    ia2 = c2 ? sia : sib;
}

// ---- the key transform in front of the assignment, and the reconstruction behind it --------
//
// With LT > 0 the sub-vectors are not taken as they are: 64 consecutive sub-vectors are 64 / LT
// whole tokens of D = LT * SUB channels (lane j of a group of LT lanes holds channels
// [SUB j, SUB (j + 1))), and each token first goes through  k~ = (k / smooth) @ H  with H the
// orthonormal Sylvester-Hadamard matrix (entries +-h in natural order), done as a fast
// Walsh-Hadamard transform across the LT lanes: in-lane butterflies over the SUB registers, then
// one butterfly per lane bit (cross-lane moves inside the row of 16, LDS permutes beyond it), then
// the scale h.  Optionally the chosen centroids go back the same way, k^ = (c @ H^T) * smooth
// (H is symmetric), and k~ itself can be written out.  This is the reference's fused key
// encode+decode (veloxquant_mlx/metal/_vecinfer.py:225-293) as a front and back end of the
// MFMA assignment.
struct KeyXform {
    const float *smooth;   // [smooth_rows, D] float32 or null
    int smooth_rows;       // 1 or the number of heads
    int64_t heads, S;      // keys are [B, heads, S, D]
    float h;               // |H[0][0]|
    void *k_hat;           // [N * SUB] reconstruction in dtype hat_dtype, or null
    int hat_dtype;
    float *k_tilde;        // [N * SUB] transformed keys, or null
};

template <int CTRL> __device__ __forceinline__ float xform_dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, x), __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, false));
}
// value of lane (lane ^ M)
template <int M> __device__ __forceinline__ float lane_xor(float x) {
    if constexpr (M == 1) return xform_dpp<0xB1>(x);        // quad_perm [1,0,3,2]
    else if constexpr (M == 2) return xform_dpp<0x4E>(x);   // quad_perm [2,3,0,1]
    else if constexpr (M == 8) return xform_dpp<0x128>(x);  // row_ror 8
    else return __shfl_xor(x, M);
}
template <int SUB, int M> __device__ __forceinline__ void lane_butterfly(float (&x)[8], int lane) {
    const bool upper = (lane & M) != 0;
#pragma unroll
    for (int e = 0; e < SUB; ++e) {
        const float p = lane_xor<M>(x[e]);
        x[e] = upper ? p - x[e] : x[e] + p;
    }
}
// unnormalised Walsh-Hadamard transform of the LT * SUB values a group of LT lanes holds
template <int SUB, int LT> __device__ __forceinline__ void wht_lanes(float (&x)[8], int lane) {
#pragma unroll
    for (int hlf = 1; hlf < SUB; hlf <<= 1)
#pragma unroll
        for (int i = 0; i < SUB; i += 2 * hlf)
#pragma unroll
            for (int k = i; k < i + hlf; ++k) {
                const float a = x[k], b = x[k + hlf];
                x[k] = a + b;
                x[k + hlf] = a - b;
            }
    if constexpr (LT > 1) lane_butterfly<SUB, 1>(x, lane);
    if constexpr (LT > 2) lane_butterfly<SUB, 2>(x, lane);
    if constexpr (LT > 4) lane_butterfly<SUB, 4>(x, lane);
    if constexpr (LT > 8) lane_butterfly<SUB, 8>(x, lane);
    if constexpr (LT > 16) lane_butterfly<SUB, 16>(x, lane);
    if constexpr (LT > 32) lane_butterfly<SUB, 32>(x, lane);
}

template <int SUB, int LT>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) void vq_assign_mfma_kernel(const void *__restrict__ x, int xt, int64_t N,
                                                             const void *__restrict__ cb, int ct, int nc,
                                                             void *__restrict__ idx, int it, KeyXform kx) {
    __shared__ float s_cb[VM_MAXC * 8];          // codebook as float32, row stride SUB
    __shared__ float s_c2[VM_MAXC];              // |c|^2, huge past the end
    __shared__ uint4 s_A[VM_TILES][64];          // MFMA A operands of every centroid tile
    __shared__ float4 s_C2[VM_TILES][64];        // MFMA accumulator inputs of every centroid tile
    __shared__ __align__(16) f16 s_xh[4][64][16];   // per wave: sub-vector high part [0..7] | remainder [8..15]
    __shared__ float s_xf[4][64][8];             // per wave: sub-vector as float32 (exact rule)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, blk = lane >> 4;
    const int ntiles = (nc + 15) / 16;

    // thread c fetches centroid c with one or two vector loads (the row is 8 to 32 bytes); a
    // codebook that is not 16-byte aligned goes element by element
    if ((reinterpret_cast<uintptr_t>(cb) & 15u) == 0) {
        if (tid < nc) {
            float row[SUB];
            if (ct == VQ_F32) {
#pragma unroll
                for (int e = 0; e < SUB; e += 4) {
                    const float4 v = *reinterpret_cast<const float4 *>((const float *)cb + tid * SUB + e);
                    row[e] = v.x; row[e + 1] = v.y; row[e + 2] = v.z; row[e + 3] = v.w;
                }
            } else {
                u32 w[SUB / 2];
                if constexpr (SUB == 8) {
                    const uint4 v = *reinterpret_cast<const uint4 *>((const u16 *)cb + tid * 8);
                    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
                } else {
                    const uint2 v = *reinterpret_cast<const uint2 *>((const u16 *)cb + tid * 4);
                    w[0] = v.x; w[1] = v.y;
                }
#pragma unroll
                for (int e = 0; e < SUB / 2; ++e) {
                    if (ct == VQ_F16) {
                        const f16x2 h = __builtin_bit_cast(f16x2, w[e]);
                        row[2 * e] = (float)h[0]; row[2 * e + 1] = (float)h[1];
                    } else {
                        row[2 * e] = __uint_as_float(w[e] << 16); row[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                    }
                }
            }
#pragma unroll
            for (int e = 0; e < SUB; ++e) s_cb[tid * SUB + e] = row[e];
        }
    } else {
        for (int i = tid; i < nc * SUB; i += 256) s_cb[i] = ld_any(cb, ct, i);
    }
    __syncthreads();
    {
        float c2 = 3.0e38f;
        if (tid < nc) {
            c2 = 0.f;
            for (int e = 0; e < SUB; ++e) c2 += s_cb[tid * SUB + e] * s_cb[tid * SUB + e];
        }
        s_c2[tid] = c2;
    }
    __syncthreads();
    // codebook as MFMA operands: A of tile j, lane (n, blk) = -2 c of centroid 16j + n (high part in
    // lane groups 0,1, remainder in 2,3); accumulator input register r = |c|^2 of centroid 16j + 4 blk + r
    for (int e4 = tid; e4 < VM_TILES * 64; e4 += 256) {
        const int j = e4 >> 6, l = e4 & 63, ln = l & 15, lb = l >> 4;
        const int ci = 16 * j + ln;
        f16x8 a;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const float c = (ci < nc && e < SUB) ? s_cb[ci * SUB + e] : 0.f;
            const f16 hi = (f16)c;
            const f16 lo = (f16)(c - (float)hi);
            a[e] = (f16)(-2.f) * (lb < 2 ? hi : lo);
        }
        s_A[j][l] = __builtin_bit_cast(uint4, a);
        const int cr = 16 * j + 4 * lb;
        s_C2[j][l] = make_float4(s_c2[cr], s_c2[cr + 1], s_c2[cr + 2], s_c2[cr + 3]);
    }
    __syncthreads();
    f16x8 A[VM_TILES];
    f32x4 C2[VM_TILES];
#pragma unroll
    for (int j = 0; j < VM_TILES; ++j) {
        A[j] = __builtin_bit_cast(f16x8, s_A[j][lane]);
        const float4 c = s_C2[j][lane];
        C2[j] = f32x4{c.x, c.y, c.z, c.w};
    }
    float cmax2 = tid < nc ? s_c2[tid] : 0.f;
    for (int i = tid + 256; i < nc; i += 256) cmax2 = fmaxf(cmax2, s_c2[i]);
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cmax2 = fmaxf(cmax2, __shfl_xor(cmax2, o));
    {   // block-wide maximum through the first slots of the (now free) wave scratch
        if (lane == 0) s_xf[wave][0][0] = cmax2;
        __syncthreads();
        cmax2 = fmaxf(fmaxf(s_xf[0][0][0], s_xf[1][0][0]), fmaxf(s_xf[2][0][0], s_xf[3][0][0]));
        __syncthreads();
    }

    const int64_t n_steps = (N + 63) / 64;
    const int64_t stride = (int64_t)gridDim.x * 4;
    const bool packed16 = SUB == 8 && xt != VQ_F32;   // one 16-byte load per sub-vector, fetched a step ahead
    auto load_raw = [&](int64_t step) {
        const int64_t sv = step * 64 + lane;
        return (packed16 && step < n_steps && sv < N) ? *reinterpret_cast<const uint4 *>((const u16 *)x + sv * 8)
                                                      : make_uint4(0, 0, 0, 0);
    };
    uint4 raw = load_raw((int64_t)blockIdx.x * 4 + wave);
    for (int64_t step = (int64_t)blockIdx.x * 4 + wave; step < n_steps; step += stride) {
        const int64_t sv = step * 64 + lane;   // this lane's sub-vector
        const uint4 raw_next = load_raw(step + stride);
        // ---- convert, split, bounce through LDS
        float xf[8];
        if (packed16) {
            const u32 w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                if (xt == VQ_F16) {
                    const f16x2 h = __builtin_bit_cast(f16x2, w[e]);
                    xf[2 * e] = (float)h[0]; xf[2 * e + 1] = (float)h[1];
                } else {
                    xf[2 * e] = __uint_as_float(w[e] << 16); xf[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) xf[e] = (e < SUB && sv < N) ? ld_any(x, xt, sv * SUB + e) : 0.f;
        }
        float sm[8];
        if constexpr (LT > 0) {
            // the lane's channels of its token: divide by the smoothing factors, transform, scale
            const int64_t token = sv / LT;
            const int64_t srow = kx.smooth_rows > 1 ? (token / kx.S) % kx.heads : 0;
#pragma unroll
            for (int e = 0; e < 8; ++e) sm[e] = 1.f;
            if (kx.smooth != nullptr && sv < N) {
                const float *sp = kx.smooth + (srow * LT + (lane & (LT - 1))) * SUB;
#pragma unroll
                for (int e = 0; e < SUB; ++e) { sm[e] = sp[e]; xf[e] = xf[e] / sm[e]; }
            }
            wht_lanes<SUB, LT>(xf, lane);
#pragma unroll
            for (int e = 0; e < SUB; ++e) xf[e] *= kx.h;
            if (kx.k_tilde != nullptr && sv < N) {
#pragma unroll
                for (int e = 0; e < SUB; e += 4)
                    *reinterpret_cast<float4 *>(kx.k_tilde + sv * SUB + e) = make_float4(xf[e], xf[e + 1], xf[e + 2], xf[e + 3]);
            }
        }
        f16x8 xh, xl;
        float x2 = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            xh[e] = (f16)xf[e];
            xl[e] = (f16)(xf[e] - (float)xh[e]);
            x2 += xf[e] * xf[e];
        }
        *reinterpret_cast<f16x8 *>(&s_xh[wave][lane][0]) = xh;
        *reinterpret_cast<f16x8 *>(&s_xh[wave][lane][8]) = xl;
        *reinterpret_cast<float4 *>(&s_xf[wave][lane][0]) = make_float4(xf[0], xf[1], xf[2], xf[3]);
        *reinterpret_cast<float4 *>(&s_xf[wave][lane][4]) = make_float4(xf[4], xf[5], xf[6], xf[7]);
        // the wave reads what its own lanes wrote: LDS serves a wave's requests in order
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");

        int my_idx = 0;
#pragma unroll 1
        for (int t = 0; t < 4; ++t) {
            // B operand: sub-vector 16t + n; lane groups 0,2 carry the high part, 1,3 the remainder
            const f16x8 B = *reinterpret_cast<const f16x8 *>(&s_xh[wave][16 * t + n][8 * (blk & 1)]);
            const float eps = 6.103515625e-05f * (__shfl(x2, 16 * t + n) + cmax2);   // 2^-14 (|v|^2 + max |c|^2)
            float k1[4], k2[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) { k1[r] = INFINITY; k2[r] = INFINITY; }
            // four centroid tiles at a time: their products are issued together, so the tracking
            // of one tile runs while the next product is still in the matrix unit (tiles past the
            // last centroid of a started group carry zero operands and a huge |c|^2: never chosen)
#pragma unroll
            for (int j4 = 0; j4 < VM_TILES; j4 += 4) {
                if (j4 < ntiles) {
                    f32x4 D[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) D[u] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A[j4 + u], B, C2[j4 + u], 0, 0, 0);
#pragma unroll
                    for (int u = 0; u < 4; ++u)
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const float key = __uint_as_float((__float_as_uint(D[u][r]) & 0xfffffff0u) | (u32)(j4 + u));
                            k2[r] = vmed3(k1[r], k2[r], key);
                            k1[r] = vmin(k1[r], key);
                        }
                }
            }
            // lane top-2 over its four rows, then over the four lane groups of the column
            float f1 = k1[0], f2 = k2[0];
            int i1 = 16 * (int)(__float_as_uint(k1[0]) & 15u) + 4 * blk, i2 = 16 * (int)(__float_as_uint(k2[0]) & 15u) + 4 * blk;
#pragma unroll
            for (int r = 1; r < 4; ++r)
                merge_top2(f1, f2, i1, i2, k1[r], k2[r], 16 * (int)(__float_as_uint(k1[r]) & 15u) + 4 * blk + r,
                           16 * (int)(__float_as_uint(k2[r]) & 15u) + 4 * blk + r);
#pragma unroll
            for (int o = 16; o <= 32; o <<= 1) {
                const float g1 = __shfl_xor(f1, o), g2 = __shfl_xor(f2, o);
                const int j1 = __shfl_xor(i1, o), j2 = __shfl_xor(i2, o);
                merge_top2(f1, f2, i1, i2, g1, g2, j1, j2);
            }
            int res = i1;
            const bool unsure = !(f2 - f1 > eps);
            if (__any(unsure)) {
                const float *xv = &s_xf[wave][16 * t + n][0];
                // Smallest tracked score outside the leading two.  A score a tracker dropped is at
                // least that tracker's second entry, so when the leading two come from different
                // trackers nothing untracked lies below g3.
                float g3 = INFINITY;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int a = 16 * (int)(__float_as_uint(k1[r]) & 15u) + 4 * blk + r;
                    const int b = 16 * (int)(__float_as_uint(k2[r]) & 15u) + 4 * blk + r;
                    if (a != i1 && a != i2) g3 = fminf(g3, k1[r]);
                    if (b != i1 && b != i2) g3 = fminf(g3, k2[r]);
                }
                g3 = fminf(g3, __shfl_xor(g3, 16));
                g3 = fminf(g3, __shfl_xor(g3, 32));
                const bool two = unsure && (i1 & 15) != (i2 & 15) && (g3 - f1 > eps) && i1 < nc && i2 < nc;
                if (two) {   // exactly two contenders: the exact rule on both
                    const float d1 = exact_dist(xv, &s_cb[i1 * SUB], SUB), d2 = exact_dist(xv, &s_cb[i2 * SUB], SUB);
                    res = (d2 < d1 || (d2 == d1 && i2 < i1)) ? i2 : i1;
                }
                const bool many = unsure && !two;
                if (__any(many)) {
                    // recompute the column's scores and apply the exact rule to every centroid the
                    // filter cannot exclude (operands from their LDS image: this path is very rare)
                    const float thr = f1 + eps;
                    float dbest = INFINITY;
                    int ibest = 0x7fffffff;
#pragma unroll 1
                    for (int j = 0; j < ntiles; ++j) {
                        const float4 c4 = s_C2[j][lane];
                        const f32x4 D = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, s_A[j][lane]), B,
                                                                              f32x4{c4.x, c4.y, c4.z, c4.w}, 0, 0, 0);
#pragma unroll 1
                        for (int r = 0; r < 4; ++r) {
                            const int ci = 16 * j + 4 * blk + r;
                            const float dr = r == 0 ? D[0] : r == 1 ? D[1] : r == 2 ? D[2] : D[3];
                            if (many && ci < nc && dr <= thr) {
                                const float d = exact_dist(xv, &s_cb[ci * SUB], SUB);
                                if (d < dbest || (d == dbest && ci < ibest)) { dbest = d; ibest = ci; }
                            }
                        }
                    }
#pragma unroll
                    for (int o = 16; o <= 32; o <<= 1) {
                        const float d = __shfl_xor(dbest, o);
                        const int ci = __shfl_xor(ibest, o);
                        if (d < dbest || (d == dbest && ci < ibest)) { dbest = d; ibest = ci; }
                    }
                    if (many) res = ibest;
                }
            }
            if (blk == t) my_idx = res;
        }
        if (sv < N) st_idx(idx, it, sv, my_idx);
        if constexpr (LT > 0) {
            if (kx.k_hat != nullptr) {   // block-uniform
                float c[8];
                const int ci = my_idx < nc ? my_idx : nc - 1;
#pragma unroll
                for (int e = 0; e < 8; ++e) c[e] = e < SUB ? s_cb[ci * SUB + e] : 0.f;
                wht_lanes<SUB, LT>(c, lane);
#pragma unroll
                for (int e = 0; e < SUB; ++e) c[e] = c[e] * kx.h * sm[e];
                if (sv < N) {
                    if (kx.hat_dtype == VQ_F32) {
#pragma unroll
                        for (int e = 0; e < SUB; e += 4)
                            *reinterpret_cast<float4 *>((float *)kx.k_hat + sv * SUB + e) = make_float4(c[e], c[e + 1], c[e + 2], c[e + 3]);
                    } else {
                        u32 w[4];
#pragma unroll
                        for (int e = 0; e < SUB; e += 2) {
                            if (kx.hat_dtype == VQ_F16) w[e / 2] = __builtin_bit_cast(u32, f16x2{(f16)c[e], (f16)c[e + 1]});
                            else w[e / 2] = (u32)f32_to_bf16(c[e]) | ((u32)f32_to_bf16(c[e + 1]) << 16);
                        }
                        if constexpr (SUB == 8) *reinterpret_cast<uint4 *>((u16 *)kx.k_hat + sv * 8) = make_uint4(w[0], w[1], w[2], w[3]);
                        else *reinterpret_cast<uint2 *>((u16 *)kx.k_hat + sv * 4) = make_uint2(w[0], w[1]);
                    }
                }
            }
        }
        raw = raw_next;
        __builtin_amdgcn_wave_barrier();   // the next step overwrites this wave's LDS slots
    }
}

bool launch_assign_mfma(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, int sub, void *idx, int it,
                        hipStream_t st) {
    if (nc > VM_MAXC || !(sub == 4 || sub == 8)) return false;
    if (xt != VQ_F32 && sub == 8 && ((uintptr_t)x & 15u)) return false;
    int64_t blocks = cdiv(cdiv(N, 64), 4);
    if (blocks > 512) blocks = 512;   // two resident blocks per compute unit
    if (blocks < 1) blocks = 1;
    const KeyXform none = {};
    if (sub == 8)
        hipLaunchKernelGGL((vq_assign_mfma_kernel<8, 0>), dim3((unsigned)blocks), dim3(256), 0, st, x, xt, N, cb, ct, nc, idx, it, none);
    else
        hipLaunchKernelGGL((vq_assign_mfma_kernel<4, 0>), dim3((unsigned)blocks), dim3(256), 0, st, x, xt, N, cb, ct, nc, idx, it, none);
    return true;
}

bool launch_encode_keys_mfma(const void *keys, int kt, int64_t B, int64_t heads, int64_t S, int64_t D, const float *smooth,
                             int smooth_rows, float h, const void *cb, int ct, int nc, int sub, void *idx, int it, void *k_hat,
                             float *k_tilde, hipStream_t st) {
    if (nc > VM_MAXC || !(sub == 4 || sub == 8) || D % sub != 0) return false;
    const int64_t lt = D / sub;
    if (!(lt == 8 || lt == 16 || lt == 32 || lt == 64)) return false;
    if (((uintptr_t)keys | (uintptr_t)k_hat | (uintptr_t)k_tilde | (uintptr_t)smooth) & 15u) return false;
    const int64_t N = B * heads * S * lt;
    int64_t blocks = cdiv(cdiv(N, 64), 4);
    if (blocks > 512) blocks = 512;
    if (blocks < 1) blocks = 1;
    const KeyXform kx = {smooth, smooth_rows, heads, S, h, k_hat, kt, k_tilde};
#define VQ_ENC(SUB, LT) hipLaunchKernelGGL((vq_assign_mfma_kernel<SUB, LT>), dim3((unsigned)blocks), dim3(256), 0, st, keys, kt, N, cb, ct, nc, idx, it, kx)
    if (sub == 8) { if (lt == 8) VQ_ENC(8, 8); else if (lt == 16) VQ_ENC(8, 16); else if (lt == 32) VQ_ENC(8, 32); else VQ_ENC(8, 64); }
    else { if (lt == 8) VQ_ENC(4, 8); else if (lt == 16) VQ_ENC(4, 16); else if (lt == 32) VQ_ENC(4, 32); else VQ_ENC(4, 64); }
#undef VQ_ENC
    return true;
}

}  // namespace vq
