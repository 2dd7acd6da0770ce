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
//   per lane and column the two smallest t are tracked at 2.5 vector operations a score: the
//   position of the score (centroid tile, accumulator register) replaces its low mantissa bits
//   (one and-or), and a PAIR of new keys a, b updates the sorted pair k1 <= k2 in three:
//   m = med3(k1, a, b), k1 = min3(k1, a, b), k2 = min(k2, m);
//   if second - first > eps (eps = 2^-14 (|v|^2 + max|c|^2): four times what the six replaced
//   mantissa bits can move a score, far above filter error and the rounding of the exact
//   rule) the first is the answer;
//   otherwise, if the two leaders come from different trackers (lanes) and no other tracked
//   score lies within eps, the exact rule decides between the two; in the remaining (rare) case
//   the column's scores are recomputed and every centroid with t <= first + eps is evaluated with
//   the exact rule, lowest index winning ties.
//
// The codebook lives in LDS as ready-made operand tiles (16 or 32 bytes a centroid, |c|^2
// beside them), 4096 centroids of four dimensions or 2048 of eight at most; a wave keeps 64
// sub-vectors in registers as four B operands and walks the tiles, four products and forty
// tracking operations a tile.  Sixteen waves to a CU (four per SIMD, 128 registers each): the
// loop is bound by vector issue, which one or two waves a SIMD do not fill.
#include <atomic>

#include "vecinfer.hpp"

namespace vq {

typedef uint32_t u32;

constexpr int VM_MAXC = 4096;

// Bare min / median-of-three: the scores are never NaN, so the canonicalising moves the
// compiler wraps around fminf would only cost issue slots in the hottest loop.
__device__ __forceinline__ float vmin(float a, float b) {
    float d;
    asm("v_min_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float vmax(float a, float b) {
    float d;
    asm("v_max_f32 %0, %1, %2" : "=v"(d) : "v"(a), "v"(b));
    return d;
}
__device__ __forceinline__ float vmin3(float a, float b, float c) {
    float d;
    asm("v_min3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
__device__ __forceinline__ float vmed3(float a, float b, float c) {
    float d;
    asm("v_med3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}
// two new keys into the sorted pair k1 <= k2
__device__ __forceinline__ void track2(float &k1, float &k2, float a, float b) {
    const float m = vmed3(k1, a, b);
    k1 = vmin3(k1, a, b);
    k2 = vmin(k2, m);
}
// a score with its low six mantissa bits replaced by `tag` (0..63 once the tile loop is unrolled: mask and
// tag are inline constants of one v_and_or_b32)
__device__ __forceinline__ float tagged(float d, int tag) {
    return __uint_as_float((__float_as_uint(d) & 0xFFFFFFC0u) | (u32)tag);
}
// the exact rule against centroid c: from the operand image when the codebook is 16-bit (its high parts are the
// centroid itself, times -2), from memory when it is float32
template <int SUB>
__device__ __forceinline__ float exact_dist_c(const float *x, const char *tiles, const void *cb, int ct, int c) {
    float cv[SUB];
    if (ct != VQ_F32) {
        const f16 *img = reinterpret_cast<const f16 *>(tiles + (size_t)c * (4 * SUB));
#pragma unroll
        for (int i = 0; i < SUB; ++i) cv[i] = (float)img[i] * -0.5f;
    } else {
#pragma unroll
        for (int i = 0; i < SUB; ++i) cv[i] = ((const float *)cb)[(int64_t)c * SUB + i];
    }
    float dist = 0.0f;
#pragma unroll
    for (int i = 0; i < SUB; ++i) {
        const float d = __fsub_rn(x[i], cv[i]);
        dist = __fadd_rn(dist, __fmul_rn(d, d));
    }
    return dist;
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


// bytes of one centroid's operand image: fp16 high parts, then fp16 remainders, of -2 c
template <int SUB> constexpr int cent_bytes() { return 4 * SUB; }

// dynamic LDS: [operand tiles: nc16 * cent_bytes][|c|^2: nc16 floats][per wave: 64 x 16 halves, 64 x 8 floats]
template <int SUB, int LT, int WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(4, 4)))
void vq_assign_mfma_kernel(const void *__restrict__ x, int xt, int64_t N, const void *__restrict__ cb, int ct, int nc,
                           void *__restrict__ idx, int it, KeyXform kx) {
    extern __shared__ __align__(16) char s_dyn[];
    __shared__ float s_red[WAVES];
    constexpr int CB = cent_bytes<SUB>();
    const int ntiles = (nc + 63) / 64 * 4, nc16 = 16 * ntiles;   // whole groups of four tiles (padded with centroids never chosen)
    char *s_tiles = s_dyn;
    float *s_c2 = reinterpret_cast<float *>(s_dyn + (size_t)nc16 * CB);
    char *s_stage = reinterpret_cast<char *>(s_c2 + nc16);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, blk = lane >> 4;
    f16 (*s_xh)[16] = reinterpret_cast<f16 (*)[16]>(s_stage + wave * 4096);          // [64][high 8 | remainder 8]
    float (*s_xf)[8] = reinterpret_cast<float (*)[8]>(s_stage + wave * 4096 + 2048);   // [64][8] float32 (exact rule)

    // ---- the codebook as operand tiles: thread c splits centroid c (one or two vector loads a row when the
    // codebook is 16-byte aligned, element by element otherwise)
    float cmax2 = 0.f;
    const bool cb_aligned = (reinterpret_cast<uintptr_t>(cb) & 15u) == 0;
    for (int c = tid; c < nc16; c += 64 * WAVES) {
        float row[SUB];
        float c2 = 3.0e38f;   // past the end: never the nearest
        if (c < nc) {
            if (!cb_aligned) {
#pragma unroll
                for (int e = 0; e < SUB; ++e) row[e] = ld_any(cb, ct, (int64_t)c * SUB + e);
            } else if (ct == VQ_F32) {
#pragma unroll
                for (int e = 0; e < SUB; e += 4) {
                    const float4 v = *reinterpret_cast<const float4 *>((const float *)cb + (int64_t)c * SUB + e);
                    row[e] = v.x; row[e + 1] = v.y; row[e + 2] = v.z; row[e + 3] = v.w;
                }
            } else {
                u32 w[SUB / 2];
                if constexpr (SUB == 8) {
                    const uint4 v = *reinterpret_cast<const uint4 *>((const u16 *)cb + (int64_t)c * 8);
                    w[0] = v.x; w[1] = v.y; w[2] = v.z; w[3] = v.w;
                } else {
                    const uint2 v = *reinterpret_cast<const uint2 *>((const u16 *)cb + (int64_t)c * 4);
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
            c2 = 0.f;
#pragma unroll
            for (int e = 0; e < SUB; ++e) c2 += row[e] * row[e];
            cmax2 = fmaxf(cmax2, c2);
        } else {
#pragma unroll
            for (int e = 0; e < SUB; ++e) row[e] = 0.f;
        }
        f16 *img = reinterpret_cast<f16 *>(s_tiles + (size_t)c * CB);
#pragma unroll
        for (int e = 0; e < SUB; ++e) {
            const f16 hi = (f16)row[e];
            const f16 lo = (f16)(row[e] - (float)hi);
            img[e] = (f16)(-2.f) * hi;
            img[SUB + e] = (f16)(-2.f) * lo;
        }
        s_c2[c] = c2;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) cmax2 = fmaxf(cmax2, __shfl_xor(cmax2, o));
    if (lane == 0) s_red[wave] = cmax2;
    __syncthreads();
    cmax2 = s_red[0];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) cmax2 = fmaxf(cmax2, s_red[w]);

    // what a lane reads of a tile.  SUB 8: lane groups 0, 1 the high parts, 2, 3 the remainders of centroid n
    // (the sub-vector side alternates high part / remainder: all four cross terms).  SUB 4: every lane group
    // the 16 bytes [high 4 | remainder 4] of centroid n; the sub-vector side carries [high | high] in lane
    // group 0, [remainder | remainder] in group 1 and zeros in groups 2, 3.
    const int a_off = SUB == 8 ? n * 32 + (blk >> 1) * 16 : n * 16;
    const int c_off = 16 * blk;                       // |c|^2 of centroids 4 blk .. 4 blk + 3 of the tile
    const bool multi = ntiles > 16;                   // more than one chunk of 256 centroids

    const int64_t n_steps = (N + 63) / 64;
    const int64_t stride = (int64_t)gridDim.x * WAVES;
    const bool packed16 = SUB == 8 && xt != VQ_F32;   // one 16-byte load per sub-vector, fetched a step ahead
    const bool packed8 = SUB == 4 && xt != VQ_F32;
    auto load_raw = [&](int64_t step) {
        const int64_t sv = step * 64 + lane;
        uint4 r = make_uint4(0, 0, 0, 0);
        if (step < n_steps && sv < N) {
            if (packed16) r = *reinterpret_cast<const uint4 *>((const u16 *)x + sv * 8);
            else if (packed8) { const uint2 t = *reinterpret_cast<const uint2 *>((const u16 *)x + sv * 4); r.x = t.x; r.y = t.y; }
        }
        return r;
    };
    uint4 raw = load_raw((int64_t)blockIdx.x * WAVES + wave);
    for (int64_t step = (int64_t)blockIdx.x * WAVES + wave; step < n_steps; step += stride) {
        const int64_t sv = step * 64 + lane;   // this lane's sub-vector
        const uint4 raw_next = load_raw(step + stride);
        // ---- convert, split, bounce through LDS
        float xf[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) xf[e] = 0.f;
        if (packed16 || packed8) {
            const u32 w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
            for (int e = 0; e < SUB / 2; ++e) {
                if (xt == VQ_F16) {
                    const f16x2 h = __builtin_bit_cast(f16x2, w[e]);
                    xf[2 * e] = (float)h[0]; xf[2 * e + 1] = (float)h[1];
                } else {
                    xf[2 * e] = __uint_as_float(w[e] << 16); xf[2 * e + 1] = __uint_as_float(w[e] & 0xffff0000u);
                }
            }
        } else {
#pragma unroll
            for (int e = 0; e < SUB; ++e) xf[e] = sv < N ? ld_any(x, xt, sv * SUB + e) : 0.f;
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
        float x2 = 0.f;   // |v|^2 for the margin only: fused multiply-adds will do
#pragma unroll
        for (int e = 0; e < 8; ++e) x2 = __builtin_fmaf(xf[e], xf[e], x2);
        if (LT == 0 && packed16 && xt == VQ_F16) {
            // fp16 sub-vectors as they came: they are their own high part, the remainder is zero
            xh = __builtin_bit_cast(f16x8, raw);
            xl = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                xh[e] = (f16)xf[e];
                xl[e] = (f16)(xf[e] - (float)xh[e]);
            }
        }
        if constexpr (SUB == 4) {   // [high | high] and [remainder | remainder]
#pragma unroll
            for (int e = 0; e < 4; ++e) { xh[4 + e] = xh[e]; xl[4 + e] = xl[e]; }
        }
        auto stage = [&]() {   // the lane's sub-vector into the wave's staging rows
            *reinterpret_cast<f16x8 *>(&s_xh[lane][0]) = xh;
            *reinterpret_cast<f16x8 *>(&s_xh[lane][8]) = xl;
            *reinterpret_cast<float4 *>(&s_xf[lane][0]) = make_float4(xf[0], xf[1], xf[2], xf[3]);
            *reinterpret_cast<float4 *>(&s_xf[lane][4]) = make_float4(xf[4], xf[5], xf[6], xf[7]);
            // the wave reads what its own lanes wrote: LDS serves a wave's requests in order
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        };
        stage();

        // B operands of the four column groups: sub-vector 16 t + n
        f16x8 B[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            B[t] = *reinterpret_cast<const f16x8 *>(&s_xh[16 * t + n][8 * (blk & 1)]);
            if (SUB == 4 && blk >= 2) B[t] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        }
        // the lane's sorted pair of every column group, over all chunks: key and chunk number
        float K1[4], K2[4];
        int Q1[4], Q2[4];
#pragma unroll
        for (int t = 0; t < 4; ++t) { K1[t] = INFINITY; K2[t] = INFINITY; Q1[t] = 0; Q2[t] = 0; }

#pragma unroll 1
        for (int t0 = 0; t0 < ntiles; t0 += 16) {
            // two sorted pairs a lane and column group: accumulator registers 0, 1 feed one, 2, 3 the other (twice
            // the trackers at the same cost: the leaders of a column less often share one)
            float k1[4], k2[4], m1[4], m2[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) { k1[t] = INFINITY; k2[t] = INFINITY; m1[t] = INFINITY; m2[t] = INFINITY; }
            const char *tp = s_tiles + (size_t)t0 * 16 * CB + a_off;
            const char *cp = reinterpret_cast<const char *>(s_c2 + t0 * 16) + c_off;
            const int left = ntiles - t0;   // tiles of this chunk (tiles past the codebook's end do not exist in LDS)
#pragma unroll
            for (int j4 = 0; j4 < 16; j4 += 4) {
                if (j4 < left) {
#pragma unroll
                    for (int j = j4; j < j4 + 4; ++j) {
                        const f16x8 A = *reinterpret_cast<const f16x8 *>(tp + j * 16 * CB);
                        const float4 c4 = *reinterpret_cast<const float4 *>(cp + j * 64);
                        const f32x4 C = {c4.x, c4.y, c4.z, c4.w};
                        f32x4 D[4];
#pragma unroll
                        for (int t = 0; t < 4; ++t) D[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, B[t], C, 0, 0, 0);
#pragma unroll
                        for (int t = 0; t < 4; ++t) {
                            track2(k1[t], k2[t], tagged(D[t][0], 4 * j), tagged(D[t][1], 4 * j + 1));
                            track2(m1[t], m2[t], tagged(D[t][2], 4 * j + 2), tagged(D[t][3], 4 * j + 3));
                        }
                    }
                }
            }
            // fold the chunk into the lane's pair (an earlier chunk keeps its place on equal keys)
            const int q = t0 >> 4;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                {   // the lane's two pairs into one (keys are distinct: they carry their register)
                    const float hi = vmax(k1[t], m1[t]);
                    k1[t] = vmin(k1[t], m1[t]);
                    k2[t] = vmin3(hi, k2[t], m2[t]);
                }
                if (!multi) { K1[t] = k1[t]; K2[t] = k2[t]; continue; }
                const bool first = k1[t] < K1[t];
                const float o1 = K1[t], o2 = K2[t];
                const int p1 = Q1[t], p2 = Q2[t];
                K1[t] = first ? k1[t] : o1;
                Q1[t] = first ? q : p1;
                // the second: of (old first, new second) when the new first leads, else of (old second, new first)
                const float sa = first ? o1 : o2, sb = first ? k2[t] : k1[t];
                const int pa = first ? p1 : p2;
                const bool keep = !(sb < sa);
                K2[t] = keep ? sa : sb;
                Q2[t] = keep ? pa : q;
            }
        }

        // ---- the pairs change hands through the staging rows (whose sub-vectors sit in registers as well): lane
        // (n, blk) collects the four lanes' pairs of column group blk -- the group its own sub-vector 16 blk + n
        // belongs to -- and decides that one column by itself: one decision a lane instead of four.
        __builtin_amdgcn_wave_barrier();   // every B operand has been read
        {
            uint4 *ex = reinterpret_cast<uint4 *>(s_stage + wave * 4096);   // [group][n][source lane group]
#pragma unroll
            for (int t = 0; t < 4; ++t)
                ex[(t * 16 + n) * 4 + blk] = make_uint4(__float_as_uint(K1[t]), __float_as_uint(K2[t]), (u32)Q1[t], (u32)Q2[t]);
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // smallest three of the eight tracked scores of the column, the first two with their origin (source lane
        // group, chunk); equal keys of different origins are different centroids: the earlier source comes first
        float f1 = INFINITY, f2 = INFINITY, g3 = INFINITY;
        int o1 = 0, o2 = 0;
        {
            const uint4 *ex = reinterpret_cast<const uint4 *>(s_stage + wave * 4096) + (blk * 16 + n) * 4;
#pragma unroll
            for (int src = 0; src < 4; ++src) {
                const uint4 e = ex[src];
                const float a[2] = {__uint_as_float(e.x), __uint_as_float(e.y)};
                const int q[2] = {(int)e.z * 4 + src, (int)e.w * 4 + src};
#pragma unroll
                for (int k = 0; k < 2; ++k) {   // insert a[k] into the sorted triple
                    const bool b1 = a[k] < f1, b2 = a[k] < f2;
                    g3 = b2 ? f2 : vmin(g3, a[k]);
                    f2 = b1 ? f1 : (b2 ? a[k] : f2);
                    o2 = b1 ? o1 : (b2 ? q[k] : o2);
                    f1 = b1 ? a[k] : f1;
                    o1 = b1 ? q[k] : o1;
                }
            }
        }
        const float eps = 6.103515625e-05f * (x2 + cmax2);   // 2^-14 (|v|^2 + max |c|^2)
        // centroid of a key: chunk * 256 + 16 * tile + 4 * lane group + register
        auto centroid = [&](float key, int org) {
            const u32 b = __float_as_uint(key) & 63u;
            return (org >> 2) * 256 + (int)((b >> 2) * 16u + (u32)(org & 3) * 4u + (b & 3u));
        };
        const int i1 = centroid(f1, o1), i2 = centroid(f2, o2);
        int my_idx = i1;
        const bool unsure = !(f2 - f1 > eps);
        if (__any(unsure)) {
            // Whatever a lane dropped (inside a tracker, or when its trackers and chunks were merged into one pair)
            // is at least that lane's second entry, so when the leading two come from different lanes nothing
            // untracked lies below g3, the third smallest tracked score.
            const bool other_lane = ((o1 ^ o2) & 3) != 0;
            const bool two = unsure && other_lane && (g3 - f1 > eps) && i1 < nc && i2 < nc;
            if (two) {   // exactly two contenders: the exact rule on both
                const float d1 = exact_dist_c<SUB>(xf, s_tiles, cb, ct, i1), d2 = exact_dist_c<SUB>(xf, s_tiles, cb, ct, i2);
                my_idx = (d2 < d1 || (d2 == d1 && i2 < i1)) ? i2 : i1;
            }
            const bool many = unsure && !two;
            const unsigned long long many_mask = __ballot(many);
            if (many_mask != 0) {
                // Recompute the scores of every such column and apply the exact rule to every centroid the filter
                // cannot exclude: the four lanes of a column work together again, so the sub-vectors go back into
                // the staging rows first.  A tile without such a centroid (nearly all) costs one product and four
                // compares.
                __builtin_amdgcn_wave_barrier();   // the exchanged pairs have been read
                stage();
                const float thr_own = f1 + eps;
#pragma unroll 1
                for (int t = 0; t < 4; ++t) {
                    if (((many_mask >> (16 * t)) & 0xFFFFull) == 0) continue;
                    const bool col = ((many_mask >> (16 * t + n)) & 1ull) != 0;   // this lane's column of group t
                    const float thr = __shfl(thr_own, 16 * t + n);
                    const float *xv = &s_xf[16 * t + n][0];
                    const f16x8 Bt = *reinterpret_cast<const f16x8 *>(&s_xh[16 * t + n][8 * (blk & 1)]);
                    const f16x8 Bz = (SUB == 4 && blk >= 2) ? f16x8{0, 0, 0, 0, 0, 0, 0, 0} : Bt;
                    float dbest = INFINITY;
                    int ibest = 0x7fffffff;
#pragma unroll 1
                    for (int j = 0; j < ntiles; ++j) {
                        const f16x8 A = *reinterpret_cast<const f16x8 *>(s_tiles + (size_t)j * 16 * CB + a_off);
                        const float4 c4 = *reinterpret_cast<const float4 *>(reinterpret_cast<const char *>(s_c2 + j * 16) + c_off);
                        const f32x4 D = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, Bz, f32x4{c4.x, c4.y, c4.z, c4.w}, 0, 0, 0);
                        const int c0 = 16 * j + 4 * blk;
                        const bool h0 = col && c0 < nc && D[0] <= thr, h1 = col && c0 + 1 < nc && D[1] <= thr;
                        const bool h2 = col && c0 + 2 < nc && D[2] <= thr, h3 = col && c0 + 3 < nc && D[3] <= thr;
                        if (!__any(h0 || h1 || h2 || h3)) continue;
#pragma unroll
                        for (int r = 0; r < 4; ++r) {
                            const bool h = r == 0 ? h0 : r == 1 ? h1 : r == 2 ? h2 : h3;
                            if (h) {
                                const float d = exact_dist_c<SUB>(xv, s_tiles, cb, ct, c0 + r);
                                if (d < dbest || (d == dbest && c0 + r < ibest)) { dbest = d; ibest = c0 + r; }
                            }
                        }
                    }
#pragma unroll
                    for (int o = 16; o <= 32; o <<= 1) {
                        const float d = __shfl_xor(dbest, o);
                        const int ci = __shfl_xor(ibest, o);
                        if (d < dbest || (d == dbest && ci < ibest)) { dbest = d; ibest = ci; }
                    }
                    if (blk == t && many) my_idx = ibest;
                }
            }
        }
        if (sv < N) st_idx(idx, it, sv, my_idx);
        if constexpr (LT > 0) {
            if (kx.k_hat != nullptr) {   // block-uniform
                float c[8];
                const int ci = my_idx < nc ? my_idx : nc - 1;
#pragma unroll
                for (int e = 0; e < 8; ++e) c[e] = e < SUB ? ld_any(cb, ct, (int64_t)ci * SUB + e) : 0.f;
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

// ---- launch: sixteen waves to a CU, as two blocks of eight or, when the codebook image is large, one of sixteen
template <int SUB, int LT, int WAVES>
static void launch_tiles_waves(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, void *idx, int it,
                               const KeyXform &kx, size_t image, int blocks_per_cu, hipStream_t st) {
    auto kernel = vq_assign_mfma_kernel<SUB, LT, WAVES>;
    // more than 64 KB of block-shared memory has to be allowed per kernel and device, once (a second
    // thread that gets here first repeats the same call)
    static std::atomic<bool> allowed[64] = {};
    int dev = 0;
    (void)hipGetDevice(&dev);
    if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {
        (void)hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024 - 256);
        if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);
    }
    int64_t blocks = cdiv(cdiv(N, 64), WAVES);
    if (blocks > 256 * blocks_per_cu) blocks = 256 * blocks_per_cu;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(kernel, dim3((unsigned)blocks), dim3(64 * WAVES), image + (size_t)WAVES * 4096, st, x, xt, N, cb, ct, nc,
                       idx, it, kx);
}

template <int SUB, int LT>
static bool launch_tiles(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, void *idx, int it, const KeyXform &kx,
                         hipStream_t st) {
    const int nc16 = (nc + 63) / 64 * 64;
    const size_t image = (size_t)nc16 * (cent_bytes<SUB>() + 4);
    if (image + 8 * 4096 <= 78 * 1024) launch_tiles_waves<SUB, LT, 8>(x, xt, N, cb, ct, nc, idx, it, kx, image, 2, st);
    else if (image + 16 * 4096 <= 159 * 1024) launch_tiles_waves<SUB, LT, 16>(x, xt, N, cb, ct, nc, idx, it, kx, image, 1, st);
    else return false;
    return true;
}

bool launch_assign_mfma(const void *x, int xt, int64_t N, const void *cb, int ct, int nc, int sub, void *idx, int it,
                        hipStream_t st) {
    if (nc > VM_MAXC || !(sub == 4 || sub == 8)) return false;
    if (xt != VQ_F32 && ((uintptr_t)x & (sub == 8 ? 15u : 7u))) return false;
    const KeyXform none = {};
    return sub == 8 ? launch_tiles<8, 0>(x, xt, N, cb, ct, nc, idx, it, none, st)
                    : launch_tiles<4, 0>(x, xt, N, cb, ct, nc, idx, it, none, st);
}

bool launch_encode_keys_mfma(const void *keys, int kt, int64_t B, int64_t heads, int64_t S, int64_t D, const float *smooth,
                             int smooth_rows, float h, const void *cb, int ct, int nc, int sub, void *idx, int it, void *k_hat,
                             float *k_tilde, hipStream_t st) {
    if (nc > VM_MAXC || !(sub == 4 || sub == 8) || D % sub != 0) return false;
    const int64_t lt = D / sub;
    if (!(lt == 8 || lt == 16 || lt == 32 || lt == 64)) return false;
    if (((uintptr_t)keys | (uintptr_t)k_hat | (uintptr_t)k_tilde | (uintptr_t)smooth) & 15u) return false;
    const int64_t N = B * heads * S * lt;
    const KeyXform kx = {smooth, smooth_rows, heads, S, h, k_hat, kt, k_tilde};
#define VQ_ENC(SUB, LT) return launch_tiles<SUB, LT>(keys, kt, N, cb, ct, nc, idx, it, kx, st)
    if (sub == 8) { if (lt == 8) VQ_ENC(8, 8); else if (lt == 16) VQ_ENC(8, 16); else if (lt == 32) VQ_ENC(8, 32); else VQ_ENC(8, 64); }
    else { if (lt == 8) VQ_ENC(4, 8); else if (lt == 16) VQ_ENC(4, 16); else if (lt == 32) VQ_ENC(4, 32); else VQ_ENC(4, 64); }
#undef VQ_ENC
}

}  // namespace vq
