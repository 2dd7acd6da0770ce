// MFMA decode attention over a packed KIVI cache (gfx950, wave64).
//
// One block of four waves per (kv head, token split).  Every wave streams units
// of 32 tokens: codes are unpacked in registers straight into fp16 MFMA operands
// (the code lands in the mantissa of a constant whose value is then removed
// exactly, followed by one packed fp16 fma with the group's scale and zero), so
// no reconstructed K or V ever touches LDS or HBM.
//
//   S^T[token, row] = K_hat[token, :] . q[row, :]   v_mfma_f32_16x16x32_f16, A = K_hat, B = q
//   O[row, chan]   += P[row, token] * V_hat[token, chan]              A = P,     B = V_hat
//
// Query rows (the H_q/H_kv heads that share the kv head) sit in the 16-wide M/N
// dimension.  Keys are packed along channels, so a lane's eight K-slots of the
// first product are eight channels of one token; values are packed along tokens
// (VQ_V_TOKEN_PACKED), so a lane's eight K-slots of the second product are eight
// tokens of one channel -- both operands come out of one 32-bit word with no
// transposition.  MFMA sums over its K index, so any assignment of channels
// (tokens) to K-slots is valid as long as A and B agree; the assignments below
// are chosen so that the accumulator layout of S^T is already the A-operand
// layout of P.
//
// Keys carry outlier channels, and rounding a reconstructed key to fp16 costs
// more than the 2e-3 output tolerance allows.  The key product is therefore
// taken on the exact integer codes with the per-channel scale folded into the
// query:  q.k_hat = sum_d (q_d s_d) c_d + sum_d q_d z_d.  The folded query q_d s_d
// is carried as an fp16 high part plus an exact fp16 remainder in spare
// columns of the same MFMA (rows [R, 2R) of the 16-wide tile), so the product
// is as accurate as a float32 one; the zero-point term is one dot product per
// (row, token group).  Values have no such outliers and are reconstructed to
// fp16 in registers.
//
// The softmax denominator is produced by the matrix unit as a ninth output tile
// against a constant ones operand, from the same fp16-rounded P that multiplies
// V_hat, so rounding of P cancels in the normalisation.
//
// The un-quantised fp16 tail is handled by one extra block per kv head that runs
// the same two products on plain rows; every block writes (max, sum, accumulator)
// partials that the shared merge kernel combines.
#include "attend.hpp"

namespace vq {

typedef uint32_t u32;

__device__ __forceinline__ f16x2 as_h2(u32 u) { return __builtin_bit_cast(f16x2, u); }
__device__ __forceinline__ u32 as_u32(f16x2 h) { return __builtin_bit_cast(u32, h); }
__device__ __forceinline__ f16x2 h2(float a) { f16x2 r = {(f16)a, (f16)a}; return r; }

// Take the two codes selected by `mask` (one per 16-bit half), place them in the
// mantissa of `magic`, remove the constant exactly and apply scale / zero.
__device__ __forceinline__ f16x2 deq2(u32 w, u32 mask, u32 magic, f16x2 off, f16x2 s, f16x2 z) {
    f16x2 v = as_h2((w & mask) | magic) - off;
    return __builtin_elementwise_fma(v, s, z);
}

// Four code pairs (eight fp16 values, one MFMA operand) from one packed word.
// BITS == 4: the word holds codes 0..7, pair p = (code p, code p + 4).
// BITS == 2: the word holds codes 0..15 and `half` picks pairs
//            (4*half + p, 4*half + p + 8), p = 0..3.
template <int BITS>
__device__ __forceinline__ f16x8 unpack8(u32 w, int half, const f16x2 (&s)[4], const f16x2 (&z)[4]) {
    f16x2 r[4];
    if (BITS == 4) {
        u32 w8 = w >> 8;
        r[0] = deq2(w, 0x000F000Fu, 0x64006400u, h2(1024.f), s[0], z[0]);
        r[1] = deq2(w, 0x00F000F0u, 0x54005400u, h2(64.f), s[1], z[1]);
        r[2] = deq2(w8, 0x000F000Fu, 0x64006400u, h2(1024.f), s[2], z[2]);
        r[3] = deq2(w8, 0x00F000F0u, 0x54005400u, h2(64.f), s[3], z[3]);
    } else {
        u32 ws = w >> (8 * half);
        r[0] = deq2(ws, 0x00030003u, 0x64006400u, h2(1024.f), s[0], z[0]);
        r[1] = deq2(ws, 0x000C000Cu, 0x5C005C00u, h2(256.f), s[1], z[1]);
        r[2] = deq2(ws, 0x00300030u, 0x54005400u, h2(64.f), s[2], z[2]);
        r[3] = deq2(ws, 0x00C000C0u, 0x4C004C00u, h2(16.f), s[3], z[3]);
    }
    f16x8 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) { o[2 * p] = r[p][0]; o[2 * p + 1] = r[p][1]; }
    return o;
}

// The same eight codes as exact small integers (no scale / zero applied).
__device__ __forceinline__ f16x2 code2(u32 w, u32 mask, u32 magic, f16x2 off) {
    return as_h2((w & mask) | magic) - off;
}
template <int BITS> __device__ __forceinline__ f16x8 unpack8_codes(u32 w, int half) {
    f16x2 r[4];
    if (BITS == 4) {
        u32 w8 = w >> 8;
        r[0] = code2(w, 0x000F000Fu, 0x64006400u, h2(1024.f));
        r[1] = code2(w, 0x00F000F0u, 0x54005400u, h2(64.f));
        r[2] = code2(w8, 0x000F000Fu, 0x64006400u, h2(1024.f));
        r[3] = code2(w8, 0x00F000F0u, 0x54005400u, h2(64.f));
    } else {
        u32 ws = w >> (8 * half);
        r[0] = code2(ws, 0x00030003u, 0x64006400u, h2(1024.f));
        r[1] = code2(ws, 0x000C000Cu, 0x5C005C00u, h2(256.f));
        r[2] = code2(ws, 0x00300030u, 0x54005400u, h2(64.f));
        r[3] = code2(ws, 0x00C000C0u, 0x4C004C00u, h2(16.f));
    }
    f16x8 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) { o[2 * p] = r[p][0]; o[2 * p + 1] = r[p][1]; }
    return o;
}

// channel (0..31 inside a lane's 32-channel slice) of K-slot pair p of k-step ks
template <int BITS> __device__ __forceinline__ constexpr int kchan_lo(int ks, int p) {
    return BITS == 4 ? 8 * ks + p : 16 * (ks / 2) + 4 * (ks % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int kchan_hi(int ks, int p) {
    return kchan_lo<BITS>(ks, p) + (BITS == 4 ? 4 : 8);
}
// token (0..31 inside a unit) of K-slot pair p of lane group blk in the P.V product
template <int BITS> __device__ __forceinline__ int vtok_lo(int blk, int p) {
    return BITS == 4 ? 8 * blk + p : 16 * (blk / 2) + 4 * (blk % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int vtok_gap() { return BITS == 4 ? 4 : 8; }

__device__ __forceinline__ float ldq(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}

template <typename M> struct MetaLd;
template <> struct MetaLd<f16> {
    // four consecutive values as two fp16 pairs
    static __device__ __forceinline__ void ld4(const f16 *p, f16 (&o)[4]) {
        uint2 u = *reinterpret_cast<const uint2 *>(p);
        f16x2 a = as_h2(u.x), b = as_h2(u.y);
        o[0] = a[0]; o[1] = a[1]; o[2] = b[0]; o[3] = b[1];
    }
    static __device__ __forceinline__ void ld4f(const f16 *p, float (&o)[4]) {
        f16 t[4];
        ld4(p, t);
        o[0] = (float)t[0]; o[1] = (float)t[1]; o[2] = (float)t[2]; o[3] = (float)t[3];
    }
};
template <> struct MetaLd<float> {
    static __device__ __forceinline__ void ld4(const float *p, f16 (&o)[4]) {
        float4 u = *reinterpret_cast<const float4 *>(p);
        o[0] = (f16)u.x; o[1] = (f16)u.y; o[2] = (f16)u.z; o[3] = (f16)u.w;
    }
    static __device__ __forceinline__ void ld4f(const float *p, float (&o)[4]) {
        float4 u = *reinterpret_cast<const float4 *>(p);
        o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
    }
};

constexpr int MF_ROWS = 16;               // M/N width of the MFMA: most query rows per kv head
constexpr int MF_D = 128;                 // head dim
constexpr int MF_PART = MF_D + 2;         // floats per partial: max, sum, accumulator
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;


// Online-softmax step for one unit of 32 tokens.  S holds the raw scores of this
// lane's column (query row i) for its eight tokens; rows of the output tiles are
// rescaled when the running maximum moves.  Returns P in the A-operand layout of
// the P.V product (pair r = tile 0 register r, tile 1 register r).
__device__ __forceinline__ f16x8 softmax_unit(const f32x4 (&S)[2], float c, float &m_run, f32x4 (&O)[9], int blk) {
    float mx = fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])),
                     fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx * c);
    if (__any(m_new > m_run)) {
        const float alpha = m_new == -INFINITY ? 1.f : exp2f(m_run - m_new);   // 0 on the first unit
        float al[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * blk + r);
#pragma unroll
        for (int n = 0; n < 9; ++n)
#pragma unroll
            for (int r = 0; r < 4; ++r) O[n][r] *= al[r];
        m_run = m_new;
    }
    const float mm = m_run == -INFINITY ? 0.f : m_run;   // a row with no visible token yet
    f16x8 P;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        P[2 * r] = (f16)__builtin_amdgcn_exp2f(S[0][r] * c - mm);
        P[2 * r + 1] = (f16)__builtin_amdgcn_exp2f(S[1][r] * c - mm);
    }
    return P;
}

// Value operand from one packed word with float32 scale / zero: the product is
// formed in float32 and rounded to fp16 once.
template <int BITS>
__device__ __forceinline__ f16x8 unpack8_f32meta(u32 w, int half, const float (&sa)[4], const float (&sb)[4],
                                                 const float (&za)[4], const float (&zb)[4]) {
    f16x8 cdes = unpack8_codes<BITS>(w, half);
    f16x8 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        o[2 * p] = (f16)fmaf((float)cdes[2 * p], sa[p], za[p]);
        o[2 * p + 1] = (f16)fmaf((float)cdes[2 * p + 1], sb[p], zb[p]);
    }
    return o;
}

// TAIL == false: grid (nsplit, B*Hkv), block sp covers tokens [sp*split_len, ...) of the
// packed prefix.  TAIL == true: grid (1, B*Hkv), the block covers the fp16 tail and writes
// partial number nsplit.  Two instantiations keep the register budget of each path apart.
template <int BITS, typename M, bool TAIL>
__global__ __launch_bounds__(256) void attend_mfma_decode_kernel(vq_attend_args a, int nsplit, int64_t split_len,
                                                                 int nparts, float *__restrict__ ws) {
    constexpr int PER = 32 / BITS;           // codes per word
    constexpr int KW = MF_D / PER;           // key words per token row
    constexpr int KWL = KW / 4;              // key words one lane loads per token (its 32 channels)
    __shared__ float s_m[4][MF_ROWS];
    __shared__ float s_l[4][MF_ROWS];
    __shared__ float s_o[4][MF_ROWS][MF_D];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i = lane & 15, blk = lane >> 4;
    const int64_t bh = blockIdx.y;
    const int sp = TAIL ? nsplit : (int)blockIdx.x;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t row0 = b * a.Hq + hkv * R;   // first query row of this kv head (Sq == 1)
    const float c = a.scale * LOG2E;

    // ---------------------------------------------------------------- packed prefix
    const int64_t t_begin = (int64_t)sp * split_len;
    int64_t t_end = t_begin + split_len;
    if (t_end > a.n_packed) t_end = a.n_packed;
    const int n_units = (int)((t_end - t_begin) / 32);

    const u32 *kp = (const u32 *)a.k_packed + bh * a.cap_tokens * KW;
    const u32 *vp = (const u32 *)a.v_packed + bh * (a.cap_tokens / PER) * MF_D;
    const int G = a.group, GV = MF_D / G;
    const int64_t GKcap = (a.cap_tokens + G - 1) / G;
    const M *ksm = (const M *)a.k_scale + bh * GKcap * MF_D + 32 * blk;
    const M *kzm = (const M *)a.k_zero + bh * GKcap * MF_D + 32 * blk;
    const M *vsm = (const M *)a.v_scale + bh * GV * a.cap_tokens;
    const M *vzm = (const M *)a.v_zero + bh * GV * a.cap_tokens;

    // Query of this lane's column: columns [0, R) carry the high part of the folded
    // query of row i, columns [R, 2R) the remainder of row i - R; the rest are zero.
    // qp: the lane's 32 channels in K-slot pair order, qn: in memory order.
    const int rq = i < R ? i : i - R;
    const bool col_used = i < 2 * R;
    f16x2 qp[16], qn[16];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            float lo = 0.f, hi = 0.f;
            if (col_used) {
                lo = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + kchan_lo<BITS>(ks, p));
                hi = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + kchan_hi<BITS>(ks, p));
            }
            qp[4 * ks + p] = f16x2{(f16)lo, (f16)hi};
        }
#pragma unroll
    for (int j = 0; j < 16; ++j) {
        float lo = 0.f, hi = 0.f;
        if (col_used) {
            lo = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + 2 * j);
            hi = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + 2 * j + 1);
        }
        qn[j] = f16x2{(f16)lo, (f16)hi};
    }
    f16x8 qB[4];
    float bias = 0.f;   // sum_d q_d z_d of row rq for the current token group
    f16x8 ones;
#pragma unroll
    for (int j = 0; j < 8; ++j) ones[j] = (f16)1.0f;

    f32x4 O[9];
#pragma unroll
    for (int n = 0; n < 9; ++n) O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;   // running max of row i (log2 domain), replicated over blk

    // token of S^T row i in tile T (see header): rows of the two tiles interleave so
    // that accumulator register r of tile T is K-slot pair r of the P.V product
    const int krow0 = vtok_lo<BITS>(i >> 2, i & 3);
    int64_t cur_group = -1;

    u32 kw[2][KWL], vw[8];
    auto load_unit = [&](int u, u32 (&kwd)[2][KWL], u32 (&vwd)[8]) {
        const int64_t base = t_begin + (int64_t)u * 32;
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const u32 *p = kp + (base + krow0 + T * vtok_gap<BITS>()) * KW + KWL * blk;
            if (BITS == 4) {
                uint4 x = *reinterpret_cast<const uint4 *>(p);
                kwd[T][0] = x.x; kwd[T][1] = x.y; kwd[T][KWL - 2] = x.z; kwd[T][KWL - 1] = x.w;
            } else {
                uint2 x = *reinterpret_cast<const uint2 *>(p);
                kwd[T][0] = x.x; kwd[T][KWL - 1] = x.y;
            }
        }
        const int64_t wrow = base / PER + (BITS == 4 ? blk : blk / 2);
        const u32 *q8 = vp + wrow * MF_D + 8 * i;
        uint4 x0 = *reinterpret_cast<const uint4 *>(q8);
        uint4 x1 = *reinterpret_cast<const uint4 *>(q8 + 4);
        vwd[0] = x0.x; vwd[1] = x0.y; vwd[2] = x0.z; vwd[3] = x0.w;
        vwd[4] = x1.x; vwd[5] = x1.y; vwd[6] = x1.z; vwd[7] = x1.w;
    };

    if constexpr (!TAIL) {
    if (wave < n_units) load_unit(wave, kw, vw);
    for (int u = wave; u < n_units; u += 4) {
        u32 kwn[2][KWL], vwn[8];
        const bool has_next = u + 4 < n_units;
        if (has_next) load_unit(u + 4, kwn, vwn);
        const int64_t base = t_begin + (int64_t)u * 32;

        // ---- new token group: fold its key scales into the query, dot its zeros with it
        const int64_t grp = base / G;
        if (grp != cur_group) {
            cur_group = grp;
            float b_part = 0.f;
            if constexpr (sizeof(M) == 2) {
                f16 sv[32];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    f16 t4[4];
                    MetaLd<M>::ld4(ksm + grp * MF_D + 4 * j, t4);
                    sv[4 * j] = t4[0]; sv[4 * j + 1] = t4[1]; sv[4 * j + 2] = t4[2]; sv[4 * j + 3] = t4[3];
                    MetaLd<M>::ld4(kzm + grp * MF_D + 4 * j, t4);
                    b_part = __builtin_amdgcn_fdot2(qn[2 * j], f16x2{t4[0], t4[1]}, b_part, false);
                    b_part = __builtin_amdgcn_fdot2(qn[2 * j + 1], f16x2{t4[2], t4[3]}, b_part, false);
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const f16x2 sp2 = f16x2{sv[kchan_lo<BITS>(ks, p)], sv[kchan_hi<BITS>(ks, p)]};
                        const f16x2 hi = qp[4 * ks + p] * sp2;
                        // q*s has at most 22 significant bits: the remainder after the fp16
                        // high part is itself an fp16 number, so this fma is exact
                        const f16x2 lo = __builtin_elementwise_fma(qp[4 * ks + p], sp2, -hi);
                        const f16x2 use = i < R ? hi : lo;
                        qB[ks][2 * p] = use[0];
                        qB[ks][2 * p + 1] = use[1];
                    }
            } else {
                float sv[32];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float t4[4];
                    MetaLd<M>::ld4f(ksm + grp * MF_D + 4 * j, t4);
                    sv[4 * j] = t4[0]; sv[4 * j + 1] = t4[1]; sv[4 * j + 2] = t4[2]; sv[4 * j + 3] = t4[3];
                    MetaLd<M>::ld4f(kzm + grp * MF_D + 4 * j, t4);
                    b_part += (float)qn[2 * j][0] * t4[0] + (float)qn[2 * j][1] * t4[1] +
                              (float)qn[2 * j + 1][0] * t4[2] + (float)qn[2 * j + 1][1] * t4[3];
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                    for (int p = 0; p < 4; ++p)
#pragma unroll
                        for (int e = 0; e < 2; ++e) {
                            const int ch = e == 0 ? kchan_lo<BITS>(ks, p) : kchan_hi<BITS>(ks, p);
                            const float t = (float)qp[4 * ks + p][e] * sv[ch];
                            const f16 hi = (f16)t;
                            const f16 lo = (f16)(t - (float)hi);
                            qB[ks][2 * p + e] = i < R ? hi : lo;
                        }
            }
            b_part += __shfl_xor(b_part, 16);
            b_part += __shfl_xor(b_part, 32);
            bias = b_part;
        }

        // ---- S^T = codes . (q s)  (two 16-token tiles, four k-steps of 32 channels)
        f32x4 S[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            S[T] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const u32 w = BITS == 4 ? kw[T][ks] : kw[T][ks / 2];
                f16x8 A = unpack8_codes<BITS>(w, ks % 2);
                S[T] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qB[ks], S[T], 0, 0, 0);
            }
        }
        // column i < R: add the remainder column i + R and the zero-point term; other columns idle
        {
            const int src = (lane & ~15) | ((i + R) & 15);
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float lo = __shfl(S[T][r], src);
                    S[T][r] = i < R ? S[T][r] + lo + bias : 0.f;
                }
        }

        // ---- online softmax for row i (this lane sees 8 of the unit's 32 tokens)
        const f16x8 P = softmax_unit(S, c, m_run, O, blk);

        // ---- value scale / zero for this lane's eight tokens, as token pairs
        const int64_t tA = base + vtok_lo<BITS>(blk, 0);
        const int64_t tB = tA + vtok_gap<BITS>();
        // ---- O += P . V_hat (eight 16-channel tiles; lane column i is channel 8*i + nt)
        // channels 8*i .. 8*i+7 lie inside one channel group (G is a multiple of 32)
        const int cg = (8 * i) / G;
        if constexpr (sizeof(M) == 2) {
            f16x2 vS[4], vZ[4];
            f16 sa[4], sb[4], za[4], zb[4];
            MetaLd<M>::ld4(vsm + cg * a.cap_tokens + tA, sa);
            MetaLd<M>::ld4(vsm + cg * a.cap_tokens + tB, sb);
            MetaLd<M>::ld4(vzm + cg * a.cap_tokens + tA, za);
            MetaLd<M>::ld4(vzm + cg * a.cap_tokens + tB, zb);
#pragma unroll
            for (int p = 0; p < 4; ++p) { vS[p] = f16x2{sa[p], sb[p]}; vZ[p] = f16x2{za[p], zb[p]}; }
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                f16x8 Bv = unpack8<BITS>(vw[nt], blk & 1, vS, vZ);
                O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, O[nt], 0, 0, 0);
            }
        } else {
            float sa[4], sb[4], za[4], zb[4];
            MetaLd<M>::ld4f(vsm + cg * a.cap_tokens + tA, sa);
            MetaLd<M>::ld4f(vsm + cg * a.cap_tokens + tB, sb);
            MetaLd<M>::ld4f(vzm + cg * a.cap_tokens + tA, za);
            MetaLd<M>::ld4f(vzm + cg * a.cap_tokens + tB, zb);
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                f16x8 Bv = unpack8_f32meta<BITS>(vw[nt], blk & 1, sa, sb, za, zb);
                O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, O[nt], 0, 0, 0);
            }
        }
        O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, O[8], 0, 0, 0);

        if (has_next) {
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int j = 0; j < KWL; ++j) kw[T][j] = kwn[T][j];
#pragma unroll
            for (int j = 0; j < 8; ++j) vw[j] = vwn[j];
        }
    }
    } else {
        // ------------------------------------------------------------ un-quantised fp16 tail
        // Same two products on plain fp16 rows: keys feed the A operand as stored,
        // values are loaded as eight rows of eight channels per lane and transposed
        // in registers into the token-major K-slots.
        const f16 *kt = (const f16 *)a.k_tail + bh * a.tail_cap * MF_D;
        const f16 *vt = (const f16 *)a.v_tail + bh * a.tail_cap * MF_D;
        f16x8 qT[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                qT[ks][2 * j] = i < R ? qn[4 * ks + j][0] : (f16)0.f;
                qT[ks][2 * j + 1] = i < R ? qn[4 * ks + j][1] : (f16)0.f;
            }
        const int n_tu = (int)((a.n_tail + 31) / 32);
        for (int u = wave; u < n_tu; u += 4) {
            const int64_t base = (int64_t)u * 32;
            f32x4 S[2];
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                const int64_t tok = base + krow0 + T * vtok_gap<BITS>();
                const f16 *p = kt + (tok < a.n_tail ? tok : 0) * MF_D + 32 * blk;
                S[T] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    f16x8 A = *reinterpret_cast<const f16x8 *>(p + 8 * ks);
                    S[T] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qT[ks], S[T], 0, 0, 0);
                }
            }
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int64_t tok = base + vtok_lo<BITS>(blk, r) + T * vtok_gap<BITS>();
                    if (i < R && tok >= a.n_tail) S[T][r] = -INFINITY;
                }
            const f16x8 P = softmax_unit(S, c, m_run, O, blk);
            f16x8 vr[8];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int64_t tA = base + vtok_lo<BITS>(blk, p), tB = tA + vtok_gap<BITS>();
                vr[2 * p] = *reinterpret_cast<const f16x8 *>(vt + (tA < a.n_tail ? tA : 0) * MF_D + 8 * i);
                vr[2 * p + 1] = *reinterpret_cast<const f16x8 *>(vt + (tB < a.n_tail ? tB : 0) * MF_D + 8 * i);
            }
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                f16x8 Bv;
#pragma unroll
                for (int j = 0; j < 8; ++j) Bv[j] = vr[j][nt];
                O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, O[nt], 0, 0, 0);
            }
            O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, O[8], 0, 0, 0);
        }
    }

    // ---------------------------------------------------------------- merge the four waves
    // accumulator register r of lane (i, blk) is row 4*blk + r, channel 8*i + nt
    if (blk == 0 && i < MF_ROWS) s_m[wave][i] = m_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * blk + r;
        if (row < R) {
            if (i == 0) s_l[wave][row] = O[8][r];
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) s_o[wave][row][8 * i + nt] = O[nt][r];
        }
    }
    __syncthreads();
    for (int e = tid; e < R * MF_D; e += 256) {
        const int row = e / MF_D, d = e % MF_D;
        float gm = fmaxf(fmaxf(s_m[0][row], s_m[1][row]), fmaxf(s_m[2][row], s_m[3][row]));
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            if (s_m[w][row] == -INFINITY) continue;
            const float f = exp2f(s_m[w][row] - gm);
            num += s_o[w][row][d] * f;
            den += s_l[w][row] * f;
        }
        float *o = ws + ((row0 + row) * nparts + sp) * MF_PART;
        o[2 + d] = num;
        if (d == 0) { o[0] = gm * LN2; o[1] = den; }
    }
}

bool mfma_decode_supported(const vq_attend_args &a) {
    if (a.D != MF_D || a.Sq != 1 || a.n_packed <= 0) return false;
    if (a.Hq % a.Hkv != 0 || 2 * (a.Hq / a.Hkv) > MF_ROWS) return false;  // high + remainder columns
    if (!(a.pack_bits == 2 || a.pack_bits == 4)) return false;
    if (!(a.group == 32 || a.group == 64 || a.group == 128)) return false;
    if (a.v_layout != VQ_V_TOKEN_PACKED) return false;
    if (a.n_packed % 32 != 0 || a.cap_tokens % 32 != 0 || a.cap_tokens % a.group != 0) return false;
    if (!(a.scale > 0.f)) return false;
    if (a.n_tail > 0 && (a.tail_dtype != VQ_F16 || (((uintptr_t)a.k_tail | (uintptr_t)a.v_tail) & 15u))) return false;
    if (a.B * a.Hkv > 65535) return false;
    const uintptr_t al = (uintptr_t)a.k_packed | (uintptr_t)a.v_packed | (uintptr_t)a.k_scale | (uintptr_t)a.k_zero |
                         (uintptr_t)a.v_scale | (uintptr_t)a.v_zero;
    if (al & 15u) return false;
    return true;
}

int launch_attend_mfma_decode(const vq_attend_args &a, int nsplit, int64_t split_len) {
    hipStream_t st = (hipStream_t)a.stream;
    const int has_tail = a.n_tail > 0 ? 1 : 0;
    const int nparts = nsplit + has_tail;
    dim3 grid((unsigned)nsplit, (unsigned)(a.B * a.Hkv));
    dim3 grid_tail(1, (unsigned)(a.B * a.Hkv));
    float *ws = (float *)a.workspace;
#define VQ_LAUNCH(BITS, M)                                                                                         \
    do {                                                                                                           \
        if (has_tail)                                                                                              \
            hipLaunchKernelGGL((attend_mfma_decode_kernel<BITS, M, true>), grid_tail, dim3(256), 0, st, a, nsplit, \
                               split_len, nparts, ws);                                                             \
        hipLaunchKernelGGL((attend_mfma_decode_kernel<BITS, M, false>), grid, dim3(256), 0, st, a, nsplit,         \
                           split_len, nparts, ws);                                                                 \
    } while (0)
    if (a.pack_bits == 4) {
        if (a.meta_dtype == VQ_F16) VQ_LAUNCH(4, f16); else VQ_LAUNCH(4, float);
    } else {
        if (a.meta_dtype == VQ_F16) VQ_LAUNCH(2, f16); else VQ_LAUNCH(2, float);
    }
#undef VQ_LAUNCH
    return VQ_OK;
}

}  // namespace vq
