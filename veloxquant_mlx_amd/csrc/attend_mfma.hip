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
__device__ __forceinline__ f16x2 h2(float a) { f16x2 r = {(f16)a, (f16)a}; return r; }
// A constant the optimiser must keep in a vector register, so that
// (w & mask) | magic becomes one v_and_or_b32 (mask in a scalar register).
__device__ __forceinline__ u32 vreg_const(u32 x) { asm volatile("" : "+v"(x)); return x; }

constexpr int MF_ROWS = 16;               // M/N width of the MFMA
constexpr int MF_D = 128;                 // head dim
constexpr int MF_PART = MF_D + 2;         // floats per partial: max, sum, accumulator
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
constexpr float RESCALE_SLACK = 8.0f;

// Magic constants: an fp16 whose mantissa field receives the code.  A 4-bit code
// in mantissa bits 4..7 of 64.0 reads 64 + code; a 2-bit code in bits 6..7 of 16.0
// reads 16 + code.
template <int BITS> struct Magic {
    static constexpr u32 bits = BITS == 4 ? 0x54005400u : 0x4C004C00u;
    static constexpr u32 mask = BITS == 4 ? 0x00F000F0u : 0x00C000C0u;
    static constexpr float off = BITS == 4 ? 64.f : 16.f;
};

// Eight codes of one packed word as fp16 values (offset + code), in K-slot pair order.
// BITS == 4: the word holds codes 0..7, pair p = (code p, code p + 4).
// BITS == 2: the word holds codes 0..15, `half` picks pairs (4*half + p, 4*half + p + 8).
// The offset is NOT removed here; callers either subtract it (values) or account
// for it in a per-group bias (keys).
template <int BITS>
__device__ __forceinline__ void unpack_raw(u32 w, int half, u32 magic, u32 (&r)[4]) {
    constexpr u32 mask = Magic<BITS>::mask;
    if (BITS == 4) {
        r[0] = ((w << 4) & mask) | magic;
        r[1] = (w & mask) | magic;
        r[2] = ((w >> 4) & mask) | magic;
        r[3] = ((w >> 8) & mask) | magic;
    } else {
        const u32 ws = w >> (8 * half);
        r[0] = ((ws << 6) & mask) | magic;
        r[1] = ((ws << 4) & mask) | magic;
        r[2] = ((ws << 2) & mask) | magic;
        r[3] = (ws & mask) | magic;
    }
}
__device__ __forceinline__ f16x8 pairs_to_h8(const f16x2 (&r)[4]) {
    f16x8 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) { o[2 * p] = r[p][0]; o[2 * p + 1] = r[p][1]; }
    return o;
}
// offset + code, exact small integers in fp16 (key operand)
template <int BITS> __device__ __forceinline__ f16x8 unpack8_offset_codes(u32 w, int half, u32 magic) {
    u32 r[4];
    unpack_raw<BITS>(w, half, magic, r);
    f16x2 h[4] = {as_h2(r[0]), as_h2(r[1]), as_h2(r[2]), as_h2(r[3])};
    return pairs_to_h8(h);
}
// code * scale + zero in packed fp16 (value operand, fp16 scale / zero)
template <int BITS>
__device__ __forceinline__ f16x8 unpack8_dequant(u32 w, int half, u32 magic, const f16x2 (&s)[4], const f16x2 (&z)[4]) {
    u32 r[4];
    unpack_raw<BITS>(w, half, magic, r);
    const f16x2 off = h2(Magic<BITS>::off);
    f16x2 h[4];
#pragma unroll
    for (int p = 0; p < 4; ++p) h[p] = __builtin_elementwise_fma(as_h2(r[p]) - off, s[p], z[p]);
    return pairs_to_h8(h);
}
// value operand with float32 scale / zero: formed in float32, rounded to fp16 once
template <int BITS>
__device__ __forceinline__ f16x8 unpack8_dequant_f32(u32 w, int half, u32 magic, const float (&sa)[4],
                                                     const float (&sb)[4], const float (&za)[4], const float (&zb)[4]) {
    u32 r[4];
    unpack_raw<BITS>(w, half, magic, r);
    const f16x2 off = h2(Magic<BITS>::off);
    f16x8 o;
#pragma unroll
    for (int p = 0; p < 4; ++p) {
        const f16x2 cd = as_h2(r[p]) - off;
        o[2 * p] = (f16)fmaf((float)cd[0], sa[p], za[p]);
        o[2 * p + 1] = (f16)fmaf((float)cd[1], sb[p], zb[p]);
    }
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
    static __device__ __forceinline__ void ld4f(const float *p, float (&o)[4]) {
        float4 u = *reinterpret_cast<const float4 *>(p);
        o[0] = u.x; o[1] = u.y; o[2] = u.z; o[3] = u.w;
    }
};

// Per-wave attention state: nine output tiles (eight of 16 channels plus the
// softmax denominator against a ones operand) and the running row maximum.
struct WaveAcc {
    f32x4 O[9];
    float m_run;   // log2 domain, row = lane % 16, replicated over the four lane groups
};

// Online-softmax step for one unit of 32 tokens.  S holds the raw scores of this
// lane's column (query row i) for its eight tokens; the output tiles are rescaled
// when the running maximum moves.  Returns P in the A-operand layout of the P.V
// product (pair r = tile 0 register r, tile 1 register r).
__device__ __forceinline__ f16x8 softmax_unit(const f32x4 (&S)[2], float c, WaveAcc &acc, int blk) {
    float mx = fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])),
                     fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    // The reference point m_run only has to stay within RESCALE_SLACK (log2 units) of the
    // true running maximum: P may then reach 2^RESCALE_SLACK, far inside fp16 range, and
    // the accumulators are rescaled a handful of times per wave instead of every time a
    // row's maximum creeps up.
    const float m_seen = mx * c;
    if (__any(m_seen > acc.m_run + RESCALE_SLACK)) {
        const float m_new = fmaxf(acc.m_run, m_seen);
        const float alpha = m_new == -INFINITY ? 1.f : exp2f(acc.m_run - m_new);   // 0 on the first unit
        float al[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * blk + r);
#pragma unroll
        for (int n = 0; n < 9; ++n)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc.O[n][r] *= al[r];
        acc.m_run = m_new;
    }
    const float mm = acc.m_run == -INFINITY ? 0.f : acc.m_run;   // a row with no visible token yet
    f16x8 P;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        P[2 * r] = (f16)__builtin_amdgcn_exp2f(S[0][r] * c - mm);
        P[2 * r + 1] = (f16)__builtin_amdgcn_exp2f(S[1][r] * c - mm);
    }
    return P;
}

__device__ __forceinline__ f16x8 ones8() {
    f16x8 o;
#pragma unroll
    for (int j = 0; j < 8; ++j) o[j] = (f16)1.0f;
    return o;
}

// ---------------------------------------------------------------------------
// Packed prefix.  A block covers n_units units of 32 tokens starting at t_begin;
// each wave takes a contiguous quarter of them, so consecutive units of a wave
// share key groups.  Loads run one unit ahead of the arithmetic: the codes and
// the value scale/zero of unit u+1, and the key scale/zero of the next token
// group when u+1 opens one, are issued before unit u is computed, so every wait
// inside the loop is for data requested a whole unit earlier.
// ---------------------------------------------------------------------------

// value scale / zero of the lane's eight tokens (tA..tA+3, tB..tB+3), one channel group
template <typename M> struct VMeta;
template <> struct VMeta<f16> {
    uint2 sa, sb, za, zb;
    __device__ __forceinline__ void load(const f16 *vs, const f16 *vz, int64_t tA, int64_t tB) {
        sa = *reinterpret_cast<const uint2 *>(vs + tA); sb = *reinterpret_cast<const uint2 *>(vs + tB);
        za = *reinterpret_cast<const uint2 *>(vz + tA); zb = *reinterpret_cast<const uint2 *>(vz + tB);
    }
};
template <> struct VMeta<float> {
    float4 sa, sb, za, zb;
    __device__ __forceinline__ void load(const float *vs, const float *vz, int64_t tA, int64_t tB) {
        sa = *reinterpret_cast<const float4 *>(vs + tA); sb = *reinterpret_cast<const float4 *>(vs + tB);
        za = *reinterpret_cast<const float4 *>(vz + tA); zb = *reinterpret_cast<const float4 *>(vz + tB);
    }
};
// key scale / zero of the lane's 32 channels for one token group, memory order
template <typename M> struct KMeta;
template <> struct KMeta<f16> {
    uint4 s[4], z[4];
    __device__ __forceinline__ void load(const f16 *ks, const f16 *kz) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s[j] = *reinterpret_cast<const uint4 *>(ks + 8 * j);
            z[j] = *reinterpret_cast<const uint4 *>(kz + 8 * j);
        }
    }
    __device__ __forceinline__ f16 sval(int ch) const {
        const uint4 &q = s[ch / 8];
        const u32 w = (ch % 8) / 2 == 0 ? q.x : (ch % 8) / 2 == 1 ? q.y : (ch % 8) / 2 == 2 ? q.z : q.w;
        return as_h2(w)[ch % 2];
    }
    __device__ __forceinline__ f16x2 zpair(int j) const {   // channels 2j, 2j+1
        const uint4 &q = z[j / 4];
        return as_h2(j % 4 == 0 ? q.x : j % 4 == 1 ? q.y : j % 4 == 2 ? q.z : q.w);
    }
};
template <> struct KMeta<float> {
    float4 s[8], z[8];
    __device__ __forceinline__ void load(const float *ks, const float *kz) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s[j] = *reinterpret_cast<const float4 *>(ks + 4 * j);
            z[j] = *reinterpret_cast<const float4 *>(kz + 4 * j);
        }
    }
    __device__ __forceinline__ float sval(int ch) const {
        const float4 &q = s[ch / 4];
        return ch % 4 == 0 ? q.x : ch % 4 == 1 ? q.y : ch % 4 == 2 ? q.z : q.w;
    }
    __device__ __forceinline__ float zval(int ch) const {
        const float4 &q = z[ch / 4];
        return ch % 4 == 0 ? q.x : ch % 4 == 1 ? q.y : ch % 4 == 2 ? q.z : q.w;
    }
};

// value of lane (lane + n) of the same 16-lane row, 0 past the row's end
template <int N> __device__ __forceinline__ float row_shl(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x100 + N, 0xF, 0xF, true));
}
__device__ __forceinline__ float row_shl_n(float x, int n, int lane) {
    switch (n) {   // n is block-uniform
        case 1: return row_shl<1>(x);
        case 2: return row_shl<2>(x);
        case 4: return row_shl<4>(x);
        case 8: return row_shl<8>(x);
        default: return __shfl(x, (lane & ~15) | ((lane + n) & 15));
    }
}

template <int BITS, typename M>
__device__ __forceinline__ void packed_units(const vq_attend_args &a, int64_t bh, int64_t row0, int R, float c,
                                             int64_t t_begin, int n_units, int lane, int wave, WaveAcc &acc,
                                             uint4 *s_q) {
    constexpr int PER = 32 / BITS;           // codes per word
    constexpr int KW = MF_D / PER;           // key words per token row
    constexpr int KWL = KW / 4;              // key words one lane loads per token (its 32 channels)
    const int i = lane & 15, blk = lane >> 4;
    const u32 magic = vreg_const(Magic<BITS>::bits);

    const u32 *kp = (const u32 *)a.k_packed + bh * a.cap_tokens * KW;
    const u32 *vp = (const u32 *)a.v_packed + bh * (a.cap_tokens / PER) * MF_D;
    const int G = a.group, GV = MF_D / G;
    const int64_t GKcap = (a.cap_tokens + G - 1) / G;
    const M *ksm = (const M *)a.k_scale + bh * GKcap * MF_D + 32 * blk;
    const M *kzm = (const M *)a.k_zero + bh * GKcap * MF_D + 32 * blk;
    // channels 8*i .. 8*i+7 of the value tiles lie inside one channel group (G is a multiple of 32)
    const M *vsm = (const M *)a.v_scale + (bh * GV + (8 * i) / G) * a.cap_tokens;
    const M *vzm = (const M *)a.v_zero + (bh * GV + (8 * i) / G) * a.cap_tokens;

    // Query of this lane's column, parked in LDS (it is only needed when a token group
    // opens): columns [0, R) carry the high part of the folded query of row i, columns
    // [R, 2R) the remainder of row i - R; the rest are zero.  s_q[0..3][lane]: the lane's
    // 32 channels in memory order, s_q[4..7][lane]: in K-slot pair order.
    {
        const int rq = i < R ? i : i - R;
        const bool col_used = i < 2 * R;
        f16x2 qn[16], qp[16];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            float lo = 0.f, hi = 0.f;
            if (col_used) {
                lo = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + 2 * j);
                hi = ldq(a.q, a.q_dtype, (row0 + rq) * MF_D + 32 * blk + 2 * j + 1);
            }
            qn[j] = f16x2{(f16)lo, (f16)hi};
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const int lo = kchan_lo<BITS>(ks, p), hi = kchan_hi<BITS>(ks, p);
                qp[4 * ks + p] = f16x2{qn[lo / 2][lo % 2], qn[hi / 2][hi % 2]};
            }
        if (wave == 0) {
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                s_q[j * 64 + lane] = make_uint4(__builtin_bit_cast(u32, qn[4 * j]), __builtin_bit_cast(u32, qn[4 * j + 1]),
                                                __builtin_bit_cast(u32, qn[4 * j + 2]), __builtin_bit_cast(u32, qn[4 * j + 3]));
                s_q[(4 + j) * 64 + lane] = make_uint4(__builtin_bit_cast(u32, qp[4 * j]), __builtin_bit_cast(u32, qp[4 * j + 1]),
                                                      __builtin_bit_cast(u32, qp[4 * j + 2]), __builtin_bit_cast(u32, qp[4 * j + 3]));
            }
        }
        __syncthreads();
    }

    f16x8 qB[4];
    float bias = 0.f;   // row bias of the current token group: sum_d q_d z_d - offset * sum_d (q s)_d
    const f16x8 ones = ones8();

    // Fold a token group's key scales into the query and dot its zeros with it.
    auto open_group = [&](const KMeta<M> &km) {
        f16x2 qn[16], qp[16];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const uint4 x = s_q[j * 64 + lane], y = s_q[(4 + j) * 64 + lane];
            qn[4 * j] = as_h2(x.x); qn[4 * j + 1] = as_h2(x.y); qn[4 * j + 2] = as_h2(x.z); qn[4 * j + 3] = as_h2(x.w);
            qp[4 * j] = as_h2(y.x); qp[4 * j + 1] = as_h2(y.y); qp[4 * j + 2] = as_h2(y.z); qp[4 * j + 3] = as_h2(y.w);
        }
        float b_part = 0.f, q_part = 0.f;
        if constexpr (sizeof(M) == 2) {
#pragma unroll
            for (int j = 0; j < 16; ++j) b_part = __builtin_amdgcn_fdot2(qn[j], km.zpair(j), b_part, false);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const f16x2 sp2 = f16x2{km.sval(kchan_lo<BITS>(ks, p)), km.sval(kchan_hi<BITS>(ks, p))};
                    const f16x2 hi = qp[4 * ks + p] * sp2;
                    // q*s has at most 22 significant bits: the remainder after the fp16
                    // high part is itself an fp16 number, so this fma is exact
                    const f16x2 lo = __builtin_elementwise_fma(qp[4 * ks + p], sp2, -hi);
                    const f16x2 use = i < R ? hi : lo;
                    q_part = __builtin_amdgcn_fdot2(use, h2(1.f), q_part, false);
                    qB[ks][2 * p] = use[0];
                    qB[ks][2 * p + 1] = use[1];
                }
        } else {
#pragma unroll
            for (int j = 0; j < 16; ++j)
                b_part += (float)qn[j][0] * km.zval(2 * j) + (float)qn[j][1] * km.zval(2 * j + 1);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int p = 0; p < 4; ++p)
#pragma unroll
                    for (int e = 0; e < 2; ++e) {
                        const int ch = e == 0 ? kchan_lo<BITS>(ks, p) : kchan_hi<BITS>(ks, p);
                        const float t = (float)qp[4 * ks + p][e] * km.sval(ch);
                        const f16 hi = (f16)t;
                        const f16 lo = (f16)(t - (float)hi);
                        const f16 use = i < R ? hi : lo;
                        q_part += (float)use;
                        qB[ks][2 * p + e] = use;
                    }
        }
        // the key operand carries offset + code: remove offset * sum_d (q s)_d here.
        // Columns [R, 2R) hold the remainder parts; their sums join the high columns'.
        float t = (i < R ? b_part : 0.f) - Magic<BITS>::off * q_part;
        t += __shfl_xor(t, 16);
        t += __shfl_xor(t, 32);
        bias = t + row_shl_n(t, R, lane);
    };

    // token of S^T row i in tile T: rows of the two tiles interleave so that accumulator
    // register r of tile T is K-slot pair r of the P.V product
    const int krow0 = vtok_lo<BITS>(i >> 2, i & 3);
    const int vt0 = vtok_lo<BITS>(blk, 0);

    struct Unit {
        u32 kw[2][KWL];
        u32 vw[8];
        VMeta<M> vm;
    };
    auto load_unit = [&](int u, Unit &d) {
        const int64_t base = t_begin + (int64_t)u * 32;
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const u32 *p = kp + (base + krow0 + T * vtok_gap<BITS>()) * KW + KWL * blk;
            if (BITS == 4) {
                uint4 x = *reinterpret_cast<const uint4 *>(p);
                d.kw[T][0] = x.x; d.kw[T][1] = x.y; d.kw[T][KWL - 2] = x.z; d.kw[T][KWL - 1] = x.w;
            } else {
                uint2 x = *reinterpret_cast<const uint2 *>(p);
                d.kw[T][0] = x.x; d.kw[T][KWL - 1] = x.y;
            }
        }
        const int64_t wrow = base / PER + (BITS == 4 ? blk : blk / 2);
        const u32 *q8 = vp + wrow * MF_D + 8 * i;
        uint4 x0 = *reinterpret_cast<const uint4 *>(q8);
        uint4 x1 = *reinterpret_cast<const uint4 *>(q8 + 4);
        d.vw[0] = x0.x; d.vw[1] = x0.y; d.vw[2] = x0.z; d.vw[3] = x0.w;
        d.vw[4] = x1.x; d.vw[5] = x1.y; d.vw[6] = x1.z; d.vw[7] = x1.w;
        d.vm.load(vsm, vzm, base + vt0, base + vt0 + vtok_gap<BITS>());
    };

    const int per_wave = (n_units + 3) / 4;
    const int u0 = wave * per_wave;
    const int u1 = u0 + per_wave < n_units ? u0 + per_wave : n_units;
    if (u0 >= u1) return;

    Unit cur;
    KMeta<M> km;
    int64_t cur_group = (t_begin + (int64_t)u0 * 32) / G;
    load_unit(u0, cur);
    km.load(ksm + cur_group * MF_D, kzm + cur_group * MF_D);
    open_group(km);

    for (int u = u0; u < u1; ++u) {
        Unit nxt;
        const bool has_next = u + 1 < u1;
        const int64_t next_group = (t_begin + (int64_t)(u + 1) * 32) / G;
        const bool new_group = has_next && next_group != cur_group;
        if (has_next) load_unit(u + 1, nxt);
        if (new_group) km.load(ksm + next_group * MF_D, kzm + next_group * MF_D);

        // ---- S^T = (offset + codes) . (q s)  (two 16-token tiles, four k-steps of 32 channels)
        f32x4 S[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            S[T] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const u32 w = BITS == 4 ? cur.kw[T][ks] : cur.kw[T][ks / 2];
                f16x8 A = unpack8_offset_codes<BITS>(w, ks % 2, magic);
                S[T] = __builtin_amdgcn_mfma_f32_16x16x32_f16(A, qB[ks], S[T], 0, 0, 0);
            }
        }
        // column i < R: add the remainder column i + R and the group bias; other columns idle
        {
            float lo[8];
#define VQ_SHL(N)                                                                             \
    _Pragma("unroll") for (int T = 0; T < 2; ++T) _Pragma("unroll") for (int r = 0; r < 4; ++r) \
        lo[4 * T + r] = row_shl<N>(S[T][r]);
            switch (R) {   // block-uniform
                case 1: VQ_SHL(1) break;
                case 2: VQ_SHL(2) break;
                case 4: VQ_SHL(4) break;
                case 8: VQ_SHL(8) break;
                default:
#pragma unroll
                    for (int T = 0; T < 2; ++T)
#pragma unroll
                        for (int r = 0; r < 4; ++r) lo[4 * T + r] = __shfl(S[T][r], (lane & ~15) | ((i + R) & 15));
            }
#undef VQ_SHL
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r) S[T][r] = i < R ? S[T][r] + lo[4 * T + r] + bias : 0.f;
        }

        const f16x8 P = softmax_unit(S, c, acc, blk);

        // ---- O += P . V_hat (eight 16-channel tiles; lane column i is channel 8*i + nt)
        if constexpr (sizeof(M) == 2) {
            const f16x2 sa0 = as_h2(cur.vm.sa.x), sa1 = as_h2(cur.vm.sa.y), sb0 = as_h2(cur.vm.sb.x), sb1 = as_h2(cur.vm.sb.y);
            const f16x2 za0 = as_h2(cur.vm.za.x), za1 = as_h2(cur.vm.za.y), zb0 = as_h2(cur.vm.zb.x), zb1 = as_h2(cur.vm.zb.y);
            const f16x2 vS[4] = {f16x2{sa0[0], sb0[0]}, f16x2{sa0[1], sb0[1]}, f16x2{sa1[0], sb1[0]}, f16x2{sa1[1], sb1[1]}};
            const f16x2 vZ[4] = {f16x2{za0[0], zb0[0]}, f16x2{za0[1], zb0[1]}, f16x2{za1[0], zb1[0]}, f16x2{za1[1], zb1[1]}};
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                f16x8 Bv = unpack8_dequant<BITS>(cur.vw[nt], blk & 1, magic, vS, vZ);
                acc.O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, acc.O[nt], 0, 0, 0);
            }
        } else {
            const float sa[4] = {cur.vm.sa.x, cur.vm.sa.y, cur.vm.sa.z, cur.vm.sa.w};
            const float sb[4] = {cur.vm.sb.x, cur.vm.sb.y, cur.vm.sb.z, cur.vm.sb.w};
            const float za[4] = {cur.vm.za.x, cur.vm.za.y, cur.vm.za.z, cur.vm.za.w};
            const float zb[4] = {cur.vm.zb.x, cur.vm.zb.y, cur.vm.zb.z, cur.vm.zb.w};
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) {
                f16x8 Bv = unpack8_dequant_f32<BITS>(cur.vw[nt], blk & 1, magic, sa, sb, za, zb);
                acc.O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, acc.O[nt], 0, 0, 0);
            }
        }
        acc.O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, acc.O[8], 0, 0, 0);

        if (new_group) {
            open_group(km);
            cur_group = next_group;
        }
        if (has_next) cur = nxt;
    }
}

// ---------------------------------------------------------------------------
// Un-quantised fp16 tail: the same two products on plain rows.  Keys feed the A
// operand as stored; values are loaded as eight rows of eight channels per lane
// and transposed in registers into the token-major K-slots.
// ---------------------------------------------------------------------------
template <int BITS>
__device__ __forceinline__ void tail_units(const vq_attend_args &a, int64_t bh, int64_t row0, int R, float c,
                                           int lane, int wave, WaveAcc &acc) {
    const int i = lane & 15, blk = lane >> 4;
    const f16 *kt = (const f16 *)a.k_tail + bh * a.tail_cap * MF_D;
    const f16 *vt = (const f16 *)a.v_tail + bh * a.tail_cap * MF_D;
    f16x8 qT[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j)
            qT[ks][j] = i < R ? (f16)ldq(a.q, a.q_dtype, (row0 + i) * MF_D + 32 * blk + 8 * ks + j) : (f16)0.f;
    const f16x8 ones = ones8();
    const int krow0 = vtok_lo<BITS>(i >> 2, i & 3);
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
        const f16x8 P = softmax_unit(S, c, acc, blk);
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
            acc.O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, acc.O[nt], 0, 0, 0);
        }
        acc.O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, acc.O[8], 0, 0, 0);
    }
}

// grid (nparts, B*Hkv): block x < nsplit covers tokens [x*split_len, ...) of the packed
// prefix, block x == nsplit (present when there is a tail) covers the fp16 tail.
template <int BITS, typename M, bool TAIL>
__global__ __launch_bounds__(256) void attend_mfma_decode_kernel(vq_attend_args a, int nsplit, int64_t split_len,
                                                                 int nparts, float *__restrict__ ws) {
    __shared__ float s_m[4][MF_ROWS];
    __shared__ float s_l[4][MF_ROWS];
    __shared__ float s_o[4][MF_ROWS][MF_D];
    __shared__ uint4 s_q[8 * 64];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: loops below stay scalar
    const int i = lane & 15, blk = lane >> 4;
    const int64_t bh = blockIdx.y;
    const int sp = TAIL ? nsplit : (int)blockIdx.x;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t row0 = b * a.Hq + hkv * R;   // first query row of this kv head (Sq == 1)
    const float c = a.scale * LOG2E;

    WaveAcc acc;
#pragma unroll
    for (int n = 0; n < 9; ++n) acc.O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.m_run = -INFINITY;

    if constexpr (TAIL) {
        tail_units<BITS>(a, bh, row0, R, c, lane, wave, acc);
    } else {
        const int64_t t_begin = (int64_t)sp * split_len;
        int64_t t_end = t_begin + split_len;
        if (t_end > a.n_packed) t_end = a.n_packed;
        packed_units<BITS, M>(a, bh, row0, R, c, t_begin, (int)((t_end - t_begin) / 32), lane, wave, acc, s_q);
    }

    // ---------------------------------------------------------------- merge the four waves
    // accumulator register r of lane (i, blk) is row 4*blk + r, channel 8*i + nt
    if (blk == 0) s_m[wave][i] = acc.m_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * blk + r;
        if (row < R) {
            if (i == 0) s_l[wave][row] = acc.O[8][r];
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) s_o[wave][row][8 * i + nt] = acc.O[nt][r];
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
    const int nparts = nsplit + (a.n_tail > 0 ? 1 : 0);
    dim3 grid((unsigned)nsplit, (unsigned)(a.B * a.Hkv));
    dim3 grid_tail(1, (unsigned)(a.B * a.Hkv));
    float *ws = (float *)a.workspace;
#define VQ_LAUNCH(BITS, M) do { if (a.n_tail > 0) hipLaunchKernelGGL((attend_mfma_decode_kernel<BITS, M, true>), grid_tail, dim3(256), 0, st, a, nsplit, split_len, nparts, ws); \
    hipLaunchKernelGGL((attend_mfma_decode_kernel<BITS, M, false>), grid, dim3(256), 0, st, a, nsplit, split_len, nparts, ws); } while (0)
    if (a.pack_bits == 4) {
        if (a.meta_dtype == VQ_F16) VQ_LAUNCH(4, f16); else VQ_LAUNCH(4, float);
    } else {
        if (a.meta_dtype == VQ_F16) VQ_LAUNCH(2, f16); else VQ_LAUNCH(2, float);
    }
#undef VQ_LAUNCH
    return VQ_OK;
}

}  // namespace vq
