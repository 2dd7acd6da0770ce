// Helpers shared by the MFMA decode kernels (gfx950, wave64).
//
// v_mfma_f32_16x16x32_f16 operand layout, lane l, n = l % 16, blk = l / 16:
//   A[i = n][k = 8*blk + j]   j = 0..7 (eight fp16 per lane)
//   B[k = 8*blk + j][n]
//   D[i = 4*blk + r][n]       r = 0..3 (four fp32 per lane)
// MFMA sums over k, so any assignment of channels (tokens) to k-slots is valid as
// long as A and B agree.
#pragma once
#include "attend.hpp"

namespace vq {

typedef uint32_t u32;
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ f16x2 as_h2(u32 u) { return __builtin_bit_cast(f16x2, u); }
__device__ __forceinline__ u32 as_u(f16x2 h) { return __builtin_bit_cast(u32, h); }
__device__ __forceinline__ f16x8 as_h8(u32 a, u32 b, u32 c, u32 d) {
    u32x4 v = {a, b, c, d};
    return __builtin_bit_cast(f16x8, v);
}
__device__ __forceinline__ f16x8 as_h8(uint4 v) { return as_h8(v.x, v.y, v.z, v.w); }
__device__ __forceinline__ f16x2 h2(float a) { f16x2 r = {(f16)a, (f16)a}; return r; }
// A constant the optimiser must keep in a vector register, so that
// (w & mask) | magic becomes one v_and_or_b32 (mask in a scalar register).
__device__ __forceinline__ u32 vreg_const(u32 x) { asm volatile("" : "+v"(x)); return x; }
// The fp16 high part of a float32 product, pinned to the value that sits in the register.  Without
// the barrier the compiler is free to evaluate `(f16)(a * b)` twice in two ways -- a float32
// multiply followed by a conversion (two roundings) where the pair is packed, and a mixed-precision
// fused multiply-add that rounds the exact product once (v_fma_mixlo_f16) where a single element
// is widened again.  When the float32 product lies exactly half-way between two fp16 numbers the
// two disagree by one fp16 step, and a remainder `t - (float)hi` formed from the second no longer
// complements the high part stored from the first (error 2^-11 relative instead of 2^-22).
__device__ __forceinline__ f16x2 pinned_h2(f16x2 h) {
    u32 u = __builtin_bit_cast(u32, h);
    asm volatile("" : "+v"(u));
    return __builtin_bit_cast(f16x2, u);
}
// {lo half of a, lo half of b} and {hi half of a, hi half of b}
__device__ __forceinline__ u32 pair_lo(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x05040100u); }
__device__ __forceinline__ u32 pair_hi(u32 a, u32 b) { return __builtin_amdgcn_perm(b, a, 0x07060302u); }

constexpr int MF_ROWS = 16;               // M/N width of the MFMA
constexpr int MF_D = 128;                 // head dim
constexpr int MF_PART = MF_D + 2;         // floats per partial: max, sum, accumulator
constexpr float LOG2E = 1.4426950408889634f;
constexpr float LN2 = 0.6931471805599453f;
// The softmax reference point only has to stay within this many log2 units of the
// true running maximum: P may then reach 2^RESCALE_SLACK, far inside fp16 range, and
// the accumulators are rescaled a handful of times per wave instead of every time a
// row's maximum creeps up.
constexpr float RESCALE_SLACK = 8.0f;

// Magic constants: an fp16 whose TOP mantissa bits receive the code, so that the constant is
// as small as it can be next to the codes (the products carry offset + code, and float32
// accumulation of the offset part costs accuracy in proportion to offset / code).  A 4-bit
// code in mantissa bits 6..9 of 16.0 reads 16 + code; a 2-bit code in bits 8..9 of 4.0 reads
// 4 + code.
template <int BITS> struct Magic {
    static constexpr u32 bits = BITS == 4 ? 0x4C004C00u : 0x44004400u;
    static constexpr u32 mask = BITS == 4 ? 0x03C003C0u : 0x03000300u;
    static constexpr float off = BITS == 4 ? 16.f : 4.f;
    static constexpr u32 neg_off_pair = BITS == 4 ? 0xCC00CC00u : 0xC400C400u;   // {-off, -off}
};

// Eight codes of one packed word as fp16 values (offset + code), in k-slot pair order.
// BITS == 4: the word holds codes 0..7, pair p = (code p, code p + 4).
// BITS == 2: `w` is the word shifted right by 8*half; it then holds codes
//            4*half + 0..3 and 4*half + 8..11 in its two byte lanes, pair p =
//            (code 4*half + p, code 4*half + p + 8).
// The offset is NOT removed here: an MFMA against a constant operand accounts for it.
template <int BITS> __device__ __forceinline__ f16x8 unpack8(u32 w, u32 magic) {
    constexpr u32 mask = Magic<BITS>::mask;
    u32 r0, r1, r2, r3;
    if (BITS == 4) {
        r0 = ((w << 6) & mask) | magic;
        r1 = ((w << 2) & mask) | magic;
        r2 = ((w >> 2) & mask) | magic;
        r3 = ((w >> 6) & mask) | magic;
    } else {
        r0 = ((w << 8) & mask) | magic;
        r1 = ((w << 6) & mask) | magic;
        r2 = ((w << 4) & mask) | magic;
        r3 = ((w << 2) & mask) | magic;
    }
    return as_h8(r0, r1, r2, r3);
}

// Two packed words at a time: a 64-bit shift (full rate on this part) moves both, and what
// crosses from one word into the other lands outside the mask.  SH > 0 shifts left.
typedef unsigned long long u64;
template <int SH> __device__ __forceinline__ u64 shift64(u64 x) {
    u64 r = x;
    if constexpr (SH > 0) asm("v_lshlrev_b64 %0, %2, %1" : "=v"(r) : "v"(x), "n"(SH));
    else if constexpr (SH < 0) asm("v_lshrrev_b64 %0, %2, %1" : "=v"(r) : "v"(x), "n"(-SH));
    return r;
}
template <int BITS, int S0, int S1, int S2, int S3>
__device__ __forceinline__ void unpack8_pair_at(u64 x, u32 magic, f16x8 &lo, f16x8 &hi) {
    constexpr u32 mask = Magic<BITS>::mask;
    const u64 t0 = shift64<S0>(x), t1 = shift64<S1>(x), t2 = shift64<S2>(x), t3 = shift64<S3>(x);
    lo = as_h8(((u32)t0 & mask) | magic, ((u32)t1 & mask) | magic, ((u32)t2 & mask) | magic, ((u32)t3 & mask) | magic);
    hi = as_h8(((u32)(t0 >> 32) & mask) | magic, ((u32)(t1 >> 32) & mask) | magic, ((u32)(t2 >> 32) & mask) | magic,
               ((u32)(t3 >> 32) & mask) | magic);
}
__device__ __forceinline__ u64 pack64(u32 lo, u32 hi) { return (u64)lo | ((u64)hi << 32); }
// unpack8 of the words w0 and w1
template <int BITS> __device__ __forceinline__ void unpack8_pair(u32 w0, u32 w1, u32 magic, f16x8 &a0, f16x8 &a1) {
    if constexpr (BITS == 4) unpack8_pair_at<4, 6, 2, -2, -6>(pack64(w0, w1), magic, a0, a1);
    else unpack8_pair_at<2, 8, 6, 4, 2>(pack64(w0, w1), magic, a0, a1);
}
// 2-bit only: unpack8 of w0 >> 8 and w1 >> 8
__device__ __forceinline__ void unpack8_pair_upper2(u32 w0, u32 w1, u32 magic, f16x8 &a0, f16x8 &a1) {
    unpack8_pair_at<2, 0, -2, -4, -6>(pack64(w0, w1), magic, a0, a1);
}

// ---- codes as fp16 SUBNORMALS (the packed decode kernel).
// A half whose exponent field is zero reads mantissa * 2^-24, and the matrix unit takes such
// operands exactly.  A code left where a shifted packed word holds it, at mantissa bit POS,
// therefore reads code * 2^(POS - 24): one AND per two codes (one per register of the
// operand) and no constant to subtract afterwards.  The other operand of the same k-slot
// carries 2^(E - POS), an exact scaling, so every product is code * value * 2^(E - 24).
// The unit aligns the products of an instruction to the largest NOMINAL exponent among them
// (-14 for every subnormal, whatever its leading zeros) and keeps about 25 bits below it: a
// code at bit POS is good to 2^-(15 + POS) of the instruction's largest other-operand value,
// which is why the fields sit at bits 2, 4, 6, 8 (2-bit) and 2, 6 (4-bit) and not lower.
template <int BITS> struct Sub {
    // mantissa bit of k-slot pair p (p = 0..3) of an operand
    static constexpr int pos(int p) { return BITS == 2 ? 2 + 2 * p : 2 + 4 * (p & 1); }
    static constexpr u32 mask(int p) { return (BITS == 2 ? 0x00030003u : 0x000F000Fu) << pos(p); }
    // exponents carried by the other operand: keys 2^(EK - pos), values 2^(EV - pos) >= 1
    static constexpr int EK = BITS == 2 ? 5 : 4;
    static constexpr int EV = BITS == 2 ? 8 : 6;
    // probabilities may reach 2^SLACK before the softmax reference moves; times 2^(EV - 2) and
    // the value scale they must stay inside fp16 (2^SLACK * 2^(EV - 2) = 2^8 either way)
    static constexpr float SLACK = BITS == 2 ? 2.f : 4.f;
    static constexpr float KSCALE = (float)(1 << (24 - EK));       // scores: accumulator * KSCALE
    static constexpr float KSCALE_INV = 1.f / (float)(1 << (24 - EK));
    static constexpr float VSCALE = (float)(1 << (24 - EV));       // outputs: accumulator * VSCALE
    static constexpr float wk(int p) { return EK >= pos(p) ? (float)(1 << (EK >= pos(p) ? EK - pos(p) : 0))
                                                           : 1.f / (float)(1 << (pos(p) > EK ? pos(p) - EK : 0)); }
    static constexpr float wv(int p) { return (float)(1 << (EV - pos(p))); }
    static constexpr float wv_inv(int p) { return 1.f / (float)(1 << (EV - pos(p))); }
};
template <int BITS> __device__ __forceinline__ f16x8 sub4(u32 w) {
    return as_h8(w & Sub<BITS>::mask(0), w & Sub<BITS>::mask(1), w & Sub<BITS>::mask(2), w & Sub<BITS>::mask(3));
}
// 4-bit: the eight codes of w0 (and of w1) as one operand each, pair p = (code p, code p + 4);
// codes 0, 1 come from the word moved up by two bits, codes 2, 3 from the word moved down by six
__device__ __forceinline__ void sub_unpack4(u32 w0, u32 w1, f16x8 &a0, f16x8 &a1) {
    const u64 x = pack64(w0, w1), l = shift64<2>(x), r = shift64<-6>(x);
    constexpr u32 m0 = Sub<4>::mask(0), m1 = Sub<4>::mask(1);
    a0 = as_h8((u32)l & m0, (u32)l & m1, (u32)r & m0, (u32)r & m1);
    a1 = as_h8((u32)(l >> 32) & m0, (u32)(l >> 32) & m1, (u32)(r >> 32) & m0, (u32)(r >> 32) & m1);
}
// 2-bit: the sixteen codes of w0 (and of w1) as two operands each: `lo*` codes 0-3 | 8-11, `up*`
// codes 4-7 | 12-15, pair p = (code p, code p + 8) of that set
__device__ __forceinline__ void sub_unpack2(u32 w0, u32 w1, f16x8 &lo0, f16x8 &up0, f16x8 &lo1, f16x8 &up1) {
    const u64 x = pack64(w0, w1), l = shift64<2>(x), r = shift64<-6>(x);
    lo0 = sub4<2>((u32)l);
    lo1 = sub4<2>((u32)(l >> 32));
    up0 = sub4<2>((u32)r);
    up1 = sub4<2>((u32)(r >> 32));
}
// largest of three / two without the quieting of signalling NaNs that fmaxf asks for (scores are never NaN)
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
    return r;
}
__device__ __forceinline__ float max_raw(float a, float b) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

// channel (0..31 inside a lane's 32-channel slice) of k-slot pair p of k-step ks
template <int BITS> __device__ __forceinline__ constexpr int kchan_lo(int ks, int p) {
    return BITS == 4 ? 8 * ks + p : 16 * (ks / 2) + 4 * (ks % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int kchan_hi(int ks, int p) {
    return kchan_lo<BITS>(ks, p) + (BITS == 4 ? 4 : 8);
}
// token (0..31 inside a unit) of k-slot pair p of lane group blk in the P.V product
template <int BITS> __device__ __forceinline__ constexpr int vtok_lo(int blk, int p) {
    return BITS == 4 ? 8 * blk + p : 16 * (blk / 2) + 4 * (blk % 2) + p;
}
template <int BITS> __device__ __forceinline__ constexpr int vtok_gap() { return BITS == 4 ? 4 : 8; }

__device__ __forceinline__ float ldq(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}

__device__ __forceinline__ f16x8 ones8() { return as_h8(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u); }

// value of lane (lane + N) of the same 16-lane row, 0 past the row's end
template <int N> __device__ __forceinline__ float row_shl(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x100 + N, 0xF, 0xF, true));
}

// load through a block-uniform base plus a 32-bit per-lane byte offset
template <typename T> __device__ __forceinline__ T ldg(const char *base, u32 off) {
    return *reinterpret_cast<const T *>(base + off);
}

// ---- asynchronous copies from global memory straight into LDS (no register in between).
// Lane l's BYTES bytes land at LDS address  lds + OFF + BYTES * l  and come from global address
// base + voff + OFF (base wave-uniform, voff a 32-bit per-lane byte offset); the instruction
// offset OFF applies to both sides.  The optimiser sees neither the LDS write nor the
// outstanding-load counter of these copies: a caller orders them against its LDS reads with
// wait_copies<N>(), which returns once at most N of the wave's copies are still in flight
// (they complete in issue order) and is a compiler barrier for memory.  m0 carries the LDS
// address; the compiler itself does not use m0 in these kernels.
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
// a wave-uniform value the register allocator must keep in scalar registers
__device__ __forceinline__ u32 uniform(u32 x) { return (u32)__builtin_amdgcn_readfirstlane((int)x); }
__device__ __forceinline__ const void *uniform(const void *p) {
    const uint64_t v = (uint64_t)(uintptr_t)p;
    return (const void *)(uintptr_t)(((uint64_t)uniform((u32)(v >> 32)) << 32) | uniform((u32)v));
}
template <int OFF> __device__ __forceinline__ void lds_copy16(const void *base, u32 voff, u32 lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 offset:%3"
                 :: "v"(voff), "s"(uniform(base)), "s"(uniform(lds)), "n"(OFF) : "memory", "m0");
}
template <int OFF> __device__ __forceinline__ void lds_copy4(const void *base, u32 voff, u32 lds) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dword %0, %1 offset:%3"
                 :: "v"(voff), "s"(uniform(base)), "s"(uniform(lds)), "n"(OFF) : "memory", "m0");
}
#pragma clang diagnostic pop
template <int N> __device__ __forceinline__ void wait_copies() {
    static_assert(N >= 0 && N < 64, "the counter has six bits");
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(N) : "memory");
}
// LDS byte address of a pointer into block-shared memory
__device__ __forceinline__ u32 lds_addr(const void *p) {
    return (u32)(uintptr_t)(__attribute__((address_space(3))) const void *)p;
}

// The query rows one block works on: RT = R * PQ rows that share a kv head, namely the R
// heads of the GQA group at PQ consecutive query positions starting at pos0.  Tile row
// j is head j % R at position pos0 + j / R.  Decode (Sq == 1) is the case PQ == 1.
struct RowTile {
    int64_t base_row;   // flattened [B, Hq, Sq] row of (b, first head of the group, position 0)
    int64_t Sq, n_total;
    // R heads of the GQA group from head h0 on (all of them unless the group has more than eight: then tiles
    // of eight heads at one position), RT = R * positions rows in all
    int R, RT, pos0, causal, h0;
    int64_t window;     // sliding window (0: none)
    __device__ __forceinline__ bool valid(int j) const { return j < RT && pos0 + j / R < Sq; }
    // first visible slot of tile row j
    __device__ __forceinline__ int64_t first(int j) const {
        int64_t pos = pos0 + j / R;
        if (pos > Sq - 1) pos = Sq - 1;
        const int64_t lo = n_total - Sq + pos + 1 - window;
        return window > 0 && lo > 0 ? lo : 0;
    }
    __device__ __forceinline__ int64_t row(int j) const { return base_row + (int64_t)(h0 + j % R) * Sq + pos0 + j / R; }
    // number of visible slots of tile row j (queries align to the end of the slots)
    __device__ __forceinline__ int64_t visible(int j) const {
        int64_t pos = pos0 + j / R;
        if (pos > Sq - 1) pos = Sq - 1;
        return causal ? n_total - Sq + pos + 1 : n_total;
    }
};

// ---------------------------------------------------------------------------
// Un-quantised fp16 / bf16 tail, run by the four waves of one block in units of 32 tokens:
//   S^T[token, row] = K[token, :] . q[row, :]          A = K as stored, B = q
//   O[row, chan]   += P[row, token] * V[token, chan]   A = P, B = V
// Values are loaded as eight rows of eight channels per lane and transposed in
// registers into the token-major k-slots.  The softmax denominator is a ninth
// output tile against a ones operand.  Writes one (max, sum, accumulator) partial
// per query row into slot `slot` of the partials.
// ---------------------------------------------------------------------------
struct TailAcc {
    f32x4 O[9];
    float m_run;   // log2 domain, row = lane % 16, replicated over the four lane groups
};

// token (0..31 inside a unit) of S^T row 4*blk + r of tile T: rows of the two tiles interleave
// so that accumulator register r of tile T is k-slot pair r of the P.V product
__device__ __forceinline__ int tail_tok(int blk, int r, int T) { return 8 * blk + r + 4 * T; }

__device__ __forceinline__ f16x8 tail_softmax_unit(const f32x4 (&S)[2], float c, TailAcc &acc, int blk) {
    float mx = fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])),
                     fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
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

// Partials another block will read in this launch go out as device-scope stores (written
// through to where every compute die sees them); otherwise plain stores.
__device__ __forceinline__ void st_partial(float *p, float v, bool device_scope) {
    if (device_scope) __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    else *p = v;
}

// Eight consecutive tail elements as fp16.  A bf16 tail is converted: exact for magnitudes in
// fp16's normal range, an absolute error below 2^-25 for smaller ones, saturating at 65504.
__device__ __forceinline__ f16x8 tail8_from_raw(const uint4 u, bool bf16) {
    if (!bf16) {
        union { uint4 u; f16x8 h; } x;
        x.u = u;
        return x.h;
    }
    const u32 w[4] = {u.x, u.y, u.z, u.w};
    f16x8 o;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const float lo = __uint_as_float(w[j] << 16), hi = __uint_as_float(w[j] & 0xffff0000u);
        o[2 * j] = (f16)fminf(fmaxf(lo, -65504.f), 65504.f);
        o[2 * j + 1] = (f16)fminf(fmaxf(hi, -65504.f), 65504.f);
    }
    return o;
}
__device__ __forceinline__ f16x8 ld_tail8(const void *base, int64_t elem, bool bf16) {
    return tail8_from_raw(*reinterpret_cast<const uint4 *>((const u16 *)base + elem), bf16);
}

// One wave's share of the tail: units w, w + T, ... of 32 tokens (w = which of the T tail waves this
// is), written as a partial of its own into slot `slot` straight from the accumulators -- no
// block-shared memory and no barrier, so the other waves of the block stream the packed prefix
// meanwhile.  s_qraw: the query rows of this kv head as fp16, q_stride halves apart.  A wave
// without units (a sequence with a shorter tail) writes an empty partial (max -inf, sum 0).
__device__ __forceinline__ void tail_wave(const vq_attend_args &a, int64_t bh, const RowTile &tile, float c, int slot,
                                          int nparts, float *__restrict__ ws, const f16 *s_qraw, int q_stride, int lane,
                                          int w, int T, bool device_scope) {
    const int i = lane & 15, blk = lane >> 4;
    const int R = tile.RT;
    // tail tokens this lane's query row sees
    int64_t n_vis = tile.visible(i < R ? i : 0) - a.n_packed;
    if (n_vis > a.n_tail) n_vis = a.n_tail;
    int64_t n_lo = tile.first(i < R ? i : 0) - a.n_packed;   // first tail token the row sees
    if (n_lo < 0) n_lo = 0;
    TailAcc acc;
#pragma unroll
    for (int n = 0; n < 9; ++n) acc.O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.m_run = -INFINITY;

    const bool bf16 = a.tail_dtype == VQ_BF16;
    const int64_t tbase = bh * a.tail_cap * MF_D;
    const f16x8 ones = ones8();
    const int n_tu = (int)((a.n_tail + 31) / 32);

    struct TUnit { f16x8 kr[2][4], vr[8]; };
    // the newest token's rows, when the call brings them, are read from where the caller holds
    // them (row n_tail - 1 of the tail is being written by this block at the same time)
    const int64_t newest = a.k_new != nullptr ? a.n_tail - 1 : -1;
    auto key_row = [&](int64_t tok, int64_t col) {
        if (tok >= a.n_tail) tok = 0;
        return tok == newest ? ld_tail8(a.k_new, bh * MF_D + col, bf16) : ld_tail8(a.k_tail, tbase + tok * MF_D + col, bf16);
    };
    auto value_row = [&](int64_t tok, int64_t col) {
        if (tok >= a.n_tail) tok = 0;
        return tok == newest ? ld_tail8(a.v_new, bh * MF_D + col, bf16) : ld_tail8(a.v_tail, tbase + tok * MF_D + col, bf16);
    };
    // every load of a unit is issued before its first product; clamped rows are masked below
    auto load = [&](int u, TUnit &d) {
        const int64_t base = (int64_t)u * 32;
#pragma unroll
        for (int Tt = 0; Tt < 2; ++Tt) {
            const int64_t tok = base + tail_tok(i >> 2, i & 3, Tt);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) d.kr[Tt][ks] = key_row(tok, 32 * blk + 8 * ks);
        }
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            d.vr[2 * p] = value_row(base + tail_tok(blk, p, 0), 8 * i);
            d.vr[2 * p + 1] = value_row(base + tail_tok(blk, p, 1), 8 * i);
        }
    };
    auto compute = [&](int u, const TUnit &d) {
        const int64_t base = (int64_t)u * 32;
        // the query operand is read again for every unit: sixteen registers that need not live across the loads
        f16x8 qT[4];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            qT[ks] = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
            if (i < R) qT[ks] = *reinterpret_cast<const f16x8 *>(s_qraw + i * q_stride + 32 * blk + 8 * ks);
        }
        f32x4 S[2];
#pragma unroll
        for (int Tt = 0; Tt < 2; ++Tt) {
            S[Tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) S[Tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(d.kr[Tt][ks], qT[ks], S[Tt], 0, 0, 0);
        }
#pragma unroll
        for (int Tt = 0; Tt < 2; ++Tt)
#pragma unroll
            for (int r = 0; r < 4; ++r)
                if (i < R && (base + tail_tok(blk, r, Tt) >= n_vis || base + tail_tok(blk, r, Tt) < n_lo)) S[Tt][r] = -INFINITY;
        const f16x8 P = tail_softmax_unit(S, c, acc, blk);
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) {   // lane column i is channel 8*i + nt
            f16x8 Bv;
#pragma unroll
            for (int j = 0; j < 8; ++j) Bv[j] = d.vr[j][nt];
            acc.O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, acc.O[nt], 0, 0, 0);
        }
        acc.O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, acc.O[8], 0, 0, 0);
    };
    // one unit in registers at a time (64 of them): the kernel runs three waves to a SIMD
    for (int u = w; u < n_tu; u += T) {
        TUnit d;
        load(u, d);
        compute(u, d);
    }
    // the partial: accumulator register r of lane (i, blk) is row 4*blk + r, channels 8*i .. 8*i + 7;
    // the maximum of row i sits in lane i of every lane group
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * blk + r;
        if (!tile.valid(row)) continue;
        float *o = ws + (tile.row(row) * nparts + slot) * MF_PART;
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) st_partial(o + 2 + 8 * i + nt, acc.O[nt][r], device_scope);
        if (i == 0) st_partial(o + 1, acc.O[8][r], device_scope);
    }
    if (blk == 0 && tile.valid(i)) st_partial(ws + (tile.row(i) * nparts + slot) * MF_PART, acc.m_run * LN2, device_scope);
}

// Combine the nparts partials of the tile's query rows into the output (the
// arithmetic of attend_merge_kernel, which shares merge_partials).  Partials written by
// other blocks of this launch are read with device-scope loads.
template <int DH = 1>
__device__ __forceinline__ void merge_rows(const vq_attend_args &a, const RowTile &tile, int nparts, const float *ws,
                                           int tid, int nthreads) {
    constexpr int DD = MF_D * DH, PART = DD + 2;
    for (int e = tid; e < tile.RT * DD; e += nthreads) {
        const int j = e / DD, d = e % DD;
        if (!tile.valid(j)) continue;
        const int64_t row = tile.row(j);
        // partials of other blocks come from beyond this XCD's L2: as few rounds of loads as possible
        const float v = merge_records<true>(ws + row * nparts * PART, nparts, PART, d);
        const int64_t oi = row * DD + d;
        if (a.out_dtype == VQ_F16) ((f16 *)a.out)[oi] = (f16)v;
        else if (a.out_dtype == VQ_BF16) ((u16 *)a.out)[oi] = f32_to_bf16(v);
        else ((float *)a.out)[oi] = v;
    }
}

// launchers of the packed-prefix kernel (it also runs the fp16 tail and, given sync counters,
// the final merge); partials are [rows][nparts][MF_PART] floats of (max, sum, accumulator)
// (one translation unit per scale / zero type and per number of query rows a block carries: 4 or 8)
void launch_mfma_packed_f16meta_r4(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_f16meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_f32meta_r4(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_f32meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
// the same for a head of 256 channels (packed prefix only)
void launch_mfma_packed_d256_f16meta_r4(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_d256_f16meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_d256_f32meta_r4(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);
void launch_mfma_packed_d256_f32meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st);

}  // namespace vq
