// MFMA decode attention over the packed prefix of a KIVI cache (gfx950, wave64).
//
// One block of eight waves per (kv head, token split), one block per CU.  Every wave streams
// units of 32 tokens and never reconstructs a key or a value: both products run on the raw
// codes, which are dropped from the packed word into the mantissa of an fp16
// constant by one and-or per two codes (value = offset + code, exact), and every
// affine term is pushed onto the matrix unit:
//
//   scores   S^T[token, row] = sum_d (off + c_td) (q s)_d          A = codes, B = folded query
//                            + sum_d z_d q_d - off * sum_d (q s)_d   the accumulator the product starts from
//   output   O[row, chan]    = sum_t (P s_g)[row, t] (off + c_t,chan)     A = P scaled per channel group (hi + remainder)
//                            - off * sum_t P[row, t] s_g[t]          extra tile, A = P, B = value scales
//                                                                    (float32 scale / zero: against ones, same A)
//                            + sum_t P[row, t] z_g[t]                same tile, B = value zeros
//   denominator               sum_t P[row, t]                        extra tile against ones
//
// Keys (per-channel scale s_d, zero z_d per token group): the scale is folded into
// the query, carried as an fp16 high part in columns [0, R) of the 16-wide tile and
// the exact fp16 remainder in columns [R, 2R), so the product is as accurate as a
// float32 one although keys carry outlier channels; the two columns are added with
// one DPP add per score.  The per-group row bias is itself a small MFMA chain
// (A = the group's zeros / a constant -off, B = the query) whose result seeds the
// score accumulators, so opening a token group costs no reductions.
//
// Values (per-token scale s_g[t], zero z_g[t] per channel group g): the scale is
// folded into the probabilities (fp16 product plus its exact fp16 remainder, so that a
// sharply peaked softmax still returns code*scale+zero to float32 accuracy).  A value
// tile covers 16 consecutive channels, which lie in one group.
//
// Query rows (the H_q/H_kv heads sharing the kv head) sit in the 16-wide M/N
// dimension.  Keys are packed along channels, so a lane's eight k-slots of the
// first product are eight channels of one token; values are packed along tokens
// (VQ_V_TOKEN_PACKED), so a lane's eight k-slots of the second product are eight
// tokens of one channel; token rows of the two score tiles interleave so that the
// accumulator layout of S^T is the A-operand layout of P.
//
// Every wave streams its units through its own ring of LDS slots, filled by copies
// that go from global memory straight into LDS and run DEPTH - 1 units ahead of the
// arithmetic: the bytes in flight per wave are set by the ring, not by the register
// file, and a unit is read into registers only when its turn comes.  The softmax
// keeps a lazily updated reference maximum, so the common path has no cross-lane
// traffic at all.
#pragma once
#include "attend_mfma.hpp"

namespace vq {

// One block of PK_WAVES waves per CU (two waves per SIMD, the register file split in two).
constexpr int PK_WAVES = 8;
constexpr int PK_THREADS = 64 * PK_WAVES;
// Every lambda below must be inlined at every call: a closure left in memory would be read back
// with vector loads, whose completion the ring's copy counter cannot tell from its own.
#define VQ_INLINE_LAMBDA __attribute__((always_inline))
#define VQ_MFMA(A, B, C) __builtin_amdgcn_mfma_f32_16x16x32_f16((A), (B), (C), 0, 0, 0)

// ---- value scale / zero of a lane's eight tokens (tA..tA+3, tB..tB+3)
template <typename M> struct TokMeta;
template <> struct TokMeta<f16> {
    uint2 a, b;
    __device__ __forceinline__ void read(const char *p, int gap_bytes) {
        a = *reinterpret_cast<const uint2 *>(p);
        b = *reinterpret_cast<const uint2 *>(p + gap_bytes);
    }
    // k-slot pair p = (token tA + p, token tB + p)
    __device__ __forceinline__ u32 pair(int p) const {
        const u32 x = p < 2 ? a.x : a.y, y = p < 2 ? b.x : b.y;
        return (p & 1) ? pair_hi(x, y) : pair_lo(x, y);
    }
};
template <> struct TokMeta<float> {
    float4 a, b;
    __device__ __forceinline__ void read(const char *p, int gap_bytes) {
        a = *reinterpret_cast<const float4 *>(p);
        b = *reinterpret_cast<const float4 *>(p + gap_bytes);
    }
    __device__ __forceinline__ float lo(int p) const { return p == 0 ? a.x : p == 1 ? a.y : p == 2 ? a.z : a.w; }
    __device__ __forceinline__ float hi(int p) const { return p == 0 ? b.x : p == 1 ? b.y : p == 2 ? b.z : b.w; }
};

// ---- key scale / zero of a lane's 32 channels for one token group, memory order
template <typename M> struct ChanMeta;
template <> struct ChanMeta<f16> {
    uint4 s[4], z[4];
    __device__ __forceinline__ void read(const char *sp, const char *zp) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s[j] = *reinterpret_cast<const uint4 *>(sp + 16 * j);
            z[j] = *reinterpret_cast<const uint4 *>(zp + 16 * j);
        }
    }
    __device__ __forceinline__ u32 sword(int w) const {   // channels 2w, 2w+1
        const uint4 &q = s[w / 4];
        return w % 4 == 0 ? q.x : w % 4 == 1 ? q.y : w % 4 == 2 ? q.z : q.w;
    }
    // {scale[lo], scale[hi]} for two channels of equal parity
    __device__ __forceinline__ u32 spair(int lo, int hi) const {
        return (lo & 1) ? pair_hi(sword(lo / 2), sword(hi / 2)) : pair_lo(sword(lo / 2), sword(hi / 2));
    }
};
template <> struct ChanMeta<float> {
    float4 s[8], z[8];
    __device__ __forceinline__ void read(const char *sp, const char *zp) {
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            s[j] = *reinterpret_cast<const float4 *>(sp + 16 * j);
            z[j] = *reinterpret_cast<const float4 *>(zp + 16 * j);
        }
    }
    static __device__ __forceinline__ float pick(const float4 &q, int e) { return e == 0 ? q.x : e == 1 ? q.y : e == 2 ? q.z : q.w; }
    __device__ __forceinline__ float sval(int ch) const { return pick(s[ch / 4], ch % 4); }
    __device__ __forceinline__ float zval(int ch) const { return pick(z[ch / 4], ch % 4); }
};

// Per-wave state of the packed kernel.  GV = channel groups per value row.
template <int GV, bool OFF_TILES> struct PackedAcc {
    f32x4 O[8];     // tile nt: channels 16*nt + n, still carrying off * sum_t (P s_g)[row, t]
    f32x4 Z;        // column g < GV: sum_t P[row, t] z_g[t]; column GV + g: sum_t P[row, t] s_g[t]
    f32x4 Off[OFF_TILES ? GV : 1];  // float32 scale / zero only: sum_t (P s_g)[row, t] from the same A operands, every column alike
    f32x4 L;        // sum_t P[row, t], every column alike
    float m_run;    // softmax reference, log2 domain, per lane column (query row)
};

template <int BITS, typename M, int GV> struct PackedUnit {
    u32 kw[2][(MF_D * BITS / 32) / 4];   // key words of the lane's 32 channels, two token rows
    u32 vw[8];                           // value words, one per 16-channel tile
    TokMeta<M> s[GV];                    // value scales of the lane's eight tokens, every group
    TokMeta<M> z;                        // lane column n < GV: value zeros of group n, else value scales of
                                         // group n % GV, of the lane's eight tokens
};

constexpr int MF_QIMG = 8 * 64;               // uint4 entries of the query image (below)
constexpr int MF_QIMG_BYTES = MF_QIMG * 16;

// A wave's ring: DEPTH unit slots, then GROUP_SLOTS group slots.  A unit slot holds what every
// unit needs, as it lies in memory:
//   key codes    32 tokens x 16*BITS bytes (4-bit: lane l's two 16-byte pieces at 16 l and 1024 + 16 l;
//                2-bit: the 16-byte piece lane l asked for at 16 l)
//   value codes  the unit's word rows, 512 bytes each
//   value scale rows (one per channel group, 32 tokens), then value zero rows
// A group slot holds the key scale and key zero (128 channels each) of a token group; the unit
// that opens a group brings them along.  Blocks start on a group boundary, so units open a
// group every UPG units and at most ceil(DEPTH / UPG) group slots are live at a time.
// The exchange arrays of the waves (tail, cross-wave merge) share the rings' bytes:
// accumulators [PK_WAVES][MF_ROWS][MF_D], zero-point sums [PK_WAVES][MF_ROWS][8], maxima and
// sums [PK_WAVES][MF_ROWS]
constexpr int EX_O = PK_WAVES * MF_ROWS * MF_D * 4, EX_Z = PK_WAVES * MF_ROWS * 8 * 4, EX_M = PK_WAVES * MF_ROWS * 4;
constexpr int EX_BYTES = EX_O + EX_Z + 2 * EX_M;
constexpr int PK_ALIGN = 128;                 // tokens: blocks start on a multiple of the largest token group

template <int BITS, typename M, int GV> struct Ring {
    static constexpr int MSZ = sizeof(M);
    static constexpr int KB = 512 * BITS, VB = 512 * BITS;
    static constexpr int VMR = GV * 32 * MSZ;      // bytes of the scale rows (and of the zero rows)
    static constexpr int KMR = MF_D * MSZ;         // bytes of a key scale (zero) row
    static constexpr int K_OFF = 0, V_OFF = KB, VS_OFF = KB + VB, VZ_OFF = VS_OFF + VMR;
    static constexpr int SLOT = VZ_OFF + VMR, GROUP_SLOT = 2 * KMR;
    // copies per unit, and per unit that opens a token group
    static constexpr int VM_COPIES = VMR > 256 ? VMR / 256 : 1, KM_COPIES = KMR / 256;
    static constexpr int UNIT_COPIES = (BITS == 4 ? 4 : 2) + 2 * VM_COPIES, GROUP_COPIES = 2 * KM_COPIES;
    static constexpr int UPG = 4 / GV;             // units per token group
    // the block has the CU's 160 KB to itself: the waves' rings next to the query image
    static constexpr int BUDGET = (160 * 1024 - MF_QIMG_BYTES - 256) / PK_WAVES;
    static constexpr int bytes_at(int depth) { return depth * SLOT + ((depth + UPG - 1) / UPG) * GROUP_SLOT; }
    // one slot in use, at least one in flight
    static constexpr int DEPTH = bytes_at(5) <= BUDGET ? 5 : bytes_at(4) <= BUDGET ? 4 : bytes_at(3) <= BUDGET ? 3 : 2;
    static constexpr int GROUP_SLOTS = (DEPTH + UPG - 1) / UPG;
    static constexpr int GROUP_OFF = DEPTH * SLOT;
    // copies issued after those of the unit about to be read: DEPTH - 1 later units, of which at
    // least (DEPTH - 1) / UPG open a group
    static constexpr int LATER = (DEPTH - 1) * UNIT_COPIES + ((DEPTH - 1) / UPG) * GROUP_COPIES;
    static constexpr int WAVE_BYTES = bytes_at(DEPTH);
    static constexpr int BYTES = PK_WAVES * WAVE_BYTES > EX_BYTES ? PK_WAVES * WAVE_BYTES : EX_BYTES;
    // Units are handed out to the waves in chunks of CHUNK consecutive units: whole token groups,
    // and at least DEPTH - 1 units, so that the copies never run more than one chunk ahead of
    // the arithmetic.
    static constexpr int CHUNK = ((DEPTH - 1 + UPG - 1) / UPG) * UPG;
};

// LDS image of the query, two operand forms of 4 k-steps x 64 lanes each:
//   [0..3]  memory order, rows in columns [0, R) only       (B operand of the zero-point product)
//   [4..7]  k-slot pair order, q in columns [0, R) and again in columns [R, 2R)
// so that  t = [4..7] * s  is the rounded product and  fma([4..7], s, -t)  its exact remainder;
// columns [0, R) keep the first, columns [R, 2R) the second.
template <int BITS>
__device__ __forceinline__ void build_query_image(const vq_attend_args &a, const RowTile &tile, int tid, f16 *s_qraw,
                                                  uint4 *s_q) {
    const int R = tile.RT;
    // raw rows: eight consecutive channels per thread, one load each
    for (int e = tid; e < MF_ROWS * MF_D / 8; e += PK_THREADS) {
        const int row = e / (MF_D / 8), d = 8 * (e % (MF_D / 8));
        f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (tile.valid(row)) {
            const int64_t i = tile.row(row) * MF_D + d;
            if (a.q_dtype == VQ_F16) v = *reinterpret_cast<const f16x8 *>((const f16 *)a.q + i);
            else {
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = (f16)ldq(a.q, a.q_dtype, i + j);
            }
        }
        *reinterpret_cast<f16x8 *>(s_qraw + 8 * e) = v;
    }
    __syncthreads();
    for (int e = tid; e < MF_QIMG; e += PK_THREADS) {
        const int form = e / 256, ks = (e / 64) % 4, l = e % 64;   // 256 entries per form
        const int n = l & 15, blk = l >> 4;
        const int rq = n < R ? n : n - R;
        const bool hi_col = n < R, lo_col = n >= R && n < 2 * R;
        f16 v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            int ch;
            if (form == 0) ch = 8 * ks + j;
            else ch = (j & 1) ? kchan_hi<BITS>(ks, j >> 1) : kchan_lo<BITS>(ks, j >> 1);
            const f16 q = (hi_col || lo_col) ? s_qraw[rq * MF_D + 32 * blk + ch] : (f16)0.f;
            v[j] = (form == 0 && !hi_col) ? (f16)0.f : q;
        }
        f16x8 o = {v[0], v[1], v[2], v[3], v[4], v[5], v[6], v[7]};
        s_q[e] = __builtin_bit_cast(uint4, o);
    }
    __syncthreads();
}

template <int BITS, typename M, int GV>
__device__ __forceinline__ void packed_units(const vq_attend_args &a, int64_t bh, int R, float c, int64_t t_begin,
                                             int n_units, int64_t lane_vis, int64_t full_vis, int lane, int wave,
                                             PackedAcc<GV, sizeof(M) != 2> &acc, const uint4 *s_q, char *ring,
                                             int *s_next, bool fixed_order) {
    constexpr int PER = 32 / BITS;           // codes per word
    constexpr int KW = MF_D / PER;           // key words per token row
    constexpr int KWL = KW / 4;              // key words one lane loads per token (its 32 channels)
    constexpr int GAP = vtok_gap<BITS>();
    constexpr int G = MF_D / GV;             // tokens per key group = channels per value group
    constexpr int TPG = 8 / GV;              // value tiles per channel group
    constexpr u32 MSZ = sizeof(M);
    const int n = lane & 15, blk = lane >> 4;
    const u32 magic = vreg_const(Magic<BITS>::bits);
    const int64_t cap = a.cap_tokens;

    // block-uniform bases, 32-bit per-lane byte offsets
    const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
    const char *vb = (const char *)a.v_packed + bh * (cap / PER) * MF_D * 4;
    const char *ksb = (const char *)a.k_scale + bh * (cap / G) * MF_D * MSZ;
    const char *kzb = (const char *)a.k_zero + bh * (cap / G) * MF_D * MSZ;
    const char *vsb = (const char *)a.v_scale + bh * GV * cap * MSZ;
    const char *vzb = (const char *)a.v_zero + bh * GV * cap * MSZ;

    using RG = Ring<BITS, M, GV>;
    using Unit = PackedUnit<BITS, M, GV>;
    char *wring = ring + wave * RG::WAVE_BYTES;
    const u32 wring_lds = lds_addr(wring);
    // ---- what a lane copies.  Key codes: token of S^T row n in tile T is vtok_lo(n / 4, n % 4) + T * GAP.
    //   4-bit: the lane's own 16 bytes (its 32 channels) of both token rows, two copies
    //   2-bit: one copy; lane (n, blk) fetches the 16-byte half blk / 2 of token row T = blk % 2
    const u32 koff = BITS == 4 ? (u32)((vtok_lo<BITS>(n >> 2, n & 3) * KW + KWL * blk) * 4)
                               : (u32)(((vtok_lo<BITS>(n >> 2, n & 3) + (blk & 1) * GAP) * KW + 4 * (blk >> 1)) * 4);
    // value codes, every scale / zero row: memory order, 16 (4) bytes per lane
    const u32 l16 = 16u * lane, l4 = 4u * lane;
    // value scale (zero) rows: byte 4*lane (+256 for a second copy) of the [GV][32] image, row g at g*cap
    constexpr int VROW = 32 * (int)MSZ;
    const u32 vmoff0 = (u32)((int64_t)(l4 / VROW) * cap * MSZ + l4 % VROW);
    const u32 vmoff1 = (u32)((int64_t)((256 + l4) / VROW) * cap * MSZ + (256 + l4) % VROW);
    constexpr u32 VM_ACTIVE = RG::VMR / 4 < 64 ? RG::VMR / 4 : 64;

    // a unit that opens a token group brings the group's key scale / zero along, into group slot `gslot`
    // blocks start on a token-group boundary; every byte offset of a unit fits 32 bits
    // (cap_tokens <= 2^24)
    const u32 unit0 = (u32)(t_begin / 32);
    auto issue_unit = [&](int u, int slot, bool opener, int gslot) VQ_INLINE_LAMBDA {
        const u32 ug = unit0 + (u32)u;   // unit number counted from token 0
        const u32 sl = wring_lds + (u32)slot * RG::SLOT;
        const char *kp = kb + ug * (u32)RG::KB;
        if constexpr (BITS == 4) {
            lds_copy16<0>(kp, koff, sl + RG::K_OFF);
            lds_copy16<GAP * KW * 4>(kp, koff, sl + RG::K_OFF + 1024 - GAP * KW * 4);
        } else {
            lds_copy16<0>(kp, koff, sl + RG::K_OFF);
        }
        const char *vp = vb + ug * (u32)RG::VB;
        lds_copy16<0>(vp, l16, sl + RG::V_OFF);
        if constexpr (BITS == 4) lds_copy16<1024>(vp, l16, sl + RG::V_OFF);
        const char *vsp = vsb + ug * (32 * MSZ), *vzp = vzb + ug * (32 * MSZ);
        if (VM_ACTIVE == 64 || lane < (int)VM_ACTIVE) {
            lds_copy4<0>(vsp, vmoff0, sl + RG::VS_OFF);
            lds_copy4<0>(vzp, vmoff0, sl + RG::VZ_OFF);
            if constexpr (RG::VM_COPIES == 2) {
                lds_copy4<0>(vsp, vmoff1, sl + RG::VS_OFF + 256);
                lds_copy4<0>(vzp, vmoff1, sl + RG::VZ_OFF + 256);
            }
        }
        if (opener) {
            const u32 goff = (ug / (u32)RG::UPG) * (u32)RG::KMR;
            const char *ksp = ksb + goff, *kzp = kzb + goff;
            const u32 gs = wring_lds + RG::GROUP_OFF + (u32)gslot * RG::GROUP_SLOT;
            lds_copy4<0>(ksp, l4, gs);
            lds_copy4<0>(kzp, l4, gs + RG::KMR);
            if constexpr (RG::KM_COPIES == 2) {
                lds_copy4<256>(ksp, l4, gs);
                lds_copy4<256>(kzp, l4, gs + RG::KMR);
            }
        }
    };

    // ---- what a lane reads back (ordinary LDS loads)
    const int vrow = BITS == 4 ? blk : blk >> 1;          // word row of the lane's eight tokens
    const u32 vshift = BITS == 2 ? 8u * (blk & 1) : 0u;
    const int tok_a = vtok_lo<BITS>(blk, 0);
    const int zrow = n < GV ? GV + n : n % GV;            // row of the [scale rows | zero rows] image
    auto read_unit = [&](int slot, Unit &d) VQ_INLINE_LAMBDA {
        const char *sl = wring + slot * RG::SLOT;
        if constexpr (BITS == 4) {
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                const uint4 x = *reinterpret_cast<const uint4 *>(sl + RG::K_OFF + 1024 * T + 16 * lane);
                d.kw[T][0] = x.x; d.kw[T][1] = x.y; d.kw[T][2] = x.z; d.kw[T][3] = x.w;
            }
        } else {
#pragma unroll
            for (int T = 0; T < 2; ++T) {
                const uint2 x = *reinterpret_cast<const uint2 *>(sl + RG::K_OFF + (16 * (2 * (blk >> 1) + T) + n) * 16 + 8 * (blk & 1));
                d.kw[T][0] = x.x; d.kw[T][1] = x.y;
            }
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
            d.vw[nt] = *reinterpret_cast<const u32 *>(sl + RG::V_OFF + vrow * 512 + (16 * nt + n) * 4);
#pragma unroll
        for (int g = 0; g < GV; ++g) d.s[g].read(sl + RG::VS_OFF + g * VROW + tok_a * (int)MSZ, GAP * (int)MSZ);
        d.z.read(sl + RG::VS_OFF + zrow * VROW + tok_a * (int)MSZ, GAP * (int)MSZ);
    };
    auto read_group = [&](int gslot, ChanMeta<M> &km) VQ_INLINE_LAMBDA {
        const char *gs = wring + RG::GROUP_OFF + gslot * RG::GROUP_SLOT;
        km.read(gs + 32 * blk * (int)MSZ, gs + RG::KMR + 32 * blk * (int)MSZ);
    };

    f16x8 qB[4];   // folded query of the open token group (high columns | remainder columns)
    f32x4 bias;    // what the score accumulators start from; every register alike
    const f16x8 ones = ones8();
    const f16x8 negoff = as_h8(Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair,
                               Magic<BITS>::neg_off_pair);

    auto open_group = [&](const ChanMeta<M> &km) VQ_INLINE_LAMBDA {
        f32x4 bt = {0.f, 0.f, 0.f, 0.f};
        if constexpr (sizeof(M) == 2) {
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) bt = VQ_MFMA(as_h8(km.z[ks]), as_h8(s_q[ks * 64 + lane]), bt);
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const uint4 qs = s_q[(4 + ks) * 64 + lane];
                const u32 qsw[4] = {qs.x, qs.y, qs.z, qs.w};
                u32 o[4];
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const f16x2 sp = as_h2(km.spair(kchan_lo<BITS>(ks, p), kchan_hi<BITS>(ks, p)));
                    const f16x2 t = as_h2(qsw[p]) * sp;   // round(q s)
                    // q*s has at most 22 significant bits: the remainder after the fp16
                    // high part is itself an fp16 number, so this fma is exact
                    const f16x2 rem = __builtin_elementwise_fma(as_h2(qsw[p]), sp, -t);
                    o[p] = n < R ? as_u(t) : as_u(rem);
                }
                qB[ks] = as_h8(o[0], o[1], o[2], o[3]);
            }
        } else {
            // float32 scale / zero: zeros split into an fp16 pair, the folded query formed
            // in float32 and split the same way
            f16x8 zh[4], zl[4];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks)
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const float z = km.zval(8 * ks + j);
                    zh[ks][j] = (f16)z;
                    zl[ks][j] = (f16)(z - (float)zh[ks][j]);
                }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const f16x8 qz = as_h8(s_q[ks * 64 + lane]);
                bt = VQ_MFMA(zh[ks], qz, bt);
                bt = VQ_MFMA(zl[ks], qz, bt);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const f16x8 qs = as_h8(s_q[(4 + ks) * 64 + lane]);
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int ch = (j & 1) ? kchan_hi<BITS>(ks, j >> 1) : kchan_lo<BITS>(ks, j >> 1);
                    const float t = (float)qs[j] * km.sval(ch);
                    const f16 hi = (f16)t;
                    const f16 lo = (f16)(t - (float)hi);
                    qB[ks][j] = n < R ? hi : lo;
                }
            }
        }
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) bt = VQ_MFMA(negoff, qB[ks], bt);
        bias = bt;
    };

    // ---- one unit: scores, softmax, output
    auto compute = [&](const Unit &cur, int64_t base) VQ_INLINE_LAMBDA {
        f32x4 S[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            f16x8 A[4];   // per k-step
            if constexpr (BITS == 4) {
                unpack8_pair<4>(cur.kw[T][0], cur.kw[T][1], magic, A[0], A[1]);
                unpack8_pair<4>(cur.kw[T][2], cur.kw[T][3], magic, A[2], A[3]);
            } else {   // word j holds k-steps 2j (low bytes) and 2j + 1 (high bytes)
                unpack8_pair<2>(cur.kw[T][0], cur.kw[T][1], magic, A[0], A[2]);
                unpack8_pair_upper2(cur.kw[T][0], cur.kw[T][1], magic, A[1], A[3]);
            }
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) S[T] = VQ_MFMA(A[ks], qB[ks], ks == 0 ? bias : S[T]);
        }
        // column n < R: add the remainder column n + R; other columns idle
#define VQ_ADD_SHL(N)                                                                         \
    _Pragma("unroll") for (int T = 0; T < 2; ++T) _Pragma("unroll") for (int r = 0; r < 4; ++r) \
        S[T][r] += row_shl<N>(S[T][r]);
        switch (R) {   // block-uniform
            case 1: VQ_ADD_SHL(1) break;
            case 2: VQ_ADD_SHL(2) break;
            case 4: VQ_ADD_SHL(4) break;
            case 8: VQ_ADD_SHL(8) break;
            default:
#pragma unroll
                for (int T = 0; T < 2; ++T)
#pragma unroll
                    for (int r = 0; r < 4; ++r) S[T][r] += __shfl(S[T][r], (lane & ~15) | ((n + R) & 15));
        }
#undef VQ_ADD_SHL
        // causal edge: tokens this lane's query row does not see (units below full_vis are
        // visible to every row of the tile)
        if (base + 32 > full_vis) {
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (base + vtok_lo<BITS>(blk, r) + T * GAP >= lane_vis) S[T][r] = -INFINITY;
        }

        // softmax against a lazily updated reference: the fast path touches no other lane
        const float mx = fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])),
                               fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
        if (__any(mx * c > acc.m_run + RESCALE_SLACK)) {
            float m_seen = mx * c;
            m_seen = fmaxf(m_seen, __shfl_xor(m_seen, 16));
            m_seen = fmaxf(m_seen, __shfl_xor(m_seen, 32));
            const float m_new = fmaxf(acc.m_run, m_seen);
            const float alpha = m_new == -INFINITY ? 1.f : exp2f(acc.m_run - m_new);   // 0 on the first unit
            float al[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * blk + r);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) acc.O[nt][r] *= al[r];
                acc.Z[r] *= al[r];
                acc.L[r] *= al[r];
                if constexpr (sizeof(M) != 2) {
#pragma unroll
                    for (int g = 0; g < GV; ++g) acc.Off[g][r] *= al[r];
                }
            }
            acc.m_run = m_new;
        }
        const float nm = acc.m_run == -INFINITY ? 0.f : -acc.m_run;   // a row with no visible token yet
        float Pf[2][4];
        u32 P[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            Pf[0][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[0][r], c, nm));
            Pf[1][r] = __builtin_amdgcn_exp2f(__builtin_fmaf(S[1][r], c, nm));
            P[r] = as_u(f16x2{(f16)Pf[0][r], (f16)Pf[1][r]});
        }
        const f16x8 P8 = as_h8(P[0], P[1], P[2], P[3]);

        // output: per channel group, A = P * s_g as an fp16 high part plus its exact fp16
        // remainder (P and s have 11 significant bits each), both multiplied into the codes
#pragma unroll
        for (int g = 0; g < GV; ++g) {
            u32 ah[4], al[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                if constexpr (sizeof(M) == 2) {
                    const f16x2 sp = as_h2(cur.s[g].pair(p));
                    const f16x2 hi = as_h2(P[p]) * sp;
                    ah[p] = as_u(hi);
                    al[p] = as_u(__builtin_elementwise_fma(as_h2(P[p]), sp, -hi));
                } else {
                    const float t0 = (float)as_h2(P[p])[0] * cur.s[g].lo(p), t1 = (float)as_h2(P[p])[1] * cur.s[g].hi(p);
                    const f16x2 hi = {(f16)t0, (f16)t1};
                    ah[p] = as_u(hi);
                    al[p] = as_u(f16x2{(f16)(t0 - (float)hi[0]), (f16)(t1 - (float)hi[1])});
                }
            }
            const f16x8 Ah = as_h8(ah[0], ah[1], ah[2], ah[3]), Al = as_h8(al[0], al[1], al[2], al[3]);
#pragma unroll
            for (int j = 0; j < TPG; j += 2) {
                const int nt = g * TPG + j;
                f16x8 Bv0, Bv1;
                if constexpr (BITS == 4) unpack8_pair<4>(cur.vw[nt], cur.vw[nt + 1], magic, Bv0, Bv1);
                else {
                    const u64 x = pack64(cur.vw[nt], cur.vw[nt + 1]) >> vshift;   // the lane's byte of each 16-token word
                    unpack8_pair<2>((u32)x, (u32)(x >> 32), magic, Bv0, Bv1);
                }
                acc.O[nt] = VQ_MFMA(Ah, Bv0, acc.O[nt]);
                acc.O[nt] = VQ_MFMA(Al, Bv0, acc.O[nt]);
                acc.O[nt + 1] = VQ_MFMA(Ah, Bv1, acc.O[nt + 1]);
                acc.O[nt + 1] = VQ_MFMA(Al, Bv1, acc.O[nt + 1]);
            }
            if constexpr (sizeof(M) != 2) {
                acc.Off[g] = VQ_MFMA(Ah, ones, acc.Off[g]);
                acc.Off[g] = VQ_MFMA(Al, ones, acc.Off[g]);
            }
        }
        if constexpr (sizeof(M) == 2) {
            acc.Z = VQ_MFMA(P8, as_h8(cur.z.pair(0), cur.z.pair(1), cur.z.pair(2), cur.z.pair(3)), acc.Z);
        } else {
            u32 zh[4], zl[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const f16x2 h = {(f16)cur.z.lo(p), (f16)cur.z.hi(p)};
                zh[p] = as_u(h);
                zl[p] = as_u(f16x2{(f16)(cur.z.lo(p) - (float)h[0]), (f16)(cur.z.hi(p) - (float)h[1])});
            }
            acc.Z = VQ_MFMA(P8, as_h8(zh[0], zh[1], zh[2], zh[3]), acc.Z);
            acc.Z = VQ_MFMA(P8, as_h8(zl[0], zl[1], zl[2], zl[3]), acc.Z);
        }
        acc.L = VQ_MFMA(P8, ones, acc.L);
    };

    // ---- the waves of a block draw chunks of CHUNK units from a shared counter (a wave that
    // is ahead simply draws more), so no wave waits for a slower one until the block's units are
    // used up.  Which wave meets which tokens then depends on timing, and with it the last bits
    // of the result; `fixed_order` deals the chunks round robin instead.  Copies run DEPTH - 1 units ahead of the arithmetic: `i_*` is where the copies are,
    // `c_*` where the arithmetic is.  Chunks being at least DEPTH - 1 units long (but for the
    // block's last), the copies have entered at most two chunks beyond the one being computed:
    // `c_next`, `c_after` queue them (NONE = nothing queued, END = the block has no more).
    constexpr int CH = RG::CHUNK;
    const int n_chunks = (n_units + CH - 1) / CH;
    int dealt = wave;   // fixed order: wave w takes chunks w, w + PK_WAVES, ...
    auto draw = [&]() VQ_INLINE_LAMBDA {   // the next chunk of the block; the value is used a chunk later
        int id = 0;
        if (fixed_order) id = (dealt += PK_WAVES);
        else if (lane == 0) id = __hip_atomic_fetch_add(s_next, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return id;
    };
    auto chunk_len = [&](int chunk) VQ_INLINE_LAMBDA { return n_units - chunk * CH < CH ? n_units - chunk * CH : CH; };
    if (wave >= n_chunks) return;   // the first PK_WAVES chunks are dealt out, the counter starts behind them
    constexpr int END = -1, NONE = -2;
    int i_chunk = wave, i_pos = 0, i_slot = 0, i_gslot = 0;
    int c_chunk = wave, c_pos = 0, c_next = NONE, c_after = NONE, c_slot = 0, c_gslot = 0;
    int in_flight = 0;
    int drawn = draw();
    auto issue_next = [&]() VQ_INLINE_LAMBDA {
        const bool opener = i_pos % RG::UPG == 0;   // chunks start on group boundaries
        issue_unit(i_chunk * CH + i_pos, i_slot, opener, i_gslot);
        i_slot = i_slot + 1 == RG::DEPTH ? 0 : i_slot + 1;
        const int g_next = i_gslot + 1 == RG::GROUP_SLOTS ? 0 : i_gslot + 1;
        i_gslot = opener ? g_next : i_gslot;
        ++in_flight;
        if (++i_pos == chunk_len(i_chunk)) {
            const int got = __builtin_amdgcn_readfirstlane(drawn);
            i_chunk = got < n_chunks ? got : END;
            i_pos = 0;
            if (c_next == NONE) c_next = i_chunk;
            else c_after = i_chunk;
            if (i_chunk >= 0) drawn = draw();
        }
    };
    // the first DEPTH - 1 passes only issue copies
    for (int pass = 1 - RG::DEPTH; c_chunk >= 0; ++pass) {
        if (i_chunk >= 0) issue_next();
        if (pass < 0) continue;
        // with a full ring exactly DEPTH - 1 units were issued behind the one awaited
        if (in_flight == RG::DEPTH) wait_copies<RG::LATER>();
        else wait_copies<0>();
        const int u = c_chunk * CH + c_pos;
        Unit cur;
        read_unit(c_slot, cur);
        const bool opens = c_pos % RG::UPG == 0;
        if (opens) {
            ChanMeta<M> km;
            read_group(c_gslot, km);
            open_group(km);
        }
        const int cg_next = c_gslot + 1 == RG::GROUP_SLOTS ? 0 : c_gslot + 1;
        c_gslot = opens ? cg_next : c_gslot;
        compute(cur, t_begin + (int64_t)u * 32);
        c_slot = c_slot + 1 == RG::DEPTH ? 0 : c_slot + 1;
        --in_flight;
        if (++c_pos == chunk_len(c_chunk)) {
            c_chunk = c_next;   // queued by then: the copies are ahead
            c_next = c_after;
            c_after = NONE;
            c_pos = 0;
        }
    }
}

// grid (nsplit, B*Hkv*tiles), PK_THREADS threads.  A block works on one tile of query rows (the GQA
// group at pq consecutive positions) and on packed tokens
// [max(0, x*split_len - tail_equiv), min(n_packed, (x+1)*split_len - tail_equiv)), cut to what the
// tile sees; block 0 first runs the fp16 tail, whose partial goes to slot nsplit.  With sync
// counters the block that finishes last for its tile merges the nparts partials into the output.
template <int BITS, typename M, int GV>
__global__ __launch_bounds__(PK_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attend_mfma_packed_kernel(vq_attend_args a, int64_t split_len, int64_t tail_equiv, int nparts, int pq, int tiles,
                               int fixed_order, float *__restrict__ ws) {
    __shared__ uint4 s_q[MF_QIMG];
    // the waves' rings; before and after the units the same bytes are the exchange buffer
    // s_o[PK_WAVES][MF_ROWS][MF_D] of the tail and of the cross-wave merge
    extern __shared__ __align__(16) char s_ring[];
    float (*s_o)[MF_ROWS][MF_D] = reinterpret_cast<float (*)[MF_ROWS][MF_D]>(s_ring);
    float (*s_z)[MF_ROWS][8] = reinterpret_cast<float (*)[MF_ROWS][8]>(s_ring + EX_O);
    float (*s_m)[MF_ROWS] = reinterpret_cast<float (*)[MF_ROWS]>(s_ring + EX_O + EX_Z);
    float (*s_l)[MF_ROWS] = reinterpret_cast<float (*)[MF_ROWS]>(s_ring + EX_O + EX_Z + EX_M);
    __shared__ int s_ticket, s_next;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: loops below stay scalar
    if (tid == 0) s_next = PK_WAVES;   // chunks 0 .. PK_WAVES - 1 are dealt to the waves up front
    const int n = lane & 15, blk = lane >> 4;
    const int by = blockIdx.y;
    const int sp = (int)blockIdx.x, nsplit = (int)gridDim.x;
    const int64_t bh = by / tiles;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    const float c = a.scale * LOG2E;

    RowTile tile;
    tile.R = (int)(a.Hq / a.Hkv);
    tile.RT = tile.R * pq;
    tile.pos0 = (int)(by % tiles) * pq;
    tile.Sq = a.Sq;
    tile.n_total = a.n_packed + a.n_tail;
    tile.causal = a.causal;
    tile.base_row = (b * a.Hq + hkv * tile.R) * a.Sq;
    const int RT = tile.RT;

    const bool single_launch = a.sync_counters != nullptr;
    // the raw query is staged in the (not yet used) output exchange buffer
    f16 *s_qraw = reinterpret_cast<f16 *>(&s_o[0][0][0]);
    build_query_image<BITS>(a, tile, tid, s_qraw, s_q);
    if (sp == 0 && a.k_new != nullptr && a.n_tail >= 1 && tid < 32) {
        // the newest token's key and value rows become the last tail row: 16 pieces of 16 bytes each
        const int piece = tid & 15;
        const bool val = tid >= 16;
        const uint4 *src = reinterpret_cast<const uint4 *>(val ? a.v_new : a.k_new) + bh * (MF_D / 8) + piece;
        uint4 *dst = reinterpret_cast<uint4 *>(const_cast<void *>(val ? a.v_tail : a.k_tail)) +
                     (bh * a.tail_cap + a.n_tail - 1) * (MF_D / 8) + piece;
        *dst = *src;
    }
    if (sp == 0 && nparts > nsplit)   // the launch has a tail slot: filled even when this sequence's tail is empty
        tail_block<PK_WAVES>(a, bh, tile, c, nsplit, nparts, ws, &s_m[0][0], &s_l[0][0], &s_o[0][0][0], s_qraw, tid,
                             wave, single_launch);

    PackedAcc<GV, sizeof(M) != 2> acc;
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) acc.O[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.Z = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.L = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.m_run = -INFINITY;
    if constexpr (sizeof(M) != 2) {
#pragma unroll
        for (int g = 0; g < GV; ++g) acc.Off[g] = f32x4{0.f, 0.f, 0.f, 0.f};
    }

    // packed tokens the rows of the tile see: all of them up to full_vis, none from max_vis on
    int64_t full_vis = tile.visible(0), max_vis = tile.visible(RT - 1);
    if (full_vis > a.n_packed) full_vis = a.n_packed;
    if (max_vis > a.n_packed) max_vis = a.n_packed;
    int64_t lane_vis = tile.visible(n < RT ? n : (n < 2 * RT ? n - RT : 0));
    if (lane_vis > a.n_packed) lane_vis = a.n_packed;

    int64_t t_begin = (int64_t)sp * split_len - tail_equiv;
    int64_t t_end = t_begin + split_len;
    if (t_begin < 0) t_begin = 0;
    if (t_end > (max_vis + 31) / 32 * 32) t_end = (max_vis + 31) / 32 * 32;
    const int n_units = t_end > t_begin ? (int)((t_end - t_begin) / 32) : 0;
    __syncthreads();   // the query staging and the tail are done with the ring's bytes
    packed_units<BITS, M, GV>(a, bh, RT, c, t_begin, n_units, lane_vis, full_vis, lane, wave, acc, s_q, s_ring,
                              &s_next, fixed_order != 0);
    __syncthreads();   // every wave has read its last slot

    // ---- merge the waves: accumulator register r of lane (n, blk) is row 4*blk + r,
    // tile nt column n is channel 16*nt + n
    if (blk == 0) s_m[wave][n] = acc.m_run;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int row = 4 * blk + r;
        if (row < RT) {
            if (n == 0) s_l[wave][row] = acc.L[r];
            if (n < 2 * GV) s_z[wave][row][n] = acc.Z[r];
#pragma unroll
            for (int nt = 0; nt < 8; ++nt)
                if constexpr (sizeof(M) == 2) s_o[wave][row][16 * nt + n] = acc.O[nt][r];
                else s_o[wave][row][16 * nt + n] = acc.O[nt][r] - Magic<BITS>::off * acc.Off[nt / (8 / GV)][r];
        }
    }
    __syncthreads();
    for (int e = tid; e < RT * MF_D; e += PK_THREADS) {
        const int row = e / MF_D, d = e % MF_D;
        if (!tile.valid(row)) continue;
        float gm = -INFINITY;
#pragma unroll
        for (int w = 0; w < PK_WAVES; ++w) gm = fmaxf(gm, s_m[w][row]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < PK_WAVES; ++w) {
            if (s_m[w][row] == -INFINITY) continue;   // a wave that had no unit, or saw nothing
            const float f = exp2f(s_m[w][row] - gm);
            const int g = d / (MF_D / GV);
            const float off_sum = sizeof(M) == 2 ? Magic<BITS>::off * s_z[w][row][GV + g] : 0.f;
            num += ((s_o[w][row][d] - off_sum) + s_z[w][row][g]) * f;
            den += s_l[w][row] * f;
        }
        float *o = ws + (tile.row(row) * nparts + sp) * MF_PART;
        st_partial(o + 2 + d, num, single_launch);
        if (d == 0) { st_partial(o, gm * LN2, single_launch); st_partial(o + 1, den, single_launch); }
    }

    // ---- last block of this tile merges the splits (no block ever waits for another).
    // Partials travel as device-scope (write-through) stores and device-scope loads, so no
    // cache-wide write-back or invalidate is needed.  What orders them against the ticket:
    // every thread waits until its own stores (these and the tail's) have been acknowledged
    // -- stores count in vmcnt on this target, and a barrier alone does not wait for them --
    // then the barrier collects the block, then one thread takes a ticket.  The merging
    // block's loads depend on the ticket's value, so they are issued after it returned.
    if (!single_launch) return;
    wait_copies<0>();
    __syncthreads();
    if (tid == 0)
        s_ticket = __hip_atomic_fetch_add(a.sync_counters + by, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    if (s_ticket != nsplit - 1) return;
    merge_rows(a, tile, nparts, ws, tid, PK_THREADS);
    if (tid == 0) __hip_atomic_store(a.sync_counters + by, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename M>
static void launch_mfma_packed(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    const dim3 grid((unsigned)p.nsplit, (unsigned)(a.B * a.Hkv * p.tiles)), block(PK_THREADS);
    const int gv = (int)(MF_D / a.group);
    // more than 64 KB of block-shared memory has to be allowed per kernel and device, once
#define VQ_LAUNCH(BITS, GV)                                                                                       \
    do {                                                                                                          \
        constexpr int ring_bytes = Ring<BITS, M, GV>::BYTES;                                                      \
        static bool allowed[64] = {};                                                                             \
        int dev = 0;                                                                                              \
        (void)hipGetDevice(&dev);                                                                                 \
        if (dev < 0 || dev >= 64 || !allowed[dev]) {                                                              \
            (void)hipFuncSetAttribute((const void *)attend_mfma_packed_kernel<BITS, M, GV>,                       \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, ring_bytes);                    \
            if (dev >= 0 && dev < 64) allowed[dev] = true;                                                        \
        }                                                                                                         \
        hipLaunchKernelGGL((attend_mfma_packed_kernel<BITS, M, GV>), grid, block, ring_bytes, st, a, p.split_len, \
                           p.tail_equiv, p.nparts, p.pq, p.tiles, p.fixed_order, ws);                             \
    } while (0)
    if (a.pack_bits == 4) {
        if (gv == 1) VQ_LAUNCH(4, 1); else if (gv == 2) VQ_LAUNCH(4, 2); else VQ_LAUNCH(4, 4);
    } else {
        if (gv == 1) VQ_LAUNCH(2, 1); else if (gv == 2) VQ_LAUNCH(2, 2); else VQ_LAUNCH(2, 4);
    }
#undef VQ_LAUNCH
}

}  // namespace vq
