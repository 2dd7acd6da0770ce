// MFMA decode attention over the packed prefix of a KIVI cache (gfx950, wave64).
//
// One block of eight waves per (kv head, token split), one block per CU.  Every wave streams
// units of 32 tokens and never reconstructs a key or a value: both products run on the raw
// codes.  A code stays where the (shifted) packed word holds it, inside the mantissa of an fp16
// SUBNORMAL -- one AND per two codes, value code * 2^(bit - 24), exact, no offset -- and the
// other operand of that k-slot carries the matching power of two (see Sub<BITS>):
//
//   scores   S^T[token, col]  = sum_d c_td (q s)_d 2^(EK - 24)     A = codes, B = folded query
//                             + 2^(EK - 24) sum_d z_d q_d            the accumulator the product starts from
//   output   O^T[chan, col]   = sum_t c_t,chan (P s_g)[t, col] 2^(EV - 24)   A = codes, B = P scaled by the
//                                                                    column's channel group (hi + remainder)
//   sums     Z[i, col]        = sum_t A_z[i, t] P[t, col]             rows i: value zeros of group i, ones
//                                                                    (the denominator)
//
// The 16 columns of a tile carry the RTP (4 or 8) query rows of the block several times over:
//   * first product: column n is query row n % RTP; columns with (n / RTP) even hold the fp16
//     high part of q*s, those with (n / RTP) odd its exact fp16 remainder, so the product is as
//     accurate as a float32 one although keys carry outlier channels.  One DPP add (rotate the
//     row of 16 lanes by RTP) gives EVERY column the full score of its row.
//   * second product: column n stands for (channel group (n / RTP) % GPP, row n % RTP): the lane
//     scales its probabilities by the value scale of ITS group only -- one operand serves all
//     channel groups at once, and a tile of 16 channels reads the columns of its own group.
//     (Per-token value scales cost 8 packed operations per unit this way, whatever the number
//     of groups.)
// Accumulators therefore sit as [channel][column]: a rescale of the running maximum is a
// per-lane factor, no cross-lane traffic.
//
// Opening a token group (keys: per-channel scale s_d, zero z_d per group of tokens) is shared
// work of the wave: every lane forms q*s (high part and remainder) for eight channels of one
// row, the pieces go through a small LDS image and come back in operand order; the row bias
// sum_d z_d q_d is one MFMA chain with the group's zeros in every operand row, so that each
// accumulator register of a lane holds the bias of the lane's column.
//
// Keys are packed along channels, so a lane's eight k-slots of the first product are eight
// channels of one token; values are packed along tokens (VQ_V_TOKEN_PACKED), so a lane's eight
// k-slots of the second product are eight tokens of one channel; token rows of the two score
// tiles interleave so that the accumulator layout of S^T is the B-operand layout of P.
//
// Every wave streams its units through its own ring of LDS slots, filled by copies that go
// from global memory straight into LDS: a slot is refilled as soon as its unit has been read
// into registers, so DEPTH units are in flight behind the arithmetic; the bytes in flight per
// wave are set by the ring, not by the register file.  The softmax keeps a lazily updated
// reference maximum, so the common path has no cross-lane traffic at all.
#pragma once
#include <atomic>

#include "attend_mfma.hpp"

namespace vq {


// One block per CU, of twelve waves (three per SIMD, 168 registers each) where twelve rings of at least
// two units fit the CU's LDS, of eight waves otherwise: Ring<...>::WAVES.  The unit loop is a chain of
// LDS round trips and dependent matrix products; the third wave of a SIMD fills what two leave idle.
constexpr int PK_MAX_WAVES = 12;
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

// How the 16 columns of the second product map to channel groups: GPP groups per probability
// operand, NP operands per unit, TPP value tiles (of 16 channels) per operand.
// GV counts the groups of the whole head (DH * 128 channels, NT = 8 * DH value tiles).
template <int GV, int RTP, int DH = 1> struct Cols {
    static constexpr int NT = 8 * DH;
    static constexpr int GPP = GV < 16 / RTP ? GV : 16 / RTP;
    static constexpr int NP = GV / GPP;
    static constexpr int TPG = NT / GV;
    static constexpr int TPP = NT / NP;
};

// Per-wave state of the packed kernel.
template <int NT = 8> struct PackedAcc {
    f32x4 O[NT];    // tile nt, register r: channel 16*nt + 4*blk + r of the lane's column, times 2^(EV - 24)
    f32x4 Z;        // register r = operand row 4*blk + r: sum_t P z_g (rows g < GV), sum_t P (rows >= 8)
    float m_run;    // softmax reference, log2 domain, of the lane's column (query row)
    float thr;      // m_run + SLACK: a score above it moves the reference
    float nm[4];    // what register r of a score tile adds before exp2: -m_run + (EV - pos(r)), the weight of
                    // its k-slot pair in the second product
};

template <int BITS, typename M, int NP, int DH = 1> struct PackedUnit {
    u32 kw[DH][2][(MF_D * BITS / 32) / 4];   // key words of the lane's 32 channels of every 128-channel half, two token rows
    u32 vw[8 * DH];                      // value words, one per 16-channel tile
    TokMeta<M> s[NP];                    // value scales of the lane's eight tokens, the lane's group of each operand
    TokMeta<M> z;                        // operand row of the sums product (see PackedAcc::Z)
};

constexpr int PK_QROW = 136;                  // halves between query rows in LDS (128 + 8: rows on different banks; a head of 256 channels: 264)
constexpr int PK_QIMG_ROW = 272;              // bytes between rows of a wave's folded-query image

// A wave's ring: DEPTH unit slots, then GROUP_SLOTS group slots, then the folded-query image.
// A unit slot holds what every unit needs, as it lies in memory:
//   key codes    32 tokens x 16*BITS bytes (4-bit: lane l's two 16-byte pieces at 16 l and 1024 + 16 l;
//                2-bit: the 16-byte piece lane l asked for at 16 l)
//   value codes  the unit's word rows, 512 bytes each
//   value scale rows (one per channel group, 32 tokens), then value zero rows
// A group slot holds the key scale and key zero (128 channels each) of a token group; the unit
// that opens a group brings them along.  Blocks start on a group boundary, so units open a
// group every UPG units.
// The exchange arrays of the waves (cross-wave merge) share the rings' bytes:
// accumulators [WAVES][MF_ROWS][MF_D], zero-point sums [WAVES][MF_ROWS][8], maxima and
// sums [WAVES][MF_ROWS]
constexpr int ex_o(int waves) { return waves * MF_ROWS * MF_D * 4; }
constexpr int ex_z(int waves) { return waves * MF_ROWS * 8 * 4; }
constexpr int ex_m(int waves) { return waves * MF_ROWS * 4; }
constexpr int ex_bytes(int waves) { return ex_o(waves) + ex_z(waves) + 2 * ex_m(waves); }
constexpr int PK_ALIGN = 128;                 // tokens: blocks start on a multiple of the largest token group
constexpr int PK_STATIC_LDS = 4096;           // query rows, constant rows, counters (static block-shared memory)

template <int BITS, typename M, int GV, int RTP, int DH = 1> struct Ring {
    static constexpr int MSZ = sizeof(M);
    static constexpr int KB = 512 * BITS * DH, VB = 512 * BITS * DH;
    static constexpr int VMR = GV * 32 * MSZ;      // bytes of the scale rows (and of the zero rows)
    static constexpr int KMR = MF_D * DH * MSZ;    // bytes of a key scale (zero) row
    static constexpr int K_OFF = 0, V_OFF = KB, VS_OFF = KB + VB, VZ_OFF = VS_OFF + VMR;
    static constexpr int SLOT = VZ_OFF + VMR, GROUP_SLOT = 2 * KMR;
    // copies per unit, and per unit that opens a token group
    static constexpr int VM_COPIES = VMR > 256 ? VMR / 256 : 1, KM_COPIES = KMR / 256;
    static constexpr int UNIT_COPIES = (BITS == 4 ? 4 : 2) * DH + 2 * VM_COPIES, GROUP_COPIES = 2 * KM_COPIES;
    static constexpr int UPG = (MF_D * DH / GV) / 32;   // units per token group
    static constexpr int QIMG = 2 * RTP * PK_QIMG_ROW * DH;
    // a group slot is read only while its group is opened, and refilled by the opener issued
    // ceil(DEPTH / UPG) openers later -- at the earliest in the same pass, after that read
    static constexpr int group_slots(int depth) { return (depth + UPG - 1) / UPG; }
    static constexpr int bytes_at(int depth) { return depth * SLOT + group_slots(depth) * GROUP_SLOT; }
    // the block has the CU's 160 KB to itself
    static constexpr int budget(int waves) { return (160 * 1024 - PK_STATIC_LDS * DH) / waves - QIMG; }
    // (float32 scale / zero: the unit loop holds more than a third of the register file, eight waves; a head of
    // 256 channels: 64 accumulator registers, eight waves, or four where eight rings of two units do not fit)
    static constexpr int WAVES = DH == 1 ? (MSZ == 2 && bytes_at(2) <= budget(PK_MAX_WAVES) ? PK_MAX_WAVES : 8)
                                         : (bytes_at(2) <= budget(8) ? 8 : 4);
    static constexpr int THREADS = 64 * WAVES;
    static constexpr int BUDGET = budget(WAVES);
    static constexpr int DEPTH = bytes_at(5) <= BUDGET ? 5 : bytes_at(4) <= BUDGET ? 4 : bytes_at(3) <= BUDGET ? 3 : 2;
    static_assert(bytes_at(DEPTH) <= BUDGET, "the rings do not fit the CU's LDS");
    static constexpr int GROUP_SLOTS = group_slots(DEPTH);
    static constexpr int GROUP_OFF = DEPTH * SLOT;
    static constexpr int QIMG_OFF = GROUP_OFF + GROUP_SLOTS * GROUP_SLOT;
    // copies issued after those of the unit about to be read: DEPTH - 1 later units, of which at
    // least (DEPTH - 1) / UPG open a group
    static constexpr int LATER = (DEPTH - 1) * UNIT_COPIES + ((DEPTH - 1) / UPG) * GROUP_COPIES;
    static constexpr int WAVE_BYTES = QIMG_OFF + QIMG;
    static constexpr int EX_BYTES = ex_o(WAVES) * DH + ex_z(WAVES) + 2 * ex_m(WAVES);
    static constexpr int BYTES = WAVES * WAVE_BYTES > EX_BYTES ? WAVES * WAVE_BYTES : EX_BYTES;
    // Units are handed out to the waves in chunks of CHUNK consecutive units: whole token groups,
    // and at least DEPTH units, so that the copies never run more than one chunk ahead of
    // the arithmetic.
    static constexpr int CHUNK = ((DEPTH + UPG - 1) / UPG) * UPG;
    static_assert(LATER < 64, "the outstanding-copy counter has six bits");
};

// The query rows of the block as fp16 in LDS, PK_QROW halves apart; rows the tile does not have are zero.
template <int RTP, int THREADS, int DH = 1>
__device__ __forceinline__ void stage_query(const vq_attend_args &a, const RowTile &tile, int tid, f16 *s_qraw) {
    constexpr int DD = MF_D * DH, PK_QROW = DD + 8;
    for (int e = tid; e < RTP * DD / 8; e += THREADS) {
        const int row = e / (DD / 8), d = 8 * (e % (DD / 8));
        f16x8 v = {0, 0, 0, 0, 0, 0, 0, 0};
        if (tile.valid(row)) {
            const int64_t i = tile.row(row) * DD + d;
            if (a.q_dtype == VQ_F16) v = *reinterpret_cast<const f16x8 *>((const f16 *)a.q + i);
            else {
#pragma unroll
                for (int j = 0; j < 8; ++j) v[j] = (f16)ldq(a.q, a.q_dtype, i + j);
            }
        }
        *reinterpret_cast<f16x8 *>(s_qraw + row * PK_QROW + d) = v;
    }
}

// value of lane (lane + N) % 16 of the same row of 16 lanes
template <int N> __device__ __forceinline__ float row_ror(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), 0x120 + N, 0xF, 0xF, true));
}

// order: bit 0 = deal the chunks round robin, bit 1 = wait for every copy in flight instead of the
// counted ones (a slower, count-free cross-check of the ring's accounting)
template <int BITS, typename M, int GV, int RTP, int DH = 1>
__device__ __forceinline__ void packed_units(const vq_attend_args &a, int64_t bh, float c, int64_t t_begin,
                                             int n_units, int lane_vis, int full_vis, int lane_lo, int lo_edge, int lane, int wave,
                                             PackedAcc<8 * DH> &acc, const f16 *s_qraw,
                                             const char *s_const, char *ring, int *s_next, int order) {
    using CL = Cols<GV, RTP, DH>;
    constexpr int DD = MF_D * DH;            // head size: DH halves of 128 channels, each worked like a head of 128
    constexpr int QROW = DD + 8;             // halves between query rows in LDS
    constexpr int PER = 32 / BITS;           // codes per word
    constexpr int KW = DD / PER;             // key words per token row
    constexpr int KWL = (MF_D / PER) / 4;    // key words one lane loads per token and half (its 32 channels)
    constexpr int HB = 16 * BITS;            // bytes of a half inside a token row of key codes
    constexpr int GAP = vtok_gap<BITS>();
    constexpr int G = DD / GV;               // tokens per key group = channels per value group
    constexpr u32 MSZ = sizeof(M);
    constexpr bool F32META = sizeof(M) != 2;
    using SB = Sub<BITS>;
    const int n = lane & 15, blk = lane >> 4;
    const float cs = c * SB::KSCALE;   // accumulated scores carry 2^(EK - 24)
    const int64_t cap = a.cap_tokens;
    const bool fixed_order = (order & 1) != 0, wait_all = (order & 2) != 0;

    // block-uniform bases, 32-bit per-lane byte offsets
    const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
    const char *vb = (const char *)a.v_packed + bh * (cap / PER) * DD * 4;
    const char *ksb = (const char *)a.k_scale + bh * (cap / G) * DD * MSZ;
    const char *kzb = (const char *)a.k_zero + bh * (cap / G) * DD * MSZ;
    const char *vsb = (const char *)a.v_scale + bh * GV * cap * MSZ;
    const char *vzb = (const char *)a.v_zero + bh * GV * cap * MSZ;

    using RG = Ring<BITS, M, GV, RTP, DH>;
    using Unit = PackedUnit<BITS, M, CL::NP, DH>;
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
    u32 vmoff[RG::VM_COPIES];   // copy c: byte 256 c + 4 lane of the image
#pragma unroll
    for (int cc = 0; cc < RG::VM_COPIES; ++cc)
        vmoff[cc] = (u32)((int64_t)((256 * cc + l4) / VROW) * cap * MSZ + (256 * cc + l4) % VROW);
    constexpr u32 VM_ACTIVE = RG::VMR / 4 < 64 ? RG::VMR / 4 : 64;

    // a unit that opens a token group brings the group's key scale / zero along, into group slot `gslot`
    // blocks start on a token-group boundary; every byte offset of a unit fits 32 bits
    // (cap_tokens <= 2^24)
    const u32 unit0 = (u32)(t_begin / 32);
    auto issue_unit = [&](int u, int slot, bool opener, int gslot) VQ_INLINE_LAMBDA {
        const u32 ug = unit0 + (u32)u;   // unit number counted from token 0
        const u32 sl = wring_lds + (u32)slot * RG::SLOT;
        const char *kp = kb + ug * (u32)RG::KB;
        // key codes: every half of the head lands as a head of 128 channels does, KB / DH bytes apart
#pragma unroll
        for (int h = 0; h < DH; ++h) {
            const u32 kh_lds = sl + RG::K_OFF + h * (RG::KB / DH);
            lds_copy16<0>(kp, koff + h * HB, kh_lds);
            if constexpr (BITS == 4) lds_copy16<GAP * KW * 4>(kp, koff + h * HB, kh_lds + 1024 - GAP * KW * 4);
        }
        // value codes: the unit's word rows as they lie in memory, a kilobyte a copy
        const char *vp = vb + ug * (u32)RG::VB;
        lds_copy16<0>(vp, l16, sl + RG::V_OFF);
        if constexpr (RG::VB >= 2048) lds_copy16<1024>(vp, l16, sl + RG::V_OFF);
        if constexpr (RG::VB >= 4096) {
            lds_copy16<2048>(vp, l16, sl + RG::V_OFF);
            lds_copy16<3072>(vp, l16, sl + RG::V_OFF);
        }
        const char *vsp = vsb + ug * (32 * MSZ), *vzp = vzb + ug * (32 * MSZ);
        if (VM_ACTIVE == 64 || lane < (int)VM_ACTIVE) {
#pragma unroll
            for (int cc = 0; cc < RG::VM_COPIES; ++cc) {
                lds_copy4<0>(vsp, vmoff[cc], sl + RG::VS_OFF + 256 * cc);
                lds_copy4<0>(vzp, vmoff[cc], sl + RG::VZ_OFF + 256 * cc);
            }
        }
        if (opener) {
            const u32 goff = (ug / (u32)RG::UPG) * (u32)RG::KMR;
            const char *ksp = ksb + goff, *kzp = kzb + goff;
            const u32 gs = wring_lds + RG::GROUP_OFF + (u32)gslot * RG::GROUP_SLOT;
            lds_copy4<0>(ksp, l4, gs);
            lds_copy4<0>(kzp, l4, gs + RG::KMR);
            if constexpr (RG::KM_COPIES >= 2) {
                lds_copy4<256>(ksp, l4, gs);
                lds_copy4<256>(kzp, l4, gs + RG::KMR);
            }
            if constexpr (RG::KM_COPIES >= 4) {
                lds_copy4<512>(ksp, l4, gs);
                lds_copy4<512>(kzp, l4, gs + RG::KMR);
                lds_copy4<768>(ksp, l4, gs);
                lds_copy4<768>(kzp, l4, gs + RG::KMR);
            }
        }
    };

    // ---- what a lane reads back (ordinary LDS loads)
    const int vrow = BITS == 4 ? blk : blk >> 1;          // word row of the lane's eight tokens
    // 2-bit: the lane's byte of each half of a 16-token word goes to mantissa bits 2..9: a rotation to
    // the right by 30 (up by two bits) for the lower byte, by 6 for the upper one
    const u32 vrot = (blk & 1) ? 6u : 30u;
    const int tok_a = vtok_lo<BITS>(blk, 0);
    // column n of the second product: channel group vgrp of every probability operand, query row n % RTP
    const int col_row = n % RTP, col_lo = (n / RTP) & 1, vgrp = (n / RTP) % CL::GPP;
    // operand row n of the sums product: zeros of group n, ones from row 8 on (rows GV .. 7 are not
    // used: they read the zeros of group 0).  Byte offset inside a slot, or inside the block's
    // constants when the row is ones.
    const bool zs_ones = n >= 8;
    const int zs_off = (zs_ones ? 0 : RG::VZ_OFF + (n < GV ? n : 0) * VROW) + tok_a * (int)MSZ;
    auto read_unit = [&](int slot, Unit &d) VQ_INLINE_LAMBDA {
        const char *sl = wring + slot * RG::SLOT;
#pragma unroll
        for (int h = 0; h < DH; ++h) {
            const char *kh = sl + RG::K_OFF + h * (RG::KB / DH);
            if constexpr (BITS == 4) {
#pragma unroll
                for (int T = 0; T < 2; ++T) {
                    const uint4 x = *reinterpret_cast<const uint4 *>(kh + 1024 * T + 16 * lane);
                    d.kw[h][T][0] = x.x; d.kw[h][T][1] = x.y; d.kw[h][T][2] = x.z; d.kw[h][T][3] = x.w;
                }
            } else {
#pragma unroll
                for (int T = 0; T < 2; ++T) {
                    const uint2 x = *reinterpret_cast<const uint2 *>(kh + (16 * (2 * (blk >> 1) + T) + n) * 16 + 8 * (blk & 1));
                    d.kw[h][T][0] = x.x; d.kw[h][T][1] = x.y;
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < CL::NT; ++nt)
            d.vw[nt] = *reinterpret_cast<const u32 *>(sl + RG::V_OFF + vrow * (4 * DD) + (16 * nt + n) * 4);
#pragma unroll
        for (int p = 0; p < CL::NP; ++p)
            d.s[p].read(sl + RG::VS_OFF + (p * CL::GPP + vgrp) * VROW + tok_a * (int)MSZ, GAP * (int)MSZ);
        d.z.read((zs_ones ? s_const : sl) + zs_off, GAP * (int)MSZ);
    };

    // ---- opening a token group
    // Writer role: lane w forms q * s for row w / 16 (+ 4 with eight rows), the eight channels of
    // k-step w % 4 of lane group (w / 4) % 4, and stores the high parts and the remainders as
    // 16-byte pieces of the folded-query image.  Reader role: lane (n, blk) fetches the four
    // pieces of its column.
    constexpr int WR = RTP / 4;                       // rows a lane writes
    const int w_row = lane >> 4, w_blk = (lane >> 2) & 3, w_ks = lane & 3;
    // first channel of the piece in k-slot pair order: pair p = (ch0 + p, ch0 + p + PAIR_GAP)
    constexpr int PAIR_GAP = BITS == 4 ? 4 : 8;
    const int w_ch0 = 32 * w_blk + (BITS == 4 ? 8 * w_ks : 16 * (w_ks >> 1) + 4 * (w_ks & 1));
    u32 qpair[DH][WR][4];
#pragma unroll
    for (int h = 0; h < DH; ++h)
#pragma unroll
        for (int u = 0; u < WR; ++u)
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const f16 *qr = s_qraw + (w_row + 4 * u) * QROW + MF_D * h + w_ch0 + p;
                // k-slot pair p of an operand sits at mantissa bit pos(p): its query side carries 2^(EK - pos(p))
                qpair[h][u][p] = as_u(f16x2{qr[0], qr[PAIR_GAP]} * h2(SB::wk(p)));
            }
    char *qimg = wring + RG::QIMG_OFF;
    constexpr int IMG = 2 * RTP * PK_QIMG_ROW;   // bytes of the folded-query image of one half
    const int w_off = w_row * PK_QIMG_ROW + w_blk * 64 + w_ks * 16;
    const int r_off = (col_lo * RTP + col_row) * PK_QIMG_ROW + blk * 64;
    // bias chain: every operand row carries the group's zeros; the query rows (high columns only;
    // remainder columns read zeros) are the other operand.  A head of 128 channels keeps them in registers;
    // a wider one, whose accumulators need the room, reads them again for every group.
    auto q_rows = [&](int h, int ks) VQ_INLINE_LAMBDA {
        f16x8 v = f16x8{0, 0, 0, 0, 0, 0, 0, 0};
        if (!col_lo) v = *reinterpret_cast<const f16x8 *>(s_qraw + col_row * QROW + MF_D * h + 32 * blk + 8 * ks);
        return v;
    };
    f16x8 q0[DH == 1 ? 4 : 1];
    if constexpr (DH == 1) {
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) q0[ks] = q_rows(0, ks);
    }

    f16x8 qB[DH][4];   // folded query of the open token group (high columns | remainder columns)
    f32x4 bias;    // what the score accumulators start from; every register alike

    auto open_group = [&](int gslot) VQ_INLINE_LAMBDA {
        const char *gs = wring + RG::GROUP_OFF + gslot * RG::GROUP_SLOT;
        f32x4 bt = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int h = 0; h < DH; ++h) {
            char *img = qimg + h * IMG;
            if constexpr (!F32META) {
                // ---- folded query, writer role
                u32 sp[4];
                const char *sh = gs + (MF_D * h + w_ch0) * 2;
                if constexpr (BITS == 4) {
                    const uint4 x = *reinterpret_cast<const uint4 *>(sh);
                    sp[0] = pair_lo(x.x, x.z); sp[1] = pair_hi(x.x, x.z); sp[2] = pair_lo(x.y, x.w); sp[3] = pair_hi(x.y, x.w);
                } else {
                    const uint2 x = *reinterpret_cast<const uint2 *>(sh);
                    const uint2 y = *reinterpret_cast<const uint2 *>(sh + 16);
                    sp[0] = pair_lo(x.x, y.x); sp[1] = pair_hi(x.x, y.x); sp[2] = pair_lo(x.y, y.y); sp[3] = pair_hi(x.y, y.y);
                }
#pragma unroll
                for (int u = 0; u < WR; ++u) {
                    u32 hi[4], lo[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const f16x2 t = as_h2(qpair[h][u][p]) * as_h2(sp[p]);   // round(q s)
                        // q*s has at most 22 significant bits: the remainder after the fp16
                        // high part is itself an fp16 number, so this fma is exact
                        hi[p] = as_u(t);
                        lo[p] = as_u(__builtin_elementwise_fma(as_h2(qpair[h][u][p]), as_h2(sp[p]), -t));
                    }
                    *reinterpret_cast<uint4 *>(img + w_off + 4 * u * PK_QIMG_ROW) = uint4{hi[0], hi[1], hi[2], hi[3]};
                    *reinterpret_cast<uint4 *>(img + w_off + (RTP + 4 * u) * PK_QIMG_ROW) = uint4{lo[0], lo[1], lo[2], lo[3]};
                }
                // ---- bias chain: the zeros of the lane's 32 channels in every operand row
                const char *zs = gs + RG::KMR + MF_D * h * 2 + 64 * blk;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks)
                    bt = VQ_MFMA(as_h8(*reinterpret_cast<const uint4 *>(zs + 16 * ks)), DH == 1 ? q0[DH == 1 ? ks : 0] : q_rows(h, ks), bt);
            } else {
                // float32 scale / zero: q * s formed in float32 and split into an fp16 pair
#pragma unroll
                for (int u = 0; u < WR; ++u) {
                    u32 hi[4], lo[4];
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const float s0 = *reinterpret_cast<const float *>(gs + (MF_D * h + w_ch0 + p) * 4);
                        const float s1 = *reinterpret_cast<const float *>(gs + (MF_D * h + w_ch0 + p + PAIR_GAP) * 4);
                        const float t0 = (float)as_h2(qpair[h][u][p])[0] * s0, t1 = (float)as_h2(qpair[h][u][p])[1] * s1;
                        const f16x2 hp = pinned_h2(f16x2{(f16)t0, (f16)t1});
                        hi[p] = as_u(hp);
                        lo[p] = as_u(f16x2{(f16)(t0 - (float)hp[0]), (f16)(t1 - (float)hp[1])});
                    }
                    *reinterpret_cast<uint4 *>(img + w_off + 4 * u * PK_QIMG_ROW) = uint4{hi[0], hi[1], hi[2], hi[3]};
                    *reinterpret_cast<uint4 *>(img + w_off + (RTP + 4 * u) * PK_QIMG_ROW) = uint4{lo[0], lo[1], lo[2], lo[3]};
                }
                // bias chain: the zeros as fp16 high parts, then their remainders, in every operand row
                const char *zs = gs + RG::KMR + MF_D * h * 4 + 128 * blk;
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) {
                    const float4 x0 = *reinterpret_cast<const float4 *>(zs + 32 * ks);
                    const float4 x1 = *reinterpret_cast<const float4 *>(zs + 32 * ks + 16);
                    const float x[8] = {x0.x, x0.y, x0.z, x0.w, x1.x, x1.y, x1.z, x1.w};
                    f16x8 oh, ol;
#pragma unroll
                    for (int j = 0; j < 8; ++j) {
                        const f16 hv = (f16)x[j];
                        oh[j] = hv;
                        ol[j] = (f16)(x[j] - (float)hv);
                    }
                    const f16x8 qr = DH == 1 ? q0[DH == 1 ? ks : 0] : q_rows(h, ks);
                    bt = VQ_MFMA(oh, qr, bt);
                    bt = VQ_MFMA(ol, qr, bt);
                }
            }
        }
        // every register of a lane holds sum z q of the lane's column; the score accumulators carry 2^(EK - 24)
#pragma unroll
        for (int r = 0; r < 4; ++r) bias[r] = bt[r] * SB::KSCALE_INV;
        // ---- folded query, reader role (the image is this wave's own: its LDS accesses run in order)
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int h = 0; h < DH; ++h)
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) qB[h][ks] = as_h8(*reinterpret_cast<const uint4 *>(qimg + h * IMG + r_off + 16 * ks));
    };

    // ---- one unit, first half: scores
    auto scores = [&](const Unit &cur, f32x4 (&S)[2]) VQ_INLINE_LAMBDA {
#pragma unroll
        for (int T = 0; T < 2; ++T) {
#pragma unroll
            for (int h = 0; h < DH; ++h) {
                f16x8 A[4];   // per k-step
                if constexpr (BITS == 4) {
                    sub_unpack4(cur.kw[h][T][0], cur.kw[h][T][1], A[0], A[1]);
                    sub_unpack4(cur.kw[h][T][2], cur.kw[h][T][3], A[2], A[3]);
                } else {   // word j holds k-steps 2j (codes 0-3 | 8-11) and 2j + 1 (codes 4-7 | 12-15)
                    sub_unpack2(cur.kw[h][T][0], cur.kw[h][T][1], A[0], A[1], A[2], A[3]);
                }
#pragma unroll
                for (int ks = 0; ks < 4; ++ks) S[T] = VQ_MFMA(A[ks], qB[h][ks], (h == 0 && ks == 0) ? bias : S[T]);
            }
        }
    };

    // ---- second half: softmax, output
    // lane_vis, full_vis, base: token positions counted from the block's first token
    const int lane_vis0 = lane_vis - tok_a;   // visible tokens counted from the lane's first token of a unit
    const int lane_lo0 = lane_lo - tok_a;     // first visible token (sliding window), counted the same way
    auto finish = [&](const Unit &cur, f32x4 (&S)[2], int base) VQ_INLINE_LAMBDA {
        // high + remainder column: every column ends up with the full score of its row
#pragma unroll
        for (int T = 0; T < 2; ++T)
#pragma unroll
            for (int r = 0; r < 4; ++r) S[T][r] += row_ror<RTP>(S[T][r]);
        // causal edge: tokens this lane's query row does not see (units below full_vis are
        // visible to every row of the tile); a real branch, taken by the last units of a block only
        // (and, under a sliding window, the first units of the sequence: tokens below lo_edge are
        // hidden from some row)
        if (base + 32 > full_vis || base < lo_edge) {
            asm volatile("" ::: "memory");
            const int lv = lane_vis0 - base, ll = lane_lo0 - base;
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (r + T * GAP >= lv || r + T * GAP < ll) S[T][r] = -INFINITY;
        }

        // softmax against a lazily updated reference: the fast path touches no other lane
        const float mx = max3_raw(max3_raw(S[0][0], S[0][1], S[0][2]), max3_raw(S[0][3], S[1][0], S[1][1]),
                                  max_raw(S[1][2], S[1][3]));
        if (__any(mx * cs > acc.thr)) {
            float m_seen = mx * cs;
            m_seen = fmaxf(m_seen, __shfl_xor(m_seen, 16));
            m_seen = fmaxf(m_seen, __shfl_xor(m_seen, 32));
            const float m_new = fmaxf(acc.m_run, m_seen);
            const float alpha = m_new == -INFINITY ? 1.f : exp2f(acc.m_run - m_new);   // 0 on the first unit
            // accumulators are [channel][column]: the factor is the lane's own
#pragma unroll
            for (int nt = 0; nt < CL::NT; ++nt)
#pragma unroll
                for (int r = 0; r < 4; ++r) acc.O[nt][r] *= alpha;
#pragma unroll
            for (int r = 0; r < 4; ++r) acc.Z[r] *= alpha;
            acc.m_run = m_new;
            acc.thr = m_new + SB::SLACK;
            const float nm = m_new == -INFINITY ? 0.f : -m_new;   // a row with no visible token yet
#pragma unroll
            for (int r = 0; r < 4; ++r) acc.nm[r] = nm + (float)(SB::EV - SB::pos(r));
        }
        // register r of either tile is k-slot pair r of the second product, whose codes sit at mantissa
        // bit pos(r): its probabilities carry 2^(EV - pos(r)), added in the exponent
        u32 P[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[0][r], cs, acc.nm[r]));
            const float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(S[1][r], cs, acc.nm[r]));
            P[r] = as_u(f16x2{(f16)p0, (f16)p1});
        }
        const f16x8 P8 = as_h8(P[0], P[1], P[2], P[3]);

        // output: B = P * s_g of the lane's channel group as an fp16 high part plus its exact fp16
        // remainder (P and s have 11 significant bits each), both multiplied into the codes
#pragma unroll
        for (int p = 0; p < CL::NP; ++p) {
            u32 bh[4], bl[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if constexpr (!F32META) {
                    const f16x2 sp = as_h2(cur.s[p].pair(j));
                    const f16x2 hi = as_h2(P[j]) * sp;
                    bh[j] = as_u(hi);
                    bl[j] = as_u(__builtin_elementwise_fma(as_h2(P[j]), sp, -hi));
                } else {
                    const float t0 = (float)as_h2(P[j])[0] * cur.s[p].lo(j), t1 = (float)as_h2(P[j])[1] * cur.s[p].hi(j);
                    const f16x2 hi = pinned_h2(f16x2{(f16)t0, (f16)t1});
                    bh[j] = as_u(hi);
                    bl[j] = as_u(f16x2{(f16)(t0 - (float)hi[0]), (f16)(t1 - (float)hi[1])});
                }
            }
            const f16x8 Bh = as_h8(bh[0], bh[1], bh[2], bh[3]), Bl = as_h8(bl[0], bl[1], bl[2], bl[3]);
#pragma unroll
            for (int j = 0; j < CL::TPP; j += 2) {
                const int nt = p * CL::TPP + j;
                f16x8 Av0, Av1;
                if constexpr (BITS == 4) sub_unpack4(cur.vw[nt], cur.vw[nt + 1], Av0, Av1);
                else {
                    Av0 = sub4<2>(__builtin_amdgcn_alignbit(cur.vw[nt], cur.vw[nt], vrot));
                    Av1 = sub4<2>(__builtin_amdgcn_alignbit(cur.vw[nt + 1], cur.vw[nt + 1], vrot));
                }
                acc.O[nt] = VQ_MFMA(Av0, Bh, acc.O[nt]);
                acc.O[nt + 1] = VQ_MFMA(Av1, Bh, acc.O[nt + 1]);
                acc.O[nt] = VQ_MFMA(Av0, Bl, acc.O[nt]);
                acc.O[nt + 1] = VQ_MFMA(Av1, Bl, acc.O[nt + 1]);
            }
        }
        // sums: operand rows = zeros of each group, ones; the weights of the probabilities are undone per
        // k-slot pair (exact powers of two)
        if constexpr (!F32META) {
            u32 zw[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) zw[j] = as_u(as_h2(cur.z.pair(j)) * h2(SB::wv_inv(j)));
            acc.Z = VQ_MFMA(as_h8(zw[0], zw[1], zw[2], zw[3]), P8, acc.Z);
        } else {
            u32 zh[4], zl[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const float z0 = cur.z.lo(j) * SB::wv_inv(j), z1 = cur.z.hi(j) * SB::wv_inv(j);
                const f16x2 h = {(f16)z0, (f16)z1};
                zh[j] = as_u(h);
                zl[j] = as_u(f16x2{(f16)(z0 - (float)h[0]), (f16)(z1 - (float)h[1])});
            }
            acc.Z = VQ_MFMA(as_h8(zh[0], zh[1], zh[2], zh[3]), P8, acc.Z);
            acc.Z = VQ_MFMA(as_h8(zl[0], zl[1], zl[2], zl[3]), P8, acc.Z);
        }
    };

    // ---- the waves of a block draw chunks of CHUNK units from a shared counter (a wave that
    // is ahead simply draws more), so no wave waits for a slower one until the block's units are
    // used up.  Which wave meets which tokens then depends on timing, and with it the last bits
    // of the result; `fixed_order` deals the chunks round robin instead.  Copies run DEPTH units
    // ahead of the arithmetic: `i_*` is where the copies are, `c_*` where the arithmetic is.
    // Chunks being at least DEPTH units long (but for the block's last), the copies have entered
    // at most two chunks beyond the one being computed: `c_next`, `c_after` queue them (NONE =
    // nothing queued, END = the block has no more).
    constexpr int CH = RG::CHUNK;
    const int n_chunks = (n_units + CH - 1) / CH;
    int dealt = wave;   // fixed order: wave w takes chunks w, w + WAVES, ...
    // 2-bit codes: every block starts its walk at a chunk of its own.  The blocks of a launch otherwise walk
    // identically laid-out heads in lockstep and their 256-byte scale / zero copies meet in the same memory
    // channels (3 % at 2 bits, where those copies are a third of the bytes; nothing at 4 bits).  Not under
    // `fixed_order`, whose results must not depend on a block's place in the grid (a layer-batched launch equals the
    // per-layer ones bit for bit there).
    const int rot = BITS == 2 && !fixed_order && n_chunks > 1 ? (int)((((unsigned)blockIdx.x * 2654435761u + (unsigned)blockIdx.y * 40503u) >> 12) % (unsigned)n_chunks) : 0;
    auto phys = [&](int id) VQ_INLINE_LAMBDA { const int q = id + rot; return q >= n_chunks ? q - n_chunks : q; };
    auto draw = [&]() VQ_INLINE_LAMBDA {   // the next chunk of the block; the value is used a chunk later
        int id = 0;
        if (fixed_order) id = (dealt += RG::WAVES);
        else if (lane == 0) id = __hip_atomic_fetch_add(s_next, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        return id;
    };
    auto chunk_len = [&](int chunk) VQ_INLINE_LAMBDA { return n_units - chunk * CH < CH ? n_units - chunk * CH : CH; };
    if (wave >= n_chunks) return;   // the first WAVES chunks are dealt out, the counter starts behind them
    constexpr int END = -1, NONE = -2;
    int i_chunk = phys(wave), i_pos = 0, i_slot = 0, i_gslot = 0;
    int c_chunk = i_chunk, c_pos = 0, c_next = NONE, c_after = NONE, c_slot = 0, c_gslot = 0;
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
            i_chunk = got < n_chunks ? phys(got) : END;
            i_pos = 0;
            if (c_next == NONE) c_next = i_chunk;
            else c_after = i_chunk;
            if (i_chunk >= 0) drawn = draw();
        }
    };
    // the ring is filled first; from then on a slot is refilled as soon as its unit sits in registers
    for (int d = 0; d < RG::DEPTH && i_chunk >= 0; ++d) issue_next();
    while (c_chunk >= 0) {
        // with a full ring exactly DEPTH - 1 units were issued behind the one awaited
        if (in_flight == RG::DEPTH && !wait_all) wait_copies<RG::LATER>();
        else wait_copies<0>();
        const int u = c_chunk * CH + c_pos;
        Unit cur;
        read_unit(c_slot, cur);
        const bool opens = c_pos % RG::UPG == 0;
        if (opens) open_group(c_gslot);
        const int cg_next = c_gslot + 1 == RG::GROUP_SLOTS ? 0 : c_gslot + 1;
        c_gslot = opens ? cg_next : c_gslot;
        f32x4 S[2];
        scores(cur, S);
        // everything of the slot (and of the group slot) has been read: refill it.  The wait is for
        // LDS reads only, whose results the products above already consumed or are about to.
        --in_flight;
        if (i_chunk >= 0) {
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            issue_next();
        }
        finish(cur, S, u * 32);
        c_slot = c_slot + 1 == RG::DEPTH ? 0 : c_slot + 1;
        if (++c_pos == chunk_len(c_chunk)) {
            c_chunk = c_next;   // queued by then: the copies are ahead
            c_next = c_after;
            c_after = NONE;
            c_pos = 0;
        }
    }
}

// grid (nsplit, B*Hkv*tiles), Ring<...>::THREADS threads.  A block works on one tile of query rows (the GQA
// group at pq consecutive positions; of a group of more than eight heads, eight at one position) and on packed tokens
// [max(0, x*split_len - tail_equiv), min(n_packed, (x+1)*split_len - tail_equiv)), cut to what the
// tile sees; in the block of split 0 the last nparts - nsplit waves first run the fp16 tail, each
// into a partial slot of its own.  With sync counters the block that finishes last for its tile
// merges the nparts partials into the output.
// DH = 2: a head of 256 channels, worked as two halves of 128 in the first product (eight k-steps into the same
// scores) and as sixteen value tiles in the second; GV counts the groups of the whole head.  Such a launch runs no
// tail waves (the fp16 tail comes as a partial of its own from the vector kernel) and takes no k_new / v_new.
template <int BITS, typename M, int GV, int RTP, int DH = 1, int WAVES = Ring<BITS, M, GV, RTP, DH>::WAVES>
__global__ __launch_bounds__(64 * WAVES) __attribute__((amdgpu_waves_per_eu(WAVES / 4, WAVES / 4)))
void attend_mfma_packed_kernel(vq_attend_args a, int64_t split_len, int64_t tail_equiv, int nparts, int pq, int tiles,
                               int order, float *__restrict__ ws) {
    using CL = Cols<GV, RTP, DH>;
    using RG = Ring<BITS, M, GV, RTP, DH>;
    constexpr int DD = MF_D * DH, QROW = DD + 8, PART = DD + 2;
    constexpr int PK_WAVES = RG::WAVES, PK_THREADS = RG::THREADS;
    constexpr int EX_O = ex_o(PK_WAVES) * DH, EX_Z = ex_z(PK_WAVES), EX_M = ex_m(PK_WAVES);
    // query rows of the block; constants: [0, 128) ones for 32 tokens in the scale / zero type, then zeros
    __shared__ __align__(16) f16 s_qraw[8 * QROW];
    __shared__ __align__(16) char s_const[512];
    // the waves' rings; after the units the same bytes are the exchange buffer
    // s_o[PK_WAVES][MF_ROWS][MF_D] of the cross-wave merge
    extern __shared__ __align__(16) char s_ring[];
    float (*s_o)[MF_ROWS][DD] = reinterpret_cast<float (*)[MF_ROWS][DD]>(s_ring);
    float (*s_z)[MF_ROWS][8] = reinterpret_cast<float (*)[MF_ROWS][8]>(s_ring + EX_O);
    float (*s_m)[MF_ROWS] = reinterpret_cast<float (*)[MF_ROWS]>(s_ring + EX_O + EX_Z);
    float (*s_l)[MF_ROWS] = reinterpret_cast<float (*)[MF_ROWS]>(s_ring + EX_O + EX_Z + EX_M);
    __shared__ int s_ticket, s_next;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: loops below stay scalar
    if (tid == 0) s_next = PK_WAVES;   // chunks 0 .. PK_WAVES - 1 are dealt to the waves up front
    if (tid < 128) {
        if (sizeof(M) == 2) reinterpret_cast<u32 *>(s_const)[tid] = tid < 16 ? 0x3C003C00u : 0u;
        else reinterpret_cast<u32 *>(s_const)[tid] = tid < 32 ? __float_as_uint(1.f) : 0u;
    }
    const int by = blockIdx.y;
    const int sp = (int)blockIdx.x, nsplit = (int)gridDim.x;
    const int64_t bh = by / tiles;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    const float c = a.scale * LOG2E;

    RowTile tile;
    const int group = (int)(a.Hq / a.Hkv);                 // query heads per kv head
    const int htiles = group > 8 ? (group + 7) / 8 : 1;   // more than eight: tiles of eight heads (pq is 1 then)
    const int t_in_bh = by % tiles;
    tile.h0 = (t_in_bh % htiles) * 8;
    tile.R = htiles > 1 ? (group - tile.h0 < 8 ? group - tile.h0 : 8) : group;
    tile.RT = tile.R * pq;
    tile.pos0 = (t_in_bh / htiles) * pq;
    tile.Sq = a.Sq;
    tile.n_total = a.n_packed + a.n_tail;
    tile.causal = a.causal;
    tile.window = a.sliding_window;
    tile.base_row = (b * a.Hq + hkv * group) * a.Sq;
    const int RT = tile.RT;

    const bool single_launch = a.sync_counters != nullptr;
    stage_query<RTP, PK_THREADS, DH>(a, tile, tid, s_qraw);
    if (DH == 1 && sp == 0 && a.k_new != nullptr && a.n_tail >= 1 && tid < 32) {
        // the newest token's key and value rows become the last tail row: 16 pieces of 16 bytes each
        const int piece = tid & 15;
        const bool val = tid >= 16;
        const uint4 *src = reinterpret_cast<const uint4 *>(val ? a.v_new : a.k_new) + bh * (MF_D / 8) + piece;
        uint4 *dst = reinterpret_cast<uint4 *>(const_cast<void *>(val ? a.v_tail : a.k_tail)) +
                     (bh * a.tail_cap + a.n_tail - 1) * (MF_D / 8) + piece;
        *dst = *src;
    }
    __syncthreads();
    // the launch has nparts - nsplit tail slots (filled even when this sequence's tail is empty): the
    // last waves of split 0 run the tail first, each into a slot of its own, while the others stream
    if constexpr (DH == 1) {
        const int tail_waves = nparts - nsplit;
        if (sp == 0 && wave >= PK_WAVES - tail_waves)
            tail_wave(a, bh, tile, c, nsplit + wave - (PK_WAVES - tail_waves), nparts, ws, s_qraw, PK_QROW, lane,
                      wave - (PK_WAVES - tail_waves), tail_waves, single_launch);
    }
    // what the unit loop derives from the lane number is formed from here on, not ahead of the tail: the tail
    // needs its 168 registers to itself
    int lane_u = lane;
    asm volatile("" : "+v"(lane_u));
    const int n = lane_u & 15, blk = lane_u >> 4;

    using SB = Sub<BITS>;
    PackedAcc<CL::NT> acc;
#pragma unroll
    for (int nt = 0; nt < CL::NT; ++nt) acc.O[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.Z = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.m_run = -INFINITY;
    acc.thr = -INFINITY;
#pragma unroll
    for (int r = 0; r < 4; ++r) acc.nm[r] = (float)(SB::EV - SB::pos(r));

    // packed tokens the rows of the tile see: all of them up to full_vis, none from max_vis on
    int64_t full_vis = tile.visible(0), max_vis = tile.visible(RT - 1);
    if (full_vis > a.n_packed) full_vis = a.n_packed;
    if (max_vis > a.n_packed) max_vis = a.n_packed;
    int64_t lane_vis = tile.visible(n % RTP < RT ? n % RTP : 0);
    if (lane_vis > a.n_packed) lane_vis = a.n_packed;

    int64_t t_begin = (int64_t)sp * split_len - tail_equiv;
    int64_t t_end = t_begin + split_len;
    if (t_begin < 0) t_begin = 0;
    if (t_end > (max_vis + 31) / 32 * 32) t_end = (max_vis + 31) / 32 * 32;
    const int n_units = t_end > t_begin ? (int)((t_end - t_begin) / 32) : 0;
    // visibility counted from the block's first token (a block holds fewer than 2^31 tokens)
    const int64_t rel_cap = (int64_t)n_units * 32 + 64;
    const int lane_rel = (int)(lane_vis - t_begin < 0 ? 0 : lane_vis - t_begin > rel_cap ? rel_cap : lane_vis - t_begin);
    const int full_rel = (int)(full_vis - t_begin < 0 ? 0 : full_vis - t_begin > rel_cap ? rel_cap : full_vis - t_begin);
    // sliding window: first token the lane's row sees, and the first token every row sees
    const int64_t lane_first = tile.first(n % RTP < RT ? n % RTP : 0) - t_begin, edge_first = tile.first(RT - 1) - t_begin;
    const int lo_rel = (int)(lane_first < 0 ? 0 : lane_first > rel_cap ? rel_cap : lane_first);
    const int edge_rel = (int)(edge_first < 0 ? 0 : edge_first > rel_cap ? rel_cap : edge_first);
    packed_units<BITS, M, GV, RTP, DH>(a, bh, c, t_begin, n_units, lane_rel, full_rel, lo_rel, edge_rel, lane_u, wave, acc, s_qraw, s_const,
                                   s_ring, &s_next, order);
    __syncthreads();   // every wave has read its last slot

    // ---- merge the waves.  Lane (n, blk): column n is query row n % RTP; tile nt, register r is
    // channel 16*nt + 4*blk + r, valid in the columns of the tile's channel group (first copy)
    const int col_row = n % RTP, col_set = n / RTP;
    if (n < RTP && blk == 0) s_m[wave][n] = acc.m_run;
    if (col_row < RT) {
#pragma unroll
        for (int nt = 0; nt < CL::NT; ++nt) {
            const int g = nt / CL::TPG;
            if (col_set == g % CL::GPP) {
#pragma unroll
                for (int r = 0; r < 4; ++r) s_o[wave][col_row][16 * nt + 4 * blk + r] = acc.O[nt][r] * SB::VSCALE;
            }
        }
        if (col_set == 0) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int i = 4 * blk + r;
                if (i < GV) s_z[wave][col_row][i] = acc.Z[r];
                if (i == 8) s_l[wave][col_row] = acc.Z[r];
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < RT * DD; e += PK_THREADS) {
        const int row = e / DD, d = e % DD;
        if (!tile.valid(row)) continue;
        float gm = -INFINITY;
#pragma unroll
        for (int w = 0; w < PK_WAVES; ++w) gm = fmaxf(gm, s_m[w][row]);
        float num = 0.f, den = 0.f;
#pragma unroll
        for (int w = 0; w < PK_WAVES; ++w) {
            if (s_m[w][row] == -INFINITY) continue;   // a wave that had no unit, or saw nothing
            const float f = exp2f(s_m[w][row] - gm);
            const int g = d / (DD / GV);
            num += (s_o[w][row][d] + s_z[w][row][g]) * f;
            den += s_l[w][row] * f;
        }
        float *o = ws + (tile.row(row) * nparts + sp) * PART;
        st_partial(o + 2 + d, num, single_launch);
        if (d == 0) { st_partial(o, gm * LN2, single_launch); st_partial(o + 1, den, single_launch); }
    }

    // ---- last block of this tile merges the splits (no block ever waits for another).
    // Partials travel as device-scope (write-through) stores and device-scope loads.  What
    // orders them against the ticket: every thread waits until its own stores (these and the
    // tail's) have been acknowledged -- stores count in vmcnt on this target, and a barrier
    // alone does not wait for them -- then the barrier collects the block, then one thread takes
    // a ticket with release-acquire ordering at device scope: the release publishes the block's
    // partials before the count moves, the acquire orders the merging block's loads after it
    // (the block barrier behind it extends that to the other threads).
    // A tile with a single run has no other block to count: the barrier has collected its own partials (the
    // packed one and the tail waves'; the tail launch of a 256-channel head ended before this one began).
    if (!single_launch) return;
    wait_copies<0>();
    __syncthreads();
    if (nsplit > 1) {
        if (tid == 0)
            s_ticket = __hip_atomic_fetch_add(a.sync_counters + by, 1, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        __syncthreads();
        if (s_ticket != nsplit - 1) return;
    }
    merge_rows<DH>(a, tile, nparts, ws, tid, PK_THREADS);
    if (nsplit > 1 && tid == 0) __hip_atomic_store(a.sync_counters + by, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

template <typename M, int RTP, int DH = 1>
static void launch_mfma_packed(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    const dim3 grid((unsigned)p.nsplit, (unsigned)(a.B * a.Hkv * p.tiles));
    const int gv = (int)(MF_D * DH / a.group);   // groups of the whole head
    // more than 64 KB of block-shared memory has to be allowed per kernel and device, once
#define VQ_LAUNCH(BITS, GV)                                                                                            \
    do {                                                                                                               \
        using RGL = Ring<BITS, M, GV, RTP, DH>;                                                                        \
        constexpr int ring_bytes = RGL::BYTES;                                                                         \
        static std::atomic<bool> allowed[64] = {};   /* set once per device; a second setter repeats the same call */ \
        int dev = 0;                                                                                                   \
        (void)hipGetDevice(&dev);                                                                                      \
        if (dev < 0 || dev >= 64 || !allowed[dev].load(std::memory_order_acquire)) {                                   \
            (void)hipFuncSetAttribute((const void *)attend_mfma_packed_kernel<BITS, M, GV, RTP, DH>,                   \
                                      hipFuncAttributeMaxDynamicSharedMemorySize, ring_bytes);                         \
            if (dev >= 0 && dev < 64) allowed[dev].store(true, std::memory_order_release);                             \
        }                                                                                                              \
        hipLaunchKernelGGL((attend_mfma_packed_kernel<BITS, M, GV, RTP, DH>), grid, dim3(RGL::THREADS),                \
                           ring_bytes, st, a, p.split_len,                                                             \
                           p.tail_equiv, p.nparts, p.pq, p.tiles, p.fixed_order, ws);                                  \
    } while (0)
    if (a.pack_bits == 4) {
        if (gv == DH) VQ_LAUNCH(4, DH); else if (gv == 2 * DH) VQ_LAUNCH(4, 2 * DH); else VQ_LAUNCH(4, 4 * DH);
    } else {
        if (gv == DH) VQ_LAUNCH(2, DH); else if (gv == 2 * DH) VQ_LAUNCH(2, 2 * DH); else VQ_LAUNCH(2, 4 * DH);
    }
#undef VQ_LAUNCH
}

}  // namespace vq
