// Vector-unit attention over [quantised prefix | tail] for the shapes the matrix-unit kernels do
// not take: any head_dim up to 256, any bit width 1..8 (3-bit words of ten codes included), both
// value layouts, any tail dtype.  Same semantics and partial format as attend_generic.hip
// (veloxquant_mlx/metal/src/scalar_affine_attend.metal:57-174: keys and values rebuilt as
// code * scale + zero in float32, online softmax, split partials merged afterwards), arranged so
// that the bytes of a kv head are read once for the query heads that share it:
//
//   * a block of four waves takes one kv head, a tile of up to four query rows (heads of the GQA
//     group x positions) and one split of the tokens;
//   * a lane owns CPL channels of a token row: the PER = 32 / bits codes of one packed word, or eight
//     of them where a word holds 16 or 32 (the accumulators of a lane are [row][channel] registers); the
//     LPT = 2^k >= D / CPL lanes of a token form a slot, a wave has 64 / LPT slots, and every
//     slot walks its own blocks of PER consecutive tokens (with token-packed values a block is
//     exactly the tokens one value word holds);
//   * no key is rebuilt: with the group's scale folded into the query (q s per channel, and
//     sum q z as the lane's share of the bias) a code costs one conversion and one fma per
//     query row; the slot's lanes add their shares with DPP moves and every lane ends up with
//     the token's scores;
//   * values likewise: the token's probability times its scale is formed once per row, a code
//     costs one fma per row into the lane's [row][channel] accumulators, zero points are summed
//     per row and added at the end;
//   * the reference maximum moves lazily (a branch the wave takes only when some score passes it).
#include "attend.hpp"
#include "attend_mfma.hpp"

namespace vq {

namespace {

constexpr int AR_NR = 4;   // query rows per block
// channels a lane owns for words of `per` codes
constexpr int ar_cpl(int per) { return per > 10 ? 8 : per; }

__device__ __forceinline__ float ar_ld(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}
// Eight 16-bit channels of a plain row (one 16-byte piece) as floats.
__device__ __forceinline__ void ar_piece8(const uint4 &v, int tag, float (&o)[8]) {
    const u32 w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        if (tag == VQ_F16) {
            const f16x2 h = __builtin_bit_cast(f16x2, w[j]);
            o[2 * j] = (float)h[0]; o[2 * j + 1] = (float)h[1];
        } else {
            o[2 * j] = __uint_as_float(w[j] << 16); o[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
        }
    }
}
template <int CTRL> __device__ __forceinline__ float ar_dpp(float x) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
// sum over the aligned group of `lpt` lanes (4, 8, 16, 32 or 64), left in every lane of the group
__device__ __forceinline__ float ar_slot_sum(float x, int lpt) {
    x += ar_dpp<0xB1>(x);                    // quad_perm [1,0,3,2]
    x += ar_dpp<0x4E>(x);                    // quad_perm [2,3,0,1]
    if (lpt >= 8) x += ar_dpp<0x141>(x);     // row_half_mirror
    if (lpt >= 16) x += ar_dpp<0x140>(x);    // row_mirror
    if (lpt >= 32) x += __shfl_xor(x, 16);
    if (lpt >= 64) x += __shfl_xor(x, 32);
    return x;
}

}  // namespace

// Rows of a tile: heads h0 .. h0 + R - 1 of the kv head's group at pq consecutive positions.
void rows_tiling(const vq_attend_args &a, int &pq, int &tiles) {
    const int64_t R = a.Hq / a.Hkv;
    pq = (a.Sq > 1 && R <= AR_NR && AR_NR % R == 0) ? (int)(AR_NR / R) : 1;
    const int64_t htiles = R > AR_NR ? cdiv(R, AR_NR) : 1;
    tiles = (int)(cdiv(a.Sq, pq) * htiles);
}

bool rows_kernel_supported(const vq_attend_args &a) {
    if (a.D < 8 || a.D > 256 || a.Hq % a.Hkv != 0) return false;
    if (!(a.scale > 0.f)) return false;
    int bits = 4;
    if (a.n_packed > 0) {
        bits = a.pack_bits;
        if (bits < 1 || bits > 8) return false;
        const int per = 32 / bits;
        if (a.group < ar_cpl(per)) return false;   // a lane's channels lie in at most two value groups
        if (a.v_layout == VQ_V_TOKEN_PACKED && a.cap_tokens % per != 0) return false;
    }
    const int64_t WL = cdiv(a.D, ar_cpl(32 / bits));   // lanes per token
    if (WL < 4 || WL > 64) return false;
    int pq, tiles;
    rows_tiling(a, pq, tiles);
    if (a.B * a.Hkv * (int64_t)tiles > 65535) return false;
    return true;
}

// NR: the rows a tile can hold (1 .. AR_NR): the per-row loops of a launch whose tiles are smaller shrink with it
template <int BITS, int NR>
__global__ __launch_bounds__(256) void attend_rows_kernel(vq_attend_args a, int64_t split_len, int pq, int tiles,
                                                          float *__restrict__ ws, int part0, int nparts) {
    constexpr int PER = 32 / BITS, CPL = ar_cpl(PER), SUBW = PER / CPL;   // SUBW lanes share a word
    constexpr uint32_t MASK = (1u << BITS) - 1u;
    __shared__ float s_q[NR][256];
    __shared__ float s_part[4][NR][258];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int sp = (int)blockIdx.x, nsplit = (int)gridDim.x, by = (int)blockIdx.y;
    const int64_t bh = by / tiles, hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    const int D = (int)a.D, g = a.k_packed != nullptr && a.group >= 1 ? (int)a.group : (1 << 30);   // plain rows: one group
    const int W = (D + PER - 1) / PER, WL = (D + CPL - 1) / CPL;   // words, lanes of a token row
    int lpt = 4;
    while (lpt < WL) lpt <<= 1;
    const int tps = 64 / lpt, slot = lane / lpt, w = lane % lpt;
    const bool live = w < WL;
    const int d0 = w * CPL, nch = !live ? 0 : (D - d0 < CPL ? D - d0 : CPL);
    const int kwi = w / SUBW, c0 = (w % SUBW) * CPL;   // the lane's word of a row, its first code in it

    RowTile tile;
    const int group = (int)(a.Hq / a.Hkv);
    const int htiles = group > AR_NR ? (group + AR_NR - 1) / AR_NR : 1;
    const int t_in_bh = by % tiles;
    tile.h0 = (t_in_bh % htiles) * AR_NR;
    tile.R = htiles > 1 ? (group - tile.h0 < AR_NR ? group - tile.h0 : AR_NR) : group;
    tile.RT = tile.R * pq;
    tile.pos0 = (t_in_bh / htiles) * pq;
    tile.Sq = a.Sq;
    tile.n_total = a.n_packed + a.n_tail;
    tile.causal = a.causal;
    tile.window = a.sliding_window;
    tile.base_row = (b * a.Hq + hkv * group) * a.Sq;

    // the tile's query rows as float32; rows the tile does not have are zeros and see nothing
    for (int e = tid; e < NR * D; e += 256) {
        const int r = e / D, d = e % D;
        s_q[r][d] = tile.valid(r) ? ar_ld(a.q, a.q_dtype, tile.row(r) * D + d) : 0.f;
    }
    __syncthreads();

    int64_t vis[NR], fst[NR];   // row r sees slots [fst, vis)
    int64_t t_lo = INT64_MAX, t_hi = 0;
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        vis[r] = tile.valid(r) ? tile.visible(r) : 0;
        fst[r] = tile.valid(r) ? tile.first(r) : 0;
        if (tile.valid(r)) {
            t_lo = fst[r] < t_lo ? fst[r] : t_lo;
            t_hi = vis[r] > t_hi ? vis[r] : t_hi;
        }
    }
    // part0 >= 0: this launch covers the tail tokens only and writes partial part0 + sp of nparts
    int64_t t0 = (part0 >= 0 ? a.n_packed : 0) + (int64_t)sp * split_len, t1 = t0 + split_len;
    if (t0 < t_lo) t0 = t_lo;
    if (t1 > t_hi) t1 = t_hi;
    // rows that see every token of [t0, t1) need no mask
    bool masked = false;
#pragma unroll
    for (int r = 0; r < NR; ++r)
        if (tile.valid(r) && (fst[r] > t0 || vis[r] < t1)) masked = true;

    float m[NR], l[NR], oz_lo[NR], oz_hi[NR], acc[NR][CPL];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        m[r] = -INFINITY;
        l[r] = oz_lo[r] = oz_hi[r] = 0.f;
#pragma unroll
        for (int j = 0; j < CPL; ++j) acc[r][j] = 0.f;
    }
    // value groups of the lane's channels: group `vg_lo` below channel index `jb`, the next one from there on
    const int vg_lo = d0 / g;
    const int jb = (vg_lo + 1) * g - d0;   // >= CPL when the lane's channels share one group
    const bool straddle = live && jb < nch;
    const int64_t GV = (D + g - 1) / g, GKcap = (a.cap_tokens + g - 1) / g;

    float qs[NR][CPL], kb[NR];
    int64_t cur_kg = -1;   // token group the folded query belongs to; -2: the tail (scale 1, zero 0)
    auto fold = [&](int64_t kg) {
        float s[CPL], z[CPL];
#pragma unroll
        for (int j = 0; j < CPL; ++j) {
            s[j] = 1.f;
            z[j] = 0.f;
            if (kg >= 0 && j < nch) {
                const int64_t mi = (bh * GKcap + kg) * D + d0 + j;
                s[j] = ar_ld(a.k_scale, a.meta_dtype, mi);
                z[j] = ar_ld(a.k_zero, a.meta_dtype, mi);
            }
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            float bsum = 0.f;
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                const float qv = j < nch ? s_q[r][d0 + j] : 0.f;
                qs[r][j] = qv * s[j];
                bsum = __builtin_fmaf(qv, z[j], bsum);
            }
            kb[r] = bsum;
        }
        cur_kg = kg;
    };

    // one token: codes (or plain values) kc of the lane's channels for the scores, vc for the output with the
    // token's value scale / zero per lane group
    auto token = [&](int64_t t, const float (&kc)[CPL], const float (&vc)[CPL], float vs_lo, float vz_lo, float vs_hi,
                     float vz_hi) {
        float s[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            float x = kb[r];
#pragma unroll
            for (int j = 0; j < CPL; ++j) x = __builtin_fmaf(qs[r][j], kc[j], x);
            s[r] = ar_slot_sum(x, lpt) * a.scale;
        }
        if (masked) {
#pragma unroll
            for (int r = 0; r < NR; ++r)
                if (t >= vis[r] || t < fst[r]) s[r] = -INFINITY;
        }
        bool up = false;
#pragma unroll
        for (int r = 0; r < NR; ++r) up |= s[r] > m[r];
        if (__any(up)) {
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                const float mn = fmaxf(m[r], s[r]);
                const float f = mn == -INFINITY ? 1.f : __expf(m[r] - mn);   // 0 when m was -inf
                m[r] = mn;
                l[r] *= f;
                oz_lo[r] *= f;
                oz_hi[r] *= f;
#pragma unroll
                for (int j = 0; j < CPL; ++j) acc[r][j] *= f;
            }
        }
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            const float p = s[r] == -INFINITY ? 0.f : __expf(s[r] - m[r]);
            l[r] += p;
            const float ps_lo = p * vs_lo, ps_hi = p * vs_hi;
            oz_lo[r] = __builtin_fmaf(p, vz_lo, oz_lo[r]);
            oz_hi[r] = __builtin_fmaf(p, vz_hi, oz_hi[r]);
#pragma unroll
            for (int j = 0; j < CPL; ++j) acc[r][j] = __builtin_fmaf(vc[j], (straddle && j >= jb) ? ps_hi : ps_lo, acc[r][j]);
        }
    };

    const int gslot = wave * tps + slot, nslots = 4 * tps;   // slots of the block
    const uint32_t *kp = (const uint32_t *)a.k_packed, *vp = (const uint32_t *)a.v_packed;
    const bool vtok = a.v_layout == VQ_V_TOKEN_PACKED;

    // ---- packed tokens of the split: blocks of PER consecutive tokens, dealt to the slots in turn
    const int64_t p1 = t1 < a.n_packed ? t1 : a.n_packed;
    if (t0 < p1) {
        const int64_t tb0 = t0 / PER, tb1 = (p1 + PER - 1) / PER;
        for (int64_t tb = tb0 + gslot; tb < tb1; tb += nslots) {
            uint32_t vw[CPL];   // token-packed values: the words of the lane's channels, PER tokens each
            if (vtok) {
#pragma unroll
                for (int j = 0; j < CPL; ++j) vw[j] = j < nch ? vp[(bh * (a.cap_tokens / PER) + tb) * D + d0 + j] : 0u;
            }
#pragma unroll 2
            for (int ii = 0; ii < PER; ++ii) {
                const int64_t t = tb * PER + ii;
                if (t < t0 || t >= p1) continue;   // the same for every lane of the slot
                if (t / g != cur_kg) fold(t / g);
                const uint32_t kw = live ? kp[(bh * a.cap_tokens + t) * W + kwi] : 0u;
                uint32_t vword = 0;
                float vs_lo, vz_lo, vs_hi = 0.f, vz_hi = 0.f;
                if (vtok) {
                    const int64_t mi = (bh * GV + (live ? vg_lo : 0)) * a.cap_tokens + t;
                    vs_lo = ar_ld(a.v_scale, a.meta_dtype, mi);
                    vz_lo = ar_ld(a.v_zero, a.meta_dtype, mi);
                    if (straddle) {
                        vs_hi = ar_ld(a.v_scale, a.meta_dtype, mi + a.cap_tokens);
                        vz_hi = ar_ld(a.v_zero, a.meta_dtype, mi + a.cap_tokens);
                    }
                } else {
                    vword = live ? vp[(bh * a.cap_tokens + t) * W + kwi] : 0u;
                    const int64_t mi = (bh * a.cap_tokens + t) * GV + (live ? vg_lo : 0);
                    vs_lo = ar_ld(a.v_scale, a.meta_dtype, mi);
                    vz_lo = ar_ld(a.v_zero, a.meta_dtype, mi);
                    if (straddle) {
                        vs_hi = ar_ld(a.v_scale, a.meta_dtype, mi + 1);
                        vz_hi = ar_ld(a.v_zero, a.meta_dtype, mi + 1);
                    }
                }
                float kc[CPL], vc[CPL];
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    kc[j] = (float)((kw >> ((c0 + j) * BITS)) & MASK);
                    vc[j] = vtok ? (float)((vw[j] >> (ii * BITS)) & MASK) : (float)((vword >> ((c0 + j) * BITS)) & MASK);
                }
                if (!live) { vs_lo = 0.f; vz_lo = 0.f; }
                token(t, kc, vc, vs_lo, vz_lo, vs_hi, vz_hi);
            }
        }
    }
    // ---- tail tokens of the split: plain rows, one token per slot and turn
    const int64_t q0 = t0 > a.n_packed ? t0 : a.n_packed;
    if (q0 < t1) {
        if (cur_kg != -2) fold(-2);
        // Lanes that own eight whole 16-bit channels (the head sizes that are multiples of 8) take their piece of a row
        // as one 16-byte load, and two tokens of a slot are requested before the first is used.
        const bool vec = CPL == 8 && a.tail_dtype != VQ_F32 && D % 8 == 0 && ((((uintptr_t)a.k_tail | (uintptr_t)a.v_tail) & 15u) == 0);
        if constexpr (CPL == 8) {
            if (vec) {
                const u16 *kt = (const u16 *)a.k_tail, *vt = (const u16 *)a.v_tail;
                for (int64_t t = q0 + gslot; t < t1; t += 2 * nslots) {
                    const bool two = t + nslots < t1;   // the same for the lanes of a slot
                    const int64_t ti = (bh * a.tail_cap + (t - a.n_packed)) * D + d0;
                    uint4 k0 = make_uint4(0, 0, 0, 0), v0 = k0, k1 = k0, v1 = k0;
                    if (live) {
                        k0 = *reinterpret_cast<const uint4 *>(kt + ti);
                        v0 = *reinterpret_cast<const uint4 *>(vt + ti);
                        if (two) {
                            k1 = *reinterpret_cast<const uint4 *>(kt + ti + (int64_t)nslots * D);
                            v1 = *reinterpret_cast<const uint4 *>(vt + ti + (int64_t)nslots * D);
                        }
                    }
                    float kc[8], vc[8];
                    ar_piece8(k0, a.tail_dtype, kc);
                    ar_piece8(v0, a.tail_dtype, vc);
                    token(t, kc, vc, 1.f, 0.f, 1.f, 0.f);
                    if (two) {
                        ar_piece8(k1, a.tail_dtype, kc);
                        ar_piece8(v1, a.tail_dtype, vc);
                        token(t + nslots, kc, vc, 1.f, 0.f, 1.f, 0.f);
                    }
                }
            }
        }
        if (!vec) {
            for (int64_t t = q0 + gslot; t < t1; t += nslots) {
                float kc[CPL], vc[CPL];
                const int64_t ti = (bh * a.tail_cap + (t - a.n_packed)) * D + d0;
#pragma unroll
                for (int j = 0; j < CPL; ++j) {
                    kc[j] = j < nch ? ar_ld(a.k_tail, a.tail_dtype, ti + j) : 0.f;
                    vc[j] = j < nch ? ar_ld(a.v_tail, a.tail_dtype, ti + j) : 0.f;
                }
                token(t, kc, vc, 1.f, 0.f, 1.f, 0.f);
            }
        }
    }

    // ---- zero points in, then the slots of the wave, then the waves of the block
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int j = 0; j < CPL; ++j) acc[r][j] += (straddle && j >= jb) ? oz_hi[r] : oz_lo[r];
    if (tps > 1) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            float mw = m[r];
            for (int off = lpt; off < 64; off <<= 1) mw = fmaxf(mw, __shfl_xor(mw, off));
            const float f = m[r] == -INFINITY ? 0.f : __expf(m[r] - mw);
            float lw = l[r] * f;
            for (int off = lpt; off < 64; off <<= 1) lw += __shfl_xor(lw, off);
#pragma unroll
            for (int j = 0; j < CPL; ++j) {
                float x = acc[r][j] * f;
                for (int off = lpt; off < 64; off <<= 1) x += __shfl_xor(x, off);
                acc[r][j] = x;
            }
            m[r] = mw;
            l[r] = lw;
        }
    }
    if (slot == 0 && live) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
#pragma unroll
            for (int j = 0; j < CPL; ++j)
                if (j < nch) s_part[wave][r][2 + d0 + j] = acc[r][j];
            if (w == 0) {
                s_part[wave][r][0] = m[r];
                s_part[wave][r][1] = l[r];
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < NR * (D + 2); e += 256) {
        const int r = e / (D + 2), c = e % (D + 2);
        if (!tile.valid(r)) continue;
        float gm = -INFINITY;
#pragma unroll
        for (int v = 0; v < 4; ++v) gm = fmaxf(gm, s_part[v][r][0]);
        float x = gm;
        if (c >= 1) {
            x = 0.f;
#pragma unroll
            for (int v = 0; v < 4; ++v)
                if (s_part[v][r][0] != -INFINITY) x += s_part[v][r][c] * __expf(s_part[v][r][0] - gm);
        }
        ws[(tile.row(r) * (part0 >= 0 ? nparts : nsplit) + (part0 >= 0 ? part0 : 0) + sp) * (D + 2) + c] = x;
    }
}

template <int BITS>
static void launch_rows_bits(const vq_attend_args &a, const AttendPlan &p, dim3 grid, hipStream_t st, float *ws) {
    const int64_t R = a.Hq / a.Hkv;
    const int rows = (int)((R > AR_NR ? AR_NR : R) * p.pq);   // rows of the largest tile
    switch (rows) {
        case 1: hipLaunchKernelGGL((attend_rows_kernel<BITS, 1>), grid, dim3(256), 0, st, a, p.split_len, p.pq, p.tiles, ws, p.part0, p.nparts); break;
        case 2: hipLaunchKernelGGL((attend_rows_kernel<BITS, 2>), grid, dim3(256), 0, st, a, p.split_len, p.pq, p.tiles, ws, p.part0, p.nparts); break;
        case 3: hipLaunchKernelGGL((attend_rows_kernel<BITS, 3>), grid, dim3(256), 0, st, a, p.split_len, p.pq, p.tiles, ws, p.part0, p.nparts); break;
        default: hipLaunchKernelGGL((attend_rows_kernel<BITS, 4>), grid, dim3(256), 0, st, a, p.split_len, p.pq, p.tiles, ws, p.part0, p.nparts); break;
    }
}

int launch_attend_rows_tail(const vq_attend_args &a, int part0, int nparts) {
    AttendPlan p = {};
    p.path = 3;
    rows_tiling(a, p.pq, p.tiles);
    p.nsplit = nparts - part0 > 1 ? nparts - part0 : 1;   // the partials past part0 are this launch's runs
    p.split_len = a.n_tail > 0 ? cdiv(a.n_tail, p.nsplit) : 1;
    p.nparts = nparts;
    p.part0 = part0;
    return launch_attend_rows(a, p);
}

int launch_attend_rows(const vq_attend_args &a, const AttendPlan &p) {
    const dim3 grid((unsigned)p.nsplit, (unsigned)(a.B * a.Hkv * p.tiles));
    hipStream_t st = (hipStream_t)a.stream;
    float *ws = (float *)a.workspace;
    switch (a.n_packed > 0 ? a.pack_bits : 4) {
        case 1: launch_rows_bits<1>(a, p, grid, st, ws); break;
        case 2: launch_rows_bits<2>(a, p, grid, st, ws); break;
        case 3: launch_rows_bits<3>(a, p, grid, st, ws); break;
        case 4: launch_rows_bits<4>(a, p, grid, st, ws); break;
        case 5: launch_rows_bits<5>(a, p, grid, st, ws); break;
        case 6: launch_rows_bits<6>(a, p, grid, st, ws); break;
        case 7: launch_rows_bits<7>(a, p, grid, st, ws); break;
        case 8: launch_rows_bits<8>(a, p, grid, st, ws); break;
        default: return VQ_ERR_UNSUPPORTED;
    }
    return VQ_OK;
}

}  // namespace vq
