// Multi-query (prefill) attention over the packed prefix of a KIVI cache on MFMA, with the
// packed tokens staged through LDS once per block of 64 query rows (gfx950, wave64).
//
// A block owns 64 query rows that share a kv head -- the GQA group at 64 / R consecutive
// query positions -- as four waves of 16 rows, and walks the packed prefix in units of 32
// tokens.  All 256 threads unpack the next unit into a double-buffered LDS tile while the
// matrix unit works on the current one:
//
//   keys     the 4-/2-bit codes become fp16 "offset + code" values (one and-or per two codes,
//            exact), channel order, [32 tokens][128 channels];
//   values   the same, transposed to [128 channels][32 tokens].
//
// Both products run on the raw codes exactly as in the decode kernel, so no reconstructed
// key or value is ever rounded to fp16.  Scores: the per-channel key scale of the open token
// group is folded into the wave's 16 query rows (fp16 high part plus exact fp16 remainder,
// two MFMAs into one accumulator), and the zero-point and offset terms seed the score
// accumulator through a short MFMA chain.  Output: the per-token value scale of each
// channel group is folded into the probabilities (high part plus exact remainder), the
// offset and zero-point terms are extra MFMA tiles.  S^T[token, row] accumulators are
// already the A operand of P.V; the softmax keeps a lazily updated reference maximum per
// row; the denominator is an extra MFMA tile against ones.  Each wave owns its rows for the
// whole run, so it writes its (max, sum, accumulator) partial straight to the workspace.
// The un-quantised tail follows the packed units through the same pipeline and the same
// code: its tiles hold plain keys and (transposed) plain values, and the scale / zero / offset
// staged with them are 1 / 0 / 0.  When there are
// fewer blocks than the chip holds twice over, the work of a block is split into runs
// handled by separate blocks; attend_merge_kernel combines the partials.
#include "attend_mfma.hpp"

namespace vq {

#define VQ_MFMA(A, B, C) __builtin_amdgcn_mfma_f32_16x16x32_f16((A), (B), (C), 0, 0, 0)

// Bare three-way maximum: the scores are never NaN, so the canonicalising moves the compiler
// wraps around fmaxf would only cost issue slots in the softmax.
__device__ __forceinline__ float vmax3(float a, float b, float c) {
    float d;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "v"(b), "v"(c));
    return d;
}

constexpr int PF_KSTRIDE = MF_D + 8;   // fp16 per token row of the key-code tile (272 B: conflict-free b128 reads)
constexpr int PF_VSTRIDE = 32 + 8;     // fp16 per channel row of the value tile (80 B)
// A unit (32 tokens of one kv head) as the 256-row blocks read it from LDS: the key tile (32 token rows of
// PF_KSTRIDE fp16, row pf_krow(token)) followed by the value tile (128 channel rows of PF_VSTRIDE fp16, tokens
// in order), padded to whole kilobytes.  vq_kivi_prefill_tiles writes units in this form to global memory; a
// launch that is given them copies them into LDS as they are.
constexpr int PF_TILE_KEYS = 32 * PF_KSTRIDE * 2;                  // bytes of the key tile
constexpr int PF_TILE_BYTES = 19 * 1024;                           // >= PF_TILE_KEYS + 128 * PF_VSTRIDE * 2
static_assert(PF_TILE_BYTES >= PF_TILE_KEYS + MF_D * PF_VSTRIDE * 2 && PF_TILE_BYTES == VQ_PREFILL_TILE_BYTES, "tile size");

// four k-slot pair registers of one unpacked word -> the same eight values in code order
__device__ __forceinline__ uint4 pairs_to_order(u32 r0, u32 r1, u32 r2, u32 r3) {
    return make_uint4(pair_lo(r0, r1), pair_lo(r2, r3), pair_hi(r0, r1), pair_hi(r2, r3));
}
template <int BITS> __device__ __forceinline__ void unpack_pairs(u32 w, u32 magic, u32 (&r)[4]) {
    const f16x8 h = unpack8<BITS>(w, magic);
    const u32x4 v = __builtin_bit_cast(u32x4, h);
    r[0] = v[0]; r[1] = v[1]; r[2] = v[2]; r[3] = v[3];
}
// One 4-bit word (8 codes) or one half of a 2-bit word -> values in code order.
// 4-bit: codes 0..7 of the word.  2-bit: lo = codes 0..7, hi = codes 8..15 of the word.
__device__ __forceinline__ uint4 word4_in_order(u32 w, u32 magic) {
    u32 r[4];
    unpack_pairs<4>(w, magic, r);   // pairs (0,4) (1,5) (2,6) (3,7)
    return pairs_to_order(r[0], r[1], r[2], r[3]);
}
__device__ __forceinline__ void word2_in_order(u32 w, u32 magic, uint4 &lo, uint4 &hi) {
    u32 a[4], b[4];
    unpack_pairs<2>(w, magic, a);        // pairs (0,8) (1,9) (2,10) (3,11)
    unpack_pairs<2>(w >> 8, magic, b);   // pairs (4,12) (5,13) (6,14) (7,15)
    lo = make_uint4(pair_lo(a[0], a[1]), pair_lo(a[2], a[3]), pair_lo(b[0], b[1]), pair_lo(b[2], b[3]));
    hi = make_uint4(pair_hi(a[0], a[1]), pair_hi(a[2], a[3]), pair_hi(b[0], b[1]), pair_hi(b[2], b[3]));
}

// packed words a thread fetches for one prefix unit before it unpacks them into LDS
template <int BITS> struct PfStage {
    u32 kw[BITS == 4 ? 2 : 1];   // key words: 16 channels of one token
    u32 vw[BITS == 4 ? 2 : 1];   // value words: 16 tokens of one channel
    uint4 meta;                  // threads 0..63: one 16-byte piece of the unit's scale / zero
};

// fp16 value scale / zero of a lane's eight consecutive tokens
template <int GV> struct PfMeta {
    uint4 s[GV];   // scales, every channel group (pair p = tokens 2p, 2p+1)
    uint4 z;       // lane column n < GV: zeros of group n; otherwise scales of group n % GV
};
__device__ __forceinline__ u32 u4_at(const uint4 &v, int p) { return p == 0 ? v.x : p == 1 ? v.y : p == 2 ? v.z : v.w; }

// token (0..31 of the unit) of S^T row i of tile T: accumulator register r of lane group blk is
// token 8 blk + 2 r + T, so a lane's P pairs are eight consecutive tokens
__device__ __forceinline__ int pf_tok(int blk, int r, int T) { return 8 * blk + 2 * r + T; }
// LDS row of token t in the key tile: even tokens first, so that the sixteen rows one score
// tile reads (tokens of equal parity) are consecutive and the b128 reads are conflict-free
__device__ __forceinline__ int pf_krow(int t) { return (t >> 1) + 16 * (t & 1); }

// grid (tiles, B*Hkv, nsplit).  The work of a block -- the packed units its rows see, then the
// tail units -- is cut into nsplit equal runs; block z takes run z and writes partial slot z.
// Scale / zero are fp16 (GV = channel groups per value row).
template <int BITS, int GV>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attend_prefill_kernel(vq_attend_args a, int qp, int nparts, float *__restrict__ ws) {
    __shared__ __align__(16) f16 s_k[2][32 * PF_KSTRIDE];
    __shared__ __align__(16) f16 s_v[2][MF_D * PF_VSTRIDE];
    // What turns the unit's tile into keys and values, staged with it: keys [scale | zero |
    // minus the code offset][128 channels] of its token group, values [scale | zero | scale as
    // the offset correction sees it][GV][32 tokens].  A tail unit holds plain values: scale 1,
    // zero 0, no offset.
    __shared__ __align__(16) f16 s_km[2][3][MF_D];
    __shared__ __align__(16) f16 s_vm[2][3][GV][32];

    constexpr int PER = 32 / BITS;
    constexpr int KW = MF_D / PER;
    constexpr int gshift = GV == 4 ? 5 : GV == 2 ? 6 : 7;   // log2 of the group size
    constexpr int TPG = 8 / GV;                             // value tiles per channel group
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, blk = lane >> 4;
    const int64_t bh = blockIdx.y;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t cap = a.cap_tokens;
    const float c = a.scale * LOG2E;
    const u32 magic = vreg_const(Magic<BITS>::bits);
    // under a causal mask the last tiles see the most tokens: they are started first
    const int pos0 = (int)(a.causal ? gridDim.x - 1 - blockIdx.x : blockIdx.x) * qp;
    const int64_t n_total = a.n_packed + a.n_tail;

    // ---- this lane's query row (as a score column): row j = 16 wave + n of the block
    const int j = 16 * wave + n;
    const int64_t pos = pos0 + j % qp;
    const bool row_ok = pos < a.Sq;
    const int64_t qrow = (b * a.Hq + hkv * R + j / qp) * a.Sq + (row_ok ? pos : a.Sq - 1);
    auto visible = [&](int64_t p) { return a.causal ? n_total - a.Sq + p + 1 : n_total; };   // slots row p sees
    const int64_t last_pos = pos0 + qp - 1 < a.Sq - 1 ? pos0 + qp - 1 : a.Sq - 1;
    const int64_t vis_lane = visible(row_ok ? pos : a.Sq - 1), vis_min = visible(pos0), vis_max = visible(last_pos);
    // packed tokens / tail tokens seen by this lane's row, by every row, by some row of the block
    const int lane_vis = (int)(vis_lane < a.n_packed ? vis_lane : a.n_packed);
    const int full_vis = (int)(vis_min < a.n_packed ? vis_min : a.n_packed);
    const int max_vis = (int)(vis_max < a.n_packed ? vis_max : a.n_packed);
    const int64_t tv_lane = vis_lane - a.n_packed, tv_min = vis_min - a.n_packed, tv_max = vis_max - a.n_packed;
    const int lane_tvis = (int)(tv_lane < 0 ? 0 : tv_lane < a.n_tail ? tv_lane : a.n_tail);
    const int full_tvis = (int)(tv_min < 0 ? 0 : tv_min < a.n_tail ? tv_min : a.n_tail);
    const int max_tvis = (int)(tv_max < 0 ? 0 : tv_max < a.n_tail ? tv_max : a.n_tail);
    const int n_punits = (max_vis + 31) / 32;
    const int n_tunits = (max_tvis + 31) / 32;
    const int n_work = n_punits + n_tunits;
    const int nsplit = (int)gridDim.z, sp = (int)blockIdx.z;
    // units below the window of the block's first row are seen by none of its rows
    const int64_t first_blk = window_first(a, n_total, pos0);
    const int w_lo = first_blk < a.n_packed ? (int)(first_blk / 32) : n_punits + (int)((first_blk - a.n_packed) / 32);
    const int w_n = n_work > w_lo ? n_work - w_lo : 0;
    const int w0 = w_lo + (int)((int64_t)w_n * sp / nsplit), w1 = w_lo + (int)((int64_t)w_n * (sp + 1) / nsplit);
    // sliding window: first packed / tail token this lane's row sees, and the first every row sees
    const int64_t first_lane = window_first(a, n_total, row_ok ? pos : a.Sq - 1), first_all = window_first(a, n_total, last_pos);
    const int lane_lo = (int)(first_lane < a.n_packed ? first_lane : a.n_packed);
    const int edge_lo = (int)(first_all < a.n_packed ? first_all : a.n_packed);
    const int lane_tlo = (int)(first_lane > a.n_packed ? first_lane - a.n_packed : 0);
    const int edge_tlo = (int)(first_all > a.n_packed ? first_all - a.n_packed : 0);

    // query as the B operand: lane (n, blk) holds channels 32 ks + 8 blk + 0..7 of row n
    f16x8 qn[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int e = 0; e < 8; ++e) qn[ks][e] = (f16)ldq(a.q, a.q_dtype, qrow * MF_D + 32 * ks + 8 * blk + e);

    // ---- producer side: block-uniform bases, per-thread offsets
    const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
    const char *vb = (const char *)a.v_packed + bh * (cap / PER) * MF_D * 4;
    const f16 *ksb = (const f16 *)a.k_scale + bh * (cap >> gshift) * MF_D;
    const f16 *kzb = (const f16 *)a.k_zero + bh * (cap >> gshift) * MF_D;
    const f16 *vsb = (const f16 *)a.v_scale + bh * GV * cap;
    const f16 *vzb = (const f16 *)a.v_zero + bh * GV * cap;
    const int kt = tid >> 3, kc = tid & 7;        // key tile: token, 16-channel chunk
    const int vc = tid & 127, vh = tid >> 7;      // value tile: channel, 16-token half
    const bool tail_bf16 = a.tail_dtype == VQ_BF16;
    const int64_t tbase = bh * a.tail_cap * MF_D;
    using Stage = PfStage<BITS>;
    auto fetch = [&](int w, Stage &st) {   // packed work units only
        if (w >= n_punits) return;
        const int64_t base = (int64_t)w * 32;
        if (BITS == 4) {
            const uint2 x = *reinterpret_cast<const uint2 *>(kb + ((base + kt) * KW + 2 * kc) * 4);
            st.kw[0] = x.x; st.kw[BITS == 4 ? 1 : 0] = x.y;
            const char *p = vb + ((base / 8 + 2 * vh) * MF_D + vc) * 4;
            st.vw[0] = *reinterpret_cast<const u32 *>(p);
            st.vw[BITS == 4 ? 1 : 0] = *reinterpret_cast<const u32 *>(p + MF_D * 4);
        } else {
            st.kw[0] = *reinterpret_cast<const u32 *>(kb + ((base + kt) * KW + kc) * 4);
            st.vw[0] = *reinterpret_cast<const u32 *>(vb + ((base / 16 + vh) * MF_D + vc) * 4);
        }
        if (tid < 32) {          // key scale (pieces 0..15) and zero (16..31) of the unit's token group
            const f16 *src = (tid < 16 ? ksb : kzb) + (base >> gshift) * MF_D + 8 * (tid & 15);
            st.meta = *reinterpret_cast<const uint4 *>(src);
        } else if (tid < 32 + 12 * GV) {   // value scale | zero | scale again: piece = (which, group, 8-token chunk)
            const int pc = tid - 32, which = pc / (4 * GV), g = (pc / 4) % GV, ch = pc % 4;
            st.meta = *reinterpret_cast<const uint4 *>((which == 1 ? vzb : vsb) + (int64_t)g * cap + base + 8 * ch);
        }
    };
    auto unpack_to_lds = [&](int w, const Stage &st, int buf) {
        if (w < n_punits) {
            // keys: 16 channels of token kt
            uint4 k0, k1;
            if (BITS == 4) { k0 = word4_in_order(st.kw[0], magic); k1 = word4_in_order(st.kw[BITS == 4 ? 1 : 0], magic); }
            else word2_in_order(st.kw[0], magic, k0, k1);
            uint4 *kd = reinterpret_cast<uint4 *>(&s_k[buf][pf_krow(kt) * PF_KSTRIDE + 16 * kc]);
            kd[0] = k0; kd[1] = k1;
            // values: 16 tokens of channel vc, still codes
            uint4 c0, c1;
            if (BITS == 4) { c0 = word4_in_order(st.vw[0], magic); c1 = word4_in_order(st.vw[BITS == 4 ? 1 : 0], magic); }
            else word2_in_order(st.vw[0], magic, c0, c1);
            uint4 *vd = reinterpret_cast<uint4 *>(&s_v[buf][vc * PF_VSTRIDE + 16 * vh]);
            vd[0] = c0; vd[1] = c1;
            if (tid < 32) *reinterpret_cast<uint4 *>(&s_km[buf][tid >> 4][8 * (tid & 15)]) = st.meta;
            else if (tid < 32 + 12 * GV) {
                const int pc = tid - 32;
                *reinterpret_cast<uint4 *>(&s_vm[buf][pc / (4 * GV)][(pc / 4) % GV][8 * (pc % 4)]) = st.meta;
            } else if (tid == 255) {
                const u32 no = Magic<BITS>::neg_off_pair;
                *reinterpret_cast<uint4 *>(&s_km[buf][2][0]) = make_uint4(no, no, no, no);
            }
        } else {
            // tail unit (few per block, fetched here): plain key row chunk; value row chunk transposed
            int64_t tok = (int64_t)(w - n_punits) * 32 + kt;
            if (tok >= a.n_tail) tok = 0;   // masked in the softmax
            const int64_t e0 = tbase + tok * MF_D + 16 * kc;
            f16x8 *kd = reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * PF_KSTRIDE + 16 * kc]);
            kd[0] = ld_tail8(a.k_tail, e0, tail_bf16);
            kd[1] = ld_tail8(a.k_tail, e0 + 8, tail_bf16);
            const f16x8 v0 = ld_tail8(a.v_tail, e0, tail_bf16), v1 = ld_tail8(a.v_tail, e0 + 8, tail_bf16);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                s_v[buf][(16 * kc + e) * PF_VSTRIDE + kt] = v0[e];
                s_v[buf][(16 * kc + 8 + e) * PF_VSTRIDE + kt] = v1[e];
            }
            const uint4 one8 = make_uint4(0x3C003C00u, 0x3C003C00u, 0x3C003C00u, 0x3C003C00u), zero8 = make_uint4(0, 0, 0, 0);
            if (tid < 32) *reinterpret_cast<uint4 *>(&s_km[buf][tid >> 4][8 * (tid & 15)]) = tid < 16 ? one8 : zero8;
            else if (tid < 32 + 12 * GV) {
                const int pc = tid - 32, which = pc / (4 * GV);
                *reinterpret_cast<uint4 *>(&s_vm[buf][which][(pc / 4) % GV][8 * (pc % 4)]) = which == 0 ? one8 : zero8;
            } else if (tid == 255) {
                *reinterpret_cast<uint4 *>(&s_km[buf][2][0]) = zero8;
            }
        }
    };
    // scale / zero of the lane's eight tokens of the unit staged in buffer buf
    using Meta = PfMeta<GV>;
    auto fetch_meta = [&](int buf, Meta &m) {
#pragma unroll
        for (int g = 0; g < GV; ++g) m.s[g] = *reinterpret_cast<const uint4 *>(&s_vm[buf][0][g][8 * blk]);
        m.z = *reinterpret_cast<const uint4 *>(&s_vm[buf][n < GV ? 1 : 2][n % GV][8 * blk]);
    };

    // ---- consumer state
    // O[nt]: channels 16 nt + n, still carrying off * sum_t P s_g; Z column g < GV = sum_t P[row, t] z_g[t],
    // column GV + g = sum_t P[row, t] s_g[t]; L = sum_t P[row, t]
    f32x4 O[8], Z = {0.f, 0.f, 0.f, 0.f}, L = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int nt = 0; nt < 8; ++nt) O[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    float m_run = -INFINITY;
    f16x8 qh[4], ql[4];
    f32x4 bias = {0.f, 0.f, 0.f, 0.f};
    const f16x8 ones = ones8();

    // fold the key scales of a token group into the query rows; seed the scores with
    // sum_d z_d q_d - off * sum_d (q s)_d
    auto open_group = [&](int buf) {
        // three short MFMA chains (zeros, high part, remainder) instead of one long one
        f32x4 bz = {0.f, 0.f, 0.f, 0.f}, bh_ = {0.f, 0.f, 0.f, 0.f}, bl = {0.f, 0.f, 0.f, 0.f};
        const f16x8 negoff = as_h8(*reinterpret_cast<const uint4 *>(&s_km[buf][2][0]));   // all lanes alike
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const f16x8 s = as_h8(*reinterpret_cast<const uint4 *>(&s_km[buf][0][32 * ks + 8 * blk]));
            const f16x8 z = as_h8(*reinterpret_cast<const uint4 *>(&s_km[buf][1][32 * ks + 8 * blk]));
            const f16x8 q8 = qn[ks];
            bz = VQ_MFMA(z, q8, bz);
            const f16x8 hi = q8 * s;
            // q*s has at most 22 significant bits: its remainder after the fp16 high part is
            // itself an fp16 number, so this fma is exact
            qh[ks] = hi;
            ql[ks] = __builtin_elementwise_fma(q8, s, -hi);
            bh_ = VQ_MFMA(negoff, qh[ks], bh_);
            bl = VQ_MFMA(negoff, ql[ks], bl);
        }
        bias = (bz + bh_) + bl;
    };

    // Softmax of one unit against the lazily updated reference.  Tokens at or past `lim` are
    // masked when the unit reaches past `full`.  Returns false, having done nothing but note the
    // new maxima in m_seen, when some row's scores outgrow the reference: the caller rescales
    // and repeats the unit.  Otherwise P is the A operand of the second product (pair r =
    // tokens 8 blk + 2 r, 8 blk + 2 r + 1).
    float m_seen = -INFINITY;
    auto softmax = [&](f32x4 (&S)[2], int base, int lim, int full, int lo, int lo_edge, u32 (&P)[4]) -> bool {
        if (base + 32 > full || base < lo_edge) {
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (base + pf_tok(blk, r, T) >= lim || base + pf_tok(blk, r, T) < lo) S[T][r] = -INFINITY;
        }
        const float mx = fmaxf(fmaxf(fmaxf(S[0][0], S[0][1]), fmaxf(S[0][2], S[0][3])),
                               fmaxf(fmaxf(S[1][0], S[1][1]), fmaxf(S[1][2], S[1][3])));
        if (__any(mx * c > m_run + RESCALE_SLACK)) {
            m_seen = mx * c;
            return false;
        }
        const float nm = m_run == -INFINITY ? 0.f : -m_run;
#pragma unroll
        for (int r = 0; r < 4; ++r)
            P[r] = as_u(f16x2{(f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[0][r], c, nm)),
                              (f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[1][r], c, nm))});
        return true;
    };
    // move the reference of every row up to what it has seen and rescale the accumulators
    auto rescale = [&]() {
        float ms = m_seen;
        ms = fmaxf(ms, __shfl_xor(ms, 16));
        ms = fmaxf(ms, __shfl_xor(ms, 32));
        const float m_new = fmaxf(m_run, ms);
        const float alpha = m_new == -INFINITY ? 1.f : exp2f(m_run - m_new);
        float al[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) al[r] = __shfl(alpha, 4 * blk + r);
#pragma unroll
        for (int r = 0; r < 4; ++r) {
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) O[nt][r] *= al[r];
            Z[r] *= al[r];
            L[r] *= al[r];
        }
        m_run = m_new;
    };

    auto compute = [&](int buf, int base, int lim, int full, int lo, int lo_edge, const Meta &vm) -> bool {
        // two accumulator chains per score tile (high and remainder part of the folded query)
        f32x4 S[2], Sl[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const f16 *kr = &s_k[buf][pf_krow(pf_tok(n >> 2, n & 3, T)) * PF_KSTRIDE + 8 * blk];
            Sl[T] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) {
                const f16x8 A = *reinterpret_cast<const f16x8 *>(kr + 32 * ks);
                S[T] = VQ_MFMA(A, qh[ks], ks == 0 ? bias : S[T]);
                Sl[T] = VQ_MFMA(A, ql[ks], Sl[T]);
            }
            S[T] += Sl[T];
        }
        u32 P[4];
        if (!softmax(S, base, lim, full, lo, lo_edge, P)) return false;
        const f16x8 P8 = as_h8(P[0], P[1], P[2], P[3]);
        // per channel group: A = P * s_g as fp16 high part plus exact fp16 remainder
#pragma unroll
        for (int g = 0; g < GV; ++g) {
            u32 ah[4], al[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const f16x2 sp2 = as_h2(u4_at(vm.s[g], p));
                const f16x2 hi = as_h2(P[p]) * sp2;
                ah[p] = as_u(hi);
                al[p] = as_u(__builtin_elementwise_fma(as_h2(P[p]), sp2, -hi));
            }
            const f16x8 Ah = as_h8(ah[0], ah[1], ah[2], ah[3]), Al = as_h8(al[0], al[1], al[2], al[3]);
#pragma unroll
            for (int jt = 0; jt < TPG; ++jt) {
                const int nt = g * TPG + jt;
                const f16x8 Bv = *reinterpret_cast<const f16x8 *>(&s_v[buf][(16 * nt + n) * PF_VSTRIDE + 8 * blk]);
                O[nt] = VQ_MFMA(Ah, Bv, O[nt]);
                O[nt] = VQ_MFMA(Al, Bv, O[nt]);
            }
        }
        Z = VQ_MFMA(P8, as_h8(vm.z), Z);
        L = VQ_MFMA(P8, ones, L);
        return true;
    };
    // ---- pipeline over the work units [w0, w1): registers hold the packed words of unit w+1
    // while unit w is computed from LDS
    // Iteration w: unpack unit w+1 (fetched during iteration w-1) into the other buffer, start
    // the fetch of unit w+2, then compute unit w; the barrier at the end makes unit w+1 visible
    // and frees the buffer of unit w.  A unit whose scores outgrow the softmax reference is
    // repeated after a rescale (a handful of times per wave) without touching the pipeline.
    Stage st;
    if (w1 > w0) {
        fetch(w0, st);
        unpack_to_lds(w0, st, 0);
        __syncthreads();
        if (w0 + 1 < w1) fetch(w0 + 1, st);
    }
    int cur_group = -1;
    bool staged = false;   // unit w+1 already unpacked (set while a unit is being repeated)
    for (int w = w0; w < w1;) {
        const int buf = (w - w0) & 1;
        if (!staged) {
            if (w + 1 < w1) unpack_to_lds(w + 1, st, buf ^ 1);
            if (w + 2 < w1) fetch(w + 2, st);
            staged = true;
        }
        // a tail unit runs through the same code: its staged scale / zero / offset make the
        // products plain ones
        const bool packed = w < n_punits;
        const int base = packed ? w * 32 : (w - n_punits) * 32;
        const int grp = packed ? (base >> gshift) : -2;
        Meta vm;
        fetch_meta(buf, vm);
        if (grp != cur_group) {
            cur_group = grp;
            open_group(buf);
        }
        if (!compute(buf, base, packed ? lane_vis : lane_tvis, packed ? full_vis : full_tvis, packed ? lane_lo : lane_tlo,
                     packed ? edge_lo : edge_tlo, vm)) {
            rescale();
            continue;
        }
        __syncthreads();
        staged = false;
        ++w;
    }

    // ---- every wave owns its 16 rows: accumulator register r of lane (n, blk) is row 4 blk + r,
    // tile nt column n is channel 16 nt + n; the row's reference maximum sits in lane 4 blk + r
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int jr = 16 * wave + 4 * blk + r;
        const int64_t pr = pos0 + jr % qp;
        const float mr = __shfl(m_run, 4 * blk + r);
        float zs[GV], ss[GV];   // zero-point and scale sums of this row: columns g and GV + g of the Z tile
#pragma unroll
        for (int g = 0; g < GV; ++g) {
            zs[g] = __shfl(Z[r], 16 * blk + g);
            ss[g] = __shfl(Z[r], 16 * blk + GV + g);
        }
        if (pr < a.Sq) {
            const int64_t row = (b * a.Hq + hkv * R + jr / qp) * a.Sq + pr;
            float *o = ws + (row * nparts + sp) * MF_PART;
#pragma unroll
            for (int nt = 0; nt < 8; ++nt) o[2 + 16 * nt + n] = (O[nt][r] - Magic<BITS>::off * ss[nt / TPG]) + zs[nt / TPG];
            if (n == 0) { o[0] = mr * LN2; o[1] = L[r]; }
        }
    }
}

// ---- 256-row blocks: keys and values reconstructed in the producer --------------------------
//
// With many query rows per kv head (a prefill chunk) the cost that matters is MFMA issue, and
// the raw-code formulation above spends 46 MFMAs per 16 rows and 32 tokens where 16 are useful.
// Here the producer turns the codes into the reconstruction itself, k^ = c s + z and
// v^ = c s + z as packed fp16 fused multiply-adds on exact fp16 codes (c s + z is formed
// exactly and rounded once to fp16, which is what the reference's cache holds: it stores the
// reconstruction cast to the input dtype, veloxquant_mlx/cache/kivi_cache.py:181-201), and the
// consumer is plain attention: 8 + 8 MFMAs per 16 rows and unit plus one for the row sums.  A
// wave owns two 16-row blocks so that every LDS read of a key or value tile feeds two MFMAs and
// everything still fits the 256 registers of two waves per SIMD (with four row blocks the
// accumulators spill into the accumulation registers and the compiler moves them back and
// forth around every product); a block is eight waves = 256 rows = the GQA group at 256 / R
// consecutive positions, one block per CU, so a unit is unpacked once for 256 rows.  Tiles,
// token order, lazily rescaled softmax and partials are those of the kernel above.
constexpr int PR_RB = 2;          // 16-row blocks per wave
constexpr int PR_THREADS = 512;

// eight scale or zero values of the storage type M as raw 16-byte pieces
template <typename M> struct Meta8 {
    static constexpr int N = (int)sizeof(M) / 2;   // pieces: 1 for fp16, 2 for float32
    uint4 u[N];
    __device__ __forceinline__ void load(const void *p) {
#pragma unroll
        for (int i = 0; i < N; ++i) u[i] = reinterpret_cast<const uint4 *>(p)[i];
    }
};
// c * s + z for eight exact fp16 codes: formed exactly and rounded once with fp16 scale / zero; in
// float32 with one rounding per operation and then rounded to fp16 with float32 scale / zero --
// in both cases what a cache that stores the reconstruction in fp16 holds
// (veloxquant_mlx/cache/kivi_cache.py:198-201)
__device__ __forceinline__ f16x8 recon8(f16x8 c, const Meta8<f16> &s, const Meta8<f16> &z) {
    return __builtin_elementwise_fma(c, as_h8(s.u[0]), as_h8(z.u[0]));
}
__device__ __forceinline__ f16x8 recon8(f16x8 c, const Meta8<float> &s, const Meta8<float> &z) {
    const float sf[8] = {__uint_as_float(s.u[0].x), __uint_as_float(s.u[0].y), __uint_as_float(s.u[0].z), __uint_as_float(s.u[0].w),
                         __uint_as_float(s.u[1].x), __uint_as_float(s.u[1].y), __uint_as_float(s.u[1].z), __uint_as_float(s.u[1].w)};
    const float zf[8] = {__uint_as_float(z.u[0].x), __uint_as_float(z.u[0].y), __uint_as_float(z.u[0].z), __uint_as_float(z.u[0].w),
                         __uint_as_float(z.u[1].x), __uint_as_float(z.u[1].y), __uint_as_float(z.u[1].z), __uint_as_float(z.u[1].w)};
    f16x8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (f16)__fadd_rn(__fmul_rn((float)c[e], sf[e]), zf[e]);
    return o;
}

// one run per row, nothing to patch afterwards, 256-row blocks: the kernel writes `out`, no merge launch follows
__host__ __device__ inline bool mfma_prefill_writes_output(const vq_attend_args &a, int nparts) {
    return nparts == 1 && a.sink_k == nullptr && (a.Hq / a.Hkv) * a.Sq >= (a.D == 2 * MF_D ? 128 : 256);
}

template <int BITS, typename M> struct PrStage {
    u32 kw;          // key word: the thread's 8 channels of one token (2-bit: the word holding them)
    u32 vw;          // value word: the thread's 8 tokens of one channel (2-bit: the word holding them)
    Meta8<M> vs, vz; // value scale / zero of those 8 tokens (the thread's channel group); a tail unit's
                     // raw key and value pieces travel in the first piece of each
};

// TILES: every unit comes ready-made from a.kv_tiles (the packed prefix and the tail alike) and is copied from
// global memory straight into a ring of four LDS buffers, four units ahead; the block then has no producer work
// on the vector unit and holds no staging registers.  BITS, GV and M play no part then.
template <int BITS, int GV, typename M, bool TILES = false>
__global__ __launch_bounds__(PR_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attend_prefill_rows_kernel(vq_attend_args a, int qp, int nparts, float *__restrict__ ws) {
    __shared__ __align__(16) f16 s_k[TILES ? 1 : 3][32 * PF_KSTRIDE];
    __shared__ __align__(16) f16 s_v[TILES ? 1 : 3][MF_D * PF_VSTRIDE];
    __shared__ __align__(16) char s_ring[TILES ? 4 * PF_TILE_BYTES : 16];
    auto key_tile = [&](int buf) -> const f16 * {
        if constexpr (TILES) return reinterpret_cast<const f16 *>(s_ring + buf * PF_TILE_BYTES);
        else return s_k[buf];
    };
    auto value_tile = [&](int buf) -> const f16 * {
        if constexpr (TILES) return reinterpret_cast<const f16 *>(s_ring + buf * PF_TILE_BYTES + PF_TILE_KEYS);
        else return s_v[buf];
    };

    constexpr int PER = 32 / BITS;
    constexpr int KW = MF_D / PER;
    constexpr int gshift = GV == 4 ? 5 : GV == 2 ? 6 : 7;   // log2 of the group size
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, blk = lane >> 4;
    // Which (row tile, (sequence, kv head), run) this block is.  Workgroups go to the eight XCDs in turn by
    // their linear number, and every XCD has its own L2: with the launch's own numbering the row tiles and runs
    // of one kv head land on all eight, and each fetches that head's keys and values from HBM for itself (68 MB
    // per launch at config 4 for 15 MB of input).  The blocks are renumbered so that a head's tiles and runs share
    // an XCD (a multiple of eight heads) or 8 / heads of them (1, 2 or 4 heads); other counts keep the launch's
    // numbering.
    unsigned tile_x = blockIdx.x, bh_y = blockIdx.y, run_z = blockIdx.z;
    if (gridDim.y % 8 == 0 || 8 % gridDim.y == 0) {
        const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned per_head = gridDim.x * gridDim.z, xcd = lin % 8, slot = lin / 8;
        unsigned within;
        if (gridDim.y % 8 == 0) {
            bh_y = xcd + 8 * (slot / per_head);
            within = slot % per_head;
        } else {
            bh_y = xcd % gridDim.y;
            within = xcd / gridDim.y + (8 / gridDim.y) * slot;
        }
        tile_x = within % gridDim.x;
        run_z = within / gridDim.x;
    }
    const int64_t bh = bh_y;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    if constexpr (TILES) {   // one kind of unit: all slots count as tail slots
        a.n_tail += a.n_packed;
        a.n_packed = 0;
    }
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t cap = a.cap_tokens;
    const float c = a.scale * LOG2E;
    const u32 magic = vreg_const(Magic<BITS>::bits);
    // under a causal mask the last tiles see the most tokens: they are started first
    const int pos0 = (int)(a.causal ? gridDim.x - 1 - tile_x : tile_x) * qp;
    const int64_t n_total = a.n_packed + a.n_tail;
    auto visible = [&](int64_t p) { return a.causal ? n_total - a.Sq + p + 1 : n_total; };   // slots row p sees

    // ---- this lane's query rows (score columns): row j = 32 wave + 16 rb + n of the block
    // the block covers qp = 256 / R positions (rounded down: a group of 3 heads 85, and the last row of the block idles)
    int lane_vis[PR_RB], lane_tvis[PR_RB];
    int lane_lo[PR_RB], lane_tlo[PR_RB];   // sliding window: first packed / tail token the row sees
    f16x8 qn[PR_RB][4];   // B operands: lane (n, blk) holds channels 32 ks + 8 blk + 0..7 of its row
#pragma unroll
    for (int rb = 0; rb < PR_RB; ++rb) {
        const int j = 16 * PR_RB * wave + 16 * rb + n;
        const int jh = (int)((unsigned)j / (unsigned)qp);   // head of the group, position in the block
        const int64_t pos = pos0 + (j - jh * qp);
        const bool row_ok = pos < a.Sq && jh < R;
        const int64_t qrow = (b * a.Hq + hkv * R + (jh < R ? jh : R - 1)) * a.Sq + (pos < a.Sq ? pos : a.Sq - 1);
        const int64_t vis = visible(row_ok ? pos : a.Sq - 1);
        lane_vis[rb] = (int)(vis < a.n_packed ? vis : a.n_packed);
        const int64_t tv = vis - a.n_packed;
        lane_tvis[rb] = (int)(tv < 0 ? 0 : tv < a.n_tail ? tv : a.n_tail);
        const int64_t first = window_first(a, n_total, row_ok ? pos : a.Sq - 1);
        lane_lo[rb] = (int)(first < a.n_packed ? first : a.n_packed);
        lane_tlo[rb] = (int)(first > a.n_packed ? first - a.n_packed : 0);
#pragma unroll
        for (int ks = 0; ks < 4; ++ks) {
            const int64_t e0 = qrow * MF_D + 32 * ks + 8 * blk;
            if (a.q_dtype == VQ_F32) {
#pragma unroll
                for (int e = 0; e < 8; ++e) qn[rb][ks][e] = (f16)((const float *)a.q)[e0 + e];
            } else {
                qn[rb][ks] = ld_tail8(a.q, e0, a.q_dtype == VQ_BF16);
            }
        }
    }
    const int64_t last_pos = pos0 + qp - 1 < a.Sq - 1 ? pos0 + qp - 1 : a.Sq - 1;
    const int64_t vis_min = visible(pos0), vis_max = visible(last_pos);
    const int full_vis = (int)(vis_min < a.n_packed ? vis_min : a.n_packed);
    const int max_vis = (int)(vis_max < a.n_packed ? vis_max : a.n_packed);
    const int64_t tv_min = vis_min - a.n_packed, tv_max = vis_max - a.n_packed;
    const int full_tvis = (int)(tv_min < 0 ? 0 : tv_min < a.n_tail ? tv_min : a.n_tail);
    const int max_tvis = (int)(tv_max < 0 ? 0 : tv_max < a.n_tail ? tv_max : a.n_tail);
    const int n_punits = (max_vis + 31) / 32;
    const int n_tunits = (max_tvis + 31) / 32;
    const int n_work = n_punits + n_tunits;
    const int nsplit = (int)gridDim.z, sp = (int)run_z;
    // units below the window of the block's first row are seen by none of its rows
    const int64_t first_blk = window_first(a, n_total, pos0);
    const int w_lo = first_blk < a.n_packed ? (int)(first_blk / 32) : n_punits + (int)((first_blk - a.n_packed) / 32);
    const int w_n = n_work > w_lo ? n_work - w_lo : 0;
    const int w0 = w_lo + (int)((int64_t)w_n * sp / nsplit), w1 = w_lo + (int)((int64_t)w_n * (sp + 1) / nsplit);
    const int64_t first_all = window_first(a, n_total, last_pos);   // below it some row of the block sees nothing
    const int edge_lo = (int)(first_all < a.n_packed ? first_all : a.n_packed);
    const int edge_tlo = (int)(first_all > a.n_packed ? first_all - a.n_packed : 0);

    // ---- producer side
    const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
    const char *vb = (const char *)a.v_packed + bh * (cap / PER) * MF_D * 4;
    const M *ksb = (const M *)a.k_scale + bh * (cap >> gshift) * MF_D;
    const M *kzb = (const M *)a.k_zero + bh * (cap >> gshift) * MF_D;
    const M *vsb = (const M *)a.v_scale + bh * GV * cap;
    const M *vzb = (const M *)a.v_zero + bh * GV * cap;
    const int kt = tid >> 4, kc = tid & 15;       // key tile: token, 8-channel chunk
    const int vc = tid & 127, vq = tid >> 7;      // value tile: channel, 8-token quarter
    const int vg = vc >> gshift;                  // channel group of the thread's value channel
    // byte offsets of the thread's key word, value word and value scale / zero piece inside a unit
    const unsigned k_off = (unsigned)((kt * KW + (BITS == 4 ? kc : kc >> 1)) * 4);
    const unsigned v_off = (unsigned)(((BITS == 4 ? vq : vq >> 1) * MF_D + vc) * 4);
    const unsigned m_off = (unsigned)(((int64_t)vg * cap + 8 * vq) * sizeof(M));
    const int tp = lane & 15, cq = 4 * wave + (lane >> 4);   // tail values: token pair, channel quad
    const bool tail_bf16 = a.tail_dtype == VQ_BF16;
    const int64_t tbase = bh * a.tail_cap * MF_D;
    const f16x8 off8 = as_h8(Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair);
    using Stage = PrStage<BITS, M>;
    Meta8<M> ksr, kzr;   // key scale / zero of the thread's 8 channels in the token group last fetched
    int meta_group = -1;
    auto fetch = [&](int w, Stage &st) {
        if (w >= n_punits) {   // tail unit: the thread's key and value pieces travel in the value-meta slots
            // a block-uniform base (the unit's first token) plus a 32-bit offset of the thread's own; a token
            // past the end of the tail reads the last one instead (masked in the softmax)
            const int64_t t0 = (int64_t)(w - n_punits) * 32;
            const int last = (int)(a.n_tail - 1 - t0);   // >= 0: the unit starts inside the tail
            const char *kt0 = (const char *)a.k_tail + (tbase + t0 * MF_D) * 2, *vt0 = (const char *)a.v_tail + (tbase + t0 * MF_D) * 2;
            st.vs.u[0] = *reinterpret_cast<const uint4 *>(kt0 + (unsigned)((kt < last ? kt : last) * (MF_D * 2) + 16 * kc));
            // values: four channels of a token pair, so that the transposed tile is written in whole words
            const int ta = 2 * tp < last ? 2 * tp : last, tb = 2 * tp + 1 < last ? 2 * tp + 1 : last;
            const uint2 va = *reinterpret_cast<const uint2 *>(vt0 + (unsigned)(ta * (MF_D * 2) + 8 * cq));
            const uint2 vb2 = *reinterpret_cast<const uint2 *>(vt0 + (unsigned)(tb * (MF_D * 2) + 8 * cq));
            st.vz.u[0] = make_uint4(va.x, va.y, vb2.x, vb2.y);
            return;
        }
        // a block-uniform base that moves with the unit plus a 32-bit offset of the thread's own: the
        // per-unit address arithmetic stays on the scalar unit
        const int64_t base = (int64_t)w * 32;
        st.kw = *reinterpret_cast<const u32 *>(kb + base * (KW * 4) + k_off);
        st.vw = *reinterpret_cast<const u32 *>(vb + (base / PER) * (MF_D * 4) + v_off);
        st.vs.load((const char *)vsb + base * sizeof(M) + m_off);
        st.vz.load((const char *)vzb + base * sizeof(M) + m_off);
        const int grp = (int)(base >> gshift);
        if (grp != meta_group) {   // block-uniform
            meta_group = grp;
            ksr.load((const char *)ksb + (int64_t)grp * (MF_D * sizeof(M)) + 8u * (unsigned)sizeof(M) * (unsigned)kc);
            kzr.load((const char *)kzb + (int64_t)grp * (MF_D * sizeof(M)) + 8u * (unsigned)sizeof(M) * (unsigned)kc);
        }
    };
    // the thread's eight codes of a word, in order, as exact fp16 numbers
    auto codes8 = [&](u32 w, int half) -> f16x8 {
        uint4 lo;
        if (BITS == 4) lo = word4_in_order(w, magic);
        else {
            uint4 hi;
            word2_in_order(w, magic, lo, hi);
            if (half) lo = hi;
        }
        return as_h8(lo) + off8;
    };
    auto unpack_to_lds = [&](int w, const Stage &st, int buf) {
        if (w < n_punits) {
            // keys: 8 channels of token kt; c s + z is formed exactly and rounded once
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * PF_KSTRIDE + 8 * kc]) = recon8(codes8(st.kw, kc & 1), ksr, kzr);
            // values: 8 tokens of channel vc
            *reinterpret_cast<f16x8 *>(&s_v[buf][vc * PF_VSTRIDE + 8 * vq]) = recon8(codes8(st.vw, vq & 1), st.vs, st.vz);
        } else {
            // tail unit: plain key row chunk; values transposed, one word (a token pair of one channel)
            // at a time: the lanes of a wave cover 16 token pairs x 4 channel quads = 64 different banks
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * PF_KSTRIDE + 8 * kc]) = tail8_from_raw(st.vs.u[0], tail_bf16);
            const f16x8 v0 = tail8_from_raw(st.vz.u[0], tail_bf16);   // channels 0..3 of the first token, then of the second
#pragma unroll
            for (int e = 0; e < 4; ++e)
                *reinterpret_cast<f16x2 *>(&s_v[buf][(4 * cq + e) * PF_VSTRIDE + 2 * tp]) = f16x2{v0[e], v0[4 + e]};
        }
    };

    // ---- consumer state: O[rb][nt] rows 16 rb + 4 blk + r of the wave, channels 16 nt + n; L the row sums
    f32x4 O[PR_RB][8], L[PR_RB];
    float m_run[PR_RB], m_seen[PR_RB];
#pragma unroll
    for (int rb = 0; rb < PR_RB; ++rb) {
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) O[rb][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
        L[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[rb] = -INFINITY;
        m_seen[rb] = -INFINITY;
    }
    const f16x8 ones = ones8();

    // move the reference of every row up to what it has seen and rescale the accumulators
    auto rescale = [&]() {
#pragma unroll
        for (int rb = 0; rb < PR_RB; ++rb) {
            float ms = m_seen[rb];
            ms = fmaxf(ms, __shfl_xor(ms, 16));
            ms = fmaxf(ms, __shfl_xor(ms, 32));
            const float m_new = fmaxf(m_run[rb], ms);
            const float alpha = m_new == -INFINITY ? 1.f : exp2f(m_run[rb] - m_new);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float al = __shfl(alpha, 4 * blk + r);
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) O[rb][nt][r] *= al;
                L[rb][r] *= al;
            }
            m_run[rb] = m_new;
        }
    };

    // The operands of a unit live in registers from one iteration to the next: the key tile's
    // rows (A) and the value tile's rows (Bv) of unit w+1 are read from LDS while unit w is
    // still being computed, so that the LDS traffic of the eight waves runs beside the products
    // and the softmax instead of in front of them.
    f16x8 A[2][4], Bv[8];
    auto load_keys = [&](int buf) {
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const f16 *kr = &key_tile(buf)[pf_krow(pf_tok(n >> 2, n & 3, T)) * PF_KSTRIDE + 8 * blk];
#pragma unroll
            for (int ks = 0; ks < 4; ++ks) A[T][ks] = *reinterpret_cast<const f16x8 *>(kr + 32 * ks);
        }
    };
    auto load_values = [&](int buf) {
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
            Bv[nt] = *reinterpret_cast<const f16x8 *>(&value_tile(buf)[(16 * nt + n) * PF_VSTRIDE + 8 * blk]);
    };

    // One unit: scores of the wave's row blocks (four independent accumulator chains side by
    // side), softmax against the lazily updated references (raised in place, with the
    // accumulators rescaled, when some row's scores outgrow its reference), second product.
    // `next` is the buffer of the following unit (stale but harmless after the last one).
    auto compute = [&](int next, int base, bool packed, int full, int lo_edge) {
        f32x4 S[PR_RB][2];
#pragma unroll
        for (int ks = 0; ks < 4; ++ks)
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int rb = 0; rb < PR_RB; ++rb)
                    S[rb][T] = VQ_MFMA(A[T][ks], qn[rb][ks], ks == 0 ? (f32x4{0.f, 0.f, 0.f, 0.f}) : S[rb][T]);
        load_keys(next);
        bool grow = false;
#pragma unroll
        for (int rb = 0; rb < PR_RB; ++rb) {
            if (base + 32 > full || base < lo_edge) {
                const int lim = packed ? lane_vis[rb] : lane_tvis[rb], lo = packed ? lane_lo[rb] : lane_tlo[rb];
#pragma unroll
                for (int T = 0; T < 2; ++T)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (base + pf_tok(blk, r, T) >= lim || base + pf_tok(blk, r, T) < lo) S[rb][T][r] = -INFINITY;
            }
            const float mx = vmax3(vmax3(S[rb][0][0], S[rb][0][1], S[rb][0][2]), vmax3(S[rb][0][3], S[rb][1][0], S[rb][1][1]),
                                   vmax3(S[rb][1][2], S[rb][1][3], S[rb][1][3]));
            m_seen[rb] = mx * c;
            grow |= mx * c > m_run[rb] + RESCALE_SLACK;
        }
        if (__any(grow)) rescale();
        f16x8 P8[PR_RB];
#pragma unroll
        for (int rb = 0; rb < PR_RB; ++rb) {
            const float nm = m_run[rb] == -INFINITY ? 0.f : -m_run[rb];
            u32 P[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                P[r] = as_u(f16x2{(f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[rb][0][r], c, nm)),
                                  (f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[rb][1][r], c, nm))});
            P8[rb] = as_h8(P[0], P[1], P[2], P[3]);
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
#pragma unroll
            for (int rb = 0; rb < PR_RB; ++rb) O[rb][nt] = VQ_MFMA(P8[rb], Bv[nt], O[rb][nt]);
#pragma unroll
        for (int rb = 0; rb < PR_RB; ++rb) L[rb] = VQ_MFMA(P8[rb], ones, L[rb]);
        load_values(next);
    };

    // ---- pipeline over the work units [w0, w1) on three LDS buffers: while unit w is computed
    // from registers, unit w+1 is read from its buffer, unit w+2 is unpacked into the third and
    // unit w+3 is requested from memory.  The producer's share comes after the unit's second product
    // (its first instructions issue while those products run); unpacking before the products in half
    // of the waves, to put the two waves of a SIMD out of step, measured 8 % slower.
    // The barrier between units waits for LDS only: __syncthreads() also waits for every outstanding
    // global load, i.e. for the unit just requested, once per unit.  For the same reason nothing
    // requested before the loop may still be pending inside it (the compiler would wait for it at
    // the loop head, and with it for whatever was requested since).
    if constexpr (TILES) {
        // A unit is 19 pieces of 1 KB; wave v copies pieces v, v + 8 and v + 16 (waves 3..7 copy piece v + 8 a second
        // time instead: every wave has three copies per unit in flight, which is what the waits count).  Four
        // buffers.  Iteration w computes unit w from registers while it reads unit w+1 from LDS into them, then waits
        // for its copies of unit w+2 (those of unit w+3 stay in flight) and meets the other waves; after that barrier
        // every wave has used unit w, so unit w+4 is requested into its buffer.  The barrier does not wait for the
        // wave's own LDS reads (nothing was written through LDS instructions): they stay in flight across it, and
        // the products that use them wait for them.  Past the end of the run the last unit is copied again.
        // (Forming the next unit's scores between this unit's exponentials, which the spare registers of this form
        // allow, was built and measured: no faster -- a product leaves the vector unit little room here.)
        const char *tiles = (const char *)a.kv_tiles + bh * a.tile_cap * PF_TILE_BYTES;
        const u32 ring = lds_addr(s_ring), lane16 = (u32)lane * 16u;
        const int third_piece = wave < 3 ? wave + 16 : wave + 8;
        auto request = [&](int w, int buf) __attribute__((always_inline)) {
            const char *src = tiles + (int64_t)(w < w1 ? w : w1 - 1) * PF_TILE_BYTES;
            const u32 dst = ring + (u32)buf * PF_TILE_BYTES;
            lds_copy16<0>(src + 1024 * wave, lane16, dst + 1024 * wave);
            lds_copy16<0>(src + 1024 * (wave + 8), lane16, dst + 1024 * (wave + 8));
            lds_copy16<0>(src + 1024 * third_piece, lane16, dst + 1024 * third_piece);
        };
        if (w1 > w0) {
            wait_global_accesses();
#pragma unroll
            for (int i = 0; i < 4; ++i) request(w0 + i, i);
            wait_copies<9>();
            lds_barrier();
            load_keys(0);
            load_values(0);
            wait_copies<6>();
            lds_barrier();
            int cur = 0;
            for (int w = w0; w < w1; ++w) {
                const int next = (cur + 1) & 3;
                compute(next, w * 32, false, full_tvis, edge_tlo);
                wait_copies<3>();
                asm volatile("s_barrier" ::: "memory");
                request(w + 4, cur);
                cur = next;
            }
            wait_copies<0>();   // nothing may land in LDS after the block has given it back
        }
    } else {
        Stage st;
        if (w1 > w0) {
            fetch(w0, st);
            unpack_to_lds(w0, st, 0);
            if (w0 + 1 < w1) {
                fetch(w0 + 1, st);
                unpack_to_lds(w0 + 1, st, 1);
            }
            if (w0 + 2 < w1) fetch(w0 + 2, st);
            __syncthreads();
            load_keys(0);
            load_values(0);
        }
        wait_global_accesses();
        int cur = 0;
        for (int w = w0; w < w1; ++w) {
            const int next = cur == 2 ? 0 : cur + 1, third = next == 2 ? 0 : next + 1;
            const bool packed = w < n_punits;
            const int base = packed ? w * 32 : (w - n_punits) * 32;
            compute(next, base, packed, packed ? full_vis : full_tvis, packed ? edge_lo : edge_tlo);
            if (w + 2 < w1) unpack_to_lds(w + 2, st, third);
            if (w + 3 < w1) fetch(w + 3, st);
            lds_barrier();
            cur = next;
        }
    }

    // ---- every wave owns its rows: accumulator register r of lane (n, blk) is row 4 blk + r of the
    // row block, tile nt column n is channel 16 nt + n; the row's reference sits in lane 4 blk + r.
    // A launch with one run per row and no protected rows to patch in writes the output itself: the merge
    // of a single record is that record normalised (mfma_prefill_writes_output decides, for the host too).
    const bool direct = mfma_prefill_writes_output(a, nparts);
#pragma unroll
    for (int rb = 0; rb < PR_RB; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int jr = 16 * PR_RB * wave + 16 * rb + 4 * blk + r;
            const int jrh = (int)((unsigned)jr / (unsigned)qp);
            const int64_t pr = pos0 + (jr - jrh * qp);
            const float mr = __shfl(m_run[rb], 4 * blk + r);
            if (pr < a.Sq && jrh < R) {
                const int64_t row = (b * a.Hq + hkv * R + jrh) * a.Sq + pr;
                if (direct) {
                    // the only record of its row: what the merge would make of it (0 for a row that sees nothing)
                    const bool seen = mr != -INFINITY && L[rb][r] > 0.f;
#pragma unroll
                    for (int nt = 0; nt < 8; ++nt) {
                        const float v = seen ? __fdiv_rn(O[rb][nt][r], L[rb][r]) : 0.f;
                        const int64_t oi = row * MF_D + 16 * nt + n;
                        if (a.out_dtype == VQ_F16) ((f16 *)a.out)[oi] = (f16)v;
                        else if (a.out_dtype == VQ_BF16) ((u16 *)a.out)[oi] = f32_to_bf16(v);
                        else ((float *)a.out)[oi] = v;
                    }
                    continue;
                }
                float *o = ws + (row * nparts + sp) * MF_PART;
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) o[2 + 16 * nt + n] = O[rb][nt][r];
                if (n == 0) { o[0] = mr * LN2; o[1] = L[rb][r]; }
            }
        }
}

// ---- units as ready-made tiles in global memory: grid (units, B*Hkv), block 512.  Unit first_unit + x of every
// (sequence, kv head): packed units are reconstructed exactly as the 256-row blocks do it (c s + z rounded once
// to fp16), tail units are the plain rows; the thread-to-piece assignment is that of the blocks' producer.
template <int BITS, int GV, typename M>
__global__ __launch_bounds__(PR_THREADS) void prefill_tiles_kernel(vq_attend_args a, int first_unit) {
    constexpr int PER = 32 / BITS;
    constexpr int KW = MF_D / PER;
    constexpr int gshift = GV == 4 ? 5 : GV == 2 ? 6 : 7;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int64_t bh = blockIdx.y, cap = a.cap_tokens;
    const int w = first_unit + (int)blockIdx.x, n_punits = (int)(a.n_packed / 32);
    char *tile = (char *)a.kv_tiles + (bh * a.tile_cap + w) * PF_TILE_BYTES;
    f16 *kdst = reinterpret_cast<f16 *>(tile), *vdst = reinterpret_cast<f16 *>(tile + PF_TILE_KEYS);
    const int kt = tid >> 4, kc = tid & 15;       // key tile: token, 8-channel chunk
    const int vc = tid & 127, vq = tid >> 7;      // value tile: channel, 8-token quarter
    if (w < n_punits) {
        const u32 magic = vreg_const(Magic<BITS>::bits);
        const f16x8 off8 = as_h8(Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair);
        auto codes8 = [&](u32 word, int half) -> f16x8 {
            uint4 lo;
            if (BITS == 4) lo = word4_in_order(word, magic);
            else {
                uint4 hi;
                word2_in_order(word, magic, lo, hi);
                if (half) lo = hi;
            }
            return as_h8(lo) + off8;
        };
        const int64_t base = (int64_t)w * 32;
        const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
        const char *vb = (const char *)a.v_packed + bh * (cap / PER) * MF_D * 4;
        const M *ksb = (const M *)a.k_scale + bh * (cap >> gshift) * MF_D, *kzb = (const M *)a.k_zero + bh * (cap >> gshift) * MF_D;
        const M *vsb = (const M *)a.v_scale + bh * GV * cap, *vzb = (const M *)a.v_zero + bh * GV * cap;
        const u32 kw = *reinterpret_cast<const u32 *>(kb + (base + kt) * (KW * 4) + (BITS == 4 ? kc : kc >> 1) * 4);
        const u32 vw = *reinterpret_cast<const u32 *>(vb + ((base / PER) + (BITS == 4 ? vq : vq >> 1)) * (MF_D * 4) + vc * 4);
        Meta8<M> ks, kz, vs, vz;
        const int64_t grp = base >> gshift;
        ks.load(ksb + grp * MF_D + 8 * kc);
        kz.load(kzb + grp * MF_D + 8 * kc);
        vs.load(vsb + (int64_t)(vc >> gshift) * cap + base + 8 * vq);
        vz.load(vzb + (int64_t)(vc >> gshift) * cap + base + 8 * vq);
        *reinterpret_cast<f16x8 *>(&kdst[pf_krow(kt) * PF_KSTRIDE + 8 * kc]) = recon8(codes8(kw, kc & 1), ks, kz);
        *reinterpret_cast<f16x8 *>(&vdst[vc * PF_VSTRIDE + 8 * vq]) = recon8(codes8(vw, vq & 1), vs, vz);
    } else {
        // tail unit; a token past the end of the tail repeats the last one (masked in the softmax)
        const bool tail_bf16 = a.tail_dtype == VQ_BF16;
        const int64_t t0 = (int64_t)(w - n_punits) * 32, tbase = bh * a.tail_cap * MF_D;
        const int last = (int)(a.n_tail - 1 - t0);
        const int tk = kt < last ? kt : last;
        *reinterpret_cast<f16x8 *>(&kdst[pf_krow(kt) * PF_KSTRIDE + 8 * kc]) = ld_tail8(a.k_tail, tbase + (t0 + tk) * MF_D + 8 * kc, tail_bf16);
        const int tp = lane & 15, cq = 4 * wave + (lane >> 4);   // token pair, channel quad
        const int ta = 2 * tp < last ? 2 * tp : last, tb = 2 * tp + 1 < last ? 2 * tp + 1 : last;
        const char *vt0 = (const char *)a.v_tail + (tbase + t0 * MF_D) * 2;
        const uint2 va = *reinterpret_cast<const uint2 *>(vt0 + ta * (MF_D * 2) + 8 * cq);
        const uint2 vb2 = *reinterpret_cast<const uint2 *>(vt0 + tb * (MF_D * 2) + 8 * cq);
        const f16x8 v0 = tail8_from_raw(make_uint4(va.x, va.y, vb2.x, vb2.y), tail_bf16);
#pragma unroll
        for (int e = 0; e < 4; ++e)
            *reinterpret_cast<f16x2 *>(&vdst[(4 * cq + e) * PF_VSTRIDE + 2 * tp]) = f16x2{v0[e], v0[4 + e]};
    }
}

// ---------------------------------------------------------------------------
// Heads of 256 channels on the same blocks: the scores run over eight k-steps instead of four, so a wave holds one
// 16-row block (a block of eight waves = 128 rows = the GQA group at 128 / R positions) where the kernel above holds
// two -- queries 32 registers, key operands 64, accumulators 32, value operands 32, as there -- and a launch forms
// the output's channels [128 v_half, 128 v_half + 128): the call is two launches that compute the same scores and
// probabilities and each take one half of the value tile.  Tiles, token order, softmax and partial format are the
// kernel's above; a record has 258 floats and the launch of the first half writes its maximum and sum.
// ---------------------------------------------------------------------------
constexpr int P2_RB = 1;

template <typename M> struct PrStage2 {
    uint4 k2;        // packed unit: the two key words (8 channels of a token in either half of the channels) and the
                     // value word; tail unit: the raw key piece of the second half
    Meta8<M> vs, vz; // value scale / zero of the thread's 8 tokens; a tail unit's raw key (first half) and value pieces
                     // travel in the first piece of each
};

template <int BITS, int GV, typename M>
__global__ __launch_bounds__(PR_THREADS) __attribute__((amdgpu_waves_per_eu(2, 2)))
void attend_prefill_rows_d256_kernel(vq_attend_args a, int qp, int nparts, int v_half, float *__restrict__ ws) {
    constexpr int DH = 2 * MF_D;          // channels of a head
    constexpr int KST = DH + 8;           // fp16 per token row of the key tile (528 B: conflict-free b128 reads)
    __shared__ __align__(16) f16 s_k[3][32 * KST];
    __shared__ __align__(16) f16 s_v[3][MF_D * PF_VSTRIDE];

    constexpr int PER = 32 / BITS;
    constexpr int KW = DH / PER;
    constexpr int gshift = GV == 8 ? 5 : GV == 4 ? 6 : 7;   // log2 of the group size
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int n = lane & 15, blk = lane >> 4;
    // Which (row tile, (sequence, kv head), run) this block is.  Workgroups go to the eight XCDs in turn by
    // their linear number, and every XCD has its own L2: with the launch's own numbering the row tiles and runs
    // of one kv head land on all eight, and each fetches that head's keys and values from HBM for itself (68 MB
    // per launch at config 4 for 15 MB of input).  The blocks are renumbered so that a head's tiles and runs share
    // an XCD (a multiple of eight heads) or 8 / heads of them (1, 2 or 4 heads); other counts keep the launch's
    // numbering.
    unsigned tile_x = blockIdx.x, bh_y = blockIdx.y, run_z = blockIdx.z;
    if (gridDim.y % 8 == 0 || 8 % gridDim.y == 0) {
        const unsigned lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
        const unsigned per_head = gridDim.x * gridDim.z, xcd = lin % 8, slot = lin / 8;
        unsigned within;
        if (gridDim.y % 8 == 0) {
            bh_y = xcd + 8 * (slot / per_head);
            within = slot % per_head;
        } else {
            bh_y = xcd % gridDim.y;
            within = xcd / gridDim.y + (8 / gridDim.y) * slot;
        }
        tile_x = within % gridDim.x;
        run_z = within / gridDim.x;
    }
    const int64_t bh = bh_y;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    take_sequence_lengths(a, b);
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t cap = a.cap_tokens;
    const float c = a.scale * LOG2E;
    const u32 magic = vreg_const(Magic<BITS>::bits);
    // under a causal mask the last tiles see the most tokens: they are started first
    const int pos0 = (int)(a.causal ? gridDim.x - 1 - tile_x : tile_x) * qp;
    const int64_t n_total = a.n_packed + a.n_tail;
    auto visible = [&](int64_t p) { return a.causal ? n_total - a.Sq + p + 1 : n_total; };   // slots row p sees

    // ---- this lane's query row (score column): row j = 16 wave + n of the block
    // the block covers qp = 128 / R positions (rounded down)
    int lane_vis[P2_RB], lane_tvis[P2_RB];
    int lane_lo[P2_RB], lane_tlo[P2_RB];   // sliding window: first packed / tail token the row sees
    f16x8 qn[P2_RB][8];   // B operands: lane (n, blk) holds channels 32 ks + 8 blk + 0..7 of its row
#pragma unroll
    for (int rb = 0; rb < P2_RB; ++rb) {
        const int j = 16 * P2_RB * wave + 16 * rb + n;
        const int jh = (int)((unsigned)j / (unsigned)qp);   // head of the group, position in the block
        const int64_t pos = pos0 + (j - jh * qp);
        const bool row_ok = pos < a.Sq && jh < R;
        const int64_t qrow = (b * a.Hq + hkv * R + (jh < R ? jh : R - 1)) * a.Sq + (pos < a.Sq ? pos : a.Sq - 1);
        const int64_t vis = visible(row_ok ? pos : a.Sq - 1);
        lane_vis[rb] = (int)(vis < a.n_packed ? vis : a.n_packed);
        const int64_t tv = vis - a.n_packed;
        lane_tvis[rb] = (int)(tv < 0 ? 0 : tv < a.n_tail ? tv : a.n_tail);
        const int64_t first = window_first(a, n_total, row_ok ? pos : a.Sq - 1);
        lane_lo[rb] = (int)(first < a.n_packed ? first : a.n_packed);
        lane_tlo[rb] = (int)(first > a.n_packed ? first - a.n_packed : 0);
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
            const int64_t e0 = qrow * DH + 32 * ks + 8 * blk;
            if (a.q_dtype == VQ_F32) {
#pragma unroll
                for (int e = 0; e < 8; ++e) qn[rb][ks][e] = (f16)((const float *)a.q)[e0 + e];
            } else {
                qn[rb][ks] = ld_tail8(a.q, e0, a.q_dtype == VQ_BF16);
            }
        }
    }
    const int64_t last_pos = pos0 + qp - 1 < a.Sq - 1 ? pos0 + qp - 1 : a.Sq - 1;
    const int64_t vis_min = visible(pos0), vis_max = visible(last_pos);
    const int full_vis = (int)(vis_min < a.n_packed ? vis_min : a.n_packed);
    const int max_vis = (int)(vis_max < a.n_packed ? vis_max : a.n_packed);
    const int64_t tv_min = vis_min - a.n_packed, tv_max = vis_max - a.n_packed;
    const int full_tvis = (int)(tv_min < 0 ? 0 : tv_min < a.n_tail ? tv_min : a.n_tail);
    const int max_tvis = (int)(tv_max < 0 ? 0 : tv_max < a.n_tail ? tv_max : a.n_tail);
    const int n_punits = (max_vis + 31) / 32;
    const int n_tunits = (max_tvis + 31) / 32;
    const int n_work = n_punits + n_tunits;
    const int nsplit = (int)gridDim.z, sp = (int)run_z;
    // units below the window of the block's first row are seen by none of its rows
    const int64_t first_blk = window_first(a, n_total, pos0);
    const int w_lo = first_blk < a.n_packed ? (int)(first_blk / 32) : n_punits + (int)((first_blk - a.n_packed) / 32);
    const int w_n = n_work > w_lo ? n_work - w_lo : 0;
    const int w0 = w_lo + (int)((int64_t)w_n * sp / nsplit), w1 = w_lo + (int)((int64_t)w_n * (sp + 1) / nsplit);
    const int64_t first_all = window_first(a, n_total, last_pos);   // below it some row of the block sees nothing
    const int edge_lo = (int)(first_all < a.n_packed ? first_all : a.n_packed);
    const int edge_tlo = (int)(first_all > a.n_packed ? first_all - a.n_packed : 0);

    // ---- producer side
    const char *kb = (const char *)a.k_packed + bh * cap * KW * 4;
    const char *vb = (const char *)a.v_packed + bh * (cap / PER) * DH * 4;
    const M *ksb = (const M *)a.k_scale + bh * (cap >> gshift) * DH;
    const M *kzb = (const M *)a.k_zero + bh * (cap >> gshift) * DH;
    const M *vsb = (const M *)a.v_scale + bh * GV * cap;
    const M *vzb = (const M *)a.v_zero + bh * GV * cap;
    const int kt = tid >> 4, kc = tid & 15;       // key tile: token, 8-channel chunk of either half of the channels
    const int vc = tid & 127, vq = tid >> 7;      // value tile: channel of this launch's half, 8-token quarter
    const int vch = MF_D * v_half + vc;           // the thread's value channel in the head
    const int vg = vch >> gshift;                 // its channel group
    // byte offsets of the thread's key words (chunks kc and kc + 16), value word and value scale / zero piece inside a unit
    const unsigned k_off = (unsigned)((kt * KW + (BITS == 4 ? kc : kc >> 1)) * 4);
    constexpr unsigned k_off2 = (BITS == 4 ? 16 : 8) * 4;
    const unsigned v_off = (unsigned)(((BITS == 4 ? vq : vq >> 1) * DH + vch) * 4);
    const unsigned m_off = (unsigned)(((int64_t)vg * cap + 8 * vq) * sizeof(M));
    const int tp = lane & 15, cq = 4 * wave + (lane >> 4);   // tail values: token pair, channel quad
    const bool tail_bf16 = a.tail_dtype == VQ_BF16;
    const int64_t tbase = bh * a.tail_cap * DH;
    const f16x8 off8 = as_h8(Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair, Magic<BITS>::neg_off_pair);
    using Stage = PrStage2<M>;
    Meta8<M> ksr[2], kzr[2];   // key scale / zero of the thread's 2 x 8 channels in the token group last fetched
    int meta_group = -1;
    auto fetch = [&](int w, Stage &st) {
        if (w >= n_punits) {   // tail unit: the thread's key and value pieces travel in the value-meta slots
            // a block-uniform base (the unit's first token) plus a 32-bit offset of the thread's own; a token
            // past the end of the tail reads the last one instead (masked in the softmax)
            const int64_t t0 = (int64_t)(w - n_punits) * 32;
            const int last = (int)(a.n_tail - 1 - t0);   // >= 0: the unit starts inside the tail
            const char *kt0 = (const char *)a.k_tail + (tbase + t0 * DH) * 2, *vt0 = (const char *)a.v_tail + (tbase + t0 * DH) * 2 + 2 * MF_D * v_half;
            st.vs.u[0] = *reinterpret_cast<const uint4 *>(kt0 + (unsigned)((kt < last ? kt : last) * (DH * 2) + 16 * kc));
            st.k2 = *reinterpret_cast<const uint4 *>(kt0 + (unsigned)((kt < last ? kt : last) * (DH * 2) + 2 * MF_D + 16 * kc));
            // values: four channels of a token pair, so that the transposed tile is written in whole words
            const int ta = 2 * tp < last ? 2 * tp : last, tb = 2 * tp + 1 < last ? 2 * tp + 1 : last;
            const uint2 va = *reinterpret_cast<const uint2 *>(vt0 + (unsigned)(ta * (DH * 2) + 8 * cq));
            const uint2 vb2 = *reinterpret_cast<const uint2 *>(vt0 + (unsigned)(tb * (DH * 2) + 8 * cq));
            st.vz.u[0] = make_uint4(va.x, va.y, vb2.x, vb2.y);
            return;
        }
        // a block-uniform base that moves with the unit plus a 32-bit offset of the thread's own: the
        // per-unit address arithmetic stays on the scalar unit
        const int64_t base = (int64_t)w * 32;
        st.k2.x = *reinterpret_cast<const u32 *>(kb + base * (KW * 4) + k_off);
        st.k2.y = *reinterpret_cast<const u32 *>(kb + base * (KW * 4) + k_off + k_off2);
        st.k2.z = *reinterpret_cast<const u32 *>(vb + (base / PER) * (DH * 4) + v_off);
        st.vs.load((const char *)vsb + base * sizeof(M) + m_off);
        st.vz.load((const char *)vzb + base * sizeof(M) + m_off);
        const int grp = (int)(base >> gshift);
        if (grp != meta_group) {   // block-uniform
            meta_group = grp;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                ksr[i].load((const char *)ksb + (int64_t)grp * (DH * sizeof(M)) + 8u * (unsigned)sizeof(M) * (unsigned)(kc + 16 * i));
                kzr[i].load((const char *)kzb + (int64_t)grp * (DH * sizeof(M)) + 8u * (unsigned)sizeof(M) * (unsigned)(kc + 16 * i));
            }
        }
    };
    // the thread's eight codes of a word, in order, as exact fp16 numbers
    auto codes8 = [&](u32 w, int half) -> f16x8 {
        uint4 lo;
        if (BITS == 4) lo = word4_in_order(w, magic);
        else {
            uint4 hi;
            word2_in_order(w, magic, lo, hi);
            if (half) lo = hi;
        }
        return as_h8(lo) + off8;
    };
    auto unpack_to_lds = [&](int w, const Stage &st, int buf) {
        if (w < n_punits) {
            // keys: 2 x 8 channels of token kt; c s + z is formed exactly and rounded once
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * KST + 8 * kc]) = recon8(codes8(st.k2.x, kc & 1), ksr[0], kzr[0]);
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * KST + MF_D + 8 * kc]) = recon8(codes8(st.k2.y, kc & 1), ksr[1], kzr[1]);
            // values: 8 tokens of channel vch
            *reinterpret_cast<f16x8 *>(&s_v[buf][vc * PF_VSTRIDE + 8 * vq]) = recon8(codes8(st.k2.z, vq & 1), st.vs, st.vz);
        } else {
            // tail unit: plain key row chunk; values transposed, one word (a token pair of one channel)
            // at a time: the lanes of a wave cover 16 token pairs x 4 channel quads = 64 different banks
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * KST + 8 * kc]) = tail8_from_raw(st.vs.u[0], tail_bf16);
            *reinterpret_cast<f16x8 *>(&s_k[buf][pf_krow(kt) * KST + MF_D + 8 * kc]) = tail8_from_raw(st.k2, tail_bf16);
            const f16x8 v0 = tail8_from_raw(st.vz.u[0], tail_bf16);   // channels 0..3 of the first token, then of the second
#pragma unroll
            for (int e = 0; e < 4; ++e)
                *reinterpret_cast<f16x2 *>(&s_v[buf][(4 * cq + e) * PF_VSTRIDE + 2 * tp]) = f16x2{v0[e], v0[4 + e]};
        }
    };

    // ---- consumer state: O[rb][nt] rows 16 rb + 4 blk + r of the wave, channels 16 nt + n; L the row sums
    f32x4 O[P2_RB][8], L[P2_RB];
    float m_run[P2_RB], m_seen[P2_RB];
#pragma unroll
    for (int rb = 0; rb < P2_RB; ++rb) {
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) O[rb][nt] = f32x4{0.f, 0.f, 0.f, 0.f};
        L[rb] = f32x4{0.f, 0.f, 0.f, 0.f};
        m_run[rb] = -INFINITY;
        m_seen[rb] = -INFINITY;
    }
    const f16x8 ones = ones8();

    // move the reference of every row up to what it has seen and rescale the accumulators
    auto rescale = [&]() {
#pragma unroll
        for (int rb = 0; rb < P2_RB; ++rb) {
            float ms = m_seen[rb];
            ms = fmaxf(ms, __shfl_xor(ms, 16));
            ms = fmaxf(ms, __shfl_xor(ms, 32));
            const float m_new = fmaxf(m_run[rb], ms);
            const float alpha = m_new == -INFINITY ? 1.f : exp2f(m_run[rb] - m_new);
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const float al = __shfl(alpha, 4 * blk + r);
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) O[rb][nt][r] *= al;
                L[rb][r] *= al;
            }
            m_run[rb] = m_new;
        }
    };

    // The operands of a unit live in registers from one iteration to the next: the key tile's
    // rows (A) and the value tile's rows (Bv) of unit w+1 are read from LDS while unit w is
    // still being computed, so that the LDS traffic of the eight waves runs beside the products
    // and the softmax instead of in front of them.
    f16x8 A[2][8], Bv[8];
    auto load_keys = [&](int buf) {
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const f16 *kr = &s_k[buf][pf_krow(pf_tok(n >> 2, n & 3, T)) * KST + 8 * blk];
#pragma unroll
            for (int ks = 0; ks < 8; ++ks) A[T][ks] = *reinterpret_cast<const f16x8 *>(kr + 32 * ks);
        }
    };
    auto load_values = [&](int buf) {
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
            Bv[nt] = *reinterpret_cast<const f16x8 *>(&s_v[buf][(16 * nt + n) * PF_VSTRIDE + 8 * blk]);
    };

    // One unit: scores of the wave's row blocks (four independent accumulator chains side by
    // side), softmax against the lazily updated references (raised in place, with the
    // accumulators rescaled, when some row's scores outgrow its reference), second product.
    // `next` is the buffer of the following unit (stale but harmless after the last one).
    auto compute = [&](int next, int base, bool packed, int full, int lo_edge) {
        f32x4 S[P2_RB][2];
#pragma unroll
        for (int ks = 0; ks < 8; ++ks)
#pragma unroll
            for (int T = 0; T < 2; ++T)
#pragma unroll
                for (int rb = 0; rb < P2_RB; ++rb)
                    S[rb][T] = VQ_MFMA(A[T][ks], qn[rb][ks], ks == 0 ? (f32x4{0.f, 0.f, 0.f, 0.f}) : S[rb][T]);
        load_keys(next);
        bool grow = false;
#pragma unroll
        for (int rb = 0; rb < P2_RB; ++rb) {
            if (base + 32 > full || base < lo_edge) {
                const int lim = packed ? lane_vis[rb] : lane_tvis[rb], lo = packed ? lane_lo[rb] : lane_tlo[rb];
#pragma unroll
                for (int T = 0; T < 2; ++T)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        if (base + pf_tok(blk, r, T) >= lim || base + pf_tok(blk, r, T) < lo) S[rb][T][r] = -INFINITY;
            }
            const float mx = vmax3(vmax3(S[rb][0][0], S[rb][0][1], S[rb][0][2]), vmax3(S[rb][0][3], S[rb][1][0], S[rb][1][1]),
                                   vmax3(S[rb][1][2], S[rb][1][3], S[rb][1][3]));
            m_seen[rb] = mx * c;
            grow |= mx * c > m_run[rb] + RESCALE_SLACK;
        }
        if (__any(grow)) rescale();
        f16x8 P8[P2_RB];
#pragma unroll
        for (int rb = 0; rb < P2_RB; ++rb) {
            const float nm = m_run[rb] == -INFINITY ? 0.f : -m_run[rb];
            u32 P[4];
#pragma unroll
            for (int r = 0; r < 4; ++r)
                P[r] = as_u(f16x2{(f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[rb][0][r], c, nm)),
                                  (f16)__builtin_amdgcn_exp2f(__builtin_fmaf(S[rb][1][r], c, nm))});
            P8[rb] = as_h8(P[0], P[1], P[2], P[3]);
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt)
#pragma unroll
            for (int rb = 0; rb < P2_RB; ++rb) O[rb][nt] = VQ_MFMA(P8[rb], Bv[nt], O[rb][nt]);
#pragma unroll
        for (int rb = 0; rb < P2_RB; ++rb) L[rb] = VQ_MFMA(P8[rb], ones, L[rb]);
        load_values(next);
    };

    // ---- pipeline over the work units [w0, w1) on three LDS buffers: while unit w is computed
    // from registers, unit w+1 is read from its buffer, unit w+2 is unpacked into the third and
    // unit w+3 is requested from memory.  The producer's share comes after the unit's second product
    // (its first instructions issue while those products run); unpacking before the products in half
    // of the waves, to put the two waves of a SIMD out of step, measured 8 % slower.
    // The barrier between units waits for LDS only: __syncthreads() also waits for every outstanding
    // global load, i.e. for the unit just requested, once per unit.  For the same reason nothing
    // requested before the loop may still be pending inside it (the compiler would wait for it at
    // the loop head, and with it for whatever was requested since).
    Stage st;
    if (w1 > w0) {
        fetch(w0, st);
        unpack_to_lds(w0, st, 0);
        if (w0 + 1 < w1) {
            fetch(w0 + 1, st);
            unpack_to_lds(w0 + 1, st, 1);
        }
        if (w0 + 2 < w1) fetch(w0 + 2, st);
        __syncthreads();
        load_keys(0);
        load_values(0);
    }
    wait_global_accesses();
    int cur = 0;
    for (int w = w0; w < w1; ++w) {
        const int next = cur == 2 ? 0 : cur + 1, third = next == 2 ? 0 : next + 1;
        const bool packed = w < n_punits;
        const int base = packed ? w * 32 : (w - n_punits) * 32;
        compute(next, base, packed, packed ? full_vis : full_tvis, packed ? edge_lo : edge_tlo);
        if (w + 2 < w1) unpack_to_lds(w + 2, st, third);
        if (w + 3 < w1) fetch(w + 3, st);
        lds_barrier();
        cur = next;
    }

    // ---- every wave owns its rows: accumulator register r of lane (n, blk) is row 4 blk + r of the
    // row block, tile nt column n is channel 16 nt + n; the row's reference sits in lane 4 blk + r.
    // A launch with one run per row and no protected rows to patch in writes the output itself: the merge
    // of a single record is that record normalised (mfma_prefill_writes_output decides, for the host too).
    const bool direct = mfma_prefill_writes_output(a, nparts);
#pragma unroll
    for (int rb = 0; rb < P2_RB; ++rb)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const int jr = 16 * P2_RB * wave + 16 * rb + 4 * blk + r;
            const int jrh = (int)((unsigned)jr / (unsigned)qp);
            const int64_t pr = pos0 + (jr - jrh * qp);
            const float mr = __shfl(m_run[rb], 4 * blk + r);
            if (pr < a.Sq && jrh < R) {
                const int64_t row = (b * a.Hq + hkv * R + jrh) * a.Sq + pr;
                if (direct) {
                    // the only record of its row: what the merge would make of it (0 for a row that sees nothing)
                    const bool seen = mr != -INFINITY && L[rb][r] > 0.f;
#pragma unroll
                    for (int nt = 0; nt < 8; ++nt) {
                        const float v = seen ? __fdiv_rn(O[rb][nt][r], L[rb][r]) : 0.f;
                        const int64_t oi = row * DH + MF_D * v_half + 16 * nt + n;
                        if (a.out_dtype == VQ_F16) ((f16 *)a.out)[oi] = (f16)v;
                        else if (a.out_dtype == VQ_BF16) ((u16 *)a.out)[oi] = f32_to_bf16(v);
                        else ((float *)a.out)[oi] = v;
                    }
                    continue;
                }
                float *o = ws + (row * nparts + sp) * (DH + 2);
#pragma unroll
                for (int nt = 0; nt < 8; ++nt) o[2 + MF_D * v_half + 16 * nt + n] = O[rb][nt][r];
                if (n == 0 && v_half == 0) { o[0] = mr * LN2; o[1] = L[rb][r]; }   // both launches form the same two
            }
        }
}

int mfma_prefill_block_rows(const vq_attend_args &a);

// the blocks of eight waves: 256 rows of 128-channel heads, 128 rows of 256-channel heads (which have no other blocks)
static bool prefill_row_blocks(const vq_attend_args &a) {
    return (a.Hq / a.Hkv) * a.Sq >= (a.D == 2 * MF_D ? 128 : 256);
}

bool mfma_prefill_supported(const vq_attend_args &a) {
    if ((a.D != MF_D && a.D != 2 * MF_D) || a.n_packed < 0 || a.Sq < 16) return false;
    if (a.Hq % a.Hkv != 0) return false;
    const int64_t R = a.Hq / a.Hkv;
    // the blocks of eight waves take any group of up to 64 heads (256 / R or 128 / R positions a block, rounded
    // down); the 64-row blocks the powers of two up to eight
    if (!(R == 1 || R == 2 || R == 4 || R == 8) && !(R >= 1 && R <= 64 && prefill_row_blocks(a))) return false;
    // (256-channel heads: 128-row blocks only, fp16 scale / zero -- float32 ones do not fit the registers beside
    // twice the key operands)
    if (a.D == 2 * MF_D && (!prefill_row_blocks(a) || (a.n_packed > 0 && a.meta_dtype != VQ_F16))) return false;
    if (a.n_packed > 0) {
        if (!(a.pack_bits == 2 || a.pack_bits == 4)) return false;
        if (!(a.group == 32 || a.group == 64 || a.group == 128)) return false;
        // float32 scale / zero: the 256-row blocks take it (they reconstruct in the producer); fewer rows stay on
        // the 8-row tiles of the decode kernel
        if (a.meta_dtype != VQ_F16 && !(a.meta_dtype == VQ_F32 && prefill_row_blocks(a))) return false;
        if (a.v_layout != VQ_V_TOKEN_PACKED) return false;
        if (a.n_packed % 32 != 0 || a.cap_tokens % 32 != 0 || a.cap_tokens % a.group != 0) return false;
        if (a.cap_tokens > ((int64_t)1 << 28)) return false;   // 32-bit byte offsets inside one (sequence, kv head) slab
    } else {
        // plain keys and values only (the tail units of the same kernels): worth the matrix unit
        // from a few hundred tokens on
        if (a.n_tail < 64 || a.packed_lens != nullptr) return false;
    }
    if (!(a.scale > 0.f)) return false;
    if (a.n_tail > 0 && (!(a.tail_dtype == VQ_F16 || a.tail_dtype == VQ_BF16) || (((uintptr_t)a.k_tail | (uintptr_t)a.v_tail) & 15u))) return false;
    if (a.B * a.Hkv > 65535) return false;
    if (a.n_tail > 0 && a.tail_cap * a.D % 8 != 0) return false;
    const uintptr_t al = (uintptr_t)a.k_packed | (uintptr_t)a.v_packed | (uintptr_t)a.k_scale | (uintptr_t)a.k_zero |
                         (uintptr_t)a.v_scale | (uintptr_t)a.v_zero;
    if (a.n_packed > 0 && (al & 15u)) return false;
    if (prefill_row_blocks(a) && a.q_dtype != VQ_F32 && ((uintptr_t)a.q & 15u)) return false;
    return true;
}

int mfma_prefill_block_rows(const vq_attend_args &a) {
    return a.D == 2 * MF_D ? 128 : prefill_row_blocks(a) ? 256 : 64;
}

bool mfma_prefill_direct_output(const vq_attend_args &a, int nparts) {
    return prefill_row_blocks(a) && mfma_prefill_writes_output(a, nparts);
}

bool mfma_prefill_uses_tiles(const vq_attend_args &a) {
    return a.kv_tiles != nullptr && a.packed_lens == nullptr && a.D == MF_D && mfma_prefill_block_rows(a) == 256 &&
           ((uintptr_t)a.kv_tiles & 15u) == 0 && a.tile_cap * 32 >= a.n_packed + a.n_tail && a.n_packed % 32 == 0;
}

int launch_prefill_tiles(const vq_attend_args &a, int64_t first_unit, int64_t n_units) {
    const char *fn = "vq_kivi_prefill_tiles";
    VQ_REQUIRE(a.D == MF_D && a.packed_lens == nullptr, VQ_ERR_UNSUPPORTED, "%s: head_dim 128 and one length for the batch only", fn);
    VQ_REQUIRE(a.B * a.Hkv <= 65535 && n_units <= 0x7fffffff, VQ_ERR_UNSUPPORTED, "%s: too many (sequence, kv head) pairs or units", fn);
    if (a.n_packed > 0) {
        VQ_REQUIRE((a.pack_bits == 2 || a.pack_bits == 4) && (a.group == 32 || a.group == 64 || a.group == 128) &&
                       (a.meta_dtype == VQ_F16 || a.meta_dtype == VQ_F32) && a.v_layout == VQ_V_TOKEN_PACKED,
                   VQ_ERR_UNSUPPORTED, "%s: 2- or 4-bit codes, groups of 32 / 64 / 128, fp16 or float32 scale / zero, token-packed values", fn);
        VQ_REQUIRE(a.n_packed % 32 == 0 && a.cap_tokens % 32 == 0 && a.cap_tokens % a.group == 0 && a.cap_tokens <= ((int64_t)1 << 28),
                   VQ_ERR_UNSUPPORTED, "%s: packed counts must be multiples of 32 and of the group", fn);
        const uintptr_t al = (uintptr_t)a.k_packed | (uintptr_t)a.v_packed | (uintptr_t)a.k_scale | (uintptr_t)a.k_zero |
                             (uintptr_t)a.v_scale | (uintptr_t)a.v_zero;
        VQ_REQUIRE((al & 15u) == 0, VQ_ERR_UNSUPPORTED, "%s: cache arrays must be 16-byte aligned", fn);
    }
    if (a.n_tail > 0)
        VQ_REQUIRE((a.tail_dtype == VQ_F16 || a.tail_dtype == VQ_BF16) && ((((uintptr_t)a.k_tail | (uintptr_t)a.v_tail) & 15u) == 0) &&
                       a.tail_cap >= a.n_tail, VQ_ERR_UNSUPPORTED, "%s: fp16 or bf16 tail, 16-byte aligned", fn);
    hipStream_t st = (hipStream_t)a.stream;
    const dim3 grid((unsigned)n_units, (unsigned)(a.B * a.Hkv));
    const int gv = a.n_packed > 0 ? (int)(MF_D / a.group) : 4;
    const bool f32 = a.n_packed > 0 && a.meta_dtype == VQ_F32;
#define VQ_TILES(BITS, GV)                                                                                                  \
    do {                                                                                                                   \
        if (f32) hipLaunchKernelGGL((prefill_tiles_kernel<BITS, GV, float>), grid, dim3(PR_THREADS), 0, st, a, (int)first_unit); \
        else hipLaunchKernelGGL((prefill_tiles_kernel<BITS, GV, f16>), grid, dim3(PR_THREADS), 0, st, a, (int)first_unit);  \
    } while (0)
    if (a.pack_bits == 4 || a.n_packed == 0) { if (gv == 1) VQ_TILES(4, 1); else if (gv == 2) VQ_TILES(4, 2); else VQ_TILES(4, 4); }
    else { if (gv == 1) VQ_TILES(2, 1); else if (gv == 2) VQ_TILES(2, 2); else VQ_TILES(2, 4); }
#undef VQ_TILES
    VQ_HIP_CHECK_LAUNCH(fn);
    return VQ_OK;
}

bool launch_attend_mfma_prefill(const vq_attend_args &a, const AttendPlan &p) {
    hipStream_t st = (hipStream_t)a.stream;
    float *ws = (float *)a.workspace;
    const int R = (int)(a.Hq / a.Hkv);
    const int rows = mfma_prefill_block_rows(a);
    const int qp = rows / R, tiles = (int)cdiv(a.Sq, qp);
    const dim3 grid((unsigned)tiles, (unsigned)(a.B * a.Hkv), (unsigned)p.nsplit), block(256);
    if (a.D == 2 * MF_D) {
        // heads of 256 channels: one launch per half of the output's channels
        const int gv2 = a.n_packed > 0 ? (int)(2 * MF_D / a.group) : 8;
#define VQ_LAUNCH2(BITS, GV)                                                                                            \
        for (int half = 0; half < 2; ++half)                                                                            \
            hipLaunchKernelGGL((attend_prefill_rows_d256_kernel<BITS, GV, f16>), grid, dim3(PR_THREADS), 0, st, a, qp, p.nparts, half, ws);
        if (a.pack_bits == 4 || a.n_packed == 0) { if (gv2 == 2) VQ_LAUNCH2(4, 2) else if (gv2 == 4) VQ_LAUNCH2(4, 4) else VQ_LAUNCH2(4, 8) }
        else { if (gv2 == 2) VQ_LAUNCH2(2, 2) else if (gv2 == 4) VQ_LAUNCH2(2, 4) else VQ_LAUNCH2(2, 8) }
#undef VQ_LAUNCH2
        return mfma_prefill_writes_output(a, p.nparts);
    }
    const int gv = a.n_packed > 0 ? (int)(MF_D / a.group) : 4;   // without packed units any instantiation serves
#define VQ_LAUNCH(BITS, GV)                                                                                          \
    do {                                                                                                             \
        if (rows == 256 && mfma_prefill_uses_tiles(a))                                                               \
            hipLaunchKernelGGL((attend_prefill_rows_kernel<4, 4, f16, true>), grid, dim3(PR_THREADS), 0, st, a, qp, p.nparts, ws); \
        else if (rows == 256 && a.n_packed > 0 && a.meta_dtype == VQ_F32)                                            \
            hipLaunchKernelGGL((attend_prefill_rows_kernel<BITS, GV, float>), grid, dim3(PR_THREADS), 0, st, a, qp, p.nparts, ws); \
        else if (rows == 256)                                                                                        \
            hipLaunchKernelGGL((attend_prefill_rows_kernel<BITS, GV, f16>), grid, dim3(PR_THREADS), 0, st, a, qp, p.nparts, ws); \
        else                                                                                                         \
            hipLaunchKernelGGL((attend_prefill_kernel<BITS, GV>), grid, block, 0, st, a, qp, p.nparts, ws);           \
    } while (0)
    if (a.pack_bits == 4 || a.n_packed == 0) { if (gv == 1) VQ_LAUNCH(4, 1); else if (gv == 2) VQ_LAUNCH(4, 2); else VQ_LAUNCH(4, 4); }
    else { if (gv == 1) VQ_LAUNCH(2, 1); else if (gv == 2) VQ_LAUNCH(2, 2); else VQ_LAUNCH(2, 4); }
#undef VQ_LAUNCH
    return rows == 256 && mfma_prefill_writes_output(a, p.nparts);
}

}  // namespace vq
