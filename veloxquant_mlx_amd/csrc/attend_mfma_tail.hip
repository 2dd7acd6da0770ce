// MFMA decode attention over the un-quantised fp16 tail of a KIVI cache, and the
// dispatch of the MFMA decode path.
//
// One block of four waves per kv head runs the two products of attention on plain
// rows, in units of 32 tokens:
//   S^T[token, row] = K[token, :] . q[row, :]      A = K as stored, B = q
//   O[row, chan]   += P[row, token] * V[token, chan]   A = P, B = V
// Values are loaded as eight rows of eight channels per lane and transposed in
// registers into the token-major k-slots.  The softmax denominator is a ninth
// output tile against a ones operand.  The block writes one (max, sum,
// accumulator) partial per query row, in slot `nsplit` of the partials the packed
// prefix kernel fills, and the shared merge kernel combines them.
#include "attend_mfma.hpp"

namespace vq {

// Per-wave attention state: nine output tiles (eight of 16 channels plus the
// softmax denominator) and the running row maximum.
struct TailAcc {
    f32x4 O[9];
    float m_run;   // log2 domain, row = lane % 16, replicated over the four lane groups
};

// Online-softmax step for one unit of 32 tokens.  S holds the raw scores of this
// lane's column (query row) for its eight tokens.  Returns P in the A-operand
// layout of the P.V product (pair r = tile 0 register r, tile 1 register r).
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

// token (0..31 inside a unit) of S^T row i of tile T: rows of the two tiles interleave so
// that accumulator register r of tile T is k-slot pair r of the P.V product
__device__ __forceinline__ int tail_tok(int blk, int r, int T) { return 8 * blk + r + 4 * T; }

__global__ __launch_bounds__(256) void attend_mfma_tail_kernel(vq_attend_args a, int nsplit, int nparts,
                                                               float *__restrict__ ws) {
    __shared__ float s_m[4][MF_ROWS];
    __shared__ float s_l[4][MF_ROWS];
    __shared__ float s_o[4][MF_ROWS][MF_D];

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15, blk = lane >> 4;
    const int64_t bh = blockIdx.x;
    const int64_t hkv = bh % a.Hkv, b = bh / a.Hkv;
    const int R = (int)(a.Hq / a.Hkv);
    const int64_t row0 = b * a.Hq + hkv * R;   // first query row of this kv head (Sq == 1)
    const float c = a.scale * LOG2E;

    TailAcc acc;
#pragma unroll
    for (int n = 0; n < 9; ++n) acc.O[n] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc.m_run = -INFINITY;

    const f16 *kt = (const f16 *)a.k_tail + bh * a.tail_cap * MF_D;
    const f16 *vt = (const f16 *)a.v_tail + bh * a.tail_cap * MF_D;
    f16x8 qT[4];
#pragma unroll
    for (int ks = 0; ks < 4; ++ks)
#pragma unroll
        for (int j = 0; j < 8; ++j)
            qT[ks][j] = i < R ? (f16)ldq(a.q, a.q_dtype, (row0 + i) * MF_D + 32 * blk + 8 * ks + j) : (f16)0.f;
    const f16x8 ones = ones8();
    const int n_tu = (int)((a.n_tail + 31) / 32);
    for (int u = wave; u < n_tu; u += 4) {
        const int64_t base = (int64_t)u * 32;
        f32x4 S[2];
#pragma unroll
        for (int T = 0; T < 2; ++T) {
            const int64_t tok = base + tail_tok(i >> 2, i & 3, T);
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
            for (int r = 0; r < 4; ++r)
                if (i < R && base + tail_tok(blk, r, T) >= a.n_tail) S[T][r] = -INFINITY;
        const f16x8 P = tail_softmax_unit(S, c, acc, blk);
        f16x8 vr[8];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const int64_t tA = base + tail_tok(blk, p, 0), tB = base + tail_tok(blk, p, 1);
            vr[2 * p] = *reinterpret_cast<const f16x8 *>(vt + (tA < a.n_tail ? tA : 0) * MF_D + 8 * i);
            vr[2 * p + 1] = *reinterpret_cast<const f16x8 *>(vt + (tB < a.n_tail ? tB : 0) * MF_D + 8 * i);
        }
#pragma unroll
        for (int nt = 0; nt < 8; ++nt) {   // lane column i is channel 8*i + nt
            f16x8 Bv;
#pragma unroll
            for (int j = 0; j < 8; ++j) Bv[j] = vr[j][nt];
            acc.O[nt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, Bv, acc.O[nt], 0, 0, 0);
        }
        acc.O[8] = __builtin_amdgcn_mfma_f32_16x16x32_f16(P, ones, acc.O[8], 0, 0, 0);
    }

    // merge the four waves: accumulator register r of lane (i, blk) is row 4*blk + r, channel 8*i + nt
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
        float *o = ws + ((row0 + row) * nparts + nsplit) * MF_PART;
        o[2 + d] = num;
        if (d == 0) { o[0] = gm * LN2; o[1] = den; }
    }
}

void launch_mfma_tail(const vq_attend_args &a, int nsplit, int nparts, float *ws, hipStream_t st) {
    hipLaunchKernelGGL(attend_mfma_tail_kernel, dim3((unsigned)(a.B * a.Hkv)), dim3(256), 0, st, a, nsplit, nparts, ws);
}

bool mfma_decode_supported(const vq_attend_args &a) {
    if (a.D != MF_D || a.Sq != 1 || a.n_packed <= 0) return false;
    if (a.Hq % a.Hkv != 0 || 2 * (a.Hq / a.Hkv) > MF_ROWS) return false;  // high + remainder columns
    if (!(a.pack_bits == 2 || a.pack_bits == 4)) return false;
    if (!(a.group == 32 || a.group == 64 || a.group == 128)) return false;
    if (a.v_layout != VQ_V_TOKEN_PACKED) return false;
    if (a.n_packed % 32 != 0 || a.cap_tokens % 32 != 0 || a.cap_tokens % a.group != 0) return false;
    if (a.cap_tokens > (1 << 24)) return false;   // per-lane byte offsets are 32-bit
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
    float *ws = (float *)a.workspace;
    if (a.n_tail > 0) launch_mfma_tail(a, nsplit, nparts, ws, st);
    if (a.meta_dtype == VQ_F16) launch_mfma_packed_f16meta(a, nsplit, split_len, nparts, ws, st);
    else launch_mfma_packed_f32meta(a, nsplit, split_len, nparts, ws, st);
    return VQ_OK;
}

}  // namespace vq
