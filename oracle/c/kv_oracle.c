/* Plain-C restatement of the KV-cache compression hot path.
 *
 * TEST INFRASTRUCTURE ONLY: linked by tests, the smoke check and the
 * benchmark's CPU-baseline leg; never by the shipped library.
 *
 * Scalar, single threaded, one IEEE float32 rounding per operation (build with
 * -ffp-contract=off).  Reference files restated (paths relative to the
 * VeloxQuant-MLX tree):
 *   group quantisation   veloxquant_mlx/metal/src/kivi_group_quant_channel.metal:35-88
 *                        veloxquant_mlx/metal/src/kivi_group_quant_token.metal:29-90
 *   word packing         veloxquant_mlx/cache/turboquant_rvq_cache.py:82-106
 *   VQ assignment        veloxquant_mlx/metal/src/vecinfer_quantize.metal:8-28
 *   decode attention     veloxquant_mlx/metal/src/scalar_affine_attend.metal:8-175
 *                        (dense float32 form of tests/metal/test_scalar_attend.py:85-115)
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* x: [BH, S, D] float32.  axis 0: groups along S (keys), scale/zero [BH, GK, D].
 * axis 1: groups along D (values), scale/zero [BH, S, GV]. */
int kvo_group_quant(const float *x, int64_t BH, int64_t S, int64_t D, int axis,
                    int group, int levels, float eps,
                    uint8_t *codes, float *scale, float *zero)
{
    if (axis == 0) {
        int64_t GK = (S + group - 1) / group;
        for (int64_t bh = 0; bh < BH; ++bh)
            for (int64_t gk = 0; gk < GK; ++gk)
                for (int64_t d = 0; d < D; ++d) {
                    int64_t s0 = gk * group, s1 = s0 + group < S ? s0 + group : S;
                    float mn = INFINITY, mx = -INFINITY;
                    for (int64_t s = s0; s < s1; ++s) {
                        float v = x[(bh * S + s) * D + d];
                        mn = v < mn ? v : mn;
                        mx = v > mx ? v : mx;
                    }
                    /* a ragged last group is padded with copies of the last live
                     * element, which is already inside [s0, s1) */
                    float sc = (mx - mn) / (float)levels;
                    if (sc < eps) sc = eps;
                    scale[(bh * GK + gk) * D + d] = sc;
                    zero[(bh * GK + gk) * D + d] = mn;
                    for (int64_t s = s0; s < s1; ++s) {
                        float v = x[(bh * S + s) * D + d];
                        float q = rintf((v - mn) / sc);
                        q = q < 0.f ? 0.f : (q > (float)levels ? (float)levels : q);
                        codes[(bh * S + s) * D + d] = (uint8_t)q;
                    }
                }
    } else {
        int64_t GV = (D + group - 1) / group;
        for (int64_t r = 0; r < BH * S; ++r)
            for (int64_t gv = 0; gv < GV; ++gv) {
                int64_t d0 = gv * group, d1 = d0 + group < D ? d0 + group : D;
                float mn = INFINITY, mx = -INFINITY;
                for (int64_t d = d0; d < d1; ++d) {
                    float v = x[r * D + d];
                    mn = v < mn ? v : mn;
                    mx = v > mx ? v : mx;
                }
                float sc = (mx - mn) / (float)levels;
                if (sc < eps) sc = eps;
                scale[r * GV + gv] = sc;
                zero[r * GV + gv] = mn;
                for (int64_t d = d0; d < d1; ++d) {
                    float q = rintf((x[r * D + d] - mn) / sc);
                    q = q < 0.f ? 0.f : (q > (float)levels ? (float)levels : q);
                    codes[r * D + d] = (uint8_t)q;
                }
            }
    }
    return 0;
}

/* codes [rows, D] -> words [rows, ceil(D / (32/bits))], LSB first. */
int kvo_pack_words(const uint8_t *codes, int64_t rows, int64_t D, int bits, uint32_t *words)
{
    int per = 32 / bits;
    int64_t W = (D + per - 1) / per;
    for (int64_t r = 0; r < rows; ++r)
        for (int64_t w = 0; w < W; ++w) {
            uint32_t acc = 0;
            for (int i = 0; i < per; ++i) {
                int64_t d = w * per + i;
                if (d < D) acc |= (uint32_t)codes[r * D + d] << (i * bits);
            }
            words[r * W + w] = acc;
        }
    return 0;
}

/* x [N, sub] float32, cb [C, sub] float32 -> idx [N] */
int kvo_vq_assign(const float *x, int64_t N, const float *cb, int C, int sub, int32_t *idx)
{
    for (int64_t n = 0; n < N; ++n) {
        float best = INFINITY;
        int bi = 0;
        for (int c = 0; c < C; ++c) {
            float dist = 0.f;
            for (int i = 0; i < sub; ++i) {
                float d = x[n * sub + i] - cb[c * sub + i];
                float sq = d * d;
                dist = dist + sq;
            }
            if (dist < best) { best = dist; bi = c; }
        }
        idx[n] = bi;
    }
    return 0;
}

/* Dense attention over reconstructed K/V, one query row per (b, h_q).
 * q [B,Hq,Sq,D]; codes [B,Hkv,S,D]; k meta [B,Hkv,GK,D]; v meta [B,Hkv,S,GV];
 * tail [B,Hkv,T,D] float32 (may be T == 0).  causal: queries aligned to the end
 * of (S + T) slots.  Accumulates in double. */
int kvo_attend(const float *q, int64_t B, int64_t Hq, int64_t Sq, int64_t D,
               const uint8_t *kc, const float *ks, const float *kz,
               const uint8_t *vc, const float *vs, const float *vz,
               int64_t Hkv, int64_t S, int group,
               const float *kt, const float *vt, int64_t T,
               float scale, int causal, float *out)
{
    int64_t GK = (S + group - 1) / group, GV = (D + group - 1) / group;
    int64_t hpk = Hq / Hkv, Stot = S + T;
    double *sc = (double *)malloc(sizeof(double) * (size_t)(Stot > 0 ? Stot : 1));
    double *acc = (double *)malloc(sizeof(double) * (size_t)D);
    if (!sc || !acc) { free(sc); free(acc); return -1; }
    for (int64_t b = 0; b < B; ++b)
        for (int64_t h = 0; h < Hq; ++h)
            for (int64_t iq = 0; iq < Sq; ++iq) {
                int64_t hk = h / hpk, bh = b * Hkv + hk;
                const float *qr = q + ((b * Hq + h) * Sq + iq) * D;
                int64_t last = causal ? (Stot - Sq + iq) : (Stot - 1);
                double m = -INFINITY;
                for (int64_t s = 0; s <= last; ++s) {
                    double dot = 0.0;
                    if (s < S) {
                        for (int64_t d = 0; d < D; ++d) {
                            float p = (float)kc[(bh * S + s) * D + d] * ks[(bh * GK + s / group) * D + d];
                            float kh = p + kz[(bh * GK + s / group) * D + d];
                            dot += (double)qr[d] * (double)kh;
                        }
                    } else {
                        for (int64_t d = 0; d < D; ++d)
                            dot += (double)qr[d] * (double)kt[(bh * T + (s - S)) * D + d];
                    }
                    sc[s] = dot * (double)scale;
                    if (sc[s] > m) m = sc[s];
                }
                double den = 0.0;
                memset(acc, 0, sizeof(double) * (size_t)D);
                for (int64_t s = 0; s <= last; ++s) {
                    double w = exp(sc[s] - m);
                    den += w;
                    if (s < S) {
                        for (int64_t d = 0; d < D; ++d) {
                            float p = (float)vc[(bh * S + s) * D + d] * vs[(bh * S + s) * GV + d / group];
                            float vh = p + vz[(bh * S + s) * GV + d / group];
                            acc[d] += w * (double)vh;
                        }
                    } else {
                        for (int64_t d = 0; d < D; ++d)
                            acc[d] += w * (double)vt[(bh * T + (s - S)) * D + d];
                    }
                }
                float *o = out + ((b * Hq + h) * Sq + iq) * D;
                for (int64_t d = 0; d < D; ++d) o[d] = last >= 0 ? (float)(acc[d] / den) : 0.f;
            }
    free(sc);
    free(acc);
    return 0;
}
