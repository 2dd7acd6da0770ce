// Layout-agnostic attention over [quantised prefix | tail] and the split merge.
//
// One wave per (query row, token split): lanes stripe the head dimension, each
// slot's key is rebuilt as code*scale+zero in float32, the dot product is
// reduced across the wave, and an online softmax accumulates the rebuilt value
// row -- the scheme of veloxquant_mlx/metal/src/scalar_affine_attend.metal:57-106
// with the split moved from SIMD groups of one threadgroup to independent
// waves whose (max, sum, accumulator) partials are merged by a second kernel
// (the merge of scalar_affine_attend.metal:149-174).
//
// This path accepts every head_dim <= 256, bit width, group size, value layout
// and tail dtype; the MFMA kernels in attend_mfma.hip cover the shapes that
// matter for throughput and share the partial format and the merge kernel.
#include "attend.hpp"

namespace vq {

__device__ __forceinline__ float ld_tag(const void *p, int tag, int64_t i) {
    if (tag == VQ_F16) return (float)((const f16 *)p)[i];
    if (tag == VQ_BF16) return bf16_to_f32(((const u16 *)p)[i]);
    return ((const float *)p)[i];
}
__device__ __forceinline__ void st_tag(void *p, int tag, int64_t i, float v) {
    if (tag == VQ_F16) ((f16 *)p)[i] = (f16)v;
    else if (tag == VQ_BF16) ((u16 *)p)[i] = f32_to_bf16(v);
    else ((float *)p)[i] = v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
    return v;
}

__global__ __launch_bounds__(256) void attend_generic_kernel(vq_attend_args a, int nsplit, int64_t split_len,
                                                             float *__restrict__ ws) {
    const int lane = threadIdx.x & 63;
    const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t rows = a.B * a.Hq * a.Sq;
    if (wid >= rows * nsplit) return;  // whole waves leave together
    const int64_t row = wid / nsplit;
    const int sp = (int)(wid % nsplit);
    const int64_t iq = row % a.Sq, h = (row / a.Sq) % a.Hq, b = row / (a.Sq * a.Hq);
    const int64_t hpk = a.Hq / a.Hkv, bh = b * a.Hkv + h / hpk;
    take_sequence_lengths(a, b);
    const int64_t D = a.D, n_total = a.n_packed + a.n_tail;
    const int64_t last = a.causal ? (n_total - a.Sq + iq) : (n_total - 1);
    int64_t t0 = (int64_t)sp * split_len, t1 = t0 + split_len;
    if (t1 > last + 1) t1 = last + 1;
    const int64_t first = window_first(a, n_total, iq);
    if (t0 < first) t0 = first;

    const int bits = a.pack_bits, per = 32 / bits, g = a.group;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t W = (D + per - 1) / per, GV = (D + g - 1) / g, GKcap = (a.cap_tokens + g - 1) / g;
    const uint32_t *kp = (const uint32_t *)a.k_packed, *vp = (const uint32_t *)a.v_packed;

    float qv[4], acc[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int64_t d = lane + 64 * j;
        qv[j] = d < D ? ld_tag(a.q, a.q_dtype, row * D + d) : 0.0f;
        acc[j] = 0.0f;
    }
    float m = -INFINITY, l = 0.0f;
    for (int64_t t = t0; t < t1; ++t) {
        float kh[4], vh[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int64_t d = lane + 64 * j;
            kh[j] = 0.0f; vh[j] = 0.0f;
            if (d >= D) continue;
            if (t < a.n_packed) {
                uint32_t kw = kp[(bh * a.cap_tokens + t) * W + d / per];
                float kc = (float)((kw >> ((d % per) * bits)) & mask);
                int64_t kmi = (bh * GKcap + t / g) * D + d;
                kh[j] = __fadd_rn(__fmul_rn(kc, ld_tag(a.k_scale, a.meta_dtype, kmi)), ld_tag(a.k_zero, a.meta_dtype, kmi));
                uint32_t vw;
                int sh;
                int64_t vmi;
                if (a.v_layout == VQ_V_CHANNEL_PACKED) {
                    vw = vp[(bh * a.cap_tokens + t) * W + d / per];
                    sh = (int)(d % per) * bits;
                    vmi = (bh * a.cap_tokens + t) * GV + d / g;
                } else {
                    vw = vp[(bh * (a.cap_tokens / per) + t / per) * D + d];
                    sh = (int)(t % per) * bits;
                    vmi = (bh * GV + d / g) * a.cap_tokens + t;
                }
                float vc = (float)((vw >> sh) & mask);
                vh[j] = __fadd_rn(__fmul_rn(vc, ld_tag(a.v_scale, a.meta_dtype, vmi)), ld_tag(a.v_zero, a.meta_dtype, vmi));
                if (a.num_splits == -2) {   // the reconstruction as a cache that stores it in fp16 holds it
                    kh[j] = (float)(f16)kh[j];
                    vh[j] = (float)(f16)vh[j];
                }
            } else {
                int64_t ti = (bh * a.tail_cap + (t - a.n_packed)) * D + d;
                kh[j] = ld_tag(a.k_tail, a.tail_dtype, ti);
                vh[j] = ld_tag(a.v_tail, a.tail_dtype, ti);
            }
        }
        float dot = qv[0] * kh[0] + qv[1] * kh[1] + qv[2] * kh[2] + qv[3] * kh[3];
        float s = wave_sum(dot) * a.scale;
        float mn = fmaxf(m, s);
        float f = __expf(m - mn), w = __expf(s - mn);
        l = l * f + w;
        m = mn;
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[j] = acc[j] * f + w * vh[j];
    }
    float *o = ws + (row * nsplit + sp) * (D + 2);
    if (lane == 0) { o[0] = m; o[1] = l; }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int64_t d = lane + 64 * j;
        if (d < D) o[2 + d] = acc[j];
    }
}

__global__ void attend_merge_kernel(const float *__restrict__ ws, int64_t rows, int nsplit, int64_t D,
                                    void *__restrict__ out, int out_dtype) {
    const int64_t n = rows * D;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = e / D, d = e % D;
        st_tag(out, out_dtype, e, merge_records<false>(ws + row * nsplit * (D + 2), nsplit, D + 2, d));
    }
}

// Up to four records per row, even D: a thread takes two neighbouring channels (the records'
// accumulators start 8 bytes into a record whose size is a multiple of 8, so the pairs are
// aligned) and reads each record's maximum and sum once for both.
__global__ void attend_merge4_kernel(const float *__restrict__ ws, int64_t rows, int nsplit, int64_t D,
                                     void *__restrict__ out, int out_dtype) {
    const int64_t half = D / 2, n = rows * half;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t row = e / half, d = 2 * (e % half);
        const float *rec = ws + row * nsplit * (D + 2);
        float m[4], l[4];
        float2 o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float *q = rec + (int64_t)(j < nsplit ? j : 0) * (D + 2);
            m[j] = j < nsplit ? q[0] : -INFINITY;
            l[j] = q[1];
            o[j] = *reinterpret_cast<const float2 *>(q + 2 + d);
        }
        const float gm = fmaxf(fmaxf(m[0], m[1]), fmaxf(m[2], m[3]));
        float den = 0.f, nx = 0.f, ny = 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (m[j] != -INFINITY) {
                const float f = __expf(m[j] - gm);
                den += l[j] * f;
                nx += o[j].x * f;
                ny += o[j].y * f;
            }
        st_tag(out, out_dtype, row * D + d, den > 0.f ? nx / den : 0.f);
        st_tag(out, out_dtype, row * D + d + 1, den > 0.f ? ny / den : 0.f);
    }
}

// Protected rows: one wave per query row redoes the merge of the row's partials keeping the sums
// apart, takes the weight of every visible stand-in out of the softmax sum (its values are stored
// as zeros, so the numerators never saw it; its key is rebuilt from the packed store as
// code * scale + zero), then folds the exact rows in with a running maximum and writes the row.
__global__ __launch_bounds__(256) void attend_sink_patch_kernel(vq_attend_args a, int nparts, const float *__restrict__ ws) {
    const int lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t rows = a.B * a.Hq * a.Sq;
    if (row >= rows) return;
    const int64_t iq = row % a.Sq, h = (row / a.Sq) % a.Hq, b = row / (a.Sq * a.Hq);
    const int64_t hpk = a.Hq / a.Hkv, bh = b * a.Hkv + h / hpk;
    take_sequence_lengths(a, b);
    const int64_t D = a.D, n_total = a.n_packed + a.n_tail;
    const int64_t last = a.causal ? (n_total - a.Sq + iq) : (n_total - 1);
    const int64_t first = window_first(a, n_total, iq);
    const int bits = a.pack_bits, per = 32 / bits, g = a.group;
    const uint32_t mask = (1u << bits) - 1u;
    const int64_t W = (D + per - 1) / per, GKcap = (a.cap_tokens + g - 1) / g;
    const uint32_t *kp = (const uint32_t *)a.k_packed;

    const float *rec = ws + row * nparts * (D + 2);
    float gm = -INFINITY;
    for (int s = 0; s < nparts; ++s) gm = fmaxf(gm, rec[(int64_t)s * (D + 2)]);
    float qv[4], num[4] = {0.f, 0.f, 0.f, 0.f}, den = 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t d = lane + 64 * j;
        qv[j] = d < D ? ld_tag(a.q, a.q_dtype, row * D + d) : 0.0f;
    }
    for (int s = 0; s < nparts; ++s) {
        const float *r = rec + (int64_t)s * (D + 2);
        if (r[0] == -INFINITY) continue;
        const float f = __expf(r[0] - gm);
        den += r[1] * f;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int64_t d = lane + 64 * j;
            if (d < D) num[j] += r[2 + d] * f;
        }
    }
    auto visible = [&](int64_t pos) { return pos >= 0 && pos < a.n_packed && pos <= last && pos >= first; };
    if (gm != -INFINITY) {
        for (int64_t j = 0; j < a.sink_cap; ++j) {
            const int64_t t = a.sink_pos[b * a.sink_cap + j];
            if (!visible(t)) continue;
            float dot = 0.f;
#pragma unroll
            for (int jj = 0; jj < 4; ++jj) {
                const int64_t d = lane + 64 * jj;
                if (d >= D) continue;
                const uint32_t kw = kp[(bh * a.cap_tokens + t) * W + d / per];
                const float kc = (float)((kw >> ((d % per) * bits)) & mask);
                const int64_t kmi = (bh * GKcap + t / g) * D + d;
                dot += qv[jj] * __fadd_rn(__fmul_rn(kc, ld_tag(a.k_scale, a.meta_dtype, kmi)), ld_tag(a.k_zero, a.meta_dtype, kmi));
            }
            den -= __expf(wave_sum(dot) * a.scale - gm);
        }
        if (den < 0.f) den = 0.f;
    }
    for (int64_t j = 0; j < a.sink_cap; ++j) {
        const int64_t t = a.sink_pos[b * a.sink_cap + j];
        if (!visible(t)) continue;
        float kh[4], vh[4], dot = 0.f;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) {
            const int64_t d = lane + 64 * jj;
            kh[jj] = vh[jj] = 0.f;
            if (d >= D) continue;
            const int64_t si = (bh * a.sink_cap + j) * D + d;
            kh[jj] = ld_tag(a.sink_k, a.sink_dtype, si);
            vh[jj] = ld_tag(a.sink_v, a.sink_dtype, si);
            dot += qv[jj] * kh[jj];
        }
        const float sc = wave_sum(dot) * a.scale;
        const float mn = fmaxf(gm, sc);
        const float f = gm == -INFINITY ? 0.f : __expf(gm - mn), w = __expf(sc - mn);
        den = den * f + w;
#pragma unroll
        for (int jj = 0; jj < 4; ++jj) num[jj] = num[jj] * f + w * vh[jj];
        gm = mn;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int64_t d = lane + 64 * j;
        if (d < D) st_tag(a.out, a.out_dtype, row * D + d, den > 0.f ? num[j] / den : 0.f);
    }
}

void launch_sink_patch(const vq_attend_args &a, int nparts) {
    const int64_t rows = a.B * a.Hq * a.Sq;
    hipLaunchKernelGGL(attend_sink_patch_kernel, dim3((unsigned)cdiv(rows, 4)), dim3(256), 0, (hipStream_t)a.stream, a, nparts,
                       (const float *)a.workspace);
}

static void launch_merge(const float *ws, int64_t rows, int nparts, int64_t D, void *out, int out_dtype, hipStream_t st) {
    const bool pairs = nparts <= 4 && D % 2 == 0 && ((uintptr_t)ws & 7u) == 0;
    int64_t g = cdiv(pairs ? rows * D / 2 : rows * D, 256);
    if (g > (1 << 20)) g = 1 << 20;
    if (g < 1) g = 1;
    if (pairs) hipLaunchKernelGGL(attend_merge4_kernel, dim3((unsigned)g), dim3(256), 0, st, ws, rows, nparts, D, out, out_dtype);
    else hipLaunchKernelGGL(attend_merge_kernel, dim3((unsigned)g), dim3(256), 0, st, ws, rows, nparts, D, out, out_dtype);
}

int launch_attend_generic(const vq_attend_args &a, int nsplit, int64_t split_len) {
    hipStream_t st = (hipStream_t)a.stream;
    const int64_t rows = a.B * a.Hq * a.Sq;
    const int64_t waves = rows * nsplit;
    hipLaunchKernelGGL(attend_generic_kernel, dim3((unsigned)cdiv(waves, 4)), dim3(256), 0, st, a, nsplit, split_len,
                       (float *)a.workspace);
    return VQ_OK;
}

void launch_merge_rows(const float *ws, int64_t rows, int nparts, int64_t D, void *out, int out_dtype, hipStream_t st) {
    launch_merge(ws, rows, nparts, D, out, out_dtype, st);
}

int launch_attend_merge(const vq_attend_args &a, int nparts) {
    launch_merge((const float *)a.workspace, a.B * a.Hq * a.Sq, nparts, a.D, a.out, a.out_dtype, (hipStream_t)a.stream);
    return VQ_OK;
}

}  // namespace vq
