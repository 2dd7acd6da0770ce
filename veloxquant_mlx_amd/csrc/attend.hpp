// Declarations shared by the attention translation units.
#pragma once
#include "common.hpp"

namespace vq {

// a batch whose sequences differ in length: the block's copy of the arguments takes the lengths
// of its own sequence
__device__ __forceinline__ void take_sequence_lengths(vq_attend_args &a, int64_t b) {
    if (a.packed_lens != nullptr) {
        a.n_packed = a.packed_lens[b];
        a.n_tail = a.tail_lens[b];
    }
}

// first slot a query at position `pos` (of Sq, aligned to the end of n_total slots) sees under a
// sliding window; 0 without one
__device__ __host__ __forceinline__ int64_t window_first(const vq_attend_args &a, int64_t n_total, int64_t pos) {
    const int64_t lo = n_total - a.Sq + pos + 1 - a.sliding_window;
    return a.sliding_window > 0 && lo > 0 ? lo : 0;
}

struct AttendPlan {
    int path;           // 0 generic waves, 1 MFMA decode (row tiles of <= 8), 2 MFMA prefill (LDS-staged, 64-row blocks),
                        // 3 vector-unit rows kernel (any head_dim / bit width, four query rows a block)
    int nsplit;         // splits along the tokens the main kernel covers
    int nparts;         // partials per query row handed to the merge kernel
    int64_t split_len;  // tokens per split (multiple of 64)
    // MFMA path: the block of split 0 also runs the fp16 tail and takes this many fewer
    // packed tokens (multiple of 64); split s covers packed tokens
    // [max(0, s*split_len - tail_equiv), min(n_packed, (s+1)*split_len - tail_equiv))
    int64_t tail_equiv;
    // MFMA path: a block works on the GQA group of one kv head at pq consecutive query
    // positions (eight heads of a group of more than eight, pq = 1); tiles such blocks per (batch, kv head)
    int pq, tiles;
    // MFMA decode path: deal token chunks to the waves round robin instead of on demand, so that
    // results are identical from run to run
    int fixed_order;
    // rows kernel over the tail only: first partial it writes (-1: the whole context, partials 0 .. nsplit - 1)
    int part0 = -1;
};

// One output element from the split partials of its query row: p points at nparts records
// of `stride` floats (max in natural-log units, sum, accumulator[D]).  CH records are
// fetched at a time with independent loads (a round costs one memory latency, so callers with
// many records pick a large CH); DEVICE_SCOPE reads partials that other blocks
// of the same launch wrote.
template <bool DEVICE_SCOPE> __device__ __forceinline__ float ld_part(const float *p) {
    if (DEVICE_SCOPE) return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return *p;
}
template <bool DEVICE_SCOPE, int CH = 8>
__device__ __forceinline__ float merge_partials(const float *p, int nparts, int64_t stride, int64_t d) {
    float gm = -INFINITY, num = 0.f, den = 0.f;
    for (int s0 = 0; s0 < nparts; s0 += CH) {
        float m[CH], l[CH], o[CH];
#pragma unroll
        for (int j = 0; j < CH; ++j) {
            const float *q = p + (int64_t)(s0 + j < nparts ? s0 + j : s0) * stride;
            m[j] = ld_part<DEVICE_SCOPE>(q);
            l[j] = ld_part<DEVICE_SCOPE>(q + 1);
            o[j] = ld_part<DEVICE_SCOPE>(q + 2 + d);
        }
        // every load of the round is issued before the first use: left to itself the scheduler
        // weaves the maxima between the loads and waits for each record in turn
        __builtin_amdgcn_sched_barrier(0);
        float cm = gm;
#pragma unroll
        for (int j = 0; j < CH; ++j)
            if (s0 + j < nparts) cm = fmaxf(cm, m[j]);
        if (cm == -INFINITY) continue;   // nothing visible so far
        const float f0 = __expf(gm - cm);   // 0 on the first chunk
        num *= f0;
        den *= f0;
#pragma unroll
        for (int j = 0; j < CH; ++j)
            if (s0 + j < nparts && m[j] != -INFINITY) {
                const float f = __expf(m[j] - cm);
                den += l[j] * f;
                num += o[j] * f;
            }
        gm = cm;
    }
    return den > 0.f ? num / den : 0.f;
}
// the round size by the number of records: one round of loads when they fit (every caller goes
// through here, so the in-kernel merge and the merge kernel add in the same order)
template <bool DEVICE_SCOPE>
__device__ __forceinline__ float merge_records(const float *p, int nparts, int64_t stride, int64_t d) {
    return nparts <= 8 ? merge_partials<DEVICE_SCOPE, 8>(p, nparts, stride, d)
           : nparts <= 16 ? merge_partials<DEVICE_SCOPE, 16>(p, nparts, stride, d)
                          : merge_partials<DEVICE_SCOPE, 36>(p, nparts, stride, d);
}


// Decides kernel and split count from shapes only, so that the workspace query
// and the launch agree.
AttendPlan plan_attend(const vq_attend_args &a);

int launch_attend_generic(const vq_attend_args &a, int nsplit, int64_t split_len);
// vector-unit kernel with the kv head's bytes shared by its query heads (attend_rows.hip): whether it takes the
// shapes, its row tiling (positions per tile, tiles per (sequence, kv head)), the launch
bool rows_kernel_supported(const vq_attend_args &a);
void rows_tiling(const vq_attend_args &a, int &pq, int &tiles);
int launch_attend_rows(const vq_attend_args &a, const AttendPlan &p);
// the same kernel over the tail tokens only, into partial `part0` of `nparts` per query row
int launch_attend_rows_tail(const vq_attend_args &a, int part0, int nparts);
int launch_attend_merge(const vq_attend_args &a, int nparts);
// protected rows (vq_attend_args.sink_k): rewrites every output row from the partials in the
// workspace, with the stand-ins' weights taken out and the exact rows put in
void launch_sink_patch(const vq_attend_args &a, int nparts);
// merges partials [rows][nparts][D + 2] of (max, sum, accumulator) into out [rows][D]
void launch_merge_rows(const float *ws, int64_t rows, int nparts, int64_t D, void *out, int out_dtype, hipStream_t st);

// MFMA decode path (attend_mfma.hip)
bool mfma_decode_supported(const vq_attend_args &a);
int mfma_row_tiles(const vq_attend_args &a);
int mfma_positions_per_tile(const vq_attend_args &a);

// MFMA prefill path (attend_prefill.hip): packed prefix into partial slot 0, tail into slot 1
bool mfma_prefill_supported(const vq_attend_args &a);
int mfma_prefill_block_rows(const vq_attend_args &a);   // 64, or 256 when a kv head has that many query rows
// returns true when the kernel wrote the output itself (one run per row: nothing to merge)
bool launch_attend_mfma_prefill(const vq_attend_args &a, const AttendPlan &p);
// that case, from the shapes alone: such a launch writes no partials and needs no workspace
bool mfma_prefill_direct_output(const vq_attend_args &a, int nparts);
// whether a launch of the 256-row blocks takes its units from a.kv_tiles
bool mfma_prefill_uses_tiles(const vq_attend_args &a);
// writes tiles [first_unit, first_unit + n_units) of every (sequence, kv head); VQ_OK or an error code
int launch_prefill_tiles(const vq_attend_args &a, int64_t first_unit, int64_t n_units);
// returns true when the kernel also merged the partials (sync counters were given)
bool launch_attend_mfma_decode(const vq_attend_args &a, const AttendPlan &p);

}  // namespace vq
