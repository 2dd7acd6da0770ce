// C entry points for attention over a packed KIVI cache: validation, the split
// plan, workspace sizing and kernel dispatch.
#include "attend.hpp"

#include <atomic>
#include <mutex>

namespace vq {

static std::atomic<int> g_fixed_order{0};

// what a tail token costs the block of split 0, in packed tokens, when the plan balances the splits
constexpr int64_t TAIL_EQUIV = 4;

AttendPlan plan_attend(const vq_attend_args &a) {
    AttendPlan p;
    // bit 0: fixed chunk order; bit 1 (fixed_order == 3): the decode kernel also waits for every copy in flight
    p.fixed_order = a.fixed_order == 1 ? 1 : a.fixed_order == 3 ? 3 : a.fixed_order == 2 ? 0 : g_fixed_order.load(std::memory_order_relaxed);
    p.path = (a.num_splits >= 0 && mfma_decode_supported(a)) ? 1 : 0;
    p.tail_equiv = 0;
    p.pq = 1;
    p.tiles = 1;
    if (a.num_splits >= 0 && mfma_prefill_supported(a)) {
        // 64-row blocks; split their work until the grid holds two blocks per compute unit
        p.path = 2;
        // 64-row blocks run two to a CU, 256-row blocks one
        const int rows = mfma_prefill_block_rows(a);
        const int64_t blocks = a.B * a.Hkv * cdiv(a.Sq, rows / (a.Hq / a.Hkv));
        const int64_t work = cdiv(a.n_packed + a.n_tail, 32);
        // (as many runs as still fit the chip in one round: a few blocks more than that would run as a second round)
        int64_t ns = a.num_splits > 0 ? a.num_splits : (rows != 64 ? 256 : 512) / (blocks > 0 ? blocks : 1);
        if (ns > 8) ns = 8;
        if (ns > work) ns = work;
        if (ns < 1) ns = 1;
        p.nsplit = (int)ns;
        p.split_len = a.n_packed;
        p.nparts = p.nsplit;
        return p;
    }
    if (p.path == 0 && a.num_splits >= 0 && rows_kernel_supported(a)) {
        // four query rows of a kv head per block; splits until the grid holds four blocks per compute unit,
        // of at least 256 tokens each
        p.path = 3;
        rows_tiling(a, p.pq, p.tiles);
        const int64_t n_total = a.n_packed + a.n_tail;
        const int64_t units = a.B * a.Hkv * p.tiles;
        int64_t ns = a.num_splits > 0 ? a.num_splits : cdiv(1024, units > 0 ? units : 1);
        const int64_t most = n_total > 256 ? n_total / 256 : 1;
        if (ns > most) ns = most;
        if (ns > 512) ns = 512;
        if (ns < 1) ns = 1;
        const int64_t len = cdiv(cdiv(n_total > 0 ? n_total : 1, ns), 64) * 64;
        p.nsplit = (int)cdiv(n_total > 0 ? n_total : 1, len);
        p.split_len = len;
        p.nparts = p.nsplit;
        return p;
    }
    // tokens the kernel splits: the MFMA path hands the tail to a few waves of the block of split 0
    // and prices a tail token at TAIL_EQUIV packed tokens when it balances the splits
    int64_t n_split = a.n_packed + a.n_tail;
    if (p.path == 1) {
        p.pq = mfma_positions_per_tile(a);
        p.tiles = mfma_row_tiles(a);
        // (a head of 256 channels: the tail is a partial of the vector kernel, none of the block's work)
        p.tail_equiv = a.n_tail > 0 && a.D == 128 ? cdiv(a.n_tail * TAIL_EQUIV, 128) * 128 : 0;
        n_split = a.n_packed + p.tail_equiv;
    }
    // the MFMA kernel wants every block to start on a boundary of the largest token group (128)
    const int64_t gran = p.path == 1 ? 128 : 64;
    const int64_t max_splits = n_split > 0 ? cdiv(n_split, gran) : 1;
    // units of parallel work before splitting: a wave per query row (generic)
    // or an eight-wave block per kv head (MFMA)
    const int64_t units = p.path == 1 ? a.B * a.Hkv * p.tiles : a.B * a.Hq * a.Sq;
    const int64_t target = p.path == 1 ? 256 : 4096;   // MFMA path: one eight-wave block per CU
    int64_t ns = a.num_splits > 0 ? a.num_splits : cdiv(target, units > 0 ? units : 1);   // < 0: choose as well
    if (ns > max_splits) ns = max_splits;
    if (ns > 512) ns = 512;
    if (ns < 1) ns = 1;
    int64_t len = cdiv(cdiv(n_split > 0 ? n_split : 1, ns), gran) * gran;
    if (p.tail_equiv > len) p.tail_equiv = len;   // split 0 may end up with the tail only
    ns = cdiv(a.n_packed + p.tail_equiv > 0 ? a.n_packed + p.tail_equiv : 1, len);
    if (p.path == 0) ns = n_split > 0 ? cdiv(n_split, len) : 1;
    p.nsplit = (int)ns;
    p.split_len = len;
    // MFMA decode path: the tail is run by up to eight waves of split 0, every wave into a partial of
    // its own.  A launch with many blocks is bound by throughput: one wave takes eight units of 32
    // tokens (the other waves stream meanwhile); a launch with few is bound by latency: one unit a wave.
    p.nparts = p.nsplit;
    if (p.path == 1 && a.n_tail > 0) {
        int64_t tw = cdiv(cdiv(a.n_tail, 32), units >= 64 ? 8 : 1);
        // (a head of 256 channels: the tail launch of the vector kernel, up to four runs of at least 16 tokens)
        const int64_t tr = cdiv(a.n_tail, 16);
        p.nparts += a.D == 128 ? (int)(tw < 1 ? 1 : tw > 8 ? 8 : tw) : (int)(tr > 4 ? 4 : tr);
    }
    return p;
}

static int64_t gcd64(int64_t x, int64_t y) { while (y) { const int64_t t = x % y; x = y; y = t; } return x; }

// Sliding window: packed tokens below the window of the call's first query are seen by none of
// its queries.  Whole stretches of them (a common multiple of 128 tokens, the token group and the
// codes of a word) are dropped by moving the buffer bases forward; the strides between sequences
// and heads stay those of cap_tokens, so the kernels address the rest as before.  What is left
// below the window inside the first stretch is masked in the kernels.
static vq_attend_args skip_below_window(const vq_attend_args &a) {
    if (a.sliding_window <= 0 || a.packed_lens != nullptr || a.n_packed <= 0) return a;
    int64_t first = a.n_packed + a.n_tail - a.Sq + 1 - a.sliding_window;   // first slot of the first query
    if (first > a.n_packed) first = a.n_packed;
    const int64_t per = 32 / a.pack_bits;
    int64_t unit = 128 / gcd64(128, a.group) * a.group;
    unit = unit / gcd64(unit, per) * per;
    const int64_t skip = first > 0 ? first / unit * unit : 0;
    if (skip <= 0) return a;
    vq_attend_args b = a;
    const int64_t W = cdiv(a.D, per), GV = cdiv(a.D, a.group), es = a.meta_dtype == VQ_F16 ? 2 : 4;
    auto fwd = [](const void *p, int64_t bytes) { return (const void *)((const char *)p + bytes); };
    b.k_packed = fwd(a.k_packed, skip * W * 4);
    b.k_scale = fwd(a.k_scale, skip / a.group * a.D * es);
    b.k_zero = fwd(a.k_zero, skip / a.group * a.D * es);
    if (a.v_layout == VQ_V_TOKEN_PACKED) {
        b.v_packed = fwd(a.v_packed, skip / per * a.D * 4);
        b.v_scale = fwd(a.v_scale, skip * es);
        b.v_zero = fwd(a.v_zero, skip * es);
    } else {
        b.v_packed = fwd(a.v_packed, skip * W * 4);
        b.v_scale = fwd(a.v_scale, skip * GV * es);
        b.v_zero = fwd(a.v_zero, skip * GV * es);
    }
    b.n_packed = a.n_packed - skip;
    if (a.kv_tiles != nullptr) b.kv_tiles = fwd(a.kv_tiles, skip / 32 * VQ_PREFILL_TILE_BYTES);   // tile_cap stays: it is the stride
    return b;
}

static int validate(const vq_attend_args *a, const char *fn) {
    VQ_REQUIRE(a != nullptr, VQ_ERR_INVALID, "%s: null argument block", fn);
    VQ_REQUIRE(a->B >= 1 && a->Hq >= 1 && a->Hkv >= 1 && a->Sq >= 1 && a->D >= 1, VQ_ERR_INVALID,
               "%s: q must be 4D with positive sizes, got B=%lld Hq=%lld Sq=%lld D=%lld", fn, (long long)a->B,
               (long long)a->Hq, (long long)a->Sq, (long long)a->D);
    VQ_REQUIRE(a->D <= 256, VQ_ERR_INVALID, "%s: D=%lld must be <= 256", fn, (long long)a->D);
    VQ_REQUIRE(a->Hq % a->Hkv == 0, VQ_ERR_INVALID,
               "%s: H_q=%lld must be a multiple of H_kv=%lld for GQA head-packing", fn, (long long)a->Hq,
               (long long)a->Hkv);
    VQ_REQUIRE(a->n_packed >= 0 && a->n_tail >= 0, VQ_ERR_INVALID, "%s: negative token count", fn);
    VQ_REQUIRE(a->n_packed + a->n_tail >= 1, VQ_ERR_INVALID, "%s: no key/value slots to attend to", fn);
    VQ_REQUIRE(a->fixed_order >= 0 && a->fixed_order <= 3, VQ_ERR_INVALID, "%s: fixed_order must be 0, 1, 2 or 3", fn);
    VQ_REQUIRE(a->sliding_window >= 0, VQ_ERR_INVALID, "%s: negative sliding window", fn);
    if (a->kv_tiles != nullptr)
        VQ_REQUIRE(((uintptr_t)a->kv_tiles & 15u) == 0 && a->tile_cap * 32 >= a->n_packed + a->n_tail, VQ_ERR_INVALID,
                   "%s: kv_tiles must be 16-byte aligned with room for all %lld slots (tile_cap %lld)", fn,
                   (long long)(a->n_packed + a->n_tail), (long long)a->tile_cap);
    if (a->sink_k != nullptr) {
        VQ_REQUIRE(a->sink_v != nullptr && a->sink_pos != nullptr && a->sink_cap >= 1, VQ_ERR_INVALID,
                   "%s: sink_k needs sink_v, sink_pos and sink_cap >= 1", fn);
        VQ_REQUIRE(is_float_tag(a->sink_dtype), VQ_ERR_INVALID, "%s: unsupported sink dtype", fn);
        VQ_REQUIRE(a->n_packed > 0, VQ_ERR_INVALID, "%s: protected rows stand for positions of the packed prefix", fn);
    }
    VQ_REQUIRE(a->Sq <= a->n_packed + a->n_tail || !a->causal, VQ_ERR_INVALID,
               "%s: S_q=%lld exceeds S_kv=%lld; queries align to the tail of the KV cache", fn, (long long)a->Sq,
               (long long)(a->n_packed + a->n_tail));
    VQ_REQUIRE(is_float_tag(a->q_dtype) && is_float_tag(a->out_dtype), VQ_ERR_INVALID, "%s: unsupported q/out dtype", fn);
    if (a->n_packed > 0) {
        VQ_REQUIRE(a->pack_bits >= 1 && a->pack_bits <= 8, VQ_ERR_INVALID, "%s: pack_bits must be in 1..8", fn);
        VQ_REQUIRE(a->group >= 1, VQ_ERR_INVALID, "%s: group_size must be >= 1", fn);
        VQ_REQUIRE(a->meta_dtype == VQ_F32 || a->meta_dtype == VQ_F16, VQ_ERR_INVALID, "%s: meta dtype must be f32/f16", fn);
        VQ_REQUIRE(a->v_layout == VQ_V_CHANNEL_PACKED || a->v_layout == VQ_V_TOKEN_PACKED, VQ_ERR_INVALID, "%s: bad v_layout", fn);
        VQ_REQUIRE(a->cap_tokens >= a->n_packed, VQ_ERR_INVALID, "%s: n_packed exceeds cap_tokens", fn);
        if (a->v_layout == VQ_V_TOKEN_PACKED)
            VQ_REQUIRE(a->cap_tokens % (32 / a->pack_bits) == 0, VQ_ERR_INVALID, "%s: cap_tokens not word aligned", fn);
    }
    if (a->n_tail > 0) {
        VQ_REQUIRE(is_float_tag(a->tail_dtype), VQ_ERR_INVALID, "%s: unsupported tail dtype", fn);
        VQ_REQUIRE(a->tail_cap >= a->n_tail, VQ_ERR_INVALID, "%s: n_tail exceeds tail_cap", fn);
    }
    return VQ_OK;
}

// Several query positions of a GQA group of 3, 5, 6 or 7 heads, fewer than 256 rows a kv head: the decode kernel's
// tiles and the 64-row prefill blocks hold groups of 1, 2, 4 and 8 (or more) heads.  Such a call runs as the next of those sizes -- every kv head's group filled up with
// heads of zeros, whose rows are computed and dropped -- when that takes a matrix-unit path and the call as given
// does not.  A prefill-sized call with more than eight heads a group runs eight of them at a time through the prefill
// blocks (one pass per eight heads, the last filled up) instead of one position a tile through the decode kernel.
// Returns the group size of the calls that run, 0 when the call runs as it is.
static int64_t padded_group(const vq_attend_args &a) {
    if (a.Sq < 2 || a.Hkv < 1 || a.Hq % a.Hkv != 0 || a.k_new != nullptr || a.num_splits < 0) return 0;
    const int64_t R = a.Hq / a.Hkv;
    if (R == 1 || R == 2 || R == 4 || R == 8) return 0;
    if ((a.Sq * a.D * (a.q_dtype == VQ_F32 ? 4 : 2)) % 16 != 0 || (a.Sq * a.D * (a.out_dtype == VQ_F32 ? 4 : 2)) % 16 != 0) return 0;
    if ((((uintptr_t)a.q | (uintptr_t)a.out) & 15u) != 0) return 0;
    const int path = plan_attend(a).path;
    vq_attend_args b = a;
    b.q = nullptr;   // stands for a 256-byte aligned buffer
    if (R > 8) {
        if (a.Sq < 16 || path == 2) return 0;
        b.Hq = a.Hkv * 8;
        return plan_attend(b).path == 2 ? 8 : 0;
    }
    if (path == 1 || path == 2) return 0;
    b.Hq = a.Hkv * (R == 3 ? 4 : 8);
    const int padded = plan_attend(b).path;
    return padded == 1 || padded == 2 ? b.Hq / a.Hkv : 0;
}

static size_t round256(size_t n) { return (n + 255) / 256 * 256; }

// rows of `row16` 16-byte pieces, in groups of R_src (src) and R_dst (dst) rows: rows [dst_off, dst_off + n_write) of
// every dst group become rows [src_off, src_off + n_write) of the same src group, zeros from the n_valid-th on
__global__ void regroup_rows_kernel(const uint4 *__restrict__ src, uint4 *__restrict__ dst, int64_t groups, int R_src,
                                    int src_off, int R_dst, int dst_off, int n_write, int n_valid, int64_t row16) {
    const int64_t n = groups * n_write * row16;
    for (int64_t e = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (int64_t)gridDim.x * blockDim.x) {
        const int64_t c = e % row16, r = (e / row16) % n_write, g = e / (row16 * n_write);
        dst[(g * R_dst + dst_off + r) * row16 + c] =
            r < n_valid ? src[(g * R_src + src_off + r) * row16 + c] : make_uint4(0u, 0u, 0u, 0u);
    }
}

static void launch_regroup(const void *src, void *dst, int64_t groups, int64_t R_src, int64_t src_off, int64_t R_dst,
                           int64_t dst_off, int64_t n_write, int64_t n_valid, int64_t row_bytes, hipStream_t st) {
    const int64_t n = groups * n_write * (row_bytes / 16);
    const int64_t blocks = cdiv(n, 256);
    hipLaunchKernelGGL(regroup_rows_kernel, dim3((unsigned)(blocks < 65535 * 16 ? blocks : 65535 * 16)), dim3(256), 0, st,
                       (const uint4 *)src, (uint4 *)dst, groups, (int)R_src, (int)src_off, (int)R_dst, (int)dst_off,
                       (int)n_write, (int)n_valid, row_bytes / 16);
}

}  // namespace vq

using namespace vq;

extern "C" int vq_kivi_attend_fixed_order(int enable) {
    return g_fixed_order.exchange(enable ? 1 : 0, std::memory_order_relaxed);
}

extern "C" size_t vq_kivi_attend_workspace(const vq_attend_args *a) {
    // the plan divides by the shapes: arguments that would not pass vq_kivi_attend need no workspace
    if (!a || a->B < 1 || a->Hq < 1 || a->Hkv < 1 || a->Sq < 1 || a->D < 1 || a->Hq % a->Hkv != 0 ||
        a->n_packed < 0 || a->n_tail < 0 || (a->n_packed > 0 && (a->pack_bits < 1 || a->pack_bits > 8 || a->group < 1)))
        return 0;
    const vq_attend_args w = skip_below_window(*a);
    if (const int64_t Rp = padded_group(w)) {
        // the padded call's own workspace, then its queries and its outputs
        vq_attend_args b = *a;
        b.Hq = a->Hkv * Rp;
        b.q = nullptr;
        const size_t rows = (size_t)(b.B * b.Hq * b.Sq) * (size_t)b.D;
        return round256(vq_kivi_attend_workspace(&b)) + round256(rows * (a->q_dtype == VQ_F32 ? 4 : 2)) +
               round256(rows * (a->out_dtype == VQ_F32 ? 4 : 2));
    }
    AttendPlan p = plan_attend(w);
    if (p.path == 2 && mfma_prefill_direct_output(w, p.nparts)) return 0;   // the kernel writes `out` itself
    return (size_t)(a->B * a->Hq * a->Sq) * (size_t)p.nparts * (size_t)(a->D + 2) * sizeof(float);
}

extern "C" int vq_kivi_prefill_tiles(const vq_attend_args *a, int64_t first_unit, int64_t n_units) {
    const char *fn = "vq_kivi_prefill_tiles";
    VQ_REQUIRE(a != nullptr, VQ_ERR_INVALID, "%s: null argument block", fn);
    VQ_REQUIRE(a->B >= 1 && a->Hkv >= 1 && a->n_packed >= 0 && a->n_tail >= 0, VQ_ERR_INVALID, "%s: bad sizes", fn);
    VQ_REQUIRE(a->kv_tiles != nullptr && ((uintptr_t)a->kv_tiles & 15u) == 0, VQ_ERR_INVALID, "%s: kv_tiles must be given, 16-byte aligned", fn);
    const int64_t units = cdiv(a->n_packed + a->n_tail, 32);
    VQ_REQUIRE(first_unit >= 0 && n_units >= 0 && first_unit + n_units <= units && units <= a->tile_cap, VQ_ERR_INVALID,
               "%s: units [%lld, %lld) do not lie inside the %lld units of the slots (tile_cap %lld)", fn, (long long)first_unit,
               (long long)(first_unit + n_units), (long long)units, (long long)a->tile_cap);
    if (a->n_packed > 0)
        VQ_REQUIRE(a->k_packed && a->v_packed && a->k_scale && a->k_zero && a->v_scale && a->v_zero, VQ_ERR_INVALID,
                   "%s: null packed-cache pointer", fn);
    if (a->n_tail > 0) VQ_REQUIRE(a->k_tail && a->v_tail, VQ_ERR_INVALID, "%s: null tail pointer", fn);
    if (n_units == 0) return VQ_OK;
    return launch_prefill_tiles(*a, first_unit, n_units);
}

extern "C" int vq_kivi_attend_plan(const vq_attend_args *a, int *path, int *nparts) {
    int rc = validate(a, "vq_kivi_attend_plan");
    if (rc != VQ_OK) return rc;
    vq_attend_args w = skip_below_window(*a);
    if (const int64_t Rp = padded_group(w)) {   // the plan of the call that runs
        w.Hq = w.Hkv * Rp;
        w.q = nullptr;
    }
    AttendPlan p = plan_attend(w);
    if (path) *path = p.path;
    if (nparts) *nparts = p.nparts;
    return VQ_OK;
}

extern "C" int vq_kivi_attend(const vq_attend_args *a_in) {
    const char *fn = "vq_kivi_attend";
    int rc = validate(a_in, fn);
    if (rc != VQ_OK) return rc;
    const vq_attend_args windowed = skip_below_window(*a_in);
    const vq_attend_args *a = &windowed;
    VQ_REQUIRE(a->q && a->out, VQ_ERR_INVALID, "%s: null q/out", fn);
    if (a->n_packed > 0)
        VQ_REQUIRE(a->k_packed && a->v_packed && a->k_scale && a->k_zero && a->v_scale && a->v_zero, VQ_ERR_INVALID,
                   "%s: null packed-cache pointer", fn);
    if (a->n_tail > 0) VQ_REQUIRE(a->k_tail && a->v_tail, VQ_ERR_INVALID, "%s: null tail pointer", fn);
    VQ_REQUIRE((a->packed_lens == nullptr) == (a->tail_lens == nullptr), VQ_ERR_INVALID,
               "%s: packed_lens and tail_lens go together", fn);
    VQ_REQUIRE((a->k_new == nullptr) == (a->v_new == nullptr), VQ_ERR_INVALID, "%s: k_new and v_new go together", fn);
    if (a->k_new != nullptr) {
        VQ_REQUIRE(a->n_tail >= 1, VQ_ERR_INVALID, "%s: k_new / v_new fill the last tail row, so n_tail must be >= 1", fn);
        VQ_REQUIRE((((uintptr_t)a->k_new | (uintptr_t)a->v_new) & 15u) == 0, VQ_ERR_UNSUPPORTED,
                   "%s: k_new / v_new must be 16-byte aligned", fn);
    }
    if (const int64_t Rp = padded_group(*a)) {
        const size_t need = vq_kivi_attend_workspace(a_in);
        VQ_REQUIRE(a_in->workspace != nullptr && a_in->workspace_bytes >= need, VQ_ERR_WORKSPACE,
                   "%s: workspace of %zu bytes required, %zu given", fn, need, a_in->workspace_bytes);
        VQ_REQUIRE(((uintptr_t)a_in->workspace & 255u) == 0, VQ_ERR_INVALID, "%s: the workspace must be 256-byte aligned", fn);
        const int64_t R = a_in->Hq / a_in->Hkv;
        vq_attend_args b = *a_in;   // the arguments as given: the inner call cuts the window itself
        b.Hq = a_in->Hkv * Rp;
        b.q = nullptr;
        const size_t inner = round256(vq_kivi_attend_workspace(&b));
        const size_t rows = (size_t)(b.B * b.Hq * b.Sq) * (size_t)b.D;
        char *base = static_cast<char *>(a_in->workspace);
        void *q_wide = base + inner;
        void *out_wide = base + inner + round256(rows * (a_in->q_dtype == VQ_F32 ? 4 : 2));
        b.q = q_wide;
        b.out = out_wide;
        b.workspace_bytes = inner;
        hipStream_t st = (hipStream_t)a_in->stream;
        const int64_t groups = a_in->B * a_in->Hkv;
        const int64_t q_row = a_in->Sq * a_in->D * (a_in->q_dtype == VQ_F32 ? 4 : 2);
        const int64_t out_row = a_in->Sq * a_in->D * (a_in->out_dtype == VQ_F32 ? 4 : 2);
        for (int64_t first = 0; first < R; first += Rp) {   // one pass for groups of up to eight heads
            const int64_t n_valid = R - first < Rp ? R - first : Rp;
            launch_regroup(a_in->q, q_wide, groups, R, first, Rp, 0, Rp, n_valid, q_row, st);
            VQ_HIP_CHECK_LAUNCH(fn);
            rc = vq_kivi_attend(&b);
            if (rc != VQ_OK) return rc;
            launch_regroup(out_wide, a_in->out, groups, Rp, 0, R, first, n_valid, n_valid, out_row, st);
            VQ_HIP_CHECK_LAUNCH(fn);
            b.tiles_stale_from = b.tile_cap;   // the first pass has brought the tiles up to date
        }
        return VQ_OK;
    }
    AttendPlan p = plan_attend(*a);
    if (a->k_new != nullptr)
        VQ_REQUIRE(p.path == 1 && a->Sq == 1, VQ_ERR_UNSUPPORTED,
                   "%s: k_new / v_new need the single-query MFMA decode path; append with vq_kv_tail_append first", fn);
    size_t need = vq_kivi_attend_workspace(a);
    VQ_REQUIRE(need == 0 || (a->workspace != nullptr && a->workspace_bytes >= need), VQ_ERR_WORKSPACE,
               "%s: workspace of %zu bytes required, %zu given", fn, need, a->workspace_bytes);
    // protected rows: the patch pass reads the partials and the original (unshifted) packed store
    auto finish = [&]() -> int {
        if (a_in->sink_k == nullptr) return VQ_OK;
        vq_attend_args full = *a_in;
        full.workspace = a->workspace;
        launch_sink_patch(full, p.nparts);
        VQ_HIP_CHECK_LAUNCH(fn);
        return VQ_OK;
    };
    if (p.path == 1) {
        if (a->D != 128 && a->n_tail > 0) {   // the tail as partial p.nsplit of every row, from the vector kernel
            rc = launch_attend_rows_tail(*a, p.nsplit, p.nparts);
            if (rc != VQ_OK) return rc;
            VQ_HIP_CHECK_LAUNCH(fn);
        }
        const bool merged = launch_attend_mfma_decode(*a, p);
        VQ_HIP_CHECK_LAUNCH(fn);
        if (merged) return finish();
    } else if (p.path == 2) {
        if (mfma_prefill_uses_tiles(*a)) {
            // bring the tiles up to date first (whole-sequence unit numbers: the arguments as given, not the windowed ones)
            const int64_t units = cdiv(a_in->n_packed + a_in->n_tail, 32);
            const int64_t from = a_in->tiles_stale_from < 0 ? 0 : a_in->tiles_stale_from;
            if (from < units) {
                rc = launch_prefill_tiles(*a_in, from, units - from);
                if (rc != VQ_OK) return rc;
            }
        }
        const bool written = launch_attend_mfma_prefill(*a, p);
        VQ_HIP_CHECK_LAUNCH(fn);
        if (written) return VQ_OK;
    } else if (p.path == 3) {
        rc = launch_attend_rows(*a, p);
        if (rc != VQ_OK) return rc;
        VQ_HIP_CHECK_LAUNCH(fn);
    } else {
        rc = launch_attend_generic(*a, p.nsplit, p.split_len);
        if (rc != VQ_OK) return rc;
        VQ_HIP_CHECK_LAUNCH(fn);
    }
    if (a_in->sink_k != nullptr) return finish();   // the patch pass does the merge as well
    rc = launch_attend_merge(*a, p.nparts);
    VQ_HIP_CHECK_LAUNCH(fn);
    return rc;
}

// ---------------------------------------------------------------------------
// vq_kivi_attend for callers that cannot allocate: the split partials and the sync counters
// live in a file-scope device array instead of a caller-provided workspace.
// ---------------------------------------------------------------------------
namespace {
constexpr size_t STATIC_WS_BYTES = (size_t)8 << 20;   // split partials
constexpr size_t STATIC_COUNTERS = 16384;             // int32 sync counters, one per (sequence, kv head, row tile)
// Every GPU the library runs on holds its own copy of this array until the process ends.  In host
// code the array's name is only a stand-in: the address kernels may use comes from
// hipGetSymbolAddress, per device.
static __device__ __align__(256) unsigned char scratch[STATIC_WS_BYTES + STATIC_COUNTERS * sizeof(int32_t)];
std::mutex g_scratch_mutex;
unsigned char *g_scratch_ptr[64] = {};

// a fill kernel, not hipMemsetAsync: the call may sit inside a stream capture
__global__ void zero_counters_kernel(int32_t *c, int n) {
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += gridDim.x * blockDim.x) c[i] = 0;
}
}  // namespace

extern "C" int vq_kivi_attend_static(const vq_attend_args *a) {
    const char *fn = "vq_kivi_attend_static";
    int rc = validate(a, fn);
    if (rc != VQ_OK) return rc;
    const size_t need = vq_kivi_attend_workspace(a);
    VQ_REQUIRE(need <= STATIC_WS_BYTES, VQ_ERR_WORKSPACE,
               "%s: these shapes need %zu bytes of split partials, the built-in scratch holds %zu; use vq_kivi_attend "
               "with a workspace of its own", fn, need, STATIC_WS_BYTES);
    vq_attend_args w = skip_below_window(*a);
    if (const int64_t Rp = padded_group(w)) {   // the call that runs: its GQA groups filled up
        w.Hq = w.Hkv * Rp;
        w.q = nullptr;
    }
    const AttendPlan p = plan_attend(w);
    VQ_REQUIRE((size_t)(a->B * a->Hkv * p.tiles) <= STATIC_COUNTERS, VQ_ERR_WORKSPACE,
               "%s: B * H_kv * row tiles = %lld exceeds the %zu built-in sync counters", fn,
               (long long)(a->B * a->Hkv * p.tiles), STATIC_COUNTERS);
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    VQ_REQUIRE(e == hipSuccess && dev >= 0 && dev < 64, VQ_ERR_HIP, "%s: no current device (%s)", fn, hipGetErrorString(e));
    unsigned char *ptr;
    {
        std::lock_guard<std::mutex> lock(g_scratch_mutex);
        if (g_scratch_ptr[dev] == nullptr) {   // once per device, with that device current
            void *sym = nullptr;
            e = hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch));
            VQ_REQUIRE(e == hipSuccess && sym != nullptr, VQ_ERR_HIP, "%s: hipGetSymbolAddress failed: %s", fn,
                       hipGetErrorString(e));
            g_scratch_ptr[dev] = static_cast<unsigned char *>(sym);
        }
        ptr = g_scratch_ptr[dev];
    }
    vq_attend_args b = *a;
    b.workspace = ptr;
    b.workspace_bytes = STATIC_WS_BYTES;
    // the counters start at zero (static storage) and every finished call leaves them at zero; a call that
    // failed half-way (a launch error) may not have, and a later call would then never reach its last ticket
    // and leave `out` unwritten: the counters are cleared again behind a failed call
    b.sync_counters = reinterpret_cast<int32_t *>(ptr + STATIC_WS_BYTES);
    rc = vq_kivi_attend(&b);
    if (rc != VQ_OK) {
        hipLaunchKernelGGL(zero_counters_kernel, dim3(16), dim3(256), 0, (hipStream_t)a->stream, b.sync_counters,
                           (int)STATIC_COUNTERS);
        (void)hipGetLastError();   // the error reported is the call's own (already recorded)
    }
    return rc;
}
