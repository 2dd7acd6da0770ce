// Shape gate and dispatch of the MFMA decode path (the kernels live in
// attend_mfma_packed.hpp, instantiated per scale/zero dtype in attend_mfma_packed_*.hip).
#include "attend_mfma.hpp"

namespace vq {

// Query positions one block takes: rows = (heads of the GQA group) x positions, at most eight
// (a high and a remainder column each in the 16-wide tile).
int mfma_positions_per_tile(const vq_attend_args &a) {
    const int64_t R = a.Hq / a.Hkv;
    if (a.Sq == 1 || R > 8) return 1;
    return (int)(8 / R);
}

// Row tiles per (sequence, kv head): positions in steps of mfma_positions_per_tile, times the tiles of
// eight heads a GQA group of more than eight falls into.
int mfma_row_tiles(const vq_attend_args &a) {
    const int64_t R = a.Hq / a.Hkv;
    return (int)(cdiv(a.Sq, mfma_positions_per_tile(a)) * (R > 8 ? cdiv(R, 8) : 1));
}

bool mfma_decode_supported(const vq_attend_args &a) {
    if ((a.D != MF_D && a.D != 2 * MF_D) || a.n_packed <= 0) return false;
    // a head of 256 channels: packed prefix only (its tail goes through the vector kernel, one more launch), no
    // token brought along by the call
    if (a.D == 2 * MF_D && (a.k_new != nullptr || !rows_kernel_supported(a))) return false;
    if (a.Hq % a.Hkv != 0) return false;
    const int64_t R = a.Hq / a.Hkv;
    // a tile has eight rows (a high and a remainder column each): the whole group at one position, a
    // power-of-two group at 8 / R positions, or eight heads of a larger group
    if (a.Sq > 1 && !(R == 1 || R == 2 || R == 4 || R >= 8)) return false;
    if (a.B * a.Hkv * (int64_t)mfma_row_tiles(a) > 65535) return false;   // grid y, sync counters
    if (!(a.pack_bits == 2 || a.pack_bits == 4)) return false;
    if (!(a.group == 32 || a.group == 64 || a.group == 128)) return false;
    if (a.v_layout != VQ_V_TOKEN_PACKED) return false;
    if (a.n_packed % 32 != 0 || a.cap_tokens % 32 != 0 || a.cap_tokens % a.group != 0) return false;
    if (a.cap_tokens > (1 << 24)) return false;   // per-lane byte offsets are 32-bit
    if (!(a.scale > 0.f)) return false;
    if (a.D == MF_D && a.n_tail > 0 &&
        (!(a.tail_dtype == VQ_F16 || a.tail_dtype == VQ_BF16) || (((uintptr_t)a.k_tail | (uintptr_t)a.v_tail) & 15u)))
        return false;
    const uintptr_t al = (uintptr_t)a.k_packed | (uintptr_t)a.v_packed | (uintptr_t)a.k_scale | (uintptr_t)a.k_zero |
                         (uintptr_t)a.v_scale | (uintptr_t)a.v_zero;
    if (al & 15u) return false;
    return true;
}

bool launch_attend_mfma_decode(const vq_attend_args &a, const AttendPlan &p) {
    hipStream_t st = (hipStream_t)a.stream;
    float *ws = (float *)a.workspace;
    // rows a block carries: the GQA group at p.pq positions, padded to 4 or 8
    const int64_t R = a.Hq / a.Hkv;
    const bool wide = (R > 8 ? 8 : R) * p.pq > 4;
    if (a.D == 2 * MF_D) {
        if (a.meta_dtype == VQ_F16) {
            if (wide) launch_mfma_packed_d256_f16meta_r8(a, p, ws, st);
            else launch_mfma_packed_d256_f16meta_r4(a, p, ws, st);
        } else {
            if (wide) launch_mfma_packed_d256_f32meta_r8(a, p, ws, st);
            else launch_mfma_packed_d256_f32meta_r4(a, p, ws, st);
        }
    } else if (a.meta_dtype == VQ_F16) {
        if (wide) launch_mfma_packed_f16meta_r8(a, p, ws, st);
        else launch_mfma_packed_f16meta_r4(a, p, ws, st);
    } else {
        if (wide) launch_mfma_packed_f32meta_r8(a, p, ws, st);
        else launch_mfma_packed_f32meta_r4(a, p, ws, st);
    }
    return a.sync_counters != nullptr;
}

}  // namespace vq
