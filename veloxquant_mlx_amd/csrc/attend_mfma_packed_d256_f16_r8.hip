// Packed-prefix MFMA decode kernels for a head of 256 channels: scale / zero stored as fp16, blocks of up to eight query rows.
#include "attend_mfma_packed.hpp"

namespace vq {

void launch_mfma_packed_d256_f16meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    launch_mfma_packed<f16, 8, 2>(a, p, ws, st);
}

}  // namespace vq
