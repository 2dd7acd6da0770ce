// Packed-prefix MFMA decode kernels for a head of 256 channels: scale / zero stored as float32, blocks of up to four query rows.
#include "attend_mfma_packed.hpp"

namespace vq {

void launch_mfma_packed_d256_f32meta_r4(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    launch_mfma_packed<float, 4, 2>(a, p, ws, st);
}

}  // namespace vq
