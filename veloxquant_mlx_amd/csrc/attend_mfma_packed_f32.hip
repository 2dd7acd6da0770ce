// Packed-prefix MFMA decode kernels for caches that store scale / zero as float32.
#include "attend_mfma_packed.hpp"

namespace vq {

void launch_mfma_packed_f32meta(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    launch_mfma_packed<float>(a, p, ws, st);
}

}  // namespace vq
