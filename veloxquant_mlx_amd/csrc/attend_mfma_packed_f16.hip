// Packed-prefix MFMA decode kernels for caches that store scale / zero as fp16.
#include "attend_mfma_packed.hpp"

namespace vq {

void launch_mfma_packed_f16meta(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    launch_mfma_packed<f16>(a, p, ws, st);
}

}  // namespace vq
