// Packed-prefix MFMA decode kernels: scale / zero stored as fp16, blocks of five to eight query rows.
#include "attend_mfma_packed.hpp"

namespace vq {

void launch_mfma_packed_f16meta_r8(const vq_attend_args &a, const AttendPlan &p, float *ws, hipStream_t st) {
    launch_mfma_packed<f16, 8>(a, p, ws, st);
}

}  // namespace vq
