// MFMA decode attention over a packed KIVI cache (placeholder until the kernel lands).
#include "attend.hpp"

namespace vq {
bool mfma_decode_supported(const vq_attend_args &) { return false; }
int launch_attend_mfma_decode(const vq_attend_args &, int, int64_t) {
    return fail(VQ_ERR_UNSUPPORTED, "MFMA decode path not built");
}
}  // namespace vq
