// Declarations shared by the attention translation units.
#pragma once
#include "common.hpp"

namespace vq {

struct AttendPlan {
    int path;           // 0 generic waves, 1 MFMA decode
    int nsplit;         // splits along the tokens the main kernel covers
    int nparts;         // partials per query row handed to the merge kernel
    int64_t split_len;  // tokens per split (multiple of 64)
};

// Decides kernel and split count from shapes only, so that the workspace query
// and the launch agree.
AttendPlan plan_attend(const vq_attend_args &a);

int launch_attend_generic(const vq_attend_args &a, int nsplit, int64_t split_len);
int launch_attend_merge(const vq_attend_args &a, int nparts);

// MFMA decode path (attend_mfma.hip)
bool mfma_decode_supported(const vq_attend_args &a);
int launch_attend_mfma_decode(const vq_attend_args &a, int nsplit, int64_t split_len);

}  // namespace vq
