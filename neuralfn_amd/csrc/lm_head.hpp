// Workspace record and launchers of the fused lm_head argmax.
#pragma once

#include "common.hpp"

namespace nfn {

// Best logit of one workgroup for one input row; the workspace holds
// [rows][workgroups] of these.
struct LmHeadCandidate {
    std::int64_t index;
    float value;
    std::uint32_t pad;
};

// Keeps the larger value; equal values keep the lower index (the reference's
// first-maximum rule, neuralfn/csrc/tile_cuda/kernels.cu:1564-1602).
__device__ __forceinline__ void better(float value, std::int64_t index, float& best_value,
                                       std::int64_t& best_index) {
    if (value > best_value || (value == best_value && index < best_index)) {
        best_value = value;
        best_index = index;
    }
}

// Pass 2: one workgroup per input row reduces `candidate_count` candidates.
void launch_lm_head_final(const LmHeadCandidate* candidates, std::int64_t candidate_count,
                          std::int64_t* indices, float* maxima, std::int64_t rows,
                          hipStream_t stream);

std::int64_t lm_head_f32_blocks(std::int64_t output_dim);
void launch_lm_head_f32(const Descriptor& descriptor, const float* input, std::int64_t rows,
                        LmHeadCandidate* candidates, std::int64_t* indices, float* maxima,
                        hipStream_t stream);

}  // namespace nfn
