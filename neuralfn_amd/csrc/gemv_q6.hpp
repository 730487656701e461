// Q6_K decode GEMV on the vector ALUs and the lm_head with fused argmax (gemv_q6.hip).
#pragma once

#include "common.hpp"
#include "lm_head.hpp"

namespace nfn {

bool gemv_q6_supports(std::uint32_t encoding, std::int64_t input_dim);

// The Q6_K projections of `set`, rows 1..16; activations are quantized inside
// the launch.  `records_out` and prologue kRecords as for launch_gemv_dot.
void launch_gemv_q6(const ProjectionSet& set, const float* first, const float* second,
                    std::uint8_t* records_out, int prologue, std::int64_t rows,
                    hipStream_t stream);

// Upper bound of the workgroups of a fused lm_head launch (= candidates per
// input row) over all input widths and token counts, for sizing the workspace.
std::int64_t lm_head_q6_max_groups(std::int64_t output_dim);
void launch_lm_head_q6(const Descriptor& descriptor, const float* input, std::int64_t rows,
                       LmHeadCandidate* candidates, std::int64_t* indices, float* maxima,
                       hipStream_t stream);

}  // namespace nfn
