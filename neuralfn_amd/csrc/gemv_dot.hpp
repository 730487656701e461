// Vector-ALU decode GEMV (gemv_dot.hip): one token, or a few tokens with the
// one-token arithmetic per row.
#pragma once

#include "common.hpp"

namespace nfn {

bool gemv_dot_supports(std::uint32_t encoding, std::int64_t input_dim);

// rows 1..16; activations are quantized inside the launch, no workspace.
void launch_gemv_dot(const ProjectionSet& set, const float* first, const float* second,
                     int prologue, std::int64_t rows, hipStream_t stream);

}  // namespace nfn
