// Q8_0 decode GEMV on the vector ALUs (gemv_q8.hip).
#pragma once

#include "common.hpp"

namespace nfn {

bool gemv_q8_supports(std::uint32_t encoding, std::int64_t input_dim);

// The Q8_0 projections of `set`, rows 1..16; activations are quantized inside
// the launch, no workspace.
void launch_gemv_q8(const ProjectionSet& set, const float* first, const float* second,
                    int prologue, std::int64_t rows, hipStream_t stream);

}  // namespace nfn
