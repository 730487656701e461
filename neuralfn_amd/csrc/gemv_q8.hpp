// Q8_0 decode GEMV on the vector ALUs (gemv_q8.hip).
#pragma once

#include "common.hpp"

namespace nfn {

bool gemv_q8_supports(std::uint32_t encoding, std::int64_t input_dim);

// The Q8_0 projections of `set`, rows 1..16; activations are quantized inside
// the launch.  `records_out` and prologue kRecords as for launch_gemv_dot.
void launch_gemv_q8(const ProjectionSet& set, const float* first, const float* second,
                    std::uint8_t* records_out, int prologue, std::int64_t rows,
                    hipStream_t stream);

}  // namespace nfn
