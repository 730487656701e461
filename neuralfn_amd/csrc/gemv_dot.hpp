// Vector-ALU decode GEMV (gemv_dot.hip): one token, or a few tokens with the
// one-token arithmetic per row.
#pragma once

#include "common.hpp"

namespace nfn {

bool gemv_dot_supports(std::uint32_t encoding, std::int64_t input_dim);

// rows 1..16; activations are quantized inside the launch.  `records_out`
// (may be null): where the launch also leaves its activation records
// (kActRecord bytes per token and 256 values) for a later launch with
// prologue kRecords, whose `first` is then that pointer.
void launch_gemv_dot(const ProjectionSet& set, const float* first, const float* second,
                     std::uint8_t* records_out, int prologue, std::int64_t rows,
                     hipStream_t stream);

// One token: hidden = residual + rms(input), normalized = rms(hidden) in the launch's own
// prologue (every workgroup for itself, the first also stores the three rows), then the
// projections of `set` on the normalized row.  All projections of one encoding, input_dim at
// most 8192.
struct DualNormArguments;
bool gemv_dot_normed_supports(const ProjectionSet& set);
void launch_gemv_dot_normed(const ProjectionSet& set, const float* input,
                            const DualNormArguments& norm, hipStream_t stream);

// One token through two projections of one shape and encoding (gate, up) with the SwiGLU
// activation at the row ends: output r = (up_r gate_r) sigmoid(gate_r), the value the SwiGLU
// prologue of the projection behind would compute from the two separate outputs.
// set.op[0]: gate, its `output` the result; set.op[1]: up.
bool gemv_dot_pairs_supports(std::uint32_t first_encoding, std::uint32_t second_encoding,
                             std::int64_t input_dim);
void launch_gemv_dot_pairs(const ProjectionSet& set, const float* input, hipStream_t stream);

}  // namespace nfn
