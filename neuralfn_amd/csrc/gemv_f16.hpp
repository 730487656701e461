// Small-batch GEMV on the fp16 matrix cores (gemv_f16.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// True when a projection of this encoding and width has this kernel.
bool gemv_f16_supports(std::uint32_t encoding, std::int64_t input_dim);

// Bytes of `workspace` a call uses: the fp16 copy of the activations and one scale per row.
std::int64_t gemv_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim);

// rows 3..16: one launch converts the activations (with the prologue applied) into
// `workspace`, then one launch per encoding present multiplies.  Prologue kHalfImage: the
// workspace already holds the converted rows and only the multiplying launches run.
void launch_gemv_f16(const ProjectionSet& set, const float* first, const float* second, int prologue,
                     std::int64_t rows, void* workspace, hipStream_t stream);

}  // namespace nfn
