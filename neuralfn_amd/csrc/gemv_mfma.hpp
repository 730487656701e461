// Matrix-core decode / small-batch GEMV (gemv_mfma.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// Workspace record of one (token, 256-value block): high plane [256], low plane
// [256], 8 float scales, 8 float sums.
constexpr int kActivationRecordBytes = 576;

// True when a projection of this encoding and width has a matrix-core kernel.
bool gemv_mfma_supports(std::uint32_t encoding, std::int64_t input_dim);

// rows == 1: one launch, activations quantized inside it.  rows 2..16: one
// quantizer launch into `workspace`, then the GEMV.
void launch_gemv_mfma(ProjectionSet set, const float* first, const float* second, int prologue,
                      std::int64_t rows, void* workspace, hipStream_t stream);

}  // namespace nfn
