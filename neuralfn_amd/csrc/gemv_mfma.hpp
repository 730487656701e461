// Matrix-core small-batch GEMV (gemv_mfma.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// Bytes of the workspace record of one (token, 256-value block); its layout is
// in wave_rows.hpp (kActRecord).  The small-batch workspace query is sized from it.
constexpr int kActivationRecordBytes = 576;

// True when a projection of this encoding and width has a matrix-core kernel.
bool gemv_mfma_supports(std::uint32_t encoding, std::int64_t input_dim);

// rows 2..16.  Up to eight rows the activations are quantized inside the
// kernel; beyond that (and for eight rows with a fused prologue) a quantizer
// launch fills `workspace` first.
void launch_gemv_mfma(ProjectionSet set, const float* first, const float* second, int prologue,
                      std::int64_t rows, void* workspace, hipStream_t stream);

// lm_head for 2..8 rows: the same kernel keeps one (value, row) candidate per
// 32-row tile and token in `candidates` ([rows][lm_head_mfma_tiles]); a second
// launch reduces them.  Only for encodings gemv_mfma_supports() accepts.
struct LmHeadCandidate;
std::int64_t lm_head_mfma_tiles(std::int64_t output_dim);
void launch_lm_head_mfma(const Descriptor& descriptor, const float* input, std::int64_t rows,
                         LmHeadCandidate* candidates, std::int64_t* indices, float* maxima,
                         hipStream_t stream);

}  // namespace nfn
