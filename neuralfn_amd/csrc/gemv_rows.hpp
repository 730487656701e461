// Verifier rows on the int8 matrix cores in the one-row arithmetic (gemv_rows.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// True when a projection of this encoding and width has the kernel.
bool gemv_rows_supports(std::uint32_t encoding, std::int64_t input_dim);

// Bytes of the operand image of `input_dim` columns (any row count up to 16).
std::int64_t gemv_rows_image_bytes(std::int64_t input_dim);

// Writes the activation records of `rows` rows (the prologue applied) to `records`
// (rows * input_dim / 256 records of 576 bytes, token by token) and the same codes in
// matrix-operand order to `image` (gemv_rows_image_bytes).
void launch_quantize_records(const float* first, const float* second, int prologue,
                             std::int64_t rows, std::int64_t input_dim, std::uint8_t* records,
                             std::uint8_t* image, hipStream_t stream);

// rows 2..16 of the set's Q4_K / Q5_K projections from the operand image.
void launch_gemv_rows(const ProjectionSet& set, const std::uint8_t* image, std::int64_t rows,
                      hipStream_t stream);

}  // namespace nfn
