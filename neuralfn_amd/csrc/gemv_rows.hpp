// Verifier rows on the int8 matrix cores in the one-row arithmetic (gemv_rows.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// True when a projection of this encoding and width has the kernel.
bool gemv_rows_supports(std::uint32_t encoding, std::int64_t input_dim);

// Writes the activation records of `rows` rows (the prologue applied) to `records`:
// rows * input_dim / 256 records of 576 bytes, token by token.
void launch_quantize_records(const float* first, const float* second, int prologue,
                             std::int64_t rows, std::int64_t input_dim, std::uint8_t* records,
                             hipStream_t stream);

// rows 2..16 of the set's Q4_K / Q5_K projections from the activation records.
void launch_gemv_rows(const ProjectionSet& set, const std::uint8_t* records, std::int64_t rows,
                      hipStream_t stream);

}  // namespace nfn
