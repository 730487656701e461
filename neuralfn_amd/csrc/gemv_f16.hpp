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

// Gate and up of an FFN (set.op[0], set.op[1]: one shape, one encoding) with
// swiglu(gate, up) stored in set.op[0].output instead of the two results.  `input` null: the
// workspace already holds the converted rows (as with prologue kHalfImage).
bool gemv_f16_pairs_supports(std::uint32_t first_encoding, std::uint32_t second_encoding,
                             std::int64_t input_dim);
void launch_gemv_f16_pairs(const ProjectionSet& set, const float* input, std::int64_t rows,
                           void* workspace, hipStream_t stream);

// lm_head for 5..16 rows: the same two launches, the multiplying one keeping (value, row)
// candidates per token instead of the logits, and a third that reduces them
// (lm_head.hip).  `workspace`: lm_head_f16_workspace_bytes(rows, input_dim) bytes.
std::int64_t lm_head_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim);
void launch_lm_head_f16(const Descriptor& descriptor, const float* input, std::int64_t rows,
                        void* workspace, std::int64_t* indices, float* maxima, hipStream_t stream);

}  // namespace nfn
