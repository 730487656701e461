// Prefill dequant-GEMM on the fp16 matrix cores (gemm_mfma.hip).
#pragma once

#include "common.hpp"

namespace nfn {

// Bytes of device workspace the fp16 path needs: a row-scaled fp16 copy of the
// activations in whole 256-row tiles, one inverse scale per row, and, where a
// small problem splits K over several workgroups per tile, one copy of the
// output per share.
std::int64_t gemm_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim,
                                      std::int64_t output_dim);
bool gemm_f16_supports(std::uint32_t encoding, std::int64_t input_dim);
// How a launch of this geometry is cut on the current device: rows of the
// output tile a workgroup owns (128 or 256) and the number of K shares (1 =
// unsplit; more = one partial output per share, summed by a second launch).
void gemm_f16_plan(std::uint32_t encoding, std::int64_t rows, std::int64_t input_dim,
                   std::int64_t output_dim, int* tile_rows, int* k_shares);
// output[rows, output_dim] = input[rows, input_dim] * W^T, float accumulation.
void launch_gemm_f16(const Descriptor& descriptor, const float* input, float* output,
                      std::int64_t rows, void* workspace, hipStream_t stream);
// The same in two steps, for several projections of one input: the activations
// go to the workspace once, then each projection runs from there (the split-K
// partial buffer behind them is reused; the launches are stream-ordered).
void convert_gemm_activations(const float* input, std::int64_t rows, std::int64_t input_dim,
                              void* workspace, hipStream_t stream);
void launch_gemm_f16_converted(const Descriptor& descriptor, float* output, std::int64_t rows,
                               void* workspace, hipStream_t stream);

}  // namespace nfn
