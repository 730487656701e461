// Verifier rows on the int8 matrix cores in the one-row arithmetic (gemv_rows.hip).
#pragma once

#include "common.hpp"

#include "wave_rows.hpp"

namespace nfn {

// Operand image of the activations, written next to the records: per block 8 KB of operand-A
// fragments, [32-value group][lane 0..63][16 bytes] (lane l: matrix row l % 32, values
// 16 (l / 32)..+15 of the group), so that a wave fetches a fragment with one coalesced load,
// then the block's 16 token scales.  Matrix row i = 8 a + 4 half + 2 c + plane holds token
// S * half + 2 a + c, which puts token S * (lane / 32) + slot into output registers 2 * slot
// (high plane) and 2 * slot + 1 (low plane); S = token slots per lane.
constexpr int kRowsImageFragments = 8 * 1024;
constexpr int kRowsImageBlock = kRowsImageFragments + 16 * 4;

__host__ __device__ constexpr int rows_token_slots(int tokens) {
    return tokens <= 4 ? 2 : tokens <= 8 ? 4 : 8;
}

// One wave's record (token, block) goes into the image: this lane's values 4 lane..+3 are the
// 32-value group lane / 8, values 4 (lane % 8)..+3 of it.
__device__ __forceinline__ void store_operand_image(std::uint8_t* image, int block, int token,
                                                    int tokens, int lane, const ActivationCodes& codes) {
    const int slots = rows_token_slots(tokens);
    const int half = token / slots;
    const int slot = token - half * slots;
    const int row = 8 * (slot >> 1) + 4 * half + 2 * (slot & 1);
    std::uint8_t* block_image = image + static_cast<std::int64_t>(block) * kRowsImageBlock;
    std::uint8_t* piece = block_image +
        (((lane >> 3) * 64 + ((lane >> 2) & 1) * 32 + row) * 16) + (lane & 3) * 4;
    *reinterpret_cast<std::uint32_t*>(piece) = codes.hi;
    *reinterpret_cast<std::uint32_t*>(piece + 16) = codes.lo;
    if (lane == 0) {
        reinterpret_cast<float*>(block_image + kRowsImageFragments)[token] =
            codes.maximum * (1.0f / kCodeRange);
    }
}

// True when a projection of this encoding and width has the kernel.
bool gemv_rows_supports(std::uint32_t encoding, std::int64_t input_dim);

// Bytes of the operand image of `input_dim` columns (any row count up to 16).
std::int64_t gemv_rows_image_bytes(std::int64_t input_dim);

// The projections of `set` whose launch adds the two halves of every row's butterfly onto the
// output (the form that pays when whole tiles would leave most of the chip idle in their last
// pass): their outputs must hold -0.0f when launch_gemv_rows starts.
// fill_launch: the fill is a launch of its own (launch_fill_outputs), which has to pay too.
ProjectionSet gemv_rows_split_set(const ProjectionSet& set, bool fill_launch);

// Fills the outputs (rows x output_dim floats each) of the projections of `clear` with -0.0f.
void launch_fill_outputs(const ProjectionSet& clear, std::int64_t rows, hipStream_t stream);

// Writes the activation records of `rows` rows (the prologue applied) to `records`
// (rows * input_dim / 256 records of 576 bytes, token by token) and the same codes in
// matrix-operand order to `image` (gemv_rows_image_bytes); fills the outputs (rows x
// output_dim floats each) of the projections of `clear` with -0.0f.
void launch_quantize_records(const float* first, const float* second, int prologue,
                             std::int64_t rows, std::int64_t input_dim, std::uint8_t* records,
                             std::uint8_t* image, const ProjectionSet& clear, hipStream_t stream);

// rows 4..16 of the set's projections from the operand image.  outputs_cleared: the outputs of
// gemv_rows_split_set(set, fill_launch) hold -0.0f (launch_quantize_records or
// launch_fill_outputs ran with that set).
void launch_gemv_rows(const ProjectionSet& set, const std::uint8_t* image, std::int64_t rows,
                      bool outputs_cleared, bool fill_launch, hipStream_t stream);

}  // namespace nfn
