// The public int8-activation ("Q8_1") path: activation quantizer and the
// int8 x K-quant dot product, single projection and 2..4 projections sharing
// one quantized row.
//
// Arithmetic follows the reference kernels: quantizer
// neuralfn/csrc/tile_cuda/kernels.cu:1527-1562, dot product :1620-1731
// (Q4_K/Q5_K round the activation scale and block sum through fp16 at use,
// Q6_K keeps the float scale), multi-projection launch :1844-1891.  One wave
// owns one output column; the 64 lanes cover the 64 four-value chunks of a
// 256-value super-block, so the single and multi launches reduce in the same
// order and agree bit for bit
// (tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:1173-1202).
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

__global__ __launch_bounds__(256) void quantize_q8_1_kernel(
    const float* __restrict__ input, std::int8_t* __restrict__ codes,
    float* __restrict__ scales, float* __restrict__ sums, std::int64_t block_count) {
    const std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * 256 + threadIdx.x;
    const std::int64_t block = index >> 5;
    if (block >= block_count) return;
    const Q8_1Value quantized = quantize_q8_1_value(input[index]);
    codes[index] = quantized.code;
    if ((threadIdx.x & 31) == 0) {
        scales[block] = quantized.scale;
        sums[block] = quantized.sum;
    }
}

__device__ __forceinline__ float through_half(float value) {
    return static_cast<float>(static_cast<_Float16>(value));
}

__device__ __forceinline__ int q6_quant(const std::uint8_t* block, int within) {
    const int half = within >> 7;
    const int position = within & 127;
    const int quarter = position >> 5;
    const int lane = position & 31;
    const std::uint32_t low = block[half * 64 + lane + ((quarter & 1) ? 32 : 0)];
    const std::uint32_t high = block[128 + half * 32 + lane];
    const int nibble = quarter < 2 ? (low & 15) : (low >> 4);
    return (nibble | (((high >> (2 * quarter)) & 3) << 4)) - 32;
}

// Partial dot product of one lane over its chunk of every super-block.
__device__ __forceinline__ float q8_1_lane_partial(
    std::uint32_t encoding, const std::uint8_t* row_data, std::int64_t input_dim,
    const std::int8_t* __restrict__ codes, const float* __restrict__ scales,
    const float* __restrict__ sums, int lane) {
    const int within = lane * 4;
    const int logical_group = within >> 5;
    const int local = within & 31;
    const std::int64_t blocks = input_dim >> 8;
    float sum = 0.0f;
    for (std::int64_t b = 0; b < blocks; ++b) {
        const int activation = *reinterpret_cast<const int*>(codes + b * 256 + within);
        const std::int64_t q8_block = b * 8 + logical_group;
        if (encoding == kEncQ6K) {
            const std::uint8_t* block = row_data + b * 210;
            std::uint32_t quantized = 0;
#pragma unroll
            for (int byte = 0; byte < 4; ++byte) {
                quantized |= static_cast<std::uint32_t>(q6_quant(block, within + byte) & 0xff)
                    << (8 * byte);
            }
            const int scale = static_cast<std::int8_t>(block[192 + (within >> 4)]);
            const int dot = __builtin_amdgcn_sdot4(static_cast<int>(quantized), activation, 0, false);
            sum += load_half(block + 208) * scales[q8_block] * static_cast<float>(scale * dot);
        } else {
            const bool q5 = encoding == kEncQ5K;
            const std::uint8_t* block = row_data + b * (q5 ? 176 : 144);
            const int outer_group = logical_group >> 1;
            const bool high_half = (logical_group & 1) != 0;
            const std::uint32_t packed = *reinterpret_cast<const std::uint32_t*>(
                block + (q5 ? 48 : 16) + outer_group * 32 + local);
            std::uint32_t quantized = (packed >> (high_half ? 4 : 0)) & 0x0f0f0f0fu;
            if (q5) {
                const std::uint32_t highs =
                    *reinterpret_cast<const std::uint32_t*>(block + 16 + local);
                const int bit = 2 * outer_group + (high_half ? 1 : 0);
                quantized |= ((highs >> bit) & 0x01010101u) << 4;
            }
            int scale, minimum;
            k_scale_min(block + 4, logical_group, &scale, &minimum);
            const int dot = __builtin_amdgcn_sdot4(static_cast<int>(quantized), activation, 0, false);
            sum += load_half(block) * through_half(scales[q8_block]) *
                static_cast<float>(scale * dot);
            if (local == 0) {
                sum -= load_half(block + 2) * static_cast<float>(minimum) *
                    through_half(sums[q8_block]);
            }
        }
    }
    return sum;
}

__global__ __launch_bounds__(256) void linear_q8_1_kernel(
    ProjectionSet set, const std::int8_t* __restrict__ codes, const float* __restrict__ scales,
    const float* __restrict__ sums, const float* __restrict__ bias,
    std::int64_t total_columns) {
    const int lane = threadIdx.x & 63;
    const std::int64_t column = static_cast<std::int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (column >= total_columns) return;
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && column >= set.op[index].first_tile) which = index;
    }
    const Projection op = set.op[which];
    const std::int64_t out_col = column - op.first_tile;
    const std::int64_t row = blockIdx.y;
    const std::int64_t input_dim = set.input_dim;
    const float partial = q8_1_lane_partial(
        op.encoding, op.data + out_col * op.row_stride, input_dim, codes + row * input_dim,
        scales + row * (input_dim >> 5), sums + row * (input_dim >> 5), lane);
    const float total = wave_sum(partial);
    if (lane == 0) {
        op.output[row * op.output_dim + out_col] =
            total + (bias != nullptr ? bias[out_col] : 0.0f);
    }
}

}  // namespace

void launch_quantize_q8_1(const float* input, std::int8_t* codes, float* scales, float* sums,
                          std::int64_t rows, std::int64_t width, hipStream_t stream) {
    const std::int64_t block_count = rows * (width / 32);
    const std::int64_t grid = (block_count * 32 + 255) / 256;
    hipLaunchKernelGGL(quantize_q8_1_kernel, dim3(static_cast<unsigned>(grid)), dim3(256), 0,
                       stream, input, codes, scales, sums, block_count);
}

void launch_linear_q8_1(ProjectionSet set, const std::int8_t* codes, const float* scales,
                        const float* sums, const float* bias, std::int64_t rows,
                        hipStream_t stream) {
    std::int64_t total_columns = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = static_cast<std::uint32_t>(total_columns);
        total_columns += set.op[index].output_dim;
    }
    const dim3 grid(static_cast<unsigned>((total_columns + 3) / 4), static_cast<unsigned>(rows), 1);
    hipLaunchKernelGGL(linear_q8_1_kernel, grid, dim3(256), 0, stream, set, codes, scales, sums,
                       bias, total_columns);
}

}  // namespace nfn
