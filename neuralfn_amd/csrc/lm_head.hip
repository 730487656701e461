// lm_head GEMV with the argmax fused in.  Pass 1: every workgroup computes the
// logits of its vocabulary rows and keeps only the best (value, index) per
// input row in the workspace.  Pass 2: one workgroup per input row reduces the
// per-workgroup candidates.  The logits are never written to memory.
//
// The reference does this as two separate operations with an 808 KB logits
// buffer in between (neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:4087-4151:
// linear, then nfn_native_tile_argmax_rows_float32_v1).  Tie rule and NaN
// behaviour are those of neuralfn/csrc/tile_cuda/kernels.cu:1564-1602.
#include "common.hpp"
#include "gemv_f32_device.hpp"
#include "kernels.hpp"
#include "lm_head.hpp"

namespace nfn {

namespace {

constexpr int kWavesPerBlock = 4;

template <int R>
__global__ __launch_bounds__(kWavesPerBlock * kWave) void lm_head_partial_kernel(
    Projection op, std::int64_t input_dim, const float* __restrict__ input, std::int64_t rows,
    int columns_per_wave, LmHeadCandidate* __restrict__ candidates) {
    __shared__ float shared_values[kWavesPerBlock][R];
    __shared__ std::int64_t shared_indices[kWavesPerBlock][R];
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const std::int64_t first_column =
        (static_cast<std::int64_t>(blockIdx.x) * kWavesPerBlock + wave) * columns_per_wave;
    float best_value[R];
    std::int64_t best_index[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        best_value[r] = -INFINITY;
        best_index[r] = 0;
    }
    const int active = static_cast<int>(rows);
    for (int step = 0; step < columns_per_wave; ++step) {
        const std::int64_t column = first_column + step;
        if (column >= op.output_dim) break;
        float sums[R];
        wave_row_partials<R, kPlain>(op.encoding, op.data + column * op.row_stride, input_dim,
                                     input, nullptr, 0, active, lane, sums);
#pragma unroll
        for (int r = 0; r < R; ++r) {
            const float logit = wave_sum(sums[r]);
            better(logit, column, best_value[r], best_index[r]);
        }
    }
    if (lane == 0) {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            shared_values[wave][r] = best_value[r];
            shared_indices[wave][r] = best_index[r];
        }
    }
    __syncthreads();
    if (threadIdx.x < R && threadIdx.x < rows) {
        float value = shared_values[0][threadIdx.x];
        std::int64_t index = shared_indices[0][threadIdx.x];
        for (int w = 1; w < kWavesPerBlock; ++w) {
            better(shared_values[w][threadIdx.x], shared_indices[w][threadIdx.x], value, index);
        }
        LmHeadCandidate candidate;
        candidate.index = index;
        candidate.value = value;
        candidate.pad = 0;
        candidates[static_cast<std::int64_t>(threadIdx.x) * gridDim.x + blockIdx.x] = candidate;
    }
}

}  // namespace

constexpr int kFinalThreads = 1024;

__global__ __launch_bounds__(kFinalThreads) void lm_head_final_kernel(
    const LmHeadCandidate* __restrict__ candidates, std::int64_t candidate_count,
    std::int64_t* __restrict__ indices, float* __restrict__ maxima) {
    constexpr int kFinalWaves = kFinalThreads / kWave;
    __shared__ float wave_values[kFinalWaves];
    __shared__ std::int64_t wave_indices[kFinalWaves];
    const std::int64_t row = blockIdx.x;
    float best_value = -INFINITY;
    std::int64_t best_index = 0;
    for (std::int64_t i = threadIdx.x; i < candidate_count; i += kFinalThreads) {
        const LmHeadCandidate c = candidates[row * candidate_count + i];
        better(c.value, c.index, best_value, best_index);
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float other_value = __shfl_xor(best_value, offset, 64);
        const std::int64_t other_index = __shfl_xor(best_index, offset, 64);
        better(other_value, other_index, best_value, best_index);
    }
    if ((threadIdx.x & 63) == 0) {
        wave_values[threadIdx.x >> 6] = best_value;
        wave_indices[threadIdx.x >> 6] = best_index;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int w = 1; w < kFinalWaves; ++w) {
            better(wave_values[w], wave_indices[w], best_value, best_index);
        }
        indices[row] = best_index;
        maxima[row] = best_value;
    }
}

void launch_lm_head_final(const LmHeadCandidate* candidates, std::int64_t candidate_count,
                          std::int64_t* indices, float* maxima, std::int64_t rows,
                          hipStream_t stream) {
    hipLaunchKernelGGL(lm_head_final_kernel, dim3(static_cast<unsigned>(rows)),
                       dim3(kFinalThreads), 0, stream, candidates, candidate_count, indices,
                       maxima);
}

std::int64_t lm_head_f32_blocks(std::int64_t output_dim) {
    // 16 vocabulary rows per wave, 64 per workgroup.
    return (output_dim + 63) / 64;
}

void launch_lm_head_f32(const Descriptor& descriptor, const float* input, std::int64_t rows,
                        LmHeadCandidate* candidates, std::int64_t* indices, float* maxima,
                        hipStream_t stream) {
    Projection op{};
    op.data = descriptor.data;
    op.output = nullptr;
    op.output_dim = descriptor.output_dim;
    op.row_stride = descriptor.row_stride_bytes;
    op.encoding = descriptor.encoding;
    const std::int64_t blocks = lm_head_f32_blocks(descriptor.output_dim);
    const dim3 grid(static_cast<unsigned>(blocks));
    const dim3 block(kWavesPerBlock * kWave);
    if (rows == 1) {
        hipLaunchKernelGGL((lm_head_partial_kernel<1>), grid, block, 0, stream, op,
                           descriptor.input_dim, input, rows, 16, candidates);
    } else if (rows <= 4) {
        hipLaunchKernelGGL((lm_head_partial_kernel<4>), grid, block, 0, stream, op,
                           descriptor.input_dim, input, rows, 16, candidates);
    } else {
        hipLaunchKernelGGL((lm_head_partial_kernel<8>), grid, block, 0, stream, op,
                           descriptor.input_dim, input, rows, 16, candidates);
    }
    launch_lm_head_final(candidates, blocks, indices, maxima, rows, stream);
}

}  // namespace nfn
