// Row argmax over float logits.  Ties select the lowest column, NaN never
// wins, an all-NaN row yields index 0 and -inf: the behaviour of the
// reference kernel (neuralfn/csrc/tile_cuda/kernels.cu:1564-1602), pinned by
// tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:1869-1904.
#include "common.hpp"
#include "kernels.hpp"
#include "lm_head.hpp"

namespace nfn {

namespace {

constexpr int kArgmaxThreads = 1024;

__global__ __launch_bounds__(kArgmaxThreads) void argmax_rows_kernel(
    const float* __restrict__ values, std::int64_t* __restrict__ indices,
    float* __restrict__ maxima, std::int64_t width) {
    __shared__ float wave_values[kArgmaxThreads / kWave];
    __shared__ std::int64_t wave_indices[kArgmaxThreads / kWave];
    const std::int64_t row = blockIdx.x;
    const float* source = values + row * width;
    float best_value = -INFINITY;
    std::int64_t best_index = 0;
    // Vector body where the row start is 16-byte aligned, scalar otherwise.
    const bool aligned = (reinterpret_cast<std::uintptr_t>(source) & 15u) == 0;
    const std::int64_t vector_count = aligned ? width / 4 : 0;
    // eight loads of a thread in flight at a time: a row is read by one workgroup, at what
    // one compute unit takes in (a 202,048-wide row: 35 us with one load at a time, 23 us so)
    constexpr int kAhead = 8;
    for (std::int64_t first = threadIdx.x; first < vector_count; first += kArgmaxThreads * kAhead) {
        float4 x[kAhead];
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const std::int64_t v = first + static_cast<std::int64_t>(u) * kArgmaxThreads;
            x[u] = reinterpret_cast<const float4*>(source)[v < vector_count ? v : vector_count - 1];
        }
#pragma unroll
        for (int u = 0; u < kAhead; ++u) {
            const std::int64_t v = first + static_cast<std::int64_t>(u) * kArgmaxThreads;
            if (v < vector_count) {
                better(x[u].x, v * 4, best_value, best_index);
                better(x[u].y, v * 4 + 1, best_value, best_index);
                better(x[u].z, v * 4 + 2, best_value, best_index);
                better(x[u].w, v * 4 + 3, best_value, best_index);
            }
        }
    }
    for (std::int64_t column = vector_count * 4 + threadIdx.x; column < width;
         column += kArgmaxThreads) {
        better(source[column], column, best_value, best_index);
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        const float other_value = __shfl_xor(best_value, offset, 64);
        const std::int64_t other_index = __shfl_xor(best_index, offset, 64);
        better(other_value, other_index, best_value, best_index);
    }
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    if (lane == 0) {
        wave_values[wave] = best_value;
        wave_indices[wave] = best_index;
    }
    __syncthreads();
    if (wave == 0) {
        best_value = lane < kArgmaxThreads / kWave ? wave_values[lane] : -INFINITY;
        best_index = lane < kArgmaxThreads / kWave ? wave_indices[lane] : 0;
#pragma unroll
        for (int offset = 8; offset > 0; offset >>= 1) {
            const float other_value = __shfl_xor(best_value, offset, 64);
            const std::int64_t other_index = __shfl_xor(best_index, offset, 64);
            better(other_value, other_index, best_value, best_index);
        }
        if (lane == 0) {
            indices[row] = best_index;
            maxima[row] = best_value;
        }
    }
}

}  // namespace

void launch_argmax_rows(const float* values, std::int64_t* indices, float* maxima,
                        std::int64_t rows, std::int64_t width, hipStream_t stream) {
    hipLaunchKernelGGL(argmax_rows_kernel, dim3(static_cast<unsigned>(rows)),
                       dim3(kArgmaxThreads), 0, stream, values, indices, maxima, width);
}

}  // namespace nfn
