// Whole-matrix dequantization to float, one thread per four consecutive
// elements.  Bit-exact with the reference's per-element decoder
// (neuralfn/csrc/tile_cuda/kernels.cu:1225-1335) and with the CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616) for Q4_K and Q5_K;
// Q6_K uses the canonical sub-scale index.
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

__global__ __launch_bounds__(256) void dequantize_kernel(
    const std::uint8_t* __restrict__ data, std::uint32_t encoding, std::int64_t row_stride,
    std::int64_t input_dim, std::int64_t count, float* __restrict__ output) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        const std::int64_t row = index / input_dim;
        const std::int64_t col = index - row * input_dim;
        output[index] = weight_value(encoding, data + row * row_stride, col);
    }
}

}  // namespace

void launch_dequantize(const Descriptor& descriptor, float* output, hipStream_t stream) {
    const std::int64_t count = descriptor.output_dim * descriptor.input_dim;
    const std::int64_t blocks = (count + 255) / 256;
    const unsigned grid = static_cast<unsigned>(blocks < (1 << 20) ? blocks : (1 << 20));
    hipLaunchKernelGGL(dequantize_kernel, dim3(grid), dim3(256), 0, stream, descriptor.data,
                       descriptor.encoding, descriptor.row_stride_bytes, descriptor.input_dim,
                       count, output);
}

}  // namespace nfn
