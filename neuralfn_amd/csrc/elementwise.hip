// The two element-wise operators whose arithmetic the fused activation
// prologues must reproduce bit for bit
// (neuralfn/csrc/tile_cuda/kernels.cu:3242-3252 sigmoid gate;
//  neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:299-317 fused forms).
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

template <int P>
__global__ __launch_bounds__(256) void elementwise_kernel(const float* __restrict__ first,
                                                          const float* __restrict__ second,
                                                          float* __restrict__ output,
                                                          std::int64_t count) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        output[index] = apply_prologue<P>(first[index], second[index]);
    }
}

unsigned grid_for(std::int64_t count) {
    const std::int64_t blocks = (count + 255) / 256;
    return static_cast<unsigned>(blocks < 65536 ? blocks : 65536);
}

}  // namespace

void launch_sigmoid_gate(const float* values, const float* gate, float* output,
                         std::int64_t count, hipStream_t stream) {
    hipLaunchKernelGGL((elementwise_kernel<kGated>), dim3(grid_for(count)), dim3(256), 0, stream,
                       values, gate, output, count);
}

void launch_swiglu(const float* gate, const float* up, float* output, std::int64_t count,
                   hipStream_t stream) {
    hipLaunchKernelGGL((elementwise_kernel<kSwiGlu>), dim3(grid_for(count)), dim3(256), 0, stream,
                       gate, up, output, count);
}

}  // namespace nfn
