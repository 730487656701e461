// Shader clock under load: one wave that waits on the side while other work
// runs, and reports how many shader cycles passed per tick of the constant
// 100 MHz device clock.  Measurement aid of the benchmark; no counterpart in
// the reference.
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

// out[0] = shader cycles, out[1] = ticks of the constant clock, out[2] = that
// clock's ticks per second.  The wait ends after `ticks` ticks, or after
// `max_polls` polls whatever the clocks say.
__global__ __launch_bounds__(64) void clock_probe_kernel(std::uint64_t* __restrict__ out,
                                                        std::int64_t ticks, int max_polls,
                                                        std::uint64_t ticks_per_second) {
    const std::uint64_t cycles_begin = clock64();
    const std::uint64_t ticks_begin = wall_clock64();
    std::uint64_t cycles_end = cycles_begin;
    std::uint64_t ticks_end = ticks_begin;
    for (int poll = 0; poll < max_polls; ++poll) {
        __builtin_amdgcn_s_sleep(32);
        cycles_end = clock64();
        ticks_end = wall_clock64();
        if (static_cast<std::int64_t>(ticks_end - ticks_begin) >= ticks) break;
    }
    if (threadIdx.x == 0) {
        out[0] = cycles_end - cycles_begin;
        out[1] = ticks_end - ticks_begin;
        out[2] = ticks_per_second;
    }
}

// What a launch costs before it computes anything: every workgroup reads its
// contiguous share of `vectors` 16-byte pieces with four loads per lane in
// flight and folds them; `sink` is written only if the fold hits one value, so
// the loads cannot be dropped and nothing is stored in practice.  With zero
// pieces it is an empty kernel of the same grid.
typedef unsigned v4u __attribute__((ext_vector_type(4)));
__global__ __launch_bounds__(512) void read_probe_kernel(const v4u* __restrict__ data,
                                                        std::int64_t vectors_per_group,
                                                        std::uint32_t* __restrict__ sink) {
    const v4u* base = data + static_cast<std::int64_t>(blockIdx.x) * vectors_per_group;
    std::uint32_t folded = 0;
    for (std::int64_t index = threadIdx.x; index < vectors_per_group; index += 4 * 512) {
        v4u piece[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const std::int64_t at = index + k * 512;
            piece[k] = base[at < vectors_per_group ? at : vectors_per_group - 1];
        }
#pragma unroll
        for (int k = 0; k < 4; ++k) folded ^= piece[k].x ^ piece[k].y ^ piece[k].z ^ piece[k].w;
    }
    if (folded == 0x9e3779b9u && vectors_per_group > 0) sink[blockIdx.x] = folded;
}

}  // namespace

void launch_read_probe(const void* data, std::int64_t nbytes, std::uint32_t* sink,
                       hipStream_t stream) {
    const int groups = compute_units();
    hipLaunchKernelGGL(read_probe_kernel, dim3(groups), dim3(512), 0, stream,
                       static_cast<const v4u*>(data), nbytes / 16 / groups, sink);
}

void launch_clock_probe(std::uint64_t* out, std::int64_t ticks, std::uint64_t ticks_per_second,
                        hipStream_t stream) {
    // a poll sleeps 32 * 64 cycles, about a microsecond: the poll limit ends a
    // wait of up to `ticks` (10 ns each) with a wide margin and no more
    const std::int64_t polls = ticks / 20 + 1024;
    hipLaunchKernelGGL(clock_probe_kernel, dim3(1), dim3(64), 0, stream, out, ticks,
                       static_cast<int>(polls < (1 << 24) ? polls : (1 << 24)), ticks_per_second);
}

}  // namespace nfn
