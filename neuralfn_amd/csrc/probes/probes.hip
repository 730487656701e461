// Measurement aids of the benchmark, built into a library of their own
// (libnfn_mi355_probes.so) that only bench.py and the probes' test load; nothing here is part
// of the path and nothing has a counterpart in the reference.
//  * shader clock under load: one wave that waits on the side while other work runs, and
//    reports how many shader cycles passed per tick of the constant 100 MHz device clock;
//  * read-only kernels of the decode grid: the floor under a launch;
//  * matrix-core rates from registers.
#include "../common.hpp"
#include "../../../include/nfn_mi355_probes.h"

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

// The same with the first `rounds` x 512 pieces per workgroup of a second buffer requested
// behind the first round of the workgroup's own loads: what a launch would gain or lose by
// pulling the next launch's first bytes into its XCD's L2 while it streams its own.
__global__ __launch_bounds__(512) void read_probe_chained_kernel(const v4u* __restrict__ data,
                                                                std::int64_t vectors_per_group,
                                                                const v4u* __restrict__ next,
                                                                int rounds,
                                                                std::uint32_t* __restrict__ sink) {
    const v4u* base = data + static_cast<std::int64_t>(blockIdx.x) * vectors_per_group;
    const v4u* ahead = next + static_cast<std::int64_t>(blockIdx.x) * vectors_per_group;
    std::uint32_t folded = 0;
    for (std::int64_t index = threadIdx.x; index < vectors_per_group; index += 8 * 512) {
        v4u piece[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            const std::int64_t at = index + k * 512;
            piece[k] = base[at < vectors_per_group ? at : vectors_per_group - 1];
        }
        if (index == threadIdx.x) {
            for (int r = 0; r < rounds; ++r) {
                const std::int64_t at = threadIdx.x + r * 512;
                folded ^= ahead[at < vectors_per_group ? at : vectors_per_group - 1].x;
            }
        }
#pragma unroll
        for (int k = 0; k < 8; ++k) folded ^= piece[k].x ^ piece[k].y ^ piece[k].z ^ piece[k].w;
    }
    if (folded == 0x9e3779b9u && vectors_per_group > 0) sink[blockIdx.x] = folded;
}

// What the matrix cores sustain per 32 x 32 x 32 step, operands in registers, for
// the three ways a prefill tile could be computed:
//   mode 0: two v_mfma_f32_32x32x16_f16 (fp16 operands, float accumulation);
//   mode 1: one v_mfma_i32_32x32x32_i8 (what an 8-bit activation would cost);
//   mode 2: two v_mfma_i32_32x32x32_i8 (the two int8 planes of a 16-bit activation
//           code) into fresh integer accumulators, then what the K-quant formats
//           force after every 32 values: 256*high + low, conversion to float and a
//           multiply-add with the sub-block's scale, for each of the 16 accumulators;
//   mode 3: one v_mfma_i32_32x32x32_i8 (an 8-bit activation per 32-value group, as the
//           reference's Q8_1 path quantizes) with the same rescale of the 16 accumulators
//           after every 32 values.
// Eight waves per compute unit and several workgroups per unit, as the GEMM runs.
typedef float probe_v16f __attribute__((ext_vector_type(16)));
typedef int probe_v16i __attribute__((ext_vector_type(16)));
typedef int probe_v4i __attribute__((ext_vector_type(4)));
typedef _Float16 probe_v8h __attribute__((ext_vector_type(8)));

template <int MODE>
__global__ __launch_bounds__(256) void mfma_rate_kernel(int steps, float* __restrict__ sink) {
    const int lane = threadIdx.x;
    probe_v16f total;
#pragma unroll
    for (int r = 0; r < 16; ++r) total[r] = 0.0f;
    probe_v4i a8 = {lane, lane * 3, lane * 5, lane * 7}, b8 = {lane * 11, lane * 13, lane * 17, lane * 19};
    probe_v8h a16, b16;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        a16[k] = static_cast<_Float16>(0.001f * static_cast<float>((lane + k) & 15));
        b16[k] = static_cast<_Float16>(0.002f * static_cast<float>((lane * 3 + k) & 15));
    }
    float scale = 1.0f + 1.0e-6f * static_cast<float>(lane);
    for (int step = 0; step < steps; ++step) {
        if constexpr (MODE == 0) {
            total = __builtin_amdgcn_mfma_f32_32x32x16_f16(a16, b16, total, 0, 0, 0);
            total = __builtin_amdgcn_mfma_f32_32x32x16_f16(b16, a16, total, 0, 0, 0);
        } else if constexpr (MODE == 1) {
            probe_v16i whole = __builtin_bit_cast(probe_v16i, total);
            whole = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8, b8, whole, 0, 0, 0);
            total = __builtin_bit_cast(probe_v16f, whole);
        } else if constexpr (MODE == 3) {
            probe_v16i zero;
#pragma unroll
            for (int r = 0; r < 16; ++r) zero[r] = 0;
            const probe_v16i dots = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8, b8, zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[r] = fmaf(static_cast<float>(dots[r]), scale, total[r]);
            }
            a8[0] += step;
            scale *= 1.0000001f;
        } else {
            probe_v16i zero;
#pragma unroll
            for (int r = 0; r < 16; ++r) zero[r] = 0;
            const probe_v16i high = __builtin_amdgcn_mfma_i32_32x32x32_i8(a8, b8, zero, 0, 0, 0);
            const probe_v16i low = __builtin_amdgcn_mfma_i32_32x32x32_i8(b8, a8, zero, 0, 0, 0);
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                total[r] = fmaf(static_cast<float>((high[r] << 8) + low[r]), scale, total[r]);
            }
            a8[0] += step;  // the next sub-block's operands and scale differ
            scale *= 1.0000001f;
        }
    }
    float folded = 0.0f;
#pragma unroll
    for (int r = 0; r < 16; ++r) folded += total[r];
    if (folded == 1.2345e30f) sink[blockIdx.x] = folded;
}

}  // namespace

void launch_mfma_rate_probe(int mode, int steps, int groups, float* sink, hipStream_t stream) {
    if (mode == 0) {
        hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(groups), dim3(256), 0, stream, steps, sink);
    } else if (mode == 1) {
        hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(groups), dim3(256), 0, stream, steps, sink);
    } else if (mode == 2) {
        hipLaunchKernelGGL(mfma_rate_kernel<2>, dim3(groups), dim3(256), 0, stream, steps, sink);
    } else {
        hipLaunchKernelGGL(mfma_rate_kernel<3>, dim3(groups), dim3(256), 0, stream, steps, sink);
    }
}

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

void launch_read_probe_chained(const void* data, std::int64_t nbytes, const void* next, int rounds,
                               std::uint32_t* sink, hipStream_t stream) {
    const int groups = compute_units();
    hipLaunchKernelGGL(read_probe_chained_kernel, dim3(groups), dim3(512), 0, stream,
                       static_cast<const v4u*>(data), nbytes / 16 / groups,
                       static_cast<const v4u*>(next), rounds, sink);
}

}  // namespace nfn

using namespace nfn;

extern "C" {

int nfn_mi355_probes_abi_version(void) { return 1; }

int nfn_mi355_shader_clock_probe_v1(std::uint64_t* cycles_and_ticks, std::int64_t microseconds,
                                    void* cuda_stream) {
    if (cycles_and_ticks == nullptr || microseconds < 1 || microseconds > 100000) return kInvalid;
    int ticks_per_millisecond = 0;  // the attribute is in kHz
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess ||
        hipDeviceGetAttribute(&ticks_per_millisecond, hipDeviceAttributeWallClockRate, device) !=
            hipSuccess ||
        ticks_per_millisecond <= 0) {
        return static_cast<int>(hipErrorNotSupported);
    }
    launch_clock_probe(cycles_and_ticks, microseconds * ticks_per_millisecond / 1000,
                       static_cast<std::uint64_t>(ticks_per_millisecond) * 1000,
                       as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_mfma_rate_probe_v1(int mode, int steps, int groups, float* sink, void* cuda_stream) {
    if (mode < 0 || mode > 3 || steps < 1 || steps > (1 << 20) || groups < 1 || groups > 65536 ||
        sink == nullptr) {
        return kInvalid;
    }
    launch_mfma_rate_probe(mode, steps, groups, sink, as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_read_probe_v1(const void* data, std::int64_t nbytes, std::uint32_t* sink,
                            void* cuda_stream) {
    if (nbytes < 0 || sink == nullptr || (nbytes > 0 && data == nullptr) ||
        reinterpret_cast<std::uintptr_t>(data) % 16 != 0) {
        return kInvalid;
    }
    launch_read_probe(data, nbytes, sink, as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_read_probe_chained_v1(const void* data, std::int64_t nbytes, const void* next,
                                    int prefetch_rounds, std::uint32_t* sink, void* cuda_stream) {
    if (nbytes <= 0 || sink == nullptr || data == nullptr || next == nullptr ||
        prefetch_rounds < 0 || prefetch_rounds > 64 ||
        reinterpret_cast<std::uintptr_t>(data) % 16 != 0 ||
        reinterpret_cast<std::uintptr_t>(next) % 16 != 0) {
        return kInvalid;
    }
    launch_read_probe_chained(data, nbytes, next, prefetch_rounds, sink, as_stream(cuda_stream));
    return launch_status();
}

}  // extern "C"
