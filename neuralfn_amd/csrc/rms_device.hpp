// Device code shared by the RMS normalisation kernels (rms.hip) and the decode GEMV that runs
// the two normalisations in its own prologue (gemv_dot.hip): the affine weight of a
// normalisation and one row of "hidden = residual + rms(input); normalized = rms(hidden)" by a
// whole workgroup, in the reference kernel's float order
// (neuralfn/csrc/tile_cuda/kernels.cu:2155-2243).
#pragma once

#include "common.hpp"

namespace nfn {

constexpr int kRmsThreads = 256;  // partial sums of the reference's order
constexpr int kRmsOwned = 32;     // columns per partial sum held in registers: rows of up to 8192

// Affine weight of one normalisation: a [1, width] packed row, or none.
struct NormWeight {
    const std::uint8_t* data;
    std::uint32_t encoding;
    int present;
    int centered;  // the stored weight is (scale - 1)
};

__device__ __forceinline__ float norm_scale(const NormWeight& weight, std::int64_t column) {
    if (!weight.present) return 1.0f;
    float scale = weight_value(weight.encoding, weight.data, column);
    if (weight.centered) scale += 1.0f;
    return scale;
}

// The scales of N columns at once.  The encoding is looked at once, outside the
// loop, so that for float and bf16 rows (what norm weights are) the N loads are
// plain and independent and go out together instead of one behind the other's
// branch.
template <int N, typename Index>
__device__ __forceinline__ void norm_scales(const NormWeight& weight, const Index (&columns)[N],
                                            float (&scale)[N]) {
    if (!weight.present) {
#pragma unroll
        for (int i = 0; i < N; ++i) scale[i] = 1.0f;
        return;
    }
    if (weight.encoding == kEncF32) {
        const float* values = reinterpret_cast<const float*>(weight.data);
#pragma unroll
        for (int i = 0; i < N; ++i) scale[i] = values[columns[i]];
    } else if (weight.encoding == kEncBF16) {
        const std::uint16_t* values = reinterpret_cast<const std::uint16_t*>(weight.data);
#pragma unroll
        for (int i = 0; i < N; ++i) scale[i] = bf16_to_float(values[columns[i]]);
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) scale[i] = weight_value(weight.encoding, weight.data, columns[i]);
    }
    if (weight.centered) {
#pragma unroll
        for (int i = 0; i < N; ++i) scale[i] += 1.0f;
    }
}

// What the decode kernel with the two normalisations in its prologue needs besides its input
// row: the other operands and where the three rows of the norm kernel's results go.
struct DualNormArguments {
    const float* residual;
    NormWeight first_weight, second_weight;
    float* hidden;
    float* captured;
    float* normalized;
    float first_eps, second_eps;
};

// The halving tree over the 256 sums of threads (0, t), additions in the order of the
// reference's tree: (p[t] + p[t+128]) + (p[t+64] + p[t+192]) is its first two levels, the last
// six run inside a wave.  Every thread of the workgroup calls it; every wave runs the tree
// for itself on the same 256 numbers (the same operations, the same result), which spares
// the barrier that handing one wave's total to the others would take.  `partials` holds
// kRmsThreads floats and may be written again after the workgroup's next barrier.
__device__ __forceinline__ float rms_tree_total(float square_sum, float* partials) {
    if (threadIdx.x < kRmsThreads) partials[threadIdx.x] = square_sum;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    const float a = partials[lane] + partials[lane + 128];
    const float b = partials[lane + 64] + partials[lane + 192];
    float value = a + b;
#pragma unroll
    for (int stride = 32; stride > 0; stride /= 2) value += __shfl_down(value, stride, 64);
    return __shfl(value, 0, 64);
}

// One row of the two normalisations by a workgroup of LOADERS x 256 threads, rows of up to
// 8192 columns, in two steps (request, finish) so that the caller can put other requests
// between the loads and the first wait.  Sum t adds the squares of columns t, t + 256, ... one after another, then
// the halving tree: the order of the 256-thread kernel; the loads are spread over LOADERS
// threads per sum (thread (q, t) loads columns t + 256 (q + LOADERS k)), which hand their
// values to thread (0, t) through `handed` (kRmsOwned x 256 floats of LDS).  After
// dual_rms_finish handed[column] holds the normalized row and every thread may read it; with
// `store` the three global rows are written as well (any of them may be null).
template <int LOADERS>
struct DualRmsOperands {
    static constexpr int kLoaded = kRmsOwned / LOADERS;
    float value[kLoaded], other[kLoaded], first_scale[kLoaded], second_scale[kLoaded];
};

// ... its loads, all requested at once; nothing waits for them here
template <int LOADERS>
__device__ __forceinline__ void dual_rms_request(DualRmsOperands<LOADERS>& operands,
                                                 const float* __restrict__ source,
                                                 const float* __restrict__ residual,
                                                 const NormWeight& first_weight,
                                                 const NormWeight& second_weight, int width) {
    constexpr int kLoaded = DualRmsOperands<LOADERS>::kLoaded;
    const int t = threadIdx.x & (kRmsThreads - 1);
    const int q = threadIdx.x / kRmsThreads;
    int clamped[kLoaded];
#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + LOADERS * i) * kRmsThreads;
        clamped[i] = min(column, width - 1);
        operands.value[i] = column < width ? source[clamped[i]] : 0.0f;
        operands.other[i] = residual[clamped[i]];
    }
    norm_scales(first_weight, clamped, operands.first_scale);
    norm_scales(second_weight, clamped, operands.second_scale);
}

// ... and the arithmetic
template <int LOADERS>
__device__ __forceinline__ void dual_rms_finish(
    DualRmsOperands<LOADERS>& operands, int width, float first_eps, float second_eps, bool store,
    float* __restrict__ hidden, float* __restrict__ captured, float* __restrict__ normalized,
    float* handed, float* partials) {
    constexpr int kLoaded = DualRmsOperands<LOADERS>::kLoaded;
    const int t = threadIdx.x & (kRmsThreads - 1);
    const int q = threadIdx.x / kRmsThreads;
    float (&value)[kLoaded] = operands.value;
    // sum t over its columns in order (a column past the end contributes fma(0, 0, sum) = sum)
    auto ordered_sum = [&]() {
        float square_sum = 0.0f;
        if (q == 0) {
#pragma unroll
            for (int k = 0; k < kRmsOwned; ++k) {
                const float v = handed[k * kRmsThreads + t];
                square_sum = fmaf(v, v, square_sum);
            }
        }
        return square_sum;
    };
#pragma unroll
    for (int i = 0; i < kLoaded; ++i) handed[(q + LOADERS * i) * kRmsThreads + t] = value[i];
    __syncthreads();
    const float first_inverse =
        1.0f / sqrtf(rms_tree_total(ordered_sum(), partials) / static_cast<float>(width) + first_eps);
#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + LOADERS * i) * kRmsThreads;
        const float sum = __fadd_rn(
            __fmul_rn(__fmul_rn(value[i], first_inverse), operands.first_scale[i]), operands.other[i]);
        value[i] = column < width ? sum : 0.0f;
        if (store && column < width) {
            if (hidden != nullptr) hidden[column] = sum;
            if (captured != nullptr) captured[column] = sum;
        }
        // every sum has read its old values: the tree's barriers lie in between
        handed[(q + LOADERS * i) * kRmsThreads + t] = value[i];
    }
    __syncthreads();
    const float second_inverse =
        1.0f / sqrtf(rms_tree_total(ordered_sum(), partials) / static_cast<float>(width) + second_eps);
#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + LOADERS * i) * kRmsThreads;
        const float result =
            __fmul_rn(__fmul_rn(value[i], second_inverse), operands.second_scale[i]);
        if (store && column < width && normalized != nullptr) normalized[column] = result;
        // (the sums have read `handed`: the tree's barriers lie in between)
        handed[(q + LOADERS * i) * kRmsThreads + t] = column < width ? result : 0.0f;
    }
    __syncthreads();
}

// Host side: the kernel argument for a norm weight descriptor (null: no weight).
inline NormWeight norm_weight(const Descriptor* descriptor, bool centered) {
    NormWeight weight{};
    if (descriptor != nullptr) {
        weight.data = descriptor->data;
        weight.encoding = descriptor->encoding;
        weight.present = 1;
        weight.centered = centered ? 1 : 0;
    }
    return weight;
}

}  // namespace nfn
