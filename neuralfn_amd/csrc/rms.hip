// Two adjacent RMS normalisations of the decode loop in one launch:
//
//   hidden            = residual_input + rms(input, first_weight, first_eps)
//   residual_output   = hidden
//   normalized_output = rms(hidden, second_weight, second_eps)
//
// and, for the one-row handoff, the activation records of normalized_output in
// the caller's small-batch workspace, so that the projection that follows can
// skip its own quantization.
//
// One workgroup per row; rows of up to 8192 columns take the kernel whose loads
// are all in flight at once (1024 threads), wider ones the 256-thread kernel that
// walks memory in batches.
// The float arithmetic follows the
// reference kernel operation for operation
// (neuralfn/csrc/tile_cuda/kernels.cu:2155-2243): thread t accumulates the
// squares of columns t, t+256, ... with fused multiply-adds, the 256 partial
// sums are added in a halving tree, normalized = (x * inverse_rms) * scale with
// two roundings, hidden = normalized + residual with one.  The only departure:
// inverse_rms is 1 / sqrt(mean + eps) with correctly rounded division and
// square root where the reference calls the device's approximate reciprocal
// square root, so the two can differ in the last bits of that one factor.
#include "common.hpp"
#include "f16_decode.hpp"
#include "gemv_rows.hpp"
#include "kernels.hpp"
#include "rms_device.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

constexpr int kBatch = 8;  // columns per thread whose loads are issued together

// 1 / sqrt(mean of squares + eps) of `values[0, width)`, the same number in every thread.
__device__ __forceinline__ float inverse_rms(const float* values, std::int64_t width, float eps,
                                             float* partials) {
    // Same order as a plain strided loop; the loads of a batch go out together
    // (a column past the end contributes fma(0, 0, sum) = sum).
    float square_sum = 0.0f;
    for (std::int64_t base = threadIdx.x; base < width; base += kBatch * kRmsThreads) {
        float value[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const std::int64_t column = base + i * kRmsThreads;
            value[i] = column < width ? values[column] : 0.0f;
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) square_sum = fmaf(value[i], value[i], square_sum);
    }
    partials[threadIdx.x] = square_sum;
    __syncthreads();
    for (int stride = kRmsThreads / 2; stride > 0; stride /= 2) {
        if (threadIdx.x < static_cast<unsigned>(stride)) {
            partials[threadIdx.x] += partials[threadIdx.x + stride];
        }
        __syncthreads();
    }
    const float result = 1.0f / sqrtf(partials[0] / static_cast<float>(width) + eps);
    __syncthreads();  // partials are reused by the next reduction
    return result;
}

template <bool HANDOFF>
__global__ __launch_bounds__(kRmsThreads) void dual_rms_add_capture_kernel(
    const float* __restrict__ input, NormWeight first_weight,
    const float* __restrict__ residual_input, float* hidden_output, NormWeight second_weight,
    float* normalized_output, float* __restrict__ residual_output, std::int64_t width,
    float first_eps, float second_eps, std::uint8_t* __restrict__ records) {
    __shared__ float partials[kRmsThreads];
    const std::int64_t row = blockIdx.x;
    const float* source = input + row * width;
    const float* residual = residual_input + row * width;
    float* hidden = hidden_output + row * width;
    float* captured = residual_output + row * width;
    float* normalized = normalized_output + row * width;

    const float first_inverse = inverse_rms(source, width, first_eps, partials);
    for (std::int64_t base = threadIdx.x; base < width; base += kBatch * kRmsThreads) {
        float value[kBatch], other[kBatch], scale[kBatch];
        std::int64_t columns[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            columns[i] = min(base + i * kRmsThreads, width - 1);
            value[i] = source[columns[i]];
            other[i] = residual[columns[i]];
        }
        norm_scales(first_weight, columns, scale);
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const std::int64_t column = base + i * kRmsThreads;
            const float sum =
                __fadd_rn(__fmul_rn(__fmul_rn(value[i], first_inverse), scale[i]), other[i]);
            if (column < width) {
                hidden[column] = sum;
                captured[column] = sum;
            }
        }
    }
    __syncthreads();  // every thread reads hidden values other threads wrote

    const float second_inverse = inverse_rms(hidden, width, second_eps, partials);
    for (std::int64_t base = threadIdx.x; base < width; base += kBatch * kRmsThreads) {
        float value[kBatch], scale[kBatch];
        std::int64_t columns[kBatch];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            columns[i] = min(base + i * kRmsThreads, width - 1);
            value[i] = hidden[columns[i]];
        }
        norm_scales(second_weight, columns, scale);
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const std::int64_t column = base + i * kRmsThreads;
            if (column < width) {
                normalized[column] = __fmul_rn(__fmul_rn(value[i], second_inverse), scale[i]);
            }
        }
    }

    if constexpr (HANDOFF) {
        __syncthreads();
        // one wave per 256-value block: the quantizer of the decode kernels
        const int lane = threadIdx.x & 63;
        const int wave = threadIdx.x >> 6;
        const int blocks = static_cast<int>(width >> 8);
        for (int block = wave; block < blocks; block += kRmsThreads / kWave) {
            const float4 x = *reinterpret_cast<const float4*>(normalized + block * 256 + lane * 4);
            store_record(records + static_cast<std::int64_t>(block) * kActRecord, lane,
                         encode_activations(x));
        }
    }
}

// Rows of up to 8192 columns: one workgroup of 1024 threads per row.  The sums
// keep the 256-thread order above (sum t adds the squares of columns t, t + 256,
// ... one after another, then the halving tree), but the loads are spread over
// four threads per sum: thread (q, t) loads columns t + 256 * (q + 4k) of every
// operand, eight per operand, so that all loads of the kernel are in flight at
// once (one thread per sum would have 104 outstanding where the hardware counts
// 63), hands its values to thread (0, t) through LDS for the ordered sum, and
// does the element-wise arithmetic of its own columns.  The second
// normalisation needs no second pass over memory.  Same arithmetic, same order,
// same bits as the kernel above.
constexpr int kOwned = kRmsOwned;
constexpr int kLoaders = 4;     // threads that share the loads of a sum
constexpr int kWideThreads = kRmsThreads * kLoaders;
constexpr int kLoaded = kOwned / kLoaders;  // columns per thread

// HANDOFF 0: nothing more; 1: the activation records of the normalized row (one row);
// 2: the normalized rows as the fp16 image of the fp16 small-batch kernel, `records` being
// the small-batch workspace of gridDim.x rows; 3: the activation records of gridDim.x rows
// (token by token) and, at `operand_image`, the same codes in matrix-operand order: what
// the exact verifier's quantizer launch leaves for its matrix-core kernel (gemv_rows.hpp).
template <int HANDOFF>
__global__ __launch_bounds__(kWideThreads) void dual_rms_resident_kernel(
    const float* __restrict__ input, NormWeight first_weight,
    const float* __restrict__ residual_input, float* __restrict__ hidden_output,
    NormWeight second_weight, float* __restrict__ normalized_output,
    float* __restrict__ residual_output, int width, float first_eps, float second_eps,
    std::uint8_t* __restrict__ records, std::uint8_t* __restrict__ operand_image) {
    __shared__ float partials[kRmsThreads + 1];
    __shared__ __attribute__((aligned(16))) float handed[kOwned * kRmsThreads];  // [k][t]: column t + 256 k
    extern __shared__ __attribute__((aligned(16))) float staged[];  // HANDOFF 1, 3: the normalized row
    __shared__ float share_factor[kHalfImageShares];  // HANDOFF 2: what a share's columns are multiplied by
    const std::int64_t row = blockIdx.x;
    const float* source = input + row * width;
    const float* residual = residual_input + row * width;
    float* hidden = hidden_output + row * width;
    float* captured = residual_output + row * width;
    float* normalized = normalized_output + row * width;
    const int t = threadIdx.x & (kRmsThreads - 1);
    const int q = threadIdx.x / kRmsThreads;

    float value[kLoaded], other[kLoaded], first_scale[kLoaded], second_scale[kLoaded];
    int clamped[kLoaded];
#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + kLoaders * i) * kRmsThreads;
        clamped[i] = min(column, width - 1);
        value[i] = column < width ? source[clamped[i]] : 0.0f;
        other[i] = residual[clamped[i]];
    }
    norm_scales(first_weight, clamped, first_scale);
    norm_scales(second_weight, clamped, second_scale);

    // sum t over its columns in order (a column past the end contributes fma(0, 0, sum) = sum)
    auto ordered_sum = [&]() {
        float square_sum = 0.0f;
        if (q == 0) {
#pragma unroll
            for (int k = 0; k < kOwned; ++k) {
                const float v = handed[k * kRmsThreads + t];
                square_sum = fmaf(v, v, square_sum);
            }
        }
        return square_sum;
    };

#pragma unroll
    for (int i = 0; i < kLoaded; ++i) handed[(q + kLoaders * i) * kRmsThreads + t] = value[i];
    __syncthreads();
    const float first_inverse =
        1.0f / sqrtf(rms_tree_total(ordered_sum(), partials) / static_cast<float>(width) + first_eps);

#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + kLoaders * i) * kRmsThreads;
        const float sum =
            __fadd_rn(__fmul_rn(__fmul_rn(value[i], first_inverse), first_scale[i]), other[i]);
        value[i] = column < width ? sum : 0.0f;
        if (column < width) {
            hidden[column] = sum;
            captured[column] = sum;
        }
        // every sum has read its old values: tree_total_wide's barriers lie in between
        handed[(q + kLoaders * i) * kRmsThreads + t] = value[i];
    }
    __syncthreads();
    const float second_inverse =
        1.0f / sqrtf(rms_tree_total(ordered_sum(), partials) / static_cast<float>(width) + second_eps);

#pragma unroll
    for (int i = 0; i < kLoaded; ++i) {
        const int column = t + (q + kLoaders * i) * kRmsThreads;
        const float result = __fmul_rn(__fmul_rn(value[i], second_inverse), second_scale[i]);
        if (column < width) {
            normalized[column] = result;
            if constexpr (HANDOFF == 1 || HANDOFF == 3) staged[column] = result;
            // (the sums have read `handed`: tree_total_wide's barriers lie in between)
            if constexpr (HANDOFF == 2) handed[column] = result;
        }
    }

    if constexpr (HANDOFF == 2) {
        // what f16_image_kernel would make of the normalized row, bit for bit: every K share of
        // the row (f16_decode.hpp) with the scale of its own largest magnitude
        static_assert(kWideThreads / kWave >= kHalfImageShares, "a wave per share");
        __syncthreads();  // the row is in `handed`
        const int rows = static_cast<int>(gridDim.x);
        const int blocks = width >> 8;
        float* inverse_scale =
            reinterpret_cast<float*>(records + static_cast<std::int64_t>(rows) * width * 2);
        const int share = threadIdx.x >> 6;
        if (share < kHalfImageShares) {
            const int end = 256 * half_image_share_begin(blocks, share + 1);
            float share_largest = 0.0f;
            for (int column = 256 * half_image_share_begin(blocks, share) + (threadIdx.x & 63); column < end;
                 column += kWave) {
                share_largest = fmaxf(share_largest, fabsf(handed[column]));
            }
#pragma unroll
            for (int offset = 32; offset > 0; offset >>= 1) {
                share_largest = fmaxf(share_largest, __shfl_xor(share_largest, offset));
            }
            const HalfImageScale scale = half_image_scale(share_largest);
            if ((threadIdx.x & 63) == 0) {
                share_factor[share] = scale.factor;
                inverse_scale[row * kHalfImageShares + share] = scale.inverse;
            }
        }
        __syncthreads();
        for (int group = threadIdx.x; group < (width >> 3); group += kWideThreads) {
            half_image_store(records, group, rows, static_cast<int>(row),
                             *reinterpret_cast<const float4*>(handed + group * 8),
                             *reinterpret_cast<const float4*>(handed + group * 8 + 4),
                             share_factor[half_image_share_of(group >> 5, blocks)]);
        }
    }

    if constexpr (HANDOFF == 1 || HANDOFF == 3) {
        __syncthreads();
        // one wave per 256-value block: the quantizer of the decode kernels
        const int lane = threadIdx.x & 63;
        const int wave = threadIdx.x >> 6;
        const int blocks = width >> 8;
        for (int block = wave; block < blocks; block += kWideThreads / kWave) {
            const float4 x = *reinterpret_cast<const float4*>(staged + block * 256 + lane * 4);
            const ActivationCodes codes = encode_activations(x);
            if constexpr (HANDOFF == 3) {
                store_record(records + (row * blocks + block) * kActRecord, lane, codes);
                store_operand_image(operand_image, block, static_cast<int>(row),
                                    static_cast<int>(gridDim.x), lane, codes);
            } else {
                store_record(records + static_cast<std::int64_t>(block) * kActRecord, lane, codes);
            }
        }
    }
}

// ---- one normalisation: output = rms(input, weight, eps) [+ residual_input],
// optionally a copy of the input (the residual the caller keeps) and the
// public Q8_1 form of the output
// (neuralfn/csrc/tile_cuda/kernels.cu:2065-2153).  Same reduction order as
// above; the Q8_1 values are those of the standalone quantizer run on the
// output, computed in registers: 32 consecutive threads hold 32 consecutive
// columns, one Q8_1 block.

struct Q8_1Outputs {
    std::int8_t* codes;
    float* scales;
    float* sums;
};

__device__ __forceinline__ void store_q8_1(const Q8_1Outputs& q8, std::int64_t index, float value,
                                           bool inside) {
    // all 32 lanes of a block are inside or outside together (width % 32 == 0)
    const Q8_1Value quantized = quantize_q8_1_value(inside ? value : 0.0f);
    if (inside) {
        q8.codes[index] = quantized.code;
        if ((threadIdx.x & 31) == 0) {
            q8.scales[index >> 5] = quantized.scale;
            q8.sums[index >> 5] = quantized.sum;
        }
    }
}

template <bool ADD, bool Q8>
__global__ __launch_bounds__(kRmsThreads) void rms_resident_kernel(
    const float* __restrict__ input, NormWeight weight, const float* __restrict__ residual_input,
    float* __restrict__ output, float* __restrict__ residual_output, int width, float eps,
    Q8_1Outputs q8) {
    __shared__ float partials[kRmsThreads];
    const std::int64_t row = blockIdx.x;
    const float* source = input + row * width;
    float value[kOwned], other[kOwned], scale[kOwned];
    int clamped[kOwned];
#pragma unroll
    for (int i = 0; i < kOwned; ++i) {
        const int column = threadIdx.x + i * kRmsThreads;
        clamped[i] = min(column, width - 1);
        value[i] = column < width ? source[clamped[i]] : 0.0f;
        other[i] = ADD ? residual_input[row * width + clamped[i]] : 0.0f;
    }
    norm_scales(weight, clamped, scale);
    float square_sum = 0.0f;
#pragma unroll
    for (int i = 0; i < kOwned; ++i) square_sum = fmaf(value[i], value[i], square_sum);
    const float inverse =
        1.0f / sqrtf(rms_tree_total(square_sum, partials) / static_cast<float>(width) + eps);
#pragma unroll
    for (int i = 0; i < kOwned; ++i) {
        const int column = threadIdx.x + i * kRmsThreads;
        const bool inside = column < width;
        const std::int64_t index = row * width + column;
        float result = __fmul_rn(__fmul_rn(value[i], inverse), scale[i]);
        if constexpr (ADD) result = __fadd_rn(result, other[i]);
        if (inside) {
            output[index] = result;
            if (residual_output != nullptr) residual_output[index] = value[i];
        }
        if constexpr (Q8) {
            if (i * kRmsThreads < width) store_q8_1(q8, index, result, inside);
        }
    }
}

template <bool ADD, bool Q8>
__global__ __launch_bounds__(kRmsThreads) void rms_wide_kernel(
    const float* __restrict__ input, NormWeight weight, const float* __restrict__ residual_input,
    float* __restrict__ output, float* __restrict__ residual_output, std::int64_t width, float eps,
    Q8_1Outputs q8) {
    __shared__ float partials[kRmsThreads];
    const std::int64_t row = blockIdx.x;
    const float* source = input + row * width;
    const float inverse = inverse_rms(source, width, eps, partials);
    // the loop runs the same number of times in every thread of a 32-lane block
    for (std::int64_t base = threadIdx.x & ~31; base < width; base += kRmsThreads) {
        const std::int64_t column = base + (threadIdx.x & 31);
        const bool inside = column < width;  // true for the whole block: width % 32 == 0 with Q8
        const std::int64_t clamped = inside ? column : width - 1;
        const std::int64_t index = row * width + column;
        const float loaded = source[clamped];
        float result = __fmul_rn(__fmul_rn(loaded, inverse), norm_scale(weight, clamped));
        if constexpr (ADD) result = __fadd_rn(result, residual_input[row * width + clamped]);
        if (inside) {
            output[index] = result;
            if (residual_output != nullptr) residual_output[index] = loaded;
        }
        if constexpr (Q8) store_q8_1(q8, index, result, inside);
    }
}

// Where the fused decode step also leaves the new key and value row (bf16 ring
// caches); key_cache null = no commit.
struct CacheRow {
    std::uint16_t* key_cache;
    std::uint16_t* value_cache;
    const float* values;  // [kv_heads, head_dim], the current value row
    std::int64_t capacity;
    std::int64_t row_stride;
};

// ---- per-head Q/K normalisation, query scale and rotary embedding in one launch
// (neuralfn/csrc/native_train/tile_ops.h:905-943; reference kernel
// neuralfn/csrc/tile_cuda/kernels.cu:2381-2473).  One workgroup per (row, head);
// a thread owns one column.  Each step is the arithmetic of the separate
// operator it replaces, in the same order (rms_resident_kernel at width =
// head_dim, the in-place scale, the rotary kernel), so the result equals the
// three calls bit for bit.  For the fused decode step the key heads' workgroups
// also write the bf16 cache row of the new key and value (the row a one-token
// attention at this position never reads).
__global__ __launch_bounds__(kRmsThreads) void qk_norm_scale_rope_kernel(
    float* __restrict__ query, float* __restrict__ key, NormWeight query_weight,
    NormWeight key_weight, int query_heads, int kv_heads, int head_dim, float eps,
    float query_scale, std::int64_t position, const std::int64_t* __restrict__ device_position,
    double theta, bool interleaved, bool apply_rope, CacheRow commit) {
    __shared__ float partials[kRmsThreads];
    __shared__ float normalized[kRmsThreads];
    if (device_position != nullptr) position = device_position[0];
    const int heads_per_row = query_heads + kv_heads;
    const int row = blockIdx.x / heads_per_row;
    const int combined = blockIdx.x - row * heads_per_row;
    const bool is_query = combined < query_heads;
    float* values = is_query
        ? query + (static_cast<std::int64_t>(row) * query_heads + combined) * head_dim
        : key + (static_cast<std::int64_t>(row) * kv_heads + combined - query_heads) * head_dim;
    const int column = threadIdx.x;
    const bool inside = column < head_dim;
    const int clamped[1] = {inside ? column : head_dim - 1};
    const float value = inside ? values[clamped[0]] : 0.0f;
    float scale[1];
    norm_scales(is_query ? query_weight : key_weight, clamped, scale);
    // the rotation's angle depends on the position alone: worked out while the loads above
    // are in flight (an empty asm keeps the compiler from moving it behind the reduction)
    RopeAngle angle{0.0, 1.0};
    if (apply_rope && column < head_dim / 2) {
        angle = rope_angle(position + row, column, head_dim, theta, false);
        asm volatile("" : "+v"(angle.sine), "+v"(angle.cosine));
    }
    const float inverse = 1.0f / sqrtf(rms_tree_total(fmaf(value, value, 0.0f), partials) /
                                           static_cast<float>(head_dim) + eps);
    float result = __fmul_rn(__fmul_rn(value, inverse), scale[0]);
    if (is_query) result = __fmul_rn(result, query_scale);
    // a key head also goes to the cache (one row only), with its value head
    const bool commits = !is_query && commit.key_cache != nullptr;
    const std::int64_t cache_index = commits
        ? (position % commit.capacity) * commit.row_stride +
            static_cast<std::int64_t>(combined - query_heads) * head_dim
        : 0;
    if (commits && inside) {
        commit.value_cache[cache_index + column] =
            to_bf16(commit.values[static_cast<std::int64_t>(combined - query_heads) * head_dim + column]);
    }
    if (!apply_rope) {
        if (inside) {
            values[column] = result;
            if (commits) commit.key_cache[cache_index + column] = to_bf16(result);
        }
        return;
    }
    normalized[column] = result;
    __syncthreads();
    const int half = head_dim / 2;
    if (column < half) {
        const int first = interleaved ? 2 * column : column;
        const int second = interleaved ? 2 * column + 1 : column + half;
        float a = normalized[first], b = normalized[second];
        rope_apply(a, b, angle);
        values[first] = a;
        values[second] = b;
        if (commits) {
            commit.key_cache[cache_index + first] = to_bf16(a);
            commit.key_cache[cache_index + second] = to_bf16(b);
        }
    }
}


}  // namespace

void launch_dual_rms_add_capture(const float* input, const Descriptor* first_weight,
                                 bool first_centered, const float* residual_input,
                                 float* hidden_output, const Descriptor* second_weight,
                                 bool second_centered, float* normalized_output,
                                 float* residual_output, std::int64_t rows, std::int64_t width,
                                 float first_eps, float second_eps, std::uint8_t* records,
                                 std::uint8_t* half_image, hipStream_t stream,
                                 std::uint8_t* operand_image) {
    const NormWeight first = norm_weight(first_weight, first_centered);
    const NormWeight second = norm_weight(second_weight, second_centered);
    const dim3 grid(static_cast<unsigned>(rows));
    if (width <= kOwned * kRmsThreads) {
        const int columns = static_cast<int>(width);
        std::uint8_t* const none = nullptr;
        if (half_image != nullptr) {
            hipLaunchKernelGGL((dual_rms_resident_kernel<2>), grid, dim3(kWideThreads), 0, stream, input,
                               first, residual_input, hidden_output, second, normalized_output,
                               residual_output, columns, first_eps, second_eps, half_image, none);
        } else if (records != nullptr && operand_image != nullptr) {
            hipLaunchKernelGGL((dual_rms_resident_kernel<3>), grid, dim3(kWideThreads),
                               static_cast<std::size_t>(columns) * sizeof(float), stream, input,
                               first, residual_input, hidden_output, second, normalized_output,
                               residual_output, columns, first_eps, second_eps, records,
                               operand_image);
        } else if (records != nullptr) {
            hipLaunchKernelGGL((dual_rms_resident_kernel<1>), grid, dim3(kWideThreads),
                               static_cast<std::size_t>(columns) * sizeof(float), stream, input,
                               first, residual_input, hidden_output, second, normalized_output,
                               residual_output, columns, first_eps, second_eps, records, none);
        } else {
            hipLaunchKernelGGL((dual_rms_resident_kernel<0>), grid, dim3(kWideThreads), 0, stream,
                               input, first, residual_input, hidden_output, second,
                               normalized_output, residual_output, columns, first_eps, second_eps,
                               records, none);
        }
        return;
    }
    if (records != nullptr) {
        hipLaunchKernelGGL((dual_rms_add_capture_kernel<true>), grid, dim3(kRmsThreads), 0, stream,
                           input, first, residual_input, hidden_output, second, normalized_output,
                           residual_output, width, first_eps, second_eps, records);
    } else {
        hipLaunchKernelGGL((dual_rms_add_capture_kernel<false>), grid, dim3(kRmsThreads), 0, stream,
                           input, first, residual_input, hidden_output, second, normalized_output,
                           residual_output, width, first_eps, second_eps, records);
    }
}

template <bool ADD, bool Q8>
static void launch_rms_variant(const float* input, const NormWeight& weight,
                               const float* residual_input, float* output, float* residual_output,
                               std::int64_t rows, std::int64_t width, float eps,
                               const Q8_1Outputs& q8, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>(rows));
    if (width <= kOwned * kRmsThreads) {
        hipLaunchKernelGGL((rms_resident_kernel<ADD, Q8>), grid, dim3(kRmsThreads), 0, stream, input,
                           weight, residual_input, output, residual_output,
                           static_cast<int>(width), eps, q8);
    } else {
        hipLaunchKernelGGL((rms_wide_kernel<ADD, Q8>), grid, dim3(kRmsThreads), 0, stream, input,
                           weight, residual_input, output, residual_output, width, eps, q8);
    }
}

void launch_rms_norm(const float* input, const Descriptor* weight, bool centered,
                     const float* residual_input, float* output, float* residual_output,
                     std::int8_t* q8_codes, float* q8_scales, float* q8_sums, std::int64_t rows,
                     std::int64_t width, float eps, hipStream_t stream) {
    const NormWeight scale = norm_weight(weight, centered);
    const Q8_1Outputs q8{q8_codes, q8_scales, q8_sums};
    const bool add = residual_input != nullptr;
    if (q8_codes != nullptr) {
        if (add) {
            launch_rms_variant<true, true>(input, scale, residual_input, output, residual_output,
                                           rows, width, eps, q8, stream);
        } else {
            launch_rms_variant<false, true>(input, scale, residual_input, output, residual_output,
                                            rows, width, eps, q8, stream);
        }
    } else if (add) {
        launch_rms_variant<true, false>(input, scale, residual_input, output, residual_output, rows,
                                        width, eps, q8, stream);
    } else {
        launch_rms_variant<false, false>(input, scale, residual_input, output, residual_output, rows,
                                         width, eps, q8, stream);
    }
}

void launch_qk_norm_scale_rope(float* query, float* key, const Descriptor* query_weight,
                               bool query_centered, const Descriptor* key_weight,
                               bool key_centered, std::int64_t rows, std::int64_t query_heads,
                               std::int64_t kv_heads, std::int64_t head_dim, float eps,
                               float query_scale, std::int64_t position,
                               const std::int64_t* device_position, float theta,
                               bool interleaved, bool apply_rope, std::uint16_t* key_cache,
                               std::uint16_t* value_cache, const float* current_value,
                               std::int64_t cache_capacity, std::int64_t cache_row_stride,
                               hipStream_t stream) {
    const CacheRow commit{key_cache, value_cache, current_value, cache_capacity, cache_row_stride};
    hipLaunchKernelGGL(qk_norm_scale_rope_kernel,
                       dim3(static_cast<unsigned>(rows * (query_heads + kv_heads))),
                       dim3(kRmsThreads), 0, stream, query, key,
                       norm_weight(query_weight, query_centered),
                       norm_weight(key_weight, key_centered), static_cast<int>(query_heads),
                       static_cast<int>(kv_heads), static_cast<int>(head_dim), eps, query_scale,
                       position, device_position, static_cast<double>(theta), interleaved,
                       apply_rope, commit);
}

}  // namespace nfn
