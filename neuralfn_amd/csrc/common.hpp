// Shared host/device definitions for the MI355X K-Quant packed-linear library.
//
// Formats follow ggml's block layouts as the reference states them
// (neuralfn/csrc/tile_cuda/vendor/llama_mmq_62bf73d/ggml/src/ggml-common.h:251-368)
// and the per-weight arithmetic of the reference's CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616), with the canonical
// Q6_K sub-scale index (neuralfn/csrc/tile_cuda/kernels.cu:1320).
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdint>

#include "../../include/nfn_mi355_tile_ops.h"

namespace nfn {

constexpr int kInvalid = 1;  // hipErrorInvalidValue; the reference returns cudaErrorInvalidValue (1)
constexpr int kWave = 64;

enum : std::uint32_t {
    kEncF32 = NFN_NATIVE_TILE_PACKED_WEIGHT_F32,
    kEncQ8_0 = NFN_MI355_PACKED_WEIGHT_Q8_0,
    kEncQ4K = NFN_NATIVE_TILE_PACKED_WEIGHT_Q4_K,
    kEncQ5K = NFN_NATIVE_TILE_PACKED_WEIGHT_Q5_K,
    kEncQ6K = NFN_NATIVE_TILE_PACKED_WEIGHT_Q6_K,
    kEncBF16 = NFN_NATIVE_TILE_PACKED_WEIGHT_BF16,
};

using Descriptor = NfnNativeTilePackedWeightDescriptorV1;

__host__ __device__ constexpr std::int64_t block_bytes(std::uint32_t encoding) {
    switch (encoding) {
        case kEncF32: return 4;
        case kEncBF16: return 2;
        case kEncQ8_0: return 34;
        case kEncQ4K: return 144;
        case kEncQ5K: return 176;
        case kEncQ6K: return 210;
        default: return 0;
    }
}

__host__ __device__ constexpr std::int64_t block_elements(std::uint32_t encoding) {
    switch (encoding) {
        case kEncF32: case kEncBF16: return 1;
        case kEncQ8_0: return 32;
        case kEncQ4K: case kEncQ5K: case kEncQ6K: return 256;
        default: return 0;
    }
}

__host__ __device__ constexpr bool is_k_quant(std::uint32_t encoding) {
    return encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K;
}

// Host-side checks (descriptor.cpp).
bool normalize_descriptor(const Descriptor* source, Descriptor* output);
bool validate_k_descriptor(const Descriptor* descriptor, std::int64_t input_dim,
                           void* stream, bool allow_q8_0);

// Compute units of the current device (256 on MI355X), cached.
constexpr int kMaxDevices = 64;

// The current device's index, 0 if it cannot be told or is beyond the tables below.
inline int current_device() {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= kMaxDevices) return 0;
    return device;
}

inline int compute_units() {
    static std::atomic<int> counts[kMaxDevices];  // 0 = not asked yet
    const int device = current_device();
    int count = counts[device].load(std::memory_order_relaxed);
    if (count == 0) {
        if (hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
            count <= 0) {
            count = 256;
        }
        counts[device].store(count, std::memory_order_relaxed);
    }
    return count;
}

// More than 64 KB of dynamic LDS has to be allowed once per kernel and device.
template <auto Kernel>
inline void allow_large_lds(int bytes = 160 * 1024) {
    static std::atomic<std::uint64_t> allowed{0};  // one bit per device
    const std::uint64_t bit = std::uint64_t(1) << current_device();
    if ((allowed.load(std::memory_order_acquire) & bit) != 0) return;
    if (hipFuncSetAttribute(reinterpret_cast<const void*>(Kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, bytes) == hipSuccess) {
        allowed.fetch_or(bit, std::memory_order_release);
    }
}

inline hipStream_t as_stream(void* stream) { return reinterpret_cast<hipStream_t>(stream); }
inline int launch_status() { return static_cast<int>(hipPeekAtLastError()); }

// What one projection of a multi-projection launch needs on the device.
struct Projection {
    const std::uint8_t* data;
    float* output;
    std::int64_t output_dim;
    std::int64_t row_stride;
    std::uint32_t encoding;
    std::uint32_t first_tile;  // first tile index of this projection in the launch
};

struct ProjectionSet {
    Projection op[4];
    int count;
    std::int64_t input_dim;
};

// Activation prologues of the fused entry points (glimmer_k_mmq.cu:299-317).
// kRecords is not a prologue of the floats: the input pointer holds activation
// records that an earlier launch quantized (the prequantized entry point,
// neuralfn/csrc/native_train/tile_ops.h:698-709).  kHalfImage likewise: the fp16 image of
// the fp16 small-batch kernel already lies in the workspace (written by the dual RMS kernel).
// kDualNorm: the input is the result of the two normalisations of a layer's input, which the
// decode kernel computes in its own prologue (one row).
enum Prologue : int { kPlain = 0, kGated = 1, kSwiGlu = 2, kRecords = 3, kHalfImage = 4, kDualNorm = 5 };

#if defined(__HIPCC__)

__device__ __forceinline__ float half_bits_to_float(std::uint32_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<unsigned short>(bits)));
}

__device__ __forceinline__ float load_half(const std::uint8_t* p) {
    return half_bits_to_float(static_cast<std::uint32_t>(p[0]) | (static_cast<std::uint32_t>(p[1]) << 8));
}

// float -> bf16 bits, round to nearest even; a NaN stays a NaN.
__device__ __forceinline__ std::uint16_t to_bf16(float value) {
    const std::uint32_t bits = __float_as_uint(value);
    if ((bits & 0x7fffffffu) > 0x7f800000u) {
        return static_cast<std::uint16_t>((bits >> 16) | 0x40u);
    }
    const std::uint32_t rounding = 0x7fffu + ((bits >> 16) & 1u);
    return static_cast<std::uint16_t>((bits + rounding) >> 16);
}

__device__ __forceinline__ float bf16_to_float(std::uint32_t bits) {
    return __uint_as_float(bits << 16);
}

// One rotary pair at `position`: angle = position / theta^(2*pair/head_dim) in
// double, [a, b] -> [a cos - b sin, b cos + a sin]
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:773-800).
// (in two steps, so that a kernel can work out the angle's sine and cosine -- a few hundred
// double-precision instructions that depend on the position only -- while its loads are in flight)
struct RopeAngle {
    double sine, cosine;
};

__device__ __forceinline__ RopeAngle rope_angle(std::int64_t position, std::int64_t pair,
                                                std::int64_t head_dim, double theta, bool inverse) {
    const double inverse_frequency =
        1.0 / pow(theta, static_cast<double>(2 * pair) / static_cast<double>(head_dim));
    double angle = static_cast<double>(position) * inverse_frequency;
    if (inverse) angle = -angle;
    RopeAngle result;
    sincos(angle, &result.sine, &result.cosine);
    return result;
}

__device__ __forceinline__ void rope_apply(float& first, float& second, const RopeAngle& angle) {
    const float lhs = first;
    const float rhs = second;
    first = static_cast<float>(lhs * angle.cosine - rhs * angle.sine);
    second = static_cast<float>(rhs * angle.cosine + lhs * angle.sine);
}

__device__ __forceinline__ void rope_rotate(float& first, float& second, std::int64_t position,
                                            std::int64_t pair, std::int64_t head_dim, double theta,
                                            bool inverse) {
    rope_apply(first, second, rope_angle(position, pair, head_dim, theta, inverse));
}

// 6-bit scale and minimum of sub-block `index` (resident_glimmer.cpp:178-186).
__device__ __forceinline__ void k_scale_min(const std::uint8_t* scales, int index,
                                            int* scale, int* minimum) {
    if (index < 4) {
        *scale = scales[index] & 63;
        *minimum = scales[index + 4] & 63;
        return;
    }
    *scale = (scales[index + 4] & 0x0f) | ((scales[index - 4] >> 6) << 4);
    *minimum = (scales[index + 4] >> 4) | ((scales[index] >> 6) << 4);
}

// 1 / (1 + exp(-x)) from the hardware's exp2 and reciprocal: the product x log2(e) keeps
// its rounding error as a correction term and the reciprocal takes one Newton step, which
// leaves about one unit in the last place; a sixth of the instructions of expf and an IEEE
// division, which a decode launch with a 16,384-column SwiGLU prologue spends on nothing
// else (SwiGLU down projection of 16,384 columns: 17.1 -> 15.7 us).  Above 88.5 the
// result is 1; below -88.5 it is 0, as where expf overflows (so that x sigmoid(x) goes to
// zero and not to x times a tiny number).
__device__ __forceinline__ float sigmoid(float x) {
    constexpr float kLog2e = 1.4426950408889634f;
    constexpr float kLn2 = 0.6931471805599453f;
    const float bounded = __builtin_amdgcn_fmed3f(x, -88.5f, 88.5f);
    const float scaled = -bounded * kLog2e;
    const float rest = fmaf(-bounded, kLog2e, -scaled);  // exact remainder of the product
    float power = __builtin_amdgcn_exp2f(scaled);
    power = fmaf(power * kLn2, rest, power);
    const float sum = 1.0f + power;
    float inverse = __builtin_amdgcn_rcpf(sum);
    inverse = fmaf(fmaf(-sum, inverse, 1.0f), inverse, inverse);
    const float result = x < -88.5f ? 0.0f : inverse;
    return x != x ? x : result;
}

// fused activation prologue; `first`/`second` follow the entry points'
// argument order: gated (input, gate), swiglu (gate, up).
template <int P>
__device__ __forceinline__ float apply_prologue(float first, float second) {
    if constexpr (P == kGated) {
        return first * sigmoid(second);
    } else if constexpr (P == kSwiGlu) {
        return (second * first) * sigmoid(first);
    } else {
        return first;
    }
}

// One weight, decoded from scratch: the slow, obviously-right form used by the
// dequantize entry point and by encodings without a tuned kernel.
__device__ __forceinline__ float weight_value(std::uint32_t encoding,
                                              const std::uint8_t* row_data,
                                              std::int64_t col) {
    if (encoding == kEncF32) {
        return reinterpret_cast<const float*>(row_data)[col];
    }
    if (encoding == kEncBF16) {
        const std::uint32_t bits = reinterpret_cast<const std::uint16_t*>(row_data)[col];
        return __uint_as_float(bits << 16);
    }
    if (encoding == kEncQ8_0) {
        const std::uint8_t* block = row_data + (col / 32) * 34;
        const int quant = static_cast<std::int8_t>(block[2 + (col & 31)]);
        return load_half(block) * static_cast<float>(quant);
    }
    const std::int64_t block_index = col >> 8;
    const int within = static_cast<int>(col & 255);
    if (encoding == kEncQ4K || encoding == kEncQ5K) {
        const bool q5 = encoding == kEncQ5K;
        const std::uint8_t* block = row_data + block_index * (q5 ? 176 : 144);
        const float d = load_half(block);
        const float dmin = load_half(block + 2);
        const int group = within >> 6;
        const int lane = within & 31;
        const bool high = (within & 32) != 0;
        int scale, minimum;
        k_scale_min(block + 4, group * 2 + (high ? 1 : 0), &scale, &minimum);
        const std::uint8_t packed = block[(q5 ? 48 : 16) + group * 32 + lane];
        int quant = high ? (packed >> 4) : (packed & 0x0f);
        if (q5) {
            const int mask = (high ? 2 : 1) << (2 * group);
            quant += (block[16 + lane] & mask) ? 16 : 0;
        }
        // Two roundings and a subtraction, never an FMA: the CPU engine's form.
        return __fsub_rn(__fmul_rn(d, static_cast<float>(scale * quant)),
                         __fmul_rn(dmin, static_cast<float>(minimum)));
    }
    const std::uint8_t* block = row_data + block_index * 210;
    const int half = within >> 7;
    const int position = within & 127;
    const int quarter = position >> 5;
    const int lane = position & 31;
    const std::uint8_t low = block[half * 64 + lane + ((quarter & 1) ? 32 : 0)];
    const std::uint8_t high = block[128 + half * 32 + lane];
    const int nibble = quarter < 2 ? (low & 0x0f) : (low >> 4);
    const int quant = (nibble | (((high >> (2 * quarter)) & 3) << 4)) - 32;
    const int scale = static_cast<std::int8_t>(block[192 + half * 8 + quarter * 2 + (lane >> 4)]);
    return __fmul_rn(__fmul_rn(load_half(block + 208), static_cast<float>(scale)),
                     static_cast<float>(quant));
}

// One value of a 32-value Q8_1 block held by 32 consecutive lanes
// (neuralfn/csrc/tile_cuda/kernels.cu:1527-1562): code = round(x * 127 / max)
// clamped to +-127, scale = 1 / (127 / max), sum = the block's float sum
// (butterfly order).  Scale and sum are the same in all 32 lanes.
struct Q8_1Value {
    std::int8_t code;
    float scale, sum;
};

__device__ __forceinline__ Q8_1Value quantize_q8_1_value(float value) {
    float maximum = fabsf(value);
    float sum = value;
#pragma unroll
    for (int offset = 16; offset > 0; offset >>= 1) {
        maximum = fmaxf(maximum, __shfl_xor(maximum, offset, 32));
        sum += __shfl_xor(sum, offset, 32);
    }
    const float inverse = maximum > 0.0f ? 127.0f / maximum : 0.0f;
    Q8_1Value result;
    result.scale = inverse > 0.0f ? 1.0f / inverse : 0.0f;
    int code = inverse > 0.0f ? static_cast<int>(roundf(value * inverse)) : 0;
    code = max(-127, min(127, code));
    result.code = static_cast<std::int8_t>(code);
    result.sum = sum;
    return result;
}

__device__ __forceinline__ float wave_sum(float value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        value += __shfl_xor(value, offset, 64);
    }
    return value;
}

// 16 bytes per lane from `source` (this lane's) to the LDS address `target` (uniform) + 16 x
// lane; counted by vmcnt like any load.  Written out as an instruction because the compiler
// holds every later LDS read back until all loads of this kind have landed, which would leave
// its ring of stages one deep; the kernels that use it wait by count themselves.
__device__ __forceinline__ void load_to_lds(const __attribute__((address_space(1))) std::uint8_t* source,
                                            std::uint8_t* target) {
    const std::uint32_t lds_address = static_cast<std::uint32_t>(
        reinterpret_cast<std::uintptr_t>((__attribute__((address_space(3))) std::uint8_t*)target));
    // (m0 carries the LDS address; it is put back, the compiler keeps no account of it)
    std::uint32_t kept;
    asm volatile(
        "s_mov_b32 %0, m0\n\ts_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off\n\ts_mov_b32 m0, %0"
        : "=&s"(kept)
        : "v"(source), "s"(lds_address)
        : "memory");
}

#endif  // __HIPCC__

}  // namespace nfn
