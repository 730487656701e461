// Float matrix-core GEMM: the exact tier at more than 16 input rows.
//
// nfn_native_tile_linear_packed_weight_float32_v1 has no workspace argument
// (neuralfn/csrc/native_train/tile_ops.h:614-620; reference kernel
// neuralfn/csrc/tile_cuda/kernels.cu:26943-26983), so the fp16 GEMM, which needs a
// scaled fp16 copy of the activations, cannot serve it.  This kernel keeps the
// float kernel's arithmetic instead: every weight is decoded by weight_value()
// (the CPU engine's two roundings and a subtraction,
// neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616), the activations stay
// float, and the products run on v_mfma_f32_32x32x2_f32, float in and float out.
// Only the order of the float additions differs from gemv_f32.hip.  The float
// matrix instruction runs at 256 flop per cycle and compute unit, a sixteenth of
// the fp16 one: 157 TFLOP/s for the chip, which is what bounds this kernel.
//
// A workgroup of four waves owns 128 input rows x 64 weight rows.  Per stage of
// 32 columns every thread loads 16 activations and the packed bytes of 8 weights
// two stages ahead, decodes the weights one stage ahead and writes both into LDS
// (rows padded to 36 floats); a wave (64 x 32 outputs, two accumulators) reads
// four values per operand row and 8 columns, which feed four instructions each:
// the instruction's k index is only a pairing of the two operands' elements, so
// the lower half of the wave takes columns 0..3 of the eight and the upper half
// 4..7.  One LDS stage and two barriers per 32 columns: 27 KB per workgroup, so
// that four workgroups share a compute unit and their loads, decoding and
// barriers run under one another's products (measured against two workgroups
// with two LDS stages: 916 against 955 us at 512 x 6,656 -> 16,384, Q4_K).
#include <type_traits>

#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

constexpr int kTileRows = 128;
constexpr int kTileCols = 64;
constexpr int kStage = 32;
constexpr int kPitch = kStage + 4;

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4_unaligned __attribute__((ext_vector_type(4), aligned(4)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef std::uint32_t u32x2_a2 __attribute__((ext_vector_type(2), aligned(2)));
typedef std::uint32_t u32x4_a4 __attribute__((ext_vector_type(4), aligned(4)));

__device__ __forceinline__ int byte_of(std::uint32_t low, std::uint32_t high, int index) {
    return static_cast<int>(((index & 4) ? high : low) >> (8 * (index & 3))) & 255;
}

// The packed bytes behind eight consecutive weights of one row (columns 32 stage + 8 part ..),
// loaded in one go and decoded a stage later.  decode() is weight_value()'s arithmetic with
// the parts that the eight weights share taken once.
template <std::uint32_t ENC>
struct EightOfQ4KOrQ5K {
    u32x4_a4 header;  // d, dmin, the twelve scale bytes
    u32x2_a2 codes, fifth;
    __device__ __forceinline__ void load(const std::uint8_t* row, std::int64_t stage, int part) {
        const std::uint8_t* block = row + (stage >> 3) * block_bytes(ENC);
        const int group = static_cast<int>(stage & 7) >> 1;
        header = *reinterpret_cast<const u32x4_a4*>(block);
        codes = *reinterpret_cast<const u32x2_a2*>(block + (ENC == kEncQ5K ? 48 : 16) + group * 32 +
                                                   part * 8);
        if constexpr (ENC == kEncQ5K) {
            fifth = *reinterpret_cast<const u32x2_a2*>(block + 16 + part * 8);
        }
    }
    __device__ __forceinline__ void decode(std::int64_t stage, float (&out)[8]) const {
        const int sub = static_cast<int>(stage & 7);
        const float d = half_bits_to_float(header.x & 0xffffu);
        const float dmin = half_bits_to_float(header.x >> 16);
        // the twelve scale bytes are header.y, .z, .w (k_scale_min's indexing)
        // (masks, not a branch: the decoding has to stay in the block of the matrix products)
        const int y = byte_of(header.y, 0, sub & 3);
        const int z = byte_of(header.z, 0, sub & 3);
        const int w = byte_of(header.w, 0, sub & 3);
        const int upper = -(sub >> 2);
        const int scale = ((y & 63) & ~upper) | (((w & 0x0f) | ((y >> 6) << 4)) & upper);
        const int minimum = ((z & 63) & ~upper) | (((w >> 4) | ((z >> 6) << 4)) & upper);
        const float offset = __fmul_rn(dmin, static_cast<float>(minimum));
        const int nibble_shift = (sub & 1) * 4;
        const int fifth_bit = sub;  // bit 2 group + (high ? 1 : 0) of the row's fifth-bit byte
#pragma unroll
        for (int index = 0; index < 8; ++index) {
            int quant = (byte_of(codes.x, codes.y, index) >> nibble_shift) & 15;
            if constexpr (ENC == kEncQ5K) {
                quant += ((byte_of(fifth.x, fifth.y, index) >> fifth_bit) & 1) << 4;
            }
            out[index] = __fsub_rn(__fmul_rn(d, static_cast<float>(scale * quant)), offset);
        }
    }
};

struct EightOfQ6K {
    u32x2_a2 low, high;
    std::uint32_t scale_and_d;  // low byte: the sub-scale; upper half: d
    __device__ __forceinline__ void load(const std::uint8_t* row, std::int64_t stage, int part) {
        const std::uint8_t* block = row + (stage >> 3) * 210;
        const int sub = static_cast<int>(stage & 7);
        const int half = sub >> 2, quarter = sub & 3;
        low = *reinterpret_cast<const u32x2_a2*>(block + half * 64 + (quarter & 1) * 32 + part * 8);
        high = *reinterpret_cast<const u32x2_a2*>(block + 128 + half * 32 + part * 8);
        const std::uint32_t scale = block[192 + half * 8 + quarter * 2 + (part >> 1)];
        const std::uint32_t d = *reinterpret_cast<const std::uint16_t*>(block + 208);
        scale_and_d = scale | (d << 16);
    }
    __device__ __forceinline__ void decode(std::int64_t stage, float (&out)[8]) const {
        const int quarter = static_cast<int>(stage & 3);
        const int scale = static_cast<std::int8_t>(scale_and_d & 255u);
        const float scaled =
            __fmul_rn(half_bits_to_float(scale_and_d >> 16), static_cast<float>(scale));
        const int nibble_shift = (quarter >> 1) * 4;
#pragma unroll
        for (int index = 0; index < 8; ++index) {
            const int nibble = (byte_of(low.x, low.y, index) >> nibble_shift) & 15;
            const int top = (byte_of(high.x, high.y, index) >> (2 * quarter)) & 3;
            out[index] = __fmul_rn(scaled, static_cast<float>((nibble | (top << 4)) - 32));
        }
    }
};

struct EightOfQ8_0 {
    u32x2_a2 codes;
    std::uint32_t d;
    __device__ __forceinline__ void load(const std::uint8_t* row, std::int64_t stage, int part) {
        const std::uint8_t* block = row + stage * 34;
        d = *reinterpret_cast<const std::uint16_t*>(block);
        codes = *reinterpret_cast<const u32x2_a2*>(block + 2 + part * 8);
    }
    __device__ __forceinline__ void decode(std::int64_t, float (&out)[8]) const {
        const float scale = half_bits_to_float(d);
#pragma unroll
        for (int index = 0; index < 8; ++index) {
            const int quant = static_cast<std::int8_t>(byte_of(codes.x, codes.y, index));
            out[index] = scale * static_cast<float>(quant);
        }
    }
};

template <std::uint32_t ENC>
struct EightUnpacked {
    float values[8];
    __device__ __forceinline__ void load(const std::uint8_t* row, std::int64_t stage, int part) {
#pragma unroll
        for (int index = 0; index < 8; ++index) {
            values[index] = weight_value(ENC, row, stage * kStage + part * 8 + index);
        }
    }
    __device__ __forceinline__ void decode(std::int64_t, float (&out)[8]) const {
#pragma unroll
        for (int index = 0; index < 8; ++index) out[index] = values[index];
    }
};

template <std::uint32_t ENC>
using EightWeights = std::conditional_t<
    ENC == kEncQ4K || ENC == kEncQ5K, EightOfQ4KOrQ5K<ENC>,
    std::conditional_t<ENC == kEncQ6K, EightOfQ6K,
                       std::conditional_t<ENC == kEncQ8_0, EightOfQ8_0, EightUnpacked<ENC>>>>;

template <std::uint32_t ENC>
__global__ __launch_bounds__(256, 4) void gemm_f32_kernel(
    const std::uint8_t* __restrict__ data, std::int64_t row_stride,
    const float* __restrict__ input, const float* __restrict__ bias,
    float* __restrict__ output, std::int64_t rows, std::int64_t input_dim,
    std::int64_t output_dim) {
    __shared__ __attribute__((aligned(16))) float a_stage[kTileRows * kPitch];
    __shared__ __attribute__((aligned(16))) float b_stage[kTileCols * kPitch];

    const int thread = threadIdx.x;
    const int lane = thread & 63;
    const int wave = thread >> 6;
    const std::int64_t row0 = static_cast<std::int64_t>(blockIdx.y) * kTileRows;
    const std::int64_t col0 = static_cast<std::int64_t>(blockIdx.x) * kTileCols;

    // Loader roles.  Rows past the end read the last row again; their results are not stored.
    const int a_row = thread >> 1;
    const int a_col = (thread & 1) * 16;
    const float* a_source =
        input + min(row0 + a_row, rows - 1) * input_dim + a_col;
    const int b_row = thread >> 2;
    const int b_col = (thread & 3) * 8;
    const std::uint8_t* b_source = data + min(col0 + b_row, output_dim - 1) * row_stride;

    // A stage's operands are requested two stages ahead, decoded one stage ahead.
    struct Requested {
        f32x4 a[4];
        EightWeights<ENC> b;
    };
    auto fetch = [&](Requested& into, std::int64_t stage) {
#pragma unroll
        for (int piece = 0; piece < 4; ++piece) {
            into.a[piece] = *reinterpret_cast<const f32x4_unaligned*>(a_source + stage * kStage +
                                                                      4 * piece);
        }
        into.b.load(b_source, stage, thread & 3);
    };
    auto keep = [&](const Requested& from, std::int64_t stage) {
        float weights[8];
        from.b.decode(stage, weights);
#pragma unroll
        for (int piece = 0; piece < 4; ++piece) {
            *reinterpret_cast<f32x4*>(&a_stage[a_row * kPitch + a_col + 4 * piece]) =
                from.a[piece];
        }
#pragma unroll
        for (int piece = 0; piece < 2; ++piece) {
            f32x4 four;
            four.x = weights[4 * piece];
            four.y = weights[4 * piece + 1];
            four.z = weights[4 * piece + 2];
            four.w = weights[4 * piece + 3];
            *reinterpret_cast<f32x4*>(&b_stage[b_row * kPitch + b_col + 4 * piece]) = four;
        }
    };

    // Consumer roles: the wave's 64 x 32 outputs.
    const int inner = lane & 31;
    const int upper = lane >> 5;
    const int a_base = ((wave & 1) * 64 + inner) * kPitch + upper * 4;
    const int b_base = ((wave >> 1) * 32 + inner) * kPitch + upper * 4;
    f32x16 sum_low = {}, sum_high = {};

    const std::int64_t stages = input_dim / kStage;
    Requested ahead_one, ahead_two;
    fetch(ahead_one, 0);
    fetch(ahead_two, stages > 1 ? 1 : 0);
    keep(ahead_one, 0);
    ahead_one = ahead_two;
    __syncthreads();
    for (std::int64_t stage = 0; stage < stages; ++stage) {
        // unconditional: past the end the last stage is read again and dropped
        fetch(ahead_two, stage + 2 < stages ? stage + 2 : stages - 1);
#pragma unroll
        for (int eight = 0; eight < kStage / 8; ++eight) {
            const f32x4 a_low = *reinterpret_cast<const f32x4*>(&a_stage[a_base + eight * 8]);
            const f32x4 a_high =
                *reinterpret_cast<const f32x4*>(&a_stage[a_base + 32 * kPitch + eight * 8]);
            const f32x4 b = *reinterpret_cast<const f32x4*>(&b_stage[b_base + eight * 8]);
            sum_low = __builtin_amdgcn_mfma_f32_32x32x2f32(a_low.x, b.x, sum_low, 0, 0, 0);
            sum_high = __builtin_amdgcn_mfma_f32_32x32x2f32(a_high.x, b.x, sum_high, 0, 0, 0);
            sum_low = __builtin_amdgcn_mfma_f32_32x32x2f32(a_low.y, b.y, sum_low, 0, 0, 0);
            sum_high = __builtin_amdgcn_mfma_f32_32x32x2f32(a_high.y, b.y, sum_high, 0, 0, 0);
            sum_low = __builtin_amdgcn_mfma_f32_32x32x2f32(a_low.z, b.z, sum_low, 0, 0, 0);
            sum_high = __builtin_amdgcn_mfma_f32_32x32x2f32(a_high.z, b.z, sum_high, 0, 0, 0);
            sum_low = __builtin_amdgcn_mfma_f32_32x32x2f32(a_low.w, b.w, sum_low, 0, 0, 0);
            sum_high = __builtin_amdgcn_mfma_f32_32x32x2f32(a_high.w, b.w, sum_high, 0, 0, 0);
        }
        __syncthreads();
        // unconditional as well: what it writes after the last stage nobody reads
        keep(ahead_one, stage + 1);
        ahead_one = ahead_two;
        __syncthreads();
    }

    // Accumulator register r of a lane: row 8 (r / 4) + 4 (lane / 32) + r % 4, column lane % 32.
    const std::int64_t column = col0 + (wave >> 1) * 32 + inner;
    if (column >= output_dim) return;
    const float offset = bias != nullptr ? bias[column] : 0.0f;
    const std::int64_t first_row = row0 + (wave & 1) * 64 + upper * 4;
#pragma unroll
    for (int index = 0; index < 16; ++index) {
        const std::int64_t row = first_row + 8 * (index / 4) + index % 4;
        if (row < rows) output[row * output_dim + column] = sum_low[index] + offset;
        if (row + 32 < rows) output[(row + 32) * output_dim + column] = sum_high[index] + offset;
    }
}

template <std::uint32_t ENC>
void launch_for(const Descriptor& weight, const float* input, const float* bias, float* output,
                std::int64_t rows, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((weight.output_dim + kTileCols - 1) / kTileCols),
                    static_cast<unsigned>((rows + kTileRows - 1) / kTileRows), 1);
    hipLaunchKernelGGL(gemm_f32_kernel<ENC>, grid, dim3(256), 0, stream, weight.data,
                       weight.row_stride_bytes, input, bias, output, rows, weight.input_dim,
                       weight.output_dim);
}

}  // namespace

bool gemm_f32_supports(const Descriptor& weight, std::int64_t rows) {
    return rows > 0 && weight.input_dim > 0 && weight.input_dim % kStage == 0 &&
           (rows + kTileRows - 1) / kTileRows <= 65535 && block_bytes(weight.encoding) != 0;
}

double gemm_f32_tile_passes(const Descriptor& weight, std::int64_t rows) {
    const double tiles = static_cast<double>((weight.output_dim + kTileCols - 1) / kTileCols) *
                         static_cast<double>((rows + kTileRows - 1) / kTileRows);
    const double units = compute_units();
    return tiles < units ? 1.0 : tiles / units;
}

void launch_gemm_f32(const Descriptor& weight, const float* input, const float* bias,
                     float* output, std::int64_t rows, hipStream_t stream) {
    switch (weight.encoding) {
        case kEncQ4K: launch_for<kEncQ4K>(weight, input, bias, output, rows, stream); break;
        case kEncQ5K: launch_for<kEncQ5K>(weight, input, bias, output, rows, stream); break;
        case kEncQ6K: launch_for<kEncQ6K>(weight, input, bias, output, rows, stream); break;
        case kEncQ8_0: launch_for<kEncQ8_0>(weight, input, bias, output, rows, stream); break;
        case kEncBF16: launch_for<kEncBF16>(weight, input, bias, output, rows, stream); break;
        default: launch_for<kEncF32>(weight, input, bias, output, rows, stream); break;
    }
}

}  // namespace nfn
