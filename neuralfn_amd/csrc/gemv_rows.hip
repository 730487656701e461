// Verifier rows (2..16 tokens) of Q4_K / Q5_K projections on the int8 matrix cores, every row
// in the one-row kernel's arithmetic bit for bit.
//
// The contract (neuralfn/csrc/native_train/tile_ops.h:685-688; the reference's kernel:
// neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1753-1925): row t of a batched call equals the
// one-row call on row t.  The one-row kernel (gemv_dot.hip) gives lane L of a wave the units
// u = L, L + 64, ... of a weight row (a unit: one 64-value pair of sub-blocks), chains
//     acc = fmaf(scale, fmaf(-dmin, float(wmin), d * fmaf(float(whi), 256, float(wlo))), acc)
// over them and sums the 64 lanes in a butterfly.  Everything up to whi / wlo / wmin is exact
// integer arithmetic, and float addition is commutative, so the result is fixed by
//   * which terms form a chain: the units 4b + p of the blocks b = c, c + 16, c + 32, ...
//     ("class" c = 0..15, p = 0..3), in that order,
//   * the balanced binary tree over the 64 chains in the order (c, p).
// Here a workgroup of 8 waves owns 32 consecutive weight rows.  v_mfma_i32_32x32x32_i8 takes
// the 32 values of a sub-block (K), 32 weight rows (operand B, lane l: row l % 32, values
// 16 (l / 32)..+15, unpacked from the 16 bytes of codes the lane loaded itself) and the two
// int8 planes of up to 16 tokens (operand A, read from the activation records a quantizer
// launch left in the workspace); a second product against the sub-block minimums, spread over
// K, gives the sums the minimums multiply.  A lane then holds, for its weight row and up to 8
// tokens, the integers of a unit, and replays the float tail above.  Wave w takes the classes
// w and 15 - w (an even share of any row length), keeps the four chains of a class per token
// in registers, and leaves (c0 + c1) + (c2 + c3) per class, token and row in LDS; after one
// barrier a thread per (token, row) adds the 16 classes in the tree's order.
// One pass over the weights for up to 16 tokens, no weight byte through LDS.
#include "common.hpp"
#include "gemv_rows.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kRowsTile = 32;
constexpr int kRowsWaves = 8;
constexpr int kRowsThreads = kRowsWaves * kWave;
constexpr int kClasses = 16;

// One wave per activation record: the (token, block) records of wave_rows.hpp.
template <int P>
__global__ __launch_bounds__(256) void quantize_records_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    std::uint8_t* __restrict__ records, int total_records) {
    const int lane = threadIdx.x & 63;
    const int record = static_cast<int>(blockIdx.x) * 4 + static_cast<int>(threadIdx.x >> 6);
    if (record >= total_records) return;
    const float4 x = load_activations<P>(first, second,
                                         static_cast<std::int64_t>(record) * 256 + lane * 4);
    store_record(records + static_cast<std::int64_t>(record) * kActRecord, lane,
                 activation_codes<P>(x));
}

template <bool Q5, int S>
struct RowsStage {
    uint4 header;   // d, dmin, 12 bytes of scales and minimums
    uint4 q[4];     // this lane's half of the four 32-byte code groups
    uint4 high;     // Q5_K: this lane's half of the high-bit bytes
    v4i a[8];       // operand A of the eight sub-blocks
    float scale[S]; // the block's activation scale of this lane's tokens
};

__device__ __forceinline__ v16i mfma_i8(v4i a, v4i b, v16i c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

// S: token slots per lane.  Token S * (lane / 32) + slot sits in output registers 2 * slot
// (high plane) and 2 * slot + 1 (low plane) of the lane; tokens = up to 2 * S.
template <std::uint32_t ENC, int S>
__global__ __launch_bounds__(kRowsThreads) void gemv_rows_kernel(
    const std::uint8_t* __restrict__ records, int tokens, int input_dim, std::uint32_t total_tiles,
    ProjectionSet set) {
    constexpr bool kQ5 = ENC == kEncQ5K;
    constexpr int kBlockBytes = kQ5 ? 176 : 144;
    constexpr int kQuants = kQ5 ? 48 : 16;
    constexpr int kTokens = 2 * S;
    __shared__ float class_sums[kClasses][kTokens][kRowsTile];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31;
    const int h = lane >> 5;
    const int blocks = input_dim >> 8;

    // the tile's projection and rows (uniform)
    const std::uint32_t tile = blockIdx.x;
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && tile >= set.op[index].first_tile) which = index;
    }
    const Projection op = pick(set, which);
    const std::int64_t row0 = static_cast<std::int64_t>(tile - op.first_tile) * kRowsTile;
    const int valid_rows =
        static_cast<int>(min(static_cast<std::int64_t>(kRowsTile), op.output_dim - row0));
    const std::uint8_t* weight_row =
        op.data + (row0 + min(j, valid_rows - 1)) * op.row_stride + h * 16;

    // operand A: row i = lane % 32 of the matrix instruction is (token, plane):
    // i = 8 a + 4 half + 2 c + plane  <->  output register 4 a + 2 c + plane of lane half `half`
    const int a_plane = j & 1;
    const int a_slot = 2 * (j >> 3) + ((j >> 1) & 1);
    const int a_token = min(a_slot < S ? S * ((j >> 2) & 1) + a_slot : 0, tokens - 1);
    const std::uint8_t* a_row = records +
        static_cast<std::int64_t>(a_token) * blocks * kActRecord + a_plane * 256 + h * 16;
    // the scales of this lane's tokens
    const std::uint8_t* scale_row[S];
#pragma unroll
    for (int slot = 0; slot < S; ++slot) {
        scale_row[slot] = records +
            static_cast<std::int64_t>(min(S * h + slot, tokens - 1)) * blocks * kActRecord + kRecordScale;
    }

    // this wave's steps: the blocks of class `wave`, then those of class 15 - wave
    const int class0 = wave;
    const int class1 = kClasses - 1 - wave;
    const int count0 = class0 < blocks ? (blocks - class0 + kClasses - 1) / kClasses : 0;
    const int count1 = class1 < blocks ? (blocks - class1 + kClasses - 1) / kClasses : 0;
    const int total = count0 + count1;

    auto block_of = [&](int step) {
        return step < count0 ? class0 + kClasses * step : class1 + kClasses * (step - count0);
    };
    auto fetch = [&](RowsStage<kQ5, S>& stage, int step) {
        // (a step past the wave's last repeats it; a wave with no block at all reads the row's last)
        const int block = min(block_of(min(step, max(total - 1, 0))), blocks - 1);
        const std::uint8_t* weights = weight_row + static_cast<std::int64_t>(block) * kBlockBytes;
        stage.header = *reinterpret_cast<const uint4*>(weights - h * 16);
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            stage.q[p] = *reinterpret_cast<const uint4*>(weights + kQuants + p * 32);
        }
        if constexpr (kQ5) stage.high = *reinterpret_cast<const uint4*>(weights + 16);
        const std::uint8_t* planes = a_row + static_cast<std::int64_t>(block) * kActRecord;
#pragma unroll
        for (int sub = 0; sub < 8; ++sub) {
            stage.a[sub] = *reinterpret_cast<const v4i*>(planes + sub * 32);
        }
#pragma unroll
        for (int slot = 0; slot < S; ++slot) {
            stage.scale[slot] = *reinterpret_cast<const float*>(
                scale_row[slot] + static_cast<std::int64_t>(block) * kActRecord);
        }
    };

    float acc[4][S];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
        for (int slot = 0; slot < S; ++slot) acc[p][slot] = 0.0f;
    }

    auto compute = [&](const RowsStage<kQ5, S>& stage) {
        const uint4 head = stage.header;
        // 6-bit scales and minimums of the eight sub-blocks, four per word
        const std::uint32_t sc_lo = head.y & 0x3f3f3f3fu;
        const std::uint32_t mn_lo = head.z & 0x3f3f3f3fu;
        const std::uint32_t sc_hi = (head.w & 0x0f0f0f0fu) | ((head.y >> 2) & 0x30303030u);
        const std::uint32_t mn_hi = ((head.w >> 4) & 0x0f0f0f0fu) | ((head.z >> 2) & 0x30303030u);
        const float d = half_bits_to_float(head.x & 0xffffu);
        const float dmin = half_bits_to_float(head.x >> 16);
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const std::uint32_t packed[4] = {stage.q[p].x, stage.q[p].y, stage.q[p].z, stage.q[p].w};
            v4i low, upper;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                std::uint32_t lo = packed[w] & 0x0f0f0f0fu;
                std::uint32_t up = (packed[w] >> 4) & 0x0f0f0f0fu;
                if constexpr (kQ5) {
                    const std::uint32_t bits[4] = {stage.high.x, stage.high.y, stage.high.z, stage.high.w};
                    const std::uint32_t shifted = bits[w] >> (2 * p);
                    lo |= (shifted & 0x01010101u) << 4;
                    up |= (shifted & 0x02020202u) << 3;
                }
                low[w] = static_cast<int>(lo);
                upper[w] = static_cast<int>(up);
            }
            const std::uint32_t sc_word = p < 2 ? sc_lo : sc_hi;
            const std::uint32_t mn_word = p < 2 ? mn_lo : mn_hi;
            const int scale_a = static_cast<int>((sc_word >> (16 * (p & 1))) & 0xffu);
            const int scale_b = static_cast<int>((sc_word >> (16 * (p & 1) + 8)) & 0xffu);
            const int min_a = static_cast<int>((mn_word >> (16 * (p & 1))) & 0xffu);
            const int min_b = static_cast<int>((mn_word >> (16 * (p & 1) + 8)) & 0xffu);
            const int spread_a = min_a * 0x01010101;
            const int spread_b = min_b * 0x01010101;
            const v4i mins_a = {spread_a, spread_a, spread_a, spread_a};
            const v4i mins_b = {spread_b, spread_b, spread_b, spread_b};
            const v16i dots_a = mfma_i8(stage.a[2 * p], low, zero);
            const v16i dots_b = mfma_i8(stage.a[2 * p + 1], upper, zero);
            // min_a * sum(codes of a) + min_b * sum(codes of b), per plane
            const v16i sums = mfma_i8(stage.a[2 * p + 1], mins_b, mfma_i8(stage.a[2 * p], mins_a, zero));
#pragma unroll
            for (int slot = 0; slot < S; ++slot) {
                const int weighted_hi = __mul24(scale_a, dots_a[2 * slot]) + __mul24(scale_b, dots_b[2 * slot]);
                const int weighted_lo =
                    __mul24(scale_a, dots_a[2 * slot + 1]) + __mul24(scale_b, dots_b[2 * slot + 1]);
                const int weighted_min = sums[2 * slot] * 256 + sums[2 * slot + 1];
                const float codes =
                    fmaf(static_cast<float>(weighted_hi), 256.0f, static_cast<float>(weighted_lo));
                const float value = fmaf(-dmin, static_cast<float>(weighted_min), d * codes);
                acc[p][slot] = fmaf(stage.scale[slot], value, acc[p][slot]);
            }
        }
    };
    // a class is complete: (c0 + c1) + (c2 + c3) per token goes to LDS
    auto finish_class = [&](int cls) {
#pragma unroll
        for (int slot = 0; slot < S; ++slot) {
            class_sums[cls][S * h + slot][j] =
                (acc[0][slot] + acc[1][slot]) + (acc[2][slot] + acc[3][slot]);
#pragma unroll
            for (int p = 0; p < 4; ++p) acc[p][slot] = 0.0f;
        }
    };

    RowsStage<kQ5, S> stages[2];
    fetch(stages[0], 0);
    if (count0 == 0) finish_class(class0);
    if (count1 == 0) finish_class(class1);
    for (int step = 0; step < total; step += 2) {
#pragma unroll
        for (int k = 0; k < 2; ++k) {
            if (step + k < total) {
                fetch(stages[1 - k], step + k + 1);
                compute(stages[k]);
                if (step + k == count0 - 1) finish_class(class0);
                if (step + k == total - 1 && count1 > 0) finish_class(class1);
            }
        }
    }
    __syncthreads();

    // a thread per (token, row): the 16 classes in the order of the one-row kernel's butterfly
    const int token = static_cast<int>(threadIdx.x) >> 5;
    if (token < kTokens && token < tokens && j < valid_rows) {
        float pairs[8];
#pragma unroll
        for (int m = 0; m < 8; ++m) {
            pairs[m] = class_sums[2 * m][token][j] + class_sums[2 * m + 1][token][j];
        }
        const float q0 = pairs[0] + pairs[1];
        const float q1 = pairs[2] + pairs[3];
        const float q2 = pairs[4] + pairs[5];
        const float q3 = pairs[6] + pairs[7];
        op.output[static_cast<std::int64_t>(token) * op.output_dim + row0 + j] = (q0 + q1) + (q2 + q3);
    }
}

template <std::uint32_t ENC>
void launch_encoding(ProjectionSet set, const std::uint8_t* records, int tokens, hipStream_t stream) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = tiles;
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kRowsTile - 1) / kRowsTile);
    }
    const dim3 grid(tiles), block(kRowsThreads);
    const int input_dim = static_cast<int>(set.input_dim);
    if (tokens <= 4) {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 2>), grid, block, 0, stream, records, tokens,
                           input_dim, tiles, set);
    } else if (tokens <= 8) {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 4>), grid, block, 0, stream, records, tokens,
                           input_dim, tiles, set);
    } else {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 8>), grid, block, 0, stream, records, tokens,
                           input_dim, tiles, set);
    }
}

}  // namespace

bool gemv_rows_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K) && input_dim % 256 == 0 &&
        input_dim <= (std::int64_t(1) << 20);
}

void launch_quantize_records(const float* first, const float* second, int prologue,
                             std::int64_t rows, std::int64_t input_dim, std::uint8_t* records,
                             hipStream_t stream) {
    const int total = static_cast<int>(rows * (input_dim >> 8));
    const dim3 grid(static_cast<unsigned>((total + 3) / 4)), block(256);
    switch (prologue) {
        case kGated:
            hipLaunchKernelGGL((quantize_records_kernel<kGated>), grid, block, 0, stream, first,
                               second, records, total);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((quantize_records_kernel<kSwiGlu>), grid, block, 0, stream, first,
                               second, records, total);
            break;
        default:
            hipLaunchKernelGGL((quantize_records_kernel<kPlain>), grid, block, 0, stream, first,
                               second, records, total);
            break;
    }
}

void launch_gemv_rows(const ProjectionSet& set, const std::uint8_t* records, std::int64_t rows,
                      hipStream_t stream) {
    const std::uint32_t encodings[2] = {kEncQ4K, kEncQ5K};
    for (const std::uint32_t encoding : encodings) {
        ProjectionSet group{};
        group.input_dim = set.input_dim;
        for (int index = 0; index < set.count; ++index) {
            if (set.op[index].encoding == encoding) group.op[group.count++] = set.op[index];
        }
        if (group.count == 0) continue;
        if (encoding == kEncQ4K) {
            launch_encoding<kEncQ4K>(group, records, static_cast<int>(rows), stream);
        } else {
            launch_encoding<kEncQ5K>(group, records, static_cast<int>(rows), stream);
        }
    }
}

}  // namespace nfn
