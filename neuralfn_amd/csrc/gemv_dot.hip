// One-token (and verifier) decode GEMV on the vector ALUs: v_dot4_i32_i8.
//
// One wave owns whole weight rows; its 64 lanes split a row into units of one
// 64-value pair of sub-blocks (32 bytes of 4-bit codes = two 16-byte loads, so
// consecutive lanes read consecutive bytes of the row).  A workgroup first
// turns the activation vector into two int8 planes (high and low byte of a
// 16-bit fixed-point code, one scale per 256 values) in LDS, laid out so that
// consecutive units read consecutive 16-byte slots; the first weight loads of
// every wave are already in flight while it does so.  Per unit a lane then
// spends 24 logic operations on unpacking and 32 dot4 on the two planes, and
// folds the 6-bit sub-scales in with 24-bit integer multiplies; one float
// conversion per unit, one butterfly per row.  No LDS round trip for weights,
// no synchronisation after the single barrier, small register footprint: the
// latency of HBM is hidden by many resident waves.
//
// Every row gets the same arithmetic whatever the number of tokens in the
// launch (T token planes are walked one after another against the same
// unpacked weights), which is the contract of the reference's verifier entry
// points (neuralfn/csrc/native_train/tile_ops.h:685-688) and of its one-row
// kernel (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:714-890).  With x = s*c,
// c = 256*hi + lo:  y += s*(d*sum_sub sc*dot(q, c) - dmin*sum_sub m*sum(c)).
#include "common.hpp"
#include "gemv_dot.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kDotWaves = 8;
constexpr int kDotThreads = kDotWaves * kWave;

// LDS image of one token's activations for a K of `blocks` super-blocks:
//   planes: eight arrays of `units` 16-byte slots, units = 4*blocks; unit
//           u = 4*block + pair reads slot u of every array:
//           array = 4*part + 2*plane + half  (part: which sub-block of the pair,
//           plane: 0 high / 1 low byte, half: which 16 of the 32 values)
//   sums:   int32 per sub-block: sum of its 32 codes
//   scale:  float per block
struct TokenImage {
    std::uint8_t* planes;
    int* sums;
    float* scale;
};

__device__ __forceinline__ int token_image_bytes(int blocks) {
    return blocks * (4 * 128 + 8 * 4 + 4 + 12);  // keeps every image 16-byte aligned
}
constexpr int token_image_bytes_host(std::int64_t blocks) {
    return static_cast<int>(blocks * (4 * 128 + 8 * 4 + 4 + 12));
}

__device__ __forceinline__ TokenImage token_image(std::uint8_t* lds, int token, int blocks) {
    std::uint8_t* base = lds + token * token_image_bytes(blocks);
    TokenImage image;
    image.planes = base;
    image.sums = reinterpret_cast<int*>(base + blocks * 512);
    image.scale = reinterpret_cast<float*>(base + blocks * 544);
    return image;
}

// Scatter the codes of block `block`, four values per lane, into the image.
__device__ __forceinline__ void quantize_block(const ActivationCodes& codes, int lane, int block,
                                               int blocks, const TokenImage& image) {
    const std::uint32_t hi = codes.hi, lo = codes.lo;
    const float maximum = codes.maximum;
    int sum = codes.sum;
    sum += dpp_move<kQuadXor1>(sum);
    sum += dpp_move<kQuadXor2>(sum);
    sum += dpp_move<kHalfMirror>(sum);
    // lane L holds values 4L..4L+3: sub-block L/8, 16-value half (L%8)/4, byte (L%4)*4
    const int units = 4 * blocks;
    const int sub = lane >> 3;
    const int unit = 4 * block + (sub >> 1);
    const int array_high = 4 * (sub & 1) + ((lane >> 2) & 1);
    std::uint8_t* slot = image.planes + (array_high * units + unit) * 16 + (lane & 3) * 4;
    *reinterpret_cast<std::uint32_t*>(slot) = hi;
    *reinterpret_cast<std::uint32_t*>(slot + 2 * units * 16) = lo;
    if ((lane & 7) == 0) image.sums[block * 8 + sub] = sum;
    if (lane == 0) image.scale[block] = maximum * (1.0f / kCodeRange);
}

template <bool Q5>
struct Stage {
    uint4 header;  // d, dmin, 12 scale bytes
    uint4 q0, q1;  // 32 bytes of 4-bit codes
    uint4 h0, h1;  // Q5_K: the block's 32 high-bit bytes
};

template <std::uint32_t ENC, int T, int P>
__global__ __launch_bounds__(kDotThreads) void gemv_dot_kernel(
    const float* __restrict__ first, const float* __restrict__ second, int tokens, int input_dim,
    int total_rows, int rows_per_group, int longer_groups, std::uint8_t* __restrict__ records_out,
    ProjectionSet set) {
    constexpr bool kQ5 = ENC == kEncQ5K;
    constexpr int kBlockBytes = kQ5 ? 176 : 144;
    constexpr int kQuants = kQ5 ? 48 : 16;
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blocks = input_dim >> 8;
    const int units = 4 * blocks;
    const int iterations = (units + kWave - 1) / kWave;
    const int token0 = blockIdx.y * T;
    const int pass_tokens = min(tokens - token0, T);
    const float* pass_first = pass_input<P>(first, token0, input_dim);
    const float* pass_second = P == kGated || P == kSwiGlu
        ? second + static_cast<std::int64_t>(token0) * input_dim : nullptr;

    // rows of this wave: dealt out evenly over the workgroups, then over the waves
    const WaveRows mine =
        wave_rows<kDotWaves>(static_cast<int>(blockIdx.x), wave, rows_per_group, longer_groups);
    const int row_begin = mine.begin;
    const int row_count = mine.count;
    const int total = row_count * iterations;

    // (1) activations of the first records this wave quantizes: loaded first so
    // that their short latency does not queue behind the weight loads.  All
    // loads are unconditional (clamped indices) to keep the load counters exact.
    const int records = pass_tokens * blocks;
    constexpr int kEarly = 4;
    float4 early[kEarly];
#pragma unroll
    for (int e = 0; e < kEarly; ++e) {
        const int record = min(wave + e * kDotWaves, records - 1);
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        early[e] = load_activations<P>(pass_first, pass_second,
                                       static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
    }

    // (2) weight loads of the first two (row, iteration) pairs
    PairCursor fetch;
    fetch.start(set, min(row_begin, total_rows - 1));
    int fetch_left = total;  // pairs not fetched yet; the cursor rests on the last one
    auto issue = [&](Stage<kQ5>& stage) {
        const int unit = min(fetch.iteration * kWave + lane, units - 1);
        const std::uint8_t* block = fetch.row + (unit >> 2) * kBlockBytes;
        stage.header = *reinterpret_cast<const uint4*>(block);
        const std::uint8_t* quants = block + kQuants + (unit & 3) * 32;
        stage.q0 = *reinterpret_cast<const uint4*>(quants);
        stage.q1 = *reinterpret_cast<const uint4*>(quants + 16);
        if constexpr (kQ5) {
            stage.h0 = *reinterpret_cast<const uint4*>(block + 16);
            stage.h1 = *reinterpret_cast<const uint4*>(block + 32);
        }
        if (--fetch_left > 0) fetch.advance(set, iterations);
    };
    Stage<kQ5> stage0, stage1;
    issue(stage0);
    issue(stage1);

    // (3) quantize; one barrier; after it the workgroup never synchronises again.
    // The first workgroup also leaves the records in the caller's workspace
    // for a later launch that shares this input.
    const bool keep_records = P != kRecords && records_out != nullptr && blockIdx.x == 0;
    auto quantize_record = [&](float4 loaded, int record) {
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        const ActivationCodes codes = activation_codes<P>(loaded);
        quantize_block(codes, lane, block, blocks, token_image(lds, token, blocks));
        if (keep_records) {
            store_record(records_out + (static_cast<std::int64_t>(token0 + token) * blocks + block) *
                             kActRecord, lane, codes);
        }
    };
#pragma unroll
    for (int e = 0; e < kEarly; ++e) {
        const int record = wave + e * kDotWaves;
        if (record < records) quantize_record(early[e], record);
    }
    for (int record = wave + kEarly * kDotWaves; record < records; record += kDotWaves) {
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        const float4 x = load_activations<P>(
            pass_first, pass_second,
            static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
        quantize_record(x, record);
    }
    __syncthreads();

    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0f;

    PairCursor work;
    work.start(set, min(row_begin, total_rows - 1));
    auto compute = [&](const Stage<kQ5>& stage) {
        const int iteration = work.iteration;
        const int raw_unit = iteration * kWave + lane;
        const bool live = raw_unit < units;
        const int unit = min(raw_unit, units - 1);
        const int block = unit >> 2;
        const int pair = unit & 3;

        // unpack: the low nibbles are sub-block 2*pair, the high nibbles 2*pair+1
        const std::uint32_t packed[8] = {stage.q0.x, stage.q0.y, stage.q0.z, stage.q0.w,
                                         stage.q1.x, stage.q1.y, stage.q1.z, stage.q1.w};
        std::uint32_t low[8], high[8];
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            low[w] = packed[w] & 0x0f0f0f0fu;
            high[w] = (packed[w] >> 4) & 0x0f0f0f0fu;
        }
        if constexpr (kQ5) {
            const std::uint32_t bits[8] = {stage.h0.x, stage.h0.y, stage.h0.z, stage.h0.w,
                                           stage.h1.x, stage.h1.y, stage.h1.z, stage.h1.w};
#pragma unroll
            for (int w = 0; w < 8; ++w) {
                // bit 2*pair of the high-bit byte belongs to the first sub-block, 2*pair+1 to the second
                const std::uint32_t shifted = bits[w] >> (2 * pair);
                low[w] |= (shifted & 0x01010101u) << 4;
                high[w] |= (shifted & 0x02020202u) << 3;
            }
        }
        // the pair's two 6-bit scales and minimums, packed [second:first] in 16 bits
        const int shift = 16 * (pair & 1);
        const std::uint32_t y = stage.header.y >> shift;
        const std::uint32_t z = stage.header.z >> shift;
        const std::uint32_t w = stage.header.w >> shift;
        const bool upper = pair >= 2;
        const std::uint32_t scales = upper ? ((w & 0x0f0fu) | ((y >> 2) & 0x3030u)) : (y & 0x3f3fu);
        const std::uint32_t minimums =
            upper ? (((w >> 4) & 0x0f0fu) | ((z >> 2) & 0x3030u)) : (z & 0x3f3fu);
        // as floats: every product and sum below stays under 2^24, so the
        // float arithmetic on the integer dot products is exact
        const float scale_a = static_cast<float>(scales & 0xffu);
        const float scale_b = static_cast<float>((scales >> 8) & 0xffu);
        const float min_a = static_cast<float>(minimums & 0xffu);
        const float min_b = static_cast<float>((minimums >> 8) & 0xffu);
        const float d = half_bits_to_float(stage.header.x & 0xffffu);
        const float dmin = half_bits_to_float(stage.header.x >> 16);

#pragma unroll
        for (int t = 0; t < T; ++t) {
            const TokenImage image = token_image(lds, t, blocks);
            const std::uint8_t* slot = image.planes + unit * 16;
            const int stride = units * 16;
            int dot_a_hi = 0, dot_a_lo = 0, dot_b_hi = 0, dot_b_lo = 0;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const v4i a_hi = *reinterpret_cast<const v4i*>(slot + (0 + half) * stride);
                const v4i a_lo = *reinterpret_cast<const v4i*>(slot + (2 + half) * stride);
                const v4i b_hi = *reinterpret_cast<const v4i*>(slot + (4 + half) * stride);
                const v4i b_lo = *reinterpret_cast<const v4i*>(slot + (6 + half) * stride);
#pragma unroll
                for (int v = 0; v < 4; ++v) {
                    const int lo_codes = static_cast<int>(low[half * 4 + v]);
                    const int hi_codes = static_cast<int>(high[half * 4 + v]);
                    dot_a_hi = __builtin_amdgcn_sdot4(lo_codes, a_hi[v], dot_a_hi, false);
                    dot_a_lo = __builtin_amdgcn_sdot4(lo_codes, a_lo[v], dot_a_lo, false);
                    dot_b_hi = __builtin_amdgcn_sdot4(hi_codes, b_hi[v], dot_b_hi, false);
                    dot_b_lo = __builtin_amdgcn_sdot4(hi_codes, b_lo[v], dot_b_lo, false);
                }
            }
            const int2 sums = *reinterpret_cast<const int2*>(image.sums + block * 8 + 2 * pair);
            const float scale = image.scale[block];
            const float weighted_hi = fmaf(scale_b, static_cast<float>(dot_b_hi),
                                           scale_a * static_cast<float>(dot_a_hi));
            const float weighted_lo = fmaf(scale_b, static_cast<float>(dot_b_lo),
                                           scale_a * static_cast<float>(dot_a_lo));
            const float weighted_min = fmaf(min_b, static_cast<float>(sums.y),
                                            min_a * static_cast<float>(sums.x));
            const float codes = fmaf(weighted_hi, 256.0f, weighted_lo);
            const float value = fmaf(-dmin, weighted_min, d * codes);
            acc[t] = fmaf(live ? scale : 0.0f, value, acc[t]);
        }

        if (iteration == iterations - 1) {
            // the row is complete: fixed-order butterfly, lane 0 writes
            float* output = work.current.output + work.local_row;
            const std::int64_t output_dim = work.current.output_dim;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float total_value = wave_total(acc[t]);
                if (lane == 0 && t < pass_tokens) {
                    output[static_cast<std::int64_t>(token0 + t) * output_dim] = total_value;
                }
                acc[t] = 0.0f;
            }
        }
        work.advance(set, iterations);
    };

    for (int n = 0; n < total; n += 2) {
        compute(stage0);
        issue(stage0);
        if (n + 1 < total) compute(stage1);
        issue(stage1);
    }
}

template <std::uint32_t ENC, int T, int P>
void launch_variant(ProjectionSet set, const float* first, const float* second,
                    std::uint8_t* records_out, int tokens, hipStream_t stream) {
    std::int64_t rows = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = static_cast<std::uint32_t>(rows);  // first row here
        rows += set.op[index].output_dim;
    }
    const std::int64_t blocks = set.input_dim >> 8;
    const std::size_t lds = static_cast<std::size_t>(T) * token_image_bytes_host(blocks);
    auto kernel = gemv_dot_kernel<ENC, T, P>;
    allow_large_lds<gemv_dot_kernel<ENC, T, P>>();
    const int passes = (tokens + T - 1) / T;
    const std::int64_t groups = decode_groups(rows, kDotWaves);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), passes), dim3(kDotThreads), lds,
                       stream, first, second, tokens, static_cast<int>(set.input_dim),
                       static_cast<int>(rows), static_cast<int>(rows / groups),
                       static_cast<int>(rows % groups), records_out, set);
}

template <std::uint32_t ENC, int P>
void launch_tokens(const ProjectionSet& set, const float* first, const float* second,
                   std::uint8_t* records_out, int tokens, hipStream_t stream) {
    // token planes of one pass must fit in LDS: four tokens up to K = 16384
    const std::int64_t image = token_image_bytes_host(set.input_dim >> 8);
    int capacity = static_cast<int>((150 * 1024) / image);
    if (capacity > 4) capacity = 4;
    const int per_pass = tokens < capacity ? tokens : capacity;
    if (per_pass <= 1) {
        launch_variant<ENC, 1, P>(set, first, second, records_out, tokens, stream);
    } else if (per_pass == 2) {
        launch_variant<ENC, 2, P>(set, first, second, records_out, tokens, stream);
    } else if (capacity >= 4) {
        launch_variant<ENC, 4, P>(set, first, second, records_out, tokens, stream);
    } else {
        launch_variant<ENC, 2, P>(set, first, second, records_out, tokens, stream);
    }
}

template <std::uint32_t ENC>
void launch_prologue(const ProjectionSet& set, const float* first, const float* second,
                     std::uint8_t* records_out, int prologue, int tokens, hipStream_t stream) {
    switch (prologue) {
        case kGated:
            launch_tokens<ENC, kGated>(set, first, second, records_out, tokens, stream);
            break;
        case kSwiGlu:
            launch_tokens<ENC, kSwiGlu>(set, first, second, records_out, tokens, stream);
            break;
        case kRecords:
            launch_tokens<ENC, kRecords>(set, first, second, nullptr, tokens, stream);
            break;
        default:
            launch_tokens<ENC, kPlain>(set, first, second, records_out, tokens, stream);
            break;
    }
}

}  // namespace

bool gemv_dot_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K) && input_dim % 256 == 0 &&
        token_image_bytes_host(input_dim >> 8) <= 150 * 1024;
}

void launch_gemv_dot(const ProjectionSet& set, const float* first, const float* second,
                     std::uint8_t* records_out, int prologue, std::int64_t rows,
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
            launch_prologue<kEncQ4K>(group, first, second, records_out, prologue,
                                     static_cast<int>(rows), stream);
        } else {
            launch_prologue<kEncQ5K>(group, first, second, records_out, prologue,
                                     static_cast<int>(rows), stream);
        }
    }
}

}  // namespace nfn
