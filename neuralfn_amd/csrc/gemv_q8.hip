// Q8_0 decode GEMV on the vector ALUs (v_dot4_i32_i8): one token, or verifier
// rows with the one-token arithmetic per row.
//
// A Q8_0 block is 34 bytes: an fp16 scale and 32 int8 codes
// (neuralfn/csrc/tile_cuda/vendor/llama_mmq_62bf73d/ggml/src/ggml-common.h:251-256;
// the reference engine itself has no Q8_0 code, this encoding is an extension).
// One wave owns whole weight rows; a lane's unit is a pair of blocks, 68 bytes
// = 17 dwords, which is 4-byte aligned (rows are 16-byte aligned since K is a
// multiple of 256): four unaligned 16-byte loads and one dword.  The codes of
// the first block start two bytes into the unit and are realigned with eight
// byte-align instructions; those of the second block are dword aligned.
//
// Activations: as in the other decode kernels, two int8 planes of a 16-bit
// fixed-point code in LDS with one scale per 256 values, quantized by the
// workgroup in the same launch, laid out per unit so that consecutive lanes
// read consecutive 16-byte slots.  y += s * (d0*(256*dot(q0,hi)+dot(q0,lo)) +
// d1*(...)); the brackets are exact integers, the reduction a fixed-order
// butterfly.
#include "common.hpp"
#include "gemv_q8.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kUnitBytes = 68;     // two blocks

struct __attribute__((packed, aligned(4))) Unaligned16 {
    std::uint32_t v[4];
};

// LDS image of one token's activations for a K of `blocks` groups of 256 values:
//   planes: eight arrays of `units` 16-byte slots, units = 4*blocks (a unit is
//           64 values); unit u reads slot u of array 2*sixteen + plane, where
//           sixteen = which 16 of its 64 values, plane 0 = high byte, 1 = low
//   scale:  float per 256 values
struct TokenImage {
    std::uint8_t* planes;
    float* scale;
};

constexpr int kImageBytesPerBlock = 4 * 128 + 16;

__host__ __device__ constexpr int token_image_bytes(std::int64_t blocks) {
    return static_cast<int>(blocks * kImageBytesPerBlock);
}

__device__ __forceinline__ TokenImage token_image(std::uint8_t* lds, int token, int blocks) {
    std::uint8_t* base = lds + token * token_image_bytes(blocks);
    TokenImage image;
    image.planes = base;
    image.scale = reinterpret_cast<float*>(base + blocks * 512);
    return image;
}

// Quantize the 256 activations of block `block`, four per lane: lane L holds
// values 4L..4L+3 = unit L/16 of the block, sixteen (L/4)%4, bytes 4*(L%4)..
__device__ __forceinline__ void quantize_block(const ActivationCodes& codes, int lane, int block,
                                               int blocks, const TokenImage& image) {
    const int units = 4 * blocks;
    const int unit = 4 * block + (lane >> 4);
    const int sixteen = (lane >> 2) & 3;
    std::uint8_t* slot = image.planes + (2 * sixteen * units + unit) * 16 + (lane & 3) * 4;
    *reinterpret_cast<std::uint32_t*>(slot) = codes.hi;
    *reinterpret_cast<std::uint32_t*>(slot + units * 16) = codes.lo;
    if (lane == 0) image.scale[block] = codes.maximum * (1.0f / kCodeRange);
}

struct Stage {
    Unaligned16 part[4];
    std::uint32_t last;
};

template <int T, int P>
__global__ __launch_bounds__(kThreads) void gemv_q8_kernel(
    const float* __restrict__ first, const float* __restrict__ second, int tokens, int input_dim,
    int total_rows, int rows_per_group, int longer_groups, std::uint8_t* __restrict__ records_out,
    ProjectionSet set) {
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blocks = input_dim >> 8;
    const int units = 4 * blocks;
    const int iterations = (units + kWave - 1) / kWave;
    const int token0 = blockIdx.y * T;
    const int pass_tokens = min(tokens - token0, T);
    const float* pass_first = pass_input<P>(first, token0, static_cast<int>(input_dim));
    const float* pass_second = P == kGated || P == kSwiGlu
        ? second + static_cast<std::int64_t>(token0) * input_dim : nullptr;

    // rows of this wave: dealt out evenly over the workgroups, then over the waves
    const WaveRows mine =
        wave_rows<kWaves>(static_cast<int>(blockIdx.x), wave, rows_per_group, longer_groups);
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
        const int record = min(wave + e * kWaves, records - 1);
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        early[e] = load_activations<P>(
            pass_first, pass_second,
            static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
    }

    // (2) weight loads of the first two (row, slice) pairs
    PairCursor fetch;
    fetch.start(set, min(row_begin, total_rows - 1));
    int fetch_left = total;  // pairs not fetched yet; the cursor rests on the last one
    auto issue = [&](Stage& stage) {
        const int unit = min(fetch.iteration * kWave + lane, units - 1);
        const std::uint8_t* source = fetch.row + unit * kUnitBytes;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            stage.part[k] = *reinterpret_cast<const Unaligned16*>(source + 16 * k);
        }
        stage.last = *reinterpret_cast<const std::uint32_t*>(source + 64);
        if (--fetch_left > 0) fetch.advance(set, iterations);
    };
    Stage stage0, stage1;
    issue(stage0);

    // (3) quantize; one barrier
    // (the first workgroup also leaves the records in the caller's workspace
    // for a later launch that shares this input)
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
        const int record = wave + e * kWaves;
        if (record < records) quantize_record(early[e], record);
    }
    for (int record = wave + kEarly * kWaves; record < records; record += kWaves) {
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        const float4 x = load_activations<P>(
            pass_first, pass_second,
            static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
        quantize_record(x, record);
    }
    // the second stage's weights are requested only now: requests that go out ahead of the
    // activation loads of waves that start later delay those, and every wave waits at
    // the barrier for all activations
    issue(stage1);
    __syncthreads();

    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0f;

    PairCursor work;
    work.start(set, min(row_begin, total_rows - 1));
    auto compute = [&](const Stage& stage) {
        const int iteration = work.iteration;
        const int raw_unit = iteration * kWave + lane;
        const bool live = raw_unit < units;
        const int unit = min(raw_unit, units - 1);
        const int block = unit >> 2;

        // the unit's 17 dwords: [d0 | codes0 0..1] [codes0 2..5] ... [codes0 30..31 | d1] [codes1 ...]
        std::uint32_t word[17];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
#pragma unroll
            for (int w = 0; w < 4; ++w) word[4 * k + w] = stage.part[k].v[w];
        }
        word[16] = stage.last;
        std::uint32_t codes0[8], codes1[8];
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            codes0[w] = __builtin_amdgcn_alignbyte(word[w + 1], word[w], 2);  // bytes 4w+2 .. 4w+5
            codes1[w] = word[9 + w];
        }
        const float d0 = half_bits_to_float(word[0] & 0xffffu);
        const float d1 = half_bits_to_float(word[8] >> 16);

#pragma unroll
        for (int t = 0; t < T; ++t) {
            const TokenImage image = token_image(lds, t, blocks);
            const std::uint8_t* slot = image.planes + unit * 16;
            const int stride = units * 16;
            int dot_hi[2] = {0, 0}, dot_lo[2] = {0, 0};
#pragma unroll
            for (int sixteen = 0; sixteen < 4; ++sixteen) {
                const v4i hi = *reinterpret_cast<const v4i*>(slot + (2 * sixteen) * stride);
                const v4i lo = *reinterpret_cast<const v4i*>(slot + (2 * sixteen + 1) * stride);
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    // values 16*sixteen + 4w .. +3 of the unit: block sixteen/2, code word 4*(sixteen%2)+w
                    const std::uint32_t q = sixteen < 2 ? codes0[4 * sixteen + w]
                                                        : codes1[4 * (sixteen - 2) + w];
                    dot_hi[sixteen >> 1] =
                        __builtin_amdgcn_sdot4(static_cast<int>(q), hi[w], dot_hi[sixteen >> 1], false);
                    dot_lo[sixteen >> 1] =
                        __builtin_amdgcn_sdot4(static_cast<int>(q), lo[w], dot_lo[sixteen >> 1], false);
                }
            }
            // |256*dot_hi + dot_lo| <= 32*127*32512 < 2^28: exact in int32
            const float value =
                fmaf(d1, static_cast<float>((dot_hi[1] << 8) + dot_lo[1]),
                     d0 * static_cast<float>((dot_hi[0] << 8) + dot_lo[0]));
            const float scale = image.scale[block];
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

template <int T, int P>
void launch_variant(ProjectionSet set, const float* first, const float* second,
                    std::uint8_t* records_out, int tokens, hipStream_t stream) {
    std::int64_t rows = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = static_cast<std::uint32_t>(rows);  // first row here
        rows += set.op[index].output_dim;
    }
    const std::size_t lds = static_cast<std::size_t>(T) * token_image_bytes(set.input_dim >> 8);
    auto kernel = gemv_q8_kernel<T, P>;
    allow_large_lds<gemv_q8_kernel<T, P>>();
    const int passes = (tokens + T - 1) / T;
    const std::int64_t groups = decode_groups(rows, kWaves);
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), passes), dim3(kThreads), lds,
                       stream, first, second, tokens, static_cast<int>(set.input_dim),
                       static_cast<int>(rows), static_cast<int>(rows / groups),
                       static_cast<int>(rows % groups), records_out, set);
}

template <int P>
void launch_tokens(const ProjectionSet& set, const float* first, const float* second,
                   std::uint8_t* records_out, int tokens, hipStream_t stream) {
    // the token images of one pass must fit in LDS
    const std::int64_t image = token_image_bytes(set.input_dim >> 8);
    int capacity = static_cast<int>((150 * 1024) / image);
    if (capacity > 4) capacity = 4;
    const int per_pass = tokens < capacity ? tokens : capacity;
    if (per_pass <= 1) {
        launch_variant<1, P>(set, first, second, records_out, tokens, stream);
    } else if (per_pass == 2 || capacity < 4) {
        launch_variant<2, P>(set, first, second, records_out, tokens, stream);
    } else {
        launch_variant<4, P>(set, first, second, records_out, tokens, stream);
    }
}

}  // namespace

bool gemv_q8_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return encoding == kEncQ8_0 && input_dim % 256 == 0 &&
        token_image_bytes(input_dim >> 8) <= 150 * 1024;
}

void launch_gemv_q8(const ProjectionSet& set, const float* first, const float* second,
                    std::uint8_t* records_out, int prologue, std::int64_t rows,
                    hipStream_t stream) {
    ProjectionSet group{};
    group.input_dim = set.input_dim;
    for (int index = 0; index < set.count; ++index) {
        if (set.op[index].encoding == kEncQ8_0) group.op[group.count++] = set.op[index];
    }
    if (group.count == 0) return;
    const int tokens = static_cast<int>(rows);
    switch (prologue) {
        case kGated: launch_tokens<kGated>(group, first, second, records_out, tokens, stream); break;
        case kSwiGlu: launch_tokens<kSwiGlu>(group, first, second, records_out, tokens, stream); break;
        case kRecords: launch_tokens<kRecords>(group, first, second, nullptr, tokens, stream); break;
        default: launch_tokens<kPlain>(group, first, second, records_out, tokens, stream); break;
    }
}

}  // namespace nfn
