// Q6_K decode GEMV on the vector ALUs (v_dot4_i32_i8), with an optional fused
// argmax for the lm_head.
//
// One wave owns whole weight rows.  Its lanes split a row into units of 64
// values: unit (block, half, sixteen) covers positions 16*sixteen .. +15 of all
// four 32-value quarters of one 128-value half of a 210-byte block, which is
// exactly three 16-byte loads (low nibbles of quarters 0/2, of quarters 1/3,
// and the 2-bit tops of all four), so consecutive lanes read neighbouring
// bytes and every loaded byte is used.  The blocks are 2-byte aligned only;
// the 16-byte loads are issued unaligned.  Four int8 sub-scales (one per
// quarter, the format has one per 16 values) and the block's fp16 scale come
// with two small loads from the same cache lines.
//
// Activations become two int8 planes in LDS (16-bit fixed-point codes, one
// scale per 256 values, quantized by the workgroup in the same launch), laid
// out per unit so that consecutive lanes read consecutive 16-byte slots.  The
// format's offset of 32 is applied through the per-16 sums of the codes:
//   y += s*d * sum_quarter sc * (256*dot(q, hi) + dot(q, lo) - 32*sum(codes)).
// The bracket is exact integer arithmetic; one float conversion and one fused
// multiply-add per quarter, one fixed-order butterfly per row.
//
// Every row gets the same arithmetic whatever the number of tokens in the
// launch, the contract of the reference's verifier entry points
// (neuralfn/csrc/native_train/tile_ops.h:685-688).  With the argmax fused in,
// each workgroup keeps the best (value, index) per token and the logits never
// reach memory; the reference runs a linear and an argmax with a logits buffer
// in between (neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:4087-4151),
// ties to the lowest index and NaN never winning as in
// neuralfn/csrc/tile_cuda/kernels.cu:1564-1602.  Block layout:
// neuralfn/csrc/native_gpt2/resident_glimmer.cpp:591-616.
#include "common.hpp"
#include "gemv_q6.hpp"
#include "lm_head.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kWavesPerUnit = 64;  // waves the grid aims at per compute unit
constexpr int kBlockBytes = 210;

struct __attribute__((packed, aligned(2))) Unaligned16 {
    std::uint32_t v[4];
};
struct __attribute__((packed, aligned(2))) Unaligned8 {
    std::uint32_t v[2];
};

// LDS image of one token's activations for a K of `blocks` blocks:
//   planes: eight arrays of `units` 16-byte slots, units = 4*blocks; unit
//           u = 4*block + 2*half + sixteen reads slot u of array 2*quarter + plane
//           (plane 0: high byte, 1: low byte of the codes)
//   sums:   int32[4] per unit: the sum of the 16 codes of each quarter
//   scale:  float per block
struct TokenImage {
    std::uint8_t* planes;
    int* sums;
    float* scale;
};

constexpr int kImageBytesPerBlock = 4 * 128 + 4 * 16 + 16;

__host__ __device__ constexpr int token_image_bytes(std::int64_t blocks) {
    return static_cast<int>(blocks * kImageBytesPerBlock);
}

__device__ __forceinline__ TokenImage token_image(std::uint8_t* lds, int token, int blocks) {
    std::uint8_t* base = lds + token * token_image_bytes(blocks);
    TokenImage image;
    image.planes = base;
    image.sums = reinterpret_cast<int*>(base + blocks * 512);
    image.scale = reinterpret_cast<float*>(base + blocks * 576);
    return image;
}

// Quantize the 256 activations of block `block`, four per lane: lane L holds
// positions 4L..4L+3 = half L/32, quarter (L/8)%4, sixteen (L/4)%2, bytes 4*(L%4)..
__device__ __forceinline__ void quantize_block(const ActivationCodes& codes, int lane, int block,
                                               int blocks, const TokenImage& image) {
    int sum = codes.sum;
    sum += dpp_move<kQuadXor1>(sum);
    sum += dpp_move<kQuadXor2>(sum);
    const int units = 4 * blocks;
    const int quarter = (lane >> 3) & 3;
    const int unit = 4 * block + 2 * (lane >> 5) + ((lane >> 2) & 1);
    std::uint8_t* slot = image.planes + (2 * quarter * units + unit) * 16 + (lane & 3) * 4;
    *reinterpret_cast<std::uint32_t*>(slot) = codes.hi;
    *reinterpret_cast<std::uint32_t*>(slot + units * 16) = codes.lo;
    if ((lane & 3) == 0) image.sums[unit * 4 + quarter] = sum;
    if (lane == 0) image.scale[block] = codes.maximum * (1.0f / kCodeRange);
}

struct Stage {
    Unaligned16 low_a;   // low nibbles: quarter 0, high nibbles: quarter 2
    Unaligned16 low_b;   // low nibbles: quarter 1, high nibbles: quarter 3
    Unaligned16 top;     // two bits per quarter
    Unaligned8 scales;   // the eight int8 sub-scales of the half
    std::uint32_t d_bits;
};

// The packed bytes of one unit: 64 values = positions 16*sixteen .. +15 of the
// four quarters of one half of a block.
struct UnitData {
    std::uint32_t low_a[4];  // low nibbles: quarter 0, high nibbles: quarter 2
    std::uint32_t low_b[4];  // low nibbles: quarter 1, high nibbles: quarter 3
    std::uint32_t top[4];    // two bits per quarter
    std::uint32_t scales_lo, scales_hi;  // the eight int8 sub-scales of the half
    std::uint32_t d_bits;
};

// acc[t] += (activation scale * d) * sum_quarter sc * (256*dot(q,hi) + dot(q,lo) - 32*sum(codes))
// for unit `unit` (= 4*block + 2*half + sixteen inside the row) and every token.
// `later` sends the unit to acc_later instead (a lane of the streaming kernel that is already
// in the wave's next row); the other accumulator takes a product with zero, which leaves it as it is.
template <int T, bool TWO = false>
__device__ __forceinline__ void accumulate_unit(const UnitData& data, std::uint8_t* lds, int blocks,
                                                int unit, bool live, float (&acc)[T],
                                                bool later = false, float* acc_later = nullptr) {
    const int units = 4 * blocks;
    const int block = unit >> 2;
    const int sixteen = unit & 1;
    // 6-bit codes of the four quarters, four bytes per word
    std::uint32_t q[4][4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        const std::uint32_t a = data.low_a[w], b = data.low_b[w], h = data.top[w];
        q[0][w] = (a & 0x0f0f0f0fu) | ((h & 0x03030303u) << 4);
        q[1][w] = (b & 0x0f0f0f0fu) | ((h & 0x0c0c0c0cu) << 2);
        q[2][w] = ((a >> 4) & 0x0f0f0f0fu) | (h & 0x30303030u);
        q[3][w] = ((b >> 4) & 0x0f0f0f0fu) | ((h >> 2) & 0x30303030u);
    }
    // sub-scale of quarter k: byte 2*k + sixteen of the half's eight
    const std::uint32_t s01 = data.scales_lo >> (8 * sixteen);
    const std::uint32_t s23 = data.scales_hi >> (8 * sixteen);
    const float scale_q[4] = {
        static_cast<float>(static_cast<std::int8_t>(s01 & 0xffu)),
        static_cast<float>(static_cast<std::int8_t>((s01 >> 16) & 0xffu)),
        static_cast<float>(static_cast<std::int8_t>(s23 & 0xffu)),
        static_cast<float>(static_cast<std::int8_t>((s23 >> 16) & 0xffu))};
    const float d = half_bits_to_float(data.d_bits);

#pragma unroll
    for (int t = 0; t < T; ++t) {
        const TokenImage image = token_image(lds, t, blocks);
        const std::uint8_t* slot = image.planes + unit * 16;
        const int stride = units * 16;
        const v4i sums = *reinterpret_cast<const v4i*>(image.sums + unit * 4);
        float unit_value = 0.0f;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const v4i hi = *reinterpret_cast<const v4i*>(slot + (2 * k) * stride);
            const v4i lo = *reinterpret_cast<const v4i*>(slot + (2 * k + 1) * stride);
            int dot_hi = 0, dot_lo = 0;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                dot_hi = __builtin_amdgcn_sdot4(static_cast<int>(q[k][w]), hi[w], dot_hi, false);
                dot_lo = __builtin_amdgcn_sdot4(static_cast<int>(q[k][w]), lo[w], dot_lo, false);
            }
            // |256*dot_hi + dot_lo| < 2^26 and 32*|sum| < 2^25: exact in int32
            const int bracket = (dot_hi << 8) + dot_lo - (sums[k] << 5);
            unit_value = fmaf(scale_q[k], static_cast<float>(bracket), unit_value);
        }
        const float scale = image.scale[block];
        const float factor = live ? scale * d : 0.0f;
        if constexpr (TWO) {
            acc[t] = fmaf(later ? 0.0f : factor, unit_value, acc[t]);
            acc_later[t] = fmaf(later ? factor : 0.0f, unit_value, acc_later[t]);
        } else {
            acc[t] = fmaf(factor, unit_value, acc[t]);
        }
    }
}

template <int T, int P, bool ARGMAX>
__global__ __launch_bounds__(kThreads) void gemv_q6_kernel(
    const float* __restrict__ first, const float* __restrict__ second, int tokens, int input_dim,
    int total_rows, int rows_per_group, int longer_groups,
    LmHeadCandidate* __restrict__ candidates, std::uint8_t* __restrict__ records_out,
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
        const std::uint8_t* block = fetch.row + (unit >> 2) * kBlockBytes;
        const int half = (unit >> 1) & 1;
        const int sixteen = unit & 1;
        const std::uint8_t* low = block + half * 64 + sixteen * 16;
        stage.low_a = *reinterpret_cast<const Unaligned16*>(low);
        stage.low_b = *reinterpret_cast<const Unaligned16*>(low + 32);
        stage.top = *reinterpret_cast<const Unaligned16*>(block + 128 + half * 32 + sixteen * 16);
        stage.scales = *reinterpret_cast<const Unaligned8*>(block + 192 + half * 8);
        stage.d_bits = *reinterpret_cast<const std::uint16_t*>(block + 208);
        if (--fetch_left > 0) fetch.advance(set, iterations);
    };
    Stage stage0, stage1;
    issue(stage0);
    issue(stage1);

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
    __syncthreads();

    float acc[T];
    float best_value[T];
    std::int64_t best_index[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        acc[t] = 0.0f;
        best_value[t] = -INFINITY;
        best_index[t] = 0;
    }

    PairCursor work;
    work.start(set, min(row_begin, total_rows - 1));
    auto compute = [&](const Stage& stage) {
        const int iteration = work.iteration;
        const int raw_unit = iteration * kWave + lane;
        const bool live = raw_unit < units;
        const int unit = min(raw_unit, units - 1);

        UnitData data;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            data.low_a[w] = stage.low_a.v[w];
            data.low_b[w] = stage.low_b.v[w];
            data.top[w] = stage.top.v[w];
        }
        data.scales_lo = stage.scales.v[0];
        data.scales_hi = stage.scales.v[1];
        data.d_bits = stage.d_bits;
        accumulate_unit<T>(data, lds, blocks, unit, live, acc);

        if (iteration == iterations - 1) {
            // the row is complete: fixed-order butterfly
            const std::int64_t output_dim = work.current.output_dim;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float total_value = wave_total(acc[t]);
                if constexpr (ARGMAX) {
                    // rows come in increasing order: a strict comparison keeps the lowest index
                    if (total_value > best_value[t]) {
                        best_value[t] = total_value;
                        best_index[t] = work.local_row;
                    }
                } else {
                    float* output = work.current.output + work.local_row;
                    if (lane == 0 && t < pass_tokens) {
                        output[static_cast<std::int64_t>(token0 + t) * output_dim] = total_value;
                    }
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

    if constexpr (ARGMAX) {
        // best of the workgroup per token: waves through LDS (the images are no longer needed)
        __syncthreads();
        float* values = reinterpret_cast<float*>(lds);
        std::int64_t* indices = reinterpret_cast<std::int64_t*>(lds + kWaves * T * 4);
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                values[wave * T + t] = best_value[t];
                indices[wave * T + t] = best_index[t];
            }
        }
        __syncthreads();
        if (threadIdx.x < static_cast<unsigned>(pass_tokens)) {
            const int t = threadIdx.x;
            float value = values[t];
            std::int64_t index = indices[t];
            for (int w = 1; w < kWaves; ++w) better(values[w * T + t], indices[w * T + t], value, index);
            LmHeadCandidate candidate;
            candidate.index = index;
            candidate.value = value;
            candidate.pad = 0;
            candidates[static_cast<std::int64_t>(token0 + t) * gridDim.x + blockIdx.x] = candidate;
        }
    }
}

// ---------------------------------------------------------------------------
// Streaming variant for rows of at least 16 blocks (K >= 4096).
//
// The kernel above gives every lane a coherent unit, which makes each load
// instruction touch sixteen separate 32-byte runs; measured, that pattern tops
// out near 4.4 TB/s whatever the arithmetic.  Here a wave copies its rows —
// contiguous in memory, the descriptor allows no padding — through a private
// LDS staging area instead: per pass 16 blocks, read as 224 consecutive 16-byte
// pieces (four load instructions whose lanes touch neighbouring bytes) and
// written to 224-byte slots, one per block, so that every piece of a block is
// 16-byte aligned in LDS.  Piece 13 of a block holds the block's last 16 bytes
// (bytes 194..209, not 208..223, so that no load reaches past the block); it
// lands at slot offset 208 and puts d at slot offset 222.  The 64 lanes then read one unit each from the slots
// and run the same arithmetic as above.  Nothing but the first barrier (for
// the activation image) synchronises the workgroup; a wave's own LDS accesses
// execute in order.
//
// A pass can straddle two rows (never three: a row is at least 16 blocks), so
// every lane keeps two running sums, for the wave's current row and the next.
// ---------------------------------------------------------------------------
constexpr int kPassBlocks = 16;
constexpr int kSlotBytes = 224;
constexpr int kPiecesPerBlock = 14;
constexpr int kPassPieces = kPassBlocks * kPiecesPerBlock;  // 224 of 256 lane slots
constexpr int kStagingBytes = kPassBlocks * kSlotBytes;

struct PassLoads {
    Unaligned16 piece[4];
};

// W: waves per workgroup (the activation images are shared by the workgroup,
// so more tokens per pass want more waves behind each image).
template <int T, int P, bool ARGMAX, int W>
__global__ __launch_bounds__(W * kWave) void gemv_q6_stream_kernel(
    const float* __restrict__ first, const float* __restrict__ second, std::int64_t input_dim,
    int tokens, int rows_per_wave, LmHeadCandidate* __restrict__ candidates,
    std::uint8_t* __restrict__ records_out, ProjectionSet set) {
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blocks = static_cast<int>(input_dim >> 8);  // per row, >= 16
    const int token0 = blockIdx.y * T;
    const int pass_tokens = min(tokens - token0, T);
    const float* pass_first = pass_input<P>(first, token0, static_cast<int>(input_dim));
    const float* pass_second = P == kGated || P == kSwiGlu
        ? second + static_cast<std::int64_t>(token0) * input_dim : nullptr;
    std::uint8_t* staging = lds + T * token_image_bytes(blocks) + wave * kStagingBytes;

    // rows and blocks of this wave: every projection owns a range of waves
    // (first_tile is its first wave), a wave a contiguous range of its rows
    const int wave_index = static_cast<int>(blockIdx.x) * W + wave;
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && wave_index >= static_cast<int>(set.op[index].first_tile)) which = index;
    }
    const Projection op = pick(set, which);
    const std::int64_t row_begin =
        static_cast<std::int64_t>(wave_index - static_cast<int>(op.first_tile)) * rows_per_wave;
    const int row_count = static_cast<int>(max(
        static_cast<std::int64_t>(0),
        min(static_cast<std::int64_t>(rows_per_wave), op.output_dim - row_begin)));
    const int wave_blocks = row_count * blocks;
    const int passes = (wave_blocks + kPassBlocks - 1) / kPassBlocks;
    // first byte of the wave's first block; a wave without rows points at the
    // last row so that its (unused) loads stay inside the tensor
    const std::uint8_t* stream = op.data +
        min(row_begin, op.output_dim - 1) * op.row_stride;
    const int stream_blocks = max(wave_blocks, 1);  // blocks that may be read from `stream`

    // Blocks are 210 bytes long, so every other block of a tensor that starts on a
    // four-byte boundary starts two bytes past one, and 16-byte loads that are not
    // word aligned run at a fraction of the rate of aligned ones.  Loads 0 and 1
    // of a pass fetch the eight blocks that start on a word (112 pieces, the last
    // 16 lanes repeat the last one), loads 2 and 3 the eight that do not: their
    // pieces are read from two bytes earlier and shifted into place with the first
    // two bytes of the next piece, which the next lane holds.  Piece 13 of such a
    // block is read from byte 194 (aligned; its bytes 12, 13 are what piece 12
    // lacks); piece 13 of an aligned block from byte 196 (aligned; d moves from
    // bytes 12, 13 to the place it has in a read from 194).  That read reaches two
    // bytes into the next block, and a shifted read two bytes into the previous
    // one: a pass that holds the last block of the tensor, or blocks that only
    // stand in for ones past the wave's range, reads every piece the plain way.
    // A tensor that does not start on a word is read the plain way throughout.
    const bool realign = (reinterpret_cast<std::uintptr_t>(op.data) & 3u) == 0;
    const int stream_parity =
        static_cast<int>((reinterpret_cast<std::uintptr_t>(stream) >> 1) & 1u);
    // the tensor's last block as a block of this wave's stream (beyond it for most waves)
    const std::int64_t blocks_to_end =
        (op.output_dim - min(row_begin, op.output_dim - 1)) * static_cast<std::int64_t>(blocks);
    const int tensor_last_block =
        static_cast<int>(min(blocks_to_end - 1, static_cast<std::int64_t>(0x7fffffff)));
    static_assert(kPassBlocks % 2 == 0, "a block of a pass keeps its alignment from pass to pass");
    // passes read the plain way: from plain_from on, and plain_also
    const int plain_from = realign ? stream_blocks / kPassBlocks : 0;
    const int plain_also = tensor_last_block / kPassBlocks;

    // which piece of a pass each of this lane's four loads fetches: loop invariant
    constexpr int kHalfPieces = kPassPieces / 2;  // of the aligned blocks, of the others
    // (source_offset: of the plain read; aligned_step: what the word-aligned read adds to it)
    int source_offset[4], aligned_step[4], target_offset[4], piece_block[4];
    bool last_piece0 = false, last_piece1 = false;  // loads k and k + 2 fetch the same piece of their blocks
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const int piece = min((k & 1) * kWave + lane, kHalfPieces - 1);
        const int pair = piece / kPiecesPerBlock;  // block pair of the pass
        const int within = piece - pair * kPiecesPerBlock;
        const int block = 2 * pair + ((k >> 1) ^ stream_parity);
        piece_block[k] = block;
        source_offset[k] = within == 13 ? 194 : within * 16;
        aligned_step[k] = k < 2 ? (within == 13 ? 2 : 0) : (within == 13 ? 0 : -2);
        target_offset[k] = block * kSlotBytes + within * 16;
        if (k == 0) last_piece0 = within == 13;
        if (k == 1) last_piece1 = within == 13;
    }
    auto issue = [&](PassLoads& loads, int pass) {
        const bool plain = pass >= plain_from || pass == plain_also;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            // blocks past the wave's range are read from its last block instead
            const int block = min(pass * kPassBlocks + piece_block[k], stream_blocks - 1);
            loads.piece[k] = *reinterpret_cast<const Unaligned16*>(
                stream + static_cast<std::int64_t>(block) * kBlockBytes + source_offset[k] +
                (plain ? 0 : aligned_step[k]));
        }
    };

    // (1) activations of the first records this wave quantizes, then (2) the
    // packed bytes of the first two passes: all in flight together
    const int records = pass_tokens * blocks;
    constexpr int kEarly = 4;
    float4 early[kEarly];
#pragma unroll
    for (int e = 0; e < kEarly; ++e) {
        const int record = min(wave + e * W, records - 1);
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        early[e] = load_activations<P>(
            pass_first, pass_second,
            static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
    }
    PassLoads loads0, loads1;
    issue(loads0, 0);

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
        const int record = wave + e * W;
        if (record < records) quantize_record(early[e], record);
    }
    for (int record = wave + kEarly * W; record < records; record += W) {
        const int token = token_of_record<T>(record, blocks);
        const int block = record - token * blocks;
        const float4 x = load_activations<P>(
            pass_first, pass_second,
            static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
        quantize_record(x, record);
    }
    // the second pass's weights are requested only now: requests that go out ahead of the
    // activation loads of waves that start later delay those, and every wave waits at
    // the barrier for all activations
    issue(loads1, min(1, max(passes - 1, 0)));
    __syncthreads();

    float acc_current[T], acc_next[T];
    float best_value[T];
    std::int64_t best_index[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
        acc_current[t] = 0.0f;
        acc_next[t] = 0.0f;
        best_value[t] = -INFINITY;
        best_index[t] = 0;
    }
    int row = 0;                 // current row, relative to row_begin
    int row_first_block = 0;     // its first block in the wave's stream
    const int my_block = lane >> 2;  // block of this lane's unit inside a pass
    const int my_unit = lane & 3;    // 2*half + sixteen
    const std::uint8_t* my_slot = staging + my_block * kSlotBytes;
    const int half = my_unit >> 1;
    const int sixteen = my_unit & 1;

    auto consume = [&](const PassLoads& loads, int pass) {
        // stage: every lane writes its pieces (lanes 32..63 of the fourth load hold
        // duplicates of the last piece and write the same bytes to the same place)
        if (pass >= plain_from || pass == plain_also) {
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                *reinterpret_cast<u32x4*>(staging + target_offset[k]) =
                    u32x4{loads.piece[k].v[0], loads.piece[k].v[1], loads.piece[k].v[2],
                          loads.piece[k].v[3]};
            }
        } else {
            // aligned blocks: only d of piece 13 moves
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const std::uint32_t v3 = loads.piece[k].v[3];
                *reinterpret_cast<u32x4*>(staging + target_offset[k]) =
                    u32x4{loads.piece[k].v[0], loads.piece[k].v[1], loads.piece[k].v[2],
                          (k == 0 ? last_piece0 : last_piece1) ? v3 << 16 : v3};
            }
            // the others: two bytes up, the last two from the next piece (piece 13 as read)
            const std::uint32_t give2 = last_piece0 ? loads.piece[2].v[3] : loads.piece[2].v[0];
            const std::uint32_t give3 = last_piece1 ? loads.piece[3].v[3] : loads.piece[3].v[0];
#pragma unroll
            for (int k = 2; k < 4; ++k) {
                const std::uint32_t v0 = loads.piece[k].v[0], v1 = loads.piece[k].v[1];
                const std::uint32_t v2 = loads.piece[k].v[2], v3 = loads.piece[k].v[3];
                // the next piece's word: from the next lane, for lane 63 from lane 0 of the next load
                const std::uint32_t wrapped = k == 2 ? __builtin_amdgcn_readfirstlane(give3) : 0u;
                const std::uint32_t next = static_cast<std::uint32_t>(__builtin_amdgcn_update_dpp(
                    static_cast<int>(wrapped), static_cast<int>(k == 2 ? give2 : give3),
                    0x130 /* wave_shl:1 */, 0xf, 0xf, false));
                const std::uint32_t shift = (k == 2 ? last_piece0 : last_piece1) ? 0u : 16u;
                *reinterpret_cast<u32x4*>(staging + target_offset[k]) =
                    u32x4{__builtin_amdgcn_alignbit(v1, v0, shift), __builtin_amdgcn_alignbit(v2, v1, shift),
                          __builtin_amdgcn_alignbit(v3, v2, shift), __builtin_amdgcn_alignbit(next, v3, shift)};
            }
        }
        // read back this lane's unit
        UnitData data;
        const u32x4 a = *reinterpret_cast<const u32x4*>(my_slot + half * 64 + sixteen * 16);
        const u32x4 b = *reinterpret_cast<const u32x4*>(my_slot + half * 64 + 32 + sixteen * 16);
        const u32x4 h = *reinterpret_cast<const u32x4*>(my_slot + 128 + half * 32 + sixteen * 16);
        const uint2 sc = *reinterpret_cast<const uint2*>(my_slot + 192 + half * 8);
        data.d_bits = *reinterpret_cast<const std::uint16_t*>(my_slot + 222);
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            data.low_a[w] = a[w];
            data.low_b[w] = b[w];
            data.top[w] = h[w];
        }
        data.scales_lo = sc.x;
        data.scales_hi = sc.y;

        const int stream_block = pass * kPassBlocks + my_block;
        const bool live = stream_block < wave_blocks;
        const int row_end_block = row_first_block + blocks;
        const bool in_next = stream_block >= row_end_block;
        // block inside its row, clamped for dead lanes
        const int block_in_row =
            min(stream_block - (in_next ? row_end_block : row_first_block), blocks - 1);
        const int unit = 4 * block_in_row + my_unit;
        accumulate_unit<T, true>(data, lds, blocks, unit, live, acc_current, in_next, acc_next);

        // the current row ends inside this pass: reduce and emit it
        if (row_end_block <= (pass + 1) * kPassBlocks && row < row_count) {
            // A row that does not start on a pass boundary has its units 4 * row_first_block
            // lanes further on than a row that does.  The butterfly must see every row the same
            // way, whatever the wave's range of rows (which changes with the launch's shape and
            // token count): move unit class u % 64 back to lane u % 64 first.
            const int turned = (4 * row_first_block) & 63;
#pragma unroll
            for (int t = 0; t < T; ++t) {
                float row_sum = acc_current[t];
                if (turned != 0) {
                    row_sum = __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(
                        ((lane + turned) & 63) << 2, __builtin_bit_cast(int, row_sum)));
                }
                const float total_value = wave_total(row_sum);
                if constexpr (ARGMAX) {
                    // rows come in increasing order: a strict comparison keeps the lowest index
                    if (total_value > best_value[t]) {
                        best_value[t] = total_value;
                        best_index[t] = row_begin + row;
                    }
                } else {
                    if (lane == 0 && t < pass_tokens) {
                        op.output[static_cast<std::int64_t>(token0 + t) * op.output_dim +
                                  row_begin + row] = total_value;
                    }
                }
                acc_current[t] = acc_next[t];
                acc_next[t] = 0.0f;
            }
            ++row;
            row_first_block = row_end_block;
        }
    };

    for (int pass = 0; pass < passes; pass += 2) {
        consume(loads0, pass);
        issue(loads0, min(pass + 2, passes - 1));
        if (pass + 1 < passes) consume(loads1, pass + 1);
        issue(loads1, min(pass + 3, passes - 1));
    }

    if constexpr (ARGMAX) {
        // best of the workgroup per token: waves through LDS (the images are no longer needed)
        __syncthreads();
        float* values = reinterpret_cast<float*>(lds);
        std::int64_t* indices = reinterpret_cast<std::int64_t*>(lds + W * T * 4);
        if (lane == 0) {
#pragma unroll
            for (int t = 0; t < T; ++t) {
                values[wave * T + t] = best_value[t];
                indices[wave * T + t] = best_index[t];
            }
        }
        __syncthreads();
        if (threadIdx.x < static_cast<unsigned>(pass_tokens)) {
            const int t = threadIdx.x;
            float value = values[t];
            std::int64_t index = indices[t];
            for (int w = 1; w < W; ++w) better(values[w * T + t], indices[w * T + t], value, index);
            LmHeadCandidate candidate;
            candidate.index = index;
            candidate.value = value;
            candidate.pad = 0;
            candidates[static_cast<std::int64_t>(token0 + t) * gridDim.x + blockIdx.x] = candidate;
        }
    }
}

struct Geometry {
    std::int64_t rows_per_wave;
    std::int64_t groups;
};

Geometry geometry(std::int64_t rows) {
    // about kWavesPerUnit waves per compute unit: the activation quantization
    // (done once per workgroup) stays a small part of a workgroup's work
    const std::int64_t waves_wanted = static_cast<std::int64_t>(compute_units()) * kWavesPerUnit;
    Geometry g;
    g.rows_per_wave = rows / waves_wanted;
    if (g.rows_per_wave < 1) g.rows_per_wave = 1;
    g.groups = (rows + g.rows_per_wave * kWaves - 1) / (g.rows_per_wave * kWaves);
    return g;
}

// The launchers return the number of workgroups along x of their (last)
// launch: with the argmax fused in, that is the number of candidates per token.
template <int T, int P, bool ARGMAX>
std::int64_t launch_variant(ProjectionSet set, const float* first, const float* second,
                            std::uint8_t* records_out, int tokens, LmHeadCandidate* candidates,
                            hipStream_t stream) {
    std::int64_t rows = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = static_cast<std::uint32_t>(rows);  // first row here
        rows += set.op[index].output_dim;
    }
    std::size_t lds = static_cast<std::size_t>(T) * token_image_bytes(set.input_dim >> 8);
    if (lds < 1024) lds = 1024;  // room for the per-wave candidates
    auto kernel = gemv_q6_kernel<T, P, ARGMAX>;
    allow_large_lds<gemv_q6_kernel<T, P, ARGMAX>>();
    const std::int64_t groups = decode_groups(rows, kWaves);
    const int passes = (tokens + T - 1) / T;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), passes), dim3(kThreads), lds,
                       stream, first, second, tokens, static_cast<int>(set.input_dim),
                       static_cast<int>(rows), static_cast<int>(rows / groups),
                       static_cast<int>(rows % groups), candidates, records_out, set);
    return groups;
}

// Rows per wave of the streaming kernel: whole multiples of eight rows once
// there are enough rows, so that a wave's block count is a multiple of the 16
// blocks of a pass for the common row lengths (26 blocks at K = 6656).
Geometry stream_geometry(std::int64_t rows, int waves_per_group) {
    Geometry g = geometry(rows);
    if (g.rows_per_wave >= 8) g.rows_per_wave &= ~std::int64_t(7);
    // few rows: up to eight per wave, as many as one workgroup per compute
    // unit would get, so that a workgroup's quantization of the activations
    // serves more than a handful of rows
    const std::int64_t resident = static_cast<std::int64_t>(compute_units()) * waves_per_group;
    const std::int64_t share = (rows + resident - 1) / resident;
    if (g.rows_per_wave < 8) g.rows_per_wave = share < 8 ? share : 8;
    g.groups = (rows + g.rows_per_wave * waves_per_group - 1) / (g.rows_per_wave * waves_per_group);
    return g;
}

// waves per workgroup of the streaming kernel for T tokens per pass
constexpr int stream_waves(int tokens_per_pass) {
    return tokens_per_pass <= 2 ? 8 : 16;
}

template <int T, int P, bool ARGMAX, int W = stream_waves(T)>
std::int64_t launch_stream(const ProjectionSet& set, const float* first, const float* second,
                           std::uint8_t* records_out, int tokens, LmHeadCandidate* candidates,
                           hipStream_t stream) {
    const std::size_t lds = static_cast<std::size_t>(T) * token_image_bytes(set.input_dim >> 8) +
        W * kStagingBytes;
    auto kernel = gemv_q6_stream_kernel<T, P, ARGMAX, W>;
    allow_large_lds<gemv_q6_stream_kernel<T, P, ARGMAX, W>>();
    const int passes = (tokens + T - 1) / T;
    // one launch: the projections take consecutive ranges of waves
    std::int64_t rows = 0;
    for (int index = 0; index < set.count; ++index) rows += set.op[index].output_dim;
    const std::int64_t rows_per_wave = stream_geometry(rows, W).rows_per_wave;
    ProjectionSet placed = set;
    std::int64_t waves = 0;
    for (int index = 0; index < placed.count; ++index) {
        placed.op[index].first_tile = static_cast<std::uint32_t>(waves);
        waves += (placed.op[index].output_dim + rows_per_wave - 1) / rows_per_wave;
    }
    const std::int64_t groups = (waves + W - 1) / W;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), passes), dim3(W * kWave), lds,
                       stream, first, second, set.input_dim, tokens, static_cast<int>(rows_per_wave),
                       candidates, records_out, placed);
    return groups;
}

bool streams(std::int64_t input_dim) { return (input_dim >> 8) >= kPassBlocks; }

template <int P, bool ARGMAX>
std::int64_t launch_tokens(const ProjectionSet& set, const float* first, const float* second,
                           std::uint8_t* records_out, int tokens, LmHeadCandidate* candidates,
                           hipStream_t stream) {
    // the token images of one pass (and the staging areas) must fit in LDS
    const std::int64_t image = token_image_bytes(set.input_dim >> 8);
    int capacity = static_cast<int>((150 * 1024 - 16 * kStagingBytes) / image);
    if (capacity > 4) capacity = 4;
    const int per_pass = tokens < capacity ? tokens : capacity;
    if (streams(set.input_dim)) {
        if (per_pass <= 1) {
            // rows of 48 blocks and more: sixteen waves share a workgroup's quantization of the
            // activations and stream side by side (19,968 -> 6,656: 29.9 -> 27.3 us, 12,288 ->
            // 6,656: 18.9 -> 16.6 us; rows of 26 blocks lose 10 % to it)
            if (set.input_dim >= 48 * 256) {
                return launch_stream<1, P, ARGMAX, 16>(set, first, second, records_out, tokens, candidates,
                                                       stream);
            }
            return launch_stream<1, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
        }
        if (per_pass == 2 || capacity < 4) {
            return launch_stream<2, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
        }
        return launch_stream<4, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
    }
    if (per_pass <= 1) {
        return launch_variant<1, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
    }
    if (per_pass == 2 || capacity < 4) {
        return launch_variant<2, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
    }
    return launch_variant<4, P, ARGMAX>(set, first, second, records_out, tokens, candidates, stream);
}

}  // namespace

bool gemv_q6_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return encoding == kEncQ6K && input_dim % 256 == 0 &&
        token_image_bytes(input_dim >> 8) <= 150 * 1024 - 16 * kStagingBytes;
}

void launch_gemv_q6(const ProjectionSet& set, const float* first, const float* second,
                    std::uint8_t* records_out, int prologue, std::int64_t rows,
                    hipStream_t stream) {
    ProjectionSet group{};
    group.input_dim = set.input_dim;
    for (int index = 0; index < set.count; ++index) {
        if (set.op[index].encoding == kEncQ6K) group.op[group.count++] = set.op[index];
    }
    if (group.count == 0) return;
    const int tokens = static_cast<int>(rows);
    switch (prologue) {
        case kGated:
            launch_tokens<kGated, false>(group, first, second, records_out, tokens, nullptr, stream);
            break;
        case kSwiGlu:
            launch_tokens<kSwiGlu, false>(group, first, second, records_out, tokens, nullptr, stream);
            break;
        case kRecords:
            launch_tokens<kRecords, false>(group, first, second, nullptr, tokens, nullptr, stream);
            break;
        default:
            launch_tokens<kPlain, false>(group, first, second, records_out, tokens, nullptr, stream);
            break;
    }
}

std::int64_t lm_head_q6_max_groups(std::int64_t output_dim) {
    // the eight-wave workgroups of the one- and two-token streaming kernel are the most numerous
    const std::int64_t a = stream_geometry(output_dim, stream_waves(1)).groups;
    const std::int64_t b = decode_groups(output_dim, kWaves);
    return a > b ? a : b;
}

void launch_lm_head_q6(const Descriptor& descriptor, const float* input, std::int64_t rows,
                       LmHeadCandidate* candidates, std::int64_t* indices, float* maxima,
                       hipStream_t stream) {
    ProjectionSet set{};
    set.count = 1;
    set.input_dim = descriptor.input_dim;
    set.op[0].data = descriptor.data;
    set.op[0].output = nullptr;
    set.op[0].output_dim = descriptor.output_dim;
    set.op[0].row_stride = descriptor.row_stride_bytes;
    set.op[0].encoding = descriptor.encoding;
    const std::int64_t groups =
        launch_tokens<kPlain, true>(set, input, nullptr, nullptr, static_cast<int>(rows), candidates,
                                    stream);
    launch_lm_head_final(candidates, groups, indices, maxima, rows, stream);
}

}  // namespace nfn
