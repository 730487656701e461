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
// folds the 6-bit sub-scales in with integer multiply-adds; two float
// conversions per unit, one butterfly per row.  No LDS round trip for weights,
// no synchronisation after the single barrier.
//
// What the launch is bound by at the sizes of one decode layer (16 MB) is the
// number of instructions a wave issues between its start and its last row, so:
// the arguments the first loads need (activation pointer, the four weight
// pointers as 48-bit addresses, the row split) are the kernel's first 14
// dwords, which arrive in registers at wave start, and everything else sits in
// a struct the kernel reads while those loads are in flight; a lane's byte
// offsets inside a row are computed once and the loads take the row address
// from scalar registers; and with one token and rows of at most two 64-unit
// slices (up to 8,192 columns) a lane's activation operands stay in registers
// for all rows of the launch instead of being read from LDS for every unit.
//
// Every row gets the same arithmetic whatever the number of tokens in the
// launch (T token planes are walked one after another against the same
// unpacked weights), which is the contract of the reference's verifier entry
// points (neuralfn/csrc/native_train/tile_ops.h:685-688) and of its one-row
// kernel (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:714-890).  With x = s*c,
// c = 256*hi + lo:  y += s*(d*sum_sub sc*dot(q, c) - dmin*sum_sub m*sum(c)).
#include "common.hpp"
#include "gemv_dot.hpp"
#include "rms_device.hpp"
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

// The activation operands of one unit for one token: the two int8 planes of
// both sub-blocks (two 16-value halves each), the sub-blocks' code sums and the
// block's scale.
struct UnitActivations {
    v4i a_hi[2], a_lo[2], b_hi[2], b_lo[2];
    int2 sums;
    float scale;
};

__device__ __forceinline__ UnitActivations load_unit_activations(const std::uint8_t* lds, int token,
                                                                 int unit, int blocks) {
    const TokenImage image = token_image(const_cast<std::uint8_t*>(lds), token, blocks);
    const int units = 4 * blocks;
    const std::uint8_t* slot = image.planes + unit * 16;
    const int stride = units * 16;
    UnitActivations acts;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        acts.a_hi[half] = *reinterpret_cast<const v4i*>(slot + (0 + half) * stride);
        acts.a_lo[half] = *reinterpret_cast<const v4i*>(slot + (2 + half) * stride);
        acts.b_hi[half] = *reinterpret_cast<const v4i*>(slot + (4 + half) * stride);
        acts.b_lo[half] = *reinterpret_cast<const v4i*>(slot + (6 + half) * stride);
    }
    acts.sums = *reinterpret_cast<const int2*>(image.sums + (unit >> 2) * 8 + 2 * (unit & 3));
    acts.scale = image.scale[unit >> 2];
    return acts;
}

// The weights of one unit, unpacked once for all tokens.
struct UnitWeights {
    std::uint32_t low[8], high[8];  // 4-bit (Q5_K: 5-bit) codes of the two sub-blocks, a byte each
    int scale_a, scale_b, min_a, min_b;  // 6-bit sub-block scales and minimums
    float d, dmin;
};

template <bool Q5>
__device__ __forceinline__ UnitWeights unpack_unit(const Stage<Q5>& stage, int pair) {
    UnitWeights weights;
    // the low nibbles are sub-block 2*pair, the high nibbles 2*pair+1
    const std::uint32_t packed[8] = {stage.q0.x, stage.q0.y, stage.q0.z, stage.q0.w,
                                     stage.q1.x, stage.q1.y, stage.q1.z, stage.q1.w};
#pragma unroll
    for (int w = 0; w < 8; ++w) {
        weights.low[w] = packed[w] & 0x0f0f0f0fu;
        weights.high[w] = (packed[w] >> 4) & 0x0f0f0f0fu;
    }
    if constexpr (Q5) {
        const std::uint32_t bits[8] = {stage.h0.x, stage.h0.y, stage.h0.z, stage.h0.w,
                                       stage.h1.x, stage.h1.y, stage.h1.z, stage.h1.w};
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            // bit 2*pair of the high-bit byte belongs to the first sub-block, 2*pair+1 to the second
            const std::uint32_t shifted = bits[w] >> (2 * pair);
            weights.low[w] |= (shifted & 0x01010101u) << 4;
            weights.high[w] |= (shifted & 0x02020202u) << 3;
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
    weights.scale_a = static_cast<int>(scales & 0xffu);
    weights.scale_b = static_cast<int>(scales >> 8);
    weights.min_a = static_cast<int>(minimums & 0xffu);
    weights.min_b = static_cast<int>(minimums >> 8);
    weights.d = half_bits_to_float(stage.header.x & 0xffffu);
    weights.dmin = half_bits_to_float(stage.header.x >> 16);
    return weights;
}

// acc += scale * (d * sum_sub sc * dot(q, codes) - dmin * sum_sub m * sum(codes)) for one
// unit and one token.  `live` is false for the lanes past the end of a row's last slice.
__device__ __forceinline__ float unit_product(const UnitWeights& weights, const UnitActivations& acts,
                                              bool live, float acc) {
    int dot_a_hi = 0, dot_a_lo = 0, dot_b_hi = 0, dot_b_lo = 0;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
        for (int v = 0; v < 4; ++v) {
            const int lo_codes = static_cast<int>(weights.low[half * 4 + v]);
            const int hi_codes = static_cast<int>(weights.high[half * 4 + v]);
            dot_a_hi = __builtin_amdgcn_sdot4(lo_codes, acts.a_hi[half][v], dot_a_hi, false);
            dot_a_lo = __builtin_amdgcn_sdot4(lo_codes, acts.a_lo[half][v], dot_a_lo, false);
            dot_b_hi = __builtin_amdgcn_sdot4(hi_codes, acts.b_hi[half][v], dot_b_hi, false);
            dot_b_lo = __builtin_amdgcn_sdot4(hi_codes, acts.b_lo[half][v], dot_b_lo, false);
        }
    }
    // Integer up to the last step: every sub-block scale times its dot product and the
    // sums of two of them stay below 2^24 (31 * 32 * 127 * 63 * 2), so the two
    // conversions are exact and the float code sum is rounded once.
    const int weighted_hi = weights.scale_a * dot_a_hi + weights.scale_b * dot_b_hi;
    const int weighted_lo = weights.scale_a * dot_a_lo + weights.scale_b * dot_b_lo;
    const int weighted_min = weights.min_a * acts.sums.x + weights.min_b * acts.sums.y;
    const float codes = fmaf(static_cast<float>(weighted_hi), 256.0f, static_cast<float>(weighted_lo));
    const float value = fmaf(-weights.dmin, static_cast<float>(weighted_min), weights.d * codes);
    return fmaf(live ? acts.scale : 0.0f, value, acc);
}

// One unit (a 64-value pair of sub-blocks of one block) against the token planes in LDS.
template <bool Q5, int T>
__device__ __forceinline__ void accumulate_unit(const Stage<Q5>& stage, const std::uint8_t* lds,
                                                int unit, bool live, int blocks, float (&acc)[T]) {
    const UnitWeights weights = unpack_unit<Q5>(stage, unit & 3);
#pragma unroll
    for (int t = 0; t < T; ++t) {
        acc[t] = unit_product(weights, load_unit_activations(lds, t, unit, blocks), live, acc[t]);
    }
}

typedef const __attribute__((address_space(1))) std::uint8_t* GlobalBytes;
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(1))) v4u* GlobalVec;

// Arguments the kernel needs late (row ends, prologues): read from the argument
// block while the first loads are in flight.
struct DotTail {
    const float* second;
    std::uint8_t* records_out;
    int tokens;
    int pad;
    float* output[4];
    std::int64_t output_dim[4];
    DualNormArguments norm;  // prologue kDualNorm only
};


// Four 48-bit device addresses in three 64-bit words.
struct PackedPointers {
    std::uint64_t a, b, c;
};
constexpr std::uint64_t kAddressMask = (std::uint64_t(1) << 48) - 1;
inline PackedPointers pack_pointers(const void* const p[4]) {
    std::uint64_t v[4];
    for (int i = 0; i < 4; ++i) v[i] = reinterpret_cast<std::uint64_t>(p[i]) & kAddressMask;
    PackedPointers packed;
    packed.a = v[0] | (v[1] << 48);
    packed.b = (v[1] >> 16) | (v[2] << 32);
    packed.c = (v[2] >> 32) | (v[3] << 16);
    return packed;
}
__device__ __forceinline__ GlobalBytes unpack_pointer(std::uint64_t a, std::uint64_t b,
                                                      std::uint64_t c, int index) {
    const std::uint64_t p0 = a & kAddressMask;
    const std::uint64_t p1 = (a >> 48) | ((b & 0xffffffffull) << 16);
    const std::uint64_t p2 = (b >> 32) | ((c & 0xffffull) << 32);
    const std::uint64_t p3 = c >> 16;
    std::uint64_t p = p0;
    p = index == 1 ? p1 : p;
    p = index == 2 ? p2 : p;
    p = index == 3 ? p3 : p;
    return reinterpret_cast<GlobalBytes>(p);
}

// Walks the (row, 64-unit slice) pairs of one wave; everything is uniform.
// HALF > 0 (pair mode, one projection slot): "row" r stands for row r of the first
// projection followed by row r of the second, HALF slices each.
struct DotCursor {
    int op, row, first_row, next_bound, iteration;
    GlobalBytes row_ptr;
    std::int64_t second_minus_first;  // pair mode: from a row of the first projection to its partner

    __device__ __forceinline__ void bounds(int b1, int b2, int b3) {
        first_row = op == 0 ? 0 : op == 1 ? b1 : op == 2 ? b2 : b3;
        next_bound = op == 0 ? b1 : op == 1 ? b2 : op == 2 ? b3 : 0x7fffffff;
    }
    __device__ __forceinline__ void start(int global_row, std::int64_t stride, std::uint64_t a,
                                          std::uint64_t b, std::uint64_t c, int b1, int b2, int b3) {
        op = (global_row >= b1 ? 1 : 0) + (global_row >= b2 ? 1 : 0) + (global_row >= b3 ? 1 : 0);
        row = global_row;
        iteration = 0;
        bounds(b1, b2, b3);
        row_ptr = unpack_pointer(a, b, c, op) + (row - first_row) * stride;
    }
    template <int HALF>
    __device__ __forceinline__ void advance(int iterations, std::int64_t stride, std::uint64_t a,
                                            std::uint64_t b, std::uint64_t c, int b1, int b2, int b3) {
        ++iteration;
        if constexpr (HALF > 0) {
            if (iteration == HALF) row_ptr += second_minus_first;
            if (iteration < 2 * HALF) return;
            iteration = 0;
            ++row;
            row_ptr += stride - second_minus_first;
            return;
        }
        if (iteration < iterations) return;
        iteration = 0;
        ++row;
        row_ptr += stride;
        if (row == next_bound) {
            ++op;
            bounds(b1, b2, b3);
            row_ptr = unpack_pointer(a, b, c, op);
        }
    }
};

// The leading arguments (14 dwords) arrive in registers at wave start: the first
// activation and weight loads depend on nothing else.  Rows of projection k are
// [bound_k, bound_k+1) of the launch (bound_0 = 0; unused bounds are INT_MAX).
// ITER > 0 (one token only): a row has exactly ITER 64-unit slices, and since a
// lane's units are then the same in every row, their activation operands stay in
// registers for the whole launch instead of being read from LDS per row.
// PAIRS (one token, ITER > 0, two projections of one shape): a wave takes row r of the first
// projection and row r of the second one after the other and stores
// swiglu(first's sum, second's sum) as output r: the gate and up projections of a
// feed-forward block with the activation folded into the row end, so that the down
// projection behind it reads one plain vector.
// WAVES: waves of a workgroup (sixteen for one token over rows of more than 8,192 columns with an
// activation prologue: twice the lanes share the evaluation of the long activation row).
template <std::uint32_t ENC, int T, int P, int ITER, int STAGES, bool PAIRS = false, int WAVES = kDotWaves>
__global__ __launch_bounds__(WAVES * kWave) void gemv_dot_kernel(
    const float* __restrict__ first, std::uint64_t data_a, std::uint64_t data_b,
    std::uint64_t data_c, int input_dim, int rows_per_group, int longer_groups, int bound1,
    int bound2, int bound3, DotTail tail) {
    static_assert(ITER == 0 || (T == 1 && ITER <= 2), "register-resident activations: one token, two slices");
    static_assert(!PAIRS || (ITER > 0 && P == kPlain), "pair mode: register-resident activations, plain input");
    constexpr int kHalf = PAIRS ? ITER : 0;
    constexpr bool kQ5 = ENC == kEncQ5K;
    constexpr int kBlockBytes = kQ5 ? 176 : 144;
    constexpr int kQuants = kQ5 ? 48 : 16;
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int blocks = input_dim >> 8;
    const int units = 4 * blocks;
    const int iterations = PAIRS ? 2 * ITER : ITER > 0 ? ITER : (units + kWave - 1) / kWave;
    const int token0 = blockIdx.y * T;
    const int pass_tokens = T == 1 ? 1 : min(tail.tokens - token0, T);
    const float* pass_first = pass_input<P>(first, token0, input_dim);
    const float* pass_second = P == kGated || P == kSwiGlu
        ? tail.second + static_cast<std::int64_t>(token0) * input_dim : nullptr;
    const std::int64_t stride = static_cast<std::int64_t>(blocks) * kBlockBytes;

    // rows of this wave: dealt out evenly over the workgroups, then over the waves
    const WaveRows mine =
        wave_rows<WAVES>(static_cast<int>(blockIdx.x), wave, rows_per_group, longer_groups);
    const int row_begin = mine.begin;
    const int row_count = mine.count;
    const int total = row_count * iterations;

    // (1) activations of the first records this wave quantizes: loaded first so
    // that their short latency does not queue behind the weight loads.  All
    // loads are unconditional (clamped indices) to keep the load counters exact.
    const int records = pass_tokens * blocks;
    // (rows of more than 8,192 columns: eight, i.e. every record of a 16,384-column row)
    constexpr int kEarly = ITER > 0 ? 4 : 8;
    float4 early[kEarly];
    constexpr int kNormLoaders = (WAVES * kWave) / kRmsThreads;
    DualRmsOperands<kNormLoaders> norm_operands;
    if constexpr (P == kDualNorm) {
        // the operands of the two normalisations instead: `first` is the row to normalise
        dual_rms_request<kNormLoaders>(norm_operands, first, tail.norm.residual,
                                       tail.norm.first_weight, tail.norm.second_weight, input_dim);
    } else {
#pragma unroll
        for (int e = 0; e < kEarly; ++e) {
            const int record = min(wave + e * WAVES, records - 1);
            const int token = token_of_record<T>(record, blocks);
            const int block = record - token * blocks;
            early[e] = load_activations<P>(pass_first, pass_second,
                                           static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
        }
    }

    // (2) weight loads of the first two (row, slice) pairs.  A stage beyond the wave's
    // last pair loads one fixed address in every lane (one cache line per instruction),
    // so the number of loads in flight is the same on every path.
    DotCursor fetch;
    fetch.second_minus_first = PAIRS ? unpack_pointer(data_a, data_b, data_c, 1) -
            unpack_pointer(data_a, data_b, data_c, 0) : 0;
    fetch.start(row_count > 0 ? row_begin : 0, stride, data_a, data_b, data_c, bound1, bound2, bound3);
    int fetch_left = total;  // pairs not fetched yet
    // A lane's byte offsets inside a row depend on the slice only (and a slice of a
    // two-slice row always lands in the same stage): computed once, added to the
    // uniform row address by the load instruction itself.
    auto unit_offset = [&](int slice) {
        const int unit = min(slice * kWave + lane, units - 1);
        return (unit >> 2) * kBlockBytes;
    };
    auto quant_offset = [&](int slice) {
        const int unit = min(slice * kWave + lane, units - 1);
        return (unit >> 2) * kBlockBytes + kQuants + (unit & 3) * 32;
    };
    const int block_offsets[2] = {unit_offset(0), unit_offset(1)};
    const int quant_offsets[2] = {quant_offset(0), quant_offset(1)};
    auto issue = [&](Stage<kQ5>& stage, int slice) {
        const bool real = fetch_left > 0;
        std::uint32_t block_offset, quants_offset;
        if constexpr (ITER > 0) {
            block_offset = real ? block_offsets[slice % ITER] : 0;
            quants_offset = real ? quant_offsets[slice % ITER] : 0;
        } else {
            const int unit = real ? min(fetch.iteration * kWave + lane, units - 1) : 0;
            block_offset = (unit >> 2) * kBlockBytes;
            quants_offset = block_offset + kQuants + (unit & 3) * 32;
        }
        GlobalBytes block = fetch.row_ptr + block_offset;
        const v4u header = *reinterpret_cast<GlobalVec>(block);
        GlobalBytes quants = fetch.row_ptr + quants_offset;
        const v4u q0 = *reinterpret_cast<GlobalVec>(quants);
        const v4u q1 = *reinterpret_cast<GlobalVec>(quants + 16);
        stage.header = make_uint4(header.x, header.y, header.z, header.w);
        stage.q0 = make_uint4(q0.x, q0.y, q0.z, q0.w);
        stage.q1 = make_uint4(q1.x, q1.y, q1.z, q1.w);
        if constexpr (kQ5) {
            const v4u h0 = *reinterpret_cast<GlobalVec>(block + 16);
            const v4u h1 = *reinterpret_cast<GlobalVec>(block + 32);
            stage.h0 = make_uint4(h0.x, h0.y, h0.z, h0.w);
            stage.h1 = make_uint4(h1.x, h1.y, h1.z, h1.w);
        }
        if (--fetch_left > 0) {
            fetch.template advance<kHalf>(iterations, stride, data_a, data_b, data_c, bound1, bound2, bound3);
        }
    };
    // STAGES register stages.  Two are requested here; a third only once this wave's
    // activations have arrived (below): weight requests that go out ahead of the activation
    // loads of waves that start later delay those, and with them the barrier every wave
    // waits at (three at the start: 6.0 us per launch of the headline workload; two: 6.0;
    // this way 5.6).  Launches of more than one workgroup per compute unit are faster with
    // two (a 16,384-row projection: 12.3 against 14.0 us).
    // With ITER > 0 the slices of consecutive steps run 0, .., ITER - 1, 0, ..; the loop
    // below is unrolled over the steps after which (stage, slice) repeats.
    static_assert(STAGES == 2 || STAGES == 3, "two or three stages");
    constexpr int kStages = STAGES;
    constexpr int kSlices = PAIRS ? 2 * ITER : ITER > 0 ? ITER : 1;
    constexpr int kPeriod = kStages % kSlices == 0 ? kStages
        : kSlices % kStages == 0                   ? kSlices
                                                   : kStages * kSlices;
    Stage<kQ5> stages[kStages];
    issue(stages[0], 0);
    issue(stages[1], 1 % kSlices);

    // (3) quantize; one barrier; after it the workgroup never synchronises again.
    // The first workgroup also leaves the records in the caller's workspace
    // for a later launch that shares this input.
    std::uint8_t* const records_out = tail.records_out;
    const bool keep_records = P != kRecords && records_out != nullptr && blockIdx.x == 0;
    if constexpr (P == kDualNorm) {
        // Every workgroup normalises the row for itself (the first one also stores the
        // results); the normalized row then waits in LDS where the records are made from it.
        __shared__ __attribute__((aligned(16))) float normalized_row[kRmsOwned * kRmsThreads];
        __shared__ float norm_partials[kRmsThreads + 1];
        dual_rms_finish<kNormLoaders>(norm_operands, input_dim, tail.norm.first_eps,
                                      tail.norm.second_eps, blockIdx.x == 0, tail.norm.hidden,
                                      tail.norm.captured, tail.norm.normalized, normalized_row,
                                      norm_partials);
#pragma unroll
        for (int e = 0; e < kEarly; ++e) {
            const int record = min(wave + e * WAVES, records - 1);
            early[e] = *reinterpret_cast<const float4*>(normalized_row + record * 256 + lane * 4);
        }
    }
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
        const int record = wave + e * WAVES;
        if (record < records) quantize_record(early[e], record);
    }
    if constexpr (P != kDualNorm) {  // (a normalised row has at most 32 records: all early)
        for (int record = wave + kEarly * WAVES; record < records; record += WAVES) {
            const int token = token_of_record<T>(record, blocks);
            const int block = record - token * blocks;
            const float4 x = load_activations<P>(
                pass_first, pass_second,
                static_cast<std::int64_t>(token) * input_dim + block * 256 + lane * 4);
            quantize_record(x, record);
        }
    }
    if constexpr (kStages == 3) issue(stages[2], 2 % kSlices);
    __syncthreads();

    UnitActivations held[ITER > 0 ? ITER : 1];
    if constexpr (ITER > 0) {
#pragma unroll
        for (int slice = 0; slice < ITER; ++slice) {
            held[slice] = load_unit_activations(lds, 0, min(slice * kWave + lane, units - 1), blocks);
        }
    }

    float acc[T];
#pragma unroll
    for (int t = 0; t < T; ++t) acc[t] = 0.0f;

    DotCursor work;
    work.second_minus_first = 0;  // only its row and iteration counters are used in pair mode
    work.start(row_count > 0 ? row_begin : 0, stride, data_a, data_b, data_c, bound1, bound2, bound3);
    float first_total = 0.0f;  // pair mode: the finished sum of the first projection's row
    // `slice`: for ITER > 0 the slice of its row this step works on
    auto compute = [&](const Stage<kQ5>& stage, int slice) {
        const int iteration = work.iteration;
        const int raw_unit = (PAIRS ? iteration % (ITER > 0 ? ITER : 1) : iteration) * kWave + lane;
        const bool live = raw_unit < units;
        const int unit = min(raw_unit, units - 1);
        if constexpr (ITER > 0) {
            acc[0] = unit_product(unpack_unit<kQ5>(stage, lane & 3), held[slice % ITER], live, acc[0]);
        } else {
            accumulate_unit<kQ5, T>(stage, lds, unit, live, blocks, acc);
        }
        if constexpr (PAIRS) {
            if (iteration == ITER - 1) {
                first_total = wave_total(acc[0]);
                acc[0] = 0.0f;
            } else if (iteration == 2 * ITER - 1) {
                const float second_total = wave_total(acc[0]);
                if (lane == 0) {
                    tail.output[0][work.row] = apply_prologue<kSwiGlu>(first_total, second_total);
                }
                acc[0] = 0.0f;
            }
        } else if (iteration == iterations - 1) {
            // the row is complete: fixed-order butterfly, lane 0 writes
            float* base = tail.output[0];
            std::int64_t output_dim = tail.output_dim[0];
#pragma unroll
            for (int k = 1; k < 4; ++k) {
                base = work.op == k ? tail.output[k] : base;
                output_dim = work.op == k ? tail.output_dim[k] : output_dim;
            }
            float* output = base + (work.row - work.first_row);
#pragma unroll
            for (int t = 0; t < T; ++t) {
                const float total_value = wave_total(acc[t]);
                if (lane == 0 && t < pass_tokens) {
                    output[static_cast<std::int64_t>(token0 + t) * output_dim] = total_value;
                }
                acc[t] = 0.0f;
            }
        }
        work.template advance<kHalf>(iterations, stride, data_a, data_b, data_c, bound1, bound2, bound3);
    };

    for (int n = 0; n < total; n += kPeriod) {
#pragma unroll
        for (int k = 0; k < kPeriod; ++k) {
            if (k == 0 || n + k < total) compute(stages[k % kStages], k % kSlices);
            issue(stages[k % kStages], (k + kStages) % kSlices);
        }
    }
}

template <std::uint32_t ENC, int T, int P>
void launch_variant(ProjectionSet set, const float* first, const float* second,
                    std::uint8_t* records_out, int tokens, hipStream_t stream,
                    const DualNormArguments* norm = nullptr) {
    std::int64_t rows = 0;
    int bounds[4] = {0, 0x7fffffff, 0x7fffffff, 0x7fffffff};
    const void* data[4] = {set.op[0].data, set.op[0].data, set.op[0].data, set.op[0].data};
    DotTail tail{};
    tail.second = second;
    tail.records_out = records_out;
    tail.tokens = tokens;
    if (norm != nullptr) tail.norm = *norm;
    for (int index = 0; index < set.count; ++index) {
        bounds[index] = static_cast<int>(rows);
        data[index] = set.op[index].data;
        tail.output[index] = set.op[index].output;
        tail.output_dim[index] = set.op[index].output_dim;
        rows += set.op[index].output_dim;
    }
    const PackedPointers packed = pack_pointers(data);
    const std::int64_t blocks = set.input_dim >> 8;
    const std::size_t lds = static_cast<std::size_t>(T) * token_image_bytes_host(blocks);
    const int passes = (tokens + T - 1) / T;
    // (up to six workgroups per unit: 6,656 -> 65,536 streams at 5.25 TB/s with six, 5.0 with four)
    const std::int64_t groups = decode_groups(rows, kDotWaves, 6);
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), passes), dim3(kDotThreads), lds,
                           stream, first, packed.a, packed.b, packed.c,
                           static_cast<int>(set.input_dim), static_cast<int>(rows / groups),
                           static_cast<int>(rows % groups), bounds[1], bounds[2], bounds[3], tail);
    };
    const std::int64_t slices = (4 * blocks + kWave - 1) / kWave;
    // (the norm prologue keeps 33 KB of static LDS: less room for the dynamic part)
    constexpr int kDynamicLds = (P == kDualNorm ? 120 : 160) * 1024;
    if constexpr (T == 1) {
        // one workgroup per compute unit: three stages, the third requested late
        const bool small = groups <= compute_units();
        if (slices == 1) {
            if (small) {
                allow_large_lds<gemv_dot_kernel<ENC, T, P, 1, 3>>(kDynamicLds);
                launch(gemv_dot_kernel<ENC, T, P, 1, 3>);
            } else {
                allow_large_lds<gemv_dot_kernel<ENC, T, P, 1, 2>>(kDynamicLds);
                launch(gemv_dot_kernel<ENC, T, P, 1, 2>);
            }
            return;
        }
        if (slices == 2) {
            if (small) {
                allow_large_lds<gemv_dot_kernel<ENC, T, P, 2, 3>>(kDynamicLds);
                launch(gemv_dot_kernel<ENC, T, P, 2, 3>);
            } else {
                allow_large_lds<gemv_dot_kernel<ENC, T, P, 2, 2>>(kDynamicLds);
                launch(gemv_dot_kernel<ENC, T, P, 2, 2>);
            }
            return;
        }
        if (small) {
            if constexpr (P == kGated || P == kSwiGlu) {
                // rows of more than 8,192 columns behind an activation prologue: sixteen waves per
                // workgroup share its evaluation (16,384 -> 6,656 with SwiGLU: 16.4 -> 15.6 us; the
                // plain input gains nothing from them)
                constexpr int kWide = 2 * kDotWaves;
                const std::int64_t wide_groups = decode_groups(rows, kWide);
                auto kernel = gemv_dot_kernel<ENC, T, P, 0, 3, false, kWide>;
                allow_large_lds<gemv_dot_kernel<ENC, T, P, 0, 3, false, kWide>>(kDynamicLds);
                hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(wide_groups), passes),
                                   dim3(kWide * kWave), lds, stream, first, packed.a, packed.b, packed.c,
                                   static_cast<int>(set.input_dim), static_cast<int>(rows / wide_groups),
                                   static_cast<int>(rows % wide_groups), bounds[1], bounds[2], bounds[3],
                                   tail);
                return;
            }
            allow_large_lds<gemv_dot_kernel<ENC, T, P, 0, 3>>(kDynamicLds);
            launch(gemv_dot_kernel<ENC, T, P, 0, 3>);
            return;
        }
    }
    allow_large_lds<gemv_dot_kernel<ENC, T, P, 0, 2>>(kDynamicLds);
    launch(gemv_dot_kernel<ENC, T, P, 0, 2>);
}

// Pair mode: `set` holds two projections of one shape and one output (slot 0), one token.
template <std::uint32_t ENC>
void launch_pairs(const ProjectionSet& set, const float* input, hipStream_t stream) {
    const std::int64_t pairs = set.op[0].output_dim;
    const void* data[4] = {set.op[0].data, set.op[1].data, set.op[0].data, set.op[0].data};
    DotTail tail{};
    tail.tokens = 1;
    tail.output[0] = set.op[0].output;
    tail.output_dim[0] = pairs;
    const PackedPointers packed = pack_pointers(data);
    const std::int64_t blocks = set.input_dim >> 8;
    const std::size_t lds = static_cast<std::size_t>(token_image_bytes_host(blocks));
    // workgroups as for the 2 x pairs weight rows of the launch, two a compute unit at most (gate
    // and up of 16,384 rows: 24.2 us with two, 24.9 with four, 25.5 with one, 26.7 with six)
    std::int64_t groups = decode_groups(2 * pairs, kDotWaves, 2);
    if (groups > pairs) groups = pairs;
    auto launch = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(groups), 1), dim3(kDotThreads), lds,
                           stream, input, packed.a, packed.b, packed.c,
                           static_cast<int>(set.input_dim), static_cast<int>(pairs / groups),
                           static_cast<int>(pairs % groups), 0x7fffffff, 0x7fffffff, 0x7fffffff, tail);
    };
    const std::int64_t slices = (4 * blocks + kWave - 1) / kWave;
    const bool small = groups <= compute_units();
    if (slices == 1) {
        if (small) {
            allow_large_lds<gemv_dot_kernel<ENC, 1, kPlain, 1, 3, true>>();
            launch(gemv_dot_kernel<ENC, 1, kPlain, 1, 3, true>);
        } else {
            allow_large_lds<gemv_dot_kernel<ENC, 1, kPlain, 1, 2, true>>();
            launch(gemv_dot_kernel<ENC, 1, kPlain, 1, 2, true>);
        }
    } else if (small) {
        allow_large_lds<gemv_dot_kernel<ENC, 1, kPlain, 2, 3, true>>();
        launch(gemv_dot_kernel<ENC, 1, kPlain, 2, 3, true>);
    } else {
        allow_large_lds<gemv_dot_kernel<ENC, 1, kPlain, 2, 2, true>>();
        launch(gemv_dot_kernel<ENC, 1, kPlain, 2, 2, true>);
    }
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

bool gemv_dot_normed_supports(const ProjectionSet& set) {
    // one launch: one encoding; register-resident activations and norm operands
    for (int index = 0; index < set.count; ++index) {
        if (set.op[index].encoding != set.op[0].encoding) return false;
    }
    return set.count > 0 && gemv_dot_supports(set.op[0].encoding, set.input_dim) &&
        set.input_dim <= kRmsOwned * kRmsThreads;
}

void launch_gemv_dot_normed(const ProjectionSet& set, const float* input,
                            const DualNormArguments& norm, hipStream_t stream) {
    if (set.op[0].encoding == kEncQ4K) {
        launch_variant<kEncQ4K, 1, kDualNorm>(set, input, nullptr, nullptr, 1, stream, &norm);
    } else {
        launch_variant<kEncQ5K, 1, kDualNorm>(set, input, nullptr, nullptr, 1, stream, &norm);
    }
}

bool gemv_dot_pairs_supports(std::uint32_t first_encoding, std::uint32_t second_encoding,
                             std::int64_t input_dim) {
    // register-resident activations: rows of at most two 64-unit slices
    return first_encoding == second_encoding && gemv_dot_supports(first_encoding, input_dim) &&
        input_dim <= 8192;
}

void launch_gemv_dot_pairs(const ProjectionSet& set, const float* input, hipStream_t stream) {
    if (set.op[0].encoding == kEncQ4K) {
        launch_pairs<kEncQ4K>(set, input, stream);
    } else {
        launch_pairs<kEncQ5K>(set, input, stream);
    }
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
