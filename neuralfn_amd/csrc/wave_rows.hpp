// Pieces shared by the wave-per-row decode kernels (gemv_dot.hip, gemv_q6.hip):
// fixed-order wave reductions on DPP, the activation load with its fused
// prologue, and the cursor that walks a wave's (row, slice) pairs.
#pragma once

#include "common.hpp"

namespace nfn {

template <int CTRL>
__device__ __forceinline__ int dpp_move(int value) {
    return __builtin_amdgcn_update_dpp(0, value, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp_move(float value) {
    return __builtin_bit_cast(float, dpp_move<CTRL>(__builtin_bit_cast(int, value)));
}

constexpr int kQuadXor1 = 0xB1;     // quad_perm [1,0,3,2]
constexpr int kQuadXor2 = 0x4E;     // quad_perm [2,3,0,1]
constexpr int kHalfMirror = 0x141;  // lane k <-> 7-k within 8 lanes
constexpr int kRowMirror = 0x140;   // lane k <-> 15-k within 16 lanes

__device__ __forceinline__ float lane_value(float v, int lane) {
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), lane));
}

// Largest of the wave's values, all of them non-negative: such floats order
// like their bit patterns, so the reduction runs on unsigned integers (one
// instruction per step with the lane exchange folded in).  Butterfly within
// rows of 16 lanes, then row 0 -> 1 and 2 -> 3, then lane 31 -> rows 2 and 3:
// lane 63 holds the result.
__device__ __forceinline__ float wave_max(float value) {
    std::uint32_t v = __float_as_uint(value);
    v = max(v, static_cast<std::uint32_t>(dpp_move<kQuadXor1>(static_cast<int>(v))));
    v = max(v, static_cast<std::uint32_t>(dpp_move<kQuadXor2>(static_cast<int>(v))));
    v = max(v, static_cast<std::uint32_t>(dpp_move<kHalfMirror>(static_cast<int>(v))));
    v = max(v, static_cast<std::uint32_t>(dpp_move<kRowMirror>(static_cast<int>(v))));
    constexpr int kRowBroadcast15 = 0x142, kRowBroadcast31 = 0x143;
    v = max(v, static_cast<std::uint32_t>(__builtin_amdgcn_update_dpp(
                   static_cast<int>(v), static_cast<int>(v), kRowBroadcast15, 0xA, 0xF, false)));
    v = max(v, static_cast<std::uint32_t>(__builtin_amdgcn_update_dpp(
                   static_cast<int>(v), static_cast<int>(v), kRowBroadcast31, 0xC, 0xF, false)));
    return __uint_as_float(static_cast<std::uint32_t>(
        __builtin_amdgcn_readlane(static_cast<int>(v), 63)));
}

// Sum over the wave in a fixed order; the total is returned in every lane.
__device__ __forceinline__ float wave_total(float v) {
    v += dpp_move<kQuadXor1>(v);
    v += dpp_move<kQuadXor2>(v);
    v += dpp_move<kHalfMirror>(v);
    v += dpp_move<kRowMirror>(v);
    return (lane_value(v, 0) + lane_value(v, 16)) + (lane_value(v, 32) + lane_value(v, 48));
}

__device__ __forceinline__ std::uint32_t perm(std::uint32_t hi, std::uint32_t lo, std::uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

constexpr float kCodeRange = 32512.0f;  // 127*256: the high byte stays in [-127, 127]

// Four activations of one lane as 16-bit fixed-point codes, code = x * 32512 /
// (largest magnitude among the wave's 256 values), rounded to nearest even and
// split into two int8 planes: code = 256*hi + lo with lo in [-128, 127].
struct ActivationCodes {
    std::uint32_t hi, lo;  // four bytes each, value order
    int sum;               // of this lane's four codes
    float maximum;         // the wave's largest magnitude; scale = maximum / 32512
};

__device__ __forceinline__ ActivationCodes encode_activations(float4 x) {
    const float local = fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w)));
    ActivationCodes codes;
    codes.maximum = wave_max(local);
    const float inverse =
        codes.maximum > 1.0e-30f ? kCodeRange * __builtin_amdgcn_rcpf(codes.maximum) : 0.0f;
    // 1.5*2^23 + 128: the low 16 bits of the sum's bit pattern are
    // round-to-nearest-even(x*inverse) + 128 in two's complement.
    constexpr float kMagic = 12582912.0f + 128.0f;
    const std::uint32_t u0 = __float_as_uint(fmaf(x.x, inverse, kMagic));
    const std::uint32_t u1 = __float_as_uint(fmaf(x.y, inverse, kMagic));
    const std::uint32_t u2 = __float_as_uint(fmaf(x.z, inverse, kMagic));
    const std::uint32_t u3 = __float_as_uint(fmaf(x.w, inverse, kMagic));
    // code + 128 = 256*hi + (lo + 128): hi is byte 1, lo is byte 0 with its top bit flipped
    const std::uint32_t p01 = perm(u1, u0, 0x05010400u);  // [u0.b0, u1.b0, u0.b1, u1.b1]
    const std::uint32_t p23 = perm(u3, u2, 0x05010400u);
    codes.lo = perm(p23, p01, 0x05040100u) ^ 0x80808080u;
    codes.hi = perm(p23, p01, 0x07060302u);
    codes.sum = (__builtin_amdgcn_sdot4(static_cast<int>(codes.hi), 0x01010101, 0, false) << 8) +
        __builtin_amdgcn_sdot4(static_cast<int>(codes.lo), 0x01010101, 0, false);
    return codes;
}

// Activation record of one (token, 256-value block) in a caller's workspace:
// what a later launch needs to skip the quantization.  [0,256) high plane,
// [256,512) low plane (value order), [512,544) eight int32 sums of the codes
// per 32 values, [544] the scale, [548] the block's largest magnitude.
constexpr int kActRecord = 576;
constexpr int kRecordSums = 512;
constexpr int kRecordScale = 544;
constexpr int kRecordMaximum = 548;

// The four values of lane `column % 256 / 4` of block `column / 256` as the
// kernels' quantizers take them: floats with the prologue applied, or for
// kRecords the raw (high word, low word, maximum) of the stored record.
template <int P>
__device__ __forceinline__ float4 load_activations(const float* __restrict__ first,
                                                   const float* __restrict__ second,
                                                   std::int64_t column) {
    if constexpr (P == kRecords) {
        const std::uint8_t* record =
            reinterpret_cast<const std::uint8_t*>(first) + (column >> 8) * kActRecord;
        const int offset = static_cast<int>(column & 255);  // 4 * lane
        float4 raw;
        raw.x = *reinterpret_cast<const float*>(record + offset);
        raw.y = *reinterpret_cast<const float*>(record + 256 + offset);
        raw.z = *reinterpret_cast<const float*>(record + kRecordMaximum);
        raw.w = 0.0f;
        return raw;
    }
    float4 x = *reinterpret_cast<const float4*>(first + column);
    if constexpr (P == kGated || P == kSwiGlu) {
        const float4 y = *reinterpret_cast<const float4*>(second + column);
        x.x = apply_prologue<P>(x.x, y.x);
        x.y = apply_prologue<P>(x.y, y.y);
        x.z = apply_prologue<P>(x.z, y.z);
        x.w = apply_prologue<P>(x.w, y.w);
    }
    return x;
}

// First input of the pass that starts at token `token0`.
template <int P>
__device__ __forceinline__ const float* pass_input(const float* first, int token0, int input_dim) {
    if constexpr (P == kRecords) {
        return reinterpret_cast<const float*>(reinterpret_cast<const std::uint8_t*>(first) +
                                              static_cast<std::int64_t>(token0) * (input_dim >> 8) * kActRecord);
    } else {
        return first + static_cast<std::int64_t>(token0) * input_dim;
    }
}

// Codes of what load_activations<P> returned.
template <int P>
__device__ __forceinline__ ActivationCodes activation_codes(float4 loaded) {
    if constexpr (P == kRecords) {
        ActivationCodes codes;
        codes.hi = __float_as_uint(loaded.x);
        codes.lo = __float_as_uint(loaded.y);
        codes.maximum = loaded.z;
        codes.sum = (__builtin_amdgcn_sdot4(static_cast<int>(codes.hi), 0x01010101, 0, false) << 8) +
            __builtin_amdgcn_sdot4(static_cast<int>(codes.lo), 0x01010101, 0, false);
        return codes;
    } else {
        return encode_activations(loaded);
    }
}

// Writes the record of one block (four values per lane) for a later launch.
__device__ __forceinline__ void store_record(std::uint8_t* record, int lane,
                                             const ActivationCodes& codes) {
    int sum = codes.sum;  // over the 8 lanes of a 32-value group
    sum += dpp_move<kQuadXor1>(sum);
    sum += dpp_move<kQuadXor2>(sum);
    sum += dpp_move<kHalfMirror>(sum);
    *reinterpret_cast<std::uint32_t*>(record + lane * 4) = codes.hi;
    *reinterpret_cast<std::uint32_t*>(record + 256 + lane * 4) = codes.lo;
    if ((lane & 7) == 0) *reinterpret_cast<int*>(record + kRecordSums + (lane >> 3) * 4) = sum;
    if (lane == 0) {
        *reinterpret_cast<float*>(record + kRecordScale) = codes.maximum * (1.0f / kCodeRange);
        *reinterpret_cast<float*>(record + kRecordMaximum) = codes.maximum;
    }
}

// Token of activation record `record` (records run token by token, `blocks`
// per token).  One token per pass: no division on the way to the first loads.
template <int T>
__device__ __forceinline__ int token_of_record(int record, int blocks) {
    if constexpr (T == 1) {
        return 0;
    } else {
        return record / blocks;
    }
}

// Projection `index` of the set, chosen with scalar selects from fields that
// were all read with static offsets: a dynamically indexed read of the kernel
// arguments is a dependent scalar load, and its first touch of a cache line
// costs a trip to memory in the middle of the kernel.
__device__ __forceinline__ Projection pick(const ProjectionSet& set, int index) {
    Projection p = set.op[0];
#pragma unroll
    for (int k = 1; k < 4; ++k) {
        const bool take = index == k;
        p.data = take ? set.op[k].data : p.data;
        p.output = take ? set.op[k].output : p.output;
        p.output_dim = take ? set.op[k].output_dim : p.output_dim;
        p.row_stride = take ? set.op[k].row_stride : p.row_stride;
        p.first_tile = take ? set.op[k].first_tile : p.first_tile;
    }
    return p;
}

// Walks the (row, iteration) pairs of one wave without divisions: everything
// here is uniform and lives in scalar registers.
struct PairCursor {
    int op;                   // projection index
    Projection current;       // its fields
    std::int64_t local_row;   // row inside that projection
    int iteration;            // which 64-unit slice of the row
    const std::uint8_t* row;  // first byte of the row

    __device__ __forceinline__ void start(const ProjectionSet& set, int global_row) {
        op = 0;
#pragma unroll
        for (int index = 1; index < 4; ++index) {
            if (index < set.count && global_row >= static_cast<int>(set.op[index].first_tile)) op = index;
        }
        current = pick(set, op);
        local_row = global_row - static_cast<int>(current.first_tile);
        iteration = 0;
        row = current.data + local_row * current.row_stride;
    }
    __device__ __forceinline__ void advance(const ProjectionSet& set, int iterations) {
        if (++iteration < iterations) return;
        iteration = 0;
        ++local_row;
        row += current.row_stride;
        if (local_row == current.output_dim && op + 1 < set.count) {
            ++op;
            current = pick(set, op);
            local_row = 0;
            row = current.data;
        }
    }
};

// The rows of one wave.  The launch deals its rows out evenly twice: over the
// workgroups (the first `longer_groups` take one more than `rows_per_group`),
// so that every compute unit streams the same number of bytes, and inside a
// workgroup over its waves (the first few take one more; they sit on different
// SIMDs).  Each wave gets a contiguous range.  No division: the quotients come
// from the host and the wave count is a power of two.
struct WaveRows {
    int begin, count;
};
template <int WAVES>
__device__ __forceinline__ WaveRows wave_rows(int group, int wave, int rows_per_group,
                                              int longer_groups) {
    static_assert((WAVES & (WAVES - 1)) == 0, "waves per workgroup must be a power of two");
    const int group_begin = group * rows_per_group + min(group, longer_groups);
    const int group_rows = rows_per_group + (group < longer_groups ? 1 : 0);
    const int base = group_rows / WAVES;
    const int extra = group_rows % WAVES;
    WaveRows rows;
    rows.begin = group_begin + wave * base + min(wave, extra);
    rows.count = base + (wave < extra ? 1 : 0);
    return rows;
}

// Workgroups of a wave-per-row decode launch.  Small launches are bound by
// fixed costs: waves start at a limited rate and every workgroup quantizes the
// whole activation vector, so one workgroup per compute unit (all resident at
// once, equally loaded) is fastest until a wave would own more than about three
// rows; from there the grid grows to up to four workgroups per unit, which a
// large weight stream needs to keep enough loads in flight.
inline std::int64_t decode_groups(std::int64_t rows, int waves_per_group, int most_per_unit = 4) {
    const std::int64_t units = compute_units();
    std::int64_t per_unit = rows / (units * waves_per_group * 3);
    if (per_unit < 1) per_unit = 1;
    if (per_unit > most_per_unit) per_unit = most_per_unit;
    std::int64_t groups = units * per_unit;
    const std::int64_t useful = (rows + waves_per_group - 1) / waves_per_group;  // a row per wave
    return groups < useful ? groups : useful;
}

}  // namespace nfn
