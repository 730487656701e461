// Device code shared by the float-activation kernels: one wave computes the
// partial dot products of one packed weight row with up to R input rows.
// Weight decode arithmetic: neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616.
#pragma once

#include "common.hpp"

namespace nfn {

template <int R, int P>
__device__ __forceinline__ void load_pair(const float* __restrict__ first,
                                          const float* __restrict__ second,
                                          std::int64_t input_dim, std::int64_t row0,
                                          int active, std::int64_t col, float (&x0)[R],
                                          float (&x1)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (r < active) {
            const std::int64_t offset = (row0 + r) * input_dim + col;
            const float2 a = *reinterpret_cast<const float2*>(first + offset);
            if constexpr (P == kPlain) {
                x0[r] = a.x;
                x1[r] = a.y;
            } else {
                const float2 b = *reinterpret_cast<const float2*>(second + offset);
                x0[r] = apply_prologue<P>(a.x, b.x);
                x1[r] = apply_prologue<P>(a.y, b.y);
            }
        } else {
            x0[r] = 0.0f;
            x1[r] = 0.0f;
        }
    }
}

template <int R, int P>
__device__ __forceinline__ float load_one(const float* __restrict__ first,
                                          const float* __restrict__ second,
                                          std::int64_t offset) {
    if constexpr (P == kPlain) {
        return first[offset];
    } else {
        return apply_prologue<P>(first[offset], second[offset]);
    }
}

// Per-lane partial sums of weight row `row_data` against rows row0..row0+active.
template <int R, int P>
__device__ __forceinline__ void wave_row_partials(
    std::uint32_t encoding, const std::uint8_t* __restrict__ row_data, std::int64_t input_dim,
    const float* __restrict__ first, const float* __restrict__ second, std::int64_t row0,
    int active, int lane, float (&sums)[R]) {
#pragma unroll
    for (int r = 0; r < R; ++r) sums[r] = 0.0f;

    if (encoding == kEncQ4K || encoding == kEncQ5K) {
        const bool q5 = encoding == kEncQ5K;
        const int group = lane >> 4;
        const int byte = (lane & 15) * 2;
        const std::int64_t blocks = input_dim >> 8;
        for (std::int64_t b = 0; b < blocks; ++b) {
            const std::uint8_t* block = row_data + b * (q5 ? 176 : 144);
            const float d = load_half(block);
            const float dmin = load_half(block + 2);
            int sc_lo, m_lo, sc_hi, m_hi;
            k_scale_min(block + 4, group * 2, &sc_lo, &m_lo);
            k_scale_min(block + 4, group * 2 + 1, &sc_hi, &m_hi);
            const std::uint32_t packed = *reinterpret_cast<const std::uint16_t*>(
                block + (q5 ? 48 : 16) + group * 32 + byte);
            int q[4] = {static_cast<int>(packed & 15), static_cast<int>((packed >> 8) & 15),
                        static_cast<int>((packed >> 4) & 15), static_cast<int>(packed >> 12)};
            if (q5) {
                const std::uint32_t high =
                    *reinterpret_cast<const std::uint16_t*>(block + 16 + byte);
                q[0] += ((high >> (2 * group)) & 1) << 4;
                q[1] += ((high >> (8 + 2 * group)) & 1) << 4;
                q[2] += ((high >> (2 * group + 1)) & 1) << 4;
                q[3] += ((high >> (8 + 2 * group + 1)) & 1) << 4;
            }
            const float off_lo = __fmul_rn(dmin, static_cast<float>(m_lo));
            const float off_hi = __fmul_rn(dmin, static_cast<float>(m_hi));
            const float w0 = __fsub_rn(__fmul_rn(d, static_cast<float>(sc_lo * q[0])), off_lo);
            const float w1 = __fsub_rn(__fmul_rn(d, static_cast<float>(sc_lo * q[1])), off_lo);
            const float w2 = __fsub_rn(__fmul_rn(d, static_cast<float>(sc_hi * q[2])), off_hi);
            const float w3 = __fsub_rn(__fmul_rn(d, static_cast<float>(sc_hi * q[3])), off_hi);
            const std::int64_t col = b * 256 + group * 64 + byte;
            float x0[R], x1[R], x2[R], x3[R];
            load_pair<R, P>(first, second, input_dim, row0, active, col, x0, x1);
            load_pair<R, P>(first, second, input_dim, row0, active, col + 32, x2, x3);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                sums[r] = fmaf(x0[r], w0, sums[r]);
                sums[r] = fmaf(x1[r], w1, sums[r]);
                sums[r] = fmaf(x2[r], w2, sums[r]);
                sums[r] = fmaf(x3[r], w3, sums[r]);
            }
        }
    } else if (encoding == kEncQ6K) {
        const int half = lane >> 5;
        const int l32 = lane & 31;
        const std::int64_t blocks = input_dim >> 8;
        for (std::int64_t b = 0; b < blocks; ++b) {
            const std::uint8_t* block = row_data + b * 210;
            const float d = load_half(block + 208);
            const std::uint32_t low_first = block[half * 64 + l32];
            const std::uint32_t low_second = block[half * 64 + 32 + l32];
            const std::uint32_t high = block[128 + half * 32 + l32];
            const std::int8_t* scales =
                reinterpret_cast<const std::int8_t*>(block + 192 + half * 8 + (l32 >> 4));
#pragma unroll
            for (int quarter = 0; quarter < 4; ++quarter) {
                const std::uint32_t low = (quarter & 1) ? low_second : low_first;
                const int nibble = quarter < 2 ? (low & 15) : (low >> 4);
                const int quant = (nibble | (((high >> (2 * quarter)) & 3) << 4)) - 32;
                const float w = __fmul_rn(
                    __fmul_rn(d, static_cast<float>(static_cast<int>(scales[quarter * 2]))),
                    static_cast<float>(quant));
                const std::int64_t col = b * 256 + half * 128 + quarter * 32 + l32;
#pragma unroll
                for (int r = 0; r < R; ++r) {
                    if (r < active) {
                        const float x =
                            load_one<R, P>(first, second, (row0 + r) * input_dim + col);
                        sums[r] = fmaf(x, w, sums[r]);
                    }
                }
            }
        }
    } else {
        // F32, BF16, Q8_0: lane-strided columns through the one-weight decoder.
        for (std::int64_t col = lane; col < input_dim; col += 64) {
            const float w = weight_value(encoding, row_data, col);
#pragma unroll
            for (int r = 0; r < R; ++r) {
                if (r < active) {
                    const float x = load_one<R, P>(first, second, (row0 + r) * input_dim + col);
                    sums[r] = fmaf(x, w, sums[r]);
                }
            }
        }
    }

}

}  // namespace nfn
