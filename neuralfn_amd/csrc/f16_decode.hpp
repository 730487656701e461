// Packed K-quant codes -> fp16 in registers, shared by the matrix-core kernels
// that multiply dequantized weights with fp16 activations (gemm_mfma.hip,
// gemv_f16.hip).  Weight layouts and decode:
// neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616.
#pragma once

#include "common.hpp"

namespace nfn {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ std::uint32_t bits_of(f16x2 value) {
    return __builtin_bit_cast(std::uint32_t, value);
}
__device__ __forceinline__ f16x2 splat(float value) {
    const _Float16 h = static_cast<_Float16>(value);
    return f16x2{h, h};
}

// Two code bytes of `word` (byte indices 2*pair, 2*pair+1) as fp16 (1024+b0, 1024+b1):
// 0x6400 is 1024.0 and its ten mantissa bits count in ones.
template <int PAIR>
__device__ __forceinline__ f16x2 bytes_to_biased_half(std::uint32_t word) {
    constexpr std::uint32_t selector = PAIR == 0 ? 0x04010400u : 0x04030402u;
    return __builtin_bit_cast(f16x2, __builtin_amdgcn_perm(0x64646464u, word, selector));
}

// (bytes + bias) * scale + shift for the four code bytes of `word`
__device__ __forceinline__ void scale_bytes(std::uint32_t word, f16x2 bias, f16x2 scale,
                                            f16x2 shift, std::uint32_t& out0,
                                            std::uint32_t& out1) {
    const f16x2 x0 = bytes_to_biased_half<0>(word) + bias;
    const f16x2 x1 = bytes_to_biased_half<1>(word) + bias;
    out0 = bits_of(__builtin_elementwise_fma(x0, scale, shift));
    out1 = bits_of(__builtin_elementwise_fma(x1, scale, shift));
}

// The fp16 copy of a small batch of activation rows that the small-batch kernel reads
// (gemv_f16.hip): [column / 8][row][8 halfs], every K share of a row (below) scaled by a power
// of two so that its largest magnitude lands near 2^14, and one float per row and share,
// [row][share], to multiply results back.
struct HalfImageScale {
    float factor, inverse;
};
// zero, subnormal-range and infinite maxima keep scale 1
__device__ __forceinline__ HalfImageScale half_image_scale(float largest) {
    const std::uint32_t exponent = (__float_as_uint(largest) >> 23) & 0xffu;
    const bool usable = exponent >= 16u && exponent <= 254u;
    HalfImageScale scale;
    scale.factor = usable ? __uint_as_float((127u + 14u + 127u - exponent) << 23) : 1.0f;
    scale.inverse = usable ? __uint_as_float((exponent - 14u) << 23) : 1.0f;
    return scale;
}
__device__ __forceinline__ float largest_of(float4 x, float largest) {
    return fmaxf(largest, fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
}
// The small-batch kernel's eight waves cut K into shares of whole blocks, share s being blocks
// blocks * s / 8 .. blocks * (s + 1) / 8, and every (row, share) has a scale of its own: a
// wave multiplies its partial sums back before the waves' sums meet.  (One scale per row
// would need the whole row before the first value can be stored; per share, the workgroups
// that convert a row share nothing.)
constexpr int kHalfImageShares = 8;
__host__ __device__ constexpr int half_image_share_begin(int blocks, int share) {
    return blocks * share / kHalfImageShares;
}
// the share that block `block` belongs to
__host__ __device__ constexpr int half_image_share_of(int block, int blocks) {
    return (kHalfImageShares * block + kHalfImageShares - 1) / blocks;
}
// columns 8 group .. 8 group + 7 of row `row` (a, then b) into the image of `rows` rows
__device__ __forceinline__ void half_image_store(std::uint8_t* image, int group, int rows, int row,
                                                 float4 a, float4 b, float factor) {
    const f16x2 h0 = {static_cast<_Float16>(a.x * factor), static_cast<_Float16>(a.y * factor)};
    const f16x2 h1 = {static_cast<_Float16>(a.z * factor), static_cast<_Float16>(a.w * factor)};
    const f16x2 h2 = {static_cast<_Float16>(b.x * factor), static_cast<_Float16>(b.y * factor)};
    const f16x2 h3 = {static_cast<_Float16>(b.z * factor), static_cast<_Float16>(b.w * factor)};
    std::uint8_t* target = image + (static_cast<std::int64_t>(group) * rows + row) * 16;
    *reinterpret_cast<u32x4*>(target) = u32x4{bits_of(h0), bits_of(h1), bits_of(h2), bits_of(h3)};
}

// Q4_K and Q5_K: d, dmin and the 6-bit scale/min pair of sub-blocks 2*pair, 2*pair+1
// out of the block's first 16 bytes
struct KBlockScales {
    std::uint32_t sc, mn;  // low byte: first sub-block, next byte: second
    f16x2 scale_a, shift_a, scale_b, shift_b;
    __device__ __forceinline__ void bits(u32x4 header, int pair) {
        const int shift = 16 * (pair & 1);
        const std::uint32_t ys = header.y >> shift, zs = header.z >> shift, ws = header.w >> shift;
        // sub-blocks 4..7 keep their 6-bit values split over two bytes; bit masks
        // instead of a branch keep the K step free of control flow
        const std::uint32_t upper = 0u - static_cast<std::uint32_t>(pair >> 1);
        sc = (((ws & 0x0f0fu) | ((ys >> 2) & 0x3030u)) & upper) | ((ys & 0x3f3fu) & ~upper);
        mn = ((((ws >> 4) & 0x0f0fu) | ((zs >> 2) & 0x3030u)) & upper) | ((zs & 0x3f3fu) & ~upper);
    }
    __device__ __forceinline__ void scales(u32x4 header) {
        const float d = half_bits_to_float(header.x & 0xffffu);
        const float dmin = half_bits_to_float(header.x >> 16);
        scale_a = splat(d * static_cast<float>(sc & 0xffu));
        scale_b = splat(d * static_cast<float>((sc >> 8) & 0xffu));
        shift_a = splat(-(dmin * static_cast<float>(mn & 0xffu)));
        shift_b = splat(-(dmin * static_cast<float>((mn >> 8) & 0xffu)));
    }
};

}  // namespace nfn
