// Prefill dequant-GEMM on the fp16 matrix cores:
//   Y[M, N] = X[M, K] * W[N, K]^T,  W packed (Q4_K / Q5_K / Q6_K / Q8_0).
//
// A workgroup (4 waves, 2 x 2) owns a 256 x 128 tile of Y and walks K in steps
// of 64.  Per step it
//   - copies its 256 x 64 slice of the activations into LDS with 16-byte loads.
//     The activations are fp16: a pre-pass scales every row by a power of two
//     so that its largest magnitude lands in [2^14, 2^15) and rounds to
//     nearest even; the epilogue multiplies the row's results by the inverse,
//     so neither large nor tiny activations leave the fp16 range,
//   - dequantizes the 128 x 64 slice of the weights: every thread turns 16
//     packed bytes (32 weights of one row) into fp16 in registers with packed
//     fp16 arithmetic (code bytes become 1024+q by a byte permute, then
//     (x-1024)*(d*sc) - dmin*m as one packed fused multiply-add) and writes
//     them to LDS — the packed bytes are read from HBM once per tile column
//     and never exist dequantized in memory,
//   - runs 32 v_mfma_f32_32x32x16_f16 per wave on a 128 x 64 sub-tile with
//     float accumulators.
// LDS is double-buffered and a step is written as 16 phases of two matrix
// instructions each, fenced against reordering, so that the dequantization,
// the LDS traffic and the global loads of later steps are issued in the shadow
// of the matrix instructions; operand fragments are read one K chunk ahead and
// packed bytes two steps ahead.  Rows are padded to 144 bytes so that the
// 16-byte operand reads of 16 lanes hit distinct banks.  Consecutive
// workgroups walk M first: with 8 XCDs picking workgroups round robin each XCD
// keeps one or two 256-row slices of X in its L2 while the packed weights
// stream through.
//
// The reference has no kernel of this kind: its small-batch path stops at 16
// rows (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1326-1328) and more rows run
// the float kernel neuralfn/csrc/tile_cuda/kernels.cu:1398-1525.  Weight
// layouts and decode: neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616.
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace nfn {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 256;
constexpr int kBN = 128;
constexpr int kBK = 64;
constexpr int kThreads = 256;
constexpr int kRowBytes = 144;  // 64 fp16 + 16 bytes of padding
constexpr int kTileA = kBM * kRowBytes;
constexpr int kTileB = kBN * kRowBytes;
constexpr int kStageBytes = kTileA + kTileB;

struct __attribute__((packed, aligned(2))) Chunk16 {
    std::uint32_t v[4];
};

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

// ---------------------------------------------------------------------------
// activations: fp32 -> row-scaled fp16, whole 256-row tiles (rows past the end
// are zeros).  One workgroup per row.
// ---------------------------------------------------------------------------
__global__ __launch_bounds__(256) void convert_activations_kernel(
    const float* __restrict__ input, std::uint16_t* __restrict__ output,
    float* __restrict__ inverse_scale, std::int64_t rows, std::int64_t width) {
    __shared__ float partial[4];
    const std::int64_t row = blockIdx.x;
    const int tid = threadIdx.x;
    uint2* target = reinterpret_cast<uint2*>(output + row * width);
    if (row >= rows) {
        for (std::int64_t i = tid; i < width / 4; i += 256) target[i] = make_uint2(0u, 0u);
        if (tid == 0) inverse_scale[row] = 0.0f;
        return;
    }
    const float4* source = reinterpret_cast<const float4*>(input + row * width);
    float largest = 0.0f;
    for (std::int64_t i = tid; i < width / 4; i += 256) {
        const float4 x = source[i];
        largest = fmaxf(fmaxf(largest, fmaxf(fabsf(x.x), fabsf(x.y))),
                        fmaxf(fabsf(x.z), fabsf(x.w)));
    }
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        largest = fmaxf(largest, __shfl_xor(largest, offset));
    }
    if ((tid & 63) == 0) partial[tid >> 6] = largest;
    __syncthreads();
    largest = fmaxf(fmaxf(partial[0], partial[1]), fmaxf(partial[2], partial[3]));
    // power-of-two scale from the exponent field; zero, subnormal, infinite or
    // NaN maxima keep scale 1
    const std::uint32_t exponent = (__float_as_uint(largest) >> 23) & 0xffu;
    const bool usable = exponent >= 16u && exponent <= 254u;
    const float scale = usable ? __uint_as_float((127u + 14u + 127u - exponent) << 23) : 1.0f;
    const float inverse = usable ? __uint_as_float((exponent - 14u) << 23) : 1.0f;
    for (std::int64_t i = tid; i < width / 4; i += 256) {
        const float4 x = source[i];
        const f16x2 lo = {static_cast<_Float16>(x.x * scale), static_cast<_Float16>(x.y * scale)};
        const f16x2 hi = {static_cast<_Float16>(x.z * scale), static_cast<_Float16>(x.w * scale)};
        target[i] = make_uint2(bits_of(lo), bits_of(hi));
    }
    if (tid == 0) inverse_scale[row] = inverse;
}

// ---------------------------------------------------------------------------
// What one thread holds of the packed weights of one K step: its row's 16
// bytes of codes for positions 16*half .. 16*half+15 of both 32-value groups
// of the step, plus the scale bytes it needs.  prepare() derives the fp16
// scale constants; word<I>() decodes code word I into positions 4I..4I+3 of
// both groups (two packed fp16 pairs each).
// ---------------------------------------------------------------------------
template <std::uint32_t ENC>
struct PackedSlice;

struct AffineConstants {
    f16x2 scale_a, shift_a, scale_b, shift_b;
};

__device__ __forceinline__ AffineConstants k_block_constants(u32x4 header, int pair) {
    const float d = half_bits_to_float(header.x & 0xffffu);
    const float dmin = half_bits_to_float(header.x >> 16);
    const int shift = 16 * (pair & 1);
    const std::uint32_t ys = header.y >> shift, zs = header.z >> shift, ws = header.w >> shift;
    // sub-blocks 4..7 keep their 6-bit values split over two bytes; bit masks
    // instead of a branch keep the K step free of control flow
    const std::uint32_t upper = 0u - static_cast<std::uint32_t>(pair >> 1);
    const std::uint32_t sc = (((ws & 0x0f0fu) | ((ys >> 2) & 0x3030u)) & upper) |
        ((ys & 0x3f3fu) & ~upper);
    const std::uint32_t mn = ((((ws >> 4) & 0x0f0fu) | ((zs >> 2) & 0x3030u)) & upper) |
        ((zs & 0x3f3fu) & ~upper);
    AffineConstants c;
    c.scale_a = splat(d * static_cast<float>(sc & 0xffu));
    c.scale_b = splat(d * static_cast<float>((sc >> 8) & 0xffu));
    c.shift_a = splat(-(dmin * static_cast<float>(mn & 0xffu)));
    c.shift_b = splat(-(dmin * static_cast<float>((mn >> 8) & 0xffu)));
    return c;
}

template <>
struct PackedSlice<kEncQ4K> {
    u32x4 header, codes;
    AffineConstants c;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 144;
        header = *reinterpret_cast<const u32x4*>(p);
        codes = *reinterpret_cast<const u32x4*>(p + 16 + pair * 32 + half * 16);
    }
    __device__ __forceinline__ void prepare(int pair, int) { c = k_block_constants(header, pair); }
    template <int I>
    __device__ __forceinline__ void word(std::uint32_t (&a)[2], std::uint32_t (&b)[2]) const {
        const f16x2 bias = splat(-1024.0f);
        scale_bytes(codes[I] & 0x0f0f0f0fu, bias, c.scale_a, c.shift_a, a[0], a[1]);
        scale_bytes((codes[I] >> 4) & 0x0f0f0f0fu, bias, c.scale_b, c.shift_b, b[0], b[1]);
    }
};

template <>
struct PackedSlice<kEncQ5K> {
    u32x4 header, codes, high;
    AffineConstants c;
    int high_shift;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 176;
        header = *reinterpret_cast<const u32x4*>(p);
        high = *reinterpret_cast<const u32x4*>(p + 16 + half * 16);
        codes = *reinterpret_cast<const u32x4*>(p + 48 + pair * 32 + half * 16);
    }
    __device__ __forceinline__ void prepare(int pair, int) {
        c = k_block_constants(header, pair);
        high_shift = 2 * pair;
    }
    template <int I>
    __device__ __forceinline__ void word(std::uint32_t (&a)[2], std::uint32_t (&b)[2]) const {
        const f16x2 bias = splat(-1024.0f);
        const std::uint32_t bits = high[I] >> high_shift;  // bit 0: first group, bit 1: second
        const std::uint32_t lo = (codes[I] & 0x0f0f0f0fu) | ((bits & 0x01010101u) << 4);
        const std::uint32_t hi = ((codes[I] >> 4) & 0x0f0f0f0fu) | ((bits & 0x02020202u) << 3);
        scale_bytes(lo, bias, c.scale_a, c.shift_a, a[0], a[1]);
        scale_bytes(hi, bias, c.scale_b, c.shift_b, b[0], b[1]);
    }
};

template <>
struct PackedSlice<kEncQ6K> {
    // a K step of 64 is two quarters (32 values each) of one half of the block:
    // quarters (0,1) or (2,3); `pair` = 2*half_of_block + (quarters 2,3 ? 1 : 0)
    u32x4 low_a, low_b, high;
    std::uint32_t sub_scales;  // the four int8 sub-scales of the two quarters
    std::uint32_t d_bits;
    f16x2 scale_a, scale_b;
    int upper;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 210;
        const int block_half = pair >> 1;
        const Chunk16 la = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + half * 16);
        const Chunk16 lb = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + 32 + half * 16);
        const Chunk16 hb = *reinterpret_cast<const Chunk16*>(p + 128 + block_half * 32 + half * 16);
        low_a = u32x4{la.v[0], la.v[1], la.v[2], la.v[3]};
        low_b = u32x4{lb.v[0], lb.v[1], lb.v[2], lb.v[3]};
        high = u32x4{hb.v[0], hb.v[1], hb.v[2], hb.v[3]};
        const std::uint8_t* s = p + 192 + block_half * 8 + (pair & 1) * 4;
        const std::uint32_t s01 = *reinterpret_cast<const std::uint16_t*>(s);
        const std::uint32_t s23 = *reinterpret_cast<const std::uint16_t*>(s + 2);
        sub_scales = s01 | (s23 << 16);
        d_bits = *reinterpret_cast<const std::uint16_t*>(p + 208);
    }
    __device__ __forceinline__ void prepare(int pair, int half) {
        const float d = half_bits_to_float(d_bits);
        // sub-scale index = quarter*2 + position/16: this thread's 16 positions share one
        const int sa = static_cast<std::int8_t>((sub_scales >> (8 * half)) & 0xffu);
        const int sb = static_cast<std::int8_t>((sub_scales >> (8 * (2 + half))) & 0xffu);
        scale_a = splat(d * static_cast<float>(sa));
        scale_b = splat(d * static_cast<float>(sb));
        upper = (pair & 1) * 4;  // quarters 2,3: high nibbles, high-bit pairs 4..7
    }
    template <int I>
    __device__ __forceinline__ void word(std::uint32_t (&a)[2], std::uint32_t (&b)[2]) const {
        const f16x2 bias = splat(-1056.0f);  // 1024 + the format's offset of 32
        const f16x2 zero = splat(0.0f);
        const std::uint32_t top = high[I] >> upper;  // bits 0,1: first quarter; 2,3: second
        const std::uint32_t qa = ((low_a[I] >> upper) & 0x0f0f0f0fu) | ((top & 0x03030303u) << 4);
        const std::uint32_t qb = ((low_b[I] >> upper) & 0x0f0f0f0fu) | ((top & 0x0c0c0c0cu) << 2);
        scale_bytes(qa, bias, scale_a, zero, a[0], a[1]);
        scale_bytes(qb, bias, scale_b, zero, b[0], b[1]);
    }
};

template <>
struct PackedSlice<kEncQ8_0> {
    // a K step of 64 is two 34-byte blocks; `pair` counts K steps inside 256 values
    u32x4 codes_a, codes_b;
    std::uint32_t d_a, d_b;
    f16x2 scale_a, scale_b;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + (block * 8 + pair * 2) * 34;
        const Chunk16 a = *reinterpret_cast<const Chunk16*>(p + 2 + half * 16);
        const Chunk16 b = *reinterpret_cast<const Chunk16*>(p + 34 + 2 + half * 16);
        codes_a = u32x4{a.v[0], a.v[1], a.v[2], a.v[3]};
        codes_b = u32x4{b.v[0], b.v[1], b.v[2], b.v[3]};
        d_a = *reinterpret_cast<const std::uint16_t*>(p);
        d_b = *reinterpret_cast<const std::uint16_t*>(p + 34);
    }
    __device__ __forceinline__ void prepare(int, int) {
        const _Float16 a = __builtin_bit_cast(_Float16, static_cast<std::uint16_t>(d_a));
        const _Float16 b = __builtin_bit_cast(_Float16, static_cast<std::uint16_t>(d_b));
        scale_a = f16x2{a, a};
        scale_b = f16x2{b, b};
    }
    template <int I>
    __device__ __forceinline__ void word(std::uint32_t (&a)[2], std::uint32_t (&b)[2]) const {
        // flipping the sign bit turns the int8 code q into the byte q+128
        const f16x2 bias = splat(-1152.0f);
        const f16x2 zero = splat(0.0f);
        scale_bytes(codes_a[I] ^ 0x80808080u, bias, scale_a, zero, a[0], a[1]);
        scale_bytes(codes_b[I] ^ 0x80808080u, bias, scale_b, zero, b[0], b[1]);
    }
};

// Eight 16-byte chunks of activations in named registers (an array here ends up
// in scratch memory).
struct ActivationSlice {
    u32x4 c0, c1, c2, c3, c4, c5, c6, c7;
};

// the six operand fragments of one K chunk of 16
struct Fragments {
    f16x8 a0, a1, a2, a3, b0, b1;
};

#define NFN_FENCE() __builtin_amdgcn_sched_barrier(0)
#define NFN_MFMA(A, B, C) C = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, B, C, 0, 0, 0)
#define NFN_READ_FRAGMENT(base, row_block, chunk) \
    (*reinterpret_cast<const f16x8*>((base) + (row_block) * 32 * kRowBytes + (chunk) * 32))
#define NFN_WRITE16(target, x, y, z, w) *reinterpret_cast<u32x4*>(target) = u32x4{x, y, z, w}

// One K step for one wave.  `current` are the fragments of K chunk 0 of this
// step (read at the end of the previous one); on return they hold chunk 0 of
// the next step.  The held slice (a_next, b_next) is dequantized into the other
// stage and refilled from global memory.
template <std::uint32_t ENC>
__device__ __forceinline__ void k_step(
    v16f (&acc)[4][2], Fragments& current, const std::uint8_t* a_read, const std::uint8_t* b_read,
    const std::uint8_t* a_read_next, const std::uint8_t* b_read_next, std::uint8_t* a_write,
    std::uint8_t* b_write, ActivationSlice& a_next, PackedSlice<ENC>& b_next, int decode_pair,
    int b_half, const std::uint8_t* a_fetch, std::int64_t a_row_bytes,
    const std::uint8_t* b_global, int fetch_step) {
    Fragments ahead;
    std::uint32_t wa[4][2], wb[4][2];

    // ---- K chunk 0: matrix ops on `current`, read chunk 1, decode ----
    b_next.prepare(decode_pair, b_half);
    ahead.a0 = NFN_READ_FRAGMENT(a_read, 0, 1);
    ahead.a1 = NFN_READ_FRAGMENT(a_read, 1, 1);
    NFN_MFMA(current.a0, current.b0, acc[0][0]);
    NFN_MFMA(current.a0, current.b1, acc[0][1]);
    NFN_FENCE();
    b_next.template word<0>(wa[0], wb[0]);
    ahead.a2 = NFN_READ_FRAGMENT(a_read, 2, 1);
    ahead.a3 = NFN_READ_FRAGMENT(a_read, 3, 1);
    NFN_MFMA(current.a1, current.b0, acc[1][0]);
    NFN_MFMA(current.a1, current.b1, acc[1][1]);
    NFN_FENCE();
    b_next.template word<1>(wa[1], wb[1]);
    ahead.b0 = NFN_READ_FRAGMENT(b_read, 0, 1);
    ahead.b1 = NFN_READ_FRAGMENT(b_read, 1, 1);
    NFN_MFMA(current.a2, current.b0, acc[2][0]);
    NFN_MFMA(current.a2, current.b1, acc[2][1]);
    NFN_FENCE();
    b_next.template word<2>(wa[2], wb[2]);
    NFN_MFMA(current.a3, current.b0, acc[3][0]);
    NFN_MFMA(current.a3, current.b1, acc[3][1]);
    NFN_FENCE();

    // ---- K chunk 1: matrix ops on `ahead`, read chunk 2 into `current`, LDS writes ----
    b_next.template word<3>(wa[3], wb[3]);
    current.a0 = NFN_READ_FRAGMENT(a_read, 0, 2);
    current.a1 = NFN_READ_FRAGMENT(a_read, 1, 2);
    NFN_MFMA(ahead.a0, ahead.b0, acc[0][0]);
    NFN_MFMA(ahead.a0, ahead.b1, acc[0][1]);
    NFN_FENCE();
    NFN_WRITE16(b_write, wa[0][0], wa[0][1], wa[1][0], wa[1][1]);
    NFN_WRITE16(b_write + 16, wa[2][0], wa[2][1], wa[3][0], wa[3][1]);
    NFN_WRITE16(b_write + 64, wb[0][0], wb[0][1], wb[1][0], wb[1][1]);
    NFN_WRITE16(b_write + 80, wb[2][0], wb[2][1], wb[3][0], wb[3][1]);
    current.a2 = NFN_READ_FRAGMENT(a_read, 2, 2);
    current.a3 = NFN_READ_FRAGMENT(a_read, 3, 2);
    NFN_MFMA(ahead.a1, ahead.b0, acc[1][0]);
    NFN_MFMA(ahead.a1, ahead.b1, acc[1][1]);
    NFN_FENCE();
    *reinterpret_cast<u32x4*>(a_write + 0 * 32 * kRowBytes) = a_next.c0;
    *reinterpret_cast<u32x4*>(a_write + 1 * 32 * kRowBytes) = a_next.c1;
    *reinterpret_cast<u32x4*>(a_write + 2 * 32 * kRowBytes) = a_next.c2;
    *reinterpret_cast<u32x4*>(a_write + 3 * 32 * kRowBytes) = a_next.c3;
    current.b0 = NFN_READ_FRAGMENT(b_read, 0, 2);
    current.b1 = NFN_READ_FRAGMENT(b_read, 1, 2);
    NFN_MFMA(ahead.a2, ahead.b0, acc[2][0]);
    NFN_MFMA(ahead.a2, ahead.b1, acc[2][1]);
    NFN_FENCE();
    *reinterpret_cast<u32x4*>(a_write + 4 * 32 * kRowBytes) = a_next.c4;
    *reinterpret_cast<u32x4*>(a_write + 5 * 32 * kRowBytes) = a_next.c5;
    *reinterpret_cast<u32x4*>(a_write + 6 * 32 * kRowBytes) = a_next.c6;
    *reinterpret_cast<u32x4*>(a_write + 7 * 32 * kRowBytes) = a_next.c7;
    NFN_MFMA(ahead.a3, ahead.b0, acc[3][0]);
    NFN_MFMA(ahead.a3, ahead.b1, acc[3][1]);
    NFN_FENCE();

    // ---- K chunk 2: matrix ops on `current`, read chunk 3 into `ahead`, refill from global ----
    const std::uint8_t* a_source = a_fetch + static_cast<std::int64_t>(fetch_step) * (kBK * 2);
    ahead.a0 = NFN_READ_FRAGMENT(a_read, 0, 3);
    ahead.a1 = NFN_READ_FRAGMENT(a_read, 1, 3);
    a_next.c0 = *reinterpret_cast<const u32x4*>(a_source + 0 * 32 * a_row_bytes);
    a_next.c1 = *reinterpret_cast<const u32x4*>(a_source + 1 * 32 * a_row_bytes);
    a_next.c2 = *reinterpret_cast<const u32x4*>(a_source + 2 * 32 * a_row_bytes);
    NFN_MFMA(current.a0, current.b0, acc[0][0]);
    NFN_MFMA(current.a0, current.b1, acc[0][1]);
    NFN_FENCE();
    ahead.a2 = NFN_READ_FRAGMENT(a_read, 2, 3);
    ahead.a3 = NFN_READ_FRAGMENT(a_read, 3, 3);
    a_next.c3 = *reinterpret_cast<const u32x4*>(a_source + 3 * 32 * a_row_bytes);
    a_next.c4 = *reinterpret_cast<const u32x4*>(a_source + 4 * 32 * a_row_bytes);
    a_next.c5 = *reinterpret_cast<const u32x4*>(a_source + 5 * 32 * a_row_bytes);
    NFN_MFMA(current.a1, current.b0, acc[1][0]);
    NFN_MFMA(current.a1, current.b1, acc[1][1]);
    NFN_FENCE();
    ahead.b0 = NFN_READ_FRAGMENT(b_read, 0, 3);
    ahead.b1 = NFN_READ_FRAGMENT(b_read, 1, 3);
    a_next.c6 = *reinterpret_cast<const u32x4*>(a_source + 6 * 32 * a_row_bytes);
    a_next.c7 = *reinterpret_cast<const u32x4*>(a_source + 7 * 32 * a_row_bytes);
    NFN_MFMA(current.a2, current.b0, acc[2][0]);
    NFN_MFMA(current.a2, current.b1, acc[2][1]);
    NFN_FENCE();
    // the packed bytes last: the waits of the step that decodes them count on this order
    b_next.load(b_global, fetch_step >> 2, fetch_step & 3, b_half);
    NFN_MFMA(current.a3, current.b0, acc[3][0]);
    NFN_MFMA(current.a3, current.b1, acc[3][1]);
    NFN_FENCE();

    // every wave has written its part of the other stage and read the last
    // fragments of this one: after the barrier the other stage may be read and
    // this one overwritten
    __syncthreads();

    // ---- K chunk 3: matrix ops on `ahead`, read chunk 0 of the next step ----
    current.a0 = NFN_READ_FRAGMENT(a_read_next, 0, 0);
    current.a1 = NFN_READ_FRAGMENT(a_read_next, 1, 0);
    NFN_MFMA(ahead.a0, ahead.b0, acc[0][0]);
    NFN_MFMA(ahead.a0, ahead.b1, acc[0][1]);
    NFN_FENCE();
    current.a2 = NFN_READ_FRAGMENT(a_read_next, 2, 0);
    current.a3 = NFN_READ_FRAGMENT(a_read_next, 3, 0);
    NFN_MFMA(ahead.a1, ahead.b0, acc[1][0]);
    NFN_MFMA(ahead.a1, ahead.b1, acc[1][1]);
    NFN_FENCE();
    current.b0 = NFN_READ_FRAGMENT(b_read_next, 0, 0);
    current.b1 = NFN_READ_FRAGMENT(b_read_next, 1, 0);
    NFN_MFMA(ahead.a2, ahead.b0, acc[2][0]);
    NFN_MFMA(ahead.a2, ahead.b1, acc[2][1]);
    NFN_FENCE();
    NFN_MFMA(ahead.a3, ahead.b0, acc[3][0]);
    NFN_MFMA(ahead.a3, ahead.b1, acc[3][1]);
    NFN_FENCE();
}

template <std::uint32_t ENC>
__global__ __launch_bounds__(kThreads) void gemm_f16_kernel(
    const std::uint8_t* __restrict__ weights, std::int64_t row_stride, std::int64_t output_dim,
    std::int64_t input_dim, const std::uint16_t* __restrict__ activations,
    const float* __restrict__ inverse_scale, float* __restrict__ output, std::int64_t rows,
    int m_tiles) {
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave >> 1;  // which 128 rows
    const int wave_n = wave & 1;   // which 64 columns
    const int m_tile = blockIdx.x % m_tiles;
    const int n_tile = blockIdx.x / m_tiles;
    const std::int64_t m0 = static_cast<std::int64_t>(m_tile) * kBM;
    const std::int64_t n0 = static_cast<std::int64_t>(n_tile) * kBN;
    const int steps = static_cast<int>(input_dim / kBK);  // a multiple of 4
    const int last = steps - 1;

    // activation copy: chunk c = tid + 256*i is row c/8 = tid/8 + 32*i, 16-byte column tid%8;
    // the workspace holds whole 256-row tiles, so no row needs a bounds check
    const std::int64_t a_row_bytes = input_dim * 2;
    const std::uint8_t* a_global = reinterpret_cast<const std::uint8_t*>(activations) +
        (m0 + (tid >> 3)) * a_row_bytes + (tid & 7) * 16;
    const int a_target = (tid >> 3) * kRowBytes + (tid & 7) * 16;
    // weights: thread -> (row, which 16 positions of the two 32-value groups)
    const int b_row = tid >> 1;
    const int b_half = tid & 1;
    const std::uint8_t* b_global = weights + min(n0 + b_row, output_dim - 1) * row_stride;
    const int b_target = kTileA + b_row * kRowBytes + b_half * 32;

    v16f acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        }
    }

    // slices in flight: while step s computes, one holds step s+1 and the other s+2
    ActivationSlice a_even, a_odd;
    PackedSlice<ENC> b_even, b_odd;
    auto fetch = [&](ActivationSlice& a, PackedSlice<ENC>& b, int step) {
        const std::uint8_t* source = a_global + static_cast<std::int64_t>(step) * (kBK * 2);
        a.c0 = *reinterpret_cast<const u32x4*>(source + 0 * 32 * a_row_bytes);
        a.c1 = *reinterpret_cast<const u32x4*>(source + 1 * 32 * a_row_bytes);
        a.c2 = *reinterpret_cast<const u32x4*>(source + 2 * 32 * a_row_bytes);
        a.c3 = *reinterpret_cast<const u32x4*>(source + 3 * 32 * a_row_bytes);
        a.c4 = *reinterpret_cast<const u32x4*>(source + 4 * 32 * a_row_bytes);
        a.c5 = *reinterpret_cast<const u32x4*>(source + 5 * 32 * a_row_bytes);
        a.c6 = *reinterpret_cast<const u32x4*>(source + 6 * 32 * a_row_bytes);
        a.c7 = *reinterpret_cast<const u32x4*>(source + 7 * 32 * a_row_bytes);
        NFN_FENCE();
        b.load(b_global, step >> 2, step & 3, b_half);
        NFN_FENCE();
    };
    fetch(a_even, b_even, 0);
    fetch(a_odd, b_odd, 1);
    NFN_FENCE();
    {
        std::uint32_t wa[4][2], wb[4][2];
        b_even.prepare(0, b_half);
        b_even.template word<0>(wa[0], wb[0]);
        b_even.template word<1>(wa[1], wb[1]);
        b_even.template word<2>(wa[2], wb[2]);
        b_even.template word<3>(wa[3], wb[3]);
        std::uint8_t* target = lds + b_target;
        NFN_WRITE16(target, wa[0][0], wa[0][1], wa[1][0], wa[1][1]);
        NFN_WRITE16(target + 16, wa[2][0], wa[2][1], wa[3][0], wa[3][1]);
        NFN_WRITE16(target + 64, wb[0][0], wb[0][1], wb[1][0], wb[1][1]);
        NFN_WRITE16(target + 80, wb[2][0], wb[2][1], wb[3][0], wb[3][1]);
        std::uint8_t* a_write = lds + a_target;
        *reinterpret_cast<u32x4*>(a_write + 0 * 32 * kRowBytes) = a_even.c0;
        *reinterpret_cast<u32x4*>(a_write + 1 * 32 * kRowBytes) = a_even.c1;
        *reinterpret_cast<u32x4*>(a_write + 2 * 32 * kRowBytes) = a_even.c2;
        *reinterpret_cast<u32x4*>(a_write + 3 * 32 * kRowBytes) = a_even.c3;
        *reinterpret_cast<u32x4*>(a_write + 4 * 32 * kRowBytes) = a_even.c4;
        *reinterpret_cast<u32x4*>(a_write + 5 * 32 * kRowBytes) = a_even.c5;
        *reinterpret_cast<u32x4*>(a_write + 6 * 32 * kRowBytes) = a_even.c6;
        *reinterpret_cast<u32x4*>(a_write + 7 * 32 * kRowBytes) = a_even.c7;
    }
    NFN_FENCE();
    fetch(a_even, b_even, 2);
    __syncthreads();

    const int operand = (lane & 31) * kRowBytes + (lane >> 5) * 16;
    const std::uint8_t* a_read0 = lds + wave_m * 128 * kRowBytes + operand;
    const std::uint8_t* b_read0 = lds + kTileA + wave_n * 64 * kRowBytes + operand;
    const std::uint8_t* a_read1 = a_read0 + kStageBytes;
    const std::uint8_t* b_read1 = b_read0 + kStageBytes;
    Fragments current;
    current.a0 = NFN_READ_FRAGMENT(a_read0, 0, 0);
    current.a1 = NFN_READ_FRAGMENT(a_read0, 1, 0);
    current.a2 = NFN_READ_FRAGMENT(a_read0, 2, 0);
    current.a3 = NFN_READ_FRAGMENT(a_read0, 3, 0);
    current.b0 = NFN_READ_FRAGMENT(b_read0, 0, 0);
    current.b1 = NFN_READ_FRAGMENT(b_read0, 1, 0);
    // Enter the loop with no load in flight: the waits inside the loop are then
    // derived from the loop's own issue order alone (slice s+1 before slice s+2),
    // not from whatever order the set-up code above was scheduled in.
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    NFN_FENCE();
    int step = 0;
    do {  // input_dim is a positive multiple of 256: at least four steps
        // stage 0 computes; step+1 (odd slice) goes to stage 1; odd slice refills with step+3
        k_step<ENC>(acc, current, a_read0, b_read0, a_read1, b_read1,
                    lds + kStageBytes + a_target, lds + kStageBytes + b_target, a_odd, b_odd,
                    (step + 1) & 3, b_half, a_global, a_row_bytes, b_global, min(step + 3, last));
        // stage 1 computes; step+2 (even slice) goes to stage 0; even slice refills with step+4
        k_step<ENC>(acc, current, a_read1, b_read1, a_read0, b_read0, lds + a_target,
                    lds + b_target, a_even, b_even, (step + 2) & 3, b_half, a_global, a_row_bytes,
                    b_global, min(step + 4, last));
        step += 2;
    } while (step < steps);

    // D register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
    const int column = lane & 31;
    const int row_base = (lane >> 5) * 4;
    const bool whole = m0 + kBM <= rows && n0 + kBN <= output_dim;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const std::int64_t tile_row = m0 + wave_m * 128 + i * 32 + row_base;
        float inverse[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) inverse[r] = inverse_scale[tile_row + 8 * (r >> 2) + (r & 3)];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const std::int64_t n = n0 + wave_n * 64 + j * 32 + column;
            float* target = output + tile_row * output_dim + n;
            if (whole) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    target[(8 * (r >> 2) + (r & 3)) * output_dim] = acc[i][j][r] * inverse[r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const std::int64_t m = tile_row + 8 * (r >> 2) + (r & 3);
                    if (m < rows && n < output_dim) {
                        output[m * output_dim + n] = acc[i][j][r] * inverse[r];
                    }
                }
            }
        }
    }
}

template <std::uint32_t ENC>
void launch_encoding(const Descriptor& descriptor, const std::uint16_t* activations,
                     const float* inverse_scale, float* output, std::int64_t rows,
                     hipStream_t stream) {
    auto kernel = gemm_f16_kernel<ENC>;
    static const bool raised =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
    (void)raised;
    const int m_tiles = static_cast<int>((rows + kBM - 1) / kBM);
    const std::int64_t n_tiles = (descriptor.output_dim + kBN - 1) / kBN;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(m_tiles * n_tiles)), dim3(kThreads),
                       2 * kStageBytes, stream, descriptor.data, descriptor.row_stride_bytes,
                       descriptor.output_dim, descriptor.input_dim, activations, inverse_scale,
                       output, rows, m_tiles);
}

std::int64_t padded_rows(std::int64_t rows) { return (rows + kBM - 1) / kBM * kBM; }

}  // namespace

std::int64_t gemm_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim) {
    // fp16 activations in whole 256-row tiles, then one float per row
    return padded_rows(rows) * input_dim * 2 + padded_rows(rows) * 4 + 256;
}

bool gemm_f16_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K ||
            encoding == kEncQ8_0) && input_dim % 256 == 0;
}

void launch_gemm_f16(const Descriptor& descriptor, const float* input, float* output,
                     std::int64_t rows, void* workspace, hipStream_t stream) {
    std::uint16_t* activations = static_cast<std::uint16_t*>(workspace);
    float* inverse_scale = reinterpret_cast<float*>(
        static_cast<std::uint8_t*>(workspace) + padded_rows(rows) * descriptor.input_dim * 2);
    hipLaunchKernelGGL(convert_activations_kernel, dim3(static_cast<unsigned>(padded_rows(rows))),
                       dim3(256), 0, stream, input, activations, inverse_scale, rows,
                       descriptor.input_dim);
    switch (descriptor.encoding) {
        case kEncQ4K:
            launch_encoding<kEncQ4K>(descriptor, activations, inverse_scale, output, rows, stream);
            break;
        case kEncQ5K:
            launch_encoding<kEncQ5K>(descriptor, activations, inverse_scale, output, rows, stream);
            break;
        case kEncQ6K:
            launch_encoding<kEncQ6K>(descriptor, activations, inverse_scale, output, rows, stream);
            break;
        default:
            launch_encoding<kEncQ8_0>(descriptor, activations, inverse_scale, output, rows, stream);
            break;
    }
}

}  // namespace nfn
