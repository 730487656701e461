// Prefill dequant-GEMM on the fp16 matrix cores:
//   Y[M, N] = X[M, K] * W[N, K]^T,  W packed (Q4_K / Q5_K / Q6_K / Q8_0).
//
// A workgroup of 4 waves owns a 256 x 128 tile of Y; wave w owns rows
// 64w .. 64w+63 and all 128 columns, and walks K in steps of 64 with 32
// v_mfma_f32_32x32x16_f16 per step and float accumulators.
//
// Activations never touch LDS.  A pre-pass converts them to fp16 once per call
// and stores them in matrix-core operand order: for every block of 32 rows and
// every K chunk of 16 the 1 KB that one operand fragment needs is contiguous,
// lane l's 16 bytes (row l%32, the 8 values of K half l/32) at offset 16*l.
// The main loop loads fragments with one fully coalesced 16-byte load per lane
// straight into the registers the matrix instruction reads, one step ahead.
// The pre-pass also scales every row by a power of two so that its largest
// magnitude lands in [2^14, 2^15); the epilogue multiplies the row's results
// by the inverse, so neither large nor tiny activations leave the fp16 range.
//
// Weights go through LDS: per step every thread turns 16 packed bytes (32
// weights of one row of the 128 x 64 slice) into fp16 in registers with packed
// fp16 arithmetic (code bytes become 1024+q by a byte permute, then
// (x-1024)*(d*sc) - dmin*m as one packed fused multiply-add) and writes them
// to a double-buffered stage; the packed bytes are read from HBM once per tile
// column and never exist dequantized in memory.  LDS writes run at about half
// the rate of reads on this chip, which is why only the smaller operand is
// staged.  Stage rows are padded to 144 bytes so that the 16-byte fragment
// reads of 16 lanes hit distinct banks.
//
// A step is written as 16 phases of two matrix instructions each, fenced
// against reordering, so that the dequantization, the LDS traffic and the
// global loads of later steps are issued in the shadow of the matrix
// instructions; weight fragments are read one K chunk ahead, packed bytes are
// loaded three steps before they are decoded.  Consecutive workgroups walk M first: with 8 XCDs picking
// workgroups round robin each XCD keeps one or two 256-row slices of X in its
// L2 while the packed weights stream through.
//
// The reference has no kernel of this kind: its small-batch path stops at 16
// rows (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1326-1328) and more rows run
// the float kernel neuralfn/csrc/tile_cuda/kernels.cu:1398-1525.  Weight
// layouts and decode: neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616.
#include "common.hpp"
#include "f16_decode.hpp"
#include "gemm_mfma.hpp"

namespace nfn {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int kBM = 256;
constexpr int kBN = 128;
constexpr int kBK = 64;
constexpr int kThreads = 256;
constexpr int kMaxShares = 4;  // K shares of a split launch at most
constexpr int kRowBytes = 144;  // 64 fp16 + 16 bytes of padding
constexpr int kStageBytes = kBN * kRowBytes;
constexpr int kFragmentBytes = 1024;  // 32 rows x 16 K values of fp16 in operand order

struct __attribute__((packed, aligned(2))) Chunk16 {
    std::uint32_t v[4];
};

// ---------------------------------------------------------------------------
// activations: fp32 -> row-scaled fp16 in operand order, whole 256-row tiles
// (rows past the end are zeros), in one launch that reads the input once.
// ---------------------------------------------------------------------------

// One wave per row, four rows per workgroup.  A lane owns groups of eight
// consecutive columns (one 16-byte piece of the fp16 copy each); rows of up to
// 8,192 columns stay in the lane's registers between the search for the row's
// largest magnitude and the conversion, wider rows are read again (from L2).
// The row's scale is the power of two that brings that magnitude into
// [2^14, 2^15); zero, subnormal, infinite or NaN maxima keep scale 1; padding
// rows get inverse 0 and zeros.
// The eight workgroups that fill one 32-row block of the operand-order copy
// are the ones a round-robin placement over the eight XCDs puts on the same
// XCD (workgroup w lands on XCD w % 8), so that the 16-byte pieces they
// scatter into the same cache lines merge in one L2 before going to memory.
// SPLIT waves share a row (each takes a contiguous part of its columns and they exchange
// their maxima through LDS): rows of up to 16,384 columns still fit the registers.
template <int HELD, int SPLIT>  // HELD: 8-column groups a lane keeps in registers; 0 = read the row twice
__global__ __launch_bounds__(256) void prepare_activations_kernel(
    const float* __restrict__ input, std::uint8_t* __restrict__ output,
    float* __restrict__ inverse_scale, std::int64_t rows, std::int64_t width) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const std::int64_t group_index = blockIdx.x;
    const std::int64_t xcd = group_index & 7;
    const std::int64_t turn = group_index >> 3;
    constexpr int kRowsPerGroup = 4 / SPLIT;
    constexpr int kGroupsPerBlock = 32 / kRowsPerGroup;  // workgroups that fill a 32-row block
    const std::int64_t block_index = (turn / kGroupsPerBlock) * 8 + xcd;  // 32-row block of the copy
    const int r = static_cast<int>(turn % kGroupsPerBlock) * kRowsPerGroup + wave / SPLIT;  // row inside it
    const int part = wave % SPLIT;  // which part of the row's columns this wave takes
    const std::int64_t row = block_index * 32 + r;
    const bool live = row < rows;
    const float* source = input + (live ? row : 0) * width;
    const std::int64_t all_groups = width / 8;
    const std::int64_t part_groups = (all_groups + SPLIT - 1) / SPLIT;
    const std::int64_t first_group = part * part_groups;
    const std::int64_t groups = min(all_groups, first_group + part_groups);  // end of this wave's groups

    float4 held_x[HELD > 0 ? HELD : 1], held_y[HELD > 0 ? HELD : 1];
    float largest = 0.0f;
    if constexpr (HELD > 0) {
#pragma unroll
        for (int j = 0; j < HELD; ++j) {
            const std::int64_t g = first_group + lane + 64 * j;
            held_x[j] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            held_y[j] = held_x[j];
            if (live && g < groups) {
                held_x[j] = *reinterpret_cast<const float4*>(source + g * 8);
                held_y[j] = *reinterpret_cast<const float4*>(source + g * 8 + 4);
            }
        }
#pragma unroll
        for (int j = 0; j < HELD; ++j) {
            const float4 x = held_x[j], y = held_y[j];
            largest = fmaxf(largest, fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
            largest = fmaxf(largest, fmaxf(fmaxf(fabsf(y.x), fabsf(y.y)), fmaxf(fabsf(y.z), fabsf(y.w))));
        }
    } else {
        for (std::int64_t g = first_group + lane; live && g < groups; g += 64) {
            const float4 x = *reinterpret_cast<const float4*>(source + g * 8);
            const float4 y = *reinterpret_cast<const float4*>(source + g * 8 + 4);
            largest = fmaxf(largest, fmaxf(fmaxf(fabsf(x.x), fabsf(x.y)), fmaxf(fabsf(x.z), fabsf(x.w))));
            largest = fmaxf(largest, fmaxf(fmaxf(fabsf(y.x), fabsf(y.y)), fmaxf(fabsf(y.z), fabsf(y.w))));
        }
    }
    // NaN never wins fmaxf: a row with NaN keeps the largest finite magnitude, as before
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        largest = fmaxf(largest, __shfl_xor(largest, offset));
    }
    if constexpr (SPLIT > 1) {
        __shared__ float maxima[4];
        if (lane == 0) maxima[wave] = largest;
        __syncthreads();
        const int first_wave = wave - part;
#pragma unroll
        for (int k = 0; k < SPLIT; ++k) largest = fmaxf(largest, maxima[first_wave + k]);
    }
    const std::uint32_t exponent = (__float_as_uint(largest) >> 23) & 0xffu;
    const bool usable = exponent >= 16u && exponent <= 254u;
    const float factor = !live ? 0.0f
        : usable ? __uint_as_float((127u + 14u + 127u - exponent) << 23) : 1.0f;
    if (lane == 0 && part == 0) {
        inverse_scale[row] = !live ? 0.0f : usable ? __uint_as_float((exponent - 14u) << 23) : 1.0f;
    }

    std::uint8_t* block = output + block_index * (width / 16) * kFragmentBytes;
    auto store = [&](std::int64_t g, float4 x, float4 y) {
        const f16x2 h0 = {static_cast<_Float16>(x.x * factor), static_cast<_Float16>(x.y * factor)};
        const f16x2 h1 = {static_cast<_Float16>(x.z * factor), static_cast<_Float16>(x.w * factor)};
        const f16x2 h2 = {static_cast<_Float16>(y.x * factor), static_cast<_Float16>(y.y * factor)};
        const f16x2 h3 = {static_cast<_Float16>(y.z * factor), static_cast<_Float16>(y.w * factor)};
        std::uint8_t* target = block + (g >> 1) * kFragmentBytes + ((g & 1) * 32 + r) * 16;
        *reinterpret_cast<u32x4*>(target) = u32x4{bits_of(h0), bits_of(h1), bits_of(h2), bits_of(h3)};
    };
    if constexpr (HELD > 0) {
#pragma unroll
        for (int j = 0; j < HELD; ++j) {
            const std::int64_t g = first_group + lane + 64 * j;
            if (g < groups) store(g, held_x[j], held_y[j]);
        }
    } else {
        for (std::int64_t g = first_group + lane; g < groups; g += 64) {
            float4 x = make_float4(0.0f, 0.0f, 0.0f, 0.0f), y = x;
            if (live) {
                x = *reinterpret_cast<const float4*>(source + g * 8);
                y = *reinterpret_cast<const float4*>(source + g * 8 + 4);
            }
            store(g, x, y);
        }
    }
}

// ---------------------------------------------------------------------------
// What one thread holds of the packed weights of one K step: its row's 16
// bytes of codes for positions 16*half .. 16*half+15 of both 32-value groups
// of the step.  Decoding is cut into pieces of
// at most eight vector instructions so that each fits behind one matrix
// instruction: prepare_bits() and prepare_scales() derive the fp16 scale
// constants; group_a<I>() / group_b<I>() decode code word I into positions
// 4I..4I+3 of the first / second group (two packed fp16 pairs).
// ---------------------------------------------------------------------------
template <std::uint32_t ENC>
struct PackedSlice;
// what all K steps of one 256-value block share; loaded once per block
template <std::uint32_t ENC>
struct BlockHeader;

template <>
struct BlockHeader<kEncQ4K> {
    u32x4 words;  // d, dmin and the twelve scale bytes
    __device__ __forceinline__ void load(const std::uint8_t* row, int block) {
        words = *reinterpret_cast<const u32x4*>(row + block * 144);
    }
};

template <>
struct PackedSlice<kEncQ4K> {
    u32x4 codes;
    KBlockScales c;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        codes = *reinterpret_cast<const u32x4*>(row + block * 144 + 16 + pair * 32 + half * 16);
    }
    __device__ __forceinline__ void prepare_bits(const BlockHeader<kEncQ4K>& header, int pair, int) {
        c.bits(header.words, pair);
    }
    __device__ __forceinline__ void prepare_scales(const BlockHeader<kEncQ4K>& header) {
        c.scales(header.words);
    }
    template <int I>
    __device__ __forceinline__ void group_a(std::uint32_t (&out)[2]) const {
        scale_bytes(codes[I] & 0x0f0f0f0fu, splat(-1024.0f), c.scale_a, c.shift_a, out[0], out[1]);
    }
    template <int I>
    __device__ __forceinline__ void group_b(std::uint32_t (&out)[2]) const {
        scale_bytes((codes[I] >> 4) & 0x0f0f0f0fu, splat(-1024.0f), c.scale_b, c.shift_b, out[0],
                    out[1]);
    }
};

template <>
struct BlockHeader<kEncQ5K> {
    u32x4 words;  // d, dmin and the twelve scale bytes
    __device__ __forceinline__ void load(const std::uint8_t* row, int block) {
        words = *reinterpret_cast<const u32x4*>(row + block * 176);
    }
};

template <>
struct PackedSlice<kEncQ5K> {
    u32x4 codes, high;
    KBlockScales c;
    int high_shift;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 176;
        high = *reinterpret_cast<const u32x4*>(p + 16 + half * 16);
        codes = *reinterpret_cast<const u32x4*>(p + 48 + pair * 32 + half * 16);
    }
    __device__ __forceinline__ void prepare_bits(const BlockHeader<kEncQ5K>& header, int pair, int) {
        c.bits(header.words, pair);
        high_shift = 2 * pair;  // bit 2*pair: first group, bit 2*pair+1: second
    }
    __device__ __forceinline__ void prepare_scales(const BlockHeader<kEncQ5K>& header) {
        c.scales(header.words);
    }
    template <int I>
    __device__ __forceinline__ void group_a(std::uint32_t (&out)[2]) const {
        const std::uint32_t bits = high[I] >> high_shift;
        const std::uint32_t q = (codes[I] & 0x0f0f0f0fu) | ((bits & 0x01010101u) << 4);
        scale_bytes(q, splat(-1024.0f), c.scale_a, c.shift_a, out[0], out[1]);
    }
    template <int I>
    __device__ __forceinline__ void group_b(std::uint32_t (&out)[2]) const {
        const std::uint32_t bits = high[I] >> high_shift;
        const std::uint32_t q = ((codes[I] >> 4) & 0x0f0f0f0fu) | ((bits & 0x02020202u) << 3);
        scale_bytes(q, splat(-1024.0f), c.scale_b, c.shift_b, out[0], out[1]);
    }
};

template <>
struct BlockHeader<kEncQ6K> {
    // sixteen int8 sub-scales in four words, then d; five plain words, so that the
    // struct has no padding for a copy to carry through scratch memory
    std::uint32_t scales_x, scales_y, scales_z, scales_w;
    std::uint32_t d_bits;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block) {
        const std::uint8_t* p = row + block * 210;
        const Chunk16 s = *reinterpret_cast<const Chunk16*>(p + 192);
        scales_x = s.v[0];
        scales_y = s.v[1];
        scales_z = s.v[2];
        scales_w = s.v[3];
        d_bits = *reinterpret_cast<const std::uint16_t*>(p + 208);
    }
};

template <>
struct PackedSlice<kEncQ6K> {
    // a K step of 64 is two quarters (32 values each) of one half of the block:
    // quarters (0,1) or (2,3); `pair` = 2*half_of_block + (quarters 2,3 ? 1 : 0)
    u32x4 low_a, low_b, high;
    f16x2 scale_a, scale_b;
    int upper, sa, sb;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 210;
        const int block_half = pair >> 1;
        const Chunk16 la = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + half * 16);
        const Chunk16 lb = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + 32 + half * 16);
        const Chunk16 hb = *reinterpret_cast<const Chunk16*>(p + 128 + block_half * 32 + half * 16);
        low_a = u32x4{la.v[0], la.v[1], la.v[2], la.v[3]};
        low_b = u32x4{lb.v[0], lb.v[1], lb.v[2], lb.v[3]};
        high = u32x4{hb.v[0], hb.v[1], hb.v[2], hb.v[3]};
    }
    __device__ __forceinline__ void prepare_bits(const BlockHeader<kEncQ6K>& header, int pair,
                                                 int half) {
        // sub-scale index = 8*half_of_block + 2*quarter + position/16: the step's four
        // are word `pair` of the sixteen, and this thread's 16 positions share one per quarter
        const std::uint32_t sub_scales = pair == 0 ? header.scales_x
            : pair == 1 ? header.scales_y : pair == 2 ? header.scales_z : header.scales_w;
        sa = static_cast<std::int8_t>((sub_scales >> (8 * half)) & 0xffu);
        sb = static_cast<std::int8_t>((sub_scales >> (8 * (2 + half))) & 0xffu);
        upper = (pair & 1) * 4;  // quarters 2,3: high nibbles, high-bit pairs 4..7
    }
    __device__ __forceinline__ void prepare_scales(const BlockHeader<kEncQ6K>& header) {
        const float d = half_bits_to_float(header.d_bits);
        scale_a = splat(d * static_cast<float>(sa));
        scale_b = splat(d * static_cast<float>(sb));
    }
    // bias: 1024 + the format's offset of 32
    template <int I>
    __device__ __forceinline__ void group_a(std::uint32_t (&out)[2]) const {
        const std::uint32_t top = high[I] >> upper;  // bits 0,1: first quarter
        const std::uint32_t q = ((low_a[I] >> upper) & 0x0f0f0f0fu) | ((top & 0x03030303u) << 4);
        scale_bytes(q, splat(-1056.0f), scale_a, splat(0.0f), out[0], out[1]);
    }
    template <int I>
    __device__ __forceinline__ void group_b(std::uint32_t (&out)[2]) const {
        const std::uint32_t top = high[I] >> upper;  // bits 2,3: second quarter
        const std::uint32_t q = ((low_b[I] >> upper) & 0x0f0f0f0fu) | ((top & 0x0c0c0c0cu) << 2);
        scale_bytes(q, splat(-1056.0f), scale_b, splat(0.0f), out[0], out[1]);
    }
};

template <>
struct BlockHeader<kEncQ8_0> {  // the scales sit next to the codes
    __device__ __forceinline__ void load(const std::uint8_t*, int) {}
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
    __device__ __forceinline__ void prepare_bits(const BlockHeader<kEncQ8_0>&, int, int) {}
    __device__ __forceinline__ void prepare_scales(const BlockHeader<kEncQ8_0>&) {
        const _Float16 a = __builtin_bit_cast(_Float16, static_cast<std::uint16_t>(d_a));
        const _Float16 b = __builtin_bit_cast(_Float16, static_cast<std::uint16_t>(d_b));
        scale_a = f16x2{a, a};
        scale_b = f16x2{b, b};
    }
    // flipping the sign bit turns the int8 code q into the byte q+128: bias 1024+128
    template <int I>
    __device__ __forceinline__ void group_a(std::uint32_t (&out)[2]) const {
        scale_bytes(codes_a[I] ^ 0x80808080u, splat(-1152.0f), scale_a, splat(0.0f), out[0], out[1]);
    }
    template <int I>
    __device__ __forceinline__ void group_b(std::uint32_t (&out)[2]) const {
        scale_bytes(codes_b[I] ^ 0x80808080u, splat(-1152.0f), scale_b, splat(0.0f), out[0], out[1]);
    }
};

// The activation fragments of one K step for one wave: row blocks 0 and 1,
// K chunks 0..3, in named registers (an array here ends up in scratch memory).
struct ActivationSlice {
    f16x8 r0k0, r0k1, r0k2, r0k3, r1k0, r1k1, r1k2, r1k3;
};

// the four weight fragments (column blocks) of one K chunk of 16
struct WeightFragments {
    f16x8 c0, c1, c2, c3;
};

#define NFN_FENCE() __builtin_amdgcn_sched_barrier(0)
#define NFN_MFMA(A, B, C) C = __builtin_amdgcn_mfma_f32_32x32x16_f16(A, B, C, 0, 0, 0)
#define NFN_READ_WEIGHTS(base, column_block, chunk) \
    (*reinterpret_cast<const f16x8*>((base) + (column_block) * 32 * kRowBytes + (chunk) * 32))
#define NFN_LOAD_ACTIVATIONS(base, row_block, chunk) \
    (*reinterpret_cast<const f16x8*>((base) + (row_block) * row_block_bytes + (chunk) * kFragmentBytes))
#define NFN_WRITE16(target, x, y, z, w) *reinterpret_cast<u32x4*>(target) = u32x4{x, y, z, w}
#define NFN_WRITE8(target, pair) *reinterpret_cast<uint2*>(target) = make_uint2((pair)[0], (pair)[1])

// One matrix instruction with the statements issued in its shadow.  A wave
// issues in order and stalls at a matrix instruction while the previous one
// occupies the pipe (32 cycles), so only what stands between two of them
// overlaps: about seven vector instructions fit.
#define NFN_SLOT(A, W, C, ...) \
    __VA_ARGS__;               \
    NFN_MFMA(A, W, C);         \
    NFN_FENCE();

// One K step for one wave: 32 slots.  A row block 0 fragment is last used in
// the fourth slot of its chunk, a row block 1 fragment in the eighth; each is
// refilled with the fragment of the next step right after.
//   a_now:    activation fragments of this step
//   current:  weight fragments of K chunk 0 of this step (read at the end of
//             the previous one); on return they hold chunk 0 of the next step
//   b_next:   packed weights of the next step: dequantized into the other
//             stage with the scales in `header`, then refilled with the packed
//             bytes of `fetch_step`
template <std::uint32_t ENC, int RB>
__device__ __forceinline__ void k_step(
    v16f (&acc)[RB][4], ActivationSlice& a_now, WeightFragments& current,
    const std::uint8_t* b_read, const std::uint8_t* b_read_next, std::uint8_t* b_write,
    PackedSlice<ENC>& b_next, const BlockHeader<ENC>& header, int decode_pair, int b_half,
    const std::uint8_t* a_fetch, std::int64_t row_block_bytes, const std::uint8_t* b_global,
    int fetch_step) {
    WeightFragments ahead;
    std::uint32_t w[2], v[2];

    if constexpr (RB == 1) {
        // One row block per wave: 16 slots carry the same side work.
        NFN_SLOT(a_now.r0k0, current.c0, acc[0][0], b_next.prepare_bits(header, decode_pair, b_half))
        NFN_SLOT(a_now.r0k0, current.c1, acc[0][1], b_next.prepare_scales(header);
                 ahead.c0 = NFN_READ_WEIGHTS(b_read, 0, 1))
        NFN_SLOT(a_now.r0k0, current.c2, acc[0][2], b_next.template group_a<0>(w);
                 ahead.c1 = NFN_READ_WEIGHTS(b_read, 1, 1))
        NFN_SLOT(a_now.r0k0, current.c3, acc[0][3], b_next.template group_a<1>(v);
                 NFN_WRITE16(b_write, w[0], w[1], v[0], v[1]); ahead.c2 = NFN_READ_WEIGHTS(b_read, 2, 1);
                 ahead.c3 = NFN_READ_WEIGHTS(b_read, 3, 1))
        NFN_SLOT(a_now.r0k1, ahead.c0, acc[0][0], b_next.template group_a<2>(w);
                 current.c0 = NFN_READ_WEIGHTS(b_read, 0, 2);
                 a_now.r0k0 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 0))
        NFN_SLOT(a_now.r0k1, ahead.c1, acc[0][1], b_next.template group_a<3>(v);
                 NFN_WRITE16(b_write + 16, w[0], w[1], v[0], v[1]); current.c1 = NFN_READ_WEIGHTS(b_read, 1, 2))
        NFN_SLOT(a_now.r0k1, ahead.c2, acc[0][2], b_next.template group_b<0>(w);
                 current.c2 = NFN_READ_WEIGHTS(b_read, 2, 2))
        NFN_SLOT(a_now.r0k1, ahead.c3, acc[0][3], b_next.template group_b<1>(v);
                 NFN_WRITE16(b_write + 64, w[0], w[1], v[0], v[1]); current.c3 = NFN_READ_WEIGHTS(b_read, 3, 2))
        NFN_SLOT(a_now.r0k2, current.c0, acc[0][0], b_next.template group_b<2>(w);
                 ahead.c0 = NFN_READ_WEIGHTS(b_read, 0, 3);
                 a_now.r0k1 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 1))
        NFN_SLOT(a_now.r0k2, current.c1, acc[0][1], b_next.template group_b<3>(v);
                 NFN_WRITE16(b_write + 80, w[0], w[1], v[0], v[1]); ahead.c1 = NFN_READ_WEIGHTS(b_read, 1, 3))
        NFN_SLOT(a_now.r0k2, current.c2, acc[0][2], ahead.c2 = NFN_READ_WEIGHTS(b_read, 2, 3))
        NFN_SLOT(a_now.r0k2, current.c3, acc[0][3], ahead.c3 = NFN_READ_WEIGHTS(b_read, 3, 3))
        __syncthreads();
        NFN_SLOT(a_now.r0k3, ahead.c0, acc[0][0], current.c0 = NFN_READ_WEIGHTS(b_read_next, 0, 0);
                 a_now.r0k2 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 2))
        NFN_SLOT(a_now.r0k3, ahead.c1, acc[0][1], current.c1 = NFN_READ_WEIGHTS(b_read_next, 1, 0))
        NFN_SLOT(a_now.r0k3, ahead.c2, acc[0][2], current.c2 = NFN_READ_WEIGHTS(b_read_next, 2, 0))
        NFN_SLOT(a_now.r0k3, ahead.c3, acc[0][3], current.c3 = NFN_READ_WEIGHTS(b_read_next, 3, 0))
        a_now.r0k3 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 3);
        NFN_FENCE();
        b_next.load(b_global, fetch_step >> 2, fetch_step & 3, b_half);
        NFN_FENCE();
        return;
    } else {
    // K chunk 0: read chunk 1, decode; every decoded group of four values is
    // written to the other stage at once (8 bytes), which keeps few registers live
    NFN_SLOT(a_now.r0k0, current.c0, acc[0][0], b_next.prepare_bits(header, decode_pair, b_half))
    NFN_SLOT(a_now.r0k0, current.c1, acc[0][1], b_next.prepare_scales(header);
             ahead.c0 = NFN_READ_WEIGHTS(b_read, 0, 1))
    NFN_SLOT(a_now.r0k0, current.c2, acc[0][2], b_next.template group_a<0>(w);
             ahead.c1 = NFN_READ_WEIGHTS(b_read, 1, 1))
    NFN_SLOT(a_now.r0k0, current.c3, acc[0][3], b_next.template group_a<1>(v);
             NFN_WRITE16(b_write, w[0], w[1], v[0], v[1]))
    NFN_SLOT(a_now.r1k0, current.c0, acc[1][0], b_next.template group_a<2>(w);
             ahead.c2 = NFN_READ_WEIGHTS(b_read, 2, 1);
             a_now.r0k0 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 0))
    NFN_SLOT(a_now.r1k0, current.c1, acc[1][1], b_next.template group_a<3>(v);
             NFN_WRITE16(b_write + 16, w[0], w[1], v[0], v[1]))
    NFN_SLOT(a_now.r1k0, current.c2, acc[1][2], b_next.template group_b<0>(w);
             ahead.c3 = NFN_READ_WEIGHTS(b_read, 3, 1))
    NFN_SLOT(a_now.r1k0, current.c3, acc[1][3], b_next.template group_b<1>(v);
             NFN_WRITE16(b_write + 64, w[0], w[1], v[0], v[1]))
    // K chunk 1: read chunk 2, finish decoding
    NFN_SLOT(a_now.r0k1, ahead.c0, acc[0][0], b_next.template group_b<2>(w);
             current.c0 = NFN_READ_WEIGHTS(b_read, 0, 2);
             a_now.r1k0 = NFN_LOAD_ACTIVATIONS(a_fetch, 1, 0))
    NFN_SLOT(a_now.r0k1, ahead.c1, acc[0][1], b_next.template group_b<3>(v);
             NFN_WRITE16(b_write + 80, w[0], w[1], v[0], v[1]))
    NFN_SLOT(a_now.r0k1, ahead.c2, acc[0][2], current.c1 = NFN_READ_WEIGHTS(b_read, 1, 2))
    NFN_SLOT(a_now.r0k1, ahead.c3, acc[0][3], (void)0)
    NFN_SLOT(a_now.r1k1, ahead.c0, acc[1][0], current.c2 = NFN_READ_WEIGHTS(b_read, 2, 2);
             a_now.r0k1 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 1))
    NFN_SLOT(a_now.r1k1, ahead.c1, acc[1][1], (void)0)
    NFN_SLOT(a_now.r1k1, ahead.c2, acc[1][2], current.c3 = NFN_READ_WEIGHTS(b_read, 3, 2))
    NFN_SLOT(a_now.r1k1, ahead.c3, acc[1][3], (void)0)
    // K chunk 2: read chunk 3
    NFN_SLOT(a_now.r0k2, current.c0, acc[0][0], ahead.c0 = NFN_READ_WEIGHTS(b_read, 0, 3);
             a_now.r1k1 = NFN_LOAD_ACTIVATIONS(a_fetch, 1, 1))
    NFN_SLOT(a_now.r0k2, current.c1, acc[0][1], (void)0)
    NFN_SLOT(a_now.r0k2, current.c2, acc[0][2], ahead.c1 = NFN_READ_WEIGHTS(b_read, 1, 3))
    NFN_SLOT(a_now.r0k2, current.c3, acc[0][3], (void)0)
    NFN_SLOT(a_now.r1k2, current.c0, acc[1][0], ahead.c2 = NFN_READ_WEIGHTS(b_read, 2, 3);
             a_now.r0k2 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 2))
    NFN_SLOT(a_now.r1k2, current.c1, acc[1][1], (void)0)
    NFN_SLOT(a_now.r1k2, current.c2, acc[1][2], ahead.c3 = NFN_READ_WEIGHTS(b_read, 3, 3))
    NFN_SLOT(a_now.r1k2, current.c3, acc[1][3], (void)0)

    // every wave has written its part of the other stage and read the last
    // fragments of this one: after the barrier the other stage may be read and
    // this one overwritten
    __syncthreads();

    // K chunk 3: read chunk 0 of the next step; the packed bytes are loaded
    // last: the waits of the step that decodes them count on this order
    NFN_SLOT(a_now.r0k3, ahead.c0, acc[0][0], current.c0 = NFN_READ_WEIGHTS(b_read_next, 0, 0);
             a_now.r1k2 = NFN_LOAD_ACTIVATIONS(a_fetch, 1, 2))
    NFN_SLOT(a_now.r0k3, ahead.c1, acc[0][1], (void)0)
    NFN_SLOT(a_now.r0k3, ahead.c2, acc[0][2], current.c1 = NFN_READ_WEIGHTS(b_read_next, 1, 0))
    NFN_SLOT(a_now.r0k3, ahead.c3, acc[0][3], (void)0)
    NFN_SLOT(a_now.r1k3, ahead.c0, acc[1][0], current.c2 = NFN_READ_WEIGHTS(b_read_next, 2, 0);
             a_now.r0k3 = NFN_LOAD_ACTIVATIONS(a_fetch, 0, 3))
    NFN_SLOT(a_now.r1k3, ahead.c1, acc[1][1], (void)0)
    NFN_SLOT(a_now.r1k3, ahead.c2, acc[1][2], current.c3 = NFN_READ_WEIGHTS(b_read_next, 3, 0))
    NFN_SLOT(a_now.r1k3, ahead.c3, acc[1][3], (void)0)
    a_now.r1k3 = NFN_LOAD_ACTIVATIONS(a_fetch, 1, 3);
    NFN_FENCE();
    b_next.load(b_global, fetch_step >> 2, fetch_step & 3, b_half);
    NFN_FENCE();
    }
}

// bytes of 256 packed values
template <std::uint32_t ENC>
constexpr int kBlockBytes = ENC == kEncQ4K ? 144 : ENC == kEncQ5K ? 176 : ENC == kEncQ6K ? 210 : 272;

// Workgroups per compute unit (= waves per SIMD): as many as the registers
// allow; while one wave waits at the barrier or for LDS, another keeps the
// matrix pipe busy.  With 256-row tiles the Q6_K decode holds too much live
// state for two.
template <std::uint32_t ENC, int RB>
constexpr int kWavesPerSimd = ENC == kEncQ6K ? RB == 1 ? 2 : 1 : RB == 1 ? (ENC == kEncQ5K ? 2 : 3) : 2;

// RB: 32-row blocks per wave; the workgroup's tile is 128*RB rows by 128 columns.
template <std::uint32_t ENC, int RB>
__global__ __launch_bounds__(kThreads)
__attribute__((amdgpu_waves_per_eu(kWavesPerSimd<ENC, RB>, kWavesPerSimd<ENC, RB>))) void gemm_f16_kernel(
    const std::uint8_t* __restrict__ weights, std::int64_t row_stride, std::int64_t output_dim,
    std::int64_t input_dim, const std::uint8_t* __restrict__ activations,
    const float* __restrict__ inverse_scale, float* __restrict__ output, std::int64_t rows,
    int m_tiles, std::int64_t split_stride) {
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // rows 64*wave .. +63 of the tile
    const int m_tile = blockIdx.x % m_tiles;
    const int n_tile = blockIdx.x / m_tiles;
    constexpr int kTileRows = 128 * RB;
    const std::int64_t m0 = static_cast<std::int64_t>(m_tile) * kTileRows;
    const std::int64_t n0 = static_cast<std::int64_t>(n_tile) * kBN;
    // blockIdx.y: which share of the K dimension (whole 256-value blocks) this
    // workgroup sums; each share writes its own copy of the output
    const int total_blocks = static_cast<int>(input_dim >> 8);
    const int first_block = total_blocks * static_cast<int>(blockIdx.y) / static_cast<int>(gridDim.y);
    const int end_block = total_blocks * (static_cast<int>(blockIdx.y) + 1) / static_cast<int>(gridDim.y);
    const int steps = (end_block - first_block) * 4;  // a positive multiple of 4
    const int last = steps - 1;
    output += blockIdx.y * split_stride;

    // activations: fragment (row block, K chunk) is 1 KB, a row block's chunks are consecutive
    const std::int64_t row_block_bytes = (input_dim / 16) * kFragmentBytes;
    const std::uint8_t* a_global = activations + (m0 / 32 + wave * RB) * row_block_bytes +
        static_cast<std::int64_t>(first_block) * 16 * kFragmentBytes + lane * 16;
    constexpr int kStepBytes = (kBK / 16) * kFragmentBytes;
    // weights: thread -> (row, which 16 positions of the two 32-value groups)
    // (sixteen consecutive lanes write sixteen consecutive stage rows: with rows of 144 bytes
    // their 16-byte pieces fall into distinct banks, as the fragment reads do)
    const int b_row = tid & 127;
    const int b_half = tid >> 7;
    const std::uint8_t* b_global = weights + min(n0 + b_row, output_dim - 1) * row_stride +
        static_cast<std::int64_t>(first_block) * kBlockBytes<ENC>;
    const int b_target = b_row * kRowBytes + b_half * 32;

    v16f acc[RB][4];
#pragma unroll
    for (int i = 0; i < RB; ++i) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
        }
    }

    // Activation fragments come from L2 (the other workgroups of this XCD read
    // the same rows): one slice, each fragment refilled right after its last use
    // with the same fragment of the next step, which leaves the load one step
    // to land.  Packed weights come from HBM or the memory-side cache: four
    // slices, each refilled right after it is decoded with the bytes of four
    // steps later (slice j holds the steps congruent to j modulo 4), which
    // gives their loads three steps.
    // The header of a 256-value block is loaded once, three or more steps
    // before the first of its four steps is decoded.
    ActivationSlice a_now;
    PackedSlice<ENC> b0, b1, b2, b3;
    BlockHeader<ENC> header_even, header_odd;  // blocks 0, 2, 4 ... and 1, 3, 5 ...
    const int last_block = (steps >> 2) - 1;
    header_even.load(b_global, 0);
    header_odd.load(b_global, min(1, last_block));
    b0.load(b_global, 0, 0, b_half);
    b1.load(b_global, 0, 1, b_half);
    b2.load(b_global, 0, 2, b_half);
    b3.load(b_global, 0, 3, b_half);
    a_now.r0k0 = NFN_LOAD_ACTIVATIONS(a_global, 0, 0);
    a_now.r0k1 = NFN_LOAD_ACTIVATIONS(a_global, 0, 1);
    a_now.r0k2 = NFN_LOAD_ACTIVATIONS(a_global, 0, 2);
    a_now.r0k3 = NFN_LOAD_ACTIVATIONS(a_global, 0, 3);
    if constexpr (RB == 2) {
        a_now.r1k0 = NFN_LOAD_ACTIVATIONS(a_global, 1, 0);
        a_now.r1k1 = NFN_LOAD_ACTIVATIONS(a_global, 1, 1);
        a_now.r1k2 = NFN_LOAD_ACTIVATIONS(a_global, 1, 2);
        a_now.r1k3 = NFN_LOAD_ACTIVATIONS(a_global, 1, 3);
    }
    {
        std::uint32_t wa[4][2], wb[4][2];
        b0.prepare_bits(header_even, 0, b_half);
        b0.prepare_scales(header_even);
        b0.template group_a<0>(wa[0]);
        b0.template group_a<1>(wa[1]);
        b0.template group_a<2>(wa[2]);
        b0.template group_a<3>(wa[3]);
        b0.template group_b<0>(wb[0]);
        b0.template group_b<1>(wb[1]);
        b0.template group_b<2>(wb[2]);
        b0.template group_b<3>(wb[3]);
        std::uint8_t* target = lds + b_target;
        NFN_WRITE16(target, wa[0][0], wa[0][1], wa[1][0], wa[1][1]);
        NFN_WRITE16(target + 16, wa[2][0], wa[2][1], wa[3][0], wa[3][1]);
        NFN_WRITE16(target + 64, wb[0][0], wb[0][1], wb[1][0], wb[1][1]);
        NFN_WRITE16(target + 80, wb[2][0], wb[2][1], wb[3][0], wb[3][1]);
    }
    b0.load(b_global, min(1, last_block), 0, b_half);  // step 4, or step 0 again
    __syncthreads();

    const int operand = (lane & 31) * kRowBytes + (lane >> 5) * 16;
    const std::uint8_t* b_read0 = lds + operand;
    const std::uint8_t* b_read1 = b_read0 + kStageBytes;
    std::uint8_t* b_write0 = lds + b_target;
    std::uint8_t* b_write1 = b_write0 + kStageBytes;
    WeightFragments current;
    current.c0 = NFN_READ_WEIGHTS(b_read0, 0, 0);
    current.c1 = NFN_READ_WEIGHTS(b_read0, 1, 0);
    current.c2 = NFN_READ_WEIGHTS(b_read0, 2, 0);
    current.c3 = NFN_READ_WEIGHTS(b_read0, 3, 0);
    // Enter the loop with no load in flight: the waits inside the loop are then
    // derived from the loop's own issue order alone, not from whatever order
    // the set-up code above was scheduled in.
    __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
    NFN_FENCE();
    const auto activations_of = [&](int step) {
        return a_global + static_cast<std::int64_t>(min(step, last)) * kStepBytes;
    };
    // Four steps: one 256-value block.  Step s computes from stage s%2 while
    // step s+1 is decoded into the other stage; the decoded slice then loads
    // step s+5 and the activation slice step s+1.  `now` holds the scales of
    // this block, `next` those of the following one (needed by the fourth step,
    // which decodes the first step of that block).
    auto block_of_four = [&](int step, const BlockHeader<ENC>& now, const BlockHeader<ENC>& next) {
        k_step<ENC, RB>(acc, a_now, current, b_read0, b_read1, b_write1, b1, now, 1, b_half,
                    activations_of(step + 1), row_block_bytes, b_global, min(step + 5, last));
        k_step<ENC, RB>(acc, a_now, current, b_read1, b_read0, b_write0, b2, now, 2, b_half,
                    activations_of(step + 2), row_block_bytes, b_global, min(step + 6, last));
        k_step<ENC, RB>(acc, a_now, current, b_read0, b_read1, b_write1, b3, now, 3, b_half,
                    activations_of(step + 3), row_block_bytes, b_global, min(step + 7, last));
        k_step<ENC, RB>(acc, a_now, current, b_read1, b_read0, b_write0, b0, next, 0, b_half,
                    activations_of(step + 4), row_block_bytes, b_global, min(step + 8, last));
    };
    // The two header register sets swap roles every block; the loop body is two
    // blocks so that no copy (and no wait for the load that feeds it) is needed.
    // An odd block count runs its first block ahead of the loop.  The loop has
    // its only exit at the end: values loaded for later steps are then live
    // around the back edge and the loads stay where they are written.
    int block = 0;
    if ((last_block & 1) == 0) {
        block_of_four(0, header_even, header_odd);
        header_even.load(b_global, min(2, last_block));
        NFN_FENCE();
        const BlockHeader<ENC> second = header_odd;
        header_odd = header_even;
        header_even = second;
        block = 1;
    }
    while (block < last_block) {
        block_of_four(block * 4, header_even, header_odd);
        header_even.load(b_global, min(block + 2, last_block));
        NFN_FENCE();
        block_of_four(block * 4 + 4, header_odd, header_even);
        header_odd.load(b_global, min(block + 3, last_block));
        NFN_FENCE();
        block += 2;
    }

    // D register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
    const int column = lane & 31;
    const int row_base = (lane >> 5) * 4;
    const bool whole = m0 + kTileRows <= rows && n0 + kBN <= output_dim;
#pragma unroll
    for (int i = 0; i < RB; ++i) {
        const std::int64_t tile_row = m0 + wave * (32 * RB) + i * 32 + row_base;
        float inverse[16];
#pragma unroll
        for (int r = 0; r < 16; ++r) inverse[r] = inverse_scale[tile_row + 8 * (r >> 2) + (r & 3)];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const std::int64_t n = n0 + j * 32 + column;
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

// Sum of the K shares: output[i] = partial[0][i] + partial[1][i] + ..., in that order.
__global__ __launch_bounds__(256) void sum_shares_kernel(const float* __restrict__ partials,
                                                         float* __restrict__ output,
                                                         std::int64_t count, int shares) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        float total = partials[index];
        for (int share = 1; share < shares; ++share) total += partials[share * count + index];
        output[index] = total;
    }
}

// Tile height and K shares of a launch, from a sweep over both on this chip.
// 256-row tiles reuse each weight fragment twice as often and win whenever
// they give every compute unit a workgroup.  A smaller problem splits K over
// several workgroups per tile (at least twelve 256-value blocks each, at most
// four shares) until the grid fills the units' two (256-row tiles) or three
// (128-row tiles) workgroup slots; the shares are summed by a second launch in
// a fixed order.  256-row tiles stay the better choice as long as two shares or
// more fit; at most 128 rows, or a K too short to split, take 128-row tiles.
// Narrow projections (an eighth of the units' count in 256-row tiles at most) take
// 128-row tiles and shares of six blocks or more.
struct Plan {
    int row_blocks;  // 32-row blocks per wave: 2 = 256-row tiles, 1 = 128-row tiles
    int shares;
};

Plan plan(std::uint32_t encoding, std::int64_t rows, std::int64_t output_dim,
          std::int64_t input_dim) {
    const std::int64_t units = compute_units();
    const std::int64_t n_tiles = (output_dim + kBN - 1) / kBN;
    const std::int64_t tall_tiles = (rows + 255) / 256 * n_tiles;
    if (tall_tiles >= units) return Plan{2, 1};
    std::int64_t longest = (input_dim >> 8) / 12;  // shares that still get twelve blocks each
    if (longest > kMaxShares) longest = kMaxShares;
    if (tall_tiles * 8 <= units) {
        // A narrow projection (a few tiles for the whole chip, e.g. 256 outputs): what it
        // takes is the length of one workgroup's walk over K, so the shares may be as short
        // as six blocks and the tiles are the small ones (1,024 x 6,656 -> 256: 53 -> 34 us).
        std::int64_t shortest = (input_dim >> 8) / 6;
        if (shortest > kMaxShares) shortest = kMaxShares;
        if (shortest < 1) shortest = 1;
        const std::int64_t tiles = (rows + 127) / 128 * n_tiles;
        std::int64_t shares = units * 3 / tiles;
        if (shares > shortest) shares = shortest;
        if (shares < 1) shares = 1;
        return Plan{1, static_cast<int>(shares)};
    }
    if (rows > 128) {
        std::int64_t shares = 2 * units / tall_tiles;
        if (shares > longest) shares = longest;
        if (shares >= 2) return Plan{2, static_cast<int>(shares)};
    }
    const std::int64_t tiles = (rows + 127) / 128 * n_tiles;
    std::int64_t shares = units * (encoding == kEncQ6K ? 2 : 3) / tiles;
    if (shares > longest) shares = longest;
    if (shares < 1) shares = 1;
    return Plan{1, static_cast<int>(shares)};
}

template <std::uint32_t ENC>
void launch_encoding(const Descriptor& descriptor, const std::uint8_t* activations,
                     const float* inverse_scale, float* output, float* partials,
                     std::int64_t rows, hipStream_t stream) {
    const std::int64_t n_tiles = (descriptor.output_dim + kBN - 1) / kBN;
    const Plan chosen = plan(ENC, rows, descriptor.output_dim, descriptor.input_dim);
    const std::int64_t count = rows * descriptor.output_dim;
    float* target = chosen.shares > 1 ? partials : output;
    const std::int64_t split_stride = chosen.shares > 1 ? count : 0;
    if (chosen.row_blocks == 2) {
        const int m_tiles = static_cast<int>((rows + 255) / 256);
        hipLaunchKernelGGL((gemm_f16_kernel<ENC, 2>),
                           dim3(static_cast<unsigned>(m_tiles * n_tiles), chosen.shares),
                           dim3(kThreads), 2 * kStageBytes, stream, descriptor.data,
                           descriptor.row_stride_bytes, descriptor.output_dim,
                           descriptor.input_dim, activations, inverse_scale, target, rows, m_tiles,
                           split_stride);
    } else {
        const int m_tiles = static_cast<int>((rows + 127) / 128);
        hipLaunchKernelGGL((gemm_f16_kernel<ENC, 1>),
                           dim3(static_cast<unsigned>(m_tiles * n_tiles), chosen.shares),
                           dim3(kThreads), 2 * kStageBytes, stream, descriptor.data,
                           descriptor.row_stride_bytes, descriptor.output_dim,
                           descriptor.input_dim, activations, inverse_scale, target, rows, m_tiles,
                           split_stride);
    }
    if (chosen.shares > 1) {
        const std::int64_t blocks = (count + 1023) / 1024;
        hipLaunchKernelGGL(sum_shares_kernel, dim3(static_cast<unsigned>(blocks < 4096 ? blocks : 4096)),
                           dim3(256), 0, stream, partials, output, count, chosen.shares);
    }
}

std::int64_t padded_rows(std::int64_t rows) { return (rows + kBM - 1) / kBM * kBM; }

// fp16 activations in whole 256-row tiles, then the inverse scale of every row (8 bytes a row
// are kept for it: the size is part of what callers were told to allocate)
std::int64_t activation_bytes(std::int64_t rows, std::int64_t input_dim) {
    return (padded_rows(rows) * input_dim * 2 + padded_rows(rows) * 8 + 255) & ~std::int64_t(255);
}

}  // namespace

std::int64_t gemm_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim,
                                      std::int64_t output_dim) {
    // the activations, then one copy of the output per K share of a split
    // launch (the encoding with the most shares bounds the others)
    const int shares = plan(kEncQ4K, rows, output_dim, input_dim).shares;
    return activation_bytes(rows, input_dim) + (shares > 1 ? shares * rows * output_dim * 4 : 0) + 256;
}

void gemm_f16_plan(std::uint32_t encoding, std::int64_t rows, std::int64_t input_dim,
                   std::int64_t output_dim, int* tile_rows, int* k_shares) {
    const Plan chosen = plan(encoding, rows, output_dim, input_dim);
    *tile_rows = 128 * chosen.row_blocks;
    *k_shares = chosen.shares;
}

bool gemm_f16_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K ||
            encoding == kEncQ8_0) && input_dim % 256 == 0;
}

void convert_gemm_activations(const float* input, std::int64_t rows, std::int64_t input_dim,
                              void* workspace, hipStream_t stream) {
    std::uint8_t* activations = static_cast<std::uint8_t*>(workspace);
    float* inverse_scale = reinterpret_cast<float*>(activations + padded_rows(rows) * input_dim * 2);
    const std::int64_t groups = input_dim / 8;
    const unsigned whole_rows = static_cast<unsigned>(padded_rows(rows) / 4);  // a wave per row
    if (groups <= 64 * 8) {
        hipLaunchKernelGGL((prepare_activations_kernel<8, 1>), dim3(whole_rows), dim3(256), 0, stream,
                           input, activations, inverse_scale, rows, input_dim);
    } else if (groups <= 64 * 16) {
        hipLaunchKernelGGL((prepare_activations_kernel<16, 1>), dim3(whole_rows), dim3(256), 0, stream,
                           input, activations, inverse_scale, rows, input_dim);
    } else if (groups <= 2 * 64 * 16) {
        hipLaunchKernelGGL((prepare_activations_kernel<16, 2>), dim3(2 * whole_rows), dim3(256), 0,
                           stream, input, activations, inverse_scale, rows, input_dim);
    } else {
        hipLaunchKernelGGL((prepare_activations_kernel<0, 1>), dim3(whole_rows), dim3(256), 0, stream,
                           input, activations, inverse_scale, rows, input_dim);
    }
}

void launch_gemm_f16(const Descriptor& descriptor, const float* input, float* output,
                     std::int64_t rows, void* workspace, hipStream_t stream) {
    convert_gemm_activations(input, rows, descriptor.input_dim, workspace, stream);
    launch_gemm_f16_converted(descriptor, output, rows, workspace, stream);
}

void launch_gemm_f16_converted(const Descriptor& descriptor, float* output, std::int64_t rows,
                               void* workspace, hipStream_t stream) {
    std::uint8_t* activations = static_cast<std::uint8_t*>(workspace);
    float* inverse_scale =
        reinterpret_cast<float*>(activations + padded_rows(rows) * descriptor.input_dim * 2);
    float* partials =
        reinterpret_cast<float*>(activations + activation_bytes(rows, descriptor.input_dim));
    switch (descriptor.encoding) {
        case kEncQ4K:
            launch_encoding<kEncQ4K>(descriptor, activations, inverse_scale, output, partials, rows,
                                     stream);
            break;
        case kEncQ5K:
            launch_encoding<kEncQ5K>(descriptor, activations, inverse_scale, output, partials, rows,
                                     stream);
            break;
        case kEncQ6K:
            launch_encoding<kEncQ6K>(descriptor, activations, inverse_scale, output, partials, rows,
                                     stream);
            break;
        default:
            launch_encoding<kEncQ8_0>(descriptor, activations, inverse_scale, output, partials, rows,
                                     stream);
            break;
    }
}

}  // namespace nfn
