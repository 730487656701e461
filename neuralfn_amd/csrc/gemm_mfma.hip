// Prefill dequant-GEMM on the bf16 matrix cores:
//   Y[M, N] = X[M, K] * W[N, K]^T,  W packed (Q4_K / Q5_K / Q6_K / Q8_0).
//
// A workgroup (4 waves, 2 x 2) owns a 256 x 128 tile of Y and walks K in steps
// of 64.  Per step it
//   - copies its 256 x 64 slice of the activations (bf16, converted once per
//     call by a small pre-pass into the workspace) into LDS with 16-byte loads,
//   - dequantizes the 128 x 64 slice of the weights: every thread turns 16
//     packed bytes (32 weights of one row: 16 of each 32-value sub-block of the
//     pair) into bf16 in registers, w = (d*sc)*q - dmin*m rounded to nearest
//     even, and writes them to LDS — the packed bytes are read from HBM once
//     per tile column and never exist dequantized in memory,
//   - runs 32 v_mfma_f32_32x32x16_bf16 per wave on a 128 x 64 sub-tile with
//     float accumulators.
// LDS is double-buffered, so the loads and the dequantization of step k+1 are
// issued between the matrix instructions of step k; rows are padded to 144
// bytes so that the 16-byte operand reads of 32 lanes hit distinct banks.
// Consecutive workgroups walk M first: with 8 XCDs picking workgroups round
// robin each XCD keeps one or two 256-row slices of X in its L2 while the
// packed weights stream through.
//
// The reference has no kernel of this kind: its small-batch path stops at 16
// rows (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1326-1328) and more rows run
// the float kernel neuralfn/csrc/tile_cuda/kernels.cu:1398-1525.  Weight
// decode arithmetic: neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616.
#include "common.hpp"
#include "gemm_mfma.hpp"

namespace nfn {

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));

constexpr int kBM = 256;
constexpr int kBN = 128;
constexpr int kBK = 64;
constexpr int kThreads = 256;
constexpr int kRowBytes = 144;  // 64 bf16 + 16 bytes of padding
constexpr int kTileA = kBM * kRowBytes;
constexpr int kTileB = kBN * kRowBytes;
constexpr int kStageBytes = kTileA + kTileB;

struct __attribute__((packed, aligned(2))) Chunk16 {
    std::uint32_t v[4];
};

__device__ __forceinline__ std::uint32_t pack_bf16(float lo, float hi) {
    const bf16x2 pair = {static_cast<__bf16>(lo), static_cast<__bf16>(hi)};
    return __builtin_bit_cast(std::uint32_t, pair);
}

// fp32 -> bf16 (round to nearest even) copy of the activations
// into whole 256-row tiles: rows past the end are written as zeros
__global__ __launch_bounds__(256) void convert_activations_kernel(
    const float* __restrict__ input, std::uint32_t* __restrict__ output, std::int64_t quads,
    std::int64_t padded_quads) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t i = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         i < padded_quads; i += stride) {
        float4 x = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
        if (i < quads) x = reinterpret_cast<const float4*>(input)[i];
        reinterpret_cast<uint2*>(output)[i] = make_uint2(pack_bf16(x.x, x.y), pack_bf16(x.z, x.w));
    }
}

// What one thread holds of the packed weights of one K step: its row's 16
// bytes of codes for positions 16*half .. 16*half+15 of both 32-value groups,
// plus the scale bytes it needs.
template <std::uint32_t ENC>
struct PackedSlice;

template <>
struct PackedSlice<kEncQ4K> {
    uint4 header;
    uint4 codes;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 144;
        header = *reinterpret_cast<const uint4*>(p);
        codes = *reinterpret_cast<const uint4*>(p + 16 + pair * 32 + half * 16);
    }
    // w[0..15]: first group, w[16..31]: second group
    __device__ __forceinline__ void decode(int pair, int, std::uint32_t (&out)[16]) const {
        const float d = half_bits_to_float(header.x & 0xffffu);
        const float dmin = half_bits_to_float(header.x >> 16);
        const std::uint32_t y = header.y, z = header.z, w = header.w;
        const int shift = 16 * (pair & 1);
        const std::uint32_t ys = y >> shift, zs = z >> shift, ws = w >> shift;
        // sub-blocks 4..7 keep their 6-bit values split over two bytes; bit masks
        // instead of a branch keep the K step one basic block
        const std::uint32_t upper = 0u - static_cast<std::uint32_t>(pair >> 1);
        const std::uint32_t sc = (((ws & 0x0f0fu) | ((ys >> 2) & 0x3030u)) & upper) |
            ((ys & 0x3f3fu) & ~upper);
        const std::uint32_t mn = ((((ws >> 4) & 0x0f0fu) | ((zs >> 2) & 0x3030u)) & upper) |
            ((zs & 0x3f3fu) & ~upper);
        const float da = d * static_cast<float>(sc & 0xffu);
        const float db = d * static_cast<float>((sc >> 8) & 0xffu);
        const float ma = dmin * static_cast<float>(mn & 0xffu);
        const float mb = dmin * static_cast<float>((mn >> 8) & 0xffu);
        const std::uint32_t words[4] = {codes.x, codes.y, codes.z, codes.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const std::uint32_t lo = words[i] & 0x0f0f0f0fu;
            const std::uint32_t hi = (words[i] >> 4) & 0x0f0f0f0fu;
            float a[4], b[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                // (d*sc)*q - dmin*m in one fused step; the bf16 rounding that
                // follows is 2^-9, far above the difference to two roundings
                a[k] = fmaf(static_cast<float>((lo >> (8 * k)) & 0xffu), da, -ma);
                b[k] = fmaf(static_cast<float>((hi >> (8 * k)) & 0xffu), db, -mb);
            }
            out[2 * i] = pack_bf16(a[0], a[1]);
            out[2 * i + 1] = pack_bf16(a[2], a[3]);
            out[8 + 2 * i] = pack_bf16(b[0], b[1]);
            out[8 + 2 * i + 1] = pack_bf16(b[2], b[3]);
        }
    }
};

template <>
struct PackedSlice<kEncQ5K> {
    uint4 header;
    uint4 codes;
    uint4 high;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 176;
        header = *reinterpret_cast<const uint4*>(p);
        high = *reinterpret_cast<const uint4*>(p + 16 + half * 16);
        codes = *reinterpret_cast<const uint4*>(p + 48 + pair * 32 + half * 16);
    }
    __device__ __forceinline__ void decode(int pair, int, std::uint32_t (&out)[16]) const {
        const float d = half_bits_to_float(header.x & 0xffffu);
        const float dmin = half_bits_to_float(header.x >> 16);
        const int shift = 16 * (pair & 1);
        const std::uint32_t ys = header.y >> shift, zs = header.z >> shift, ws = header.w >> shift;
        // sub-blocks 4..7 keep their 6-bit values split over two bytes; bit masks
        // instead of a branch keep the K step one basic block
        const std::uint32_t upper = 0u - static_cast<std::uint32_t>(pair >> 1);
        const std::uint32_t sc = (((ws & 0x0f0fu) | ((ys >> 2) & 0x3030u)) & upper) |
            ((ys & 0x3f3fu) & ~upper);
        const std::uint32_t mn = ((((ws >> 4) & 0x0f0fu) | ((zs >> 2) & 0x3030u)) & upper) |
            ((zs & 0x3f3fu) & ~upper);
        const float da = d * static_cast<float>(sc & 0xffu);
        const float db = d * static_cast<float>((sc >> 8) & 0xffu);
        const float ma = dmin * static_cast<float>(mn & 0xffu);
        const float mb = dmin * static_cast<float>((mn >> 8) & 0xffu);
        const std::uint32_t words[4] = {codes.x, codes.y, codes.z, codes.w};
        const std::uint32_t bits[4] = {high.x, high.y, high.z, high.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const std::uint32_t shifted = bits[i] >> (2 * pair);
            const std::uint32_t lo = (words[i] & 0x0f0f0f0fu) | ((shifted & 0x01010101u) << 4);
            const std::uint32_t hi = ((words[i] >> 4) & 0x0f0f0f0fu) | ((shifted & 0x02020202u) << 3);
            float a[4], b[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a[k] = fmaf(static_cast<float>((lo >> (8 * k)) & 0xffu), da, -ma);
                b[k] = fmaf(static_cast<float>((hi >> (8 * k)) & 0xffu), db, -mb);
            }
            out[2 * i] = pack_bf16(a[0], a[1]);
            out[2 * i + 1] = pack_bf16(a[2], a[3]);
            out[8 + 2 * i] = pack_bf16(b[0], b[1]);
            out[8 + 2 * i + 1] = pack_bf16(b[2], b[3]);
        }
    }
};

template <>
struct PackedSlice<kEncQ6K> {
    // a K step of 64 is two quarters (32 values each) of one half of the block:
    // quarters (0,1) or (2,3); `pair` = 2*half_of_block + (quarters 2,3 ? 1 : 0)
    uint4 low_a, low_b, high;
    std::uint32_t scale_bytes;  // the four int8 sub-scales of the two quarters
    std::uint32_t d_bits;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + block * 210;
        const int block_half = pair >> 1;
        const Chunk16 la = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + half * 16);
        const Chunk16 lb = *reinterpret_cast<const Chunk16*>(p + block_half * 64 + 32 + half * 16);
        const Chunk16 hb = *reinterpret_cast<const Chunk16*>(p + 128 + block_half * 32 + half * 16);
        low_a = make_uint4(la.v[0], la.v[1], la.v[2], la.v[3]);
        low_b = make_uint4(lb.v[0], lb.v[1], lb.v[2], lb.v[3]);
        high = make_uint4(hb.v[0], hb.v[1], hb.v[2], hb.v[3]);
        const std::uint8_t* s = p + 192 + block_half * 8 + (pair & 1) * 4;
        scale_bytes = static_cast<std::uint32_t>(s[0]) | (static_cast<std::uint32_t>(s[1]) << 8) |
            (static_cast<std::uint32_t>(s[2]) << 16) | (static_cast<std::uint32_t>(s[3]) << 24);
        d_bits = static_cast<std::uint32_t>(p[208]) | (static_cast<std::uint32_t>(p[209]) << 8);
    }
    __device__ __forceinline__ void decode(int pair, int half, std::uint32_t (&out)[16]) const {
        const float d = half_bits_to_float(d_bits);
        const int upper = (pair & 1) * 4;  // quarters 2,3: high nibbles, high-bit pairs 4..7
        // sub-scale index = quarter*2 + lane/16: this thread's 16 values sit in one 16-group
        const int sa = static_cast<std::int8_t>((scale_bytes >> (8 * half)) & 0xffu);
        const int sb = static_cast<std::int8_t>((scale_bytes >> (8 * (2 + half))) & 0xffu);
        const float da = __fmul_rn(d, static_cast<float>(sa));
        const float db = __fmul_rn(d, static_cast<float>(sb));
        const std::uint32_t la[4] = {low_a.x, low_a.y, low_a.z, low_a.w};
        const std::uint32_t lb[4] = {low_b.x, low_b.y, low_b.z, low_b.w};
        const std::uint32_t hb[4] = {high.x, high.y, high.z, high.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const std::uint32_t na = (la[i] >> upper) & 0x0f0f0f0fu;
            const std::uint32_t nb = (lb[i] >> upper) & 0x0f0f0f0fu;
            const std::uint32_t ha = hb[i] >> upper;  // bits 0,1 -> first quarter
            const std::uint32_t qa = na | ((ha & 0x03030303u) << 4);
            const std::uint32_t qb = nb | (((ha >> 2) & 0x03030303u) << 4);
            float a[4], b[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a[k] = fmaf(static_cast<float>((qa >> (8 * k)) & 0xffu), da, -32.0f * da);
                b[k] = fmaf(static_cast<float>((qb >> (8 * k)) & 0xffu), db, -32.0f * db);
            }
            out[2 * i] = pack_bf16(a[0], a[1]);
            out[2 * i + 1] = pack_bf16(a[2], a[3]);
            out[8 + 2 * i] = pack_bf16(b[0], b[1]);
            out[8 + 2 * i + 1] = pack_bf16(b[2], b[3]);
        }
    }
};

template <>
struct PackedSlice<kEncQ8_0> {
    // a K step of 64 is two 34-byte blocks; `pair` counts K steps inside 256 values
    uint4 codes_a, codes_b;
    std::uint32_t d_a, d_b;
    __device__ __forceinline__ void load(const std::uint8_t* row, int block, int pair, int half) {
        const std::uint8_t* p = row + (block * 8 + pair * 2) * 34;
        const Chunk16 a = *reinterpret_cast<const Chunk16*>(p + 2 + half * 16);
        const Chunk16 b = *reinterpret_cast<const Chunk16*>(p + 34 + 2 + half * 16);
        codes_a = make_uint4(a.v[0], a.v[1], a.v[2], a.v[3]);
        codes_b = make_uint4(b.v[0], b.v[1], b.v[2], b.v[3]);
        d_a = static_cast<std::uint32_t>(p[0]) | (static_cast<std::uint32_t>(p[1]) << 8);
        d_b = static_cast<std::uint32_t>(p[34]) | (static_cast<std::uint32_t>(p[35]) << 8);
    }
    __device__ __forceinline__ void decode(int, int, std::uint32_t (&out)[16]) const {
        const float da = half_bits_to_float(d_a);
        const float db = half_bits_to_float(d_b);
        const std::uint32_t wa[4] = {codes_a.x, codes_a.y, codes_a.z, codes_a.w};
        const std::uint32_t wb[4] = {codes_b.x, codes_b.y, codes_b.z, codes_b.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float a[4], b[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                a[k] = __fmul_rn(da, static_cast<float>(static_cast<std::int8_t>((wa[i] >> (8 * k)) & 0xffu)));
                b[k] = __fmul_rn(db, static_cast<float>(static_cast<std::int8_t>((wb[i] >> (8 * k)) & 0xffu)));
            }
            out[2 * i] = pack_bf16(a[0], a[1]);
            out[2 * i + 1] = pack_bf16(a[2], a[3]);
            out[8 + 2 * i] = pack_bf16(b[0], b[1]);
            out[8 + 2 * i + 1] = pack_bf16(b[2], b[3]);
        }
    }
};

typedef std::uint32_t u32x4 __attribute__((ext_vector_type(4)));

// Eight 16-byte chunks of activations in named registers (an array here ends up
// in scratch memory).
struct ActivationSlice {
    u32x4 c0, c1, c2, c3, c4, c5, c6, c7;
};
#define NFN_EACH_CHUNK(X) X(0) X(1) X(2) X(3) X(4) X(5) X(6) X(7)

__device__ __forceinline__ void load_slice(ActivationSlice& a, const std::uint8_t* source,
                                           std::int64_t row_bytes) {
#define NFN_LOAD_CHUNK(i) a.c##i = *reinterpret_cast<const u32x4*>(source + i * 32 * row_bytes);
    NFN_EACH_CHUNK(NFN_LOAD_CHUNK)
#undef NFN_LOAD_CHUNK
}

__device__ __forceinline__ void store_slice(const ActivationSlice& a, std::uint8_t* target) {
#define NFN_STORE_CHUNK(i) *reinterpret_cast<u32x4*>(target + i * 32 * kRowBytes) = a.c##i;
    NFN_EACH_CHUNK(NFN_STORE_CHUNK)
#undef NFN_STORE_CHUNK
}

// One K step: the 32 matrix instructions of `stage`, the dequantization of the
// slice held in (a_next, b_next) into `other`, and the loads that refill them.
// The scheduling groups at the end ask for that work to be issued between the
// matrix instructions rather than after them.
template <std::uint32_t ENC>
__device__ __forceinline__ void k_step(
    v16f (&acc)[4][2], const std::uint8_t* a_read, const std::uint8_t* b_read,
    std::uint8_t* a_write, std::uint8_t* b_write, ActivationSlice& a_next,
    PackedSlice<ENC>& b_next, int decode_pair, int b_half,
    const std::uint8_t* a_global, std::int64_t a_row_bytes, const std::uint8_t* b_global,
    int fetch_step) {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        bf16x8 a[4], b[2];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            a[i] = *reinterpret_cast<const bf16x8*>(a_read + i * 32 * kRowBytes + kk * 32);
        }
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            b[j] = *reinterpret_cast<const bf16x8*>(b_read + j * 32 * kRowBytes + kk * 32);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    // dequantize the held slice into the other stage
    std::uint32_t w[16];
    b_next.decode(decode_pair, b_half, w);
    *reinterpret_cast<uint4*>(b_write) = make_uint4(w[0], w[1], w[2], w[3]);
    *reinterpret_cast<uint4*>(b_write + 16) = make_uint4(w[4], w[5], w[6], w[7]);
    *reinterpret_cast<uint4*>(b_write + 64) = make_uint4(w[8], w[9], w[10], w[11]);
    *reinterpret_cast<uint4*>(b_write + 80) = make_uint4(w[12], w[13], w[14], w[15]);
    store_slice(a_next, a_write);
    // refill
    load_slice(a_next, a_global + static_cast<std::int64_t>(fetch_step) * (kBK * 2), a_row_bytes);
    b_next.load(b_global, fetch_step >> 2, fetch_step & 3, b_half);

    // 32 x {1 matrix op, 1 LDS read, 4 vector ops}, LDS writes and global loads spread over them
#pragma unroll
    for (int g = 0; g < 32; ++g) {
        __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
        if (g < 24) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
        if (g >= 12 && g < 24) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);
        if (g >= 22) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
    }
}

template <std::uint32_t ENC>
__global__ __launch_bounds__(kThreads) void gemm_bf16_kernel(
    const std::uint8_t* __restrict__ weights, std::int64_t row_stride, std::int64_t output_dim,
    std::int64_t input_dim, const std::uint16_t* __restrict__ activations,
    float* __restrict__ output, std::int64_t rows, int m_tiles) {
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

    ActivationSlice a_even, a_odd;  // hold steps s+2 (even s) and s+1 while step s computes
    PackedSlice<ENC> b_even, b_odd;
    auto fetch = [&](ActivationSlice& a, PackedSlice<ENC>& b, int step) {
        load_slice(a, a_global + static_cast<std::int64_t>(step) * (kBK * 2), a_row_bytes);
        b.load(b_global, step >> 2, step & 3, b_half);
    };
    fetch(a_even, b_even, 0);
    fetch(a_odd, b_odd, 1);
    {
        std::uint32_t w[16];
        b_even.decode(0, b_half, w);
        std::uint8_t* target = lds + b_target;
        *reinterpret_cast<uint4*>(target) = make_uint4(w[0], w[1], w[2], w[3]);
        *reinterpret_cast<uint4*>(target + 16) = make_uint4(w[4], w[5], w[6], w[7]);
        *reinterpret_cast<uint4*>(target + 64) = make_uint4(w[8], w[9], w[10], w[11]);
        *reinterpret_cast<uint4*>(target + 80) = make_uint4(w[12], w[13], w[14], w[15]);
        store_slice(a_even, lds + a_target);
    }
    fetch(a_even, b_even, 2);
    __syncthreads();

    const int operand = (lane & 31) * kRowBytes + (lane >> 5) * 16;
    const std::uint8_t* a_read0 = lds + wave_m * 128 * kRowBytes + operand;
    const std::uint8_t* b_read0 = lds + kTileA + wave_n * 64 * kRowBytes + operand;
    for (int step = 0; step < steps; step += 2) {
        // stage 0 computes; step+1 (odd slice) goes to stage 1; odd slice refills with step+3
        k_step<ENC>(acc, a_read0, b_read0, lds + kStageBytes + a_target,
                    lds + kStageBytes + b_target, a_odd, b_odd, (step + 1) & 3, b_half, a_global,
                    a_row_bytes, b_global, min(step + 3, last));
        __syncthreads();
        // stage 1 computes; step+2 (even slice) goes to stage 0; even slice refills with step+4
        k_step<ENC>(acc, a_read0 + kStageBytes, b_read0 + kStageBytes, lds + a_target,
                    lds + b_target, a_even, b_even, (step + 2) & 3, b_half, a_global, a_row_bytes,
                    b_global, min(step + 4, last));
        __syncthreads();
    }

    // D register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
    const int column = lane & 31;
    const int row_base = (lane >> 5) * 4;
    const bool whole = m0 + kBM <= rows && n0 + kBN <= output_dim;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const std::int64_t n = n0 + wave_n * 64 + j * 32 + column;
            float* target = output + (m0 + wave_m * 128 + i * 32 + row_base) * output_dim + n;
            if (whole) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    target[(8 * (r >> 2) + (r & 3)) * output_dim] = acc[i][j][r];
                }
            } else {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const std::int64_t m = m0 + wave_m * 128 + i * 32 + 8 * (r >> 2) + row_base + (r & 3);
                    if (m < rows && n < output_dim) output[m * output_dim + n] = acc[i][j][r];
                }
            }
        }
    }
}

template <std::uint32_t ENC>
void launch_encoding(const Descriptor& descriptor, const std::uint16_t* activations, float* output,
                     std::int64_t rows, hipStream_t stream) {
    auto kernel = gemm_bf16_kernel<ENC>;
    static const bool raised =
        hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) == hipSuccess;
    (void)raised;
    const int m_tiles = static_cast<int>((rows + kBM - 1) / kBM);
    const std::int64_t n_tiles = (descriptor.output_dim + kBN - 1) / kBN;
    hipLaunchKernelGGL(kernel, dim3(static_cast<unsigned>(m_tiles * n_tiles)), dim3(kThreads),
                       2 * kStageBytes, stream, descriptor.data, descriptor.row_stride_bytes,
                       descriptor.output_dim, descriptor.input_dim, activations, output, rows,
                       m_tiles);
}

}  // namespace

std::int64_t gemm_bf16_workspace_bytes(std::int64_t rows, std::int64_t input_dim) {
    const std::int64_t padded_rows = (rows + kBM - 1) / kBM * kBM;
    return padded_rows * input_dim * 2 + 256;
}

bool gemm_bf16_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K ||
            encoding == kEncQ8_0) && input_dim % 256 == 0;
}

void launch_gemm_bf16(const Descriptor& descriptor, const float* input, float* output,
                      std::int64_t rows, void* workspace, hipStream_t stream) {
    std::uint16_t* activations = static_cast<std::uint16_t*>(workspace);
    const std::int64_t quads = rows * descriptor.input_dim / 4;
    const std::int64_t padded_quads = (rows + kBM - 1) / kBM * kBM * descriptor.input_dim / 4;
    const std::int64_t blocks = (padded_quads + 255) / 256;
    hipLaunchKernelGGL(convert_activations_kernel,
                       dim3(static_cast<unsigned>(blocks < 65536 ? blocks : 65536)), dim3(256), 0,
                       stream, input, reinterpret_cast<std::uint32_t*>(activations), quads,
                       padded_quads);
    switch (descriptor.encoding) {
        case kEncQ4K: launch_encoding<kEncQ4K>(descriptor, activations, output, rows, stream); break;
        case kEncQ5K: launch_encoding<kEncQ5K>(descriptor, activations, output, rows, stream); break;
        case kEncQ6K: launch_encoding<kEncQ6K>(descriptor, activations, output, rows, stream); break;
        default: launch_encoding<kEncQ8_0>(descriptor, activations, output, rows, stream); break;
    }
}

}  // namespace nfn
