// Small-batch (3..16 rows) GEMV on the fp16 matrix cores.
//
// A small launch first turns the activations into fp16, every K share of a
// row (the blocks one wave of the main kernel multiplies) scaled by the power
// of two that brings its largest magnitude into [2^14, 2^15), and stores them
// in the caller's workspace by groups of eight columns:
// [column / 8][row][8 values], so that the 16 bytes one lane feeds to a matrix
// instruction are contiguous and the lanes of a quarter wave read one segment.
// Fused prologues (sigmoid gate, SwiGLU) are applied there.
//
// In the main kernel a workgroup of 8 waves owns tiles of 16 consecutive
// weight rows (persistent: tiles blockIdx.x, blockIdx.x + gridDim.x, ...).
// The waves split K by 256-value blocks and meet once per tile in a
// fixed-order sum.  Per block a lane (row i = lane % 16, quarter j = lane / 16)
// loads its share of the packed bytes of row i straight into registers (the
// block's header and a quarter of its codes), dequantizes them to fp16 with
// packed arithmetic and feeds eight v_mfma_f32_16x16x32_f16: operand B is the
// weights (column = weight row), operand A the activations (row = token).
// The K index of a matrix instruction is only a pairing of A and B elements,
// so every format picks the eight columns a lane contributes from the bytes
// it already holds; the activation address follows that choice.  Weights are
// read from HBM once.  Q4_K and Q5_K bytes go from memory to the registers of
// the lane that decodes them; Q6_K (rows of up to 8,192 columns) and Q8_0
// blocks are brought into a per-wave ring in LDS first, whole, and read from
// there (the RING form below, with the measurements that chose it).
//
// Arithmetic it replaces: the reference's small-batch kernel
// (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1174-1303), which multiplies 8-bit
// activation codes with the integer codes; here the weights are dequantized
// ((q * d*sc - dmin*m) rounded to fp16, 11 significant bits) and the
// activations keep 11 significant bits each, which stays within 2e-3 of the
// float-activation CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:655-679) like the prefill
// GEMM with the same number formats.  Results do not depend on the launch
// geometry: the sum over K runs block by block inside a wave and the eight
// waves' partial sums are added in wave order.
#include "common.hpp"
#include "f16_decode.hpp"
#include "gemv_f16.hpp"
#include "lm_head.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef int i32x4 __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
constexpr int kDepth = 4;  // blocks in flight per wave

// ---- activations: fp32 -> fp16 scaled per row and K share, [column / 8][row][8] ----

constexpr int kImageThreads = 256;
constexpr int kImageHeld = 2;  // 8-column groups a thread keeps: shares of up to 16 blocks are read once
static_assert(kHalfImageShares == kWaves, "a share of the image is a wave's share of K");

// One workgroup per (row, share): blockIdx.x = row * kWaves + share.
template <int P>
__global__ __launch_bounds__(kImageThreads) void f16_image_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    std::uint8_t* __restrict__ image, float* __restrict__ inverse_scale, int tokens,
    int input_dim) {
    __shared__ float maxima[kImageThreads / kWave];
    const int token = blockIdx.x / kWaves;
    const int share = blockIdx.x - token * kWaves;
    const int blocks = input_dim >> 8;
    const int group0 = 32 * half_image_share_begin(blocks, share);  // 32 groups of 8 columns a block
    const int groups = 32 * half_image_share_begin(blocks, share + 1) - group0;
    const std::int64_t base = static_cast<std::int64_t>(token) * input_dim;
    const bool held = groups <= kImageThreads * kImageHeld;  // uniform
    float4 x[kImageHeld][2];
    float largest = 0.0f;
    if (held) {
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j) {
            const int g = threadIdx.x + kImageThreads * j;
            x[j][0] = make_float4(0.0f, 0.0f, 0.0f, 0.0f);
            x[j][1] = x[j][0];
            if (g < groups) {
                x[j][0] = load_activations<P>(first, second, base + (group0 + g) * 8);
                x[j][1] = load_activations<P>(first, second, base + (group0 + g) * 8 + 4);
            }
        }
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j) largest = largest_of(x[j][1], largest_of(x[j][0], largest));
    } else {
        for (int g = threadIdx.x; g < groups; g += kImageThreads) {
            largest = largest_of(load_activations<P>(first, second, base + (group0 + g) * 8), largest);
            largest = largest_of(load_activations<P>(first, second, base + (group0 + g) * 8 + 4), largest);
        }
    }
    // NaN never wins fmaxf: a share with NaN keeps its largest finite magnitude
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) largest = fmaxf(largest, __shfl_xor(largest, offset));
    if ((threadIdx.x & 63) == 0) maxima[threadIdx.x >> 6] = largest;
    __syncthreads();
#pragma unroll
    for (int w = 0; w < kImageThreads / kWave; ++w) largest = fmaxf(largest, maxima[w]);
    const HalfImageScale scale = half_image_scale(largest);
    if (threadIdx.x == 0) inverse_scale[token * kWaves + share] = scale.inverse;
    auto store = [&](int g, float4 a, float4 b) {
        half_image_store(image, group0 + g, tokens, token, a, b, scale.factor);
    };
    if (held) {
#pragma unroll
        for (int j = 0; j < kImageHeld; ++j) {
            const int g = threadIdx.x + kImageThreads * j;
            if (g < groups) store(g, x[j][0], x[j][1]);
        }
    } else {
        for (int g = threadIdx.x; g < groups; g += kImageThreads) {
            store(g, load_activations<P>(first, second, base + (group0 + g) * 8),
                  load_activations<P>(first, second, base + (group0 + g) * 8 + 4));
        }
    }
}

// ---- what one lane holds of one 256-value block of its weight row ---------------
// load(): the packed bytes (header and this quarter's codes) of the block at
//   `block` (uniform) + `row` (this lane's byte offset, 32 bits): a scalar base
//   and a 32-bit lane offset, the addressing form that needs no address arithmetic.
// prepare(): the fp16 scale constants.
// operand<M>(): the eight weights of matrix instruction M as fp16.
// lane_group(j) + step_group(m): which group of eight columns of the block those are.

typedef const __attribute__((address_space(1))) std::uint8_t* GlobalBytes;
typedef const __attribute__((address_space(1))) u32x4* GlobalVec;
typedef const __attribute__((address_space(1))) f16x8* GlobalFragment;

__device__ __forceinline__ f16x8 as_operand(std::uint32_t a, std::uint32_t b, std::uint32_t c,
                                            std::uint32_t d) {
    return __builtin_bit_cast(f16x8, u32x4{a, b, c, d});
}

// kQuadFetch: the packed bytes are fetched by quads of lanes instead of by the lanes that use
//   them, and change_lanes() moves them there (see the kernel).

template <std::uint32_t ENC>
struct PackedBlock;

// Pieces of a row's packed bytes where a wave has laid them out in LDS (load_tile() below):
// aligned to two bytes only (a Q6_K block is 210 bytes long, and a tensor may start anywhere).
struct __attribute__((packed, aligned(2))) TilePiece16 {
    std::uint32_t v[4];
};
struct __attribute__((packed, aligned(2))) TilePiece8 {
    std::uint32_t v[2];
};
struct __attribute__((packed, aligned(2))) TilePiece4 {
    std::uint32_t v;
};
__device__ __forceinline__ u32x4 tile_read16(const std::uint8_t* at) {
    const TilePiece16 piece = *reinterpret_cast<const TilePiece16*>(at);
    return u32x4{piece.v[0], piece.v[1], piece.v[2], piece.v[3]};
}

// The value of the lane whose number times four is `source` (any permutation of the lanes).
__device__ __forceinline__ std::uint32_t from_lane(int source, std::uint32_t value) {
    return static_cast<std::uint32_t>(__builtin_amdgcn_ds_bpermute(source, static_cast<int>(value)));
}
__device__ __forceinline__ u32x4 from_lane(int source, u32x4 value) {
    return u32x4{from_lane(source, value[0]), from_lane(source, value[1]), from_lane(source, value[2]),
                 from_lane(source, value[3])};
}

// Q4_K: a 16-byte piece c of the 128 code bytes holds values 16*(c%2)..+15 of
// sub-blocks 2*(c/2) (low nibbles) and 2*(c/2)+1 (high nibbles).  Quarter j
// takes pieces j and j + 4; instructions 0..3 use the first, 4..7 the second:
// M % 4 = 2*(high nibbles) + (second eight values).
template <>
struct PackedBlock<kEncQ4K> {
    static constexpr int kBytes = 144;
    static constexpr bool kQuadFetch = false;
    __device__ __forceinline__ void change_lanes(int) {}
    u32x4 header, piece[2];
    KBlockScales scales[2];
    __device__ __forceinline__ void load(GlobalBytes block, std::uint32_t row, int j) {
        header = *reinterpret_cast<GlobalVec>(block + row);
        const std::uint32_t mine = row + 16 + 16 * j;
        piece[0] = *reinterpret_cast<GlobalVec>(block + mine);
        piece[1] = *reinterpret_cast<GlobalVec>(block + mine + 64);
    }
    // the same registers from the block at `at` in LDS
    __device__ __forceinline__ void load_tile(const std::uint8_t* at, int j) {
        header = tile_read16(at);
        piece[0] = tile_read16(at + 16 + 16 * j);
        piece[1] = tile_read16(at + 80 + 16 * j);
    }
    __device__ __forceinline__ void prepare(int j) {
        scales[0].bits(header, j >> 1);
        scales[0].scales(header);
        scales[1].bits(header, (j >> 1) + 2);
        scales[1].scales(header);
    }
    __device__ __forceinline__ static int lane_group(int j) { return 8 * (j >> 1) + 2 * (j & 1); }
    static constexpr int step_group(int m) { return 16 * (m >> 2) + 4 * ((m >> 1) & 1) + (m & 1); }
    template <int M>
    __device__ __forceinline__ f16x8 operand() const {
        constexpr int kPiece = M >> 2, kHigh = (M >> 1) & 1, kWord = 2 * (M & 1);
        const KBlockScales& s = scales[kPiece];
        const std::uint32_t a = (kHigh ? piece[kPiece][kWord] >> 4 : piece[kPiece][kWord]) & 0x0f0f0f0fu;
        const std::uint32_t b =
            (kHigh ? piece[kPiece][kWord + 1] >> 4 : piece[kPiece][kWord + 1]) & 0x0f0f0f0fu;
        std::uint32_t out[4];
        scale_bytes(a, splat(-1024.0f), kHigh ? s.scale_b : s.scale_a, kHigh ? s.shift_b : s.shift_a,
                    out[0], out[1]);
        scale_bytes(b, splat(-1024.0f), kHigh ? s.scale_b : s.scale_a, kHigh ? s.shift_b : s.shift_a,
                    out[2], out[3]);
        return as_operand(out[0], out[1], out[2], out[3]);
    }
};

// Q5_K: as Q4_K, and bit s of high-bit byte v is the fifth bit of value v of
// sub-block s; both pieces of a quarter cover values 16*(j%2)..+15.
template <>
struct PackedBlock<kEncQ5K> {
    static constexpr int kBytes = 176;
    static constexpr bool kQuadFetch = false;
    __device__ __forceinline__ void change_lanes(int) {}
    u32x4 header, fifth, piece[2];
    KBlockScales scales[2];
    int fifth_shift;  // sub-block of the first piece's low nibbles
    __device__ __forceinline__ void load(GlobalBytes block, std::uint32_t row, int j) {
        header = *reinterpret_cast<GlobalVec>(block + row);
        fifth = *reinterpret_cast<GlobalVec>(block + (row + 16 + 16 * (j & 1)));
        const std::uint32_t mine = row + 48 + 16 * j;
        piece[0] = *reinterpret_cast<GlobalVec>(block + mine);
        piece[1] = *reinterpret_cast<GlobalVec>(block + mine + 64);
    }
    __device__ __forceinline__ void load_tile(const std::uint8_t* at, int j) {
        header = tile_read16(at);
        fifth = tile_read16(at + 16 + 16 * (j & 1));
        piece[0] = tile_read16(at + 48 + 16 * j);
        piece[1] = tile_read16(at + 112 + 16 * j);
    }
    __device__ __forceinline__ void prepare(int j) {
        scales[0].bits(header, j >> 1);
        scales[0].scales(header);
        scales[1].bits(header, (j >> 1) + 2);
        scales[1].scales(header);
        fifth_shift = 2 * (j >> 1);
    }
    __device__ __forceinline__ static int lane_group(int j) { return PackedBlock<kEncQ4K>::lane_group(j); }
    static constexpr int step_group(int m) { return PackedBlock<kEncQ4K>::step_group(m); }
    template <int M>
    __device__ __forceinline__ f16x8 operand() const {
        constexpr int kPiece = M >> 2, kHigh = (M >> 1) & 1, kWord = 2 * (M & 1);
        const KBlockScales& s = scales[kPiece];
        const int shift = fifth_shift + 4 * kPiece + kHigh;  // the sub-block's bit
        std::uint32_t out[4];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const std::uint32_t word = piece[kPiece][kWord + w];
            const std::uint32_t nibbles = (kHigh ? word >> 4 : word) & 0x0f0f0f0fu;
            const std::uint32_t bit = ((fifth[kWord + w] >> shift) & 0x01010101u) << 4;
            scale_bytes(nibbles | bit, splat(-1024.0f), kHigh ? s.scale_b : s.scale_a,
                        kHigh ? s.shift_b : s.shift_a, out[2 * w], out[2 * w + 1]);
        }
        return as_operand(out[0], out[1], out[2], out[3]);
    }
};

// Q6_K: value v (0..31) of quarter q (0..3) of half n (0, 1) of the block has
// its low nibble in ql[64n + 32*(q%2) + v] (high nibble for q >= 2) and bits
// 2q, 2q+1 of qh[32n + v] on top; one int8 sub-scale per 16 values.  Quarter j
// of the wave takes values 16*(j%2)..+15 of every quarter of half j/2:
// instruction M = 2q + (second eight values).
template <>
struct PackedBlock<kEncQ6K> {
    static constexpr int kBytes = 210;
    // its parts are aligned to two bytes only, and a lane's unaligned 16-byte load is slow on
    // its own; the four of a quad, side by side in one row, are not
    static constexpr bool kQuadFetch = true;
    u32x4 low_a, low_b, top;
    std::uint32_t sub_scales[2];  // the eight of this lane's half
    std::uint32_t d_bits;
    f16x2 scale[4];  // per quarter
    __device__ __forceinline__ void load(GlobalBytes block, std::uint32_t row, int j) {
        const int n = j >> 1, h = j & 1;
        // the block is 210 bytes long: its parts are aligned to two bytes only
        typedef std::uint32_t Words4 __attribute__((ext_vector_type(4), aligned(2)));
        typedef std::uint32_t Words2 __attribute__((ext_vector_type(2), aligned(2)));
        typedef const __attribute__((address_space(1))) Words4* GlobalWords4;
        typedef const __attribute__((address_space(1))) Words2* GlobalWords2;
        typedef const __attribute__((address_space(1))) std::uint16_t* GlobalHalf;
        const std::uint32_t low = row + 64 * n + 16 * h;
        const Words4 a = *reinterpret_cast<GlobalWords4>(block + low);
        const Words4 b = *reinterpret_cast<GlobalWords4>(block + low + 32);
        const Words4 t = *reinterpret_cast<GlobalWords4>(block + (row + 128 + 32 * n + 16 * h));
        const Words2 s = *reinterpret_cast<GlobalWords2>(block + (row + 192 + 8 * n));
        low_a = u32x4{a[0], a[1], a[2], a[3]};
        low_b = u32x4{b[0], b[1], b[2], b[3]};
        top = u32x4{t[0], t[1], t[2], t[3]};
        sub_scales[0] = s[0];
        sub_scales[1] = s[1];
        d_bits = *reinterpret_cast<GlobalHalf>(block + (row + 208));
    }
    __device__ __forceinline__ void load_tile(const std::uint8_t* at, int j) {
        const int n = j >> 1, h = j & 1;
        low_a = tile_read16(at + 64 * n + 16 * h);
        low_b = tile_read16(at + 64 * n + 16 * h + 32);
        top = tile_read16(at + 128 + 32 * n + 16 * h);
        const TilePiece8 s = *reinterpret_cast<const TilePiece8*>(at + 192 + 8 * n);
        sub_scales[0] = s.v[0];
        sub_scales[1] = s.v[1];
        d_bits = *reinterpret_cast<const std::uint16_t*>(at + 208);
    }
    __device__ __forceinline__ void change_lanes(int source) {
        low_a = from_lane(source, low_a);
        low_b = from_lane(source, low_b);
        top = from_lane(source, top);
        sub_scales[0] = from_lane(source, sub_scales[0]);
        sub_scales[1] = from_lane(source, sub_scales[1]);
        d_bits = from_lane(source, d_bits);
    }
    __device__ __forceinline__ void prepare(int j) {
        const float d = half_bits_to_float(d_bits);
        const int within = 8 * (j & 1);
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            // sub-scale 8n + 2q + j%2: byte (2q + j%2) % 4 of word q/2 of this half's eight
            const std::uint32_t pair = sub_scales[q >> 1] >> (16 * (q & 1));
            const int value = static_cast<std::int8_t>((pair >> within) & 0xffu);
            scale[q] = splat(d * static_cast<float>(value));
        }
    }
    __device__ __forceinline__ static int lane_group(int j) { return 16 * (j >> 1) + 2 * (j & 1); }
    static constexpr int step_group(int m) { return 4 * (m >> 1) + (m & 1); }
    template <int M>
    __device__ __forceinline__ f16x8 operand() const {
        constexpr int kQuarter = M >> 1, kWord = 2 * (M & 1);
        std::uint32_t out[4];
#pragma unroll
        for (int w = 0; w < 2; ++w) {
            const std::uint32_t low = (kQuarter & 1) ? low_b[kWord + w] : low_a[kWord + w];
            const std::uint32_t nibbles = (kQuarter >= 2 ? low >> 4 : low) & 0x0f0f0f0fu;
            const std::uint32_t bits = top[kWord + w];
            const std::uint32_t upper =
                (kQuarter < 2 ? bits << (4 - 2 * kQuarter) : bits >> (2 * kQuarter - 4)) & 0x30303030u;
            // bias: 1024 + the format's offset of 32
            scale_bytes(nibbles | upper, splat(-1056.0f), scale[kQuarter], splat(0.0f), out[2 * w],
                        out[2 * w + 1]);
        }
        return as_operand(out[0], out[1], out[2], out[3]);
    }
};

// Q8_0: eight 34-byte blocks (fp16 scale, 32 int8 codes) per 256 values.  Quarter j takes
// blocks 2j and 2j + 1; instruction M uses codes 8*(M%4)..+7 of block 2j + M/4.
template <>
struct PackedBlock<kEncQ8_0> {
    static constexpr int kBytes = 272;
    static constexpr bool kQuadFetch = false;
    __device__ __forceinline__ void change_lanes(int) {}
    __device__ __forceinline__ void load_tile(const std::uint8_t* at, int j) {
        const std::uint8_t* mine = at + 68 * j;
        std::uint32_t word[17];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const u32x4 four = tile_read16(mine + 16 * q);
            word[4 * q] = four[0];
            word[4 * q + 1] = four[1];
            word[4 * q + 2] = four[2];
            word[4 * q + 3] = four[3];
        }
        word[16] = reinterpret_cast<const TilePiece4*>(mine + 64)->v;
        take(word);
    }
    std::uint32_t codes[2][8];
    std::uint32_t d_bits[2];
    f16x2 scale[2];
    __device__ __forceinline__ void load(GlobalBytes block, std::uint32_t row, int j) {
        // The quarter's two blocks are 68 bytes = 17 aligned words: the first block's codes
        // start in the middle of word 0 and are shifted into place, the second block's
        // scale is the upper half of word 8 and its codes are words 9..16.
        typedef const __attribute__((address_space(1))) std::uint32_t* GlobalWord;
        const std::uint32_t mine = row + 68 * j;
        std::uint32_t word[17];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const u32x4 four = *reinterpret_cast<GlobalVec>(block + (mine + 16 * q));
            word[4 * q] = four[0];
            word[4 * q + 1] = four[1];
            word[4 * q + 2] = four[2];
            word[4 * q + 3] = four[3];
        }
        word[16] = *reinterpret_cast<GlobalWord>(block + (mine + 64));
        take(word);
    }
    __device__ __forceinline__ void take(const std::uint32_t (&word)[17]) {
        d_bits[0] = word[0] & 0xffffu;
        d_bits[1] = word[8] >> 16;
#pragma unroll
        for (int w = 0; w < 8; ++w) {
            codes[0][w] = __builtin_amdgcn_alignbit(word[w + 1], word[w], 16);
            codes[1][w] = word[9 + w];
        }
    }
    __device__ __forceinline__ void prepare(int) {
#pragma unroll
        for (int b = 0; b < 2; ++b) {
            const _Float16 d = __builtin_bit_cast(_Float16, static_cast<std::uint16_t>(d_bits[b]));
            scale[b] = f16x2{d, d};
        }
    }
    __device__ __forceinline__ static int lane_group(int j) { return 8 * j; }
    static constexpr int step_group(int m) { return m; }
    template <int M>
    __device__ __forceinline__ f16x8 operand() const {
        constexpr int kBlock = M >> 2, kWord = 2 * (M & 3);
        std::uint32_t out[4];
        // flipping the sign bit turns the int8 code q into the byte q + 128: bias 1024 + 128
        scale_bytes(codes[kBlock][kWord] ^ 0x80808080u, splat(-1152.0f), scale[kBlock], splat(0.0f),
                    out[0], out[1]);
        scale_bytes(codes[kBlock][kWord + 1] ^ 0x80808080u, splat(-1152.0f), scale[kBlock],
                    splat(0.0f), out[2], out[3]);
        return as_operand(out[0], out[1], out[2], out[3]);
    }
};

// Projection a tile belongs to.
__device__ __forceinline__ Projection tile_projection(const ProjectionSet& set, std::uint32_t tile) {
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && tile >= set.op[index].first_tile) which = index;
    }
    return pick(set, which);
}

constexpr int kGroupTiles = 2;  // tiles a workgroup accumulates side by side

// A workgroup takes its tiles in groups of up to kGroupTiles and K in chunks of
// 8 x kDepth blocks.  Per (group, chunk) a wave loads the activation fragments
// of its share of the chunk (at most kDepth blocks) once, into registers, and
// walks the group's tiles: step s of every tile uses fragment set s and stage
// s, so only packed weights stream, kDepth steps (one tile) ahead.  Rows of up
// to 8,192 columns are one chunk: the fragments are loaded once per launch.
// After the last chunk the eight waves' partial sums of the group meet in LDS.
//
// kArgmax (the lm_head, one projection): instead of storing the results, the wave that adds up
// a tile keeps for each of its (row of the tile, token) pairs the best result over the
// workgroup's tiles, and at the end writes one (value, row) candidate per token:
// `candidates` is [tokens][kGroupTiles x workgroups].  Ties keep the lower row and NaN never
// wins, as in the row argmax (neuralfn/csrc/tile_cuda/kernels.cu:1564-1602).
//
// kPairs (gate and up of an FFN, two projections of one shape): a group is tile T of the first
// projection beside tile T of the second, and the wave that adds up the first adds up both and
// stores swiglu(first, second), the value the SwiGLU prologue of the projection behind would
// compute from the two outputs: one [rows, output_dim] result instead of two.
enum Mode : int { kStore = 0, kArgmax = 1, kPairs = 2 };

// RING: how the packed weights reach the lanes.  In the plain form every lane loads the bytes
// it decodes, 16 rows x (a quarter of) one block per instruction: a wave instruction touches
// 16 to 32 cache lines for 1 KB, and the launch is bound by the rate at which the vector
// cache looks lines up (the Q6_K lm_head read this way and nothing else: 4.05 TB/s).  In the
// RING form a load instruction brings whole blocks of several rows, every row's block as
// neighbouring 16-byte pieces (5.4 to 5.7 TB/s for the same bytes), and brings them straight
// into LDS (global_load_lds_dwordx4: lane l's 16 bytes land at the instruction's LDS address
// + 16 l; the source may start at any byte), into a ring of block steps that belongs to the
// wave alone; no register waits for a load.  Every lane then reads its row's pieces from
// LDS, where two-byte alignment costs nothing.  The arithmetic and its order are those of
// the plain form.
template <std::uint32_t ENC>
struct Ring {
    static constexpr int kBytes = PackedBlock<ENC>::kBytes;
    static constexpr int kRowLanes = (kBytes + 15) / 16;  // 16-byte pieces of a row's block
    static constexpr int kRowPitch = 16 * kRowLanes;      // a row's place in a stage
    // bytes a row's last piece reaches past its block (Q6_K: 14): the last piece of a
    // projection's very last block is not loaded this way
    static constexpr int kOver = kRowPitch - kBytes;
    static constexpr int kRowsPerLoad = kWave / kRowLanes;
    static constexpr int kLoads = (kTileRows + kRowsPerLoad - 1) / kRowsPerLoad;  // per block step
    static constexpr int kStageBytes = kTileRows * kRowPitch;
    // as many stages as fit beside the kernel's other LDS (36 KB) in the 160 KB of a unit
    // (a fifth Q6_K stage in place of the second buffer of partial sums, which costs a second
    // barrier per group: the lm_head at 16 rows 227 -> 236 us)
    static constexpr int kFit = 120 * 1024 / (kWaves * kStageBytes);
    static constexpr int kStages = kFit < 6 ? kFit : 6;
    static constexpr unsigned kLdsBytes = kWaves * kStages * kStageBytes;
};

// A tile of 16 weight rows as both the fetching and the multiplying side see it (uniform).
struct TileShape {
    const __attribute__((address_space(1))) std::uint8_t* base;  // its first row
    std::uint32_t stride;  // bytes between rows
    int last;              // last row that exists
    int final_row;         // the projection's last row if it is one of the tile's, else -1
};

template <std::uint32_t ENC, int MODE, bool RING>
__global__ __launch_bounds__(kThreads) void gemv_f16_kernel(
    const std::uint8_t* __restrict__ image, const float* __restrict__ inverse_scale, int tokens,
    std::uint32_t total_tiles, int input_dim, LmHeadCandidate* __restrict__ candidates,
    ProjectionSet set) {
    using Block = PackedBlock<ENC>;
    using Lds = Ring<ENC>;
    constexpr bool ARGMAX = MODE == kArgmax;
    constexpr bool PAIRS = MODE == kPairs;
    __shared__ float partial[2 * kGroupTiles * kWaves * kWave * 4];
    extern __shared__ __attribute__((aligned(16))) std::uint8_t ring_lds[];  // RING: [wave][stage][row][kRowPitch]

    const int lane = threadIdx.x & 63;
    // the wave index is uniform; saying so keeps tile bookkeeping in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15;
    const int j = lane >> 4;
    const int blocks = input_dim >> 8;
    // K is cut into kWaves shares of blocks * share / kWaves .. blocks * (share + 1) / kWaves;
    // which wave takes which share is free (sums meet in share order).  Waves w and w + 4 run
    // on one SIMD, and with this choice the shares that are one block longer than the others
    // spread over the four SIMDs for every remainder of blocks / 8 (26 blocks: shares 3 and 7;
    // the Q6_K lm_head 250 -> 238 us, Q4_K gate and up at 16 rows 38.4 -> 37.6 us).
    const int share = (0x63571240 >> (4 * wave)) & 7;
    const int begin = blocks * share / kWaves;
    const int end = blocks * (share + 1) / kWaves;
    const int count = end - begin;
    const int chunks = ((blocks + kWaves - 1) / kWaves + kDepth - 1) / kDepth;  // the same for every wave

    // The 16 bytes of group g of eight columns for token i: image + (g * tokens + i) * 16, as
    // a uniform part (block and instruction) and this lane's part (its quarter and token).
    // Lanes past the last token read token 0 again: a row of A only reaches its own row of
    // the result, and those rows are never stored.
    const GlobalBytes global_image = (GlobalBytes)image;
    const std::uint32_t group_bytes = static_cast<std::uint32_t>(tokens) * 16;
    const std::uint32_t lane_fragment =
        static_cast<std::uint32_t>(Block::lane_group(j)) * group_bytes + (i < tokens ? i : 0) * 16;
    f16x8 fragments[kDepth][8];
    auto load_fragments = [&](int chunk) {
#pragma unroll
        for (int s = 0; s < kDepth; ++s) {
            const int block = begin + max(min(chunk * kDepth + s, count - 1), 0);
            const GlobalBytes block_image = global_image + static_cast<std::int64_t>(block) * 32 * group_bytes;
#pragma unroll
            for (int m = 0; m < 8; ++m) {
                fragments[s][m] = *reinterpret_cast<GlobalFragment>(
                    block_image + Block::step_group(m) * group_bytes + lane_fragment);
            }
        }
    };

    // register r of quarter j of the result: token 4j + r; what this wave's sums of that token
    // are multiplied back by (the scale of the token's share of K that the wave has)
    f32x4 token_scale;
#pragma unroll
    for (int r = 0; r < 4; ++r) token_scale[r] = inverse_scale[min(4 * j + r, tokens - 1) * kWaves + share];

    // this workgroup's tiles: blockIdx.x + n * gridDim.x
    const int tile_count =
        static_cast<int>((total_tiles - blockIdx.x + gridDim.x - 1) / gridDim.x);
    // (kPairs: total_tiles counts the tiles of one projection and a group is one of them twice)
    const int groups = PAIRS ? tile_count : (tile_count + kGroupTiles - 1) / kGroupTiles;
    auto tiles_of_group = [&](int group) {
        return PAIRS ? kGroupTiles : min(kGroupTiles, tile_count - group * kGroupTiles);
    };
    // tile `slot` of group `group` (both exist)
    auto tile_shape = [&](int group, int slot) {
        const int index = PAIRS ? group : group * kGroupTiles + slot;
        const std::uint32_t tile = blockIdx.x + static_cast<std::uint32_t>(index) * gridDim.x;
        const Projection op = PAIRS ? pick(set, slot) : tile_projection(set, tile);
        const std::int64_t row0 = static_cast<std::int64_t>(tile - (PAIRS ? 0u : op.first_tile)) * kTileRows;
        TileShape shape;
        shape.last = static_cast<int>(min(static_cast<std::int64_t>(kTileRows - 1), op.output_dim - 1 - row0));
        shape.base = (GlobalBytes)op.data + row0 * op.row_stride;
        shape.stride = static_cast<std::uint32_t>(op.row_stride);
        shape.final_row = row0 + shape.last == op.output_dim - 1 ? shape.last : -1;
        return shape;
    };

    // Every wave walks the same stream of (group, chunk, tile of the group, step)
    // in uniform control flow (a group's tiles: kGroupTiles, fewer in the last group).
    //
    // Plain form: weight loads run kDepth steps ahead; they are
    // unconditional (a step without work reads the first bytes of the first
    // projection, one line for the whole wave), so a step waits for nothing but
    // its own.  The fetch cursor walks the same stream, one tile ahead.
    // kQuadFetch: lane l asks for quarter l % 4 of row l / 4, so that the four lanes of a quad
    // read neighbouring bytes of one row; the matrix instruction wants quarter l / 16 of row
    // l % 16 in lane l, and a step's registers change lanes before use (Q6_K at 16 rows,
    // 6,656 -> 202,048: 299 -> 234 us; the formats with aligned blocks lose 3-7 % to it).
    constexpr bool QUADS = Block::kQuadFetch && !RING;
    const int load_row = QUADS ? lane >> 2 : i;
    const int load_quarter = QUADS ? lane & 3 : j;
    const int taken_from = 4 * (4 * i + j);  // the lane that fetched this lane's row and quarter, x 4
    int fetch_group = 0, fetch_chunk = 0, fetch_slot = 0;
    GlobalBytes fetch_tile = nullptr;  // first row of the tile being fetched (uniform)
    std::uint32_t fetch_row = 0;       // this lane's row of it, in bytes
    bool fetch_live = true;
    auto fetch_setup = [&]() {
        const int index = PAIRS ? fetch_group : fetch_group * kGroupTiles + fetch_slot;
        fetch_live = fetch_group < groups && index < tile_count;
        const TileShape shape = fetch_live ? tile_shape(fetch_group, fetch_slot) : tile_shape(0, 0);
        fetch_tile = shape.base;
        fetch_row = static_cast<std::uint32_t>(min(load_row, shape.last)) * shape.stride;  // rows past the end repeat the last one
    };
    auto fetch_advance = [&]() {  // to the next (group, chunk, tile of the group)
        if (++fetch_slot >= (PAIRS ? kGroupTiles : min(kGroupTiles, tile_count - fetch_group * kGroupTiles))) {
            fetch_slot = 0;
            if (++fetch_chunk == chunks) {
                fetch_chunk = 0;
                ++fetch_group;
            }
        }
        fetch_setup();
    };
    auto fetch = [&](PackedBlock<ENC>& stage, int s) {
        const int local = fetch_chunk * kDepth + s;  // block of this wave's K range
        const bool work = fetch_live && local < count;
        const GlobalBytes source = work
            ? fetch_tile + static_cast<std::int64_t>(begin + local) * Block::kBytes : (GlobalBytes)set.op[0].data;
        stage.load(source, work ? fetch_row : 0u, work ? load_quarter : 0);
    };
    PackedBlock<ENC> stages[RING ? 1 : kDepth];

    // RING form: a cursor over the steps that have work runs kStages - 1 of them ahead.  A
    // step's kLoads instructions each bring the block of kRowsPerLoad rows; lane l of one has
    // piece l % kRowLanes of row l / kRowLanes.  Past the last step the cursor keeps issuing
    // (the first 16 bytes of the first projection), so that the count of loads in flight that
    // a step waits by stays what it is.  What a step needs is kept ready: a pointer that moves
    // on by a block, and every lane's offsets from it, which change with the tile only.
    std::uint8_t* const my_ring = ring_lds + wave * (Lds::kStages * Lds::kStageBytes);
    const int piece_row = lane / Lds::kRowLanes;
    const int piece = lane - piece_row * Lds::kRowLanes;
    int ring_group = 0, ring_chunk = 0, ring_slot = -1;
    int ring_step = 0, ring_steps = 0;  // of the cursor's (tile, chunk)
    int ring_final_step = -1;           // the step that is the projection's very last block, if one is
    int ring_last = 0, ring_final_row = -1;
    std::uint32_t ring_stride = 0;
    int ring_stage = 0;                 // where the next step lands
    GlobalBytes ring_ptr = (GlobalBytes)set.op[0].data;  // row 0 of the tile, the step's block
    std::uint32_t ring_bump = 0;                         // what a step moves it by
    std::uint32_t ring_offset[Lds::kLoads];              // this lane's piece in each instruction
    auto ring_enter = [&]() {  // the next (tile, chunk) in which this wave has steps
        for (;;) {
            if (++ring_slot >= tiles_of_group(ring_group)) {
                ring_slot = 0;
                if (++ring_chunk == chunks) {
                    ring_chunk = 0;
                    ++ring_group;
                }
            }
            if (ring_group >= groups) {  // done: the same 16 bytes from now on
                ring_ptr = (GlobalBytes)set.op[0].data;
                ring_bump = 0;
                ring_step = 0;
                ring_steps = 0x7fffffff;
                ring_final_step = -1;
#pragma unroll
                for (int q = 0; q < Lds::kLoads; ++q) ring_offset[q] = 0;
                return;
            }
            ring_steps = min(kDepth, count - ring_chunk * kDepth);
            if (ring_steps > 0) break;
        }
        const TileShape shape = tile_shape(ring_group, ring_slot);
        const int first = begin + ring_chunk * kDepth;
        ring_ptr = shape.base + static_cast<std::int64_t>(first) * Block::kBytes;
        ring_bump = Block::kBytes;
        ring_step = 0;
        ring_last = shape.last;
        ring_final_row = shape.final_row;
        ring_stride = shape.stride;
        ring_final_step =
            Lds::kOver > 0 && shape.final_row >= 0 && first + ring_steps == blocks ? ring_steps - 1 : -1;
#pragma unroll
        for (int q = 0; q < Lds::kLoads; ++q) {
            const int row = q * Lds::kRowsPerLoad + piece_row;  // (rows past the end repeat the last one)
            ring_offset[q] = static_cast<std::uint32_t>(min(row, shape.last)) * shape.stride + 16u * piece;
        }
    };
    auto ring_issue = [&]() {
        // the reads of the step that lay in this stage have returned
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        std::uint8_t* const stage = my_ring + ring_stage * Lds::kStageBytes;
        ring_stage = ring_stage + 1 == Lds::kStages ? 0 : ring_stage + 1;
        if (ring_step != ring_final_step) {
#pragma unroll
            for (int q = 0; q < Lds::kLoads; ++q) {
                // the lanes of instruction q that have a row of the tile
                const int rows = min(kTileRows - q * Lds::kRowsPerLoad, Lds::kRowsPerLoad);  // (a constant)
                if (lane < rows * Lds::kRowLanes) {
                    load_to_lds(ring_ptr + ring_offset[q], stage + q * Lds::kRowsPerLoad * Lds::kRowPitch);
                }
            }
        } else if constexpr (Lds::kOver > 0) {
            // The projection's very last block: its last piece would reach past the projection.
            // The lanes that have it stand back, and the bytes of it that exist go by hand
            // (into every row that repeats the final one).
            static_assert(Lds::kOver == 14 || Lds::kOver == 0, "the last piece holds two bytes of the block");
#pragma unroll
            for (int q = 0; q < Lds::kLoads; ++q) {
                const int row = q * Lds::kRowsPerLoad + piece_row;
                const bool past = min(row, ring_last) == ring_final_row && piece == Lds::kRowLanes - 1;
                if (piece_row < Lds::kRowsPerLoad && row < kTileRows && !past) {
                    load_to_lds(ring_ptr + ring_offset[q], stage + q * Lds::kRowsPerLoad * Lds::kRowPitch);
                }
            }
            typedef const __attribute__((address_space(1))) std::uint16_t* GlobalHalf;
            if (lane < kTileRows && min(lane, ring_last) == ring_final_row) {
                const std::uint16_t two = *reinterpret_cast<GlobalHalf>(
                    ring_ptr + (static_cast<std::uint32_t>(ring_final_row) * ring_stride + Block::kBytes - 2));
                *reinterpret_cast<std::uint16_t*>(stage + lane * Lds::kRowPitch + Block::kBytes - 2) = two;
            }
        }
        ring_ptr += ring_bump;
        if (++ring_step == ring_steps) ring_enter();
    };
    int read_stage = 0;  // where the next step to multiply waits

    // RING: the step behind the one being multiplied, read from its stage while that one's
    // matrix instructions run
    PackedBlock<ENC> ahead;
    auto ring_read_ahead = [&]() {
        // all but the loads of the kStages - 1 steps behind the next one have landed
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(Lds::kLoads * (Lds::kStages - 1)) : "memory");
        ahead.load_tile(my_ring + read_stage * Lds::kStageBytes + i * Lds::kRowPitch, j);
        read_stage = read_stage + 1 == Lds::kStages ? 0 : read_stage + 1;
    };
    // RING, rows of one chunk: the launch's only fragments are requested with the first weights,
    // not behind the wait for them
    const bool fragments_first = RING && chunks == 1;
    if constexpr (RING) {
        ring_enter();
        // (ahead of the weights, so that the first step's wait by count covers them)
        if (fragments_first) load_fragments(0);
#pragma unroll
        for (int s = 0; s < Lds::kStages; ++s) ring_issue();
        ring_read_ahead();
    } else {
        fetch_setup();
#pragma unroll
        for (int s = 0; s < kDepth; ++s) fetch(stages[s], s);
        fetch_advance();
    }

    // ARGMAX: the running best of every (lane, result register) of the waves that add up tiles
    // lives in LDS between tiles, so that the main loop holds no register for it
    __shared__ f32x4 best_values[ARGMAX ? kGroupTiles * kWave : 1];
    __shared__ i32x4 best_rows[ARGMAX ? kGroupTiles * kWave : 1];
    if constexpr (ARGMAX) {
        if (wave < kGroupTiles) {
            best_values[wave * kWave + lane] = f32x4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
            best_rows[wave * kWave + lane] = i32x4{0, 0, 0, 0};
        }
    }

    for (int group = 0; group < groups; ++group) {
        f32x4 acc[kGroupTiles];
#pragma unroll
        for (int t = 0; t < kGroupTiles; ++t) acc[t] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
        const int group_tiles = tiles_of_group(group);
        for (int chunk = 0; chunk < chunks; ++chunk) {
            if (chunks > 1 || (group == 0 && !fragments_first)) load_fragments(chunk);
            const int chunk_count = min(kDepth, count - chunk * kDepth);  // this wave's blocks of the chunk
#pragma unroll
            for (int t = 0; t < kGroupTiles; ++t) {
                if (t >= group_tiles) break;
#pragma unroll
                for (int s = 0; s < kDepth; ++s) {
                    if (RING && s >= chunk_count) break;  // (the plain form fetches in every step)
                    PackedBlock<ENC>& stage = stages[RING ? 0 : s];
                    if (s < chunk_count) {
                        const f16x8 (&a)[8] = fragments[s];
                        if constexpr (RING) {
                            stage = ahead;
                            ring_issue();  // into the stage that `ahead` came from
                        }
                        if constexpr (QUADS) stage.change_lanes(taken_from);
                        stage.prepare(j);
                        f32x4 sum = acc[t];
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[0], stage.template operand<0>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[1], stage.template operand<1>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[2], stage.template operand<2>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[3], stage.template operand<3>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[4], stage.template operand<4>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[5], stage.template operand<5>(), sum, 0, 0, 0);
                        // RING: the next step's registers, as late as its LDS reads still hide
                        // behind this step's last instructions
                        if constexpr (RING) ring_read_ahead();
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[6], stage.template operand<6>(), sum, 0, 0, 0);
                        sum = __builtin_amdgcn_mfma_f32_16x16x32_f16(a[7], stage.template operand<7>(), sum, 0, 0, 0);
                        acc[t] = sum;
                    }
                    if constexpr (!RING) fetch(stage, s);
                }
                if constexpr (!RING) fetch_advance();
            }
        }
        // Cross-wave sums in share order, wave t adds up tile t of the group; the
        // two buffers alternate so one barrier per group is enough.
        float* buffer = partial + (group & 1) * kGroupTiles * kWaves * kWave * 4;
#pragma unroll
        for (int t = 0; t < kGroupTiles; ++t) {
            if (t < group_tiles) {
                *reinterpret_cast<f32x4*>(buffer + ((t * kWaves + share) * kWave + lane) * 4) =
                    acc[t] * token_scale;
            }
        }
        __syncthreads();
        if constexpr (PAIRS) {
            if (wave == 0) {
                const std::uint32_t tile = blockIdx.x + static_cast<std::uint32_t>(group) * gridDim.x;
                const std::int64_t row = static_cast<std::int64_t>(tile) * kTileRows + i;
                f32x4 first = *reinterpret_cast<const f32x4*>(buffer + lane * 4);
                f32x4 second = *reinterpret_cast<const f32x4*>(buffer + (kWaves * kWave + lane) * 4);
#pragma unroll
                for (int w = 1; w < kWaves; ++w) {
                    first += *reinterpret_cast<const f32x4*>(buffer + (w * kWave + lane) * 4);
                    second += *reinterpret_cast<const f32x4*>(buffer + ((kWaves + w) * kWave + lane) * 4);
                }
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int token = 4 * j + r;
                    if (token < tokens && row < set.op[0].output_dim) {
                        set.op[0].output[static_cast<std::int64_t>(token) * set.op[0].output_dim + row] =
                            apply_prologue<kSwiGlu>(first[r], second[r]);
                    }
                }
            }
            continue;
        }
        if (wave < group_tiles) {
            const float* mine = buffer + wave * kWaves * kWave * 4;
            const std::uint32_t tile =
                blockIdx.x + static_cast<std::uint32_t>(group * kGroupTiles + wave) * gridDim.x;
            const Projection op = tile_projection(set, tile);
            const std::int64_t row = static_cast<std::int64_t>(tile - op.first_tile) * kTileRows + i;
            f32x4 sum = *reinterpret_cast<const f32x4*>(mine + lane * 4);
#pragma unroll
            for (int w = 1; w < kWaves; ++w) {
                sum += *reinterpret_cast<const f32x4*>(mine + (w * kWave + lane) * 4);
            }
            if constexpr (ARGMAX) {
                f32x4 best_value = best_values[wave * kWave + lane];
                i32x4 best_row = best_rows[wave * kWave + lane];
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const float result = sum[r];
                    // rows past the end and NaN results stand back; a later tile's rows are
                    // higher, so that an equal result does not replace an earlier one
                    const bool wins = row < op.output_dim && result > best_value[r];
                    best_value[r] = wins ? result : best_value[r];
                    best_row[r] = wins ? static_cast<int>(row) : best_row[r];
                }
                best_values[wave * kWave + lane] = best_value;
                best_rows[wave * kWave + lane] = best_row;
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int token = 4 * j + r;
                    if (token < tokens && row < op.output_dim) {
                        op.output[static_cast<std::int64_t>(token) * op.output_dim + row] = sum[r];
                    }
                }
            }
        }
    }
    // RING: the loads issued past the last step still write this workgroup's LDS
    if constexpr (RING) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if constexpr (ARGMAX) {
        if (wave < kGroupTiles) {  // the waves that added up tiles
            const f32x4 mine_value = best_values[wave * kWave + lane];
            const i32x4 mine_row = best_rows[wave * kWave + lane];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float best_value = mine_value[r];
                std::int64_t best_row = mine_row[r];
                // over the 16 rows of a tile: the lanes of a quarter
#pragma unroll
                for (int offset = 8; offset > 0; offset >>= 1) {
                    const float other_value = __shfl_xor(best_value, offset, 64);
                    const std::int64_t other_row = __shfl_xor(best_row, offset, 64);
                    better(other_value, other_row, best_value, best_row);
                }
                const int token = 4 * j + r;
                if (i == 0 && token < tokens) {
                    LmHeadCandidate candidate;
                    candidate.index = best_row;
                    candidate.value = best_value;
                    candidate.pad = 0;
                    candidates[static_cast<std::int64_t>(token) * (kGroupTiles * gridDim.x) +
                               kGroupTiles * blockIdx.x + wave] = candidate;
                }
            }
        }
    }
}

constexpr std::uint32_t kMaxArgmaxGroups = 512;  // workgroups of an lm_head launch at most

// Workgroups of a launch over `tiles` tiles: one per compute unit (persistent), fewer when
// there are fewer tiles.
std::uint32_t grid_of(std::uint32_t tiles, bool argmax) {
    std::uint32_t slots = static_cast<std::uint32_t>(compute_units());
    if (argmax && slots > kMaxArgmaxGroups) slots = kMaxArgmaxGroups;
    return tiles < slots ? tiles : slots;
}

// Which form a launch takes (16 rows, graph replay, plain -> RING in us):
//   Q8_0 6,656 -> 16,384: 34.3 -> 32.9, -> 65,536: 120.7 -> 98.3, 16,384 -> 6,656: 40.4 -> 35.6;
//   Q6_K 6,656 -> 65,536: 93.4 -> 86.4, 2,048 -> 16,384: 22.6 -> 20.6, the lm_head 245 -> 227,
//        but 16,384 -> 6,656: 35.0 -> 35.9 (its fragments are loaded per group there);
//   Q4_K 6,656 -> 16,384: 27.8 -> 30.2, Q5_K: 31.0 -> 33.7 (fewer bytes for the same
//        arithmetic: the extra instructions of a RING step cost more than its loads save).
template <std::uint32_t ENC>
bool ring_form(const ProjectionSet& set) {
    if (ENC == kEncQ8_0) return true;
    if (ENC == kEncQ6K) return set.input_dim <= 32 * 256;
    return false;
}

// `candidates` non-null: the lm_head form (one projection), which returns its workgroup count.
template <std::uint32_t ENC>
std::uint32_t launch_encoding(ProjectionSet set, const std::uint8_t* image, const float* inverse_scale,
                              int tokens, LmHeadCandidate* candidates, hipStream_t stream) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = tiles;
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kTileRows - 1) / kTileRows);
    }
    const std::uint32_t grid = grid_of(tiles, candidates != nullptr);
    if (ring_form<ENC>(set)) {
        constexpr unsigned kLds = Ring<ENC>::kLdsBytes;
        if (candidates != nullptr) {
            allow_large_lds<gemv_f16_kernel<ENC, kArgmax, true>>(kLds);  // (beside 36 KB of static LDS)
            hipLaunchKernelGGL((gemv_f16_kernel<ENC, kArgmax, true>), dim3(grid), dim3(kThreads), kLds,
                               stream, image, inverse_scale, tokens, tiles,
                               static_cast<int>(set.input_dim), candidates, set);
        } else {
            allow_large_lds<gemv_f16_kernel<ENC, kStore, true>>(kLds);
            hipLaunchKernelGGL((gemv_f16_kernel<ENC, kStore, true>), dim3(grid), dim3(kThreads), kLds,
                               stream, image, inverse_scale, tokens, tiles,
                               static_cast<int>(set.input_dim), candidates, set);
        }
    } else if (candidates != nullptr) {
        hipLaunchKernelGGL((gemv_f16_kernel<ENC, kArgmax, false>), dim3(grid), dim3(kThreads), 0, stream,
                           image, inverse_scale, tokens, tiles, static_cast<int>(set.input_dim),
                           candidates, set);
    } else {
        hipLaunchKernelGGL((gemv_f16_kernel<ENC, kStore, false>), dim3(grid), dim3(kThreads), 0, stream,
                           image, inverse_scale, tokens, tiles, static_cast<int>(set.input_dim),
                           candidates, set);
    }
    return grid;
}

// The pair form: two projections of one shape and encoding, one result.
template <std::uint32_t ENC>
void launch_pair(const ProjectionSet& set, const std::uint8_t* image, const float* inverse_scale,
                 int tokens, hipStream_t stream) {
    const std::uint32_t tiles =
        static_cast<std::uint32_t>((set.op[0].output_dim + kTileRows - 1) / kTileRows);
    if (ring_form<ENC>(set)) {
        allow_large_lds<gemv_f16_kernel<ENC, kPairs, true>>(Ring<ENC>::kLdsBytes);
        hipLaunchKernelGGL((gemv_f16_kernel<ENC, kPairs, true>), dim3(grid_of(tiles, false)), dim3(kThreads),
                           Ring<ENC>::kLdsBytes, stream, image, inverse_scale, tokens, tiles,
                           static_cast<int>(set.input_dim), static_cast<LmHeadCandidate*>(nullptr), set);
    } else {
        hipLaunchKernelGGL((gemv_f16_kernel<ENC, kPairs, false>), dim3(grid_of(tiles, false)), dim3(kThreads),
                           0, stream, image, inverse_scale, tokens, tiles,
                           static_cast<int>(set.input_dim), static_cast<LmHeadCandidate*>(nullptr), set);
    }
}

std::uint32_t launch_by_encoding(const ProjectionSet& group, std::uint32_t encoding,
                                 const std::uint8_t* image, const float* inverse_scale, int tokens,
                                 LmHeadCandidate* candidates, hipStream_t stream) {
    if (encoding == kEncQ4K) {
        return launch_encoding<kEncQ4K>(group, image, inverse_scale, tokens, candidates, stream);
    } else if (encoding == kEncQ5K) {
        return launch_encoding<kEncQ5K>(group, image, inverse_scale, tokens, candidates, stream);
    } else if (encoding == kEncQ6K) {
        return launch_encoding<kEncQ6K>(group, image, inverse_scale, tokens, candidates, stream);
    }
    return launch_encoding<kEncQ8_0>(group, image, inverse_scale, tokens, candidates, stream);
}

}  // namespace

bool gemv_f16_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K ||
            encoding == kEncQ8_0) &&
        input_dim % 256 == 0 && input_dim <= 65536;
}

std::int64_t gemv_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim) {
    return rows * input_dim * 2 + rows * kWaves * 4;
}

void launch_gemv_f16(const ProjectionSet& set, const float* first, const float* second, int prologue,
                     std::int64_t rows, void* workspace, hipStream_t stream) {
    std::uint8_t* image = static_cast<std::uint8_t*>(workspace);
    float* inverse_scale = reinterpret_cast<float*>(image + rows * set.input_dim * 2);
    const int tokens = static_cast<int>(rows);
    const int input_dim = static_cast<int>(set.input_dim);
    const dim3 grid(static_cast<unsigned>(rows * kWaves));
    switch (prologue) {
        case kHalfImage:  // an earlier launch left the image in the workspace
            break;
        case kGated:
            hipLaunchKernelGGL((f16_image_kernel<kGated>), grid, dim3(kImageThreads), 0, stream, first,
                               second, image, inverse_scale, tokens, input_dim);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((f16_image_kernel<kSwiGlu>), grid, dim3(kImageThreads), 0, stream, first,
                               second, image, inverse_scale, tokens, input_dim);
            break;
        default:
            hipLaunchKernelGGL((f16_image_kernel<kPlain>), grid, dim3(kImageThreads), 0, stream, first,
                               second, image, inverse_scale, tokens, input_dim);
            break;
    }
    // one launch per encoding present
    const std::uint32_t encodings[4] = {kEncQ4K, kEncQ5K, kEncQ6K, kEncQ8_0};
    for (const std::uint32_t encoding : encodings) {
        ProjectionSet group{};
        group.input_dim = set.input_dim;
        for (int index = 0; index < set.count; ++index) {
            if (set.op[index].encoding == encoding) group.op[group.count++] = set.op[index];
        }
        if (group.count == 0) continue;
        launch_by_encoding(group, encoding, image, inverse_scale, tokens, nullptr, stream);
    }
}

bool gemv_f16_pairs_supports(std::uint32_t first_encoding, std::uint32_t second_encoding,
                             std::int64_t input_dim) {
    return first_encoding == second_encoding && gemv_f16_supports(first_encoding, input_dim);
}

void launch_gemv_f16_pairs(const ProjectionSet& set, const float* input, std::int64_t rows,
                           void* workspace, hipStream_t stream) {
    std::uint8_t* image = static_cast<std::uint8_t*>(workspace);
    float* inverse_scale = reinterpret_cast<float*>(image + rows * set.input_dim * 2);
    const int tokens = static_cast<int>(rows);
    if (input != nullptr) {
        hipLaunchKernelGGL((f16_image_kernel<kPlain>), dim3(static_cast<unsigned>(rows * kWaves)),
                           dim3(kImageThreads), 0, stream, input, nullptr, image, inverse_scale, tokens,
                           static_cast<int>(set.input_dim));
    }
    switch (set.op[0].encoding) {
        case kEncQ4K: launch_pair<kEncQ4K>(set, image, inverse_scale, tokens, stream); break;
        case kEncQ5K: launch_pair<kEncQ5K>(set, image, inverse_scale, tokens, stream); break;
        case kEncQ6K: launch_pair<kEncQ6K>(set, image, inverse_scale, tokens, stream); break;
        default: launch_pair<kEncQ8_0>(set, image, inverse_scale, tokens, stream); break;
    }
}

// Workspace of the lm_head form: the fp16 copy and its row scales, then the candidates.
namespace {
std::int64_t lm_head_image_bytes(std::int64_t rows, std::int64_t input_dim) {
    return (rows * input_dim * 2 + rows * kWaves * 4 + 255) & ~std::int64_t(255);
}
}  // namespace

std::int64_t lm_head_f16_workspace_bytes(std::int64_t rows, std::int64_t input_dim) {
    return lm_head_image_bytes(rows, input_dim) +
        rows * kGroupTiles * kMaxArgmaxGroups * static_cast<std::int64_t>(sizeof(LmHeadCandidate));
}

void launch_lm_head_f16(const Descriptor& descriptor, const float* input, std::int64_t rows,
                        void* workspace, std::int64_t* indices, float* maxima, hipStream_t stream) {
    std::uint8_t* image = static_cast<std::uint8_t*>(workspace);
    float* inverse_scale = reinterpret_cast<float*>(image + rows * descriptor.input_dim * 2);
    LmHeadCandidate* candidates =
        reinterpret_cast<LmHeadCandidate*>(image + lm_head_image_bytes(rows, descriptor.input_dim));
    const int tokens = static_cast<int>(rows);
    hipLaunchKernelGGL((f16_image_kernel<kPlain>), dim3(static_cast<unsigned>(rows * kWaves)),
                       dim3(kImageThreads), 0, stream, input, nullptr, image, inverse_scale, tokens,
                       static_cast<int>(descriptor.input_dim));
    ProjectionSet set{};
    set.count = 1;
    set.input_dim = descriptor.input_dim;
    set.op[0].data = descriptor.data;
    set.op[0].output = nullptr;
    set.op[0].output_dim = descriptor.output_dim;
    set.op[0].row_stride = descriptor.row_stride_bytes;
    set.op[0].encoding = descriptor.encoding;
    const std::uint32_t groups =
        launch_by_encoding(set, descriptor.encoding, image, inverse_scale, tokens, candidates, stream);
    launch_lm_head_final(candidates, static_cast<std::int64_t>(kGroupTiles) * groups, indices, maxima,
                         rows, stream);
}

}  // namespace nfn
