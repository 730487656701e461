// Decode / small-batch GEMV on the int8 matrix cores.
//
// One workgroup (4 waves) owns a tile of 16 consecutive weight rows; the waves
// split the K dimension by super-block ranges and meet once, at the end, in a
// fixed-order sum.  Per 256-value super-block a wave
//   1. copies its 16 x block_bytes of packed weights from HBM to a private LDS
//      tile with fully coalesced 16-byte loads (prefetched DEPTH blocks ahead),
//   2. turns the 256 activations of that block into two int8 planes (the high
//      and low byte of a 16-bit fixed-point code, one scale per 32 values) —
//      in this launch for one token, or read from the workspace for 2..8,
//   3. unpacks 4/5/6/8-bit codes to int8 straight from LDS in the operand
//      layout of v_mfma_i32_16x16x32_i8 (weights are the B operand: lane
//      l holds row l%16, k-chunk l/16; the token planes are rows of A),
//   4. scales the int32 dot products of each 32-value sub-block in float.
// Every weight byte is read from HBM exactly once per launch.
//
// Arithmetic it replaces: the reference's one-row and small-batch kernels
// (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:714-890, 1174-1303), which
// quantize activations to 8 bits; here 16 bits are kept so the result stays
// within 2e-3 of the float-activation CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:655-679).
//   y[t][j] = sum_blocks d*sum_sub sc_sub*s[t][sub]*(256*dot(q,hi) + dot(q,lo))
//                        - dmin*sum_sub m_sub*S[t][sub]
// with s the activation scale and S the float sum of the 32 activations.
#include "common.hpp"
#include "gemv_mfma.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kTileRows = 16;
constexpr int kWaves = 4;
constexpr int kThreads = kWaves * kWave;
constexpr float kCodeRange = 32512.0f;  // 127*256: high byte stays in [-127, 127]
constexpr int kActRecord = kActivationRecordBytes;

struct __attribute__((packed, aligned(2))) Chunk16 {
    std::uint32_t v[4];
};

template <std::uint32_t ENC>
struct Format;
template <>
struct Format<kEncQ4K> {
    static constexpr int kBlockBytes = 144;
    static constexpr int kChunks = 9;    // 16-byte chunks copied per block
    static constexpr int kLdsRow = 144;  // (kLdsRow/4) % 64 must be 4*odd: conflict-free reads
    static constexpr bool kAligned = true;
    static constexpr bool kHasMin = true;
};
template <>
struct Format<kEncQ5K> {
    static constexpr int kBlockBytes = 176;
    static constexpr int kChunks = 11;
    static constexpr int kLdsRow = 176;
    static constexpr bool kAligned = true;
    static constexpr bool kHasMin = true;
};
template <>
struct Format<kEncQ6K> {
    static constexpr int kBlockBytes = 210;
    static constexpr int kChunks = 14;  // 224 bytes: the tail reads into the next block
    static constexpr int kLdsRow = 240;
    static constexpr bool kAligned = false;
    static constexpr bool kHasMin = false;
};
template <>
struct Format<kEncQ8_0> {
    static constexpr int kBlockBytes = 272;  // eight 34-byte blocks
    static constexpr int kChunks = 17;
    static constexpr int kLdsRow = 272;
    static constexpr bool kAligned = false;
    static constexpr bool kHasMin = false;
};

constexpr int kMaxLdsTile = kTileRows * 272;

template <int CTRL>
__device__ __forceinline__ float dpp_move(float value) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, value), CTRL, 0xF, 0xF, true));
}

// Reductions over the 8 lanes that share one 32-value group: quad xor 1, quad
// xor 2, then the mirrored half row (lane k <-> 7-k) brings in the other quad.
__device__ __forceinline__ float group8_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));
    v = fmaxf(v, dpp_move<0x4E>(v));
    v = fmaxf(v, dpp_move<0x141>(v));
    return v;
}
__device__ __forceinline__ float group8_sum(float v) {
    v += dpp_move<0xB1>(v);
    v += dpp_move<0x4E>(v);
    v += dpp_move<0x141>(v);
    return v;
}

__device__ __forceinline__ std::uint32_t perm(std::uint32_t hi, std::uint32_t lo, std::uint32_t sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

// Quantize four consecutive activations held by this lane; the 8 lanes of a
// 32-value group agree on one scale.  Returns the packed high and low planes.
struct QuantizedQuad {
    std::uint32_t hi;
    std::uint32_t lo;
    float scale;  // activation = scale * (256*hi + lo)
    float sum;    // float sum of the 32 inputs of the group
    int isum;     // sum over the group of (256*hi + lo), for formats with an offset code
};

__device__ __forceinline__ QuantizedQuad quantize_quad(float x0, float x1, float x2, float x3) {
    QuantizedQuad q;
    const float local = fmaxf(fmaxf(fabsf(x0), fabsf(x1)), fmaxf(fabsf(x2), fabsf(x3)));
    const float maximum = group8_max(local);
    q.sum = group8_sum((x0 + x1) + (x2 + x3));
    const float inverse = maximum > 0.0f ? kCodeRange / maximum : 0.0f;
    q.scale = maximum * (1.0f / kCodeRange);
    // 1.5*2^23 + 128: the low 16 bits of the sum's bit pattern are
    // round-to-nearest-even(x*inverse) + 128 in two's complement.
    constexpr float kMagic = 12582912.0f + 128.0f;
    const std::uint32_t u0 = __float_as_uint(fmaf(x0, inverse, kMagic));
    const std::uint32_t u1 = __float_as_uint(fmaf(x1, inverse, kMagic));
    const std::uint32_t u2 = __float_as_uint(fmaf(x2, inverse, kMagic));
    const std::uint32_t u3 = __float_as_uint(fmaf(x3, inverse, kMagic));
    // code + 128 = 256*hi + (lo + 128): hi is byte 1, lo is byte 0 with its top bit flipped.
    const std::uint32_t p01 = perm(u1, u0, 0x05010400u);  // [u0.b0, u1.b0, u0.b1, u1.b1]
    const std::uint32_t p23 = perm(u3, u2, 0x05010400u);
    q.lo = perm(p23, p01, 0x05040100u) ^ 0x80808080u;
    q.hi = perm(p23, p01, 0x07060302u);
    q.isum = 0;
    return q;
}

struct TileContext {
    Projection op;
    std::int64_t row0;
    int valid_rows;
};

// Per-lane float scale factors of one super-block of this lane's weight row.
template <std::uint32_t ENC>
struct BlockScales;

template <>
struct BlockScales<kEncQ4K> {
    float d, dmin;
    float sc[8];
    float mn[8];
    __device__ __forceinline__ void load(const std::uint8_t* row) {
        const uint4 h = *reinterpret_cast<const uint4*>(row);
        d = half_bits_to_float(h.x & 0xffffu);
        dmin = half_bits_to_float(h.x >> 16);
        const std::uint32_t sc_lo = h.y & 0x3f3f3f3fu;
        const std::uint32_t mn_lo = h.z & 0x3f3f3f3fu;
        const std::uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
        const std::uint32_t mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            sc[i] = static_cast<float>((sc_lo >> (8 * i)) & 0xffu);
            mn[i] = static_cast<float>((mn_lo >> (8 * i)) & 0xffu);
            sc[4 + i] = static_cast<float>((sc_hi >> (8 * i)) & 0xffu);
            mn[4 + i] = static_cast<float>((mn_hi >> (8 * i)) & 0xffu);
        }
    }
};
template <>
struct BlockScales<kEncQ5K> : BlockScales<kEncQ4K> {};

__device__ __forceinline__ long pack_long(std::uint32_t lo, std::uint32_t hi) {
    return static_cast<long>((static_cast<unsigned long>(hi) << 32) | lo);
}

// Where one lane finds the activation planes and scales of (token, super-block).
struct ActSource {
    const std::uint8_t* planes;  // hi plane at +0, lo plane at +256
    const float* scales;         // 8 scales then 8 sums
};

// Process one super-block: 8 sub-block MFMAs and their float post-scaling.
// `tile` is this wave's LDS copy of the 16 rows of the block.
template <std::uint32_t ENC, int TPG, typename ActFn>
__device__ __forceinline__ void process_block(const std::uint8_t* tile, int j, int kq,
                                              ActFn&& activation, float (&acc)[TPG]);

template <int TPG, bool Q5, typename ActFn>
__device__ __forceinline__ void process_block_q45(const std::uint8_t* tile, int j, int kq,
                                                  ActFn&& activation, float (&acc)[TPG]) {
    constexpr int kRow = Q5 ? 176 : 144;
    const std::uint8_t* row = tile + j * kRow;
    BlockScales<kEncQ4K> scales;
    scales.load(row);
    std::uint32_t high0 = 0, high1 = 0;
    if constexpr (Q5) {
        const uint2 h = *reinterpret_cast<const uint2*>(row + 16 + kq * 8);
        high0 = h.x;
        high1 = h.y;
    }
    const std::uint8_t* quants = row + (Q5 ? 48 : 16) + kq * 8;
    float block_acc[TPG];
    float block_min[TPG];
#pragma unroll
    for (int u = 0; u < TPG; ++u) {
        block_acc[u] = 0.0f;
        block_min[u] = 0.0f;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const uint2 packed = *reinterpret_cast<const uint2*>(quants + g * 32);
        std::uint32_t lo0 = packed.x & 0x0f0f0f0fu;
        std::uint32_t lo1 = packed.y & 0x0f0f0f0fu;
        std::uint32_t hi0 = (packed.x >> 4) & 0x0f0f0f0fu;
        std::uint32_t hi1 = (packed.y >> 4) & 0x0f0f0f0fu;
        if constexpr (Q5) {
            // bit 2g of the high-bit byte belongs to sub-block 2g, bit 2g+1 to 2g+1
            lo0 |= ((high0 >> (2 * g)) & 0x01010101u) << 4;
            lo1 |= ((high1 >> (2 * g)) & 0x01010101u) << 4;
            hi0 |= ((high0 >> (2 * g + 1)) & 0x01010101u) << 4;
            hi1 |= ((high1 >> (2 * g + 1)) & 0x01010101u) << 4;
        }
#pragma unroll
        for (int part = 0; part < 2; ++part) {
            const int sub = 2 * g + part;
            const long b = part == 0 ? pack_long(lo0, lo1) : pack_long(hi0, hi1);
            const long a = activation.operand(sub);
            v4i dot = {0, 0, 0, 0};
            dot = __builtin_amdgcn_mfma_i32_16x16x32_i8(a, b, dot, 0, 0, 0);
#pragma unroll
            for (int u = 0; u < TPG; ++u) {
                const int code = (dot[2 * u] << 8) + dot[2 * u + 1];
                block_acc[u] = fmaf(static_cast<float>(code),
                                    scales.sc[sub] * activation.scale(u, sub), block_acc[u]);
                block_min[u] = fmaf(scales.mn[sub], activation.sum(u, sub), block_min[u]);
            }
        }
    }
#pragma unroll
    for (int u = 0; u < TPG; ++u) {
        acc[u] = fmaf(scales.d, block_acc[u], acc[u]);
        acc[u] = fmaf(-scales.dmin, block_min[u], acc[u]);
    }
}

// Activations quantized by this wave into its own LDS record (one token).
struct FusedActivation {
    const std::uint8_t* record;  // LDS: hi[256] lo[256] scale[8] sum[8]
    int plane_offset;            // which plane this lane feeds to the A operand
    int kq;
    float scales[8];
    float sums[8];
    __device__ __forceinline__ void load_scalars() {
        const float4* p = reinterpret_cast<const float4*>(record + 512);
        const float4 a = p[0], b = p[1], c = p[2], d = p[3];
        scales[0] = a.x; scales[1] = a.y; scales[2] = a.z; scales[3] = a.w;
        scales[4] = b.x; scales[5] = b.y; scales[6] = b.z; scales[7] = b.w;
        sums[0] = c.x; sums[1] = c.y; sums[2] = c.z; sums[3] = c.w;
        sums[4] = d.x; sums[5] = d.y; sums[6] = d.z; sums[7] = d.w;
    }
    __device__ __forceinline__ long operand(int sub) const {
        const uint2 v = *reinterpret_cast<const uint2*>(record + plane_offset + sub * 32 + kq * 8);
        return pack_long(v.x, v.y);
    }
    __device__ __forceinline__ float scale(int, int sub) const { return scales[sub]; }
    __device__ __forceinline__ float sum(int, int sub) const { return sums[sub]; }
};

// Activations quantized earlier into the workspace (2..8 tokens per pass).
template <int TPG>
struct WorkspaceActivation {
    const std::uint8_t* operand_base;  // this lane's plane of its A row, or a valid dummy
    int kq;
    float scales[TPG][8];
    float sums[TPG][8];
    __device__ __forceinline__ void load_scalars(const std::uint8_t* const (&records)[TPG]) {
#pragma unroll
        for (int u = 0; u < TPG; ++u) {
            const float4* p = reinterpret_cast<const float4*>(records[u] + 512);
            const float4 a = p[0], b = p[1], c = p[2], d = p[3];
            scales[u][0] = a.x; scales[u][1] = a.y; scales[u][2] = a.z; scales[u][3] = a.w;
            scales[u][4] = b.x; scales[u][5] = b.y; scales[u][6] = b.z; scales[u][7] = b.w;
            sums[u][0] = c.x; sums[u][1] = c.y; sums[u][2] = c.z; sums[u][3] = c.w;
            sums[u][4] = d.x; sums[u][5] = d.y; sums[u][6] = d.z; sums[u][7] = d.w;
        }
    }
    __device__ __forceinline__ long operand(int sub) const {
        const uint2 v = *reinterpret_cast<const uint2*>(operand_base + sub * 32 + kq * 8);
        return pack_long(v.x, v.y);
    }
    __device__ __forceinline__ float scale(int u, int sub) const { return scales[u][sub]; }
    __device__ __forceinline__ float sum(int u, int sub) const { return sums[u][sub]; }
};

template <std::uint32_t ENC, int TPG, typename Act>
__device__ __forceinline__ void dispatch_block(const std::uint8_t* tile, int j, int kq, Act& act,
                                               float (&acc)[TPG]) {
    if constexpr (ENC == kEncQ4K) {
        process_block_q45<TPG, false>(tile, j, kq, act, acc);
    } else if constexpr (ENC == kEncQ5K) {
        process_block_q45<TPG, true>(tile, j, kq, act, acc);
    }
}

template <std::uint32_t ENC>
__device__ __forceinline__ uint4 load_chunk(const std::uint8_t* p) {
    if constexpr (Format<ENC>::kAligned) {
        return *reinterpret_cast<const uint4*>(p);
    } else {
        const Chunk16 c = *reinterpret_cast<const Chunk16*>(p);
        return make_uint4(c.v[0], c.v[1], c.v[2], c.v[3]);
    }
}

// The whole K loop of one wave for one tile.
template <std::uint32_t ENC, int TPG, bool FUSED, int P, int DEPTH>
__device__ __forceinline__ void run_tile(const TileContext& ctx, std::int64_t input_dim,
                                         const float* __restrict__ first,
                                         const float* __restrict__ second,
                                         const std::uint8_t* __restrict__ workspace,
                                         int tokens, std::uint8_t* wave_tile,
                                         std::uint8_t* wave_record, int lane, int wave,
                                         float (&acc)[TPG]) {
    using F = Format<ENC>;
    constexpr int kTotalChunks = kTileRows * F::kChunks;
    constexpr int kLoads = (kTotalChunks + kWave - 1) / kWave;
    const int j = lane & 15;
    const int kq = lane >> 4;
    const std::int64_t blocks = input_dim >> 8;
    const std::int64_t begin = blocks * wave / kWaves;
    const std::int64_t end = blocks * (wave + 1) / kWaves;

    // Per-lane source pointers and LDS offsets of the chunks this lane copies.
    const std::uint8_t* source[kLoads];
    int target[kLoads];
    const std::uint8_t* data_end = ctx.op.data + ctx.op.output_dim * ctx.op.row_stride;
#pragma unroll
    for (int i = 0; i < kLoads; ++i) {
        const int chunk = i * kWave + lane;
        const int row = chunk / F::kChunks;
        const int col = chunk - row * F::kChunks;
        const int clamped = min(row, ctx.valid_rows - 1);
        source[i] = ctx.op.data + (ctx.row0 + clamped) * ctx.op.row_stride + col * 16;
        target[i] = row * F::kLdsRow + col * 16;
    }
    (void)data_end;

    uint4 staged[DEPTH][kLoads];
    auto fetch = [&](int slot, std::int64_t block) {
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            if (i * kWave + lane < kTotalChunks) {
                const std::uint8_t* p = source[i] + block * F::kBlockBytes;
                if constexpr (!F::kAligned) {
                    // the last chunk of a block reads past it; keep it inside the tensor
                    p = p + 16 <= data_end ? p : data_end - 16;
                }
                staged[slot][i] = load_chunk<ENC>(p);
            }
        }
    };

#pragma unroll
    for (int d = 0; d < DEPTH; ++d) {
        if (begin + d < end) fetch(d, begin + d);
    }

    // Which activation plane this lane supplies as a row of the A operand.
    const int a_group = j >> 2;          // which lane group's tokens
    const int a_slot = (j & 3) >> 1;     // token slot within the group
    const int a_term = j & 1;            // 0: high plane, 1: low plane
    const int a_token = a_group * TPG + (a_slot < TPG ? a_slot : 0);
    const bool a_valid = a_slot < TPG && a_token < tokens;

    for (std::int64_t base = begin; base < end; base += DEPTH) {
#pragma unroll
        for (int d = 0; d < DEPTH; ++d) {
            const std::int64_t block = base + d;
            if (block < end) {
                // (1) staged weights -> private LDS tile
#pragma unroll
                for (int i = 0; i < kLoads; ++i) {
                    if (i * kWave + lane < kTotalChunks) {
                        *reinterpret_cast<uint4*>(wave_tile + target[i]) = staged[d][i];
                    }
                }
                if (block + DEPTH < end) fetch(d, block + DEPTH);

                if constexpr (FUSED) {
                    // (2) quantize this block's 256 activations of the one token
                    const std::int64_t column = block * 256 + lane * 4;
                    float4 x = *reinterpret_cast<const float4*>(first + column);
                    if constexpr (P != kPlain) {
                        const float4 y = *reinterpret_cast<const float4*>(second + column);
                        x.x = apply_prologue<P>(x.x, y.x);
                        x.y = apply_prologue<P>(x.y, y.y);
                        x.z = apply_prologue<P>(x.z, y.z);
                        x.w = apply_prologue<P>(x.w, y.w);
                    }
                    const QuantizedQuad q = quantize_quad(x.x, x.y, x.z, x.w);
                    *reinterpret_cast<std::uint32_t*>(wave_record + lane * 4) = q.hi;
                    *reinterpret_cast<std::uint32_t*>(wave_record + 256 + lane * 4) = q.lo;
                    if ((lane & 7) == 0) {
                        *reinterpret_cast<float*>(wave_record + 512 + (lane >> 3) * 4) = q.scale;
                        *reinterpret_cast<float*>(wave_record + 544 + (lane >> 3) * 4) = q.sum;
                    }
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    FusedActivation act;
                    act.record = wave_record;
                    act.plane_offset = a_term * 256;
                    act.kq = kq;
                    act.load_scalars();
                    dispatch_block<ENC, TPG>(wave_tile, j, kq, act, acc);
                } else {
                    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                    __builtin_amdgcn_wave_barrier();
                    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
                    WorkspaceActivation<TPG> act;
                    const std::uint8_t* records[TPG];
#pragma unroll
                    for (int u = 0; u < TPG; ++u) {
                        const int token = min(kq * TPG + u, tokens - 1);
                        records[u] = workspace + (token * blocks + block) * kActRecord;
                    }
                    const int token = a_valid ? a_token : 0;
                    act.operand_base =
                        workspace + (token * blocks + block) * kActRecord + a_term * 256;
                    act.kq = kq;
                    act.load_scalars(records);
                    dispatch_block<ENC, TPG>(wave_tile, j, kq, act, acc);
                }
                // the next block's LDS writes must not pass this block's reads
                __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
                __builtin_amdgcn_wave_barrier();
            }
        }
    }
}

template <int TPG, bool FUSED, int P, int DEPTH>
__global__ __launch_bounds__(kThreads) void gemv_mfma_kernel(
    ProjectionSet set, const float* __restrict__ first, const float* __restrict__ second,
    const std::uint8_t* __restrict__ workspace, int tokens, int token_stride_tiles) {
    __shared__ __attribute__((aligned(16))) std::uint8_t tiles[kWaves][kMaxLdsTile];
    __shared__ __attribute__((aligned(16))) std::uint8_t records[kWaves][640];
    __shared__ float partial[kWaves][kWave][TPG];

    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const std::uint32_t tile_index = blockIdx.x;
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && tile_index >= set.op[index].first_tile) which = index;
    }
    TileContext ctx;
    ctx.op = set.op[which];
    ctx.row0 = static_cast<std::int64_t>(tile_index - ctx.op.first_tile) * kTileRows;
    ctx.valid_rows =
        static_cast<int>(min(static_cast<std::int64_t>(kTileRows), ctx.op.output_dim - ctx.row0));

    // Passes over the tokens when there are more than one pass can hold.
    const int token0 = blockIdx.y * 4 * TPG;
    const int pass_tokens = min(tokens - token0, 4 * TPG);
    const std::int64_t blocks = set.input_dim >> 8;
    const std::uint8_t* pass_workspace =
        FUSED ? nullptr : workspace + static_cast<std::int64_t>(token0) * blocks * kActRecord;
    const float* pass_first = first;
    const float* pass_second = second;

    float acc[TPG];
#pragma unroll
    for (int u = 0; u < TPG; ++u) acc[u] = 0.0f;

    switch (ctx.op.encoding) {
        case kEncQ4K:
            run_tile<kEncQ4K, TPG, FUSED, P, DEPTH>(ctx, set.input_dim, pass_first, pass_second,
                                                   pass_workspace, pass_tokens, tiles[wave],
                                                   records[wave], lane, wave, acc);
            break;
        case kEncQ5K:
            run_tile<kEncQ5K, TPG, FUSED, P, DEPTH>(ctx, set.input_dim, pass_first, pass_second,
                                                   pass_workspace, pass_tokens, tiles[wave],
                                                   records[wave], lane, wave, acc);
            break;
        default:
            break;
    }

#pragma unroll
    for (int u = 0; u < TPG; ++u) partial[wave][lane][u] = acc[u];
    __syncthreads();
    if (wave == 0) {
        const int j = lane & 15;
        const int kq = lane >> 4;
#pragma unroll
        for (int u = 0; u < TPG; ++u) {
            const int token = kq * TPG + u;
            const float total = ((partial[0][lane][u] + partial[1][lane][u]) +
                                 partial[2][lane][u]) + partial[3][lane][u];
            if (token < pass_tokens && j < ctx.valid_rows) {
                ctx.op.output[static_cast<std::int64_t>(token0 + token) * ctx.op.output_dim +
                              ctx.row0 + j] = total;
            }
        }
    }
    (void)token_stride_tiles;
}

// ---- activation quantizer for the multi-token passes -----------------------

template <int P>
__global__ __launch_bounds__(256) void quantize_activations_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    std::uint8_t* __restrict__ workspace, std::int64_t total_blocks) {
    // one wave per (token, super-block) record
    const int lane = threadIdx.x & 63;
    const std::int64_t record = static_cast<std::int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (record >= total_blocks) return;
    const std::int64_t column = record * 256 + lane * 4;
    float4 x = *reinterpret_cast<const float4*>(first + column);
    if constexpr (P != kPlain) {
        const float4 y = *reinterpret_cast<const float4*>(second + column);
        x.x = apply_prologue<P>(x.x, y.x);
        x.y = apply_prologue<P>(x.y, y.y);
        x.z = apply_prologue<P>(x.z, y.z);
        x.w = apply_prologue<P>(x.w, y.w);
    }
    const QuantizedQuad q = quantize_quad(x.x, x.y, x.z, x.w);
    std::uint8_t* out = workspace + record * kActRecord;
    *reinterpret_cast<std::uint32_t*>(out + lane * 4) = q.hi;
    *reinterpret_cast<std::uint32_t*>(out + 256 + lane * 4) = q.lo;
    if ((lane & 7) == 0) {
        *reinterpret_cast<float*>(out + 512 + (lane >> 3) * 4) = q.scale;
        *reinterpret_cast<float*>(out + 544 + (lane >> 3) * 4) = q.sum;
    }
}

template <int TPG, bool FUSED, int P>
void launch_variant(const ProjectionSet& set, const float* first, const float* second,
                    const std::uint8_t* workspace, int tokens, std::uint32_t tiles, int passes,
                    hipStream_t stream) {
    hipLaunchKernelGGL((gemv_mfma_kernel<TPG, FUSED, P, 4>), dim3(tiles, passes), dim3(kThreads),
                       0, stream, set, first, second, workspace, tokens, 0);
}

}  // namespace

bool gemv_mfma_supports(std::uint32_t encoding) {
    return encoding == kEncQ4K || encoding == kEncQ5K;
}

void launch_gemv_mfma(ProjectionSet set, const float* first, const float* second, int prologue,
                      std::int64_t rows, void* workspace, hipStream_t stream) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = tiles;
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kTileRows - 1) / kTileRows);
    }
    const int tokens = static_cast<int>(rows);
    if (tokens == 1) {
        switch (prologue) {
            case kGated:
                launch_variant<1, true, kGated>(set, first, second, nullptr, 1, tiles, 1, stream);
                break;
            case kSwiGlu:
                launch_variant<1, true, kSwiGlu>(set, first, second, nullptr, 1, tiles, 1, stream);
                break;
            default:
                launch_variant<1, true, kPlain>(set, first, second, nullptr, 1, tiles, 1, stream);
                break;
        }
        return;
    }
    // 2..16 tokens: quantize once into the workspace, then one or two passes.
    const std::int64_t records = rows * (set.input_dim >> 8);
    const dim3 grid(static_cast<unsigned>((records + 3) / 4));
    std::uint8_t* ws = static_cast<std::uint8_t*>(workspace);
    switch (prologue) {
        case kGated:
            hipLaunchKernelGGL((quantize_activations_kernel<kGated>), grid, dim3(256), 0, stream,
                               first, second, ws, records);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((quantize_activations_kernel<kSwiGlu>), grid, dim3(256), 0, stream,
                               first, second, ws, records);
            break;
        default:
            hipLaunchKernelGGL((quantize_activations_kernel<kPlain>), grid, dim3(256), 0, stream,
                               first, second, ws, records);
            break;
    }
    if (tokens <= 4) {
        launch_variant<1, false, kPlain>(set, nullptr, nullptr, ws, tokens, tiles, 1, stream);
    } else {
        launch_variant<2, false, kPlain>(set, nullptr, nullptr, ws, tokens, tiles,
                                         (tokens + 7) / 8, stream);
    }
}

}  // namespace nfn
