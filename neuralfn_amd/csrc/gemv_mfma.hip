// Small-batch (2..16 rows) GEMV on the int8 matrix cores.
//
// A small quantizer launch first turns the activations into two int8 planes
// (high and low byte of a 16-bit fixed-point code, one scale per 256 values)
// in the caller's workspace.  In the main kernel a workgroup of 8 waves owns
// tiles of 32 consecutive weight rows (persistent: it walks tiles blockIdx.x,
// blockIdx.x + gridDim.x, ...).  The waves split the K dimension by
// super-block ranges and meet once per tile in a fixed-order sum.  Per
// 256-value super-block a wave
//   1. stores its 32 x block_bytes of packed weights, loaded with coalesced
//      16-byte accesses several blocks ahead (across tile boundaries), into a
//      private LDS tile,
//   2. unpacks 4/5/6-bit codes to int8 straight from LDS in the operand layout
//      of v_mfma_i32_32x32x32_i8 (weights are the B operand: lane l holds row
//      l%32, k-half l/32; the token planes are rows of A),
//   3. weights the int32 dot products of every sub-block with its integer
//      sub-scale (24-bit multiply-add) and converts to float once per block.
// Every weight byte is read from HBM exactly once per launch.
//
// Arithmetic it replaces: the reference's small-batch kernel
// (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1174-1303), which quantizes
// activations to 8 bits; here 16 bits are kept so the result stays within 2e-3
// of the float-activation CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:655-679).  With x = s*c,
// c = 256*hi + lo the 16-bit code of an activation and s its block scale:
//   Q4_K/Q5_K: y += s*(d*sum_sub sc*dot(q, c) - dmin*sum_sub m*sum(c))
//   Q6_K:      y += s*d*sum_16 sc8*dot(q - 32, c)
#include "common.hpp"
#include "gemv_mfma.hpp"
#include "lm_head.hpp"
#include "wave_rows.hpp"

#include <type_traits>

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

constexpr int kTileRows = 32;
constexpr int kWaves = 8;
constexpr int kThreads = kWaves * kWave;
static_assert(kActRecord == kActivationRecordBytes, "record size is part of the workspace contract");

struct __attribute__((packed, aligned(2))) Chunk16 {
    std::uint32_t v[4];
};

template <std::uint32_t ENC>
struct Format;
template <>
struct Format<kEncQ4K> {
    static constexpr int kBlockBytes = 144;
    static constexpr int kChunks = 9;    // 16-byte chunks copied per block
    static constexpr int kLdsRow = 144;  // (kLdsRow/4) % 64 is 4*odd: conflict-free operand reads
    static constexpr bool kAligned = true;
    static constexpr int kDepth = 4;     // packed blocks in flight per wave
};
template <>
struct Format<kEncQ5K> {
    static constexpr int kBlockBytes = 176;
    static constexpr int kChunks = 11;
    static constexpr int kLdsRow = 176;
    static constexpr bool kAligned = true;
    static constexpr int kDepth = 3;
};
template <>
struct Format<kEncQ6K> {
    static constexpr int kBlockBytes = 210;
    static constexpr int kChunks = 14;  // 224 bytes: the tail reads into the next block
    static constexpr int kLdsRow = 240;
    static constexpr bool kAligned = false;
    static constexpr int kDepth = 3;
};

// Quantize the 256 activations of one block, four per lane, and write the
// record (planes, per-32 code sums, scale) to `record` (LDS or workspace).
__device__ __forceinline__ void quantize_block(float4 x, int lane, std::uint8_t* record) {
    store_record(record, lane, encode_activations(x));
}

// Token <-> operand-row bookkeeping of v_mfma_i32_32x32x32_i8.  Output register
// r of lane l holds row 8*(r/4) + 4*(l/32) + r%4 of column l%32.
//  Q4_K/Q5_K: a token takes two A rows (high, low plane).  Token t = 2u + h sits
//    in registers 2u, 2u+1 of lane half h: up to 16 tokens, S = ceil(tokens/2)
//    register pairs per lane.
//  Q6_K: a 32-wide MFMA spans two 16-value groups with different sub-scales,
//    so a token takes four A rows (high/low x first/second 16) and a lane
//    feeds zeros where its k-half is not the row's: token t = 2q + h sits in
//    registers 4q..4q+3 of lane half h: up to 8 tokens.
template <bool Q6>
struct OperandRow {
    int token;
    int plane;
    bool keep;  // false: this lane's k-half is outside the row, feed zeros
    __device__ __forceinline__ OperandRow(int i, int kc) {
        if constexpr (Q6) {
            const int row4 = i >> 2;
            const int within = i & 3;
            plane = within & 1;
            keep = (within >> 1) == kc;
            token = 2 * (row4 >> 1) + (row4 & 1);
        } else {
            const int pair = i >> 1;
            plane = i & 1;
            keep = true;
            const int u = 2 * (pair >> 2) + (pair & 1);
            const int h = (pair >> 1) & 1;
            token = 2 * u + h;
        }
    }
};

// Activation side of one super-block as one lane sees it.
template <int S>
struct BlockActivation {
    const std::uint8_t* operand_base;  // record + plane offset of this lane's A row
    bool keep;
    int kc;
    float scale[S];
    int sums[S][8];
    __device__ __forceinline__ v4i operand(int sub) const {
        v4i v = *reinterpret_cast<const v4i*>(operand_base + sub * 32 + kc * 16);
        if (!keep) v = v4i{0, 0, 0, 0};
        return v;
    }
};

__device__ __forceinline__ int byte_of(std::uint32_t packed, int index) {
    return static_cast<int>((packed >> (8 * index)) & 0xffu);
}
__device__ __forceinline__ int signed_byte_of(std::uint32_t packed, int index) {
    return static_cast<int>(static_cast<std::int32_t>(packed << (24 - 8 * index)) >> 24);
}

__device__ __forceinline__ v16i mfma32(v4i a, v4i b) {
    const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, zero, 0, 0, 0);
}

// ---- Q4_K / Q5_K ------------------------------------------------------------
template <int S, bool Q5>
__device__ __forceinline__ void process_block_q45(const std::uint8_t* tile, int j, int kc,
                                                  const BlockActivation<S>& act,
                                                  float (&acc)[S]) {
    constexpr int kRow = Q5 ? 176 : 144;
    const std::uint8_t* row = tile + j * kRow;
    const uint4 h = *reinterpret_cast<const uint4*>(row);
    v4i high = {0, 0, 0, 0};
    if constexpr (Q5) high = *reinterpret_cast<const v4i*>(row + 16 + kc * 16);
    const std::uint8_t* quants = row + (Q5 ? 48 : 16) + kc * 16;
    // 6-bit scales and minimums of the eight sub-blocks, packed four per word
    const std::uint32_t sc_lo = h.y & 0x3f3f3f3fu;
    const std::uint32_t mn_lo = h.z & 0x3f3f3f3fu;
    const std::uint32_t sc_hi = (h.w & 0x0f0f0f0fu) | ((h.y >> 2) & 0x30303030u);
    const std::uint32_t mn_hi = ((h.w >> 4) & 0x0f0f0f0fu) | ((h.z >> 2) & 0x30303030u);
    int acc_hi[S], acc_lo[S], acc_min[S];
#pragma unroll
    for (int u = 0; u < S; ++u) {
        acc_hi[u] = 0;
        acc_lo[u] = 0;
        acc_min[u] = 0;
    }
#pragma unroll
    for (int g = 0; g < 4; ++g) {
        const v4i packed = *reinterpret_cast<const v4i*>(quants + g * 32);
        v4i low, upper;
#pragma unroll
        for (int w = 0; w < 4; ++w) {
            const std::uint32_t word = static_cast<std::uint32_t>(packed[w]);
            std::uint32_t lo = word & 0x0f0f0f0fu;
            std::uint32_t up = (word >> 4) & 0x0f0f0f0fu;
            if constexpr (Q5) {
                // bit 2g of the high-bit byte belongs to sub-block 2g, bit 2g+1 to 2g+1
                const std::uint32_t bits = static_cast<std::uint32_t>(high[w]);
                lo |= (g < 2 ? bits << (4 - 2 * g) : bits >> (2 * g - 4)) & 0x10101010u;
                up |= (g < 2 ? bits << (3 - 2 * g) : bits >> (2 * g - 3)) & 0x10101010u;
            }
            low[w] = static_cast<int>(lo);
            upper[w] = static_cast<int>(up);
        }
        // Up to eight tokens both matrix instructions of the group go out before
        // either result is read: the second runs while the first one's products
        // are scaled.  Beyond that the second result costs more in registers
        // than the overlap returns.
        constexpr int kInFlight = S <= 4 ? 2 : 1;
#pragma unroll
        for (int first = 0; first < 2; first += kInFlight) {
            v16i dots[kInFlight];
#pragma unroll
            for (int part = 0; part < kInFlight; ++part) {
                const int sub = 2 * g + first + part;
                dots[part] = mfma32(act.operand(sub), (sub & 1) == 0 ? low : upper);
            }
#pragma unroll
            for (int part = 0; part < kInFlight; ++part) {
                const int sub = 2 * g + first + part;
                const int sc = byte_of(sub < 4 ? sc_lo : sc_hi, sub & 3);
                const int mn = byte_of(sub < 4 ? mn_lo : mn_hi, sub & 3);
#pragma unroll
                for (int u = 0; u < S; ++u) {
                    acc_hi[u] += __mul24(sc, dots[part][2 * u]);
                    acc_lo[u] += __mul24(sc, dots[part][2 * u + 1]);
                    acc_min[u] += __mul24(mn, act.sums[u][sub]);
                }
            }
        }
    }
    const float d = half_bits_to_float(h.x & 0xffffu);
    const float dmin = half_bits_to_float(h.x >> 16);
#pragma unroll
    for (int u = 0; u < S; ++u) {
        const float codes = fmaf(static_cast<float>(acc_hi[u]), 256.0f, static_cast<float>(acc_lo[u]));
        const float value = fmaf(-dmin, static_cast<float>(acc_min[u]), d * codes);
        acc[u] = fmaf(act.scale[u], value, acc[u]);
    }
}

// ---- Q6_K ---------------------------------------------------------------------
template <int S>
__device__ __forceinline__ void process_block_q6(const std::uint8_t* tile, int j, int kc,
                                                 const BlockActivation<S>& act, float (&acc)[S]) {
    const std::uint8_t* row = tile + j * 240;
    const uint4 sc = *reinterpret_cast<const uint4*>(row + 192);
    const std::uint32_t scales[4] = {sc.x, sc.y, sc.z, sc.w};
    int acc_hi[S], acc_lo[S];
#pragma unroll
    for (int u = 0; u < S; ++u) {
        acc_hi[u] = 0;
        acc_lo[u] = 0;
    }
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const v4i ql_a = *reinterpret_cast<const v4i*>(row + half * 64 + kc * 16);
        const v4i ql_b = *reinterpret_cast<const v4i*>(row + half * 64 + 32 + kc * 16);
        const v4i qh = *reinterpret_cast<const v4i*>(row + 128 + half * 32 + kc * 16);
        // the codes of quarter `quarter` as signed bytes
        auto unpack = [&](int quarter) {
            v4i q;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const std::uint32_t ql = static_cast<std::uint32_t>((quarter & 1) ? ql_b[w] : ql_a[w]);
                const std::uint32_t nib = (quarter < 2 ? ql : ql >> 4) & 0x0f0f0f0fu;
                const std::uint32_t bits = static_cast<std::uint32_t>(qh[w]);
                // bits 2q, 2q+1 of the high byte move to bits 4, 5
                const std::uint32_t top =
                    (quarter < 2 ? bits << (4 - 2 * quarter) : bits >> (2 * quarter - 4)) & 0x30303030u;
                // q - 32 with no borrow between bytes: ((q | 0x80) - 0x20) ^ 0x80
                q[w] = static_cast<int>(((nib | top | 0x80808080u) - 0x20202020u) ^ 0x80808080u);
            }
            return q;
        };
        // the matrix instructions go out two at a time: the second runs while
        // the first one's products are scaled
        // (up to four tokens; beyond that two results in flight cost more in
        // registers than the overlap returns)
        constexpr int kInFlight = S <= 2 ? 2 : 1;
#pragma unroll
        for (int first = 0; first < 4; first += kInFlight) {
            v16i dots[kInFlight];
#pragma unroll
            for (int part = 0; part < kInFlight; ++part) {
                dots[part] = mfma32(act.operand(half * 4 + first + part), unpack(first + part));
            }
#pragma unroll
            for (int part = 0; part < kInFlight; ++part) {
                const int sub = half * 4 + first + part;
                // a lane's k-half is one 16-value group: rows of the first group
                // carry zeros in k-half 1 and the other way round
                const int s0 = signed_byte_of(scales[sub >> 1], (2 * sub) & 3);
                const int s1 = signed_byte_of(scales[sub >> 1], (2 * sub + 1) & 3);
#pragma unroll
                for (int u = 0; u < S; ++u) {
                    acc_hi[u] += __mul24(s0, dots[part][4 * u]) + __mul24(s1, dots[part][4 * u + 2]);
                    acc_lo[u] += __mul24(s0, dots[part][4 * u + 1]) + __mul24(s1, dots[part][4 * u + 3]);
                }
            }
        }
    }
    const float d = half_bits_to_float(*reinterpret_cast<const std::uint16_t*>(row + 208));
#pragma unroll
    for (int u = 0; u < S; ++u) {
        const float codes = fmaf(static_cast<float>(acc_hi[u]), 256.0f, static_cast<float>(acc_lo[u]));
        acc[u] = fmaf(act.scale[u], d * codes, acc[u]);
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

__device__ __forceinline__ void wave_lds_fence() {
    // LDS traffic of one wave is in order; this only pins the compiler.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// Projection a tile belongs to.
__device__ __forceinline__ Projection tile_projection(const ProjectionSet& set, std::uint32_t tile) {
    int which = 0;
#pragma unroll
    for (int index = 1; index < 4; ++index) {
        if (index < set.count && tile >= set.op[index].first_tile) which = index;
    }
    return pick(set, which);
}

// Where the results of a tile go.
struct TileOutput {
    float* output;
    std::int64_t output_dim;
    std::int64_t row0;
    int valid_rows;
    __device__ __forceinline__ TileOutput(const ProjectionSet& set, std::uint32_t tile) {
        const Projection op = tile_projection(set, tile);
        row0 = static_cast<std::int64_t>(tile - op.first_tile) * kTileRows;
        valid_rows = static_cast<int>(min(static_cast<std::int64_t>(kTileRows), op.output_dim - row0));
        output = op.output;
        output_dim = op.output_dim;
    }
};

// Where the chunks a lane copies for one tile come from.
template <std::uint32_t ENC>
struct TileSource {
    using F = Format<ENC>;
    static constexpr int kTotalChunks = kTileRows * F::kChunks;
    static constexpr int kLoads = (kTotalChunks + kWave - 1) / kWave;
    const std::uint8_t* base;      // first byte of the tile's first row (uniform)
    const std::uint8_t* data_end;  // end of the tensor (uniform)
    std::uint32_t offset[kLoads];  // byte offset of this lane's chunk i from base

    __device__ __forceinline__ void setup(const ProjectionSet& set, std::uint32_t tile, int lane) {
        const Projection op = tile_projection(set, tile);
        const std::int64_t row0 = static_cast<std::int64_t>(tile - op.first_tile) * kTileRows;
        const int valid_rows =
            static_cast<int>(min(static_cast<std::int64_t>(kTileRows), op.output_dim - row0));
        base = op.data + row0 * op.row_stride;
        data_end = op.data + op.output_dim * op.row_stride;
        const std::uint32_t stride = static_cast<std::uint32_t>(op.row_stride);
#pragma unroll
        for (int i = 0; i < kLoads; ++i) {
            // lanes past the last chunk repeat it: same bytes to the same LDS
            // address, and no lane-masked load to blur the load counters
            const int chunk = min(i * kWave + lane, kTotalChunks - 1);
            const int row = chunk / F::kChunks;
            const int col = chunk - row * F::kChunks;
            offset[i] = static_cast<std::uint32_t>(min(row, valid_rows - 1)) * stride + col * 16;
        }
    }
};

// Q6_K blocks are 210 bytes: every other block of a row starts two bytes past a word, and a
// 16-byte load that is not word aligned runs at a fraction of an aligned one's rate.  Such a
// chunk is read from two bytes earlier and moved into place when it goes to LDS
// (store_block), with the first word of the next chunk, which the next lane holds.
// `flags` remembers per load: bit i: moved down two bytes; bit 8 + i: read at the tensor's end.
// REALIGN false keeps the loads where the chunks are: the lm_head at two to eight tokens has
// no vector instructions to spare for the moving (263 us as read, 272 us realigned), the short
// launches of a decode layer are waiting for memory (17.2 -> 16.1 us on the attention
// projections at four tokens).
template <std::uint32_t ENC, bool REALIGN>
__device__ __forceinline__ void fetch_block(const TileSource<ENC>& src, std::int64_t block,
                                            int lane, uint4 (&staged)[TileSource<ENC>::kLoads],
                                            std::uint32_t& flags) {
    using F = Format<ENC>;
    const std::uint8_t* block_base = src.base + block * F::kBlockBytes;
    flags = 0;
#pragma unroll
    for (int i = 0; i < TileSource<ENC>::kLoads; ++i) {
        const std::uint8_t* p = block_base + src.offset[i];
        if constexpr (F::kAligned) {
            staged[i] = load_chunk<ENC>(p);
        } else {
            const std::uint32_t two =
                REALIGN ? static_cast<std::uint32_t>(reinterpret_cast<std::uintptr_t>(p)) & 2u : 0u;
            p -= two;
            // The last chunk of a block reads past it; only its first two bytes (the block's
            // d) are used.  At the very end of the tensor the 16 bytes before the end are
            // read instead, whose last two bytes they are.
            const bool past = p + 16 > src.data_end;
            staged[i] = load_chunk<ENC>(past ? src.data_end - 16 : p);
            flags |= (two >> 1) << i;
            flags |= (past ? 1u : 0u) << (8 + i);
        }
    }
}

template <std::uint32_t ENC, bool REALIGN>
__device__ __forceinline__ void store_block(const uint4 (&staged)[TileSource<ENC>::kLoads],
                                            std::uint32_t flags, int lane,
                                            std::uint8_t* wave_tile) {
    using F = Format<ENC>;
#pragma unroll
    for (int i = 0; i < TileSource<ENC>::kLoads; ++i) {
        const int chunk = min(i * kWave + lane, TileSource<ENC>::kTotalChunks - 1);
        const int row = chunk / F::kChunks;
        const int col = chunk - row * F::kChunks;
        if constexpr (!F::kAligned) {
            const uint4 read = staged[i];
            // the next chunk's first word: the next lane's, for lane 63 lane 0 of the next load
            // (a row's last chunk needs none: its two bytes are in the words it read)
            const std::uint32_t wrapped = i + 1 < TileSource<ENC>::kLoads
                ? __builtin_amdgcn_readfirstlane(staged[i + 1 < TileSource<ENC>::kLoads ? i + 1 : i].x)
                : 0u;
            const bool moved = REALIGN && ((flags >> i) & 1u) != 0;
            const bool past = ((flags >> (8 + i)) & 1u) != 0;
            // (a chunk read at the tensor's end holds those two bytes in its last word)
            const std::uint32_t next = static_cast<std::uint32_t>(__builtin_amdgcn_update_dpp(
                static_cast<int>(wrapped), static_cast<int>(past ? read.w : read.x),
                0x130 /* wave_shl:1 */, 0xf, 0xf, false));
            uint4 placed;
            placed.x = moved ? __builtin_amdgcn_alignbit(read.y, read.x, 16) : read.x;
            placed.y = moved ? __builtin_amdgcn_alignbit(read.z, read.y, 16) : read.y;
            placed.z = moved ? __builtin_amdgcn_alignbit(read.w, read.z, 16) : read.z;
            placed.w = moved ? __builtin_amdgcn_alignbit(next, read.w, 16) : read.w;
            if (past) placed.x = read.w >> 16;
            *reinterpret_cast<uint4*>(wave_tile + row * F::kLdsRow + col * 16) = placed;
            continue;
        }
        *reinterpret_cast<uint4*>(wave_tile + row * F::kLdsRow + col * 16) = staged[i];
    }
}

// Where the int8 activation planes of a launch come from.
//   kWorkspace: a quantizer launch wrote them to the caller's workspace.
//   kResident:  every wave quantizes the activations of its own K range once,
//               at the start, into LDS records it keeps for all its tiles; the
//               float inputs are loaded before the first packed chunks and are
//               dead before the main loop starts.  Needs LDS for tokens x blocks
//               records.
//   kStream:    every wave quantizes block by block; the float inputs of the
//               blocks in flight sit in registers next to the packed chunks, so
//               the prefetch depth is two.  No LDS limit on K.
constexpr int kWorkspace = 0;
constexpr int kResident = 1;
constexpr int kStream = 2;
constexpr int kEarlyBlocks = 4;  // blocks per wave whose inputs are loaded before the weights

template <std::uint32_t ENC, int MODE>
constexpr int prefetch_depth() {
    return MODE == kStream ? 2 : Format<ENC>::kDepth;
}

// float4 registers one block's inputs take in a lane
template <int S, int P>
constexpr int input_registers() {
    return 2 * S * (P == kPlain ? 1 : 2);
}

// ARGMAX: instead of storing the results the workgroup keeps, per token, the
// best (value, row) of each tile in `candidates` ([tokens][tiles]); a second
// launch reduces them, so the logits of an lm_head never reach memory.
template <std::uint32_t ENC, int S, int MODE, int P, bool ARGMAX>
__global__ __launch_bounds__(kThreads) void gemv_mfma_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    const std::uint8_t* __restrict__ workspace, int tokens, std::uint32_t total_tiles,
    int pass_capacity, int input_dim, LmHeadCandidate* __restrict__ candidates,
    ProjectionSet set) {
    using F = Format<ENC>;
    using Source = TileSource<ENC>;
    constexpr bool kQ6 = ENC == kEncQ6K;
    constexpr int kTokens = 2 * S;
    constexpr int kDepth = prefetch_depth<ENC, MODE>();
    constexpr int kTileBytes = kTileRows * F::kLdsRow;
    extern __shared__ __attribute__((aligned(16))) std::uint8_t lds[];

    const int lane = threadIdx.x & 63;
    // the wave index is uniform; saying so keeps tile bookkeeping in scalar registers
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31;
    const int kc = lane >> 5;
    const std::int64_t blocks = input_dim >> 8;
    // K is cut into kWaves shares; which wave takes which is free (the sums meet in share
    // order).  Waves w and w + 4 run on one SIMD: with this choice the shares that are one
    // block longer than the others spread over the four SIMDs (26 blocks: shares 3 and 7).
    const int share = (0x63571240 >> (4 * wave)) & 7;
    const std::int64_t begin = blocks * share / kWaves;
    const std::int64_t end = blocks * (share + 1) / kWaves;
    const int count = static_cast<int>(end - begin);
    const int max_count = static_cast<int>((blocks + kWaves - 1) / kWaves);

    // LDS: [waves][tile] | [2][waves][lanes][S] partial sums | records:
    // kResident [waves][max_count][tokens], kStream [waves][tokens]
    std::uint8_t* wave_tile = lds + wave * kTileBytes;
    float* partial = reinterpret_cast<float*>(lds + kWaves * kTileBytes);
    std::uint8_t* wave_records = lds + kWaves * kTileBytes + 2 * kWaves * kWave * S * 4 +
        wave * (MODE == kResident ? max_count : 1) * kTokens * kActRecord;

    const int token0 = blockIdx.y * pass_capacity;
    const int pass_tokens = min(tokens - token0, pass_capacity);
    const std::uint8_t* pass_workspace = MODE == kWorkspace
        ? workspace + static_cast<std::int64_t>(token0) * blocks * kActRecord : nullptr;
    const float* pass_first =
        MODE == kWorkspace ? nullptr : first + static_cast<std::int64_t>(token0) * input_dim;
    const float* pass_second = MODE == kWorkspace || P == kPlain
        ? nullptr : second + static_cast<std::int64_t>(token0) * input_dim;
    // float inputs of block `block` of this wave's range for token slot t
    auto load_input = [&](int block, int t) {
        const int token = min(t, pass_tokens - 1);
        return load_activations<P>(pass_first, pass_second,
                                   static_cast<std::int64_t>(token) * input_dim +
                                       (begin + block) * 256 + lane * 4);
    };

    // kResident: the inputs of the first blocks go out before anything else
    float4 early[MODE == kResident ? kEarlyBlocks : 1][MODE == kResident ? kTokens : 1];
    if constexpr (MODE == kResident) {
#pragma unroll
        for (int b = 0; b < kEarlyBlocks; ++b) {
#pragma unroll
            for (int t = 0; t < kTokens; ++t) early[b][t] = load_input(max(min(b, count - 1), 0), t);
        }
    }

    // Every wave walks the same flat stream of (tile, step) pairs: its tiles are
    // blockIdx.x, blockIdx.x + gridDim.x, ..., and a tile takes max_count steps
    // for every wave (a wave whose K range is one block shorter idles in the
    // last step), so the waves meet at the end of a tile in uniform control
    // flow.  Loads run kDepth steps ahead of the arithmetic.  They are all
    // unconditional (indices are clamped instead) and the loop body is
    // unrolled over the kDepth register sets, so the compiler knows exactly
    // how many loads were issued after the one a step needs and a step waits
    // for nothing but its own chunks and activations.
    const std::uint32_t first_tile = blockIdx.x;
    const int steps = max_count;
    const int tile_count = static_cast<int>((total_tiles - first_tile + gridDim.x - 1) / gridDim.x);
    const int total = tile_count * steps;

    Source fetch_source;
    std::uint32_t fetch_tile = first_tile;
    int fetch_step = 0;
    fetch_source.setup(set, fetch_tile, lane);
    uint4 staged[kDepth][Source::kLoads];
    std::uint32_t staged_flags[kDepth];
    float4 inputs[MODE == kStream ? kDepth : 1][MODE == kStream ? kTokens : 1];
    auto fetch = [&](uint4 (&chunks)[Source::kLoads], std::uint32_t& chunk_flags,
                     float4 (&slot)[MODE == kStream ? kTokens : 1]) {
        const int block = max(min(fetch_step, count - 1), 0);
        if constexpr (MODE == kStream) {
            // the float activations of the block go out ahead of its chunks
#pragma unroll
            for (int t = 0; t < kTokens; ++t) slot[t] = load_input(block, t);
        }
        fetch_block<ENC, !ARGMAX>(fetch_source, begin + block, lane, chunks, chunk_flags);
        if (++fetch_step == steps) {
            fetch_step = 0;
            if (fetch_tile + gridDim.x < total_tiles) {
                fetch_tile += gridDim.x;
                fetch_source.setup(set, fetch_tile, lane);
            } else {
                // stream exhausted: the remaining (never used) fetches all hit one line
#pragma unroll
                for (int i = 0; i < Source::kLoads; ++i) fetch_source.offset[i] = 0;
            }
        }
    };
    // kResident: only the first block's weights are requested ahead of the quantization, the
    // rest after it.  Weight requests that go out ahead of the activation loads of waves
    // that start later delay those, and every wave waits for its activations first (all
    // four blocks ahead: 12.5 us per launch of the headline workload at four tokens; one:
    // 10.8; none: 11.8).
    constexpr int kAhead = MODE == kResident ? 1 : kDepth;
#pragma unroll
    for (int d = 0; d < kAhead; ++d) fetch(staged[d], staged_flags[d], inputs[MODE == kStream ? d : 0]);

    if constexpr (MODE == kResident) {
#pragma unroll
        for (int b = 0; b < kEarlyBlocks; ++b) {
#pragma unroll
            for (int t = 0; t < kTokens; ++t) {
                if (b < count && t < pass_tokens) {
                    quantize_block(early[b][t], lane, wave_records + (b * kTokens + t) * kActRecord);
                }
            }
        }
        // a longer K range: the rest one block at a time
        for (int b = kEarlyBlocks; b < count; ++b) {
#pragma unroll
            for (int t = 0; t < kTokens; ++t) {
                const float4 x = load_input(b, t);
                if (t < pass_tokens) {
                    quantize_block(x, lane, wave_records + (b * kTokens + t) * kActRecord);
                }
            }
        }
        wave_lds_fence();
    }
#pragma unroll
    for (int d = kAhead; d < kDepth; ++d) fetch(staged[d], staged_flags[d], inputs[MODE == kStream ? d : 0]);

    // Which A row this lane supplies.
    const OperandRow<kQ6> a_row(j, kc);
    const bool a_valid = a_row.token < pass_tokens && a_row.token < kTokens;
    const int operand_token = a_valid ? a_row.token : 0;

    std::uint32_t tile = first_tile;
    int work_step = 0;
    int parity = 0;
    float acc[S];
#pragma unroll
    for (int u = 0; u < S; ++u) acc[u] = 0.0f;

    auto step = [&](uint4 (&chunks)[Source::kLoads], std::uint32_t& chunk_flags,
                    float4 (&slot)[MODE == kStream ? kTokens : 1], int position) {
        if (position < total) {
            if (work_step < count) {
                store_block<ENC, !ARGMAX>(chunks, chunk_flags, lane, wave_tile);
                if constexpr (MODE == kStream) {
#pragma unroll
                    for (int t = 0; t < kTokens; ++t) {
                        if (t < pass_tokens) {
                            quantize_block(slot[t], lane, wave_records + t * kActRecord);
                        }
                    }
                }
                wave_lds_fence();

                BlockActivation<S> act;
                act.kc = kc;
                act.keep = a_row.keep;
                // records of this block: one per token, in LDS or in the workspace
                const std::uint8_t* records = MODE == kWorkspace
                    ? pass_workspace + (begin + work_step) * kActRecord
                    : wave_records + (MODE == kResident ? work_step * kTokens * kActRecord : 0);
                const std::int64_t token_stride =
                    MODE == kWorkspace ? blocks * kActRecord : kActRecord;
                act.operand_base = records + operand_token * token_stride + a_row.plane * 256;
#pragma unroll
                for (int u = 0; u < S; ++u) {
                    const int token = min(2 * u + kc, pass_tokens - 1);
                    const std::uint8_t* record = records + token * token_stride;
                    act.scale[u] = *reinterpret_cast<const float*>(record + kRecordScale);
                    if constexpr (!kQ6) {
                        const int4 s0 = *reinterpret_cast<const int4*>(record + kRecordSums);
                        const int4 s1 = *reinterpret_cast<const int4*>(record + kRecordSums + 16);
                        act.sums[u][0] = s0.x; act.sums[u][1] = s0.y;
                        act.sums[u][2] = s0.z; act.sums[u][3] = s0.w;
                        act.sums[u][4] = s1.x; act.sums[u][5] = s1.y;
                        act.sums[u][6] = s1.z; act.sums[u][7] = s1.w;
                    }
                }
                if constexpr (ENC == kEncQ4K) {
                    process_block_q45<S, false>(wave_tile, j, kc, act, acc);
                } else if constexpr (ENC == kEncQ5K) {
                    process_block_q45<S, true>(wave_tile, j, kc, act, acc);
                } else {
                    process_block_q6<S>(wave_tile, j, kc, act, acc);
                }
                wave_lds_fence();  // the next block's stores stay behind these reads
            }
            if (++work_step == steps) {
                // Cross-wave sum in a fixed order; the two buffers alternate so
                // one barrier per tile is enough.
                float* mine = partial + ((parity * kWaves + share) * kWave + lane) * S;
#pragma unroll
                for (int u = 0; u < S; ++u) mine[u] = acc[u];
                __syncthreads();
                if (wave == (parity ? kWaves - 1 : 0)) {
                    const TileOutput out(set, tile);
#pragma unroll
                    for (int u = 0; u < S; ++u) {
                        const int token = 2 * u + kc;
                        float sum = partial[((parity * kWaves + 0) * kWave + lane) * S + u];
#pragma unroll
                        for (int w = 1; w < kWaves; ++w) {
                            sum += partial[((parity * kWaves + w) * kWave + lane) * S + u];
                        }
                        if constexpr (ARGMAX) {
                            // best of the tile's 32 rows within each half of the wave
                            float value = j < out.valid_rows ? sum : -INFINITY;
                            std::int64_t index = out.row0 + j;
#pragma unroll
                            for (int offset = 16; offset > 0; offset >>= 1) {
                                const float other_value = __shfl_xor(value, offset, 64);
                                const std::int64_t other_index = __shfl_xor(index, offset, 64);
                                better(other_value, other_index, value, index);
                            }
                            if (j == 0 && token < pass_tokens) {
                                LmHeadCandidate candidate;
                                candidate.index = index;
                                candidate.value = value;
                                candidate.pad = 0;
                                candidates[static_cast<std::int64_t>(token0 + token) * total_tiles +
                                           tile] = candidate;
                            }
                        } else if (token < pass_tokens && j < out.valid_rows) {
                            out.output[static_cast<std::int64_t>(token0 + token) * out.output_dim +
                                       out.row0 + j] = sum;
                        }
                    }
                }
                parity ^= 1;
                work_step = 0;
                tile += gridDim.x;
#pragma unroll
                for (int u = 0; u < S; ++u) acc[u] = 0.0f;
            }
        }
        fetch(chunks, chunk_flags, slot);
    };

    for (int position = 0; position < total; position += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            step(staged[d], staged_flags[d], inputs[MODE == kStream ? d : 0], position + d);
        }
    }
}

// ---- activation quantizer for the passes that do not quantize in the kernel --

template <int P>
__global__ __launch_bounds__(256) void quantize_activations_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    std::uint8_t* __restrict__ workspace, std::int64_t total_blocks) {
    // one wave per (token, super-block) record
    const int lane = threadIdx.x & 63;
    const std::int64_t record = static_cast<std::int64_t>(blockIdx.x) * 4 + (threadIdx.x >> 6);
    if (record >= total_blocks) return;
    const float4 x = load_activations<P>(first, second, record * 256 + lane * 4);
    quantize_block(x, lane, workspace + record * kActRecord);
}

void launch_quantizer(const float* first, const float* second, int prologue, std::int64_t records,
                      std::uint8_t* workspace, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((records + 3) / 4));
    switch (prologue) {
        case kGated:
            hipLaunchKernelGGL((quantize_activations_kernel<kGated>), grid, dim3(256), 0, stream,
                               first, second, workspace, records);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((quantize_activations_kernel<kSwiGlu>), grid, dim3(256), 0, stream,
                               first, second, workspace, records);
            break;
        default:
            hipLaunchKernelGGL((quantize_activations_kernel<kPlain>), grid, dim3(256), 0, stream,
                               first, second, workspace, records);
            break;
    }
}

// What one launch needs beyond the projections.
struct Pass {
    const float* first;
    const float* second;
    int prologue;
    std::uint8_t* workspace;
    int tokens;
    bool* quantized;  // whether the quantizer launch of this call has been enqueued
    LmHeadCandidate* candidates;  // lm_head: per-tile candidates instead of outputs
    hipStream_t stream;
};

constexpr std::size_t kLdsBudget = 150 * 1024;

template <std::uint32_t ENC, int S, int MODE>
std::size_t lds_bytes(std::int64_t blocks) {
    const std::size_t max_count = static_cast<std::size_t>((blocks + kWaves - 1) / kWaves);
    const std::size_t records = MODE == kResident ? max_count : MODE == kStream ? 1 : 0;
    return static_cast<std::size_t>(kWaves) * kTileRows * Format<ENC>::kLdsRow +
        2u * kWaves * kWave * S * 4 + kWaves * records * 2u * S * kActRecord;
}

template <std::uint32_t ENC, int S, int MODE, int P, bool ARGMAX>
void launch_variant(ProjectionSet set, const Pass& pass) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = tiles;
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kTileRows - 1) / kTileRows);
    }
    if (MODE == kWorkspace && !*pass.quantized) {
        launch_quantizer(pass.first, pass.second, pass.prologue,
                         static_cast<std::int64_t>(pass.tokens) * (set.input_dim >> 8),
                         pass.workspace, pass.stream);
        *pass.quantized = true;
    }
    auto kernel = gemv_mfma_kernel<ENC, S, MODE, P, ARGMAX>;
    allow_large_lds<gemv_mfma_kernel<ENC, S, MODE, P, ARGMAX>>();
    const int pass_capacity = 2 * S;
    const int passes = (pass.tokens + pass_capacity - 1) / pass_capacity;
    // persistent grid: one workgroup per compute unit, fewer when there are fewer tiles
    const std::uint32_t grid = tiles < static_cast<std::uint32_t>(compute_units())
        ? tiles : static_cast<std::uint32_t>(compute_units());
    const std::size_t lds = lds_bytes<ENC, S, MODE>(set.input_dim >> 8);
    hipLaunchKernelGGL(kernel, dim3(grid, passes), dim3(kThreads), lds, pass.stream, pass.first,
                       pass.second, pass.workspace, pass.tokens, tiles, pass_capacity,
                       static_cast<int>(set.input_dim), pass.candidates, set);
}

// Resident records where LDS holds them and the inputs of the early blocks fit
// in registers, streamed quantization where only the latter holds, the
// quantizer launch otherwise.
template <std::uint32_t ENC, int S, int P, bool ARGMAX>
void launch_tokens(const ProjectionSet& set, const Pass& pass) {
    constexpr bool kResidentFits = kEarlyBlocks * input_registers<S, P>() <= 16;
    constexpr bool kStreamFits = 2 * input_registers<S, P>() <= 16;
    if constexpr (kResidentFits) {
        if (lds_bytes<ENC, S, kResident>(set.input_dim >> 8) <= kLdsBudget) {
            launch_variant<ENC, S, kResident, P, ARGMAX>(set, pass);
            return;
        }
    }
    if constexpr (kStreamFits) {
        // Streamed quantization repeats for every tile of a workgroup: with two or more
        // tiles each, one quantizer launch and records read from the workspace are cheaper.
        std::int64_t tiles = 0;
        for (int index = 0; index < set.count; ++index) {
            tiles += (set.op[index].output_dim + kTileRows - 1) / kTileRows;
        }
        if (tiles < 2 * static_cast<std::int64_t>(compute_units()) || pass.workspace == nullptr) {
            launch_variant<ENC, S, kStream, P, ARGMAX>(set, pass);
            return;
        }
    }
    launch_variant<ENC, S, kWorkspace, kPlain, ARGMAX>(set, pass);
}

template <std::uint32_t ENC, int P, bool ARGMAX>
void launch_prologue(const ProjectionSet& set, const Pass& pass) {
    constexpr bool kQ6 = ENC == kEncQ6K;
    if (pass.tokens <= 2) {
        launch_tokens<ENC, 1, P, ARGMAX>(set, pass);
    } else if (pass.tokens <= 4) {
        launch_tokens<ENC, 2, P, ARGMAX>(set, pass);
    } else if (pass.tokens <= 8 || kQ6) {
        launch_tokens<ENC, 4, P, ARGMAX>(set, pass);
    } else {
        if constexpr (!kQ6 && !ARGMAX) launch_tokens<ENC, 8, P, false>(set, pass);
    }
}

template <std::uint32_t ENC>
void launch_encoding(const ProjectionSet& set, const Pass& pass) {
    if (pass.candidates != nullptr) {
        launch_prologue<ENC, kPlain, true>(set, pass);
        return;
    }
    switch (pass.prologue) {
        case kGated: launch_prologue<ENC, kGated, false>(set, pass); break;
        case kSwiGlu: launch_prologue<ENC, kSwiGlu, false>(set, pass); break;
        default: launch_prologue<ENC, kPlain, false>(set, pass); break;
    }
}

void launch_groups(const ProjectionSet& set, const Pass& pass) {
    // one launch per encoding present
    const std::uint32_t encodings[3] = {kEncQ4K, kEncQ5K, kEncQ6K};
    for (const std::uint32_t encoding : encodings) {
        ProjectionSet group{};
        group.input_dim = set.input_dim;
        for (int index = 0; index < set.count; ++index) {
            if (set.op[index].encoding == encoding) group.op[group.count++] = set.op[index];
        }
        if (group.count == 0) continue;
        if (encoding == kEncQ4K) {
            launch_encoding<kEncQ4K>(group, pass);
        } else if (encoding == kEncQ5K) {
            launch_encoding<kEncQ5K>(group, pass);
        } else {
            launch_encoding<kEncQ6K>(group, pass);
        }
    }
}

}  // namespace

bool gemv_mfma_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K) &&
        input_dim % 256 == 0 && input_dim <= 65536;
}

void launch_gemv_mfma(ProjectionSet set, const float* first, const float* second, int prologue,
                      std::int64_t rows, void* workspace, hipStream_t stream) {
    bool quantized = false;
    const Pass pass{first, second, prologue, static_cast<std::uint8_t*>(workspace),
                    static_cast<int>(rows), &quantized, nullptr, stream};
    launch_groups(set, pass);
}

std::int64_t lm_head_mfma_tiles(std::int64_t output_dim) {
    return (output_dim + kTileRows - 1) / kTileRows;
}

void launch_lm_head_mfma(const Descriptor& descriptor, const float* input, std::int64_t rows,
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
    bool quantized = false;  // up to eight rows always quantize in the kernel
    const Pass pass{input, nullptr, kPlain, nullptr, static_cast<int>(rows), &quantized, candidates,
                    stream};
    launch_groups(set, pass);
    launch_lm_head_final(candidates, lm_head_mfma_tiles(descriptor.output_dim), indices, maxima,
                         rows, stream);
}

}  // namespace nfn
