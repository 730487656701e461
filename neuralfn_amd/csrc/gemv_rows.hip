// Verifier rows (4..16 tokens) of K-quant projections on the int8 matrix cores, every row in
// the one-row kernel's arithmetic bit for bit.
//
// The contract (neuralfn/csrc/native_train/tile_ops.h:685-688; the reference's kernel:
// neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1753-1925): row t of a batched call equals the
// one-row call on row t.  The one-row kernels (gemv_dot.hip, gemv_q6.hip, gemv_q8.hip) give
// lane L of a wave the units u = L, L + 64, ... of a weight row (a unit: 64 values), chain one
// fused multiply-add per unit,
//   Q4_K, Q5_K  acc = fmaf(scale, fmaf(-dmin, float(wmin), d * fmaf(float(whi), 256, float(wlo))), acc)
//   Q6_K        acc = fmaf(scale * d, ((sc0 * float(b0) + sc1 * float(b1)) + ...) in fused steps, acc)
//   Q8_0        acc = fmaf(scale, fmaf(d1, float(b1), d0 * float(b0)), acc)
// over them and sum the 64 lanes in a butterfly.  Everything up to the integers in these
// formulas is exact integer arithmetic, and float addition is commutative, so the result is
// fixed by
//   * which terms form a chain: the units 4b + p of the blocks b = c, c + 16, c + 32, ...
//     ("class" c = 0..15, p = 0..3; a block: 256 values), in that order,
//   * the balanced binary tree over the 64 chains in the order (c, p).
// Here a workgroup of 8 waves owns 32 consecutive weight rows.  A matrix instruction takes
// the values of a scale group (K: 32 values, 16 for Q6_K), 32 weight rows (operand B, lane l:
// row l % 32, half l / 32 of the group; the packed bytes are loaded coalesced and change lanes
// through a private LDS tile per wave) and the two int8 planes of up to 16 tokens (operand A,
// fetched in operand order from the image a quantizer launch left in the workspace beside the
// activation records: lanes that each pick their own 16 bytes out of sixteen records cost the
// memory pipeline four times the instructions' coalesced rate).  For Q4_K / Q5_K a second
// product against the sub-block minimums, spread over K, gives the sums the minimums
// multiply; Q6_K's offset of 32 is taken off the codes before the product.  A lane then holds,
// for its weight row and up to 8 tokens, the integers of a unit, and replays the float tail
// above.  Wave w takes the classes w and 15 - w (an even share of any row length), keeps the
// four chains of a class per token in registers, and leaves (c0 + c1) + (c2 + c3) per class,
// token and row in LDS; after one barrier a thread per (token, row) adds the 16 classes in the
// tree's order.  A workgroup walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ... with the
// loads of the next tile's first block in flight under the last block of the one before.
// One pass over the weights for up to 16 tokens.
#include "common.hpp"
#include "gemv_rows.hpp"
#include "wave_rows.hpp"

namespace nfn {

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef unsigned v4u __attribute__((ext_vector_type(4)));

constexpr int kRowsTile = 32;
constexpr int kRowsWaves = 8;
constexpr int kRowsThreads = kRowsWaves * kWave;
constexpr int kClasses = 16;
constexpr int kMaxRowsBlocks = 256;  // input_dim up to 65,536: the blocks whose scales a workgroup keeps

constexpr int kImageFragments = kRowsImageFragments;
constexpr int kImageBlock = kRowsImageBlock;

// One wave per activation record: writes the (token, block) record of wave_rows.hpp and the
// token's share of the block's operand image.
// Workgroups past those of the records fill the outputs of `clear` with -0.0f, 1024 floats a
// workgroup: the split form of the kernel below adds the two halves of a row's butterfly
// onto them (-0 + x is x for every x, -0 included).
template <int P>
__global__ __launch_bounds__(256) void quantize_records_kernel(
    const float* __restrict__ first, const float* __restrict__ second,
    std::uint8_t* __restrict__ records, std::uint8_t* __restrict__ image, int blocks, int tokens,
    int record_groups, ProjectionSet clear) {
    if (static_cast<int>(blockIdx.x) >= record_groups) {
        std::int64_t chunk = static_cast<std::int64_t>(blockIdx.x) - record_groups;
#pragma unroll
        for (int index = 0; index < 4; ++index) {
            if (index >= clear.count) break;
            const std::int64_t floats = clear.op[index].output_dim * tokens;
            const std::int64_t chunks = (floats + 1023) >> 10;
            if (chunk < chunks) {
                float* output = clear.op[index].output;
                const std::int64_t begin = (chunk << 10) + threadIdx.x * 4;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (begin + e < floats) output[begin + e] = -0.0f;
                }
                return;
            }
            chunk -= chunks;
        }
        return;
    }
    const int lane = threadIdx.x & 63;
    const int record = static_cast<int>(blockIdx.x) * 4 + static_cast<int>(threadIdx.x >> 6);
    if (record >= blocks * tokens) return;
    const float4 x = load_activations<P>(first, second,
                                         static_cast<std::int64_t>(record) * 256 + lane * 4);
    const ActivationCodes codes = activation_codes<P>(x);
    store_record(records + static_cast<std::int64_t>(record) * kActRecord, lane, codes);
    const int token = record / blocks;
    const int block = record - token * blocks;
    store_operand_image(image, block, token, tokens, lane, codes);
}

// How a block (256 values of one weight row) lies in memory and in a wave's LDS tile.
//   Q4_K / Q5_K: 144 / 176 bytes, 16-byte aligned; the tile is the same bytes row after row.
//   Q8_0: eight 34-byte blocks = 272 bytes; rows are as aligned as the tensor is.
//   Q6_K: 210 bytes, so every other block starts two bytes past a word.  A block is fetched as
//     fourteen 16-byte pieces from the word at or before its first byte (pieces 0..12 in a
//     row, piece 13 from byte 196, so that no load reaches past the word that holds the
//     block's last byte) and written to its 240-byte LDS slot two bytes down when it started
//     past a word: in LDS every block starts at byte 16 of its slot.
template <std::uint32_t ENC>
struct RowsFormat {
    static constexpr bool kQ6 = ENC == kEncQ6K;
    static constexpr bool kQ8 = ENC == kEncQ8_0;
    static constexpr int kBlockBytes = ENC == kEncQ4K ? 144 : ENC == kEncQ5K ? 176 : kQ6 ? 210 : 272;
    static constexpr int kChunks = kQ6 ? 14 : kBlockBytes / 16;  // 16-byte pieces of a block
    static constexpr int kTileChunks = kRowsTile * kChunks;      // of a block of 32 rows
    static constexpr int kLoads = (kTileChunks + kWave - 1) / kWave;
    static constexpr int kSlotBytes = kQ6 ? 240 : kBlockBytes;   // a row's place in the LDS tile
    static constexpr int kSlotOrigin = kQ6 ? 16 : 0;             // where the block starts in it
    static constexpr int kTileBytes = kRowsTile * kSlotBytes;
};

struct __attribute__((packed, aligned(2))) RowsPiece {
    std::uint32_t v[4];
};
struct __attribute__((packed, aligned(2))) RowsHalfPiece {
    std::uint32_t v[2];
};

typedef int v2i __attribute__((ext_vector_type(2)));

// The packed bytes of 32 rows x one block as a wave loads them, coalesced: one set of
// registers (they go to the LDS tile as soon as they arrive, and the next block's request
// reuses them).
template <std::uint32_t ENC>
struct RowsPacked {
    v4u chunk[RowsFormat<ENC>::kLoads];
    std::uint32_t shifted;  // Q6_K: bit i = piece i of this lane starts two bytes past a word
};

// Operand A of the eight 32-value groups of a block: two sets, used by the matrix instructions
// where they arrive.
struct RowsOperands {
    v4i a[8];
};

__device__ __forceinline__ v16i mfma_i8(v4i a, v4i b, v16i c) {
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

// K = 16: operands of 8 bytes a lane (lane l: row l % 32, values 8 (l / 32)..+7)
__device__ __forceinline__ v16i mfma_i8_k16(v2i a, v2i b, v16i c) {
    return __builtin_amdgcn_mfma_i32_32x32x16_i8(__builtin_bit_cast(long, a), __builtin_bit_cast(long, b),
                                                 c, 0, 0, 0);
}

__device__ __forceinline__ void rows_lds_fence() {
    // LDS traffic of one wave is in order; this only pins the compiler.
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// SPLIT: a workgroup computes one half of a row's butterfly, the classes 0..7 (the first
// left_groups workgroups) or 8..15 (the others), a wave one class, and adds (q0 + q1) or
// (q2 + q3) onto the output, which the quantizer launch has filled with -0: two terms commute,
// so the sum is the one-row kernel's whichever half arrives first.  Twice the work units of
// about half the length, shared out over the workgroups by what the halves cost (a row of 26
// blocks has 16 on the left and 10 on the right): for tile counts that leave much of the
// chip idle in the last pass over whole tiles (272 tiles on 256 units).
template <std::uint32_t ENC, int S, bool SPLIT>
__global__ __launch_bounds__(kRowsThreads) void gemv_rows_kernel(
    const std::uint8_t* __restrict__ image, int tokens, int input_dim, std::uint32_t total_tiles,
    std::uint32_t left_groups, ProjectionSet set) {
    constexpr bool kQ5 = ENC == kEncQ5K;
    using F = RowsFormat<ENC>;
    constexpr int kBlockBytes = F::kBlockBytes;
    constexpr int kQuants = kQ5 ? 48 : 16;
    constexpr int kTokens = 2 * S;
    // (two buffers of class sums: the workgroup's waves meet once per tile)
    constexpr int kOwnClasses = SPLIT ? kClasses / 2 : kClasses;
    __shared__ float class_sums[2][kOwnClasses][kTokens][kRowsTile];
    __shared__ __attribute__((aligned(16))) std::uint8_t packed_tiles[kRowsWaves][F::kTileBytes];

    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int j = lane & 31;
    const int h = lane >> 5;
    const int blocks = input_dim >> 8;

    // A workgroup walks the tiles blockIdx.x, blockIdx.x + gridDim.x, ...; the loads of a
    // tile's first block go out under the arithmetic of the tile before.
    const bool right_half = SPLIT && blockIdx.x >= left_groups;
    const std::uint32_t first_tile = right_half ? blockIdx.x - left_groups : blockIdx.x;
    const std::uint32_t tile_stride =
        SPLIT ? (right_half ? gridDim.x - left_groups : left_groups) : gridDim.x;
    const int my_tiles = static_cast<int>((total_tiles - first_tile + tile_stride - 1) / tile_stride);
    auto projection_of = [&](std::uint32_t tile) {
        int which = 0;
#pragma unroll
        for (int index = 1; index < 4; ++index) {
            if (index < set.count && tile >= set.op[index].first_tile) which = index;
        }
        return pick(set, which);
    };

    // What the loads of a tile need: its first row and, per lane, where the pieces it copies
    // per block lie: piece n = 64 i + lane of the 32 x kChunks, kChunks to a row (the lanes
    // past the last piece repeat it), and where in the LDS tile each goes.
    const std::uint8_t* tile_rows;
    std::uint32_t chunk_offset[F::kLoads];
    std::uint32_t row_parity = 0;  // Q6_K: bit i = the row of piece i starts two bytes past a word
    // (Q4_K, Q5_K, Q8_0: the LDS tile is the same bytes row after row, piece n at byte 16 n)
    std::uint32_t lds_offset[F::kQ6 ? F::kLoads : 1];
    if constexpr (F::kQ6) {
#pragma unroll
        for (int i = 0; i < F::kLoads; ++i) {
            const int chunk = i * kWave + lane;
            const int row = chunk / F::kChunks;
            const int col = chunk - row * F::kChunks;
            lds_offset[i] = row * F::kSlotBytes + F::kSlotOrigin + (col == 13 ? 196 : col * 16);
        }
    }
    const int last_slot = min((F::kLoads - 1) * kWave + lane, F::kTileChunks - 1) * 16;
    auto aim = [&](std::uint32_t tile) {
        const Projection op = projection_of(tile);
        const std::int64_t row0 = static_cast<std::int64_t>(tile - op.first_tile) * kRowsTile;
        const int valid_rows =
            static_cast<int>(min(static_cast<std::int64_t>(kRowsTile), op.output_dim - row0));
        tile_rows = op.data + row0 * op.row_stride;
        row_parity = 0;
#pragma unroll
        for (int i = 0; i < F::kLoads; ++i) {
            const int chunk = min(i * kWave + lane, F::kTileChunks - 1);
            const int row = chunk / F::kChunks;
            const int col = chunk - row * F::kChunks;
            const int within = F::kQ6 && col == 13 ? 196 : col * 16;
            const std::uint32_t row_offset = static_cast<std::uint32_t>(min(row, valid_rows - 1)) *
                    static_cast<std::uint32_t>(op.row_stride);
            chunk_offset[i] = row_offset + within;
            if constexpr (F::kQ6) {
                const std::uint32_t address_low = static_cast<std::uint32_t>(
                    reinterpret_cast<std::uintptr_t>(tile_rows)) + row_offset;
                row_parity |= ((address_low >> 1) & 1u) << i;
            }
        }
    };
    std::uint8_t* const my_tile = packed_tiles[wave];
    const std::uint8_t* const my_row = my_tile + j * F::kSlotBytes + F::kSlotOrigin;

    // this wave's steps of a tile: the blocks of class `wave`, then those of class 15 - wave
    // (SPLIT: the one class 8 (right half) + wave)
    const int class0 = SPLIT ? (right_half ? 8 : 0) + wave : wave;
    const int class1 = kClasses - 1 - wave;
    const int count0 = class0 < blocks ? (blocks - class0 + kClasses - 1) / kClasses : 0;
    int count1 = class1 < blocks ? (blocks - class1 + kClasses - 1) / kClasses : 0;
    if constexpr (SPLIT) {
        // (no second class; a value the optimizer cannot see through, so that the walk below
        // compiles as it does for two classes: with a known zero it is scheduled with far
        // more registers, and spills)
        count1 = 0;
        asm volatile("" : "+s"(count1));
    }
    const int total = count0 + count1;

    auto block_of = [&](int step) {
        return step < count0 ? class0 + kClasses * step : class1 + kClasses * (step - count0);
    };
    std::uint32_t fetch_tile = first_tile;
    int fetch_step = 0;
    aim(fetch_tile);
    // the loads of the next step of the walk; past its end the last block again
    auto fetch = [&](RowsPacked<ENC>& stage, RowsOperands& operands) {
        const int block = min(block_of(min(fetch_step, max(total - 1, 0))), blocks - 1);
        const std::uint8_t* weights = tile_rows + static_cast<std::int64_t>(block) * kBlockBytes;
        // (a Q6_K block with an odd index lies two bytes further from a word than its row does)
        const std::uint32_t shifted = F::kQ6 ? row_parity ^ (0u - static_cast<std::uint32_t>(block & 1)) : 0u;
        if constexpr (F::kQ6) stage.shifted = shifted;
#pragma unroll
        for (int i = 0; i < F::kLoads; ++i) {
            if constexpr (F::kQ6 || F::kQ8) {
                // (Q8_0 rows are only as aligned as the tensor; Q6_K pieces start on a word)
                const std::uint32_t back = F::kQ6 ? ((shifted >> i) & 1u) * 2u : 0u;
                const RowsPiece piece = *reinterpret_cast<const RowsPiece*>(weights + chunk_offset[i] - back);
                stage.chunk[i] = v4u{piece.v[0], piece.v[1], piece.v[2], piece.v[3]};
            } else {
                stage.chunk[i] = *reinterpret_cast<const v4u*>(weights + chunk_offset[i]);
            }
        }
        const std::uint8_t* fragments = image + static_cast<std::int64_t>(block) * kImageBlock;
#pragma unroll
        for (int sub = 0; sub < 8; ++sub) {
            if constexpr (F::kQ6) {
                // the sixteen values 16 s..+15 of a 32-value group are what the image keeps for
                // lanes 32 s..+31: this lane takes bytes 8 h..+7 of row j's sixteen, for s = 0, 1
                const std::uint8_t* mine = fragments + sub * 1024 + j * 16 + h * 8;
                const v2i lower = *reinterpret_cast<const v2i*>(mine);
                const v2i upper = *reinterpret_cast<const v2i*>(mine + 512);
                operands.a[sub] = v4i{lower[0], lower[1], upper[0], upper[1]};
            } else {
                operands.a[sub] = *reinterpret_cast<const v4i*>(fragments + sub * 1024 + lane * 16);
            }
        }
        if (++fetch_step >= total && fetch_tile + tile_stride < total_tiles) {
            fetch_step = 0;
            fetch_tile += tile_stride;
            aim(fetch_tile);
        }
    };

    constexpr int kMaxSteps = kMaxRowsBlocks / kRowsWaves;
    __shared__ __attribute__((aligned(16))) float step_scales[kRowsWaves][kMaxSteps][16];

    float acc[4][S];
#pragma unroll
    for (int p = 0; p < 4; ++p) {
#pragma unroll
        for (int slot = 0; slot < S; ++slot) acc[p][slot] = 0.0f;
    }

    // the packed bytes change lanes through the wave's LDS tile
    auto stage_to_lds = [&](const RowsPacked<ENC>& stage) {
        if constexpr (F::kQ6) {
#pragma unroll
            for (int i = 0; i < F::kLoads; ++i) {
                const std::uint32_t back = ((stage.shifted >> i) & 1u) * 2u;
                RowsPiece piece;
                piece.v[0] = stage.chunk[i][0];
                piece.v[1] = stage.chunk[i][1];
                piece.v[2] = stage.chunk[i][2];
                piece.v[3] = stage.chunk[i][3];
                *reinterpret_cast<RowsPiece*>(my_tile + lds_offset[i] - back) = piece;
            }
        } else {
#pragma unroll
            for (int i = 0; i + 1 < F::kLoads; ++i) {
                *reinterpret_cast<v4u*>(my_tile + lane * 16 + i * (kWave * 16)) = stage.chunk[i];
            }
            *reinterpret_cast<v4u*>(my_tile + last_slot) = stage.chunk[F::kLoads - 1];
        }
    };

    auto compute = [&](const RowsOperands& stage, int step) {
        const v16i zero = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
        float scale[S];
#pragma unroll
        for (int slot = 0; slot < S; ++slot) scale[slot] = step_scales[wave][step][S * h + slot];
        if constexpr (F::kQ6) {
            // Q6_K (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:591-616): per half of 128
            // values 64 bytes of low nibbles (quarters 0 / 2 in bytes 0..31, 1 / 3 in 32..63) and
            // 32 bytes of 2-bit tops; 16 int8 sub-scales (half, quarter, sixteen) and d.  This
            // lane decodes values 8 h..+7 of both sixteens of every quarter of row j.
            const RowsPiece sub_scales = *reinterpret_cast<const RowsPiece*>(my_row + 192);
            const float d = half_bits_to_float(*reinterpret_cast<const std::uint16_t*>(my_row + 208));
            float factor[S];
#pragma unroll
            for (int slot = 0; slot < S; ++slot) factor[slot] = scale[slot] * d;
            // The codes go into the product as 4 (q - 32), which is their six bits moved to the
            // top of a byte with the highest one flipped; the sub-scales as sc / 4, so that
            // every product sc * bracket keeps its value (both factors are exact) and every
            // rounding of the one-row kernel's chain happens on the same number.
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                float quarter_scale[8];
#pragma unroll
                for (int w = 0; w < 2; ++w) {
                    const std::uint32_t biased = sub_scales.v[2 * half + w] ^ 0x80808080u;
#pragma unroll
                    for (int byte = 0; byte < 4; ++byte) {
                        quarter_scale[4 * w + byte] =
                            fmaf(static_cast<float>((biased >> (8 * byte)) & 0xffu), 0.25f, -32.0f);
                    }
                }
#pragma unroll
                for (int s = 0; s < 2; ++s) {
                    const std::uint8_t* at = my_row + half * 64 + s * 16 + h * 8;
                    const RowsHalfPiece low_a = *reinterpret_cast<const RowsHalfPiece*>(at);
                    const RowsHalfPiece low_b = *reinterpret_cast<const RowsHalfPiece*>(at + 32);
                    const RowsHalfPiece top =
                        *reinterpret_cast<const RowsHalfPiece*>(my_row + 128 + half * 32 + s * 16 + h * 8);
                    v2i codes[4];
#pragma unroll
                    for (int w = 0; w < 2; ++w) {
                        const std::uint32_t a = low_a.v[w], b = low_b.v[w];
                        const std::uint32_t t = top.v[w] ^ 0xaaaaaaaau;
                        codes[0][w] = static_cast<int>(((a << 2) & 0x3c3c3c3cu) | ((t << 6) & 0xc0c0c0c0u));
                        codes[1][w] = static_cast<int>(((b << 2) & 0x3c3c3c3cu) | ((t << 4) & 0xc0c0c0c0u));
                        codes[2][w] = static_cast<int>(((a >> 2) & 0x3c3c3c3cu) | ((t << 2) & 0xc0c0c0c0u));
                        codes[3][w] = static_cast<int>(((b >> 2) & 0x3c3c3c3cu) | (t & 0xc0c0c0c0u));
                    }
                    // quarter after quarter, so that one product's sixteen integers are live
                    float unit_value[S];
#pragma unroll
                    for (int slot = 0; slot < S; ++slot) unit_value[slot] = 0.0f;
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        const v4i both = stage.a[4 * half + k];
                        const v2i fragment = s == 0 ? v2i{both[0], both[1]} : v2i{both[2], both[3]};
                        const v16i dots = mfma_i8_k16(fragment, codes[k], zero);
#pragma unroll
                        for (int slot = 0; slot < S; ++slot) {
                            // |4 (256 hi + lo)| <= 4 * 16 * 32 * 32512 < 2^27: exact in int32
                            const int bracket = (dots[2 * slot] << 8) + dots[2 * slot + 1];
                            unit_value[slot] =
                                fmaf(quarter_scale[2 * k + s], static_cast<float>(bracket), unit_value[slot]);
                        }
                    }
#pragma unroll
                    for (int slot = 0; slot < S; ++slot) {
                        acc[2 * half + s][slot] = fmaf(factor[slot], unit_value[slot], acc[2 * half + s][slot]);
                    }
                }
            }
            rows_lds_fence();  // the next block's stores stay behind these reads
        } else if constexpr (F::kQ8) {
            // Q8_0: eight blocks of an fp16 scale and 32 int8 codes; the codes are operand B as
            // they lie, this lane's sixteen of each block from byte 34 b + 2 + 16 h
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const std::uint8_t* pair = my_row + 68 * p;
                const RowsPiece c0 = *reinterpret_cast<const RowsPiece*>(pair + 2 + 16 * h);
                const RowsPiece c1 = *reinterpret_cast<const RowsPiece*>(pair + 36 + 16 * h);
                const float d0 = half_bits_to_float(*reinterpret_cast<const std::uint16_t*>(pair));
                const float d1 = half_bits_to_float(*reinterpret_cast<const std::uint16_t*>(pair + 34));
                const v16i dots0 = mfma_i8(stage.a[2 * p], v4i{static_cast<int>(c0.v[0]), static_cast<int>(c0.v[1]),
                                                                static_cast<int>(c0.v[2]), static_cast<int>(c0.v[3])}, zero);
                const v16i dots1 = mfma_i8(stage.a[2 * p + 1], v4i{static_cast<int>(c1.v[0]), static_cast<int>(c1.v[1]),
                                                                    static_cast<int>(c1.v[2]), static_cast<int>(c1.v[3])}, zero);
#pragma unroll
                for (int slot = 0; slot < S; ++slot) {
                    // |256 hi + lo| <= 32 * 127 * 32512 < 2^28: exact in int32
                    const int bracket0 = (dots0[2 * slot] << 8) + dots0[2 * slot + 1];
                    const int bracket1 = (dots1[2 * slot] << 8) + dots1[2 * slot + 1];
                    const float value = fmaf(d1, static_cast<float>(bracket1), d0 * static_cast<float>(bracket0));
                    acc[p][slot] = fmaf(scale[slot], value, acc[p][slot]);
                }
            }
            rows_lds_fence();  // the next block's stores stay behind these reads
        } else {
            // Q4_K / Q5_K: a lane needs the header of row j and its half of the row's codes
            const uint4 head = *reinterpret_cast<const uint4*>(my_row);
            uint4 high = make_uint4(0, 0, 0, 0);
            if constexpr (kQ5) high = *reinterpret_cast<const uint4*>(my_row + 16 + h * 16);
            uint4 quants[4];
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                quants[p] = *reinterpret_cast<const uint4*>(my_row + kQuants + p * 32 + h * 16);
            }
            rows_lds_fence();  // the next block's stores stay behind these reads
            // 6-bit scales and minimums of the eight sub-blocks, four per word
            const std::uint32_t sc_lo = head.y & 0x3f3f3f3fu;
            const std::uint32_t mn_lo = head.z & 0x3f3f3f3fu;
            const std::uint32_t sc_hi = (head.w & 0x0f0f0f0fu) | ((head.y >> 2) & 0x30303030u);
            const std::uint32_t mn_hi = ((head.w >> 4) & 0x0f0f0f0fu) | ((head.z >> 2) & 0x30303030u);
            const float d = half_bits_to_float(head.x & 0xffffu);
            const float dmin = half_bits_to_float(head.x >> 16);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                const std::uint32_t packed[4] = {quants[p].x, quants[p].y, quants[p].z, quants[p].w};
                v4i low, upper;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    std::uint32_t lo = packed[w] & 0x0f0f0f0fu;
                    std::uint32_t up = (packed[w] >> 4) & 0x0f0f0f0fu;
                    if constexpr (kQ5) {
                        const std::uint32_t bits[4] = {high.x, high.y, high.z, high.w};
                        const std::uint32_t shifted = bits[w] >> (2 * p);
                        lo |= (shifted & 0x01010101u) << 4;
                        up |= (shifted & 0x02020202u) << 3;
                    }
                    low[w] = static_cast<int>(lo);
                    upper[w] = static_cast<int>(up);
                }
                const std::uint32_t sc_word = p < 2 ? sc_lo : sc_hi;
                const std::uint32_t mn_word = p < 2 ? mn_lo : mn_hi;
                const int scale_a = static_cast<int>((sc_word >> (16 * (p & 1))) & 0xffu);
                const int scale_b = static_cast<int>((sc_word >> (16 * (p & 1) + 8)) & 0xffu);
                const int min_a = static_cast<int>((mn_word >> (16 * (p & 1))) & 0xffu);
                const int min_b = static_cast<int>((mn_word >> (16 * (p & 1) + 8)) & 0xffu);
                const int spread_a = static_cast<int>(__umul24(min_a, 0x010101u)) | (min_a << 24);
                const int spread_b = static_cast<int>(__umul24(min_b, 0x010101u)) | (min_b << 24);
                const v4i mins_a = {spread_a, spread_a, spread_a, spread_a};
                const v4i mins_b = {spread_b, spread_b, spread_b, spread_b};
                // the sub-block scales times 256, opaque to the optimizer: it would otherwise factor
                // scale * (256 * hi + lo) out and pay a full 32-bit multiplication for it
                int scale_a256, scale_b256;
                asm("v_lshlrev_b32 %0, 8, %1" : "=v"(scale_a256) : "v"(scale_a));
                asm("v_lshlrev_b32 %0, 8, %1" : "=v"(scale_b256) : "v"(scale_b));
                const v16i dots_a = mfma_i8(stage.a[2 * p], low, zero);
                const v16i dots_b = mfma_i8(stage.a[2 * p + 1], upper, zero);
                // min_a * sum(codes of a) + min_b * sum(codes of b), per plane
                const v16i sums = mfma_i8(stage.a[2 * p + 1], mins_b, mfma_i8(stage.a[2 * p], mins_a, zero));
#pragma unroll
                for (int slot = 0; slot < S; ++slot) {
                    float codes;
                    if constexpr (kQ5) {
                        const int weighted_hi =
                            __mul24(scale_a, dots_a[2 * slot]) + __mul24(scale_b, dots_b[2 * slot]);
                        const int weighted_lo =
                            __mul24(scale_a, dots_a[2 * slot + 1]) + __mul24(scale_b, dots_b[2 * slot + 1]);
                        codes = fmaf(static_cast<float>(weighted_hi), 256.0f, static_cast<float>(weighted_lo));
                    } else {
                        // 4-bit codes: 256 * weighted_hi + weighted_lo stays below 2^31
                        // (2 * 63 * 32 * 15 * (127 * 256 + 128)), and one conversion rounds the
                        // exact integer as the fused multiply-add of the two exact floats does
                        // (a chain of multiply-adds: the empty statements keep the optimizer from
                        // turning it into a tree with one more instruction)
                        int weighted = __mul24(scale_a256, dots_a[2 * slot]);
                        asm("" : "+v"(weighted));
                        weighted += __mul24(scale_b256, dots_b[2 * slot]);
                        asm("" : "+v"(weighted));
                        weighted += __mul24(scale_a, dots_a[2 * slot + 1]);
                        asm("" : "+v"(weighted));
                        weighted += __mul24(scale_b, dots_b[2 * slot + 1]);
                        codes = static_cast<float>(weighted);
                    }
                    const int weighted_min = sums[2 * slot] * 256 + sums[2 * slot + 1];
                    const float value = fmaf(-dmin, static_cast<float>(weighted_min), d * codes);
                    acc[p][slot] = fmaf(scale[slot], value, acc[p][slot]);
                }
            }
        }
    };
    // a class is complete: (c0 + c1) + (c2 + c3) per token goes to LDS
    int parity = 0;
    auto finish_class = [&](int cls) {
#pragma unroll
        for (int slot = 0; slot < S; ++slot) {
            class_sums[parity][cls & (kOwnClasses - 1)][S * h + slot][j] =
                (acc[0][slot] + acc[1][slot]) + (acc[2][slot] + acc[3][slot]);
#pragma unroll
            for (int p = 0; p < 4; ++p) acc[p][slot] = 0.0f;
        }
    };
    // a tile is complete: after the barrier a thread per (token, row) adds the 16 classes in
    // the order of the one-row kernel's butterfly
    std::uint32_t work_tile = first_tile;
    auto finish_tile = [&]() {
        __syncthreads();
        const Projection op = projection_of(work_tile);
        const std::int64_t row0 = static_cast<std::int64_t>(work_tile - op.first_tile) * kRowsTile;
        const int valid_rows =
            static_cast<int>(min(static_cast<std::int64_t>(kRowsTile), op.output_dim - row0));
        const int token = static_cast<int>(threadIdx.x) >> 5;
        if (token < kTokens && token < tokens && j < valid_rows) {
            float pairs[kOwnClasses / 2];
#pragma unroll
            for (int m = 0; m < kOwnClasses / 2; ++m) {
                pairs[m] = class_sums[parity][2 * m][token][j] + class_sums[parity][2 * m + 1][token][j];
            }
            float* output = op.output + (static_cast<std::int64_t>(token) * op.output_dim + row0 + j);
            if constexpr (SPLIT) {
                // this half of the butterfly; the other workgroup's joins it in either order
                // (a compare-and-swap loop: the sum is a vector-ALU addition like every other)
                const float mine = (pairs[0] + pairs[1]) + (pairs[2] + pairs[3]);
                unsigned int* word = reinterpret_cast<unsigned int*>(output);
                unsigned int seen = __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                while (true) {
                    const unsigned int wanted = __float_as_uint(__uint_as_float(seen) + mine);
                    if (__hip_atomic_compare_exchange_strong(word, &seen, wanted, __ATOMIC_RELAXED,
                                                             __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) {
                        break;
                    }
                }
            } else {
                const float q0 = pairs[0] + pairs[1];
                const float q1 = pairs[2] + pairs[3];
                const float q2 = pairs[4] + pairs[5];
                const float q3 = pairs[6] + pairs[7];
                *output = (q0 + q1) + (q2 + q3);
            }
        }
        parity ^= 1;
        work_tile += tile_stride;
    };

    if (total == 0) {
        // (rows of fewer blocks than classes: this wave only takes part in the sums)
        for (int n = 0; n < my_tiles; ++n) {
            finish_class(class0);
            if constexpr (!SPLIT) finish_class(class1);
            finish_tile();
        }
        return;
    }
    // One set of registers for the packed bytes, two named ones for the operands (an array of
    // them indexed in the loop ends up in scratch memory).  A block's loads are requested when
    // the block before has gone to LDS, so one block's arithmetic covers them; the second is
    // requested only when the first has arrived: more requests at the start of a launch make
    // it slower on this chip, not faster.  Past the end of the walk a request repeats the last
    // block, so that the number of loads in flight is the same on every path.
    RowsPacked<ENC> packed;
    RowsOperands even, odd;
    fetch(packed, even);
    // the activation scales of this wave's blocks, 16 tokens each: once into LDS (requested
    // behind the first block's loads, so that nothing waits for them alone)
    for (int index = lane; index < total * 16; index += kWave) {
        const int block = block_of(index >> 4);
        step_scales[wave][index >> 4][index & 15] = reinterpret_cast<const float*>(
            image + static_cast<std::int64_t>(block) * kImageBlock + kImageFragments)[index & 15];
    }
    int work_step = 0;
    // (class0 = wave has at least as many blocks as class1 = 15 - wave; a class without
    // blocks leaves the zeros the sums start from)
    auto finish_step = [&]() {
        if (work_step == count0 - 1) finish_class(class0);
        if (work_step == total - 1) {
            if constexpr (!SPLIT) finish_class(class1);
            finish_tile();
            work_step = 0;
        } else {
            ++work_step;
        }
    };
    const int steps = my_tiles * total;
    for (int step = 0; step < steps; step += 2) {
        stage_to_lds(packed);
        rows_lds_fence();
        fetch(packed, odd);
        compute(even, work_step);
        finish_step();
        if (step + 1 < steps) {
            stage_to_lds(packed);
            rows_lds_fence();
            fetch(packed, even);
            compute(odd, work_step);
            finish_step();
        }
    }
}

std::uint32_t tiles_of(const ProjectionSet& set) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kRowsTile - 1) / kRowsTile);
    }
    return tiles;
}

// How a launch of `tiles` tiles of rows of `blocks` blocks is shared out.  Costs in blocks a
// SIMD works through (two of a workgroup's eight waves to a SIMD, waves w and w + 4): a whole
// tile gives wave w the classes w and 15 - w, the split form the class w (left half) or 8 + w
// (right half); a block and a half per work unit for its first loads, its barrier and its
// stores (measured: 1.1 us a block, 1.6 us a unit at 16 tokens).
struct RowsPlan {
    bool split;
    std::uint32_t left_groups;   // split: workgroups on the left halves
    std::uint32_t groups;        // workgroups of the launch
};

// fill_launch: the outputs are filled by a launch of its own (a prequantized call has no
// quantizer launch to do it), which the split form must win back as well (two blocks' time).
RowsPlan plan_rows(std::uint32_t tiles, std::int64_t input_dim, bool may_split, bool fill_launch = false) {
    const std::uint32_t units = static_cast<std::uint32_t>(compute_units());
    const int blocks = static_cast<int>(input_dim >> 8);
    const auto count = [blocks](int cls) { return cls < blocks ? (blocks - cls + kClasses - 1) / kClasses : 0; };
    int whole = 0, left = 0, right = 0;
    for (int simd = 0; simd < 4; ++simd) {
        const int a = simd, b = simd + 4;
        const int whole_here = count(a) + count(kClasses - 1 - a) + count(b) + count(kClasses - 1 - b);
        const int left_here = count(a) + count(b);
        const int right_here = count(8 + a) + count(8 + b);
        whole = whole_here > whole ? whole_here : whole;
        left = left_here > left ? left_here : left;
        right = right_here > right ? right_here : right;
    }
    const auto passes = [tiles](std::uint32_t groups) { return (tiles + groups - 1) / groups; };
    RowsPlan plan{false, 0, tiles < units ? tiles : units};
    if (!may_split || units < 2) return plan;
    // costs in half blocks
    const std::uint64_t whole_cost = static_cast<std::uint64_t>(passes(plan.groups)) * (2 * whole + 3);
    std::uint64_t best = ~std::uint64_t(0);
    std::uint32_t best_left = 0, best_right = 0;
    for (std::uint32_t left_groups = 1; left_groups < units; ++left_groups) {
        const std::uint32_t l = left_groups < tiles ? left_groups : tiles;
        const std::uint32_t r = units - left_groups < tiles ? units - left_groups : tiles;
        const std::uint64_t left_cost = static_cast<std::uint64_t>(passes(l)) * (2 * left + 3);
        const std::uint64_t right_cost = static_cast<std::uint64_t>(passes(r)) * (2 * right + 3);
        const std::uint64_t cost = left_cost > right_cost ? left_cost : right_cost;
        if (cost < best) {
            best = cost;
            best_left = l;
            best_right = r;
        }
    }
    // (the split form has to win by a tenth: the model is that coarse)
    if (fill_launch) best += 4;
    if (best * 10 <= whole_cost * 9) {
        plan.split = true;
        plan.left_groups = best_left;
        plan.groups = best_left + best_right;
    }
    return plan;
}

template <std::uint32_t ENC, bool SPLIT>
void launch_form(const ProjectionSet& set, const std::uint8_t* image, int tokens, std::uint32_t tiles,
                 const RowsPlan& plan, hipStream_t stream) {
    const dim3 grid(plan.groups), block(kRowsThreads);
    const int input_dim = static_cast<int>(set.input_dim);
    if (tokens <= 4) {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 2, SPLIT>), grid, block, 0, stream, image, tokens,
                           input_dim, tiles, plan.left_groups, set);
    } else if (tokens <= 8) {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 4, SPLIT>), grid, block, 0, stream, image, tokens,
                           input_dim, tiles, plan.left_groups, set);
    } else {
        hipLaunchKernelGGL((gemv_rows_kernel<ENC, 8, SPLIT>), grid, block, 0, stream, image, tokens,
                           input_dim, tiles, plan.left_groups, set);
    }
}

template <std::uint32_t ENC>
void launch_encoding(ProjectionSet set, const std::uint8_t* image, int tokens, bool outputs_cleared,
                     bool fill_launch, hipStream_t stream) {
    std::uint32_t tiles = 0;
    for (int index = 0; index < set.count; ++index) {
        set.op[index].first_tile = tiles;
        tiles += static_cast<std::uint32_t>((set.op[index].output_dim + kRowsTile - 1) / kRowsTile);
    }
    const RowsPlan plan = plan_rows(tiles, set.input_dim, outputs_cleared, fill_launch);
    if (plan.split) {
        launch_form<ENC, true>(set, image, tokens, tiles, plan, stream);
    } else {
        launch_form<ENC, false>(set, image, tokens, tiles, plan, stream);
    }
}

// the projections of one encoding, in the order of the set
ProjectionSet encoding_group(const ProjectionSet& set, std::uint32_t encoding) {
    ProjectionSet group{};
    group.input_dim = set.input_dim;
    for (int index = 0; index < set.count; ++index) {
        if (set.op[index].encoding == encoding) group.op[group.count++] = set.op[index];
    }
    return group;
}

constexpr std::uint32_t kRowsEncodings[4] = {kEncQ4K, kEncQ5K, kEncQ6K, kEncQ8_0};

}  // namespace

bool gemv_rows_supports(std::uint32_t encoding, std::int64_t input_dim) {
    return (encoding == kEncQ4K || encoding == kEncQ5K || encoding == kEncQ6K || encoding == kEncQ8_0) &&
        input_dim % 256 == 0 && input_dim <= kMaxRowsBlocks * 256;
}

std::int64_t gemv_rows_image_bytes(std::int64_t input_dim) {
    return (input_dim >> 8) * kImageBlock;
}

ProjectionSet gemv_rows_split_set(const ProjectionSet& set, bool fill_launch) {
    ProjectionSet split{};
    split.input_dim = set.input_dim;
    for (const std::uint32_t encoding : kRowsEncodings) {
        const ProjectionSet group = encoding_group(set, encoding);
        if (group.count == 0 || !plan_rows(tiles_of(group), set.input_dim, true, fill_launch).split) continue;
        for (int index = 0; index < group.count; ++index) split.op[split.count++] = group.op[index];
    }
    return split;
}

void launch_quantize_records(const float* first, const float* second, int prologue,
                             std::int64_t rows, std::int64_t input_dim, std::uint8_t* records,
                             std::uint8_t* image, const ProjectionSet& clear, hipStream_t stream) {
    const int blocks = static_cast<int>(input_dim >> 8);
    const int tokens = static_cast<int>(rows);
    const int record_groups = (blocks * tokens + 3) / 4;
    std::int64_t fill_groups = 0;
    for (int index = 0; index < clear.count; ++index) {
        fill_groups += (clear.op[index].output_dim * rows + 1023) >> 10;
    }
    const dim3 grid(static_cast<unsigned>(record_groups + fill_groups)), block(256);
    switch (prologue) {
        case kGated:
            hipLaunchKernelGGL((quantize_records_kernel<kGated>), grid, block, 0, stream, first,
                               second, records, image, blocks, tokens, record_groups, clear);
            break;
        case kSwiGlu:
            hipLaunchKernelGGL((quantize_records_kernel<kSwiGlu>), grid, block, 0, stream, first,
                               second, records, image, blocks, tokens, record_groups, clear);
            break;
        default:
            hipLaunchKernelGGL((quantize_records_kernel<kPlain>), grid, block, 0, stream, first,
                               second, records, image, blocks, tokens, record_groups, clear);
            break;
    }
}

void launch_fill_outputs(const ProjectionSet& clear, std::int64_t rows, hipStream_t stream) {
    std::int64_t fill_groups = 0;
    for (int index = 0; index < clear.count; ++index) {
        fill_groups += (clear.op[index].output_dim * rows + 1023) >> 10;
    }
    if (fill_groups == 0) return;
    // (the quantizer kernel with no records to write)
    hipLaunchKernelGGL((quantize_records_kernel<kPlain>), dim3(static_cast<unsigned>(fill_groups)),
                       dim3(256), 0, stream, static_cast<const float*>(nullptr),
                       static_cast<const float*>(nullptr), static_cast<std::uint8_t*>(nullptr),
                       static_cast<std::uint8_t*>(nullptr), 0, static_cast<int>(rows), 0, clear);
}

void launch_gemv_rows(const ProjectionSet& set, const std::uint8_t* image, std::int64_t rows,
                      bool outputs_cleared, bool fill_launch, hipStream_t stream) {
    for (const std::uint32_t encoding : kRowsEncodings) {
        const ProjectionSet group = encoding_group(set, encoding);
        if (group.count == 0) continue;
        const int tokens = static_cast<int>(rows);
        switch (encoding) {
            case kEncQ4K: launch_encoding<kEncQ4K>(group, image, tokens, outputs_cleared, fill_launch, stream); break;
            case kEncQ5K: launch_encoding<kEncQ5K>(group, image, tokens, outputs_cleared, fill_launch, stream); break;
            case kEncQ6K: launch_encoding<kEncQ6K>(group, image, tokens, outputs_cleared, fill_launch, stream); break;
            default: launch_encoding<kEncQ8_0>(group, image, tokens, outputs_cleared, fill_launch, stream); break;
        }
    }
}

}  // namespace nfn
