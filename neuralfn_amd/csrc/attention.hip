// Attention of the decode loop over a bf16 key/value cache: the one-token
// grouped-query form and the block form of the verifier and the proposal
// model (semantics: neuralfn/csrc/native_train/tile_ops.h:308-339, 445-486;
// reference kernels: neuralfn/csrc/tile_cuda/kernels.cu:2475-2824, 2924-3075).
//
// One workgroup per (query row, query head), up to eight waves.  A wave takes
// every active-th tile of 64 keys, keeps a running (maximum, denominator,
// accumulator), and the workgroup merges the waves through LDS at the end.
// The query sits in LDS and is read as a broadcast.  Two kernels: a vector
// form for head sizes that are multiples of 32 (everything in 16-byte pieces,
// all loads of a phase in flight together) and a generic element-wise form.
// The one-token form is the block form with one query row whose own key is
// the only block row.  A third kernel serves head_dim 128 with four or more
// query heads per key/value head on the matrix cores, one workgroup per group
// of up to 16 such heads: the split one-token form and blocks of many rows.
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

constexpr int kMaxWaves = 8;   // 512 threads: 256 vector registers per lane
constexpr int kMaxHeadDim = 256;
constexpr int kMaxSplits = 128;    // most shares of one head's keys in the split form
constexpr int kVectorSplits = 32;  // ... when every query head has workgroups of its own
constexpr int kOwned = kMaxHeadDim / kWave;  // output dimensions per lane

struct AttentionArguments {
    const float* query;
    const float* block_key;
    const float* block_value;
    const std::uint16_t* key_cache;
    const std::uint16_t* value_cache;
    float* output;
    std::int64_t query_heads;
    std::int64_t kv_heads;
    std::int64_t head_dim;
    std::uint32_t heads_per_kv;  // query_heads / kv_heads
    std::int64_t context_length;
    std::int64_t block_rows;
    std::int64_t sliding_window;
    std::int64_t cache_capacity;
    std::int64_t cache_row_stride;
    float scale;
    int causal;
    // Split form: workgroup (x, y) takes the y-th of `splits` shares of the row's
    // tiles and leaves (maximum, denominator, accumulator) in `partials`
    // instead of an output row; null for the ordinary form.
    float* partials;
    int splits;
    // One-token form with the position in device memory (read when the kernel
    // runs, so that one captured graph serves every token): context_length is
    // *device_position and the window is `sliding_window` keys, or everything
    // from key 0 when `whole_context`.  Null for a position known at launch.
    const std::int64_t* device_position;
    int whole_context;
};

// Resolves a device-side position into the fields the kernels work with.
__device__ __forceinline__ void resolve_position(AttentionArguments& a) {
    if (a.device_position == nullptr) return;
    const std::int64_t position = a.device_position[0];
    a.context_length = position;
    if (a.whole_context) a.sliding_window = position + 1;
}

// floats per (query row, query head, split) in the partial buffer
__host__ __device__ constexpr std::int64_t partial_floats(std::int64_t head_dim) {
    return head_dim + 2;
}

__device__ __forceinline__ float wave_max_f(float value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        value = fmaxf(value, __shfl_xor(value, offset));
    }
    return value;
}

__device__ __forceinline__ float wave_sum_f(float value) {
#pragma unroll
    for (int offset = 32; offset > 0; offset >>= 1) {
        value += __shfl_xor(value, offset);
    }
    return value;
}

// ---------------------------------------------------------------------------
// Generic form: any head_dim, any alignment; element-wise loads.  A lane owns
// one key for the scores and the output dimensions lane, lane + 64, ... for
// the weighted sum.
// ---------------------------------------------------------------------------
__device__ __forceinline__ float score_cache_key(const float* q, const std::uint16_t* key,
                                                 int head_dim) {
    float dot = 0.0f;
    for (int d = 0; d < head_dim; ++d) dot = fmaf(q[d], bf16_to_float(key[d]), dot);
    return dot;
}

__device__ __forceinline__ float score_block_key(const float* q, const float* key, int head_dim,
                                                 bool as_cached) {
    float dot = 0.0f;
    for (int d = 0; d < head_dim; ++d) {
        float k = key[d];
        if (as_cached) k = bf16_to_float(to_bf16(k));
        dot = fmaf(q[d], k, dot);
    }
    return dot;
}

// The key range of one query row, and how many waves share it.  The split
// depends on the row's key count only, not on the launch: a row of a causal
// block then sums in the same order as the one-token call at the same
// position, and gives the same bits.
struct KeyRange {
    std::int64_t first, last;
    int active;
};

__device__ __forceinline__ KeyRange key_range(const AttentionArguments& a, std::int64_t query_row,
                                              int waves) {
    const std::int64_t query_position = a.context_length + query_row;
    const bool causal = a.causal != 0;
    KeyRange range;
    range.first = query_position - a.sliding_window + (causal ? 1 : 0);
    if (range.first < 0) range.first = 0;
    range.last = query_position;
    if (!causal) {
        const std::int64_t end = a.context_length + a.block_rows - 1;
        range.last =
            a.sliding_window < end - query_position ? query_position + a.sliding_window : end;
    }
    std::int64_t tiles = (range.last - range.first) / kWave + 1;
    if (a.partials != nullptr) {
        // this workgroup's share: whole tiles, contiguous; an empty share has last < first
        const std::int64_t share = (tiles + a.splits - 1) / a.splits;
        const std::int64_t begin = static_cast<std::int64_t>(blockIdx.y) * share;
        const std::int64_t end = begin + share < tiles ? begin + share : tiles;
        const std::int64_t share_last = range.first + end * kWave - 1;
        range.first += begin * kWave;
        if (share_last < range.last) range.last = share_last;
        tiles = end > begin ? end - begin : 0;
    }
    range.active = static_cast<int>(tiles < waves ? tiles : waves);
    return range;
}

__global__ __launch_bounds__(kMaxWaves * kWave) void attention_generic_kernel(AttentionArguments a) {
    __shared__ __attribute__((aligned(16))) float q[kMaxHeadDim];
    __shared__ float wave_maximum[kMaxWaves];
    __shared__ float wave_denominator[kMaxWaves];
    __shared__ float wave_accumulator[kMaxWaves][kMaxHeadDim];

    resolve_position(a);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int head_dim = static_cast<int>(a.head_dim);
    // query_heads and the grid fit 32 bits (checked by the caller): no 64-bit division
    const std::uint32_t heads = static_cast<std::uint32_t>(a.query_heads);
    const std::int64_t query_row = blockIdx.x / heads;
    const std::int64_t query_head = blockIdx.x % heads;
    const std::int64_t kv_head = static_cast<std::uint32_t>(query_head) / a.heads_per_kv;
    const bool causal = a.causal != 0;
    const KeyRange range = key_range(a, query_row, waves);
    const std::int64_t last = range.last;
    const int active = range.active;

    const float* query = a.query + (query_row * a.query_heads + query_head) * a.head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) q[d] = query[d];
    __syncthreads();

    float maximum = -INFINITY;
    float denominator = 0.0f;
    float accumulator[kOwned];
#pragma unroll
    for (int j = 0; j < kOwned; ++j) accumulator[j] = 0.0f;

    for (std::int64_t tile = range.first + static_cast<std::int64_t>(wave) * kWave;
         wave < active && tile <= last; tile += static_cast<std::int64_t>(active) * kWave) {
        const std::int64_t key_position = tile + lane;
        const bool live = key_position <= last;
        float score = -INFINITY;
        if (live) {
            if (key_position >= a.context_length) {
                const std::int64_t block_row = key_position - a.context_length;
                const float* key = a.block_key + (block_row * a.kv_heads + kv_head) * a.head_dim;
                score = score_block_key(q, key, head_dim, causal && block_row < query_row);
            } else {
                const std::uint16_t* key = a.key_cache +
                    (key_position % a.cache_capacity) * a.cache_row_stride + kv_head * a.head_dim;
                score = score_cache_key(q, key, head_dim);
            }
            score *= a.scale;
        }
        // the tile has at least one live key, so its maximum is finite
        const float next_maximum = fmaxf(maximum, wave_max_f(score));
        const float keep = expf(maximum - next_maximum);  // 0 on the first tile
        const float weight = live ? expf(score - next_maximum) : 0.0f;
        denominator = denominator * keep + wave_sum_f(weight);
#pragma unroll
        for (int j = 0; j < kOwned; ++j) accumulator[j] *= keep;
        maximum = next_maximum;

        const int count = static_cast<int>(last - tile + 1 < kWave ? last - tile + 1 : kWave);
        for (int k = 0; k < count; ++k) {
            const float weight_k = __uint_as_float(
                __builtin_amdgcn_readlane(__float_as_uint(weight), k));
            const std::int64_t position = tile + k;
            if (position >= a.context_length) {
                const std::int64_t block_row = position - a.context_length;
                const float* value =
                    a.block_value + (block_row * a.kv_heads + kv_head) * a.head_dim;
                const bool as_cached = causal && block_row < query_row;
#pragma unroll
                for (int j = 0; j < kOwned; ++j) {
                    const int d = lane + j * kWave;
                    if (d < head_dim) {
                        float v = value[d];
                        if (as_cached) v = bf16_to_float(to_bf16(v));
                        accumulator[j] = fmaf(weight_k, v, accumulator[j]);
                    }
                }
            } else {
                const std::uint16_t* value = a.value_cache +
                    (position % a.cache_capacity) * a.cache_row_stride + kv_head * a.head_dim;
#pragma unroll
                for (int j = 0; j < kOwned; ++j) {
                    const int d = lane + j * kWave;
                    if (d < head_dim) {
                        accumulator[j] = fmaf(weight_k, bf16_to_float(value[d]), accumulator[j]);
                    }
                }
            }
        }
    }

    if (lane == 0) {
        wave_maximum[wave] = maximum;
        wave_denominator[wave] = denominator;
    }
#pragma unroll
    for (int j = 0; j < kOwned; ++j) {
        const int d = lane + j * kWave;
        if (d < head_dim) wave_accumulator[wave][d] = accumulator[j];
    }
    __syncthreads();

    // merge the active waves: each of them had at least one tile, so every
    // maximum is finite
    float overall = wave_maximum[0];
    for (int w = 1; w < active; ++w) overall = fmaxf(overall, wave_maximum[w]);
    float total = 0.0f;
    for (int w = 0; w < active; ++w) {
        total = fmaf(wave_denominator[w], expf(wave_maximum[w] - overall), total);
    }
    float* output = a.output + (query_row * a.query_heads + query_head) * a.head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) {
        float sum = 0.0f;
        for (int w = 0; w < active; ++w) {
            sum = fmaf(wave_accumulator[w][d], expf(wave_maximum[w] - overall), sum);
        }
        output[d] = sum / total;
    }
}

// ---------------------------------------------------------------------------
// Vector form: head_dim 32, 64, 128 or 256, rows 16-byte aligned, a ring of at
// least 64 rows.  Everything moves in 16-byte pieces.  Scores: a lane owns one
// key and reads its head_dim / 8 pieces.  Weighted sum: LANES_PER_KEY =
// head_dim / 8 lanes share a value row; lane (g, i) = (lane / LANES_PER_KEY,
// lane % LANES_PER_KEY) owns dimensions 8i .. 8i+7 of the keys g, g + G,
// g + 2G ... of the tile (G = 64 / LANES_PER_KEY keys per load instruction),
// so a tile's values arrive with LANES_PER_KEY load instructions; the G
// partial sums of a dimension meet in a butterfly once, after the last tile.
// A tile that lies wholly in the cache (all but the last one or two of a row)
// runs straight-line code with up to sixteen loads per lane in flight; a tile
// that holds block rows takes the same sums in the same order through a
// slower path that can fetch either kind of row.
// ---------------------------------------------------------------------------
struct Piece {
    float v[8];
};

__device__ __forceinline__ Piece unpack_bf16(uint4 packed) {
    Piece p;
    p.v[0] = __uint_as_float(packed.x << 16);
    p.v[1] = __uint_as_float(packed.x & 0xffff0000u);
    p.v[2] = __uint_as_float(packed.y << 16);
    p.v[3] = __uint_as_float(packed.y & 0xffff0000u);
    p.v[4] = __uint_as_float(packed.z << 16);
    p.v[5] = __uint_as_float(packed.z & 0xffff0000u);
    p.v[6] = __uint_as_float(packed.w << 16);
    p.v[7] = __uint_as_float(packed.w & 0xffff0000u);
    return p;
}

__device__ __forceinline__ Piece from_floats(float4 low, float4 high, bool as_cached) {
    Piece p = {{low.x, low.y, low.z, low.w, high.x, high.y, high.z, high.w}};
    if (as_cached) {
#pragma unroll
        for (int e = 0; e < 8; ++e) p.v[e] = bf16_to_float(to_bf16(p.v[e]));
    }
    return p;
}

__device__ __forceinline__ float dot_piece(const float* q, const Piece& p, float dot) {
    const float4 q0 = *reinterpret_cast<const float4*>(q);
    const float4 q1 = *reinterpret_cast<const float4*>(q + 4);
    dot = fmaf(q0.x, p.v[0], dot);
    dot = fmaf(q0.y, p.v[1], dot);
    dot = fmaf(q0.z, p.v[2], dot);
    dot = fmaf(q0.w, p.v[3], dot);
    dot = fmaf(q1.x, p.v[4], dot);
    dot = fmaf(q1.y, p.v[5], dot);
    dot = fmaf(q1.z, p.v[6], dot);
    dot = fmaf(q1.w, p.v[7], dot);
    return dot;
}

// Ties two values together for the compiler: whatever is computed from either after this
// point cannot be scheduled before both have their values here.  (Used to bound how many
// registers a long unrolled stretch holds at once.)
template <typename A, typename B>
__device__ __forceinline__ void tie(A& first, B& second) {
    asm volatile("" : "+v"(first), "+v"(second));
    __builtin_amdgcn_sched_barrier(0);
}

template <int LANES_PER_KEY>
__global__ __launch_bounds__(kMaxWaves * kWave) void attention_vector_kernel(AttentionArguments a) {
    constexpr int kPieces = LANES_PER_KEY;             // head_dim / 8
    constexpr int kKeysPerLoad = kWave / LANES_PER_KEY;
    __shared__ __attribute__((aligned(16))) float q[kMaxHeadDim];
    __shared__ float wave_maximum[kMaxWaves];
    __shared__ float wave_denominator[kMaxWaves];
    __shared__ __attribute__((aligned(16))) float wave_accumulator[kMaxWaves][kMaxHeadDim];

    resolve_position(a);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    constexpr int head_dim = kPieces * 8;
    // query_heads and the grid fit 32 bits (checked by the caller): no 64-bit division
    const std::uint32_t heads = static_cast<std::uint32_t>(a.query_heads);
    const std::int64_t query_row = blockIdx.x / heads;
    const std::int64_t query_head = blockIdx.x % heads;
    const std::int64_t kv_head = static_cast<std::uint32_t>(query_head) / a.heads_per_kv;
    const bool causal = a.causal != 0;
    const KeyRange range = key_range(a, query_row, waves);
    const std::int64_t last = range.last;
    const int active = range.active;
    const std::int64_t head_offset = kv_head * head_dim;
    const std::int64_t block_stride = a.kv_heads * head_dim;

    const float* query = a.query + (query_row * a.query_heads + query_head) * head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) q[d] = query[d];
    __syncthreads();

    // Ring rows without a division per key: the slot of a wave's first tile and
    // of its tile-to-tile step are computed once, the rest is compare-and-subtract
    // (the ring has at least 64 rows here).
    const std::int64_t capacity = a.cache_capacity;
    const std::int64_t tile_step = static_cast<std::int64_t>(active) * kWave;
    const std::int64_t slot_step = tile_step % capacity;
    std::int64_t tile_slot = (range.first + static_cast<std::int64_t>(wave) * kWave) % capacity;
    const auto ring_row = [capacity](std::int64_t slot) {  // slot < 2 * capacity
        return slot >= capacity ? slot - capacity : slot;
    };

    const int group = lane / LANES_PER_KEY;  // which key of a load instruction
    const int piece = lane % LANES_PER_KEY;  // which 8 dimensions

    float maximum = -INFINITY;
    float denominator = 0.0f;
    float accumulator[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) accumulator[e] = 0.0f;

    // running maximum, denominator and accumulator take in a tile's scores;
    // returns this lane's weight exp(score - maximum)
    const auto fold = [&](float raw_score, bool live) {
        const float score = live ? raw_score * a.scale : -INFINITY;
        const float next_maximum = fmaxf(maximum, wave_max_f(score));
        const float keep = expf(maximum - next_maximum);  // 0 on the first tile
        const float weight = live ? expf(score - next_maximum) : 0.0f;
        denominator = denominator * keep + wave_sum_f(weight);
#pragma unroll
        for (int e = 0; e < 8; ++e) accumulator[e] *= keep;
        maximum = next_maximum;
        return weight;
    };
    // this lane's 8 dimensions of the cached value row of key k of the tile whose first
    // row is ring slot `slot` (keys past the range repeat the last one)
    const auto cached_value_piece = [&](std::int64_t slot, int k, int in_tile) {
        const int clamped = k < in_tile ? k : in_tile;
        return reinterpret_cast<const uint4*>(
            a.value_cache + ring_row(slot + clamped) * a.cache_row_stride + head_offset)[piece];
    };

    // Scores: lane = key.  Weighted sum: lane = (key of the load, 8 dimensions);
    // every form adds the keys of the tile in the same order, key g, g + G, ...
    std::int64_t tile = range.first + static_cast<std::int64_t>(wave) * kWave;

    // A wave's tiles that lie wholly in the cache come first.  Keys and values of such a
    // tile are requested before anything of it is used, and the keys of the next such
    // tile (if it is a full one) while the weighted sum of the current one runs.
    if constexpr (kPieces <= 16) {
        uint4 key_raw[kPieces];
        bool requested_ahead = false;  // wave-uniform
        // bytes from a load's first value row to this lane's 8 dimensions (fits 32 bits:
        // the launcher bounds the row stride)
        const std::uint32_t value_lane_offset =
            static_cast<std::uint32_t>(group) * static_cast<std::uint32_t>(a.cache_row_stride) * 2u +
            static_cast<std::uint32_t>(piece) * 16u;
        for (; wave < active && tile <= last && tile + kWave - 1 < a.context_length;
             tile += tile_step, tile_slot = ring_row(tile_slot + slot_step)) {
            const int in_tile = static_cast<int>(last - tile < kWave - 1 ? last - tile : kWave - 1);
            const bool live = lane <= in_tile;
            const int my_key = live ? lane : in_tile;
            uint4 value_raw[kPieces];
            if (!requested_ahead) {
                const uint4* key = reinterpret_cast<const uint4*>(
                    a.key_cache + ring_row(tile_slot + my_key) * a.cache_row_stride + head_offset);
#pragma unroll
                for (int u = 0; u < kPieces; ++u) key_raw[u] = key[u];
            }
            if (in_tile == kWave - 1 && tile_slot + kWave <= capacity) {
                // a full tile that does not wrap: one wave-uniform row address per load
                // and the same 32-bit lane offset for all of them
                const char* rows = reinterpret_cast<const char*>(
                    a.value_cache + tile_slot * a.cache_row_stride + head_offset);
                const std::int64_t load_stride = kKeysPerLoad * a.cache_row_stride * 2;
#pragma unroll
                for (int u = 0; u < kPieces; ++u) {
                    value_raw[u] = *reinterpret_cast<const uint4*>(rows + u * load_stride +
                                                                   value_lane_offset);
                }
            } else {
#pragma unroll
                for (int u = 0; u < kPieces; ++u) {
                    value_raw[u] = cached_value_piece(tile_slot, u * kKeysPerLoad + group, in_tile);
                }
            }
            // the query comes out of shared memory a few pieces at a time (all of it at
            // once would take as many registers as the tile's keys and values together)
            // (four pieces at a time; the offset, tied to the running score, keeps the
            // compiler from holding the whole query in registers)
            int query_offset = 0;
            float score = 0.0f;
#pragma unroll
            for (int u = 0; u < kPieces; ++u) {
                if (u % 4 == 0) tie(query_offset, score);
                score = dot_piece(q + query_offset + u * 8, unpack_bf16(key_raw[u]), score);
            }
            const std::int64_t next_end = tile + tile_step + kWave - 1;
            requested_ahead = next_end <= last && next_end < a.context_length;
            // the next keys go into the registers the scores have just freed: their loads
            // must come after the last use of the current keys
            int next_lane = lane;
            tie(next_lane, score);
            if (requested_ahead) {
                const uint4* next_key = reinterpret_cast<const uint4*>(
                    a.key_cache +
                    ring_row(ring_row(tile_slot + slot_step) + next_lane) * a.cache_row_stride +
                    head_offset);
#pragma unroll
                for (int u = 0; u < kPieces; ++u) key_raw[u] = next_key[u];
            }
            const float weight = fold(score, live);
            float weight_of[kPieces];
#pragma unroll
            for (int u = 0; u < kPieces; ++u) {
                weight_of[u] = __shfl(weight, u * kKeysPerLoad + group);
            }
            // values are unpacked a few loads at a time: unpacking all of them at once
            // would not fit the registers beside the keys requested ahead
#pragma unroll
            for (int u = 0; u < kPieces; ++u) {
                if (u % 2 == 0) tie(value_raw[u].x, accumulator[0]);
                const Piece value = unpack_bf16(value_raw[u]);
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    accumulator[e] = fmaf(weight_of[u], value.v[e], accumulator[e]);
                }
            }
        }
    }

    // The remaining tiles: those that hold rows of the block, and with more than 128
    // dimensions a head also the cached ones (16 loads in flight at a time).
    for (; wave < active && tile <= last;
         tile += tile_step, tile_slot = ring_row(tile_slot + slot_step)) {
        // Keys past the range repeat the last key of the tile with weight 0.
        const int in_tile = static_cast<int>(last - tile < kWave - 1 ? last - tile : kWave - 1);
        const bool live = lane <= in_tile;
        const int my_key = live ? lane : in_tile;
        const bool cache_only = tile + kWave - 1 < a.context_length;  // wave-uniform

        if (kPieces > 16 && cache_only) {
            const uint4* key = reinterpret_cast<const uint4*>(
                a.key_cache + ring_row(tile_slot + my_key) * a.cache_row_stride + head_offset);
            float score = 0.0f;
            int query_offset = 0;
#pragma unroll
            for (int c = 0; c < kPieces; c += 16) {
                uint4 raw[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) raw[u] = key[c + u];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    if (u % 4 == 0) tie(query_offset, score);
                    score = dot_piece(q + query_offset + (c + u) * 8, unpack_bf16(raw[u]), score);
                }
            }
            const float weight = fold(score, live);
#pragma unroll
            for (int t0 = 0; t0 < kPieces; t0 += 16) {
                uint4 raw[16];
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    raw[u] = cached_value_piece(tile_slot, (t0 + u) * kKeysPerLoad + group, in_tile);
                }
#pragma unroll
                for (int u = 0; u < 16; ++u) {
                    const float weight_k = __shfl(weight, (t0 + u) * kKeysPerLoad + group);
                    const Piece value = unpack_bf16(raw[u]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        accumulator[e] = fmaf(weight_k, value.v[e], accumulator[e]);
                    }
                }
            }
        } else {
            float score = 0.0f;
            int query_offset = 0;
            const std::int64_t key_position = tile + my_key;
            if (key_position >= a.context_length) {
                const std::int64_t block_row = key_position - a.context_length;
                const float4* key = reinterpret_cast<const float4*>(
                    a.block_key + block_row * block_stride + head_offset);
                const bool as_cached = causal && block_row < query_row;
                for (int c = 0; c < kPieces; c += 4) {
                    float4 raw[8];
#pragma unroll
                    for (int u = 0; u < 8; ++u) raw[u] = key[2 * c + u];
                    tie(query_offset, score);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        score = dot_piece(q + query_offset + (c + u) * 8,
                                          from_floats(raw[2 * u], raw[2 * u + 1], as_cached), score);
                    }
                }
            } else {
                const uint4* key = reinterpret_cast<const uint4*>(
                    a.key_cache + ring_row(tile_slot + my_key) * a.cache_row_stride + head_offset);
                for (int c = 0; c < kPieces; c += 4) {
                    uint4 raw[4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) raw[u] = key[c + u];
                    tie(query_offset, score);
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        score = dot_piece(q + query_offset + (c + u) * 8, unpack_bf16(raw[u]), score);
                    }
                }
            }
            const float weight = fold(score, live);
            for (int t0 = 0; t0 < kPieces; t0 += 4) {
                if (t0 * kKeysPerLoad > in_tile) break;  // wave-uniform: only dead keys left
                uint4 cached[4];
                float4 low[4], high[4];
                float weights[4];
                bool from_block[4], as_cached[4];
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int k = (t0 + u) * kKeysPerLoad + group;
                    const int clamped = k < in_tile ? k : in_tile;
                    const std::int64_t position = tile + clamped;
                    weights[u] = __shfl(weight, k);
                    from_block[u] = position >= a.context_length;
                    const std::int64_t block_row = from_block[u] ? position - a.context_length : 0;
                    as_cached[u] = causal && block_row < query_row;
                    const std::int64_t slot = from_block[u] ? 0 : ring_row(tile_slot + clamped);
                    cached[u] = reinterpret_cast<const uint4*>(
                        a.value_cache + slot * a.cache_row_stride + head_offset)[piece];
                    const float4* row = reinterpret_cast<const float4*>(
                        a.block_value + block_row * block_stride + head_offset);
                    low[u] = row[2 * piece];
                    high[u] = row[2 * piece + 1];
                }
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const Piece from_cache = unpack_bf16(cached[u]);
                    const Piece block = from_floats(low[u], high[u], as_cached[u]);
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float value = from_block[u] ? block.v[e] : from_cache.v[e];
                        accumulator[e] = fmaf(weights[u], value, accumulator[e]);
                    }
                }
            }
        }
    }

    // the partial sums of the key groups meet; group 0 ends up with the totals
#pragma unroll
    for (int offset = LANES_PER_KEY; offset < kWave; offset <<= 1) {
#pragma unroll
        for (int e = 0; e < 8; ++e) accumulator[e] += __shfl_xor(accumulator[e], offset);
    }
    if (lane == 0) {
        wave_maximum[wave] = maximum;
        wave_denominator[wave] = denominator;
    }
    if (group == 0) {
        float* target = &wave_accumulator[wave][piece * 8];
        *reinterpret_cast<float4*>(target) =
            make_float4(accumulator[0], accumulator[1], accumulator[2], accumulator[3]);
        *reinterpret_cast<float4*>(target + 4) =
            make_float4(accumulator[4], accumulator[5], accumulator[6], accumulator[7]);
    }
    __syncthreads();

    float overall = active > 0 ? wave_maximum[0] : -INFINITY;
    for (int w = 1; w < active; ++w) overall = fmaxf(overall, wave_maximum[w]);
    float total = 0.0f;
    for (int w = 0; w < active; ++w) {
        total = fmaf(wave_denominator[w], expf(wave_maximum[w] - overall), total);
    }
    if (a.partials != nullptr) {
        // unnormalised, relative to this share's maximum; an empty share says (-inf, 0, 0)
        float* partial = a.partials +
            ((query_row * a.query_heads + query_head) * a.splits + blockIdx.y) *
                partial_floats(head_dim);
        if (tid == 0) {
            partial[0] = overall;
            partial[1] = total;
        }
        for (int d = tid; d < head_dim; d += blockDim.x) {
            float sum = 0.0f;
            for (int w = 0; w < active; ++w) {
                sum = fmaf(wave_accumulator[w][d], expf(wave_maximum[w] - overall), sum);
            }
            partial[2 + d] = sum;
        }
        return;
    }
    float* output = a.output + (query_row * a.query_heads + query_head) * head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) {
        float sum = 0.0f;
        for (int w = 0; w < active; ++w) {
            sum = fmaf(wave_accumulator[w][d], expf(wave_maximum[w] - overall), sum);
        }
        output[d] = sum / total;
    }
}

// Split form, second launch: one workgroup per (query row, query head) merges
// the shares.  Four threads share an output dimension and take every fourth
// share each, so that the loads of many shares are in flight together (read
// one after the other, 32 shares cost more than the attention itself).
constexpr int kMergeLanes = 4;

__global__ __launch_bounds__(kMaxHeadDim * kMergeLanes) void attention_merge_kernel(
    const float* __restrict__ partials, float* __restrict__ output, int splits, int head_dim) {
    __shared__ float factor[kMaxSplits];
    __shared__ float wave_part[2][kMaxHeadDim * kMergeLanes / kWave];
    __shared__ float lane_sum[kMergeLanes][kMaxHeadDim];
    const std::int64_t stride = partial_floats(head_dim);
    const float* mine = partials + static_cast<std::int64_t>(blockIdx.x) * splits * stride;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int dims = static_cast<int>(blockDim.x) / kMergeLanes;  // head_dim rounded up to waves

    // thread s holds share s (at most 128 shares, at least 256 threads)
    const float maximum = tid < splits ? mine[tid * stride] : -INFINITY;
    const float denominator = tid < splits ? mine[tid * stride + 1] : 0.0f;
    const float wave_maximum = wave_max_f(maximum);
    if (lane == 0) wave_part[0][wave] = wave_maximum;
    __syncthreads();
    const float overall = fmaxf(wave_part[0][0], wave_part[0][1]);
    const float mine_factor = expf(maximum - overall);  // 0 for an empty share
    if (tid < splits) factor[tid] = mine_factor;
    const float wave_total = wave_sum_f(denominator * mine_factor);
    if (lane == 0) wave_part[1][wave] = wave_total;
    __syncthreads();
    const float total = wave_part[1][0] + wave_part[1][1];

    const int d = tid % dims;
    const int share_lane = tid / dims;
    float sum = 0.0f;
    if (d < head_dim) {
#pragma unroll 4
        for (int s = share_lane; s < splits; s += kMergeLanes) {
            sum = fmaf(mine[s * stride + 2 + d], factor[s], sum);
        }
    }
    lane_sum[share_lane][d] = sum;
    __syncthreads();
    if (share_lane == 0 && d < head_dim) {
        const float all = (lane_sum[0][d] + lane_sum[1][d]) + (lane_sum[2][d] + lane_sum[3][d]);
        output[static_cast<std::int64_t>(blockIdx.x) * head_dim + d] = all / total;
    }
}

// ---------------------------------------------------------------------------
// Grouped form on the matrix cores (head_dim 128): one workgroup per (query row,
// key/value head, group of up to 16 of its query heads[, share of the keys]).
// All query heads of a group read a key/value row once.  Same semantics as the
// vector kernel for one-token calls and blocks, with or without the split.
//
// Lane = (j, i) = (lane / 16, lane % 16).  Both products run on
// v_mfma_f32_16x16x32_bf16 with float operands cut into three bf16 terms whose sum
// is the float, so that every product is exact (cache rows are bf16 already).
//
// Scores of 16 keys x 16 heads, one accumulator per 32 dimensions: operand A is the
// cached key as it lies in memory (lane (j, i): key i, dimensions 8j..8j+7 of the
// 32), operand B the query of head i.  The result leaves lane (j, i) with keys
// 4j..4j+3 of head i, for four blocks of 16 keys a tile.
//
// Weighted sum over 32 keys at a time: operand A is the weights of head i as the
// lane holds them (the instruction's k index 8j + e read as "key 4j + e % 4 of
// block e / 4" of the 32), operand B wants, for one dimension, the values of those
// eight keys -- a column of the cache.  A wave therefore stages its tile's value
// rows in LDS (rows of 272 bytes: a row's 256 and a pad that spreads the four j
// over the banks) and reads them back a dword at a time: dimensions 2i and 2i + 1
// of a key, whose halves go to two instructions (column i standing for dimension
// 32p + 2i in one and 32p + 2i + 1 in the other).
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kGroupWaves = 8;
constexpr int kGroupHeads = 16;
constexpr int kGroupHeadDim = 128;
constexpr int kGroupRowPad = 4;  // floats between the rows of a wave's result in LDS
constexpr int kStageRowBytes = 2 * kGroupHeadDim + 16;  // a staged value row and its pad
constexpr int kStageBytes = kWave * kStageRowBytes;      // a wave's tile of value rows
constexpr int kGroupMinHeads = 4;  // fewer query heads per key/value head: the vector form

struct QueryTerms {
    bf16x8 high, middle, low;
};

// x = high + middle + low exactly, every term a bf16: each term takes the next eight
// significant bits of what is left (truncation, so the remainders are exact)
__device__ __forceinline__ QueryTerms split_query(const float (&x)[8]) {
    std::uint32_t words[3][4];
#pragma unroll
    for (int w = 0; w < 4; ++w) {
        std::uint32_t term[3][2];
#pragma unroll
        for (int half = 0; half < 2; ++half) {
            float rest = x[2 * w + half];
#pragma unroll
            for (int t = 0; t < 3; ++t) {
                term[t][half] = __float_as_uint(rest) & 0xffff0000u;
                rest -= __uint_as_float(term[t][half]);
            }
        }
#pragma unroll
        for (int t = 0; t < 3; ++t) {
            words[t][w] = __builtin_amdgcn_perm(term[t][1], term[t][0], 0x07060302u);
        }
    }
    QueryTerms terms;
    terms.high = __builtin_bit_cast(bf16x8, make_uint4(words[0][0], words[0][1], words[0][2], words[0][3]));
    terms.middle = __builtin_bit_cast(bf16x8, make_uint4(words[1][0], words[1][1], words[1][2], words[1][3]));
    terms.low = __builtin_bit_cast(bf16x8, make_uint4(words[2][0], words[2][1], words[2][2], words[2][3]));
    return terms;
}

// eight floats as the bf16 row the cache would hold of them
__device__ __forceinline__ uint4 pack_as_cached(float4 low, float4 high) {
    const auto pair = [](float first, float second) {
        return static_cast<std::uint32_t>(to_bf16(first)) |
            (static_cast<std::uint32_t>(to_bf16(second)) << 16);
    };
    return make_uint4(pair(low.x, low.y), pair(low.z, low.w), pair(high.x, high.y),
                      pair(high.z, high.w));
}

__global__ __launch_bounds__(kGroupWaves * kWave) void attention_grouped_kernel(AttentionArguments a) {
    // waves x kStageBytes: a value tile per wave; at the end the waves' results
    // (maxima, denominators, accumulators: less than that) in the same memory
    extern __shared__ __attribute__((aligned(16))) std::uint8_t grouped_lds[];

    resolve_position(a);
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int j = lane >> 4;
    const int i = lane & 15;
    std::uint8_t* stage = grouped_lds + wave * kStageBytes;
    // workgroup = (query row, key/value head, group of its query heads); all fit 32 bits
    const std::uint32_t groups_per_kv = (a.heads_per_kv + kGroupHeads - 1) / kGroupHeads;
    const std::uint32_t groups_per_row = static_cast<std::uint32_t>(a.kv_heads) * groups_per_kv;
    const std::int64_t query_row = blockIdx.x / groups_per_row;
    const std::uint32_t in_row = blockIdx.x % groups_per_row;
    const std::uint32_t kv_head = in_row / groups_per_kv;
    const std::uint32_t head_group = in_row % groups_per_kv;
    const int heads_here = static_cast<int>(
        a.heads_per_kv - head_group * kGroupHeads < kGroupHeads
            ? a.heads_per_kv - head_group * kGroupHeads : kGroupHeads);
    const std::int64_t first_head =
        static_cast<std::int64_t>(kv_head) * a.heads_per_kv + head_group * kGroupHeads;
    const KeyRange range = key_range(a, query_row, waves);
    const int active = range.active;
    // Keys that are bf16 rows go through the matrix cores in tiles: the cache and, for a
    // causal block, the rows before the query's own (the cache will hold them rounded).
    // The others are float rows, taken one at a time: the query's own row, or every
    // row of a block that is not causal.
    const std::int64_t tiled_end = a.causal != 0 ? a.context_length + query_row : a.context_length;
    const std::int64_t tiled_last = range.last < tiled_end ? range.last : tiled_end - 1;
    const std::int64_t float_first = range.first > tiled_end ? range.first : tiled_end;
    const std::int64_t head_offset = static_cast<std::int64_t>(kv_head) * kGroupHeadDim;
    const std::int64_t block_stride = a.kv_heads * kGroupHeadDim;

    // query of head i, dimensions 32s + 8j .. + 7 (zeros for the heads a group lacks), as
    // operand B of the score instructions
    const float* query =
        a.query + (query_row * a.query_heads + first_head + i) * kGroupHeadDim + 8 * j;
    QueryTerms q[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
        float x[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        if (i < heads_here) {
            const float4 low = *reinterpret_cast<const float4*>(query + 32 * s);
            const float4 high = *reinterpret_cast<const float4*>(query + 32 * s + 4);
            x[0] = low.x, x[1] = low.y, x[2] = low.z, x[3] = low.w;
            x[4] = high.x, x[5] = high.y, x[6] = high.z, x[7] = high.w;
        }
        q[s] = split_query(x);
    }

    const std::int64_t capacity = a.cache_capacity;
    const std::int64_t tile_step = static_cast<std::int64_t>(active) * kWave;
    const std::int64_t slot_step = tile_step % capacity;
    std::int64_t tile_slot = (range.first + static_cast<std::int64_t>(wave) * kWave) % capacity;
    const auto ring_row = [capacity](std::int64_t slot) {  // slot < 2 * capacity
        return slot >= capacity ? slot - capacity : slot;
    };

    float maximum = -INFINITY;  // of head i; the same in the four lanes (., i)
    float denominator = 0.0f;
    f32x4 accumulator[8];  // [2p + parity][r]: head 4j + r, dimension 32p + 2i + parity
#pragma unroll
    for (int e = 0; e < 8; ++e) accumulator[e] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
    // what a lane wrote to its wave's stage is seen by the other lanes after this, and
    // the compiler moves no LDS access across it
    const auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };

    // the accumulator rows (heads 4j + r) are scaled by their heads' factors
    const auto rescale = [&](float keep) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float keep_r = __shfl(keep, 4 * j + r);
#pragma unroll
            for (int e = 0; e < 8; ++e) accumulator[e][r] *= keep_r;
        }
    };
    const auto across_j_max = [](float value) {
        value = fmaxf(value, __shfl_xor(value, 16));
        return fmaxf(value, __shfl_xor(value, 32));
    };
    const auto across_j_sum = [](float value) {
        value += __shfl_xor(value, 16);
        return value + __shfl_xor(value, 32);
    };

    // Loads of one tile of up to 64 bf16 rows starting at key `tile` (ring slot `slot`).
    // Keys past the range repeat the last key of the tile (their weight will be 0).
    uint4 key_raw[4][4], value_raw[4][4];
    // ... a full tile that lies in the cache and does not wrap: one pointer per lane
    // and operand, the rest are wave-uniform steps
    const auto load_straight = [&](std::int64_t slot) {
        const std::uint16_t* key_rows =
            a.key_cache + (slot + i) * a.cache_row_stride + head_offset + 8 * j;
        const std::uint16_t* value_rows =
            a.value_cache + (slot + 4 * j) * a.cache_row_stride + head_offset + 8 * i;
#pragma unroll
        for (int block = 0; block < 4; ++block) {
            const std::uint16_t* row = key_rows + block * 16 * a.cache_row_stride;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                key_raw[block][s] = *reinterpret_cast<const uint4*>(row + 32 * s);
            }
        }
#pragma unroll
        for (int block = 0; block < 4; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                value_raw[block][r] = *reinterpret_cast<const uint4*>(
                    value_rows + (block * 16 + r) * a.cache_row_stride);
            }
        }
    };
    // ... any tile: rows of the block are read as floats and rounded the way the cache
    // commit rounds them
    const auto load_general = [&](std::int64_t tile, std::int64_t slot, int in_tile) {
        const auto key_piece = [&](int key, int s) {
            if (tile + key >= a.context_length) {
                const float* row = a.block_key +
                    (tile + key - a.context_length) * block_stride + head_offset + 8 * j + 32 * s;
                return pack_as_cached(*reinterpret_cast<const float4*>(row),
                                      *reinterpret_cast<const float4*>(row + 4));
            }
            return *reinterpret_cast<const uint4*>(
                a.key_cache + ring_row(slot + key) * a.cache_row_stride + head_offset + 8 * j +
                32 * s);
        };
        const auto value_piece = [&](int key) {
            if (tile + key >= a.context_length) {
                const float* row = a.block_value +
                    (tile + key - a.context_length) * block_stride + head_offset + 8 * i;
                return pack_as_cached(*reinterpret_cast<const float4*>(row),
                                      *reinterpret_cast<const float4*>(row + 4));
            }
            return *reinterpret_cast<const uint4*>(
                a.value_cache + ring_row(slot + key) * a.cache_row_stride + head_offset + 8 * i);
        };
        for (int block = 0; block < 4; ++block) {
            const int key = block * 16 + i < in_tile ? block * 16 + i : in_tile;
#pragma unroll
            for (int s = 0; s < 4; ++s) key_raw[block][s] = key_piece(key, s);
        }
        for (int block = 0; block < 4; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int wanted = block * 16 + 4 * j + r;
                value_raw[block][r] = value_piece(wanted < in_tile ? wanted : in_tile);
            }
        }
    };
    const auto is_straight = [&](std::int64_t tile, std::int64_t slot) {  // wave-uniform
        return tile + kWave - 1 <= tiled_last && tile + kWave - 1 < a.context_length &&
            slot + kWave <= capacity;
    };

    for (std::int64_t tile = range.first + static_cast<std::int64_t>(wave) * kWave;
         wave < active && tile <= tiled_last;
         tile += tile_step, tile_slot = ring_row(tile_slot + slot_step)) {
        const int in_tile =
            static_cast<int>(tiled_last - tile < kWave - 1 ? tiled_last - tile : kWave - 1);
        if (is_straight(tile, tile_slot)) {
            load_straight(tile_slot);
        } else {
            load_general(tile, tile_slot, in_tile);
        }

        // scores: the small terms of the query first
        f32x4 score[4];
#pragma unroll
        for (int block = 0; block < 4; ++block) score[block] = f32x4{0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int term = 0; term < 3; ++term) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const bf16x8 query_term = term == 0 ? q[s].low : term == 1 ? q[s].middle : q[s].high;
#pragma unroll
                for (int block = 0; block < 4; ++block) {
                    score[block] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                        __builtin_bit_cast(bf16x8, key_raw[block][s]), query_term, score[block], 0,
                        0, 0);
                }
            }
        }

        float tile_maximum = -INFINITY;
#pragma unroll
        for (int block = 0; block < 4; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const bool live = block * 16 + 4 * j + r <= in_tile;
                score[block][r] = live ? score[block][r] * a.scale : -INFINITY;
                tile_maximum = fmaxf(tile_maximum, score[block][r]);
            }
        }
        const float next_maximum = fmaxf(maximum, across_j_max(tile_maximum));
        const float keep = __expf(maximum - next_maximum);  // 0 on the first tile
        float weights = 0.0f;
#pragma unroll
        for (int block = 0; block < 4; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                score[block][r] = __expf(score[block][r] - next_maximum);  // 0 for a dead key
                weights += score[block][r];
            }
        }
        denominator = denominator * keep + across_j_sum(weights);
        maximum = next_maximum;
        rescale(keep);

        // the tile's value rows into the stage: key block * 16 + 4j + r, dimensions 8i..
        wave_sync();  // the reads of the previous tile are done
#pragma unroll
        for (int block = 0; block < 4; ++block) {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                *reinterpret_cast<uint4*>(stage + (block * 16 + 4 * j + r) * kStageRowBytes + 16 * i) =
                    value_raw[block][r];
            }
        }
        wave_sync();
#pragma unroll
        for (int half = 0; half < 2; ++half) {  // 32 keys: blocks 2 * half and 2 * half + 1
            const float weights_here[8] = {
                score[2 * half][0], score[2 * half][1], score[2 * half][2], score[2 * half][3],
                score[2 * half + 1][0], score[2 * half + 1][1], score[2 * half + 1][2],
                score[2 * half + 1][3]};
            const QueryTerms weight = split_query(weights_here);
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                // element e of the operands: key 16 * (2 * half + e / 4) + 4j + e % 4
                std::uint32_t pair[8];
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int key = 16 * (2 * half + e / 4) + 4 * j + e % 4;
                    pair[e] = *reinterpret_cast<const std::uint32_t*>(
                        stage + key * kStageRowBytes + 64 * p + 4 * i);
                }
                // dimensions 32p + 2i and 32p + 2i + 1 of the eight keys: the low halves of
                // two dwords side by side, and the high halves (v_perm_b32 byte selectors)
                uint4 even, odd;
                even.x = __builtin_amdgcn_perm(pair[1], pair[0], 0x05040100u);
                even.y = __builtin_amdgcn_perm(pair[3], pair[2], 0x05040100u);
                even.z = __builtin_amdgcn_perm(pair[5], pair[4], 0x05040100u);
                even.w = __builtin_amdgcn_perm(pair[7], pair[6], 0x05040100u);
                odd.x = __builtin_amdgcn_perm(pair[1], pair[0], 0x07060302u);
                odd.y = __builtin_amdgcn_perm(pair[3], pair[2], 0x07060302u);
                odd.z = __builtin_amdgcn_perm(pair[5], pair[4], 0x07060302u);
                odd.w = __builtin_amdgcn_perm(pair[7], pair[6], 0x07060302u);
                const bf16x8 even_values = __builtin_bit_cast(bf16x8, even);
                const bf16x8 odd_values = __builtin_bit_cast(bf16x8, odd);
                accumulator[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.low, even_values, accumulator[2 * p], 0, 0, 0);
                accumulator[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.low, odd_values, accumulator[2 * p + 1], 0, 0, 0);
                accumulator[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.middle, even_values, accumulator[2 * p], 0, 0, 0);
                accumulator[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.middle, odd_values, accumulator[2 * p + 1], 0, 0, 0);
                accumulator[2 * p] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.high, even_values, accumulator[2 * p], 0, 0, 0);
                accumulator[2 * p + 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    weight.high, odd_values, accumulator[2 * p + 1], 0, 0, 0);
            }
        }
    }

    // Float rows of the block, dealt over the waves that have work (the one-token form has
    // one, the query's own key, and its first wave takes it).
    for (std::int64_t position = float_first + wave; wave < active && position <= range.last;
         position += active) {
        const std::int64_t block_row = position - a.context_length;
        const float* key = a.block_key + block_row * block_stride + head_offset + 8 * j;
        float dot = 0.0f;
        if (i < heads_here) {
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                const float4 q_low = *reinterpret_cast<const float4*>(query + 32 * s);
                const float4 q_high = *reinterpret_cast<const float4*>(query + 32 * s + 4);
                const float4 k_low = *reinterpret_cast<const float4*>(key + 32 * s);
                const float4 k_high = *reinterpret_cast<const float4*>(key + 32 * s + 4);
                dot = fmaf(q_low.x, k_low.x, dot);
                dot = fmaf(q_low.y, k_low.y, dot);
                dot = fmaf(q_low.z, k_low.z, dot);
                dot = fmaf(q_low.w, k_low.w, dot);
                dot = fmaf(q_high.x, k_high.x, dot);
                dot = fmaf(q_high.y, k_high.y, dot);
                dot = fmaf(q_high.z, k_high.z, dot);
                dot = fmaf(q_high.w, k_high.w, dot);
            }
        }
        const float score = across_j_sum(dot) * a.scale;
        const float next_maximum = fmaxf(maximum, score);
        const float keep = expf(maximum - next_maximum);
        const float weight = expf(score - next_maximum);
        denominator = denominator * keep + weight;
        maximum = next_maximum;
        rescale(keep);
        const float* value_row = a.block_value + block_row * block_stride + head_offset + 2 * i;
        float value[8];  // [2p + parity]: dimension 32p + 2i + parity
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            const float2 two = *reinterpret_cast<const float2*>(value_row + 32 * p);
            value[2 * p] = two.x;
            value[2 * p + 1] = two.y;
        }
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const float weight_r = __shfl(weight, 4 * j + r);
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                accumulator[e][r] = fmaf(weight_r, value[e], accumulator[e][r]);
            }
        }
    }

    // the stages have been read; the waves' results take their place
    __syncthreads();
    constexpr int kRowFloats = kGroupHeadDim + kGroupRowPad;
    float* wave_maximum = reinterpret_cast<float*>(grouped_lds);           // [waves][16]
    float* wave_denominator = wave_maximum + waves * kGroupHeads;           // [waves][16]
    float* wave_accumulator = wave_denominator + waves * kGroupHeads;       // [waves][16][132]
    if (j == 0) {
        wave_maximum[wave * kGroupHeads + i] = maximum;
        wave_denominator[wave * kGroupHeads + i] = denominator;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        float* target = wave_accumulator + (wave * kGroupHeads + 4 * j + r) * kRowFloats + 2 * i;
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            *reinterpret_cast<float2*>(target + 32 * p) =
                make_float2(accumulator[2 * p][r], accumulator[2 * p + 1][r]);
        }
    }
    __syncthreads();

    // The waves' results meet; a thread takes eight dimensions of a head.  The split form
    // leaves them unnormalised, relative to the share's maximum (an empty share says
    // (-inf, 0, 0)); otherwise the output row is written.
    for (int item = tid; item < heads_here * (kGroupHeadDim / 8); item += blockDim.x) {
        const int head = item / (kGroupHeadDim / 8);
        const int piece = item % (kGroupHeadDim / 8);
        float overall = active > 0 ? wave_maximum[head] : -INFINITY;
        for (int w = 1; w < active; ++w) {
            overall = fmaxf(overall, wave_maximum[w * kGroupHeads + head]);
        }
        float sum[8] = {0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f, 0.0f};
        float total = 0.0f;
        for (int w = 0; w < active; ++w) {
            const float factor = expf(wave_maximum[w * kGroupHeads + head] - overall);
            const float* row = wave_accumulator + (w * kGroupHeads + head) * kRowFloats + 8 * piece;
            const float4 low = *reinterpret_cast<const float4*>(row);
            const float4 high = *reinterpret_cast<const float4*>(row + 4);
            sum[0] = fmaf(low.x, factor, sum[0]);
            sum[1] = fmaf(low.y, factor, sum[1]);
            sum[2] = fmaf(low.z, factor, sum[2]);
            sum[3] = fmaf(low.w, factor, sum[3]);
            sum[4] = fmaf(high.x, factor, sum[4]);
            sum[5] = fmaf(high.y, factor, sum[5]);
            sum[6] = fmaf(high.z, factor, sum[6]);
            sum[7] = fmaf(high.w, factor, sum[7]);
            total = fmaf(wave_denominator[w * kGroupHeads + head], factor, total);
        }
        const std::int64_t row_index = query_row * a.query_heads + first_head + head;
        if (a.partials != nullptr) {
            // a partial row starts 8-byte aligned, and so does its third float
            float* partial =
                a.partials + (row_index * a.splits + blockIdx.y) * partial_floats(kGroupHeadDim);
            if (piece == 0) *reinterpret_cast<float2*>(partial) = make_float2(overall, total);
            float2* target = reinterpret_cast<float2*>(partial + 2 + 8 * piece);
            target[0] = make_float2(sum[0], sum[1]);
            target[1] = make_float2(sum[2], sum[3]);
            target[2] = make_float2(sum[4], sum[5]);
            target[3] = make_float2(sum[6], sum[7]);
        } else {
            float4* target =
                reinterpret_cast<float4*>(a.output + row_index * kGroupHeadDim + 8 * piece);
            target[0] = make_float4(sum[0] / total, sum[1] / total, sum[2] / total, sum[3] / total);
            target[1] = make_float4(sum[4] / total, sum[5] / total, sum[6] / total, sum[7] / total);
        }
    }
}

bool vector_form_fits(const AttentionArguments& arguments) {
    const auto aligned = [](const void* pointer) {
        return reinterpret_cast<std::uintptr_t>(pointer) % 16 == 0;
    };
    const std::int64_t head_dim = arguments.head_dim;
    return (head_dim == 32 || head_dim == 64 || head_dim == 128 || head_dim == 256) &&
        arguments.cache_row_stride % 8 == 0 && arguments.cache_row_stride < (1 << 24) &&
        arguments.cache_capacity >= kWave &&
        aligned(arguments.key_cache) && aligned(arguments.value_cache) &&
        aligned(arguments.block_key) && aligned(arguments.block_value);
}

// The matrix-core kernel: head_dim 128, enough query heads per key/value head to fill
// a useful part of its 16-head tiles, 16-byte aligned rows everywhere.
bool grouped_form_fits(const AttentionArguments& arguments) {
    const auto aligned = [](const void* pointer) {
        return reinterpret_cast<std::uintptr_t>(pointer) % 16 == 0;
    };
    return vector_form_fits(arguments) && arguments.head_dim == kGroupHeadDim &&
        arguments.heads_per_kv >= kGroupMinHeads && aligned(arguments.query) &&
        aligned(arguments.output);
}

// `tiles_per_group`: the most 64-key tiles one workgroup has to cover.
void launch_attention(const AttentionArguments& arguments, std::int64_t query_rows,
                      std::int64_t tiles_per_group, hipStream_t stream) {
    std::int64_t waves = tiles_per_group;
    if (waves < 1) waves = 1;
    if (waves > kMaxWaves) waves = kMaxWaves;
    const std::int64_t head_dim = arguments.head_dim;
    const unsigned splits = arguments.partials != nullptr ? arguments.splits : 1;
    // A workgroup that walks a whole key range alone takes its rows in at what one
    // compute unit can pull from memory, whatever the arithmetic costs: the matrix-core
    // kernel pays where its workgroups are many (the split form) or where the vector
    // kernel's would not fit the chip at once (blocks of many rows).
    if (grouped_form_fits(arguments) &&
        (arguments.partials != nullptr || query_rows * arguments.query_heads > compute_units())) {
        static_assert(kGroupWaves == kMaxWaves, "one wave rule for both kernels");
        const std::int64_t groups = arguments.kv_heads *
            ((arguments.heads_per_kv + kGroupHeads - 1) / kGroupHeads);
        allow_large_lds<attention_grouped_kernel>(kGroupWaves * kStageBytes);
        hipLaunchKernelGGL(attention_grouped_kernel,
                           dim3(static_cast<unsigned>(query_rows * groups), splits),
                           dim3(static_cast<unsigned>(waves * kWave)),
                           static_cast<std::size_t>(waves) * kStageBytes, stream, arguments);
        return;
    }
    const dim3 grid(static_cast<unsigned>(query_rows * arguments.query_heads), splits);
    const dim3 block(static_cast<unsigned>(waves * kWave));
    if (!vector_form_fits(arguments)) {
        hipLaunchKernelGGL(attention_generic_kernel, grid, block, 0, stream, arguments);
    } else if (head_dim == 32) {
        hipLaunchKernelGGL(attention_vector_kernel<4>, grid, block, 0, stream, arguments);
    } else if (head_dim == 64) {
        hipLaunchKernelGGL(attention_vector_kernel<8>, grid, block, 0, stream, arguments);
    } else if (head_dim == 128) {
        hipLaunchKernelGGL(attention_vector_kernel<16>, grid, block, 0, stream, arguments);
    } else {
        hipLaunchKernelGGL(attention_vector_kernel<32>, grid, block, 0, stream, arguments);
    }
}

AttentionArguments decode_arguments(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d) {
    AttentionArguments a{};
    a.query = d.query;
    a.block_key = d.current_key;
    a.block_value = d.current_value;
    a.key_cache = d.key_cache_bf16;
    a.value_cache = d.value_cache_bf16;
    a.output = d.output;
    a.query_heads = d.query_heads;
    a.kv_heads = d.kv_heads;
    a.head_dim = d.head_dim;
    a.heads_per_kv = static_cast<std::uint32_t>(d.query_heads / d.kv_heads);
    a.context_length = d.position;
    a.block_rows = 1;
    a.sliding_window = d.position - d.first_key_position + 1;
    a.cache_capacity = d.cache_capacity;
    a.cache_row_stride = d.cache_row_stride;
    a.scale = d.scale;
    a.causal = 1;
    return a;
}

std::int64_t tiles_of(std::int64_t keys) { return (keys + kWave - 1) / kWave; }

}  // namespace

void launch_gqa_decode(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d, hipStream_t stream) {
    const AttentionArguments a = decode_arguments(d);
    launch_attention(a, 1, tiles_of(a.sliding_window), stream);
}

void launch_gqa_decode_device_position(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d,
                                       const std::int64_t* device_position,
                                       std::int64_t sliding_window, bool whole_context,
                                       hipStream_t stream) {
    AttentionArguments a = decode_arguments(d);
    a.device_position = device_position;
    a.sliding_window = sliding_window;
    a.whole_context = whole_context ? 1 : 0;
    // the key count is not known here: the largest workgroup, of which as many
    // waves work as the row has tiles
    launch_attention(a, 1, kMaxWaves, stream);
}

std::int64_t gqa_decode_split_workspace_bytes(std::int64_t query_heads, std::int64_t head_dim) {
    return query_heads * kMaxSplits * partial_floats(head_dim) * 4;
}

namespace {

// Split form.  `tiles`: the 64-key tiles of the longest row, or with a position in
// device memory the most it can have (the shares are cut from each row's real key
// count when the kernel runs; surplus shares are empty).  `partial_bytes` bounds the
// shares; with room for fewer than two the ordinary form runs.
void launch_split(AttentionArguments a, std::int64_t query_rows, std::int64_t tiles,
                  float* partials, std::int64_t partial_bytes, hipStream_t stream) {
    // As many shares as fill the chip with about one workgroup per compute unit (a
    // workgroup of the matrix-core kernel serves up to 16 query heads, one of the
    // vector kernel a single head), then up to eight waves a share.
    a.partials = partials;  // (decides the kernel)
    const bool grouped = grouped_form_fits(a);
    const std::int64_t groups = query_rows *
        (grouped ? a.kv_heads * ((a.heads_per_kv + kGroupHeads - 1) / kGroupHeads) : a.query_heads);
    const std::int64_t share_bytes = query_rows * a.query_heads * partial_floats(a.head_dim) * 4;
    std::int64_t splits = compute_units() / groups;
    if (splits > (grouped ? kMaxSplits : kVectorSplits)) splits = grouped ? kMaxSplits : kVectorSplits;
    if (splits > tiles) splits = tiles;
    // One query row: at least two tiles a share, two waves a workgroup.  A 2,048-key window
    // in 16 shares of two waves takes 11.1 us with its merge, in 32 shares of one wave 12.1 us
    // (12 or 24 shares: 11.7; 8: 11.9); long contexts and blocks are not touched by this
    // (32,768 keys: 128 shares 15.1 us, 96: 15.4, 64: 17.1; a 16-row block: 8..24 shares 16.1 us).
    if (query_rows == 1 && grouped && 2 * splits > tiles && tiles >= 4) splits = (tiles + 1) / 2;
    if (splits < 2) splits = 2;
    if (splits > partial_bytes / share_bytes) splits = partial_bytes / share_bytes;
    if (splits < 2) {
        a.partials = nullptr;
        launch_attention(a, query_rows, tiles, stream);
        return;
    }
    a.splits = static_cast<int>(splits);
    launch_attention(a, query_rows, (tiles + splits - 1) / splits, stream);
    const int threads = static_cast<int>((a.head_dim + kWave - 1) / kWave * kWave) * kMergeLanes;
    hipLaunchKernelGGL(attention_merge_kernel,
                       dim3(static_cast<unsigned>(query_rows * a.query_heads)), dim3(threads), 0,
                       stream, partials, a.output, a.splits, static_cast<int>(a.head_dim));
}

}  // namespace

void launch_gqa_decode_split(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d, float* partials,
                             hipStream_t stream) {
    const AttentionArguments a = decode_arguments(d);
    const std::int64_t tiles = tiles_of(a.sliding_window);
    if (!vector_form_fits(a) || tiles < 2) {
        launch_attention(a, 1, tiles, stream);  // nothing to split, or no vector form: one launch
        return;
    }
    launch_split(a, 1, tiles, partials, gqa_decode_split_workspace_bytes(d.query_heads, d.head_dim),
                 stream);
}

void launch_gqa_decode_split_device_position(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d,
                                             const std::int64_t* device_position,
                                             std::int64_t sliding_window, bool whole_context,
                                             float* partials, hipStream_t stream) {
    AttentionArguments a = decode_arguments(d);
    a.device_position = device_position;
    a.sliding_window = sliding_window;
    a.whole_context = whole_context ? 1 : 0;
    if (!vector_form_fits(a)) {
        launch_attention(a, 1, kMaxWaves, stream);
        return;
    }
    // a global layer sees at most the ring and the row's own key
    launch_split(a, 1, tiles_of(whole_context ? d.cache_capacity + 1 : sliding_window), partials,
                 gqa_decode_split_workspace_bytes(d.query_heads, d.head_dim), stream);
}

void launch_block_attention(const NfnNativeTileDFlashBlockAttentionDescriptorV1& d, float* partials,
                            std::int64_t partial_bytes, hipStream_t stream) {
    AttentionArguments a{};
    a.query = d.query;
    a.block_key = d.block_key;
    a.block_value = d.block_value;
    a.key_cache = d.key_cache_bf16;
    a.value_cache = d.value_cache_bf16;
    a.output = d.output;
    a.query_heads = d.query_heads;
    a.kv_heads = d.kv_heads;
    a.head_dim = d.head_dim;
    a.heads_per_kv = static_cast<std::uint32_t>(d.query_heads / d.kv_heads);
    a.context_length = d.context_length;
    a.block_rows = d.block_rows;
    a.sliding_window = d.sliding_window;
    a.cache_capacity = d.cache_capacity;
    a.cache_row_stride = d.cache_row_stride;
    a.scale = d.scale;
    a.causal = (d.flags & NFN_NATIVE_TILE_BLOCK_ATTENTION_CAUSAL) != 0 ? 1 : 0;
    std::int64_t longest = d.context_length + d.block_rows;  // never more keys than exist
    if (d.sliding_window < longest) {
        const std::int64_t window = a.causal ? d.sliding_window : 2 * d.sliding_window + 1;
        if (window < longest) longest = window;
    }
    const std::int64_t tiles = tiles_of(longest);
    if (partials != nullptr && vector_form_fits(a) && tiles >= 2) {
        launch_split(a, d.query_rows, tiles, partials, partial_bytes, stream);
    } else {
        launch_attention(a, d.query_rows, tiles, stream);
    }
}

}  // namespace nfn
