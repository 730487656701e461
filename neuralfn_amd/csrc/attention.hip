// Attention of the decode loop over a bf16 key/value cache: the one-token
// grouped-query form and the block form of the verifier and the proposal
// model (semantics: neuralfn/csrc/native_train/tile_ops.h:308-339, 445-486;
// reference kernels: neuralfn/csrc/tile_cuda/kernels.cu:2475-2824, 2924-3075).
//
// One workgroup per (query row, query head), up to sixteen waves.  A wave takes
// every waves-th tile of 64 keys.  Inside a tile a lane owns one key for the
// scores (it walks the key's head_dim values in 16-byte pieces against the
// query, which sits in LDS and is read as a broadcast), the wave reduces the
// tile's maximum and sum once, and for the weighted sum of the values a lane
// owns the output dimensions lane, lane + 64, ...: the weight of key k comes
// from lane k by a lane read, the value row is read coalesced.  Every wave
// keeps a running (maximum, denominator, accumulator) and the workgroup
// merges them through LDS at the end.  The one-token form is the block form
// with one query row whose own key is the only block row.
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

constexpr int kMaxWaves = 16;
constexpr int kMaxHeadDim = 256;
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
    std::int64_t context_length;
    std::int64_t block_rows;
    std::int64_t sliding_window;
    std::int64_t cache_capacity;
    std::int64_t cache_row_stride;
    float scale;
    int causal;
};

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

// q . k for one key held by this lane.  VEC: head_dim is a multiple of 8 and
// every row starts 16-byte aligned.
template <bool VEC>
__device__ __forceinline__ float score_cache_key(const float* q, const std::uint16_t* key,
                                                 int head_dim) {
    float dot = 0.0f;
    if constexpr (VEC) {
        for (int d = 0; d < head_dim; d += 8) {
            const uint4 packed = *reinterpret_cast<const uint4*>(key + d);
            const float4 q0 = *reinterpret_cast<const float4*>(q + d);
            const float4 q1 = *reinterpret_cast<const float4*>(q + d + 4);
            dot = fmaf(q0.x, __uint_as_float(packed.x << 16), dot);
            dot = fmaf(q0.y, __uint_as_float(packed.x & 0xffff0000u), dot);
            dot = fmaf(q0.z, __uint_as_float(packed.y << 16), dot);
            dot = fmaf(q0.w, __uint_as_float(packed.y & 0xffff0000u), dot);
            dot = fmaf(q1.x, __uint_as_float(packed.z << 16), dot);
            dot = fmaf(q1.y, __uint_as_float(packed.z & 0xffff0000u), dot);
            dot = fmaf(q1.z, __uint_as_float(packed.w << 16), dot);
            dot = fmaf(q1.w, __uint_as_float(packed.w & 0xffff0000u), dot);
        }
    } else {
        for (int d = 0; d < head_dim; ++d) dot = fmaf(q[d], bf16_to_float(key[d]), dot);
    }
    return dot;
}

template <bool VEC>
__device__ __forceinline__ float score_block_key(const float* q, const float* key, int head_dim,
                                                 bool as_cached) {
    float dot = 0.0f;
    if constexpr (VEC) {
        for (int d = 0; d < head_dim; d += 4) {
            float4 k = *reinterpret_cast<const float4*>(key + d);
            const float4 qv = *reinterpret_cast<const float4*>(q + d);
            if (as_cached) {
                k.x = bf16_to_float(to_bf16(k.x));
                k.y = bf16_to_float(to_bf16(k.y));
                k.z = bf16_to_float(to_bf16(k.z));
                k.w = bf16_to_float(to_bf16(k.w));
            }
            dot = fmaf(qv.x, k.x, dot);
            dot = fmaf(qv.y, k.y, dot);
            dot = fmaf(qv.z, k.z, dot);
            dot = fmaf(qv.w, k.w, dot);
        }
    } else {
        for (int d = 0; d < head_dim; ++d) {
            float k = key[d];
            if (as_cached) k = bf16_to_float(to_bf16(k));
            dot = fmaf(q[d], k, dot);
        }
    }
    return dot;
}

template <bool VEC>
__global__ __launch_bounds__(kMaxWaves * kWave) void attention_kernel(AttentionArguments a) {
    __shared__ __attribute__((aligned(16))) float q[kMaxHeadDim];
    __shared__ float wave_maximum[kMaxWaves];
    __shared__ float wave_denominator[kMaxWaves];
    __shared__ float wave_accumulator[kMaxWaves][kMaxHeadDim];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int waves = static_cast<int>(blockDim.x >> 6);
    const int head_dim = static_cast<int>(a.head_dim);
    const std::int64_t query_row = blockIdx.x / a.query_heads;
    const std::int64_t query_head = blockIdx.x - query_row * a.query_heads;
    const std::int64_t kv_head = query_head * a.kv_heads / a.query_heads;
    const std::int64_t query_position = a.context_length + query_row;
    const bool causal = a.causal != 0;
    std::int64_t first = query_position - a.sliding_window + (causal ? 1 : 0);
    if (first < 0) first = 0;
    std::int64_t last = query_position;
    if (!causal) {
        const std::int64_t end = a.context_length + a.block_rows - 1;
        last = a.sliding_window < end - query_position ? query_position + a.sliding_window : end;
    }

    const float* query = a.query + (query_row * a.query_heads + query_head) * a.head_dim;
    for (int d = tid; d < head_dim; d += blockDim.x) q[d] = query[d];
    __syncthreads();

    float maximum = -INFINITY;
    float denominator = 0.0f;
    float accumulator[kOwned];
#pragma unroll
    for (int j = 0; j < kOwned; ++j) accumulator[j] = 0.0f;

    // How many waves share the keys depends on this row's key count only, not
    // on the launch: a row of a causal block then sums in the same order as
    // the one-token call at the same position, and gives the same bits.
    const std::int64_t tiles = (last - first) / kWave + 1;
    const int active = static_cast<int>(tiles < waves ? tiles : waves);
    for (std::int64_t tile = first + static_cast<std::int64_t>(wave) * kWave;
         wave < active && tile <= last; tile += static_cast<std::int64_t>(active) * kWave) {
        const std::int64_t key_position = tile + lane;
        const bool live = key_position <= last;
        float score = -INFINITY;
        if (live) {
            if (key_position >= a.context_length) {
                const std::int64_t block_row = key_position - a.context_length;
                const float* key = a.block_key + (block_row * a.kv_heads + kv_head) * a.head_dim;
                score = score_block_key<VEC>(q, key, head_dim, causal && block_row < query_row);
            } else {
                const std::uint16_t* key = a.key_cache +
                    (key_position % a.cache_capacity) * a.cache_row_stride + kv_head * a.head_dim;
                score = score_cache_key<VEC>(q, key, head_dim);
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

void launch_attention(const AttentionArguments& arguments, std::int64_t query_rows,
                      std::int64_t longest_key_range, hipStream_t stream) {
    std::int64_t waves = (longest_key_range + kWave - 1) / kWave;
    if (waves < 1) waves = 1;
    if (waves > kMaxWaves) waves = kMaxWaves;
    const auto aligned = [](const void* pointer) {
        return reinterpret_cast<std::uintptr_t>(pointer) % 16 == 0;
    };
    const bool vectors = arguments.head_dim % 8 == 0 && arguments.cache_row_stride % 8 == 0 &&
        aligned(arguments.key_cache) && aligned(arguments.block_key);
    const dim3 grid(static_cast<unsigned>(query_rows * arguments.query_heads));
    const dim3 block(static_cast<unsigned>(waves * kWave));
    if (vectors) {
        hipLaunchKernelGGL(attention_kernel<true>, grid, block, 0, stream, arguments);
    } else {
        hipLaunchKernelGGL(attention_kernel<false>, grid, block, 0, stream, arguments);
    }
}

}  // namespace

void launch_gqa_decode(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& d, hipStream_t stream) {
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
    a.context_length = d.position;
    a.block_rows = 1;
    a.sliding_window = d.position - d.first_key_position + 1;
    a.cache_capacity = d.cache_capacity;
    a.cache_row_stride = d.cache_row_stride;
    a.scale = d.scale;
    a.causal = 1;
    launch_attention(a, 1, a.sliding_window, stream);
}

void launch_block_attention(const NfnNativeTileDFlashBlockAttentionDescriptorV1& d,
                            hipStream_t stream) {
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
    launch_attention(a, d.query_rows, longest, stream);
}

}  // namespace nfn
