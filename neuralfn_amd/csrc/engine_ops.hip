// The small operators of the decode loop around the packed linears: token
// embedding, rotary position embedding, the bf16 cache commit, the logit
// transform, add and scale.  Each is a few kilobytes of traffic per call at
// decode time and bound by its launch; they exist so that the reference's
// resident engine finds every operator it requires in one library
// (neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:431-495).
//
// Arithmetic follows the reference's CPU engine
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:773-800 rope, 1895-1903
// logit transform), which computes angles and the soft cap in double; the
// reference's device kernels (neuralfn/csrc/tile_cuda/kernels.cu:2346-2376,
// 3254-3264) compute the same formulas in float.
#include "common.hpp"
#include "kernels.hpp"

namespace nfn {

namespace {

constexpr int kThreads = 256;

unsigned blocks_for(std::int64_t count, std::int64_t limit = 1 << 20) {
    const std::int64_t blocks = (count + kThreads - 1) / kThreads;
    return static_cast<unsigned>(blocks < limit ? blocks : limit);
}

// ---- embedding ------------------------------------------------------------
// TOKENS: 0 = one token passed by value, 1 = one int64 token in device memory,
// 2 = int32 tokens in device memory, one per row.
template <int TOKENS>
__global__ __launch_bounds__(kThreads) void embedding_kernel(
    const std::uint8_t* __restrict__ data, std::uint32_t encoding, std::int64_t row_stride,
    std::int64_t vocabulary, std::int64_t width, std::int64_t host_token,
    const void* __restrict__ device_tokens, float* __restrict__ output, std::int64_t count) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        const std::int64_t row = index / width;
        const std::int64_t col = index - row * width;
        std::int64_t token = host_token;
        if constexpr (TOKENS == 1) token = static_cast<const std::int64_t*>(device_tokens)[0];
        if constexpr (TOKENS == 2) token = static_cast<const std::int32_t*>(device_tokens)[row];
        const bool known = token >= 0 && token < vocabulary;
        output[index] = known ? weight_value(encoding, data + token * row_stride, col) : 0.0f;
    }
}

// ---- rotary position embedding ---------------------------------------------
// One thread per (row, head, pair).
__global__ __launch_bounds__(kThreads) void rope_kernel(
    float* __restrict__ query, float* __restrict__ key, std::int64_t rows,
    std::int64_t query_heads, std::int64_t kv_heads, std::int64_t head_dim,
    std::int64_t start_position, double theta, bool interleaved, bool inverse) {
    const std::int64_t half = head_dim / 2;
    const std::int64_t pairs_per_row = (query_heads + kv_heads) * half;
    const std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= rows * pairs_per_row) return;
    const std::int64_t row = index / pairs_per_row;
    const std::int64_t local = index - row * pairs_per_row;
    const std::int64_t head = local / half;
    const std::int64_t pair = local - head * half;
    float* values = head < query_heads
        ? query + (row * query_heads + head) * head_dim
        : key + (row * kv_heads + head - query_heads) * head_dim;
    const std::int64_t first = interleaved ? 2 * pair : pair;
    const std::int64_t second = interleaved ? 2 * pair + 1 : pair + half;
    rope_rotate(values[first], values[second], start_position + row, pair, head_dim, theta, inverse);
}

// ---- cache commit -----------------------------------------------------------
__global__ __launch_bounds__(kThreads) void cache_commit_kernel(
    const float* __restrict__ keys, const float* __restrict__ values,
    std::uint16_t* __restrict__ key_cache, std::uint16_t* __restrict__ value_cache,
    std::int64_t width, std::int64_t rows, std::int64_t position,
    const std::int64_t* __restrict__ device_position, std::int64_t capacity,
    std::int64_t row_stride) {
    const std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= rows * width) return;
    if (device_position != nullptr) position = device_position[0];
    const std::int64_t row = index / width;
    const std::int64_t column = index - row * width;
    const std::int64_t target = ((position + row) % capacity) * row_stride + column;
    key_cache[target] = to_bf16(keys[index]);
    value_cache[target] = to_bf16(values[index]);
}

// Rows 0..rows-1 of a staged block into the rings of up to 64 layers, one launch
// (neuralfn/csrc/tile_cuda/kernels.cu:2862-2901).  blockIdx = (columns, row, layer).
struct CacheLayers {
    NfnNativeTileGlimmerCacheLayerV1 layer[64];
};

__global__ __launch_bounds__(kThreads) void cache_commit_layers_kernel(
    const float* __restrict__ keys, const float* __restrict__ values, std::int64_t width,
    std::int64_t position, std::int64_t layer_stride, CacheLayers layers) {
    const std::int64_t column = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (column >= width) return;
    const std::int64_t row = blockIdx.y;
    const NfnNativeTileGlimmerCacheLayerV1& layer = layers.layer[blockIdx.z];
    const std::int64_t source = blockIdx.z * layer_stride + row * width + column;
    const std::int64_t target =
        ((position + row) % layer.cache_capacity) * layer.cache_row_stride + column;
    layer.key_cache_bf16[target] = to_bf16(keys[source]);
    layer.value_cache_bf16[target] = to_bf16(values[source]);
}

// [tap, source_row, hidden] -> [row, tap, hidden] for rows source_row_offset .. +rows-1
// (neuralfn/csrc/tile_cuda/kernels.cu:2903-2922).
__global__ __launch_bounds__(kThreads) void pack_target_taps_kernel(
    const float* __restrict__ tap_major, float* __restrict__ row_major, std::int64_t source_rows,
    std::int64_t source_row_offset, std::int64_t tap_count, std::int64_t hidden_width,
    std::int64_t count) {
    const std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
    if (index >= count) return;
    const std::int64_t hidden = index % hidden_width;
    const std::int64_t row_tap = index / hidden_width;
    const std::int64_t tap = row_tap % tap_count;
    const std::int64_t row = row_tap / tap_count;
    row_major[index] = tap_major[(tap * source_rows + source_row_offset + row) * hidden_width + hidden];
}

// ---- element-wise -------------------------------------------------------------
__global__ __launch_bounds__(kThreads) void logit_transform_kernel(float* __restrict__ logits,
                                                                  std::int64_t count,
                                                                  double multiplier,
                                                                  double softcap) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        const double value = static_cast<double>(logits[index]);
        logits[index] = static_cast<float>(softcap * tanh((multiplier * value) / softcap));
    }
}

__global__ __launch_bounds__(kThreads) void add_kernel(const float* __restrict__ lhs,
                                                      const float* __restrict__ rhs,
                                                      float* __restrict__ out,
                                                      std::int64_t count) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        out[index] = __fadd_rn(lhs[index], rhs[index]);
    }
}

__global__ __launch_bounds__(kThreads) void scale_kernel(float* __restrict__ values,
                                                        std::int64_t count, float scale) {
    const std::int64_t stride = static_cast<std::int64_t>(gridDim.x) * blockDim.x;
    for (std::int64_t index = static_cast<std::int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
         index < count; index += stride) {
        values[index] = __fmul_rn(values[index], scale);
    }
}

}  // namespace

void launch_embedding(const Descriptor& table, int token_source, std::int64_t host_token,
                      const void* device_tokens, float* output, std::int64_t rows,
                      hipStream_t stream) {
    const std::int64_t count = rows * table.input_dim;
    const dim3 grid(blocks_for(count)), block(kThreads);
    if (token_source == 0) {
        hipLaunchKernelGGL(embedding_kernel<0>, grid, block, 0, stream, table.data, table.encoding,
                           table.row_stride_bytes, table.output_dim, table.input_dim, host_token,
                           device_tokens, output, count);
    } else if (token_source == 1) {
        hipLaunchKernelGGL(embedding_kernel<1>, grid, block, 0, stream, table.data, table.encoding,
                           table.row_stride_bytes, table.output_dim, table.input_dim, host_token,
                           device_tokens, output, count);
    } else {
        hipLaunchKernelGGL(embedding_kernel<2>, grid, block, 0, stream, table.data, table.encoding,
                           table.row_stride_bytes, table.output_dim, table.input_dim, host_token,
                           device_tokens, output, count);
    }
}

void launch_rope(float* query, float* key, std::int64_t rows, std::int64_t query_heads,
                 std::int64_t kv_heads, std::int64_t head_dim, std::int64_t start_position,
                 float theta, bool interleaved, bool inverse, hipStream_t stream) {
    const std::int64_t count = rows * (query_heads + kv_heads) * (head_dim / 2);
    hipLaunchKernelGGL(rope_kernel, dim3(blocks_for(count, std::int64_t(1) << 31)), dim3(kThreads),
                       0, stream, query, key, rows, query_heads, kv_heads, head_dim,
                       start_position, static_cast<double>(theta), interleaved, inverse);
}

void launch_cache_commit(const float* keys, const float* values, std::uint16_t* key_cache,
                         std::uint16_t* value_cache, std::int64_t width, std::int64_t rows,
                         std::int64_t position, const std::int64_t* device_position,
                         std::int64_t capacity, std::int64_t row_stride, hipStream_t stream) {
    hipLaunchKernelGGL(cache_commit_kernel,
                       dim3(blocks_for(rows * width, std::int64_t(1) << 31)), dim3(kThreads), 0,
                       stream, keys, values, key_cache, value_cache, width, rows, position,
                       device_position, capacity, row_stride);
}

void launch_cache_commit_layers(const NfnNativeTileGlimmerCacheCommitLayersDescriptorV1& d,
                                hipStream_t stream) {
    CacheLayers layers{};
    for (std::int64_t index = 0; index < d.layer_count; ++index) layers.layer[index] = d.layers[index];
    const std::int64_t width = d.kv_heads * d.head_dim;
    hipLaunchKernelGGL(cache_commit_layers_kernel,
                       dim3(blocks_for(width), static_cast<unsigned>(d.rows),
                            static_cast<unsigned>(d.layer_count)),
                       dim3(kThreads), 0, stream, d.staged_keys, d.staged_values, width, d.position,
                       d.source_layer_stride, layers);
}

void launch_pack_target_taps(const float* tap_major, float* row_major, std::int64_t source_rows,
                             std::int64_t source_row_offset, std::int64_t rows,
                             std::int64_t tap_count, std::int64_t hidden_width,
                             hipStream_t stream) {
    const std::int64_t count = rows * tap_count * hidden_width;
    hipLaunchKernelGGL(pack_target_taps_kernel, dim3(blocks_for(count, std::int64_t(1) << 31)),
                       dim3(kThreads), 0, stream, tap_major, row_major, source_rows,
                       source_row_offset, tap_count, hidden_width, count);
}

void launch_logit_transform(float* logits, std::int64_t count, float multiplier, float softcap,
                            hipStream_t stream) {
    hipLaunchKernelGGL(logit_transform_kernel, dim3(blocks_for(count)), dim3(kThreads), 0, stream,
                       logits, count, static_cast<double>(multiplier),
                       static_cast<double>(softcap));
}

void launch_add(const float* lhs, const float* rhs, float* out, std::int64_t count,
                hipStream_t stream) {
    hipLaunchKernelGGL(add_kernel, dim3(blocks_for(count)), dim3(kThreads), 0, stream, lhs, rhs,
                       out, count);
}

void launch_scale(float* values, std::int64_t count, float scale, hipStream_t stream) {
    hipLaunchKernelGGL(scale_kernel, dim3(blocks_for(count)), dim3(kThreads), 0, stream, values,
                       count, scale);
}

}  // namespace nfn
