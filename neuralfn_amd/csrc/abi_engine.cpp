// extern "C" surface of the decode loop's operators around the packed linears:
// argument checks as the reference's wrappers make them
// (neuralfn/csrc/native_train/tile_ops.cu:3601-3800, 4734-4775, 5013-5030,
// 5150-5260, 5348-5362, 5421-5445, 6377-6388, 6944-6951), then one launch.
#include "common.hpp"
#include "kernels.hpp"

#include <cmath>
#include <limits>
#include <mutex>

namespace nfn {

namespace {

constexpr std::int64_t kMaxHeadDim = 256;
constexpr std::int64_t kMaxBlockRows = 64;
constexpr std::int64_t kLimit = std::numeric_limits<std::int64_t>::max();

bool positive_finite(float value) { return std::isfinite(value) && value > 0.0f; }

// Workspaces an engine lent to the reference-named attention entry points
// (nfn_mi355_attention_workspace_v1), one per (device, stream): a loan serves
// only calls issued on the stream it was made for, whose work is ordered, so
// two calls never write the same partial results at once.
struct LentWorkspace {
    int device = -1;
    void* stream = nullptr;
    float* memory = nullptr;  // null = free slot
    std::int64_t nbytes = 0;
};
constexpr int kMaxLoans = 32;
std::mutex lent_mutex;
LentWorkspace lent_workspaces[kMaxLoans];

// The workspace lent for `stream` on the current device (memory null if none).
LentWorkspace lent_here(void* stream) {
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) return LentWorkspace{};
    std::lock_guard<std::mutex> guard(lent_mutex);
    for (const LentWorkspace& loan : lent_workspaces) {
        if (loan.memory != nullptr && loan.device == device && loan.stream == stream) return loan;
    }
    return LentWorkspace{};
}

// ... if it is also large enough for the one-token split form of this geometry.
float* lent_partials(void* stream, std::int64_t query_heads, std::int64_t head_dim) {
    const LentWorkspace lent = lent_here(stream);
    if (lent.memory == nullptr) return nullptr;
    const std::int64_t required = gqa_decode_split_workspace_bytes(query_heads, head_dim);
    return lent.nbytes >= required ? lent.memory : nullptr;
}

// kv_heads * head_dim, both positive, fits and does not exceed the row stride
bool cache_rows_fit(std::int64_t kv_heads, std::int64_t head_dim, std::int64_t row_stride) {
    return kv_heads <= kLimit / head_dim && kv_heads * head_dim <= row_stride;
}

// One thread per element (or pair) and no grid-stride loop in these kernels:
// the count must fit a grid of 256-thread workgroups.
constexpr std::int64_t kMaxThreads = std::int64_t(0x7fffffff) * 256;

bool rope_arguments_valid(const float* query, const float* key, std::int64_t rows,
                          std::int64_t query_heads, std::int64_t kv_heads, std::int64_t head_dim,
                          std::int64_t position, float theta, std::uint32_t layout) {
    if (query == nullptr || key == nullptr || rows <= 0 || query_heads <= 0 || kv_heads <= 0 ||
        query_heads % kv_heads != 0 || head_dim <= 0 || head_dim > kMaxHeadDim ||
        head_dim % 2 != 0 || position < 0 || position > kLimit - rows || !positive_finite(theta) ||
        (layout != NFN_NATIVE_TILE_GLIMMER_ROPE_HALF_SPLIT &&
         layout != NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED)) {
        return false;
    }
    // rows * (query_heads + kv_heads) * head_dim / 2 pairs, without overflow on the way
    const std::int64_t half = head_dim / 2;
    if (query_heads > kMaxThreads / half || kv_heads > query_heads) return false;
    const std::int64_t pairs_per_row = (query_heads + kv_heads) * half;
    return rows <= kMaxThreads / pairs_per_row;
}

bool commit_descriptor_valid(const NfnNativeTileGlimmerCacheCommitDescriptorV1* d) {
    return d != nullptr && d->struct_size >= sizeof(*d) &&
        d->version == NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 && d->flags == 0 &&
        d->reserved0 == 0 && d->reserved1 == 0 && d->reserved2 == 0 &&
        d->current_key != nullptr && d->current_value != nullptr &&
        d->key_cache_bf16 != nullptr && d->value_cache_bf16 != nullptr && d->kv_heads > 0 &&
        d->head_dim > 0 && d->head_dim <= kMaxHeadDim && d->position >= 0 &&
        d->cache_capacity > 0 && d->cache_row_stride > 0 &&
        cache_rows_fit(d->kv_heads, d->head_dim, d->cache_row_stride);
}

// Shared checks of the two qk_norm_scale_rope forms and of the fused decode step.
// `normalized_*` receive the checked weight descriptors; a null weight leaves
// its output untouched and reports "no weight" through the returned pointers.
bool qk_norm_arguments_valid(const float* query, const float* key, const Descriptor* query_weight,
                             const Descriptor* key_weight, std::int64_t rows,
                             std::int64_t query_heads, std::int64_t kv_heads,
                             std::int64_t head_dim, float eps, float query_scale,
                             std::int64_t position, float theta, std::uint32_t layout,
                             Descriptor* normalized_query, Descriptor* normalized_key) {
    if (rows > kMaxBlockRows || !positive_finite(eps) || !positive_finite(query_scale) ||
        !rope_arguments_valid(query, key, rows, query_heads, kv_heads, head_dim, position, theta,
                              layout) ||
        query_heads + kv_heads > std::numeric_limits<std::int32_t>::max() / kMaxBlockRows) {
        return false;
    }
    const auto weight_valid = [head_dim](const Descriptor* weight, Descriptor* normalized) {
        return weight == nullptr ||
            (normalize_descriptor(weight, normalized) && normalized->output_dim == 1 &&
             normalized->input_dim == head_dim);
    };
    return weight_valid(query_weight, normalized_query) && weight_valid(key_weight, normalized_key);
}

bool gqa_descriptor_valid(const NfnNativeTileGlimmerGqaDecodeDescriptorV1* d) {
    return !(d == nullptr || d->struct_size < sizeof(*d) ||
        d->version != NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 || d->flags != 0 ||
        d->reserved0 != 0 || d->reserved1 != 0 || d->query == nullptr ||
        d->current_key == nullptr || d->current_value == nullptr ||
        d->key_cache_bf16 == nullptr || d->value_cache_bf16 == nullptr || d->output == nullptr ||
        d->query_heads <= 0 || d->kv_heads <= 0 || d->query_heads % d->kv_heads != 0 ||
        d->head_dim <= 0 || d->head_dim > kMaxHeadDim || d->position < 0 ||
        d->position == kLimit || d->first_key_position < 0 ||
        d->first_key_position > d->position || d->cache_capacity <= 0 ||
        d->cache_row_stride <= 0 || !positive_finite(d->scale) ||
        !cache_rows_fit(d->kv_heads, d->head_dim, d->cache_row_stride) ||
        d->query_heads > std::numeric_limits<std::int32_t>::max());
}

bool block_descriptor_valid(const NfnNativeTileDFlashBlockAttentionDescriptorV1* d) {
    return d != nullptr && d->struct_size >= sizeof(*d) &&
        d->version == NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 &&
        (d->flags & ~static_cast<std::uint32_t>(NFN_NATIVE_TILE_BLOCK_ATTENTION_CAUSAL)) == 0 &&
        d->reserved0 == 0 && d->reserved1 == 0 && d->query != nullptr &&
        d->block_key != nullptr && d->block_value != nullptr && d->key_cache_bf16 != nullptr &&
        d->value_cache_bf16 != nullptr && d->output != nullptr && d->query_rows > 0 &&
        d->block_rows > 0 && d->query_rows <= d->block_rows && d->block_rows <= kMaxBlockRows &&
        d->query_heads > 0 && d->kv_heads > 0 && d->query_heads % d->kv_heads == 0 &&
        d->head_dim > 0 && d->head_dim <= kMaxHeadDim && d->context_length >= 0 &&
        d->context_length <= kLimit - kMaxBlockRows && d->sliding_window > 0 &&
        d->cache_capacity >= d->sliding_window && d->cache_row_stride > 0 &&
        positive_finite(d->scale) &&
        cache_rows_fit(d->kv_heads, d->head_dim, d->cache_row_stride) &&
        d->query_heads <= std::numeric_limits<std::int32_t>::max() / kMaxBlockRows;
}

// Shared body of the fused decode entry points; device_position null = the
// position and first key of the descriptor; split_partials non-null = the
// split attention form with that workspace.
int run_fused_decode(const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* d,
                     const std::int64_t* device_position, std::int64_t sliding_window,
                     float* split_partials) {
    const bool on_device = device_position != nullptr;
    if (d == nullptr || d->struct_size < sizeof(*d) ||
        d->version != NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 || d->flags != 0 ||
        d->reserved0 != 0 || d->reserved1 != 0 || d->current_value == nullptr ||
        d->key_cache_bf16 == nullptr || d->value_cache_bf16 == nullptr || d->output == nullptr ||
        d->query_heads > 256 || d->position == kLimit || d->first_key_position < 0 ||
        d->first_key_position > d->position || d->cache_capacity <= 0 ||
        d->cache_row_stride <= 0 || !positive_finite(d->attention_scale) ||
        d->has_query_norm_weight > 1 || d->has_key_norm_weight > 1 ||
        d->query_norm_centered > 1 || d->key_norm_centered > 1 || d->apply_rope > 1 ||
        (on_device && (sliding_window <= 0 || sliding_window > d->cache_capacity))) {
        return kInvalid;
    }
    Descriptor query_weight{}, key_weight{};
    const Descriptor* query_source = d->has_query_norm_weight != 0 ? &d->query_norm_weight : nullptr;
    const Descriptor* key_source = d->has_key_norm_weight != 0 ? &d->key_norm_weight : nullptr;
    if (!qk_norm_arguments_valid(d->query, d->key, query_source, key_source, 1, d->query_heads,
                                 d->kv_heads, d->head_dim, d->norm_eps, d->query_scale,
                                 d->position, d->rope_theta, d->rope_layout, &query_weight,
                                 &key_weight) ||
        !cache_rows_fit(d->kv_heads, d->head_dim, d->cache_row_stride)) {
        return kInvalid;
    }
    const hipStream_t stream = as_stream(d->cuda_stream);
    if (split_partials == nullptr) split_partials = lent_partials(d->cuda_stream, d->query_heads, d->head_dim);
    // The new cache row is written by the first launch, before the attention
    // runs: right as long as the attention does not read that ring row, which
    // holds for every key range shorter than the ring (and for the device
    // form, whose window is at most the ring).  Otherwise the commit follows.
    const bool commit_first = on_device || d->position - d->first_key_position < d->cache_capacity;
    launch_qk_norm_scale_rope(d->query, d->key, query_source != nullptr ? &query_weight : nullptr,
                              d->query_norm_centered != 0,
                              key_source != nullptr ? &key_weight : nullptr,
                              d->key_norm_centered != 0, 1, d->query_heads, d->kv_heads,
                              d->head_dim, d->norm_eps, d->query_scale, d->position,
                              device_position, d->rope_theta,
                              d->rope_layout == NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED,
                              d->apply_rope != 0, commit_first ? d->key_cache_bf16 : nullptr,
                              d->value_cache_bf16, d->current_value, d->cache_capacity,
                              d->cache_row_stride, stream);
    NfnNativeTileGlimmerGqaDecodeDescriptorV1 attention{};
    attention.query = d->query;
    attention.current_key = d->key;
    attention.current_value = d->current_value;
    attention.key_cache_bf16 = d->key_cache_bf16;
    attention.value_cache_bf16 = d->value_cache_bf16;
    attention.output = d->output;
    attention.query_heads = d->query_heads;
    attention.kv_heads = d->kv_heads;
    attention.head_dim = d->head_dim;
    attention.position = d->position;
    attention.first_key_position = d->first_key_position;
    attention.cache_capacity = d->cache_capacity;
    attention.cache_row_stride = d->cache_row_stride;
    attention.scale = d->attention_scale;
    if (on_device && split_partials != nullptr) {
        launch_gqa_decode_split_device_position(attention, device_position, sliding_window,
                                                d->apply_rope == 0, split_partials, stream);
    } else if (on_device) {
        // a local layer (rope applied) sees its window, a global one everything
        launch_gqa_decode_device_position(attention, device_position, sliding_window,
                                          d->apply_rope == 0, stream);
    } else if (split_partials != nullptr) {
        launch_gqa_decode_split(attention, split_partials, stream);
    } else {
        launch_gqa_decode(attention, stream);
    }
    if (!commit_first) {
        launch_cache_commit(d->key, d->current_value, d->key_cache_bf16, d->value_cache_bf16,
                            d->kv_heads * d->head_dim, 1, d->position, nullptr, d->cache_capacity,
                            d->cache_row_stride, stream);
    }
    return launch_status();
}

}  // namespace

}  // namespace nfn

using namespace nfn;

extern "C" {

int nfn_native_tile_glimmer_embedding_gather_float32_v1(const Descriptor* descriptor,
                                                        std::int64_t token_id, float* output) {
    Descriptor table{};
    if (!normalize_descriptor(descriptor, &table) || token_id < 0 ||
        token_id >= table.output_dim || output == nullptr) {
        return kInvalid;
    }
    launch_embedding(table, 0, token_id, nullptr, output, 1, as_stream(table.cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_embedding_gather_device_i64_float32_v1(const Descriptor* descriptor,
                                                                   const std::int64_t* token_id,
                                                                   float* output) {
    Descriptor table{};
    if (!normalize_descriptor(descriptor, &table) || token_id == nullptr || output == nullptr) {
        return kInvalid;
    }
    launch_embedding(table, 1, 0, token_id, output, 1, as_stream(table.cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_embedding_batch_i32_float32_v1(const Descriptor* descriptor,
                                                           const std::int32_t* token_ids,
                                                           float* output, std::int64_t rows) {
    Descriptor table{};
    if (!normalize_descriptor(descriptor, &table) || token_ids == nullptr || output == nullptr ||
        rows <= 0 || rows > kLimit / table.input_dim) {
        return kInvalid;
    }
    launch_embedding(table, 2, 0, token_ids, output, rows, as_stream(table.cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_positioned_rope_float32_v1(float* query, float* key,
                                                       std::int64_t query_heads,
                                                       std::int64_t kv_heads,
                                                       std::int64_t head_dim,
                                                       std::int64_t position, float theta,
                                                       std::uint32_t layout, void* cuda_stream) {
    if (!rope_arguments_valid(query, key, 1, query_heads, kv_heads, head_dim, position, theta,
                              layout)) {
        return kInvalid;
    }
    launch_rope(query, key, 1, query_heads, kv_heads, head_dim, position, theta,
                layout == NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED, false, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_positioned_rope_batch_float32_v1(
    float* query, float* key, std::int64_t rows, std::int64_t query_heads, std::int64_t kv_heads,
    std::int64_t head_dim, std::int64_t start_position, float theta, std::uint32_t layout,
    bool inverse, void* cuda_stream) {
    if (!rope_arguments_valid(query, key, rows, query_heads, kv_heads, head_dim, start_position,
                              theta, layout)) {
        return kInvalid;
    }
    launch_rope(query, key, rows, query_heads, kv_heads, head_dim, start_position, theta,
                layout == NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED, inverse,
                as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1(
    float* query, float* key, const Descriptor* query_norm_weight,
    const Descriptor* key_norm_weight, std::int64_t rows, std::int64_t query_heads,
    std::int64_t kv_heads, std::int64_t head_dim, float eps, bool query_norm_centered,
    bool key_norm_centered, float query_scale, std::int64_t position, float theta,
    std::uint32_t layout, bool apply_rope, void* cuda_stream) {
    Descriptor query_weight{}, key_weight{};
    if (!qk_norm_arguments_valid(query, key, query_norm_weight, key_norm_weight, rows, query_heads,
                                 kv_heads, head_dim, eps, query_scale, position, theta, layout,
                                 &query_weight, &key_weight)) {
        return kInvalid;
    }
    launch_qk_norm_scale_rope(query, key, query_norm_weight != nullptr ? &query_weight : nullptr,
                              query_norm_centered,
                              key_norm_weight != nullptr ? &key_weight : nullptr,
                              key_norm_centered, rows, query_heads, kv_heads, head_dim, eps,
                              query_scale, position, nullptr, theta,
                              layout == NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED, apply_rope,
                              nullptr, nullptr, nullptr, 0, 0, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_qk_norm_scale_rope_float32_v1(
    float* query, float* key, const Descriptor* query_norm_weight,
    const Descriptor* key_norm_weight, std::int64_t query_heads, std::int64_t kv_heads,
    std::int64_t head_dim, float eps, bool query_norm_centered, bool key_norm_centered,
    float query_scale, std::int64_t position, float theta, std::uint32_t layout, bool apply_rope,
    void* cuda_stream) {
    return nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1(
        query, key, query_norm_weight, key_norm_weight, 1, query_heads, kv_heads, head_dim, eps,
        query_norm_centered, key_norm_centered, query_scale, position, theta, layout, apply_rope,
        cuda_stream);
}

int nfn_native_tile_glimmer_fused_decode_attention_float32_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* d) {
    return run_fused_decode(d, nullptr, 0, nullptr);
}

int nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* d,
    const std::int64_t* device_position, std::int64_t sliding_window) {
    if (device_position == nullptr) return kInvalid;
    return run_fused_decode(d, device_position, sliding_window, nullptr);
}

int nfn_mi355_fused_decode_attention_split_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* d, void* workspace,
    std::int64_t workspace_nbytes) {
    if (d == nullptr || workspace == nullptr ||
        reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    const std::int64_t required =
        nfn_mi355_gqa_decode_split_workspace_bytes_v1(d->query_heads, d->head_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    return run_fused_decode(d, nullptr, 0, static_cast<float*>(workspace));
}

int nfn_mi355_fused_decode_attention_split_device_position_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* d,
    const std::int64_t* device_position, std::int64_t sliding_window, void* workspace,
    std::int64_t workspace_nbytes) {
    if (d == nullptr || device_position == nullptr || workspace == nullptr ||
        reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    const std::int64_t required =
        nfn_mi355_gqa_decode_split_workspace_bytes_v1(d->query_heads, d->head_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    return run_fused_decode(d, device_position, sliding_window, static_cast<float*>(workspace));
}

int nfn_native_tile_glimmer_gqa_decode_float32_v1(
    const NfnNativeTileGlimmerGqaDecodeDescriptorV1* d) {
    if (!gqa_descriptor_valid(d)) return kInvalid;
    if (float* partials = lent_partials(d->cuda_stream, d->query_heads, d->head_dim)) {
        launch_gqa_decode_split(*d, partials, as_stream(d->cuda_stream));
    } else {
        launch_gqa_decode(*d, as_stream(d->cuda_stream));
    }
    return launch_status();
}

int nfn_mi355_attention_workspace_v1(void* workspace, std::int64_t workspace_nbytes,
                                     void* cuda_stream) {
    if ((workspace == nullptr) != (workspace_nbytes == 0) || workspace_nbytes < 0 ||
        reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    int device = -1;
    if (hipGetDevice(&device) != hipSuccess) return kInvalid;
    std::lock_guard<std::mutex> guard(lent_mutex);
    LentWorkspace* slot = nullptr;
    for (LentWorkspace& loan : lent_workspaces) {
        if (loan.memory != nullptr && loan.device == device && loan.stream == cuda_stream) {
            slot = &loan;
            break;
        }
        if (loan.memory == nullptr && slot == nullptr) slot = &loan;
    }
    if (workspace == nullptr) {  // taking back what was never lent is not an error
        if (slot != nullptr && slot->memory != nullptr) *slot = LentWorkspace{};
        return 0;
    }
    if (slot == nullptr) return kInvalid;  // every slot holds another stream's loan
    slot->device = device;
    slot->stream = cuda_stream;
    slot->memory = static_cast<float*>(workspace);
    slot->nbytes = workspace_nbytes;
    return 0;
}

std::int64_t nfn_mi355_gqa_decode_split_workspace_bytes_v1(std::int64_t query_heads,
                                                           std::int64_t head_dim) {
    if (query_heads <= 0 || query_heads > std::numeric_limits<std::int32_t>::max() ||
        head_dim <= 0 || head_dim > kMaxHeadDim) {
        return 0;
    }
    return (gqa_decode_split_workspace_bytes(query_heads, head_dim) + 255) & ~std::int64_t(255);
}

int nfn_mi355_gqa_decode_split_v1(const NfnNativeTileGlimmerGqaDecodeDescriptorV1* d,
                                  void* workspace, std::int64_t workspace_nbytes) {
    if (!gqa_descriptor_valid(d) || workspace == nullptr ||
        reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    const std::int64_t required =
        nfn_mi355_gqa_decode_split_workspace_bytes_v1(d->query_heads, d->head_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    launch_gqa_decode_split(*d, static_cast<float*>(workspace), as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_cache_commit_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitDescriptorV1* d) {
    if (!commit_descriptor_valid(d) || d->kv_heads * d->head_dim > kMaxThreads) return kInvalid;
    launch_cache_commit(d->current_key, d->current_value, d->key_cache_bf16, d->value_cache_bf16,
                        d->kv_heads * d->head_dim, 1, d->position, nullptr, d->cache_capacity,
                        d->cache_row_stride, as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_cache_commit_rows_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitDescriptorV1* d, std::int64_t rows) {
    if (!commit_descriptor_valid(d) || rows <= 0 || rows > kMaxBlockRows ||
        d->position > kLimit - rows || d->kv_heads * d->head_dim > kMaxThreads / rows) {
        return kInvalid;
    }
    launch_cache_commit(d->current_key, d->current_value, d->key_cache_bf16, d->value_cache_bf16,
                        d->kv_heads * d->head_dim, rows, d->position, nullptr, d->cache_capacity,
                        d->cache_row_stride, as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_native_tile_dflash_block_attention_float32_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* d) {
    if (!block_descriptor_valid(d)) return kInvalid;
    const LentWorkspace lent = lent_here(d->cuda_stream);
    launch_block_attention(*d, lent.memory, lent.nbytes, as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_mi355_dflash_block_attention_split_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* d, void* workspace,
    std::int64_t workspace_nbytes) {
    if (!block_descriptor_valid(d) || workspace == nullptr || workspace_nbytes <= 0 ||
        reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    launch_block_attention(*d, static_cast<float*>(workspace), workspace_nbytes,
                           as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_cache_commit_layers_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitLayersDescriptorV1* d) {
    if (d == nullptr || d->struct_size < sizeof(*d) ||
        d->version != NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 || d->flags != 0 ||
        d->reserved0 != 0 || d->reserved1 != 0 || d->reserved2 != 0 ||
        d->staged_keys == nullptr || d->staged_values == nullptr || d->layers == nullptr ||
        d->layer_count <= 0 || d->layer_count > 64 || d->source_rows <= 0 ||
        d->source_rows > kMaxBlockRows || d->rows <= 0 || d->rows > d->source_rows ||
        d->kv_heads <= 0 || d->head_dim <= 0 || d->head_dim > kMaxHeadDim || d->position < 0 ||
        d->position > kLimit - d->rows || d->source_layer_stride <= 0 ||
        d->kv_heads > kMaxThreads / d->head_dim) {
        return kInvalid;
    }
    const std::int64_t width = d->kv_heads * d->head_dim;
    if (width > kLimit / d->source_rows || d->source_layer_stride < d->source_rows * width ||
        d->source_layer_stride > kLimit / d->layer_count) {
        return kInvalid;
    }
    for (std::int64_t index = 0; index < d->layer_count; ++index) {
        const NfnNativeTileGlimmerCacheLayerV1& layer = d->layers[index];
        if (layer.key_cache_bf16 == nullptr || layer.value_cache_bf16 == nullptr ||
            layer.cache_capacity <= 0 || layer.cache_row_stride < width) {
            return kInvalid;
        }
    }
    launch_cache_commit_layers(*d, as_stream(d->cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_pack_target_taps_float32_v1(const float* tap_major, float* row_major,
                                                        std::int64_t source_rows,
                                                        std::int64_t source_row_offset,
                                                        std::int64_t rows, std::int64_t tap_count,
                                                        std::int64_t hidden_width,
                                                        void* cuda_stream) {
    if (tap_major == nullptr || row_major == nullptr || source_rows <= 0 ||
        source_rows > kMaxBlockRows || source_row_offset < 0 || rows <= 0 ||
        rows > kMaxBlockRows || source_row_offset + rows > source_rows || tap_count <= 0 ||
        tap_count > 64 || hidden_width <= 0 || hidden_width > 65536) {
        return kInvalid;
    }
    launch_pack_target_taps(tap_major, row_major, source_rows, source_row_offset, rows, tap_count,
                            hidden_width, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_dflash_block_attention_short_split_float32_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* d, float* score_workspace,
    std::int64_t score_workspace_nbytes) {
    // the reference's geometry (glimmer_k_mmq.cu:1928-1929, 2432-2472): tiles of 8 keys, 128 keys at most
    constexpr std::int64_t kKeysPerScoreTile = 8;
    constexpr std::int64_t kMaxKeys = 128;
    if (d == nullptr || score_workspace == nullptr || d->query_rows <= 0 || d->query_rows > 16 ||
        d->query_heads != 32 || d->head_dim != 128 || d->cuda_stream == nullptr ||
        d->block_rows <= 0 || d->context_length < 0 || d->sliding_window <= 0 ||
        d->context_length > kLimit - kMaxBlockRows) {
        return kInvalid;
    }
    const std::int64_t available = d->context_length + d->block_rows;
    const std::int64_t maximum_keys = d->sliding_window < available ? d->sliding_window : available;
    if (maximum_keys > kMaxKeys) return kInvalid;
    const std::int64_t score_tiles = (maximum_keys + kKeysPerScoreTile - 1) / kKeysPerScoreTile;
    const std::int64_t score_count = d->query_rows * d->query_heads * score_tiles * kKeysPerScoreTile;
    if (score_workspace_nbytes < score_count * 4) return kInvalid;
    // everything else is the general entry point's business, checks included
    return nfn_native_tile_dflash_block_attention_float32_v1(d);
}

int nfn_native_tile_glimmer_logit_transform_float32_v1(float* logits, std::int64_t count,
                                                       float multiplier, float softcap,
                                                       void* cuda_stream) {
    if (logits == nullptr || count <= 0 || !positive_finite(multiplier) ||
        !positive_finite(softcap)) {
        return kInvalid;
    }
    launch_logit_transform(logits, count, multiplier, softcap, as_stream(cuda_stream));
    return launch_status();
}

// The reference checks only the count here (tile_ops.cu:6377-6388); null
// pointers would fault in its kernel, this build refuses them.
int nfn_native_tile_add_float32(const float* lhs, const float* rhs, float* out, std::int64_t n,
                                void* cuda_stream) {
    if (n <= 0 || lhs == nullptr || rhs == nullptr || out == nullptr) return kInvalid;
    launch_add(lhs, rhs, out, n, as_stream(cuda_stream));
    return launch_status();
}

// The reference launches whatever it is given (tile_ops.cu:6944-6951); an
// empty or null array is refused here, anything else is scaled.
int nfn_native_tile_scale_inplace_float32(float* values, std::int64_t n, float scale,
                                          void* cuda_stream) {
    if (values == nullptr || n <= 0) return kInvalid;
    launch_scale(values, n, scale, as_stream(cuda_stream));
    return launch_status();
}

}  // extern "C"
