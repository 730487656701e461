// Descriptor validation: the fail-closed gate in front of every launch.
// Follows normalize_packed_weight_descriptor
// (neuralfn/csrc/native_train/tile_ops.cu:3303-3366) and the stricter
// small-batch validator (neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:1363-1390).
#include "common.hpp"

#include <limits>

namespace nfn {

namespace {

bool checked_positive_product(std::int64_t left, std::int64_t right, std::int64_t* output) {
    if (left <= 0 || right <= 0 ||
        left > std::numeric_limits<std::int64_t>::max() / right) {
        return false;
    }
    *output = left * right;
    return true;
}

}  // namespace

bool normalize_descriptor(const Descriptor* source, Descriptor* output) {
    if (source == nullptr || output == nullptr ||
        source->struct_size < sizeof(Descriptor) ||
        source->version != NFN_NATIVE_TILE_PACKED_WEIGHT_V1 || source->flags != 0 ||
        source->reserved0 != 0 || source->reserved1 != 0 || source->data == nullptr ||
        source->data_nbytes <= 0 || source->output_dim <= 0 || source->input_dim <= 0 ||
        source->row_stride_bytes <= 0) {
        return false;
    }
    // device addresses have 48 bits (the decode kernels pass four of them in six dwords)
    if ((reinterpret_cast<std::uintptr_t>(source->data) >> 48) != 0) return false;
    const std::int64_t elements = block_elements(source->encoding);
    const std::int64_t bytes = block_bytes(source->encoding);
    if (elements == 0 || source->input_dim % elements != 0) {
        return false;  // unknown encodings never fall through to a float read
    }
    std::int64_t stride = 0;
    std::int64_t total = 0;
    if (!checked_positive_product(source->input_dim / elements, bytes, &stride) ||
        !checked_positive_product(source->output_dim, stride, &total) ||
        source->row_stride_bytes != stride || source->data_nbytes != total) {
        return false;
    }
    *output = *source;
    output->struct_size = sizeof(Descriptor);
    return true;
}

bool validate_k_descriptor(const Descriptor* descriptor, std::int64_t input_dim,
                           void* stream, bool allow_q8_0) {
    Descriptor normalized;
    if (!normalize_descriptor(descriptor, &normalized)) return false;
    if (normalized.input_dim != input_dim || input_dim % 256 != 0) return false;
    if (!is_k_quant(normalized.encoding) &&
        !(allow_q8_0 && normalized.encoding == kEncQ8_0)) {
        return false;
    }
    // A descriptor may name no stream or the stream of the call, nothing else.
    return normalized.cuda_stream == nullptr || normalized.cuda_stream == stream;
}

}  // namespace nfn
