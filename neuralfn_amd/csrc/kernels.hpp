// Launchers implemented by the .hip files; called by the C ABI in abi.cpp.
#pragma once

#include "common.hpp"

namespace nfn {

// dequant.hip
void launch_dequantize(const Descriptor& descriptor, float* output, hipStream_t stream);

// gemv_f32.hip — exact float-activation path, rows in tiles of up to 8.
void launch_gemv_f32(ProjectionSet set, const float* first, const float* second, int prologue,
                     const float* bias, std::int64_t rows, hipStream_t stream);

// gemm_f32.hip — the same arithmetic on the float matrix cores, for many rows of one
// projection: input_dim a multiple of 32.  gemm_f32_tile_passes: how many of its
// 128 x 64 tiles a compute unit works through one after another (at least 1).
bool gemm_f32_supports(const Descriptor& weight, std::int64_t rows);
double gemm_f32_tile_passes(const Descriptor& weight, std::int64_t rows);
void launch_gemm_f32(const Descriptor& weight, const float* input, const float* bias,
                     float* output, std::int64_t rows, hipStream_t stream);

// q8_1.hip — the public int8-activation path.
void launch_quantize_q8_1(const float* input, std::int8_t* codes, float* scales, float* sums,
                          std::int64_t rows, std::int64_t width, hipStream_t stream);
void launch_linear_q8_1(ProjectionSet set, const std::int8_t* codes, const float* scales,
                        const float* sums, const float* bias, std::int64_t rows,
                        hipStream_t stream);

// argmax.hip
void launch_argmax_rows(const float* values, std::int64_t* indices, float* maxima,
                        std::int64_t rows, std::int64_t width, hipStream_t stream);

// elementwise.hip
void launch_sigmoid_gate(const float* values, const float* gate, float* output,
                         std::int64_t count, hipStream_t stream);
void launch_swiglu(const float* gate, const float* up, float* output, std::int64_t count,
                   hipStream_t stream);

// rms.hip — two adjacent RMS normalisations of the decode loop in one launch;
// `records` (may be null, else one row only): the small-batch workspace that
// receives the activation records of normalized_output.  `half_image` (may be null,
// else rows of at most 8,192 columns): the small-batch workspace of `rows` rows that
// receives normalized_output as the fp16 small-batch kernel's image.  `operand_image` (may
// be null; with `records`, rows of at most 8,192 columns): the records are those of all
// `rows` rows, token by token, and the same codes go to `operand_image` in the order the
// exact verifier's matrix-core kernel reads them (gemv_rows.hpp).
void launch_dual_rms_add_capture(const float* input, const Descriptor* first_weight,
                                 bool first_centered, const float* residual_input,
                                 float* hidden_output, const Descriptor* second_weight,
                                 bool second_centered, float* normalized_output,
                                 float* residual_output, std::int64_t rows, std::int64_t width,
                                 float first_eps, float second_eps, std::uint8_t* records,
                                 std::uint8_t* half_image, hipStream_t stream,
                                 std::uint8_t* operand_image = nullptr);

// One normalisation: output = rms(input, weight, eps) (+ residual_input when
// given); residual_output (may be null) receives a copy of the input; the
// q8 pointers (all or none) receive the public Q8_1 form of the output.
void launch_rms_norm(const float* input, const Descriptor* weight, bool centered,
                     const float* residual_input, float* output, float* residual_output,
                     std::int8_t* q8_codes, float* q8_scales, float* q8_sums, std::int64_t rows,
                     std::int64_t width, float eps, hipStream_t stream);

// rms.hip — per-head Q/K normalisation, query scale and rotary embedding of
// `rows` rows in one launch; row r is at position + r.  A non-null
// device_position replaces `position` when the kernel runs.  With key_cache
// non-null (rows == 1) the new key and current_value rows also go to the bf16
// rings at `position`.
void launch_qk_norm_scale_rope(float* query, float* key, const Descriptor* query_weight,
                               bool query_centered, const Descriptor* key_weight,
                               bool key_centered, std::int64_t rows, std::int64_t query_heads,
                               std::int64_t kv_heads, std::int64_t head_dim, float eps,
                               float query_scale, std::int64_t position,
                               const std::int64_t* device_position, float theta,
                               bool interleaved, bool apply_rope, std::uint16_t* key_cache,
                               std::uint16_t* value_cache, const float* current_value,
                               std::int64_t cache_capacity, std::int64_t cache_row_stride,
                               hipStream_t stream);

// engine_ops.hip — the small operators around the packed linears.
// token_source: 0 = host_token, 1 = one int64 in device memory, 2 = int32 per row.
void launch_embedding(const Descriptor& table, int token_source, std::int64_t host_token,
                      const void* device_tokens, float* output, std::int64_t rows,
                      hipStream_t stream);
void launch_rope(float* query, float* key, std::int64_t rows, std::int64_t query_heads,
                 std::int64_t kv_heads, std::int64_t head_dim, std::int64_t start_position,
                 float theta, bool interleaved, bool inverse, hipStream_t stream);
void launch_cache_commit(const float* keys, const float* values, std::uint16_t* key_cache,
                         std::uint16_t* value_cache, std::int64_t width, std::int64_t rows,
                         std::int64_t position, const std::int64_t* device_position,
                         std::int64_t capacity, std::int64_t row_stride, hipStream_t stream);
void launch_cache_commit_layers(const NfnNativeTileGlimmerCacheCommitLayersDescriptorV1& descriptor,
                                hipStream_t stream);
void launch_pack_target_taps(const float* tap_major, float* row_major, std::int64_t source_rows,
                             std::int64_t source_row_offset, std::int64_t rows,
                             std::int64_t tap_count, std::int64_t hidden_width,
                             hipStream_t stream);
void launch_logit_transform(float* logits, std::int64_t count, float multiplier, float softcap,
                            hipStream_t stream);
void launch_add(const float* lhs, const float* rhs, float* out, std::int64_t count,
                hipStream_t stream);
void launch_scale(float* values, std::int64_t count, float scale, hipStream_t stream);

// attention.hip — descriptors already checked.
void launch_gqa_decode(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& descriptor,
                       hipStream_t stream);
// `partials` (16-byte aligned, `partial_bytes` bytes) or null: with it the keys of every
// row are shared out over workgroups as in the split one-token form.
void launch_block_attention(const NfnNativeTileDFlashBlockAttentionDescriptorV1& descriptor,
                            float* partials, std::int64_t partial_bytes, hipStream_t stream);
// One-token attention with the keys of every head dealt over several
// workgroups; `partials` holds gqa_decode_split_workspace_bytes() bytes.
// One-token attention whose position is read from device memory when the kernel
// runs; the keys are the last `sliding_window` ones, or all when whole_context.
void launch_gqa_decode_device_position(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& descriptor,
                                       const std::int64_t* device_position,
                                       std::int64_t sliding_window, bool whole_context,
                                       hipStream_t stream);
std::int64_t gqa_decode_split_workspace_bytes(std::int64_t query_heads, std::int64_t head_dim);
void launch_gqa_decode_split(const NfnNativeTileGlimmerGqaDecodeDescriptorV1& descriptor,
                             float* partials, hipStream_t stream);
// The same with the position read from device memory when the kernels run (the
// meaning of `sliding_window` and `whole_context` as in the one-launch form).
void launch_gqa_decode_split_device_position(
    const NfnNativeTileGlimmerGqaDecodeDescriptorV1& descriptor, const std::int64_t* device_position,
    std::int64_t sliding_window, bool whole_context, float* partials, hipStream_t stream);

}  // namespace nfn
