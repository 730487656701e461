/*
 * C ABI of libnfn_mi355_tile_ops.so — the K-Quant packed-linear operators of
 * NeuralFn's tile-ops sidecar, implemented for AMD MI355X (gfx950).
 *
 * Every `nfn_native_tile_*` entry point below keeps the name, argument order
 * and meaning of the declaration it replaces in the reference's
 * neuralfn/csrc/native_train/tile_ops.h (cited per function), so the
 * reference's resident engine can dlopen this library through its
 * `tile_ops_lib` option.  `nfn_mi355_*` entry points are additions; each says
 * what it adds and that no reference counterpart exists.
 *
 * Conventions (reference: tile_ops.cu:4504-4713, glimmer_k_mmq.cu:2349-2649):
 *  - Return `int`: 0 on success, 1 (invalid value) for every argument or
 *    descriptor violation, any other value is a HIP runtime error code that
 *    nfn_native_tile_ops_error_string() turns into text.
 *  - All data pointers are device pointers.  Descriptor structs and arrays of
 *    descriptor/output pointers are host memory, read during the call only.
 *  - The caller owns every buffer.  No entry point allocates, frees,
 *    synchronises or keeps a pointer after it returns.
 *  - `cuda_stream` is an opaque stream handle: here a hipStream_t.  Null is the
 *    default stream.  Entry points without a stream argument use
 *    descriptor->cuda_stream.
 *  - Work is enqueued; the status reflects argument checks and the launch.
 *  - Tensors: input [rows, input_dim] row-major float; each output
 *    [rows, output_dim] row-major float; bias [output_dim] float, added after
 *    the reduction.
 */
#ifndef NFN_MI355_TILE_OPS_H
#define NFN_MI355_TILE_OPS_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Encoding ids (tile_ops.h:11-26).  8 = ggml Q8_0 is an addition: the reference
 * accepts only 0, 12, 13, 14, 30 (and a training-only 31, rejected here). */
enum {
    NFN_NATIVE_TILE_PACKED_WEIGHT_V1 = 1,
    NFN_NATIVE_TILE_K_QUANT_MMQ_V1 = 1,
    NFN_NATIVE_TILE_PACKED_WEIGHT_F32 = 0,
    NFN_MI355_PACKED_WEIGHT_Q8_0 = 8,
    NFN_NATIVE_TILE_PACKED_WEIGHT_Q4_K = 12,
    NFN_NATIVE_TILE_PACKED_WEIGHT_Q5_K = 13,
    NFN_NATIVE_TILE_PACKED_WEIGHT_Q6_K = 14,
    NFN_NATIVE_TILE_PACKED_WEIGHT_BF16 = 30
};

/* One [output_dim, input_dim] row-major packed matrix (tile_ops.h:293-307).
 * 72 bytes.  Row r starts at data + r*row_stride_bytes; rows are unpadded:
 * row_stride_bytes == input_dim/block_elements*block_bytes and
 * data_nbytes == output_dim*row_stride_bytes, or validation fails. */
typedef struct NfnNativeTilePackedWeightDescriptorV1 {
    uint32_t struct_size;
    uint32_t version;   /* NFN_NATIVE_TILE_PACKED_WEIGHT_V1 */
    uint32_t encoding;
    uint32_t flags;     /* 0 */
    const uint8_t* data;
    int64_t data_nbytes;
    int64_t output_dim;
    int64_t input_dim;
    int64_t row_stride_bytes;
    uint32_t reserved0; /* 0 */
    uint32_t reserved1; /* 0 */
    void* cuda_stream;
} NfnNativeTilePackedWeightDescriptorV1;

/* ---- versions (tile_ops.h:601-606; engine requires the first four == 1,
 *      resident_glimmer_cuda.cpp:496-501) -------------------------------- */
int nfn_native_tile_ops_abi_version(void);
int nfn_native_tile_strict_math_abi_version(void);
int nfn_native_tile_packed_weight_abi_version(void);
int nfn_native_tile_glimmer_inference_abi_version(void);
int nfn_native_tile_k_quant_mmq_abi_version(void);

/* tile_ops.h:1096.  Never returns null. */
const char* nfn_native_tile_ops_error_string(int code);

/* ---- validation and dequantization (tile_ops.h:609-613) ----------------- */
int nfn_native_tile_packed_weight_validate_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor);
/* output: [output_dim, input_dim] float, bit-exact with the reference's
 * packed_weight_value_device (kernels.cu:1225-1322). */
int nfn_native_tile_packed_weight_dequantize_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    float* output);

/* ---- generic float-activation linear, any row count (tile_ops.h:614-620):
 *      float weights times float activations, no quantization of the input.
 *      It has no workspace argument, so every row count keeps that float
 *      arithmetic (17 rows and more on the float matrix instruction);
 *      nfn_mi355_k_quant_gemm_float32_v1 is the fp16 matrix-core route. -- */
int nfn_native_tile_linear_packed_weight_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const float* input,
    const float* bias,
    float* output,
    int64_t rows,
    bool has_bias);

/* ---- public Q8_1 activation path (tile_ops.h:624-640, 743-756) ----------
 * q8_values: rows*width int8; q8_scales, q8_sums: rows*(width/32) float. */
int nfn_native_tile_quantize_q8_1_float32_v1(
    const float* input,
    int8_t* q8_values,
    float* q8_scales,
    float* q8_sums,
    int64_t rows,
    int64_t width,
    void* cuda_stream);
int nfn_native_tile_linear_packed_weight_q8_1_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const int8_t* q8_values,
    const float* q8_scales,
    const float* q8_sums,
    const float* bias,
    float* output,
    int64_t rows,
    bool has_bias);
int nfn_native_tile_linear_packed_weight_q8_1_multi_decode_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor0,
    const NfnNativeTilePackedWeightDescriptorV1* descriptor1,
    const NfnNativeTilePackedWeightDescriptorV1* descriptor2,
    const NfnNativeTilePackedWeightDescriptorV1* descriptor3,
    const int8_t* q8_values,
    const float* q8_scales,
    const float* q8_sums,
    float* output0,
    float* output1,
    float* output2,
    float* output3,
    int64_t projection_count,
    void* cuda_stream);

/* ---- decode / small-batch K-quant path (tile_ops.h:647-739) --------------
 * 1..4 projections that share one input, rows 1..16, Q4_K/Q5_K/Q6_K (and
 * Q8_0 here).  `workspace` is caller-owned scratch whose layout is private to
 * this library; its size comes from the query.  The query returns 0 when rows
 * is outside 1..16 or input_dim is not a multiple of 128. */
int64_t nfn_native_tile_k_quant_mmq_workspace_bytes_v1(int64_t rows, int64_t input_dim);
int nfn_native_tile_k_quant_mmq_multi_linear_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* input,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* input := input / (1 + expf(-gate)), fused (tile_ops.h:659-672). */
int nfn_native_tile_k_quant_mmq_multi_linear_gated_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* input,
    const float* gate,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* input := (up * gate) * (1 / (1 + expf(-gate))), fused (tile_ops.h:673-684). */
int nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* gate,
    const float* up,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* Verifier variants: every row gets exactly the one-row arithmetic
 * (tile_ops.h:685-729). */
int nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* input,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* Same as the entry point above for an input whose activation records are
 * already in `workspace`: left there by one of the three
 * nfn_native_tile_k_quant_mmvq_multi_linear* entry points around this one,
 * called on that input with the same `rows`, or by the dual-RMS handoff below
 * (one row).  Skips only the
 * activation quantization (tile_ops.h:698-709).  Refused when a projection has
 * no kernel that reads the records. */
int nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
int nfn_native_tile_k_quant_mmvq_multi_linear_gated_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* input,
    const float* gate,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
int nfn_native_tile_k_quant_mmvq_multi_linear_swiglu_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* gate,
    const float* up,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* One-row decode GEMV (tile_ops.h:730-739). */
int nfn_native_tile_k_quant_mmvq_linear_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const float* input,
    float* output,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);
/* The gate and up projections of a feed-forward block for one token with the
 * SwiGLU activation at the row ends: output[r] = (up_r * gate_r) * sigmoid(gate_r),
 * output_dim floats.  No counterpart in the reference, whose engine runs the
 * grouped one-row call on [gate, up] and then
 * nfn_native_tile_k_quant_mmvq_multi_linear_swiglu_float32_v1 on the two
 * results (resident_glimmer_cuda.cpp:2233-2585, glimmer_k_mmq.cu:299-317):
 * here the down projection behind reads one plain vector of output_dim floats
 * instead of two, and the plain call on `output` gives the bits of the SwiGLU
 * call on the separate results.  gate and up: the same encoding (Q4_K or
 * Q5_K), shape and row stride; input_dim a multiple of 256, at most 8192. */
int nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* gate,
    const NfnNativeTilePackedWeightDescriptorV1* up,
    const float* input,
    float* output,
    void* cuda_stream);

/* The same pair for a block of 5..16 rows (a verifier block) on the fp16
 * small-batch kernel: output[row][r] = (up * gate) * sigmoid(gate) of the two
 * projections' results, rows x output_dim floats, which the plain small-batch
 * call behind then reads (the bits of the SwiGLU call on the separate results).
 * No counterpart in the reference (it runs the grouped small-batch call and
 * nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1,
 * tile_ops.h:650-684).  input null: the workspace already holds the rows as
 * nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1 left them.  gate and up: the
 * same encoding (Q4_K, Q5_K, Q6_K or Q8_0), shape and row stride; the workspace
 * as for the small-batch calls. */
int nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* gate,
    const NfnNativeTilePackedWeightDescriptorV1* up,
    const float* input,
    float* output,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);

/* ---- the normalisation step upstream of the decode projections ----------
 * hidden = residual_input + rms(input, first_weight, first_eps);
 * residual_output = hidden; normalized_output = rms(hidden, second_weight,
 * second_eps), with rms(x, w, eps) = x / sqrt(mean(x^2) + eps) * (w or 1, plus
 * 1 when centered).  A weight is null or a [1, width] F32/BF16 descriptor;
 * width <= 65536; eps finite and > 0 (tile_ops.h:836-858,
 * tile_ops.cu:4901-4950). */
/* One normalisation, output = rms(input, weight, eps), and its fused forms:
 * with a copy of the input kept as the residual, with that and the public
 * Q8_1 form of the output (bit-identical to nfn_native_tile_quantize_q8_1 run
 * on the output; width a multiple of 32), and with a residual added to the
 * result (tile_ops.h:786-829, tile_ops.cu:4777-4899). */
int nfn_native_tile_glimmer_rms_norm_affine_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* weight,
    float* output,
    int64_t rows,
    int64_t width,
    float eps,
    bool centered,
    void* cuda_stream);
int nfn_native_tile_glimmer_rms_norm_affine_capture_residual_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* weight,
    float* output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float eps,
    bool centered,
    void* cuda_stream);
int nfn_native_tile_glimmer_rms_norm_affine_capture_residual_q8_1_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* weight,
    float* output,
    float* residual_output,
    int8_t* q8_values,
    float* q8_scales,
    float* q8_sums,
    int64_t rows,
    int64_t width,
    float eps,
    bool centered,
    void* cuda_stream);
int nfn_native_tile_glimmer_rms_norm_affine_add_residual_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* weight,
    const float* residual_input,
    float* output,
    int64_t rows,
    int64_t width,
    float eps,
    bool centered,
    void* cuda_stream);
int nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    void* cuda_stream);
/* The reference's multi-row specialization of the entry point above: same
 * results, F32 norm weights only (tile_ops.h:859-873). */
int nfn_native_tile_glimmer_dual_rms_add_capture_cooperative_batch_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    void* cuda_stream);
/* One-row variant that also leaves the activation records of
 * normalized_output in the small-batch workspace, for
 * nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1
 * (tile_ops.h:874-894, tile_ops.cu:4952-5010).  rows must be 1, width a
 * multiple of 256, the workspace at least
 * nfn_native_tile_k_quant_mmq_workspace_bytes_v1(1, width) bytes. */
int nfn_native_tile_glimmer_dual_rms_add_capture_mmvq_q8_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    void* mmvq_workspace,
    int64_t mmvq_workspace_nbytes,
    void* cuda_stream);
/* The same handoff for a block of 5..16 rows (the verifier's block, a prefill
 * chunk): the reference's pair (tile_ops.h:874-894 producer, :698-709 consumer)
 * takes one row only, and at these row counts the small-batch entry points
 * spend a launch per call on converting their input.  Here the norm kernel
 * also leaves normalized_output in mmq_workspace in the form the
 * nfn_native_tile_k_quant_mmq_* calls convert their input to, and
 * nfn_mi355_k_quant_mmq_multi_linear_prequantized_float32_v1 multiplies from
 * it: the same bits as the mmq call on normalized_output, one launch less per
 * projection group.  width: a multiple of 256, at most 8192; the workspace at
 * least nfn_native_tile_k_quant_mmq_workspace_bytes_v1(rows, width) bytes; the
 * consumer fails closed unless every projection is Q4_K, Q5_K, Q6_K or Q8_0. */
int nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    void* mmq_workspace,
    int64_t mmq_workspace_nbytes,
    void* cuda_stream);

/* The handoff for a block of 4..16 rows in the exact verifier's family.  No counterpart in
 * the reference: its pair (tile_ops.h:874-894 producer, :698-709 consumer) takes one row,
 * and the engine's verifier therefore runs the norm and then
 * nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1, whose first launch here quantizes
 * the rows.  This producer leaves the activation records of all rows and their
 * matrix-operand copy in mmvq_workspace, as that launch would, and the reference's own
 * consumer nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1 (same rows, same
 * workspace) multiplies from them: the bits of the mmvq call on normalized_output, one
 * launch less per projection group.  width: a multiple of 256, at most 8192; the workspace
 * at least nfn_native_tile_k_quant_mmq_workspace_bytes_v1(rows, width) bytes. */
int nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t rows,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    void* mmvq_workspace,
    int64_t mmvq_workspace_nbytes,
    void* cuda_stream);
/* One row: the two normalisations and the projections of their result in one
 * launch.  No counterpart in the reference, whose engine calls
 * nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1 and then the grouped
 * one-row call on normalized_output (resident_glimmer_cuda.cpp:2890-2956):
 * here every workgroup of the projection launch normalises the row in its own
 * prologue (the arithmetic and the float order of the norm kernel,
 * kernels.cu:2155-2243) and the first also stores the three rows, which saves
 * the norm kernel's launch in front of a launch of one workgroup per compute
 * unit.  The same bits as the two calls.  The arguments up to second_centered
 * are those of the dual RMS call for one row; width a multiple of 256 up to
 * 8192; 1..4 projections of one encoding (Q4_K or Q5_K) and input_dim = width.
 * No aliasing: every workgroup reads `input` and `residual_input` while the
 * first one stores the three result rows, so hidden_output, normalized_output,
 * residual_output and the projection outputs must not overlap either input row
 * (status 1 otherwise).  A caller that normalises in place, as the engine does
 * with residual_output == residual_input, keeps its two calls or alternates
 * between two residual buffers. */
int nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1(
    const float* input,
    const NfnNativeTilePackedWeightDescriptorV1* first_weight,
    const float* residual_input,
    float* hidden_output,
    const NfnNativeTilePackedWeightDescriptorV1* second_weight,
    float* normalized_output,
    float* residual_output,
    int64_t width,
    float first_eps,
    bool first_centered,
    float second_eps,
    bool second_centered,
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    float* const* outputs,
    int64_t operation_count,
    void* cuda_stream);
int nfn_mi355_k_quant_mmq_multi_linear_prequantized_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);

/* ---- row argmax, ties to the lowest column (tile_ops.h:757-764) --------- */
int nfn_native_tile_argmax_rows_float32_v1(
    const float* values,
    int64_t* output_indices,
    float* output_values,
    int64_t rows,
    int64_t width,
    void* cuda_stream);

/* ---- element-wise operators the fused prologues must equal bit for bit
 *      (tile_ops.h:998-1003, 3251-3256) ----------------------------------- */
int nfn_native_tile_glimmer_sigmoid_gate_float32_v1(
    const float* values,
    const float* gate,
    float* output,
    int64_t count,
    void* cuda_stream);
int nfn_native_tile_swiglu_float32(
    const float* gate,
    const float* up,
    float* out,
    int64_t n,
    void* cuda_stream);

/* ==== the decode loop's remaining operators ===============================
 * The operators the reference's resident engine requires from the sidecar
 * besides the packed linears (resident_glimmer_cuda.cpp:431-495): token
 * embedding, rotary position embedding, one-token and block attention over a
 * bf16 cache, the cache commit, the logit transform, add and scale.
 * Arithmetic: the CPU engine's (resident_glimmer.cpp:773-800, 1716-1800,
 * 1895-1903), computed in float except where a comment says double. */

enum {
    NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 = 1,      /* tile_ops.h:34 */
    NFN_NATIVE_TILE_GLIMMER_ROPE_HALF_SPLIT = 0,   /* tile_ops.h:35 */
    NFN_NATIVE_TILE_GLIMMER_ROPE_INTERLEAVED = 1,  /* tile_ops.h:36 */
    NFN_NATIVE_TILE_BLOCK_ATTENTION_CAUSAL = 1     /* tile_ops.h:37 */
};

/* Row `token_id` of a packed [vocabulary, width] matrix, dequantized to
 * output[width] (tile_ops.h:770-785; bit-exact with ...dequantize_float32_v1).
 * The stream is descriptor->cuda_stream.  The first form checks the token on
 * the host; the device forms write zeros for a token outside the vocabulary. */
int nfn_native_tile_glimmer_embedding_gather_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    int64_t token_id,
    float* output);
int nfn_native_tile_glimmer_embedding_gather_device_i64_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const int64_t* token_id, /* device */
    float* output);
int nfn_native_tile_glimmer_embedding_batch_i32_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const int32_t* token_ids, /* device, [rows] */
    float* output,            /* [rows, width] */
    int64_t rows);

/* Rotary position embedding in place (tile_ops.h:895-904, 1016-1027):
 * query [rows, query_heads, head_dim], key [rows, kv_heads, head_dim]; row r
 * is at position start_position + r; pair i of a head is elements (i,
 * i + head_dim/2) for HALF_SPLIT and (2i, 2i+1) for INTERLEAVED; angle =
 * position / theta^(2i/head_dim), computed in double as the CPU engine does
 * (resident_glimmer.cpp:773-800); `inverse` rotates by the negative angle.
 * head_dim even, at most 256. */
int nfn_native_tile_glimmer_positioned_rope_float32_v1(
    float* query,
    float* key,
    int64_t query_heads,
    int64_t kv_heads,
    int64_t head_dim,
    int64_t position,
    float theta,
    uint32_t layout,
    void* cuda_stream);
int nfn_native_tile_glimmer_positioned_rope_batch_float32_v1(
    float* query,
    float* key,
    int64_t rows,
    int64_t query_heads,
    int64_t kv_heads,
    int64_t head_dim,
    int64_t start_position,
    float theta,
    uint32_t layout,
    bool inverse,
    void* cuda_stream);

/* Per-head RMS normalisation of query and key (optional [1, head_dim] weights),
 * query *= query_scale, then the rotary embedding when apply_rope, in place, in
 * one launch (tile_ops.h:905-943).  Equal bit for bit to
 * rms_norm_affine(rows = heads, width = head_dim) on query and on key,
 * scale_inplace on query and positioned_rope, which is the reference probe's rule
 * (tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:461-610).  The batch form
 * handles rows 1..64, row r at position + r. */
int nfn_native_tile_glimmer_qk_norm_scale_rope_float32_v1(
    float* query,
    float* key,
    const NfnNativeTilePackedWeightDescriptorV1* query_norm_weight,
    const NfnNativeTilePackedWeightDescriptorV1* key_norm_weight,
    int64_t query_heads,
    int64_t kv_heads,
    int64_t head_dim,
    float eps,
    bool query_norm_centered,
    bool key_norm_centered,
    float query_scale,
    int64_t position,
    float theta,
    uint32_t layout,
    bool apply_rope,
    void* cuda_stream);
int nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1(
    float* query,
    float* key,
    const NfnNativeTilePackedWeightDescriptorV1* query_norm_weight,
    const NfnNativeTilePackedWeightDescriptorV1* key_norm_weight,
    int64_t rows,
    int64_t query_heads,
    int64_t kv_heads,
    int64_t head_dim,
    float eps,
    bool query_norm_centered,
    bool key_norm_centered,
    float query_scale,
    int64_t position,
    float theta,
    uint32_t layout,
    bool apply_rope,
    void* cuda_stream);

/* One-token causal attention of query_heads heads over kv_heads cached heads
 * (tile_ops.h:308-339, 944-945).  Keys first_key_position .. position-1 are
 * rows (p % cache_capacity) of the bf16 caches, key `position` is
 * current_key/current_value in float and not yet in the cache.  Query head h
 * uses cached head h*kv_heads/query_heads.  output[query_heads, head_dim] =
 * softmax(scale * q.k) . v.  Read-only on the caches. */
typedef struct NfnNativeTileGlimmerGqaDecodeDescriptorV1 {
    uint32_t struct_size;
    uint32_t version; /* NFN_NATIVE_TILE_GLIMMER_INFERENCE_V1 */
    uint32_t flags;   /* 0 */
    uint32_t reserved0;
    const float* query;
    const float* current_key;
    const float* current_value;
    const uint16_t* key_cache_bf16;
    const uint16_t* value_cache_bf16;
    float* output;
    int64_t query_heads;
    int64_t kv_heads;
    int64_t head_dim; /* 1..256 */
    int64_t position;
    int64_t first_key_position; /* 0..position */
    int64_t cache_capacity;
    int64_t cache_row_stride; /* elements, >= kv_heads*head_dim */
    float scale;              /* finite, > 0 */
    uint32_t reserved1;
    void* cuda_stream;
} NfnNativeTileGlimmerGqaDecodeDescriptorV1;
int nfn_native_tile_glimmer_gqa_decode_float32_v1(
    const NfnNativeTileGlimmerGqaDecodeDescriptorV1* descriptor);

/* Writes current_key/current_value [kv_heads*head_dim] (rows of them for the
 * second form, 1..64, row r at position + r) into row (position %
 * cache_capacity) of the bf16 caches, rounding to nearest even
 * (tile_ops.h:341-359, 955-959). */
typedef struct NfnNativeTileGlimmerCacheCommitDescriptorV1 {
    uint32_t struct_size;
    uint32_t version;
    uint32_t flags;
    uint32_t reserved0;
    const float* current_key;
    const float* current_value;
    uint16_t* key_cache_bf16;
    uint16_t* value_cache_bf16;
    int64_t kv_heads;
    int64_t head_dim;
    int64_t position;
    int64_t cache_capacity;
    int64_t cache_row_stride;
    uint32_t reserved1;
    uint32_t reserved2;
    void* cuda_stream;
} NfnNativeTileGlimmerCacheCommitDescriptorV1;
int nfn_native_tile_glimmer_cache_commit_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitDescriptorV1* descriptor);
int nfn_native_tile_glimmer_cache_commit_rows_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitDescriptorV1* descriptor,
    int64_t rows);

/* The three dependent per-layer decode steps in one call (tile_ops.h:361-405,
 * 946-947): qk_norm_scale_rope on query/key (in place), gqa_decode with key as
 * the current key, and the bf16 cache commit of key/current_value at
 * `position`.  The norm weights are embedded by value; has_*_norm_weight == 0
 * makes the corresponding descriptor inert.  Here it is two launches on the
 * descriptor's stream (the norm/rope kernel also writes the cache row, which a
 * one-token attention at this position does not read; a key range as long as
 * the ring gets the commit as a third launch, after the attention), with the
 * arithmetic of the separate calls, so it equals them bit for bit. */
typedef struct NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1 {
    uint32_t struct_size;
    uint32_t version;
    uint32_t flags;
    uint32_t reserved0;
    float* query;
    float* key;
    const float* current_value;
    uint16_t* key_cache_bf16;
    uint16_t* value_cache_bf16;
    float* output;
    NfnNativeTilePackedWeightDescriptorV1 query_norm_weight;
    NfnNativeTilePackedWeightDescriptorV1 key_norm_weight;
    int64_t query_heads; /* at most 256 */
    int64_t kv_heads;
    int64_t head_dim;
    int64_t position;
    int64_t first_key_position;
    int64_t cache_capacity;
    int64_t cache_row_stride;
    float norm_eps;
    float query_scale;
    float rope_theta;
    float attention_scale;
    uint32_t rope_layout;
    uint32_t has_query_norm_weight;
    uint32_t has_key_norm_weight;
    uint32_t query_norm_centered;
    uint32_t key_norm_centered;
    uint32_t apply_rope;
    uint32_t reserved1;
    void* cuda_stream;
} NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1;
int nfn_native_tile_glimmer_fused_decode_attention_float32_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* descriptor);

/* The same with the position in device memory (tile_ops.h:948-954): `position`
 * and `first_key_position` of the descriptor are ignored, the kernels read
 * *device_position when they run, so one captured graph serves every token.
 * With apply_rope (a local layer) the keys are the last `sliding_window` ones,
 * otherwise all from key 0.  1 <= sliding_window <= cache_capacity. */
int nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* descriptor,
    const int64_t* device_position,
    int64_t sliding_window);

/* Rows 0..rows-1 of a staged verification block, laid out [layer, source_rows,
 * kv_heads*head_dim] float, into the bf16 rings of up to 64 layers in one
 * launch (tile_ops.h:416-453, 960-961).  `layers` is a host array read during
 * the call; the cache pointers inside it are device pointers. */
typedef struct NfnNativeTileGlimmerCacheLayerV1 {
    uint16_t* key_cache_bf16;
    uint16_t* value_cache_bf16;
    int64_t cache_capacity;
    int64_t cache_row_stride;
} NfnNativeTileGlimmerCacheLayerV1;
typedef struct NfnNativeTileGlimmerCacheCommitLayersDescriptorV1 {
    uint32_t struct_size;
    uint32_t version;
    uint32_t flags;
    uint32_t reserved0;
    const float* staged_keys;
    const float* staged_values;
    const NfnNativeTileGlimmerCacheLayerV1* layers;
    int64_t layer_count; /* 1..64 */
    int64_t source_rows; /* 1..64 */
    int64_t rows;        /* 1..source_rows */
    int64_t kv_heads;
    int64_t head_dim;
    int64_t position;
    int64_t source_layer_stride; /* elements, >= source_rows*kv_heads*head_dim */
    uint32_t reserved1;
    uint32_t reserved2;
    void* cuda_stream;
} NfnNativeTileGlimmerCacheCommitLayersDescriptorV1;
int nfn_native_tile_glimmer_cache_commit_layers_bf16_v1(
    const NfnNativeTileGlimmerCacheCommitLayersDescriptorV1* descriptor);

/* [tap, source_row, hidden] -> [row, tap, hidden] for source rows
 * source_row_offset .. source_row_offset + rows - 1 (tile_ops.h:962-973). */
int nfn_native_tile_glimmer_pack_target_taps_float32_v1(
    const float* tap_major,
    float* row_major,
    int64_t source_rows,
    int64_t source_row_offset,
    int64_t rows,
    int64_t tap_count,
    int64_t hidden_width,
    void* cuda_stream);

/* Attention of a block of query_rows rows (positions context_length + r) over
 * the cached context and the block's own block_rows keys (tile_ops.h:445-486,
 * 974-975).  Causal (flags = NFN_NATIVE_TILE_BLOCK_ATTENTION_CAUSAL): keys
 * max(0, p - sliding_window + 1) .. p; block rows before the query's own are
 * rounded to bf16 on read, as a token-at-a-time decode would have cached them,
 * the query's own row stays float.  Not causal: keys max(0, p - sliding_window)
 * .. min(context_length + block_rows - 1, p + sliding_window), block rows in
 * float.  block_key/block_value: [block_rows, kv_heads, head_dim] float;
 * query, output: [query_rows, query_heads, head_dim].  block_rows <= 64. */
typedef struct NfnNativeTileDFlashBlockAttentionDescriptorV1 {
    uint32_t struct_size;
    uint32_t version;
    uint32_t flags;
    uint32_t reserved0;
    const float* query;
    const float* block_key;
    const float* block_value;
    const uint16_t* key_cache_bf16;
    const uint16_t* value_cache_bf16;
    float* output;
    int64_t query_rows;
    int64_t block_rows;
    int64_t query_heads;
    int64_t kv_heads;
    int64_t head_dim;
    int64_t context_length;
    int64_t sliding_window;
    int64_t cache_capacity; /* >= sliding_window */
    int64_t cache_row_stride;
    float scale;
    uint32_t reserved1;
    void* cuda_stream;
} NfnNativeTileDFlashBlockAttentionDescriptorV1;
int nfn_native_tile_dflash_block_attention_float32_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* descriptor);

/* The reference's short-context specialisation of the block attention
 * (tile_ops.h:976-982): same descriptor and result, a caller-supplied score
 * workspace, and a narrow geometry (32 query heads, head size 128, at most 16
 * query rows, at most 128 keys, a non-null stream) outside of which it fails
 * closed so that the caller keeps the general entry point.  Here the general
 * kernel serves it and the workspace stays untouched; the checks, including
 * the workspace size, are the reference's (glimmer_k_mmq.cu:2432-2472). */
int nfn_native_tile_dflash_block_attention_short_split_float32_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* descriptor,
    float* score_workspace,
    int64_t score_workspace_nbytes);

/* logits[i] = softcap * tanh(multiplier * logits[i] / softcap), in place, in
 * double as the CPU engine computes it (tile_ops.h:1004-1009;
 * resident_glimmer.cpp:1895-1903).  multiplier, softcap finite and > 0. */
int nfn_native_tile_glimmer_logit_transform_float32_v1(
    float* logits,
    int64_t count,
    float multiplier,
    float softcap,
    void* cuda_stream);

/* out[i] = lhs[i] + rhs[i] (tile_ops.h:1262-1267); values[i] *= scale
 * (tile_ops.h:1818-1822). */
int nfn_native_tile_add_float32(
    const float* lhs,
    const float* rhs,
    float* out,
    int64_t n,
    void* cuda_stream);
int nfn_native_tile_scale_inplace_float32(
    float* values,
    int64_t n,
    float scale,
    void* cuda_stream);

/* ==== additions: no counterpart in the reference ========================= */

/* Version of the additions below, 2: an engine that binds any nfn_mi355_* symbol checks it
 * the way it checks the reference's four version symbols (resident_glimmer_cuda.cpp:496-501).
 * Version 2: nfn_mi355_attention_workspace_v1 takes the stream the loan is for as a third
 * argument (a caller built against the two-argument form must not call it); the measurement
 * probes live in a library of their own (nfn_mi355_probes.h); the small-batch workspace of
 * four rows and more also holds the activations in matrix-operand order (the query
 * nfn_native_tile_k_quant_mmq_workspace_bytes_v1 returns the larger size);
 * nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1 is new. */
int nfn_mi355_abi_version(void);

/* lm_head GEMV with the argmax fused in: logits never reach memory.  The
 * reference runs mmvq_linear into an 808 KB logits buffer and then
 * argmax_rows over it (resident_glimmer_cuda.cpp:4087-4151, 2661-2704); this
 * is both in one call.  rows 1..16 (a verifier block); beyond 8 rows for the
 * four packed formats at an input_dim of at most 16,384, for which the
 * workspace query, which does not know input_dim, sizes the fp16 copy of the
 * rows that the 5..16-row form (Q6_K: 2..16) keeps there.  Ties go to the lowest index; NaN
 * never wins.  output_indices: int64[rows]; output_values: float[rows]. */
int64_t nfn_mi355_lm_head_argmax_workspace_bytes_v1(int64_t rows, int64_t output_dim);
int nfn_mi355_lm_head_argmax_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const float* input,
    int64_t* output_indices,
    float* output_values,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    void* cuda_stream);

/* nfn_mi355_lm_head_argmax_v1 for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc) and therefore have no workspace to pass.  No counterpart in the
 * reference.  Same arguments without the workspace, same kernels, same
 * results bit for bit: the candidate records of the first pass live in a
 * device array inside the library, NFN_MI355_LM_HEAD_NO_ALLOC_SCRATCH_BYTES
 * per GPU, held from library load until the process ends.  The call allocates
 * and frees nothing.  A problem whose workspace
 * (nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, output_dim)) exceeds that
 * size is refused with NFN_MI355_STATUS_STATIC_SCRATCH_EXCEEDED; the full
 * 202,048-row vocabulary at 8 rows needs 808,192 bytes and fits, and so do
 * its 16 rows (786,688 bytes).  Every call
 * on a GPU uses that GPU's one array: calls that overlap on a device
 * (different streams, concurrently replayed graphs) race on it.  The first
 * call on a device looks the array's address up in the runtime
 * (hipGetSymbolAddress); make that call before a capture begins. */
#define NFN_MI355_LM_HEAD_NO_ALLOC_SCRATCH_BYTES (1 << 20)
#define NFN_MI355_STATUS_STATIC_SCRATCH_EXCEEDED 0x4e46
int nfn_mi355_lm_head_argmax_no_alloc_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const float* input,
    int64_t* output_indices,
    float* output_values,
    int64_t rows,
    void* cuda_stream);

/* Prefill dequant-GEMM for any row count: output[rows, output_dim] =
 * input[rows, input_dim] * W^T.  The reference's small-batch entry points stop
 * at 16 rows (glimmer_k_mmq.cu:1326-1328) and its only route for more rows is
 * the generic linear above.  mode selects the MFMA operand type. */
enum {
    NFN_MI355_GEMM_F16 = 0, /* weights dequantized to fp16 in LDS, activations
                               row-scaled fp16, fp16 MFMA, float accumulate */
    NFN_MI355_GEMM_INT8 = 1 /* reserved: int8 activations per 32 values on the
                               int8 MFMA; refused (workspace query returns 0) */
};
int64_t nfn_mi355_k_quant_gemm_workspace_bytes_v1(
    int64_t rows, int64_t input_dim, int64_t output_dim, int mode);
int nfn_mi355_k_quant_gemm_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor,
    const float* input,
    float* output,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    int mode,
    void* cuda_stream);

/* How the call above cuts a problem of this geometry on the current device
 * (no counterpart in the reference; for tests and benchmarks that want to know
 * which launch form they exercised): *tile_rows = output rows per workgroup
 * tile (128 or 256), *k_shares = workgroups that share the K range of a tile
 * (1 = unsplit; with more, each writes a partial output into the workspace and
 * a second launch adds them in share order).  0 on success, 1 for an encoding
 * or width the matrix-core path does not take, or the reserved mode. */
int nfn_mi355_k_quant_gemm_plan_v1(
    uint32_t encoding,
    int64_t rows,
    int64_t input_dim,
    int64_t output_dim,
    int mode,
    int* tile_rows,
    int* k_shares);

/* The same for 1..4 projections of one input (Q/K/V, gate/up), the way the
 * small-batch entry points group them: the activations are converted once and
 * every projection runs from that copy.  All descriptors share input_dim (a
 * multiple of 256) and are Q4_K, Q5_K, Q6_K or Q8_0.  The workspace is the
 * largest of the single-projection sizes (the query above with each
 * output_dim).  Results are those of the single-projection call, bit for bit. */
int nfn_mi355_k_quant_gemm_multi_float32_v1(
    const NfnNativeTilePackedWeightDescriptorV1* const* descriptors,
    const float* input,
    float* const* outputs,
    int64_t operation_count,
    int64_t rows,
    void* workspace,
    int64_t workspace_nbytes,
    int mode,
    void* cuda_stream);

/* One-token attention with a workspace: nfn_native_tile_glimmer_gqa_decode_float32_v1
 * runs one workgroup per query head because it has nowhere to put partial
 * results; with a workspace the keys of every head are dealt over many
 * workgroups (up to 128 shares) and a second launch merges their partial sums.
 * With head_dim 128 and four or more query heads per key/value head a
 * workgroup serves up to 16 query heads of one key/value head on the matrix
 * cores, so a cache row is read once for all of them.  Same descriptor,
 * same semantics, same tolerance against the double-precision formula; the
 * summation order differs, so the bits can differ from the ordinary entry
 * point (and the causal-block equality rule is stated for that one).  The
 * workspace is 16-byte aligned device memory of
 * nfn_mi355_gqa_decode_split_workspace_bytes_v1(query_heads, head_dim) bytes
 * (0 = unsupported geometry), private to one call at a time. */
int64_t nfn_mi355_gqa_decode_split_workspace_bytes_v1(int64_t query_heads, int64_t head_dim);
int nfn_mi355_gqa_decode_split_v1(
    const NfnNativeTileGlimmerGqaDecodeDescriptorV1* descriptor,
    void* workspace,
    int64_t workspace_nbytes);

/* nfn_native_tile_glimmer_fused_decode_attention_float32_v1 with the split
 * attention form above: three launches (norm/rope/commit, attention shares,
 * merge).  Same descriptor, same workspace as nfn_mi355_gqa_decode_split_v1. */
int nfn_mi355_fused_decode_attention_split_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* descriptor,
    void* workspace,
    int64_t workspace_nbytes);

/* nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1
 * (position read from device memory when the kernels run, so one captured
 * graph serves every token) with the split attention form: the shares are cut
 * from the row's real key count on the device.  Arguments as in the two entry
 * points it combines. */
int nfn_mi355_fused_decode_attention_split_device_position_v1(
    const NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1* descriptor,
    const int64_t* device_position,
    int64_t sliding_window,
    void* workspace,
    int64_t workspace_nbytes);

/* nfn_native_tile_dflash_block_attention_float32_v1 with a workspace: the keys
 * of every query row are shared out over workgroups like those of the
 * one-token split form (as many shares as the workspace has room for,
 * query_rows * query_heads * (head_dim + 2) floats each; with room for fewer
 * than two the ordinary form runs).  Same descriptor, same semantics and
 * tolerance; the bits can differ from the ordinary entry point.  The workspace
 * of the one-token form is a good size for blocks of up to 16 rows. */
int nfn_mi355_dflash_block_attention_split_v1(
    const NfnNativeTileDFlashBlockAttentionDescriptorV1* descriptor,
    void* workspace,
    int64_t workspace_nbytes);

/* Lends the attention entry points that have no workspace argument
 * (nfn_native_tile_glimmer_gqa_decode_float32_v1, the fused decode-attention
 * call and its device-position form, nfn_native_tile_dflash_block_attention_float32_v1
 * and its short_split form) a workspace for the split forms above, so
 * that an engine's unchanged call sites take it: from this call on they run as
 * their nfn_mi355_*_split_* counterparts whenever the workspace is on the
 * current device, was lent for the stream the call is issued on
 * (descriptor->cuda_stream) and is large enough for the call's geometry
 * (nfn_mi355_gqa_decode_split_workspace_bytes_v1; a block takes as many shares
 * as fit), and as before otherwise.  One loan per (device, stream), at most 32
 * at a time; lending again for the same stream replaces the loan;
 * (nullptr, 0, stream) takes that stream's loan back.  No counterpart in the
 * reference.  The memory stays the caller's.  Calls on the loan's stream run
 * in stream order, so they never write the workspace at once; calls on other
 * streams do not see it.  What still races: graphs captured from that stream
 * and replayed concurrently with each other or with it -- give such graphs
 * the explicit *_split_v1 entry points with a workspace each.  Calls already
 * captured into a graph keep the form they were captured with.  0 on success,
 * 1 for a misaligned pointer, a size without a pointer, or a 33rd loan. */
int nfn_mi355_attention_workspace_v1(void* workspace, int64_t workspace_nbytes, void* cuda_stream);

#ifdef __cplusplus
}
#endif

#endif /* NFN_MI355_TILE_OPS_H */
