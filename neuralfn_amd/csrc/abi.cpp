// extern "C" surface of libnfn_mi355_tile_ops.so: argument checks, then one or
// two launches on the caller's stream.  Nothing here allocates, synchronises
// or keeps state between calls.  Reference wrappers:
// neuralfn/csrc/native_train/tile_ops.cu:4504-4713 and
// neuralfn/csrc/tile_cuda/glimmer_k_mmq.cu:2349-2649.
#include "common.hpp"
#include "gemv_dot.hpp"
#include "gemm_mfma.hpp"
#include "gemv_f16.hpp"
#include "gemv_mfma.hpp"
#include "gemv_q6.hpp"
#include "gemv_q8.hpp"
#include "gemv_rows.hpp"
#include "kernels.hpp"
#include "lm_head.hpp"
#include "rms_device.hpp"

#include <cmath>
#include <limits>

namespace nfn {

namespace {

constexpr std::int64_t kMaxSmallRows = 16;
constexpr std::int64_t kMaxOperations = 4;
constexpr std::int64_t kFirstHalfRows = 5;  // rows from which the fp16 matrix-core kernel takes a batch
// ... and Q6_K from three rows: its int8 kernel reads the 210-byte blocks lane by lane, the
// fp16 one brings them into LDS whole (6,656 -> 4,096 at 4 rows: 22.0 -> 19.2 us, the lm_head at
// 3 and 4 rows: 257 -> 226 us; Q4_K and Q5_K the other way round: 21.7 -> 27.3 us at
// 6,656 -> 16,384)
constexpr std::int64_t kFirstHalfRowsQ6 = 3;
std::int64_t first_half_rows(std::uint32_t encoding) {
    return encoding == kEncQ6K ? kFirstHalfRowsQ6 : kFirstHalfRows;
}
// rows from which the verifier family's Q4_K / Q5_K projections run on the int8 matrix cores
// (one pass over the weights behind a quantizer launch; below: the dot kernel's token passes,
// which are faster up to three rows: 9.0 / 12.4 / 13.9 us per launch of the attention
// projections at 2 / 3 / 4 rows against 12.8 for the matrix-core kernel at any of them)
constexpr std::int64_t kFirstVerifierMatrixRows = 4;
// Private activation records of the small-batch path, 576 bytes per token and
// 256 values (two int8 planes of a 16-bit fixed-point code, group sums, scale,
// block maximum): 72 bytes per 32 values, the unit the workspace is sized in.
constexpr std::int64_t kActivationGroupBytes = kActivationRecordBytes / 8;

// Bytes of the activation records of `rows` rows, rounded up to 256.
std::int64_t record_bytes(std::int64_t rows, std::int64_t input_dim) {
    const std::int64_t groups = (input_dim + 31) / 32;
    return (rows * groups * kActivationGroupBytes + 255) & ~std::int64_t(255);
}

// Records, and behind them, from the row count on at which the verifier family runs on the
// matrix cores, the same codes in matrix-operand order (gemv_rows.hpp).
std::int64_t small_batch_workspace_bytes(std::int64_t rows, std::int64_t input_dim) {
    if (rows < 1 || rows > kMaxSmallRows || input_dim <= 0 || input_dim % 128 != 0) return 0;
    const std::int64_t groups = (input_dim + 31) / 32;
    if (groups > std::numeric_limits<std::int64_t>::max() / (2 * kActivationGroupBytes * kMaxSmallRows)) {
        return 0;
    }
    std::int64_t raw = record_bytes(rows, input_dim);
    if (rows >= kFirstVerifierMatrixRows && input_dim % 256 == 0) {
        raw += gemv_rows_image_bytes(input_dim);
    }
    return (raw + 255) & ~std::int64_t(255);
}

bool ranges_overlap(const void* a, std::int64_t a_bytes, const void* b, std::int64_t b_bytes) {
    const std::uintptr_t pa = reinterpret_cast<std::uintptr_t>(a);
    const std::uintptr_t pb = reinterpret_cast<std::uintptr_t>(b);
    return pa < pb + static_cast<std::uintptr_t>(b_bytes) && pb < pa + static_cast<std::uintptr_t>(a_bytes);
}

Projection make_projection(const Descriptor& descriptor, float* output) {
    Projection op{};
    op.data = descriptor.data;
    op.output = output;
    op.output_dim = descriptor.output_dim;
    op.row_stride = descriptor.row_stride_bytes;
    op.encoding = descriptor.encoding;
    op.first_tile = 0;
    return op;
}

// Shared body of the small-batch entry points.
// `verifier`: every row must get the one-row arithmetic bit for bit.
int run_small_batch(bool verifier, const Descriptor* const* descriptors, const float* first,
                    const float* second, int prologue, float* const* outputs,
                    std::int64_t operation_count, std::int64_t rows, void* workspace,
                    std::int64_t workspace_nbytes, void* stream) {
    if (descriptors == nullptr || first == nullptr || outputs == nullptr ||
        operation_count < 1 || operation_count > kMaxOperations || workspace == nullptr ||
        workspace_nbytes <= 0 || ((prologue == kGated || prologue == kSwiGlu) && second == nullptr)) {
        return kInvalid;
    }
    const std::int64_t input_dim = descriptors[0] == nullptr ? 0 : descriptors[0]->input_dim;
    ProjectionSet set{};
    set.count = static_cast<int>(operation_count);
    set.input_dim = input_dim;
    for (std::int64_t index = 0; index < operation_count; ++index) {
        if (outputs[index] == nullptr ||
            !validate_k_descriptor(descriptors[index], input_dim, stream, true)) {
            return kInvalid;
        }
        set.op[index] = make_projection(*descriptors[index], outputs[index]);
    }
    const std::int64_t required = small_batch_workspace_bytes(rows, input_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    // One or two rows, and the verifier entry points at any row count: the
    // vector-ALU kernels.  Otherwise 3 and 4 rows: the int8 matrix-core kernel,
    // which quantizes inside the kernel; 5..16 rows (Q6_K: 3..16): the fp16 matrix-core kernel
    // behind its conversion launch (Q8_0 below five rows: its dot kernel).
    // Encodings and widths without either: the float kernel.
    // (two rows are also faster on the dot kernels: they walk the token planes
    // against the same unpacked weights)
    const bool one_row_arithmetic = rows <= 2 || verifier;
    const bool verifier_matrix = verifier && rows >= kFirstVerifierMatrixRows;
    ProjectionSet dot{}, dot6{}, dot8{}, matrix{}, half{}, exact{}, verifier_rows{};
    dot.input_dim = dot6.input_dim = dot8.input_dim = matrix.input_dim = half.input_dim =
        exact.input_dim = verifier_rows.input_dim = input_dim;
    for (int index = 0; index < set.count; ++index) {
        const std::uint32_t encoding = set.op[index].encoding;
        ProjectionSet* target = &exact;
        if (verifier_matrix && gemv_rows_supports(encoding, input_dim)) {
            target = &verifier_rows;
        } else if (one_row_arithmetic && gemv_dot_supports(encoding, input_dim)) {
            target = &dot;
        } else if (one_row_arithmetic && gemv_q6_supports(encoding, input_dim)) {
            target = &dot6;
        } else if (rows >= first_half_rows(encoding) && !verifier && gemv_f16_supports(encoding, input_dim)) {
            target = &half;
        } else if (gemv_q8_supports(encoding, input_dim)) {
            target = &dot8;  // Q8_0 below five rows and in the verifier family: its dot kernel
        } else if (rows >= 2 && gemv_mfma_supports(encoding, input_dim)) {
            target = &matrix;
        }
        target->op[target->count++] = set.op[index];
    }
    // Prequantized input: only the dot kernels read activation records.
    if (prologue == kRecords && (matrix.count > 0 || half.count > 0 || exact.count > 0)) return kInvalid;
    // An fp16 image in the workspace: only the fp16 small-batch kernel reads one.
    if (prologue == kHalfImage && half.count != set.count) return kInvalid;
    // In the verifier family the dot kernels leave their activation records in
    // the workspace, where a following prequantized call with the same input
    // finds them (neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:3649-3666).
    std::uint8_t* records =
        verifier && prologue != kRecords ? static_cast<std::uint8_t*>(workspace) : nullptr;
    const float* dot_first = first;
    const float* dot_second = second;
    int dot_prologue = prologue;
    if (verifier_matrix && input_dim % 256 == 0) {
        // The matrix-core kernel reads the activations in operand order: a quantizer launch
        // writes that image behind the records (whatever the encodings of this call, so that a
        // prequantized call behind it finds both), and the dot kernels of the other encodings
        // read the records instead of quantizing again.
        std::uint8_t* image = static_cast<std::uint8_t*>(workspace) + record_bytes(rows, input_dim);
        // The quantizer launch can also prepare the outputs for the kernel's split form, unless
        // one of them overlaps what that launch reads.
        // (a prequantized call has no such launch: a fill launch of its own where that pays)
        const bool fill_launch = prologue == kRecords;
        ProjectionSet clear = gemv_rows_split_set(verifier_rows, fill_launch);
        if (fill_launch) {
            launch_fill_outputs(clear, rows, as_stream(stream));
        } else {
            const std::int64_t input_bytes = rows * input_dim * static_cast<std::int64_t>(sizeof(float));
            for (int index = 0; index < clear.count; ++index) {
                const std::int64_t bytes =
                    rows * clear.op[index].output_dim * static_cast<std::int64_t>(sizeof(float));
                if (ranges_overlap(clear.op[index].output, bytes, first, input_bytes) ||
                    (second != nullptr && ranges_overlap(clear.op[index].output, bytes, second, input_bytes))) {
                    clear.count = 0;
                    break;
                }
            }
            launch_quantize_records(first, second, prologue, rows, input_dim,
                                    static_cast<std::uint8_t*>(workspace), image, clear,
                                    as_stream(stream));
        }
        if (verifier_rows.count > 0) {
            launch_gemv_rows(verifier_rows, image, rows, clear.count > 0, fill_launch, as_stream(stream));
        }
        dot_first = static_cast<const float*>(workspace);
        dot_second = nullptr;
        dot_prologue = kRecords;
        records = nullptr;
    }
    if (dot.count > 0) {
        launch_gemv_dot(dot, dot_first, dot_second, records, dot_prologue, rows, as_stream(stream));
    }
    if (dot6.count > 0) {
        launch_gemv_q6(dot6, dot_first, dot_second, records, dot_prologue, rows, as_stream(stream));
    }
    if (dot8.count > 0) {
        launch_gemv_q8(dot8, dot_first, dot_second, records, dot_prologue, rows, as_stream(stream));
    }
    if (matrix.count > 0) {
        launch_gemv_mfma(matrix, first, second, prologue, rows, workspace, as_stream(stream));
    }
    if (half.count > 0) {
        launch_gemv_f16(half, first, second, prologue, rows, workspace, as_stream(stream));
    }
    if (exact.count > 0) {
        launch_gemv_f32(exact, first, second, prologue, nullptr, rows, as_stream(stream));
    }
    return launch_status();
}

}  // namespace

}  // namespace nfn

using namespace nfn;

extern "C" {

int nfn_native_tile_ops_abi_version(void) { return 1; }
// Strict math: no fast-math flags, correctly rounded division and square root,
// no contraction of the reference's two-rounding weight decode.
int nfn_native_tile_strict_math_abi_version(void) { return 1; }
int nfn_native_tile_packed_weight_abi_version(void) { return NFN_NATIVE_TILE_PACKED_WEIGHT_V1; }
int nfn_native_tile_glimmer_inference_abi_version(void) { return 1; }
int nfn_native_tile_k_quant_mmq_abi_version(void) { return NFN_NATIVE_TILE_K_QUANT_MMQ_V1; }
int nfn_mi355_abi_version(void) { return 2; }

const char* nfn_native_tile_ops_error_string(int code) {
    if (code == NFN_MI355_STATUS_STATIC_SCRATCH_EXCEEDED) {
        return "the problem needs more scratch than the no-allocation entry point holds";
    }
    const char* text = hipGetErrorString(static_cast<hipError_t>(code));
    return text != nullptr ? text : "unknown error";
}

}  // extern "C"

namespace {

// The generic linear has two exact kernels: the vector one decodes every weight once per 8
// input rows, the matrix-core one once per 128.  Rates measured on MI355X at 6,656 columns:
// the vector kernel decodes 4.6e11 (Q4_K, Q5_K), 3.0e11 (Q6_K) or 2.4e11 (others) weights a
// second and a launch of it takes at least 6 us; a 128 x 64 tile of the matrix-core kernel
// takes 300 us alone on its compute unit (3.6e11 flop/s) and 229 us when the unit works
// through several (4.8e11 flop/s).
bool float_matrix_cores_pay(const Descriptor& weight, std::int64_t rows) {
    if (rows <= 16 || !gemm_f32_supports(weight, rows)) return false;
    const double weights =
        static_cast<double>(weight.output_dim) * static_cast<double>(weight.input_dim);
    const double decoded_per_us = weight.encoding == kEncQ4K || weight.encoding == kEncQ5K ? 4.6e5
                                  : weight.encoding == kEncQ6K                             ? 3.0e5
                                                                                           : 2.4e5;
    // the vector kernel's passes of eight rows are workgroups of one launch, not launches one
    // after another: the launch floor counts once
    const double vector_work_us = static_cast<double>((rows + 7) / 8) * weights / decoded_per_us;
    const double vector_us = vector_work_us < 6.0 ? 6.0 : vector_work_us;
    const double tile_flop = 128.0 * 64.0 * 2.0 * static_cast<double>(weight.input_dim);
    const double passes = gemm_f32_tile_passes(weight, rows);
    const double alone_us = tile_flop / 3.6e5;
    const double matrix_us = passes * tile_flop / 4.8e5 < alone_us ? alone_us : passes * tile_flop / 4.8e5;
    return matrix_us + 4.0 < vector_us;
}

}  // namespace

extern "C" {

int nfn_native_tile_packed_weight_validate_v1(const Descriptor* descriptor) {
    Descriptor normalized{};
    return normalize_descriptor(descriptor, &normalized) ? 0 : kInvalid;
}

int nfn_native_tile_packed_weight_dequantize_float32_v1(const Descriptor* descriptor,
                                                        float* output) {
    Descriptor normalized{};
    if (!normalize_descriptor(descriptor, &normalized) || output == nullptr) return kInvalid;
    launch_dequantize(normalized, output, as_stream(normalized.cuda_stream));
    return launch_status();
}

int nfn_native_tile_linear_packed_weight_float32_v1(const Descriptor* descriptor,
                                                    const float* input, const float* bias,
                                                    float* output, std::int64_t rows,
                                                    bool has_bias) {
    Descriptor normalized{};
    if (!normalize_descriptor(descriptor, &normalized) || input == nullptr ||
        output == nullptr || rows <= 0 || (has_bias && bias == nullptr)) {
        return kInvalid;
    }
    const hipStream_t stream = as_stream(normalized.cuda_stream);
    if (float_matrix_cores_pay(normalized, rows)) {
        launch_gemm_f32(normalized, input, has_bias ? bias : nullptr, output, rows, stream);
        return launch_status();
    }
    ProjectionSet set{};
    set.count = 1;
    set.input_dim = normalized.input_dim;
    set.op[0] = make_projection(normalized, output);
    constexpr std::int64_t kChunk = 65535 * 8;
    for (std::int64_t row = 0; row < rows; row += kChunk) {
        const std::int64_t count = rows - row < kChunk ? rows - row : kChunk;
        set.op[0].output = output + row * normalized.output_dim;
        launch_gemv_f32(set, input + row * normalized.input_dim, nullptr, kPlain,
                        has_bias ? bias : nullptr, count, stream);
    }
    return launch_status();
}

int nfn_native_tile_quantize_q8_1_float32_v1(const float* input, std::int8_t* q8_values,
                                             float* q8_scales, float* q8_sums,
                                             std::int64_t rows, std::int64_t width,
                                             void* cuda_stream) {
    if (input == nullptr || q8_values == nullptr || q8_scales == nullptr ||
        q8_sums == nullptr || rows <= 0 || width <= 0 || width % 32 != 0) {
        return kInvalid;
    }
    launch_quantize_q8_1(input, q8_values, q8_scales, q8_sums, rows, width,
                         as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_linear_packed_weight_q8_1_float32_v1(
    const Descriptor* descriptor, const std::int8_t* q8_values, const float* q8_scales,
    const float* q8_sums, const float* bias, float* output, std::int64_t rows, bool has_bias) {
    Descriptor normalized{};
    if (!normalize_descriptor(descriptor, &normalized) || q8_values == nullptr ||
        q8_scales == nullptr || q8_sums == nullptr || output == nullptr || rows <= 0 ||
        (has_bias && bias == nullptr) || normalized.input_dim % 256 != 0 ||
        !is_k_quant(normalized.encoding)) {
        return kInvalid;
    }
    ProjectionSet set{};
    set.count = 1;
    set.input_dim = normalized.input_dim;
    const hipStream_t stream = as_stream(normalized.cuda_stream);
    const std::int64_t groups = normalized.input_dim / 32;
    constexpr std::int64_t kChunk = 65535;
    for (std::int64_t row = 0; row < rows; row += kChunk) {
        const std::int64_t count = rows - row < kChunk ? rows - row : kChunk;
        set.op[0] = make_projection(normalized, output + row * normalized.output_dim);
        launch_linear_q8_1(set, q8_values + row * normalized.input_dim, q8_scales + row * groups,
                           q8_sums + row * groups, has_bias ? bias : nullptr, count, stream);
    }
    return launch_status();
}

int nfn_native_tile_linear_packed_weight_q8_1_multi_decode_float32_v1(
    const Descriptor* descriptor0, const Descriptor* descriptor1, const Descriptor* descriptor2,
    const Descriptor* descriptor3, const std::int8_t* q8_values, const float* q8_scales,
    const float* q8_sums, float* output0, float* output1, float* output2, float* output3,
    std::int64_t projection_count, void* cuda_stream) {
    const Descriptor* descriptors[4] = {descriptor0, descriptor1, descriptor2, descriptor3};
    float* outputs[4] = {output0, output1, output2, output3};
    if (projection_count < 2 || projection_count > 4 || q8_values == nullptr ||
        q8_scales == nullptr || q8_sums == nullptr) {
        return kInvalid;
    }
    ProjectionSet set{};
    set.count = static_cast<int>(projection_count);
    for (int index = 0; index < 4; ++index) {
        if (index >= projection_count) {
            // Unused slots must be null (tile_ops.cu:4669-4683).
            if (descriptors[index] != nullptr || outputs[index] != nullptr) return kInvalid;
            continue;
        }
        Descriptor normalized{};
        if (descriptors[index] == nullptr || outputs[index] == nullptr ||
            !normalize_descriptor(descriptors[index], &normalized) ||
            normalized.input_dim % 256 != 0 || !is_k_quant(normalized.encoding)) {
            return kInvalid;
        }
        if (index == 0) set.input_dim = normalized.input_dim;
        if (normalized.input_dim != set.input_dim) return kInvalid;
        set.op[index] = make_projection(normalized, outputs[index]);
    }
    launch_linear_q8_1(set, q8_values, q8_scales, q8_sums, nullptr, 1, as_stream(cuda_stream));
    return launch_status();
}

std::int64_t nfn_native_tile_k_quant_mmq_workspace_bytes_v1(std::int64_t rows,
                                                            std::int64_t input_dim) {
    return small_batch_workspace_bytes(rows, input_dim);
}

int nfn_native_tile_k_quant_mmq_multi_linear_float32_v1(
    const Descriptor* const* descriptors, const float* input, float* const* outputs,
    std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    return run_small_batch(false, descriptors, input, nullptr, kPlain, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmq_multi_linear_gated_float32_v1(
    const Descriptor* const* descriptors, const float* input, const float* gate,
    float* const* outputs, std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    if (gate == nullptr) return kInvalid;
    return run_small_batch(false, descriptors, input, gate, kGated, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1(
    const Descriptor* const* descriptors, const float* gate, const float* up,
    float* const* outputs, std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    if (gate == nullptr || up == nullptr) return kInvalid;
    return run_small_batch(false, descriptors, gate, up, kSwiGlu, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1(
    const Descriptor* const* descriptors, const float* input, float* const* outputs,
    std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    return run_small_batch(true, descriptors, input, nullptr, kPlain, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1(
    const Descriptor* const* descriptors, float* const* outputs, std::int64_t operation_count,
    std::int64_t rows, void* workspace, std::int64_t workspace_nbytes, void* cuda_stream) {
    // The workspace holds the activation records of `rows` rows, left there by
    // a verifier-family call on the same input or by the dual-RMS handoff.
    return run_small_batch(true, descriptors, static_cast<const float*>(workspace), nullptr,
                           kRecords, outputs, operation_count, rows, workspace, workspace_nbytes,
                           cuda_stream);
}

int nfn_mi355_k_quant_mmq_multi_linear_prequantized_float32_v1(
    const Descriptor* const* descriptors, float* const* outputs, std::int64_t operation_count,
    std::int64_t rows, void* workspace, std::int64_t workspace_nbytes, void* cuda_stream) {
    // The workspace holds the fp16 image of `rows` rows, left there by
    // nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1.
    if (rows < 5) return kInvalid;
    return run_small_batch(false, descriptors, static_cast<const float*>(workspace), nullptr,
                           kHalfImage, outputs, operation_count, rows, workspace, workspace_nbytes,
                           cuda_stream);
}

int nfn_native_tile_k_quant_mmvq_multi_linear_gated_float32_v1(
    const Descriptor* const* descriptors, const float* input, const float* gate,
    float* const* outputs, std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    if (gate == nullptr) return kInvalid;
    return run_small_batch(true, descriptors, input, gate, kGated, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmvq_multi_linear_swiglu_float32_v1(
    const Descriptor* const* descriptors, const float* gate, const float* up,
    float* const* outputs, std::int64_t operation_count, std::int64_t rows, void* workspace,
    std::int64_t workspace_nbytes, void* cuda_stream) {
    if (gate == nullptr || up == nullptr) return kInvalid;
    return run_small_batch(true, descriptors, gate, up, kSwiGlu, outputs, operation_count, rows,
                           workspace, workspace_nbytes, cuda_stream);
}

int nfn_native_tile_k_quant_mmvq_linear_float32_v1(const Descriptor* descriptor,
                                                   const float* input, float* output,
                                                   void* workspace,
                                                   std::int64_t workspace_nbytes,
                                                   void* cuda_stream) {
    const Descriptor* descriptors[1] = {descriptor};
    float* outputs[1] = {output};
    return run_small_batch(true, descriptors, input, nullptr, kPlain, outputs, 1, 1, workspace,
                           workspace_nbytes, cuda_stream);
}

int nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1(const Descriptor* gate, const Descriptor* up,
                                                     const float* input, float* output,
                                                     void* cuda_stream) {
    if (gate == nullptr || up == nullptr || input == nullptr || output == nullptr ||
        !validate_k_descriptor(gate, gate->input_dim, cuda_stream, false) ||
        !validate_k_descriptor(up, gate->input_dim, cuda_stream, false) ||
        gate->output_dim != up->output_dim || gate->output_dim > 0x3fffffff ||
        !gemv_dot_pairs_supports(gate->encoding, up->encoding, gate->input_dim)) {
        return kInvalid;
    }
    ProjectionSet set{};
    set.count = 2;
    set.input_dim = gate->input_dim;
    set.op[0] = make_projection(*gate, output);
    set.op[1] = make_projection(*up, output);
    if (set.op[0].row_stride != set.op[1].row_stride) return kInvalid;
    launch_gemv_dot_pairs(set, input, as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1(const Descriptor* gate, const Descriptor* up,
                                                    const float* input, float* output,
                                                    std::int64_t rows, void* workspace,
                                                    std::int64_t workspace_nbytes,
                                                    void* cuda_stream) {
    if (gate == nullptr || up == nullptr || output == nullptr || workspace == nullptr ||
        rows < kFirstHalfRows || rows > kMaxSmallRows ||
        !validate_k_descriptor(gate, gate->input_dim, cuda_stream, true) ||
        !validate_k_descriptor(up, gate->input_dim, cuda_stream, true) ||
        gate->output_dim != up->output_dim ||
        gate->row_stride_bytes != up->row_stride_bytes ||
        !gemv_f16_pairs_supports(gate->encoding, up->encoding, gate->input_dim)) {
        return kInvalid;
    }
    const std::int64_t required = small_batch_workspace_bytes(rows, gate->input_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    ProjectionSet set{};
    set.count = 2;
    set.input_dim = gate->input_dim;
    set.op[0] = make_projection(*gate, output);
    set.op[1] = make_projection(*up, output);
    launch_gemv_f16_pairs(set, input, rows, workspace, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_argmax_rows_float32_v1(const float* values, std::int64_t* output_indices,
                                           float* output_values, std::int64_t rows,
                                           std::int64_t width, void* cuda_stream) {
    if (values == nullptr || output_indices == nullptr || output_values == nullptr ||
        rows <= 0 || width <= 0 || rows > 0x7fffffff) {
        return kInvalid;
    }
    launch_argmax_rows(values, output_indices, output_values, rows, width,
                       as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_sigmoid_gate_float32_v1(const float* values, const float* gate,
                                                    float* output, std::int64_t count,
                                                    void* cuda_stream) {
    if (values == nullptr || gate == nullptr || output == nullptr || count <= 0) return kInvalid;
    launch_sigmoid_gate(values, gate, output, count, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_swiglu_float32(const float* gate, const float* up, float* out,
                                   std::int64_t n, void* cuda_stream) {
    if (gate == nullptr || up == nullptr || out == nullptr || n <= 0) return kInvalid;
    launch_swiglu(gate, up, out, n, as_stream(cuda_stream));
    return launch_status();
}

// The four single-normalisation entry points
// (neuralfn/csrc/native_train/tile_ops.cu:4777-4899) share one body.
static int run_rms_norm(const float* input, const Descriptor* weight, const float* residual_input,
                        bool wants_residual_input, float* output, float* residual_output,
                        bool wants_residual_output, std::int8_t* q8_values, float* q8_scales,
                        float* q8_sums, bool wants_q8, std::int64_t rows, std::int64_t width,
                        float eps, bool centered, void* cuda_stream) {
    Descriptor normalized{};
    if (input == nullptr || output == nullptr || rows <= 0 || width <= 0 || width > 65536 ||
        !std::isfinite(eps) || !(eps > 0.0f) ||
        (wants_residual_input && residual_input == nullptr) ||
        (wants_residual_output && residual_output == nullptr) ||
        (wants_q8 && (q8_values == nullptr || q8_scales == nullptr || q8_sums == nullptr ||
                      width % 32 != 0)) ||
        (weight != nullptr && (!normalize_descriptor(weight, &normalized) ||
                               normalized.output_dim != 1 || normalized.input_dim != width))) {
        return kInvalid;
    }
    launch_rms_norm(input, weight != nullptr ? &normalized : nullptr, centered,
                    wants_residual_input ? residual_input : nullptr, output,
                    wants_residual_output ? residual_output : nullptr,
                    wants_q8 ? q8_values : nullptr, q8_scales, q8_sums, rows, width, eps,
                    as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_rms_norm_affine_float32_v1(
    const float* input, const Descriptor* weight, float* output, std::int64_t rows,
    std::int64_t width, float eps, bool centered, void* cuda_stream) {
    return run_rms_norm(input, weight, nullptr, false, output, nullptr, false, nullptr, nullptr,
                        nullptr, false, rows, width, eps, centered, cuda_stream);
}

int nfn_native_tile_glimmer_rms_norm_affine_capture_residual_float32_v1(
    const float* input, const Descriptor* weight, float* output, float* residual_output,
    std::int64_t rows, std::int64_t width, float eps, bool centered, void* cuda_stream) {
    return run_rms_norm(input, weight, nullptr, false, output, residual_output, true, nullptr,
                        nullptr, nullptr, false, rows, width, eps, centered, cuda_stream);
}

int nfn_native_tile_glimmer_rms_norm_affine_capture_residual_q8_1_float32_v1(
    const float* input, const Descriptor* weight, float* output, float* residual_output,
    std::int8_t* q8_values, float* q8_scales, float* q8_sums, std::int64_t rows,
    std::int64_t width, float eps, bool centered, void* cuda_stream) {
    return run_rms_norm(input, weight, nullptr, false, output, residual_output, true, q8_values,
                        q8_scales, q8_sums, true, rows, width, eps, centered, cuda_stream);
}

int nfn_native_tile_glimmer_rms_norm_affine_add_residual_float32_v1(
    const float* input, const Descriptor* weight, const float* residual_input, float* output,
    std::int64_t rows, std::int64_t width, float eps, bool centered, void* cuda_stream) {
    return run_rms_norm(input, weight, residual_input, true, output, nullptr, false, nullptr,
                        nullptr, nullptr, false, rows, width, eps, centered, cuda_stream);
}

// Shared argument checks of the two dual-RMS entry points
// (neuralfn/csrc/native_train/tile_ops.cu:4901-5010): a norm weight is absent
// or a valid [1, width] descriptor.
static bool dual_rms_arguments_valid(const float* input, const Descriptor* first_weight,
                                     const float* residual_input, float* hidden_output,
                                     const Descriptor* second_weight, float* normalized_output,
                                     float* residual_output, std::int64_t rows, std::int64_t width,
                                     float first_eps, float second_eps, Descriptor* first,
                                     Descriptor* second) {
    const auto valid_weight = [&](const Descriptor* source, Descriptor* target) {
        return source == nullptr ||
            (normalize_descriptor(source, target) && target->output_dim == 1 &&
             target->input_dim == width);
    };
    return input != nullptr && residual_input != nullptr && hidden_output != nullptr &&
        normalized_output != nullptr && residual_output != nullptr && rows > 0 && width > 0 &&
        width <= 65536 && std::isfinite(first_eps) && first_eps > 0.0f &&
        std::isfinite(second_eps) && second_eps > 0.0f && valid_weight(first_weight, first) &&
        valid_weight(second_weight, second);
}

int nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t rows, std::int64_t width, float first_eps,
    bool first_centered, float second_eps, bool second_centered, void* cuda_stream) {
    Descriptor first{}, second{};
    if (!dual_rms_arguments_valid(input, first_weight, residual_input, hidden_output,
                                  second_weight, normalized_output, residual_output, rows, width,
                                  first_eps, second_eps, &first, &second)) {
        return kInvalid;
    }
    launch_dual_rms_add_capture(input, first_weight != nullptr ? &first : nullptr, first_centered,
                                residual_input, hidden_output,
                                second_weight != nullptr ? &second : nullptr, second_centered,
                                normalized_output, residual_output, rows, width, first_eps,
                                second_eps, nullptr, nullptr, as_stream(cuda_stream));
    return launch_status();
}

int nfn_native_tile_glimmer_dual_rms_add_capture_cooperative_batch_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t rows, std::int64_t width, float first_eps,
    bool first_centered, float second_eps, bool second_centered, void* cuda_stream) {
    // The reference's multi-row specialization takes F32 norm weights only
    // (tile_ops.h:859-862); the arithmetic is the ordinary entry point's, which
    // here already runs one workgroup per row with all loads in flight at once.
    if ((first_weight != nullptr && first_weight->encoding != kEncF32) ||
        (second_weight != nullptr && second_weight->encoding != kEncF32)) {
        return kInvalid;
    }
    return nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1(
        input, first_weight, residual_input, hidden_output, second_weight, normalized_output,
        residual_output, rows, width, first_eps, first_centered, second_eps, second_centered,
        cuda_stream);
}

int nfn_native_tile_glimmer_dual_rms_add_capture_mmvq_q8_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t rows, std::int64_t width, float first_eps,
    bool first_centered, float second_eps, bool second_centered, void* mmvq_workspace,
    std::int64_t mmvq_workspace_nbytes, void* cuda_stream) {
    Descriptor first{}, second{};
    // One row only; the records are those of the small-batch workspace, so the
    // width must be one the small-batch entry points take.
    const std::int64_t required = rows == 1 ? small_batch_workspace_bytes(1, width) : 0;
    if (mmvq_workspace == nullptr || rows != 1 || width % 256 != 0 || required == 0 ||
        mmvq_workspace_nbytes < required ||
        !dual_rms_arguments_valid(input, first_weight, residual_input, hidden_output,
                                  second_weight, normalized_output, residual_output, rows, width,
                                  first_eps, second_eps, &first, &second)) {
        return kInvalid;
    }
    launch_dual_rms_add_capture(input, first_weight != nullptr ? &first : nullptr, first_centered,
                                residual_input, hidden_output,
                                second_weight != nullptr ? &second : nullptr, second_centered,
                                normalized_output, residual_output, rows, width, first_eps,
                                second_eps, static_cast<std::uint8_t*>(mmvq_workspace), nullptr,
                                as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t width, float first_eps, bool first_centered,
    float second_eps, bool second_centered, const Descriptor* const* descriptors,
    float* const* outputs, std::int64_t operation_count, void* cuda_stream) {
    Descriptor first{}, second{};
    if (descriptors == nullptr || outputs == nullptr || operation_count < 1 ||
        operation_count > kMaxOperations || width % 256 != 0 ||
        !dual_rms_arguments_valid(input, first_weight, residual_input, hidden_output,
                                  second_weight, normalized_output, residual_output, 1, width,
                                  first_eps, second_eps, &first, &second)) {
        return kInvalid;
    }
    ProjectionSet set{};
    set.count = static_cast<int>(operation_count);
    set.input_dim = width;
    for (std::int64_t index = 0; index < operation_count; ++index) {
        if (outputs[index] == nullptr ||
            !validate_k_descriptor(descriptors[index], width, cuda_stream, false)) {
            return kInvalid;
        }
        set.op[index] = make_projection(*descriptors[index], outputs[index]);
    }
    if (!gemv_dot_normed_supports(set)) return kInvalid;
    // Every workgroup of the launch reads `input` and `residual_input` in its prologue and the
    // first one stores the three rows: a row stored over one that is still being read would
    // change what later workgroups normalise.  In-place calls (the engine's residual_output ==
    // residual_input) therefore keep to the two-call form.
    const auto overlaps = [width](const float* read, const float* written) {
        const auto a = reinterpret_cast<std::uintptr_t>(read);
        const auto b = reinterpret_cast<std::uintptr_t>(written);
        const std::uintptr_t bytes = static_cast<std::uintptr_t>(width) * sizeof(float);
        return a < b + bytes && b < a + bytes;
    };
    const float* const read_rows[2] = {input, residual_input};
    const float* const written_rows[3] = {hidden_output, residual_output, normalized_output};
    for (const float* read : read_rows) {
        for (const float* written : written_rows) {
            if (overlaps(read, written)) return kInvalid;
        }
    }
    for (std::int64_t index = 0; index < operation_count; ++index) {
        // (the projections' outputs are written while other workgroups may still read the rows)
        const auto out = reinterpret_cast<std::uintptr_t>(outputs[index]);
        const std::uintptr_t out_bytes =
            static_cast<std::uintptr_t>(set.op[index].output_dim) * sizeof(float);
        for (const float* read : read_rows) {
            const auto a = reinterpret_cast<std::uintptr_t>(read);
            if (a < out + out_bytes && out < a + static_cast<std::uintptr_t>(width) * sizeof(float)) {
                return kInvalid;
            }
        }
    }
    DualNormArguments norm{};
    norm.residual = residual_input;
    norm.first_weight = norm_weight(first_weight != nullptr ? &first : nullptr, first_centered);
    norm.second_weight = norm_weight(second_weight != nullptr ? &second : nullptr, second_centered);
    norm.hidden = hidden_output;
    norm.captured = residual_output;
    norm.normalized = normalized_output;
    norm.first_eps = first_eps;
    norm.second_eps = second_eps;
    launch_gemv_dot_normed(set, input, norm, as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t rows, std::int64_t width, float first_eps,
    bool first_centered, float second_eps, bool second_centered, void* mmq_workspace,
    std::int64_t mmq_workspace_nbytes, void* cuda_stream) {
    Descriptor first{}, second{};
    // Row counts that the small-batch entry points run on the fp16 kernel, rows that the
    // register-resident norm kernel takes, a width that kernel reads.
    const bool rows_fit = rows >= 5 && rows <= kMaxSmallRows;
    const std::int64_t required = rows_fit ? small_batch_workspace_bytes(rows, width) : 0;
    if (mmq_workspace == nullptr || !rows_fit || width % 256 != 0 || width > 8192 ||
        required == 0 || mmq_workspace_nbytes < required ||
        !dual_rms_arguments_valid(input, first_weight, residual_input, hidden_output,
                                  second_weight, normalized_output, residual_output, rows, width,
                                  first_eps, second_eps, &first, &second)) {
        return kInvalid;
    }
    launch_dual_rms_add_capture(input, first_weight != nullptr ? &first : nullptr, first_centered,
                                residual_input, hidden_output,
                                second_weight != nullptr ? &second : nullptr, second_centered,
                                normalized_output, residual_output, rows, width, first_eps,
                                second_eps, nullptr, static_cast<std::uint8_t*>(mmq_workspace),
                                as_stream(cuda_stream));
    return launch_status();
}

int nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1(
    const float* input, const Descriptor* first_weight, const float* residual_input,
    float* hidden_output, const Descriptor* second_weight, float* normalized_output,
    float* residual_output, std::int64_t rows, std::int64_t width, float first_eps,
    bool first_centered, float second_eps, bool second_centered, void* mmvq_workspace,
    std::int64_t mmvq_workspace_nbytes, void* cuda_stream) {
    Descriptor first{}, second{};
    // Row counts that the exact verifier's entry points run on the matrix-core kernel, rows
    // that the register-resident norm kernel takes.
    const bool rows_fit = rows >= kFirstVerifierMatrixRows && rows <= kMaxSmallRows;
    const std::int64_t required = rows_fit ? small_batch_workspace_bytes(rows, width) : 0;
    if (mmvq_workspace == nullptr || !rows_fit || width % 256 != 0 || width > 8192 ||
        required == 0 || mmvq_workspace_nbytes < required ||
        !dual_rms_arguments_valid(input, first_weight, residual_input, hidden_output,
                                  second_weight, normalized_output, residual_output, rows, width,
                                  first_eps, second_eps, &first, &second)) {
        return kInvalid;
    }
    std::uint8_t* records = static_cast<std::uint8_t*>(mmvq_workspace);
    launch_dual_rms_add_capture(input, first_weight != nullptr ? &first : nullptr, first_centered,
                                residual_input, hidden_output,
                                second_weight != nullptr ? &second : nullptr, second_centered,
                                normalized_output, residual_output, rows, width, first_eps,
                                second_eps, records, nullptr, as_stream(cuda_stream),
                                records + record_bytes(rows, width));
    return launch_status();
}

namespace {
// Widest input the fp16 form of the lm_head takes: the workspace query does not know the
// input width and sizes that form's fp16 copy of the rows for this one.
constexpr std::int64_t kLmHeadHalfWidth = 16384;
// rows from which the fp16 form runs: those of the small-batch call, so that the fused result
// is the maximum of that call's logits; two rows of Q6_K as well (there the small-batch call
// keeps the one-row arithmetic, which no fused form of two rows has: 249 -> 225 us)
constexpr std::int64_t kLmHeadOtherRows = 8;  // rows up to which the other forms run
constexpr std::int64_t kLmHeadFirstHalfRowsQ6 = 2;

bool lm_head_half_form(const nfn::Descriptor& weight, std::int64_t rows) {
    const std::int64_t first_rows =
        weight.encoding == nfn::kEncQ6K ? kLmHeadFirstHalfRowsQ6 : first_half_rows(weight.encoding);
    // (its kernel keeps row numbers in 32 bits)
    return rows >= first_rows && rows <= 16 && weight.input_dim <= kLmHeadHalfWidth &&
        weight.output_dim <= std::numeric_limits<std::int32_t>::max() &&
        nfn::gemv_f16_supports(weight.encoding, weight.input_dim);
}
}  // namespace

std::int64_t nfn_mi355_lm_head_argmax_workspace_bytes_v1(std::int64_t rows,
                                                         std::int64_t output_dim) {
    if (rows < 1 || rows > 16 || output_dim <= 0) return 0;
    std::int64_t raw = 0;
    if (rows <= kLmHeadOtherRows) {
        // room for either kernel's per-workgroup candidates
        std::int64_t groups = lm_head_f32_blocks(output_dim);
        if (lm_head_q6_max_groups(output_dim) > groups) groups = lm_head_q6_max_groups(output_dim);
        if (lm_head_mfma_tiles(output_dim) > groups) groups = lm_head_mfma_tiles(output_dim);
        raw = rows * groups * static_cast<std::int64_t>(sizeof(LmHeadCandidate));
    }
    if (rows >= kLmHeadFirstHalfRowsQ6) {  // (the query does not know the encoding either)
        raw = std::max(raw, lm_head_f16_workspace_bytes(rows, kLmHeadHalfWidth));
    }
    return (raw + 255) & ~std::int64_t(255);
}

int nfn_mi355_lm_head_argmax_v1(const Descriptor* descriptor, const float* input,
                                std::int64_t* output_indices, float* output_values,
                                std::int64_t rows, void* workspace,
                                std::int64_t workspace_nbytes, void* cuda_stream) {
    Descriptor normalized{};
    if (!normalize_descriptor(descriptor, &normalized) || input == nullptr ||
        output_indices == nullptr || output_values == nullptr || workspace == nullptr ||
        (normalized.cuda_stream != nullptr && normalized.cuda_stream != cuda_stream)) {
        return kInvalid;
    }
    const std::int64_t required =
        nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, normalized.output_dim);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    // Five rows and more (Q6_K: two): the fp16 matrix-core kernel (one pass over the weights
    // for up to sixteen rows), the only form beyond eight rows.  Two rows and more: the int8
    // matrix-core kernel (one pass for up to four rows).  One row of Q6_K: the streaming
    // dot kernel.
    if (lm_head_half_form(normalized, rows)) {
        launch_lm_head_f16(normalized, input, rows, workspace, output_indices, output_values,
                           as_stream(cuda_stream));
    } else if (rows > kLmHeadOtherRows) {
        return kInvalid;
    } else if (rows >= 2 && gemv_mfma_supports(normalized.encoding, normalized.input_dim)) {
        launch_lm_head_mfma(normalized, input, rows, static_cast<LmHeadCandidate*>(workspace),
                            output_indices, output_values, as_stream(cuda_stream));
    } else if (gemv_q6_supports(normalized.encoding, normalized.input_dim)) {
        launch_lm_head_q6(normalized, input, rows, static_cast<LmHeadCandidate*>(workspace),
                          output_indices, output_values, as_stream(cuda_stream));
    } else {
        launch_lm_head_f32(normalized, input, rows, static_cast<LmHeadCandidate*>(workspace),
                           output_indices, output_values, as_stream(cuda_stream));
    }
    return launch_status();
}

std::int64_t nfn_mi355_k_quant_gemm_workspace_bytes_v1(std::int64_t rows, std::int64_t input_dim,
                                                       std::int64_t output_dim, int mode) {
    if (rows <= 0 || input_dim <= 0 || input_dim % 256 != 0 || output_dim <= 0 ||
        mode != NFN_MI355_GEMM_F16) {
        return 0;
    }
    return gemm_f16_workspace_bytes(rows, input_dim, output_dim);
}

int nfn_mi355_k_quant_gemm_plan_v1(std::uint32_t encoding, std::int64_t rows, std::int64_t input_dim,
                                   std::int64_t output_dim, int mode, int* tile_rows,
                                   int* k_shares) {
    if (tile_rows == nullptr || k_shares == nullptr || rows <= 0 || output_dim <= 0 ||
        input_dim <= 0 || mode != NFN_MI355_GEMM_F16 || !gemm_f16_supports(encoding, input_dim)) {
        return kInvalid;
    }
    gemm_f16_plan(encoding, rows, input_dim, output_dim, tile_rows, k_shares);
    return 0;
}

int nfn_mi355_k_quant_gemm_float32_v1(const Descriptor* descriptor, const float* input,
                                      float* output, std::int64_t rows, void* workspace,
                                      std::int64_t workspace_nbytes, int mode,
                                      void* cuda_stream) {
    Descriptor normalized{};
    if (input == nullptr || output == nullptr || workspace == nullptr || rows <= 0 ||
        !validate_k_descriptor(descriptor, descriptor == nullptr ? 0 : descriptor->input_dim,
                               cuda_stream, true) ||
        !normalize_descriptor(descriptor, &normalized)) {
        return kInvalid;
    }
    const std::int64_t required = nfn_mi355_k_quant_gemm_workspace_bytes_v1(
        rows, normalized.input_dim, normalized.output_dim, mode);
    if (required == 0 || workspace_nbytes < required) return kInvalid;
    if (gemm_f16_supports(normalized.encoding, normalized.input_dim)) {
        if (reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) return kInvalid;
        launch_gemm_f16(normalized, input, output, rows, workspace, as_stream(cuda_stream));
        return launch_status();
    }
    ProjectionSet set{};
    set.count = 1;
    set.input_dim = normalized.input_dim;
    set.op[0] = make_projection(normalized, output);
    constexpr std::int64_t kChunk = 65535 * 8;
    for (std::int64_t row = 0; row < rows; row += kChunk) {
        const std::int64_t count = rows - row < kChunk ? rows - row : kChunk;
        set.op[0].output = output + row * normalized.output_dim;
        launch_gemv_f32(set, input + row * normalized.input_dim, nullptr, kPlain, nullptr, count,
                        as_stream(cuda_stream));
    }
    return launch_status();
}

int nfn_mi355_k_quant_gemm_multi_float32_v1(const Descriptor* const* descriptors, const float* input,
                                            float* const* outputs, std::int64_t operation_count,
                                            std::int64_t rows, void* workspace,
                                            std::int64_t workspace_nbytes, int mode,
                                            void* cuda_stream) {
    if (descriptors == nullptr || input == nullptr || outputs == nullptr || workspace == nullptr ||
        operation_count < 1 || operation_count > kMaxOperations || rows <= 0 ||
        mode != NFN_MI355_GEMM_F16 || reinterpret_cast<std::uintptr_t>(workspace) % 16 != 0) {
        return kInvalid;
    }
    Descriptor normalized[kMaxOperations];
    std::int64_t required = 0;
    for (std::int64_t index = 0; index < operation_count; ++index) {
        const Descriptor* descriptor = descriptors[index];
        if (outputs[index] == nullptr ||
            !validate_k_descriptor(descriptor, descriptors[0] == nullptr ? 0 : descriptors[0]->input_dim,
                                   cuda_stream, true) ||
            !normalize_descriptor(descriptor, &normalized[index]) ||
            !gemm_f16_supports(normalized[index].encoding, normalized[index].input_dim)) {
            return kInvalid;
        }
        const std::int64_t bytes = nfn_mi355_k_quant_gemm_workspace_bytes_v1(
            rows, normalized[index].input_dim, normalized[index].output_dim, mode);
        if (bytes == 0) return kInvalid;
        if (bytes > required) required = bytes;
    }
    if (workspace_nbytes < required) return kInvalid;
    const hipStream_t stream = as_stream(cuda_stream);
    convert_gemm_activations(input, rows, normalized[0].input_dim, workspace, stream);
    for (std::int64_t index = 0; index < operation_count; ++index) {
        launch_gemm_f16_converted(normalized[index], outputs[index], rows, workspace, stream);
    }
    return launch_status();
}

}  // extern "C"
