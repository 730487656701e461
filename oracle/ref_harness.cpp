// Harness that exposes the reference engine's own CPU K-Quant arithmetic
// through a small C ABI.  TEST INFRASTRUCTURE ONLY.
//
// The reference keeps linear() in an anonymous namespace
// (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:653-679) and
// GlimmerModel::WeightView public (resident_glimmer.h:293-300), so the only way
// to execute them is a translation unit that textually includes
// resident_glimmer.cpp.  The Makefile passes that file with -include from the
// reference checkout where it lies; nothing of the reference is copied into
// this repository.  The resulting library is used to validate the CPU
// restatement in kquant_oracle.cpp and, optionally, as the timed CPU baseline.

#include <atomic>
#include <cstdint>
#include <vector>

#ifndef NFN_REF_INCLUDED
#error "build with -include <reference>/neuralfn/csrc/native_gpt2/resident_glimmer.cpp -DNFN_REF_INCLUDED"
#endif

namespace {

using View = neuralfn::resident_glimmer::GlimmerModel::WeightView;

bool make_view(std::uint32_t encoding, const std::uint8_t* data, std::int64_t out_dim,
               std::int64_t in_dim, View* view) {
    std::int64_t stride = 0;
    switch (encoding) {
        case 0: view->encoding = View::Encoding::F32; stride = in_dim * 4; break;
        case 30: view->encoding = View::Encoding::BF16; stride = in_dim * 2; break;
        case 12: view->encoding = View::Encoding::Q4K; stride = in_dim / 256 * 144; break;
        case 13: view->encoding = View::Encoding::Q5K; stride = in_dim / 256 * 176; break;
        case 14: view->encoding = View::Encoding::Q6K; stride = in_dim / 256 * 210; break;
        default: return false;
    }
    view->data = data;
    view->rows = out_dim;
    view->cols = in_dim;
    view->row_stride_bytes = stride;
    view->nbytes = out_dim * stride;
    return true;
}

}  // namespace

extern "C" {

float nfr_fp16_to_float(std::uint16_t bits) {
    std::uint8_t bytes[2];
    std::memcpy(bytes, &bits, 2);
    return neuralfn::resident_glimmer::fp16_to_float(bytes);
}

void nfr_k_scale_min(const std::uint8_t* scales, int index, int* scale, int* minimum) {
    neuralfn::resident_glimmer::k_scale_min(scales, index, scale, minimum);
}

int nfr_dequantize(std::uint32_t encoding, const std::uint8_t* data, std::int64_t out_dim,
                   std::int64_t in_dim, float* out) {
    View view;
    if (!make_view(encoding, data, out_dim, in_dim, &view)) return 1;
    for (std::int64_t row = 0; row < out_dim; ++row) {
        for (std::int64_t col = 0; col < in_dim; ++col) {
            out[row * in_dim + col] = view.value(row, col);
        }
    }
    return 0;
}

// One call of the reference's linear() per input row, as the engine does
// (resident_glimmer.cpp:1937-1941 runs one hidden row at a time).
int nfr_linear(std::uint32_t encoding, const std::uint8_t* data, std::int64_t out_dim,
               std::int64_t in_dim, const float* input, std::int64_t rows, float* output) {
    View view;
    if (!make_view(encoding, data, out_dim, in_dim, &view)) return 1;
    const std::atomic<bool> cancelled{false};
    try {
        for (std::int64_t row = 0; row < rows; ++row) {
            const std::vector<float> source(input + row * in_dim, input + (row + 1) * in_dim);
            std::vector<float> result;
            neuralfn::resident_glimmer::linear(source, view, &result, cancelled);
            std::copy(result.begin(), result.end(), output + row * out_dim);
        }
    } catch (const std::exception&) {
        return 2;
    }
    return 0;
}

// The reference's CPU RMSNorm (resident_glimmer.cpp:713-745) with an optional
// F32 weight row.
int nfr_rms_norm(const float* input, const float* weight, int centered, std::int64_t width,
                 double epsilon, float* output) {
    View view;
    if (weight != nullptr) {
        if (!make_view(0, reinterpret_cast<const std::uint8_t*>(weight), 1, width, &view)) return 1;
        view.centered = centered != 0;
    }
    const std::atomic<bool> cancelled{false};
    try {
        const std::vector<float> source(input, input + width);
        std::vector<float> result;
        neuralfn::resident_glimmer::rms_norm(source, weight != nullptr ? &view : nullptr, epsilon,
                                            &result, cancelled);
        std::copy(result.begin(), result.end(), output);
    } catch (const std::exception&) {
        return 2;
    }
    return 0;
}

std::int64_t nfr_argmax(const float* values, std::int64_t count) {
    const std::vector<float> logits(values, values + count);
    return neuralfn::resident_glimmer::argmax_token(logits);
}

// The reference's CPU rotary position embedding (resident_glimmer.cpp:773-800),
// in place on `heads` heads of one position.
int nfr_apply_rope(float* values, std::int64_t heads, std::int64_t head_dim, std::int64_t position,
                   double theta, int interleaved) {
    const std::atomic<bool> cancelled{false};
    try {
        std::vector<float> buffer(values, values + heads * head_dim);
        neuralfn::resident_glimmer::apply_rope(&buffer, heads, head_dim, position, theta,
                                               interleaved != 0, cancelled);
        std::copy(buffer.begin(), buffer.end(), values);
    } catch (const std::exception&) {
        return 2;
    }
    return 0;
}

// The reference's CPU per-head norm (resident_glimmer.cpp:746-771) with an
// optional F32 weight row.
int nfr_qk_norm(float* values, std::int64_t heads, std::int64_t head_dim, const float* weight,
                double epsilon, double scalar) {
    View view;
    if (weight != nullptr &&
        !make_view(0, reinterpret_cast<const std::uint8_t*>(weight), 1, head_dim, &view)) {
        return 1;
    }
    const std::atomic<bool> cancelled{false};
    try {
        std::vector<float> buffer(values, values + heads * head_dim);
        neuralfn::resident_glimmer::qk_norm_in_place(&buffer, heads, head_dim,
                                                     weight != nullptr ? &view : nullptr, epsilon,
                                                     scalar, cancelled);
        std::copy(buffer.begin(), buffer.end(), values);
    } catch (const std::exception&) {
        return 2;
    }
    return 0;
}

}  // extern "C"
