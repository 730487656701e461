// Host-side weight quantizers: float rows -> ggml Q4_K / Q5_K / Q6_K / Q8_0
// blocks.  They exist to make synthetic packed tensors for the parity tests
// and the benchmark; no kernel depends on them.
//
// The reference has no quantizer (it only reads GGUF files written by
// llama.cpp), so these restate the published ggml algorithms
// (ggml-quants.c: quantize_row_q4_K_ref, quantize_row_q5_K_ref,
// quantize_row_q6_K_ref, quantize_row_q8_0_ref with make_qkx2_quants and
// make_qx_quants) against the block layouts the reference vendors in
// neuralfn/csrc/tile_cuda/vendor/llama_mmq_62bf73d/ggml/src/ggml-common.h:251-368.
// Parity of the *encoding choice* with llama.cpp is unpinned and irrelevant to
// kernel parity: kernel and oracle consume the same packed bytes.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <thread>
#include <vector>

namespace {

constexpr float kGroupMaxEps = 1e-15f;

inline int nearest_int(float value) {
    // Round half to even through the float magic constant, as ggml does.
    const float shifted = value + 12582912.f;
    int bits;
    std::memcpy(&bits, &shifted, sizeof(bits));
    return (bits & 0x007fffff) - 0x00400000;
}

std::uint16_t float_to_half_bits(float value) {
    std::uint32_t bits;
    std::memcpy(&bits, &value, sizeof(bits));
    const std::uint32_t sign = (bits >> 16) & 0x8000u;
    const std::uint32_t magnitude = bits & 0x7fffffffu;
    std::uint32_t half;
    if (magnitude >= 0x7f800000u) {
        half = magnitude > 0x7f800000u ? 0x7e00u : 0x7c00u;
    } else if (magnitude >= 0x477ff000u) {
        half = 0x7c00u;
    } else if (magnitude >= 0x38800000u) {
        const std::uint32_t shifted = magnitude - 0x38000000u;
        half = (shifted + 0x0fffu + ((shifted >> 13) & 1u)) >> 13;
    } else if (magnitude >= 0x33000000u) {
        float positive;
        std::memcpy(&positive, &magnitude, sizeof(positive));
        half = static_cast<std::uint32_t>(std::nearbyint(std::ldexp(positive, 24)));
    } else {
        half = 0;
    }
    return static_cast<std::uint16_t>(sign | half);
}

float half_bits_to_float(std::uint16_t bits) {
    const int exponent = (bits >> 10) & 0x1f;
    const int mantissa = bits & 0x3ff;
    float value;
    if (exponent == 0) value = std::ldexp(static_cast<float>(mantissa), -24);
    else if (exponent == 31) value = mantissa ? NAN : INFINITY;
    else value = std::ldexp(1.0f + mantissa / 1024.0f, exponent - 15);
    return (bits & 0x8000) ? -value : value;
}

void store_half(std::uint8_t* target, float value) {
    const std::uint16_t bits = float_to_half_bits(value);
    std::memcpy(target, &bits, 2);
}

float make_qkx2_quants(int n, int nmax, const float* x, const float* weights, std::uint8_t* L,
                       float* the_min, std::uint8_t* Laux, float rmin, float rdelta, int nstep) {
    float min = x[0];
    float max = x[0];
    float sum_w = weights[0];
    float sum_x = sum_w * x[0];
    for (int i = 1; i < n; ++i) {
        if (x[i] < min) min = x[i];
        if (x[i] > max) max = x[i];
        const float w = weights[i];
        sum_w += w;
        sum_x += w * x[i];
    }
    if (min > 0) min = 0;
    if (max == min) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        *the_min = -min;
        return 0.f;
    }
    float iscale = nmax / (max - min);
    float scale = 1 / iscale;
    float best_error = 0;
    for (int i = 0; i < n; ++i) {
        const int l = nearest_int(iscale * (x[i] - min));
        L[i] = static_cast<std::uint8_t>(std::max(0, std::min(nmax, l)));
        const float diff = scale * L[i] + min - x[i];
        best_error += weights[i] * diff * diff;
    }
    for (int is = 0; is <= nstep; ++is) {
        iscale = (rmin + rdelta * is + nmax) / (max - min);
        float sum_l = 0, sum_l2 = 0, sum_xl = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * (x[i] - min));
            l = std::max(0, std::min(nmax, l));
            Laux[i] = static_cast<std::uint8_t>(l);
            const float w = weights[i];
            sum_l += w * l;
            sum_l2 += w * l * l;
            sum_xl += w * l * x[i];
        }
        const float D = sum_w * sum_l2 - sum_l * sum_l;
        if (D > 0) {
            float this_scale = (sum_w * sum_xl - sum_x * sum_l) / D;
            float this_min = (sum_l2 * sum_x - sum_l * sum_xl) / D;
            if (this_min > 0) {
                this_min = 0;
                this_scale = sum_xl / sum_l2;
            }
            float error = 0;
            for (int i = 0; i < n; ++i) {
                const float diff = this_scale * Laux[i] + this_min - x[i];
                error += weights[i] * diff * diff;
            }
            if (error < best_error) {
                for (int i = 0; i < n; ++i) L[i] = Laux[i];
                best_error = error;
                scale = this_scale;
                min = this_min;
            }
        }
    }
    *the_min = -min;
    return scale;
}

void scale_min_of(int j, const std::uint8_t* q, std::uint8_t* d, std::uint8_t* m) {
    if (j < 4) {
        *d = q[j] & 63;
        *m = q[j + 4] & 63;
    } else {
        *d = (q[j + 4] & 0xF) | ((q[j - 4] >> 6) << 4);
        *m = (q[j + 4] >> 4) | ((q[j - 0] >> 6) << 4);
    }
}

// Shared front half of Q4_K and Q5_K: choose sub-block scales/mins, pack the
// 12 scale bytes and the two half-precision super-block factors, then
// requantize against the packed values.  `block` points at d.
void quantize_k45_block(const float* x, std::uint8_t* block, int nmax, float rmin, float rdelta,
                        int nstep, std::uint8_t* L) {
    std::uint8_t Laux[32];
    float weights[32];
    float mins[8];
    float scales[8];
    float max_scale = 0;
    float max_min = 0;
    for (int j = 0; j < 8; ++j) {
        float sum_x2 = 0;
        for (int l = 0; l < 32; ++l) sum_x2 += x[32 * j + l] * x[32 * j + l];
        const float av_x = std::sqrt(sum_x2 / 32);
        for (int l = 0; l < 32; ++l) weights[l] = av_x + std::fabs(x[32 * j + l]);
        scales[j] = make_qkx2_quants(32, nmax, x + 32 * j, weights, L + 32 * j, &mins[j], Laux,
                                     rmin, rdelta, nstep);
        max_scale = std::max(max_scale, scales[j]);
        max_min = std::max(max_min, mins[j]);
    }
    const float inv_scale = max_scale > 0 ? 63.f / max_scale : 0.f;
    const float inv_min = max_min > 0 ? 63.f / max_min : 0.f;
    std::uint8_t* packed = block + 4;
    std::memset(packed, 0, 12);
    for (int j = 0; j < 8; ++j) {
        std::uint8_t ls = static_cast<std::uint8_t>(nearest_int(inv_scale * scales[j]));
        std::uint8_t lm = static_cast<std::uint8_t>(nearest_int(inv_min * mins[j]));
        ls = std::min<std::uint8_t>(63, ls);
        lm = std::min<std::uint8_t>(63, lm);
        if (j < 4) {
            packed[j] = ls;
            packed[j + 4] = lm;
        } else {
            packed[j + 4] = (ls & 0xF) | ((lm & 0xF) << 4);
            packed[j - 4] |= ((ls >> 4) << 6);
            packed[j - 0] |= ((lm >> 4) << 6);
        }
    }
    store_half(block, max_scale / 63.f);
    store_half(block + 2, max_min / 63.f);
    std::uint16_t d_bits, dmin_bits;
    std::memcpy(&d_bits, block, 2);
    std::memcpy(&dmin_bits, block + 2, 2);
    const float d_all = half_bits_to_float(d_bits);
    const float dmin_all = half_bits_to_float(dmin_bits);
    for (int j = 0; j < 8; ++j) {
        std::uint8_t sc, m;
        scale_min_of(j, packed, &sc, &m);
        const float d = d_all * sc;
        if (!d) continue;
        const float dm = dmin_all * m;
        for (int ii = 0; ii < 32; ++ii) {
            int l = nearest_int((x[32 * j + ii] + dm) / d);
            l = std::max(0, std::min(nmax, l));
            L[32 * j + ii] = static_cast<std::uint8_t>(l);
        }
    }
}

void quantize_q4_k_block(const float* x, std::uint8_t* block) {
    std::uint8_t L[256];
    quantize_k45_block(x, block, 15, -1.f, 0.1f, 20, L);
    std::uint8_t* q = block + 16;
    for (int j = 0; j < 256; j += 64) {
        for (int l = 0; l < 32; ++l) q[l] = L[j + l] | (L[j + l + 32] << 4);
        q += 32;
    }
}

void quantize_q5_k_block(const float* x, std::uint8_t* block) {
    std::uint8_t L[256];
    quantize_k45_block(x, block, 31, -0.5f, 0.1f, 15, L);
    std::uint8_t* qh = block + 16;
    std::uint8_t* ql = block + 48;
    std::memset(qh, 0, 32);
    std::uint8_t m1 = 1, m2 = 2;
    for (int n = 0; n < 256; n += 64) {
        for (int j = 0; j < 32; ++j) {
            int l1 = L[n + j];
            if (l1 > 15) { l1 -= 16; qh[j] |= m1; }
            int l2 = L[n + j + 32];
            if (l2 > 15) { l2 -= 16; qh[j] |= m2; }
            ql[j] = static_cast<std::uint8_t>(l1 | (l2 << 4));
        }
        m1 <<= 2;
        m2 <<= 2;
        ql += 32;
    }
}

float make_qx_quants(int n, int nmax, const float* x, std::int8_t* L) {
    float max = 0;
    float amax = 0;
    for (int i = 0; i < n; ++i) {
        const float ax = std::fabs(x[i]);
        if (ax > amax) { amax = ax; max = x[i]; }
    }
    if (amax < kGroupMaxEps) {
        for (int i = 0; i < n; ++i) L[i] = 0;
        return 0.f;
    }
    float iscale = -nmax / max;
    float sumlx = 0;
    float suml2 = 0;
    for (int i = 0; i < n; ++i) {
        int l = nearest_int(iscale * x[i]);
        l = std::max(-nmax, std::min(nmax - 1, l));
        L[i] = static_cast<std::int8_t>(l + nmax);
        const float w = x[i] * x[i];
        sumlx += w * x[i] * l;
        suml2 += w * l * l;
    }
    float scale = suml2 ? sumlx / suml2 : 0.0f;
    float best = scale * sumlx;
    for (int is = -9; is <= 9; ++is) {
        if (is == 0) continue;
        iscale = -(nmax + 0.1f * is) / max;
        sumlx = suml2 = 0;
        for (int i = 0; i < n; ++i) {
            int l = nearest_int(iscale * x[i]);
            l = std::max(-nmax, std::min(nmax - 1, l));
            const float w = x[i] * x[i];
            sumlx += w * x[i] * l;
            suml2 += w * l * l;
        }
        if (suml2 > 0 && sumlx * sumlx > best * suml2) {
            for (int i = 0; i < n; ++i) {
                const int l = nearest_int(iscale * x[i]);
                L[i] = static_cast<std::int8_t>(nmax + std::max(-nmax, std::min(nmax - 1, l)));
            }
            scale = sumlx / suml2;
            best = scale * sumlx;
        }
    }
    return scale;
}

void quantize_q6_k_block(const float* x, std::uint8_t* block) {
    std::int8_t L[256];
    float scales[16];
    float max_scale = 0;
    float max_abs_scale = 0;
    for (int ib = 0; ib < 16; ++ib) {
        const float scale = make_qx_quants(16, 32, x + 16 * ib, L + 16 * ib);
        scales[ib] = scale;
        const float abs_scale = std::fabs(scale);
        if (abs_scale > max_abs_scale) {
            max_abs_scale = abs_scale;
            max_scale = scale;
        }
    }
    if (max_abs_scale < kGroupMaxEps) {
        std::memset(block, 0, 210);
        return;
    }
    const float iscale = -128.f / max_scale;
    store_half(block + 208, 1 / iscale);
    std::int8_t* packed_scales = reinterpret_cast<std::int8_t*>(block + 192);
    for (int ib = 0; ib < 16; ++ib) {
        packed_scales[ib] = static_cast<std::int8_t>(std::min(127, nearest_int(iscale * scales[ib])));
    }
    std::uint16_t d_bits;
    std::memcpy(&d_bits, block + 208, 2);
    const float d_all = half_bits_to_float(d_bits);
    for (int j = 0; j < 16; ++j) {
        const float d = d_all * packed_scales[j];
        if (!d) continue;
        for (int ii = 0; ii < 16; ++ii) {
            int l = nearest_int(x[16 * j + ii] / d);
            l = std::max(-32, std::min(31, l));
            L[16 * j + ii] = static_cast<std::int8_t>(l + 32);
        }
    }
    std::uint8_t* ql = block;
    std::uint8_t* qh = block + 128;
    for (int j = 0; j < 256; j += 128) {
        for (int l = 0; l < 32; ++l) {
            const std::uint8_t q1 = L[j + l + 0] & 0xF;
            const std::uint8_t q2 = L[j + l + 32] & 0xF;
            const std::uint8_t q3 = L[j + l + 64] & 0xF;
            const std::uint8_t q4 = L[j + l + 96] & 0xF;
            ql[l + 0] = q1 | (q3 << 4);
            ql[l + 32] = q2 | (q4 << 4);
            qh[l] = static_cast<std::uint8_t>((L[j + l] >> 4) | ((L[j + l + 32] >> 4) << 2) |
                                              ((L[j + l + 64] >> 4) << 4) |
                                              ((L[j + l + 96] >> 4) << 6));
        }
        ql += 64;
        qh += 32;
    }
}

void quantize_q8_0_block(const float* x, std::uint8_t* block) {
    float amax = 0.0f;
    for (int j = 0; j < 32; ++j) amax = std::max(amax, std::fabs(x[j]));
    const float d = amax / 127.f;
    const float id = d ? 1.0f / d : 0.0f;
    store_half(block, d);
    for (int j = 0; j < 32; ++j) {
        block[2 + j] = static_cast<std::uint8_t>(static_cast<std::int8_t>(std::round(x[j] * id)));
    }
}

}  // namespace

extern "C" {

// Quantize a row-major [rows, cols] float matrix into `output`
// (rows * cols/block_elements * block_bytes bytes).  encoding: 8, 12, 13, 14.
// Returns 0, or 1 for an unsupported encoding or a ragged column count.
int nfn_mi355_quantize_rows(std::uint32_t encoding, const float* input, std::int64_t rows,
                            std::int64_t cols, std::uint8_t* output, int threads) {
    std::int64_t elements = 256;
    std::int64_t bytes = 0;
    void (*quantize)(const float*, std::uint8_t*) = nullptr;
    switch (encoding) {
        case 8: elements = 32; bytes = 34; quantize = quantize_q8_0_block; break;
        case 12: bytes = 144; quantize = quantize_q4_k_block; break;
        case 13: bytes = 176; quantize = quantize_q5_k_block; break;
        case 14: bytes = 210; quantize = quantize_q6_k_block; break;
        default: return 1;
    }
    if (rows <= 0 || cols <= 0 || cols % elements != 0) return 1;
    const std::int64_t blocks_per_row = cols / elements;
    const std::int64_t total = rows * blocks_per_row;
    int workers = threads > 0 ? threads
                              : static_cast<int>(std::max(1u, std::thread::hardware_concurrency()));
    workers = static_cast<int>(std::min<std::int64_t>(workers, std::max<std::int64_t>(1, total / 64)));
    auto work = [&](std::int64_t begin, std::int64_t end) {
        for (std::int64_t index = begin; index < end; ++index) {
            quantize(input + index * elements, output + index * bytes);
        }
    };
    if (workers <= 1) {
        work(0, total);
        return 0;
    }
    std::vector<std::thread> pool;
    for (int w = 0; w < workers; ++w) {
        pool.emplace_back(work, total * w / workers, total * (w + 1) / workers);
    }
    for (auto& thread : pool) thread.join();
    return 0;
}

}  // extern "C"
