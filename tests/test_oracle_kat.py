"""Pins the CPU oracle before anything is compared against it.

Known-answer blocks are the reference's own (tests/test_native_gguf.py:510-553
and tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:640-681); everything else is
fixed by closed forms that a dropped term, a wrong index or a swapped nibble
would break.
"""
import struct

import numpy as np
import pytest

from neuralfn_amd import kquant

SCALES = bytes((1, 2, 3, 4, 5, 6, 7, 8, 0, 0, 0, 0))


def test_fp16_decode_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    expected = bits.view(np.float16).astype(np.float32)
    actual = np.array([oracle.fp16_to_float(int(b)) for b in bits], dtype=np.float32)
    nan = np.isnan(expected)
    assert np.array_equal(np.isnan(actual), nan)
    assert np.array_equal(actual[~nan].view(np.uint32), expected[~nan].view(np.uint32))


def _scale_min_bitfield(scales: bytes, j: int):
    """ggml's get_scale_min_k4 restated over one 96-bit little-endian integer."""
    word = int.from_bytes(scales, "little")

    def byte(i):
        return (word >> (8 * i)) & 0xFF

    if j < 4:
        return byte(j) & 63, byte(j + 4) & 63
    scale = (byte(j + 4) & 0xF) | ((byte(j - 4) >> 6) << 4)
    minimum = (byte(j + 4) >> 4) | ((byte(j) >> 6) << 4)
    return scale, minimum


def test_k_scale_min_roundtrip(oracle):
    # Pack chosen 6-bit scales/mins the way ggml's quantizer does, then decode.
    rng = np.random.default_rng(7)
    for _ in range(200):
        ls = rng.integers(0, 64, 8)
        lm = rng.integers(0, 64, 8)
        packed = bytearray(12)
        for j in range(8):
            if j < 4:
                packed[j] = ls[j]
                packed[j + 4] = lm[j]
            else:
                packed[j + 4] = (ls[j] & 0xF) | ((lm[j] & 0xF) << 4)
                packed[j - 4] |= (ls[j] >> 4) << 6
                packed[j] |= (lm[j] >> 4) << 6
        for j in range(8):
            assert oracle.k_scale_min(bytes(packed), j) == (ls[j], lm[j])
            assert _scale_min_bitfield(bytes(packed), j) == (ls[j], lm[j])


def test_q4_k_known_answer(oracle):
    block = struct.pack("<ee", 1.0, 0.5) + SCALES + bytes([0x21] * 128)
    v = oracle.dequantize(kquant.Q4_K, np.frombuffer(block, np.uint8), 1, 256)[0]
    assert np.all(v[:32] == -1.5)
    assert np.all(v[32:64] == 1.0)
    assert np.all(v[64:96] == -0.5)
    assert np.all(v[96:128] == 4.0)
    # sub-blocks 4..7: scale/min come from the split 6-bit fields (all zero high
    # bits here): scale = byte[j+4]&15, min = byte[j+4]>>4 with bytes 8..11 = 0.
    assert np.all(v[128:] == 0.0)


def test_q5_k_known_answer(oracle):
    high = bytearray(32)
    high[0] = 3
    block = struct.pack("<ee", 1.0, 0.5) + SCALES + bytes(high) + bytes([0x21] * 128)
    v = oracle.dequantize(kquant.Q5_K, np.frombuffer(block, np.uint8), 1, 256)[0]
    assert (v[0], v[1], v[32], v[33]) == (14.5, -1.5, 33.0, 1.0)


def test_q6_k_known_answer_and_as_written_divergence(oracle):
    block = bytes(128) + bytes(64) + struct.pack("<16b", *range(1, 17)) + struct.pack("<e", 0.5)
    data = np.frombuffer(block, np.uint8)
    v = oracle.dequantize(kquant.Q6_K, data, 1, 256)[0]
    assert (v[0], v[16], v[32], v[64], v[128]) == (-16.0, -32.0, -48.0, -80.0, -144.0)
    # The reference CPU engine (resident_glimmer.cpp:614) drops `lane/16`:
    # element 16 then uses sub-scale 0 instead of 1.
    w = oracle.dequantize(kquant.Q6_K, data, 1, 256, q6_as_written=True)[0]
    assert w[16] == -16.0 and w[0] == -16.0 and w[32] == -48.0
    assert np.count_nonzero(v != w) == 128


def test_q6_k_every_position(oracle):
    # One distinct 6-bit code per element, unit scales: checks nibble/2-bit routing.
    codes = (np.arange(256) * 7 + 3) % 64
    ql = np.zeros(128, np.uint8)
    qh = np.zeros(64, np.uint8)
    for e, q in enumerate(codes):
        half, pos = divmod(e, 128)
        quarter, lane = divmod(pos, 32)
        byte = half * 64 + lane + (32 if quarter in (1, 3) else 0)
        ql[byte] |= (q & 15) << (0 if quarter < 2 else 4)
        qh[half * 32 + lane] |= (q >> 4) << (2 * quarter)
    block = ql.tobytes() + qh.tobytes() + struct.pack("<16b", *([1] * 16)) + struct.pack("<e", 1.0)
    v = oracle.dequantize(kquant.Q6_K, np.frombuffer(block, np.uint8), 1, 256)[0]
    assert np.array_equal(v, (codes - 32).astype(np.float32))


def test_q4_q5_every_position(oracle):
    codes = (np.arange(256) * 5 + 1) % 32
    for encoding, mask in ((kquant.Q4_K, 15), (kquant.Q5_K, 31)):
        q = codes & mask
        ql = np.zeros(128, np.uint8)
        qh = np.zeros(32, np.uint8)
        for e, code in enumerate(q):
            group, pos = divmod(e, 64)
            high, lane = divmod(pos, 32)
            ql[group * 32 + lane] |= (code & 15) << (4 * high)
            if code > 15:
                qh[lane] |= (2 if high else 1) << (2 * group)
        scales = bytes([1] * 4 + [0] * 4 + [1] * 4)  # all scales 1, all mins 0
        body = (qh.tobytes() if encoding == kquant.Q5_K else b"") + ql.tobytes()
        block = struct.pack("<ee", 1.0, 0.0) + scales + body
        v = oracle.dequantize(encoding, np.frombuffer(block, np.uint8), 1, 256)[0]
        assert np.array_equal(v, q.astype(np.float32))


def test_q8_0_closed_form(oracle):
    # Parity unpinned in the reference (no Q8_0 code there): closed form only.
    q = np.arange(-16, 16, dtype=np.int8)
    block = struct.pack("<e", 0.25) + q.tobytes()
    v = oracle.dequantize(kquant.Q8_0, np.frombuffer(block, np.uint8), 1, 32)[0]
    assert np.array_equal(v, q.astype(np.float32) * 0.25)


@pytest.mark.parametrize("encoding", [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0])
def test_linear_equals_dequantize_then_double_dot(oracle, encoding):
    out_dim, in_dim, rows = 5, 512, 5
    packed = kquant.patterned_bytes(encoding, out_dim, in_dim)
    r = np.arange(rows)[:, None]
    c = np.arange(in_dim)[None, :]
    x = (((r * 37 + c * 13) % 257 - 128) / 257.0).astype(np.float32)
    bias = ((np.arange(out_dim) - 2) / 7.0).astype(np.float32)
    w = oracle.dequantize(encoding, packed, out_dim, in_dim)
    expected = (x.astype(np.float64) @ w.astype(np.float64).T).astype(np.float32)
    y = oracle.linear(encoding, packed, out_dim, in_dim, x)
    # Same double products; numpy's pairwise/BLAS order may differ in the last bit.
    np.testing.assert_allclose(y, expected, rtol=0, atol=1e-6)
    y_written = oracle.linear(encoding, packed, out_dim, in_dim, x, as_written=True)
    assert np.array_equal(y.view(np.uint32), y_written.view(np.uint32))
    y_bias = oracle.linear(encoding, packed, out_dim, in_dim, x, bias=bias)
    assert np.array_equal(y_bias, y + bias[None, :])


def test_linear_sequential_double_order(oracle):
    # Cancellation makes the accumulation order visible: 1e8 + 1 - 1e8 in double
    # keeps the 1 only if the terms are added in column order.
    w = np.zeros((1, 4), np.float32)
    w[0] = [1.0, 1.0, 1.0, 0.0]
    x = np.array([[1e8, 1.0, -1e8, 0.0]], np.float32)
    y = oracle.linear(kquant.F32, w.view(np.uint8).reshape(-1), 1, 4, x)
    assert y[0, 0] == 1.0


def test_q8_1_quantizer_exact_scale(oracle):
    # tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:899-920: codes*2^-5 with a
    # +-127 pair gives scale exactly 1/32 and returns the codes unchanged.
    rows, width = 3, 512
    x = np.zeros((rows, width), np.float32)
    expected = np.zeros((rows, width), np.int32)
    for row in range(rows):
        for block in range(width // 32):
            for lane in range(32):
                code = 0
                if lane == 0:
                    code = -127
                elif lane == 1:
                    code = 127
                elif lane == 2:
                    code = 64 - 2 * (row % 5)
                elif lane >= 4:
                    magnitude = 1 + (block * 11 + (lane // 2) * 7 + row * 3) % 96
                    code = magnitude if lane % 2 == 0 else -magnitude
                expected[row, block * 32 + lane] = code
                x[row, block * 32 + lane] = code * 0.03125
    codes, scales, sums = oracle.quantize_q8_1(x)
    assert np.array_equal(codes.astype(np.int32), expected)
    assert np.all(scales == np.float32(1.0) / (np.float32(127.0) / np.float32(127 * 0.03125)))
    np.testing.assert_allclose(sums, x.reshape(rows, -1, 32).sum(-1), atol=2e-5)


def test_q8_1_zero_block_and_rounding(oracle):
    x = np.zeros((1, 64), np.float32)
    x[0, 32:] = np.linspace(-1, 1, 32, dtype=np.float32)
    codes, scales, sums = oracle.quantize_q8_1(x)
    assert np.all(codes[0, :32] == 0) and scales[0, 0] == 0.0
    inverse = np.float32(127.0) / np.float32(1.0)
    ref = np.clip(np.sign(x[0, 32:]) * np.floor(np.abs(x[0, 32:] * inverse) + 0.5), -127, 127)
    assert np.array_equal(codes[0, 32:], ref.astype(np.int8))  # half away from zero


def test_round_through_fp16(oracle):
    rng = np.random.default_rng(3)
    values = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.integers(-8, 5, 2000),
        np.array([0.0, 65504.0, 65519.9, 65520.0, 1e-8, 6e-8, 2.98e-8, 2.99e-8], np.float32),
    ]).astype(np.float32)
    with np.errstate(over="ignore"):
        expected = values.astype(np.float16).astype(np.float32)
    actual = np.array([oracle.round_through_fp16(float(v)) for v in values], np.float32)
    assert np.array_equal(actual.view(np.uint32), expected.view(np.uint32))


def test_argmax_first_maximum(oracle):
    width = 202048
    values = np.full(width, -9.0, np.float32)
    values[17] = 10.0
    values[123] = 10.0
    assert oracle.argmax(values) == 17
    values[:] = -9.0
    values[-1] = 5.5
    assert oracle.argmax(values) == width - 1
    values[:] = -9.0
    values[0] = -1.0
    assert oracle.argmax(values) == 0


def test_worker_count_follows_reference_cap(oracle):
    # min(count, ceil(count/128), hardware, 32)  (resident_glimmer.cpp:193-196)
    assert oracle.worker_count(100) == 1
    assert oracle.worker_count(129, cap=2) == 2
    assert oracle.worker_count(10**6, cap=64) <= 32


def test_rms_norm_closed_form(oracle):
    # x / sqrt(mean(x^2) + eps) * (w or 1, plus 1 when centered), in double
    # (resident_glimmer.cpp:713-745); one rounding to float per element.
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1536).astype(np.float32)
    w = rng.standard_normal(1536).astype(np.float32)
    inverse = 1.0 / np.sqrt(np.mean(x.astype(np.float64) ** 2) + 1e-6)
    assert np.array_equal(oracle.rms_norm(x, None, False, 1e-6),
                          (x.astype(np.float64) * inverse).astype(np.float32))
    assert np.array_equal(oracle.rms_norm(x, w, False, 1e-6),
                          (x.astype(np.float64) * inverse * w.astype(np.float64)).astype(np.float32))
    assert np.array_equal(
        oracle.rms_norm(x, w, True, 1e-6),
        (x.astype(np.float64) * inverse * (w.astype(np.float64) + 1.0)).astype(np.float32))
    # a constant row normalises to +-1 (eps negligible)
    assert np.allclose(oracle.rms_norm(np.full(512, -3.0, np.float32), None, False, 1e-12), -1.0)


def test_dual_rms_strict_order_and_double_form(oracle):
    # The device order (kernels.cu:2155-2243) restated independently in numpy:
    # 256 strided float partial sums (products are exact in double, each step
    # rounds once like a fused multiply-add), a halving tree, float arithmetic after.
    def inverse_rms(values, eps):
        partials = np.zeros(256, dtype=np.float32)
        for start in range(0, values.size, 256):
            chunk = values[start:start + 256].astype(np.float64)
            lanes = chunk.size
            partials[:lanes] = (chunk * chunk + partials[:lanes].astype(np.float64)).astype(np.float32)
        stride = 128
        while stride:
            partials[:stride] = partials[:stride] + partials[stride:2 * stride]
            stride //= 2
        mean = np.float32(partials[0] / np.float32(values.size))
        return np.float32(1.0) / np.sqrt(np.float32(mean + np.float32(eps)), dtype=np.float32)

    rows, width = 2, 6656
    index = np.arange(rows * width)
    x = (((index % 37) - 18) / 11.0).astype(np.float32).reshape(rows, width)  # probe :222-225
    residual = np.random.default_rng(6).standard_normal((rows, width)).astype(np.float32)
    weight = np.random.default_rng(7).standard_normal(width).astype(np.float32)
    hidden, normalized = oracle.dual_rms_add_capture(x, residual, weight, True, None, False,
                                                     1e-8, 1e-5)
    for row in range(rows):
        first = inverse_rms(x[row], 1e-8)
        expected_hidden = (x[row] * first) * (weight + np.float32(1.0)) + residual[row]
        assert np.array_equal(hidden[row], expected_hidden.astype(np.float32))
        second = inverse_rms(hidden[row], 1e-5)
        assert np.array_equal(normalized[row], hidden[row] * second)
        # the double form of the CPU engine, at the reference probe's tolerance (:243-256)
        reference_hidden = oracle.rms_norm(x[row], weight, True, 1e-8) + residual[row]
        assert np.max(np.abs(hidden[row] - reference_hidden)) <= 2e-5
        assert np.max(np.abs(normalized[row] - oracle.rms_norm(reference_hidden, None, False, 1e-5))) <= 2e-5

