"""Pins of the oracle functions that the GPU tests use as the comparand of the fused
prologues and of the public Q8_1 path: nfo_sigmoid_gate, nfo_swiglu, nfo_linear_q8_1.

* sigmoid gate and SwiGLU against the reference's own CPU stand-in for its sidecar
  (tests/cpp/fake_glimmer_tile_ops.cpp:570, :1105) — live where oracle/_ref is built,
  and against the vectors that stand-in wrote (tests/golden/make_prologue_vectors.py)
  everywhere.  The stand-in writes SwiGLU as gate/(1+exp(-gate))*up, the device form
  (glimmer_k_mmq.cu:299-317) as (up*gate)*(1/(1+exp(-gate))): the same value up to
  float rounding of three operations, hence a relative bound of 4 ulp rather than
  bit equality.  The sigmoid gate is the same expression in both and must be bit-equal.
* both also against float64 numpy closed forms, with asymmetric inputs so that
  swapping the operands fails.
* linear_q8_1 against an independent float64 numpy statement
  (round_fp16(scale) * code) @ dequantized.T (kernels.cu:1697-1718: the scale goes
  through fp16 for Q4_K/Q5_K, stays float for Q6_K).
"""
import ctypes
from pathlib import Path

import numpy as np
import pytest

from neuralfn_amd import kquant

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_prologue_vectors.npz"
ULP = float(np.finfo(np.float32).eps)


@pytest.fixture(scope="module")
def golden():
    if not GOLDEN.exists():
        pytest.fail("tests/golden/reference_prologue_vectors.npz is missing")
    return np.load(GOLDEN)


def test_sigmoid_gate_equals_reference_vectors_bit_for_bit(oracle, golden):
    ours = oracle.sigmoid_gate(golden["values"], golden["gate"])
    assert np.array_equal(ours.view(np.uint32), golden["sigmoid_gate"].view(np.uint32))


def test_swiglu_equals_reference_vectors_to_rounding(oracle, golden):
    ours = oracle.swiglu(golden["gate"], golden["up"])
    theirs = golden["swiglu"]
    assert np.all(np.abs(ours - theirs) <= 4 * ULP * np.abs(theirs) + 1e-44)
    # and it is the SwiGLU of (gate, up), not of (up, gate)
    swapped = oracle.swiglu(golden["up"], golden["gate"])
    assert np.max(np.abs(swapped - theirs)) > 0.1


def test_prologues_equal_float64_closed_forms(oracle, golden):
    values, gate, up = (golden[k].astype(np.float64) for k in ("values", "gate", "up"))
    sigmoid = 1.0 / (1.0 + np.exp(-gate))
    gated = oracle.sigmoid_gate(golden["values"], golden["gate"])
    assert np.all(np.abs(gated - values * sigmoid) <= 4 * ULP * np.abs(values * sigmoid) + 1e-44)
    swiglu = oracle.swiglu(golden["gate"], golden["up"])
    assert np.all(np.abs(swiglu - up * gate * sigmoid) <= 4 * ULP * np.abs(up * gate * sigmoid) + 1e-44)
    # swapped operands are a different function on these inputs
    assert np.max(np.abs(oracle.sigmoid_gate(golden["gate"], golden["values"]) - values * sigmoid)) > 0.1


def test_prologues_equal_live_reference_stand_in(oracle, golden):
    if not oracle.sidecar_reference_available():
        pytest.skip("reference CPU sidecar not built (no reference checkout here)")
    lib = ctypes.CDLL(str(oracle.SIDECAR_REF_LIB), mode=ctypes.RTLD_LOCAL)
    pointer, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.nfn_native_tile_glimmer_sigmoid_gate_float32_v1.argtypes = [pointer, pointer, pointer, i64, pointer]
    lib.nfn_native_tile_swiglu_float32.argtypes = [pointer, pointer, pointer, i64, pointer]
    rng = np.random.default_rng(77)
    values = (rng.standard_normal(3000) * 2.0 + 1.0).astype(np.float32)
    gate = (rng.standard_normal(3000) * 5.0).astype(np.float32)
    up = rng.uniform(-1.0, 3.0, 3000).astype(np.float32)
    theirs = np.empty_like(values)
    assert lib.nfn_native_tile_glimmer_sigmoid_gate_float32_v1(
        values.ctypes.data, gate.ctypes.data, theirs.ctypes.data, values.size, None) == 0
    assert np.array_equal(oracle.sigmoid_gate(values, gate).view(np.uint32), theirs.view(np.uint32))
    assert lib.nfn_native_tile_swiglu_float32(
        gate.ctypes.data, up.ctypes.data, theirs.ctypes.data, gate.size, None) == 0
    ours = oracle.swiglu(gate, up)
    assert np.all(np.abs(ours - theirs) <= 4 * ULP * np.abs(theirs) + 1e-44)


@pytest.mark.parametrize("encoding", [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K])
@pytest.mark.parametrize("with_bias", [False, True])
def test_linear_q8_1_equals_independent_float64_statement(oracle, encoding, with_bias):
    out_dim, in_dim, rows = 37, 768, 3
    packed = kquant.quantize(encoding, kquant.synthetic_weights(300 + encoding, out_dim, in_dim))
    rng = np.random.default_rng(9 + encoding)
    # activations of very different magnitude per row, so that a scale indexed by the
    # wrong row or group shows; scales that fp16 rounding changes
    x = (rng.standard_normal((rows, in_dim)) * np.array([[0.03], [1.0], [40.0]])).astype(np.float32)
    codes, scales, _sums = oracle.quantize_q8_1(x)
    bias = rng.standard_normal(out_dim).astype(np.float32) if with_bias else None
    ours = oracle.linear_q8_1(encoding, packed, out_dim, in_dim, codes, scales, bias)

    weights = oracle.dequantize(encoding, packed, out_dim, in_dim).astype(np.float64)
    used = scales.astype(np.float16).astype(np.float32) if encoding != kquant.Q6_K else scales
    assert encoding == kquant.Q6_K or not np.array_equal(used, scales)  # the rounding is not a no-op here
    # the activation the int8 path sees: one float product per element, then float64 from there on
    activation = (np.repeat(used, 32, axis=1) * codes.astype(np.float32)).astype(np.float32)
    expected = activation.astype(np.float64) @ weights.T
    if with_bias:
        expected = expected + bias.astype(np.float64)
    scale = np.max(np.abs(expected))
    assert np.max(np.abs(ours - expected)) <= 2e-7 * scale
    # what the pin excludes: the unrounded scale (Q4_K/Q5_K), or codes used without their scale
    if encoding != kquant.Q6_K:
        unrounded = (np.repeat(scales, 32, axis=1) * codes).astype(np.float64) @ weights.T
        if with_bias:
            unrounded = unrounded + bias
        assert np.max(np.abs(ours - unrounded)) > 1e-5 * scale


def test_round_through_fp16_equals_numpy(oracle):
    rng = np.random.default_rng(3)
    samples = np.concatenate([
        rng.standard_normal(2000).astype(np.float32) * 10.0 ** rng.integers(-9, 5, 2000),
        np.array([0.0, -0.0, 65504.0, 65519.0, 6e-8, 5.96e-8, 2.98e-8, 1e-10, -3.1e-5], np.float32),
    ]).astype(np.float32)
    samples = samples[np.abs(samples) < 65520.0]
    for value in samples:
        assert np.float32(oracle.round_through_fp16(float(value))).view(np.uint32) == \
            np.float32(np.float16(value)).view(np.uint32), value
