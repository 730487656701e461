"""The oracle against the reference engine's own compiled CPU code.

`make -C oracle ref` compiles the reference's resident_glimmer*.cpp where they
lie and exposes WeightView::value and linear() (oracle/ref_harness.cpp).  That
library exists only where the reference checkout does; elsewhere these tests
fall back to the committed vectors under tests/golden/, which
tests/golden/make_reference_vectors.py wrote from that same library.
"""
from pathlib import Path

import numpy as np
import pytest

from neuralfn_amd import kquant

GOLDEN = Path(__file__).resolve().parent / "golden" / "reference_linear_vectors.npz"
ENCODINGS = [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K]


def _random_packed(encoding, out_dim, in_dim, seed):
    """Random bytes with finite half-precision scales (every bit pattern of the
    quant fields is exercised; scale fields keep their exponent small)."""
    rng = np.random.default_rng(seed)
    _, nbytes = kquant.BLOCKS[encoding]
    blocks = rng.integers(0, 256, (out_dim * in_dim // 256, nbytes), dtype=np.uint8)
    d_offsets = (0, 2) if encoding in (kquant.Q4_K, kquant.Q5_K) else (208,)
    for offset in d_offsets:
        blocks[:, offset + 1] = (blocks[:, offset + 1] & 0x83) | 0x24  # exponent 9..12
    return blocks.reshape(-1)


needs_ref = pytest.mark.skipif(
    not __import__("oracle.kquant_oracle", fromlist=["x"]).reference_available(),
    reason="reference harness not built (no reference checkout here)")


@needs_ref
def test_fp16_and_scale_min_match_reference(oracle):
    r = oracle.ref()
    for bits in range(0, 65536, 7):
        a = oracle.fp16_to_float(bits)
        b = float(r.nfr_fp16_to_float(bits))
        assert (np.isnan(a) and np.isnan(b)) or np.float32(a).view(np.uint32) == np.float32(b).view(np.uint32)


@needs_ref
@pytest.mark.parametrize("encoding", ENCODINGS)
def test_dequantize_matches_reference_bit_for_bit(oracle, encoding):
    out_dim, in_dim = 6, 1024
    packed = _random_packed(encoding, out_dim, in_dim, 11 + encoding)
    reference = oracle.ref_dequantize(encoding, packed, out_dim, in_dim)
    as_written = oracle.dequantize(encoding, packed, out_dim, in_dim, q6_as_written=True)
    assert np.array_equal(as_written.view(np.uint32), reference.view(np.uint32))
    canonical = oracle.dequantize(encoding, packed, out_dim, in_dim)
    if encoding == kquant.Q6_K:
        # The reference CPU engine's Q6_K differs from the canonical layout in
        # elements 16..31 of every 32 (resident_glimmer.cpp:614), nowhere else.
        differs = (canonical != reference).reshape(out_dim, -1, 32)
        assert not differs[:, :, :16].any()
        assert differs[:, :, 16:].any()
    else:
        assert np.array_equal(canonical.view(np.uint32), reference.view(np.uint32))


@needs_ref
@pytest.mark.parametrize("encoding", ENCODINGS)
def test_linear_matches_reference_bit_for_bit(oracle, encoding):
    out_dim, in_dim, rows = 160, 512, 3  # >128 rows so the reference goes multi-threaded
    packed = _random_packed(encoding, out_dim, in_dim, 5 + encoding)
    x = kquant.synthetic_activations(99, rows, in_dim)
    reference = oracle.ref_linear(encoding, packed, out_dim, in_dim, x)
    for as_written in (False, True):
        y = oracle.linear(encoding, packed, out_dim, in_dim, x, q6_as_written=True,
                          as_written=as_written)
        assert np.array_equal(y.view(np.uint32), reference.view(np.uint32))


@pytest.mark.parametrize("encoding", ENCODINGS)
def test_linear_matches_committed_reference_vectors(oracle, encoding):
    if not GOLDEN.exists():
        pytest.fail("tests/golden/reference_linear_vectors.npz is missing")
    data = np.load(GOLDEN)
    name = kquant.NAMES[encoding]
    packed, x = data[f"{name}_packed"], data[f"{name}_input"]
    out_dim, in_dim = int(data[f"{name}_shape"][0]), int(data[f"{name}_shape"][1])
    y = oracle.linear(encoding, packed, out_dim, in_dim, x, q6_as_written=True)
    assert np.array_equal(y.view(np.uint32), data[f"{name}_output"].view(np.uint32))
    w = oracle.dequantize(encoding, packed, out_dim, in_dim, q6_as_written=True)
    assert np.array_equal(w.view(np.uint32), data[f"{name}_weights"].view(np.uint32))


@needs_ref
@pytest.mark.parametrize("centered", [False, True])
def test_rms_norm_matches_reference_bit_for_bit(oracle, centered):
    rng = np.random.default_rng(21)
    x = rng.standard_normal(6656).astype(np.float32)
    weight = rng.standard_normal(6656).astype(np.float32)
    assert np.array_equal(oracle.rms_norm(x, weight, centered, 1e-6),
                          oracle.ref_rms_norm(x, weight, centered, 1e-6))
    assert np.array_equal(oracle.rms_norm(x, None, False, 1e-8),
                          oracle.ref_rms_norm(x, None, False, 1e-8))

