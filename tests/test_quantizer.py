"""The host quantizers produce valid blocks that reconstruct their input to the
accuracy each format allows (they exist to make test and benchmark tensors)."""
import numpy as np
import pytest

from neuralfn_amd import kquant

# relative RMS reconstruction error of N(0, 0.02) weights, generous upper bounds
LIMITS = {kquant.Q4_K: 0.09, kquant.Q5_K: 0.045, kquant.Q6_K: 0.025, kquant.Q8_0: 0.008}


@pytest.mark.parametrize("encoding", sorted(LIMITS))
def test_quantize_roundtrip(oracle, encoding):
    w = kquant.synthetic_weights(5, 16, 1024)
    packed = kquant.quantize(encoding, w)
    assert packed.size == kquant.packed_nbytes(encoding, 16, 1024)
    back = oracle.dequantize(encoding, packed, 16, 1024)
    error = np.sqrt(np.mean((back - w) ** 2)) / np.sqrt(np.mean(w ** 2))
    assert np.isfinite(back).all()
    assert error < LIMITS[encoding], error
    assert error > LIMITS[encoding] / 20  # not a pass-through


def test_quantize_is_deterministic_and_thread_independent():
    w = kquant.synthetic_weights(9, 64, 512)
    a = kquant.quantize(kquant.Q4_K, w, threads=1)
    b = kquant.quantize(kquant.Q4_K, w, threads=4)
    assert np.array_equal(a, b)


def test_zero_rows_quantize_to_zero(oracle):
    w = np.zeros((2, 256), np.float32)
    for encoding in LIMITS:
        back = oracle.dequantize(encoding, kquant.quantize(encoding, w), 2, 256)
        assert not back.any()
