"""Writes tests/golden/reference_linear_vectors.npz from the compiled reference.

Run in a container that has the reference checkout, after `make -C oracle ref`:
    python tests/golden/make_reference_vectors.py
Inputs are seeded random packed bytes (finite scales) and bf16-rounded N(0,1)
activations; outputs are what the reference's own WeightView::value and
linear() (neuralfn/csrc/native_gpt2/resident_glimmer.cpp:542-616, 655-679)
return for them.  Only these vectors travel; the reference does not.
"""
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "tests"))

from neuralfn_amd import kquant  # noqa: E402
from oracle import kquant_oracle  # noqa: E402
from test_oracle_vs_reference import _random_packed  # noqa: E402


def main() -> None:
    out = {}
    for encoding in (kquant.Q4_K, kquant.Q5_K, kquant.Q6_K):
        name = kquant.NAMES[encoding]
        out_dim, in_dim, rows = 8, 512, 2
        packed = _random_packed(encoding, out_dim, in_dim, 1000 + encoding)
        x = kquant.synthetic_activations(2000 + encoding, rows, in_dim)
        out[f"{name}_shape"] = np.array([out_dim, in_dim], np.int64)
        out[f"{name}_packed"] = packed
        out[f"{name}_input"] = x
        out[f"{name}_weights"] = kquant_oracle.ref_dequantize(encoding, packed, out_dim, in_dim)
        out[f"{name}_output"] = kquant_oracle.ref_linear(encoding, packed, out_dim, in_dim, x)
    target = Path(__file__).resolve().parent / "reference_linear_vectors.npz"
    np.savez_compressed(target, **out)
    print(target, target.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
