"""Writes tests/golden/reference_prologue_vectors.npz from the reference's CPU stand-in
for its sidecar (tests/cpp/fake_glimmer_tile_ops.cpp:570 sigmoid gate, :1105 SwiGLU),
compiled by `make -C oracle ref` into oracle/_ref/libnfn_cpu_sidecar_ref.so.

Run in a container that has the reference checkout:
    python tests/golden/make_prologue_vectors.py
Inputs are seeded and asymmetric (values, gates and ups come from different
distributions), so that an operand swap changes the output.  Only these
vectors travel; the reference does not.
"""
import ctypes
import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

from oracle import kquant_oracle  # noqa: E402

TARGET = Path(__file__).resolve().parent / "reference_prologue_vectors.npz"
COUNT = 4096


def inputs():
    rng = np.random.default_rng(20240611)
    values = (rng.standard_normal(COUNT) * 3.0 + 0.5).astype(np.float32)
    gate = (rng.standard_normal(COUNT) * 4.0 - 1.0).astype(np.float32)
    up = rng.uniform(-2.0, 5.0, COUNT).astype(np.float32)
    # the ends of the range: saturated sigmoid on both sides, zero, tiny gates
    gate[:8] = [0.0, -0.0, 1e-30, -1e-30, 30.0, -30.0, 88.0, -88.0]
    return values, gate, up


def reference_outputs(values, gate, up):
    lib = ctypes.CDLL(str(kquant_oracle.SIDECAR_REF_LIB), mode=ctypes.RTLD_LOCAL)
    pointer, i64 = ctypes.c_void_p, ctypes.c_int64
    lib.nfn_native_tile_glimmer_sigmoid_gate_float32_v1.argtypes = [pointer, pointer, pointer, i64, pointer]
    lib.nfn_native_tile_swiglu_float32.argtypes = [pointer, pointer, pointer, i64, pointer]
    gated = np.empty_like(values)
    status = lib.nfn_native_tile_glimmer_sigmoid_gate_float32_v1(
        values.ctypes.data, gate.ctypes.data, gated.ctypes.data, values.size, None)
    assert status == 0
    swiglu = np.empty_like(gate)
    status = lib.nfn_native_tile_swiglu_float32(
        gate.ctypes.data, up.ctypes.data, swiglu.ctypes.data, gate.size, None)
    assert status == 0
    return gated, swiglu


def main() -> None:
    values, gate, up = inputs()
    gated, swiglu = reference_outputs(values, gate, up)
    np.savez_compressed(TARGET, values=values, gate=gate, up=up, sigmoid_gate=gated, swiglu=swiglu)
    print(TARGET, TARGET.stat().st_size, "bytes")


if __name__ == "__main__":
    main()
