"""Packed K-Quant formats and synthetic tensors (host side, numpy).

Block layouts are ggml's, as the reference vendors them in
neuralfn/csrc/tile_cuda/vendor/llama_mmq_62bf73d/ggml/src/ggml-common.h:251-368;
encoding ids are those of neuralfn/csrc/native_train/tile_ops.h:11-26 plus 8 for
Q8_0.  The quantizers live in the host library built from
csrc/host/kquant_quantize.cpp.
"""
from __future__ import annotations

import ctypes
from pathlib import Path

import numpy as np

F32 = 0
Q8_0 = 8
Q4_K = 12
Q5_K = 13
Q6_K = 14
BF16 = 30

#: encoding id -> (elements per block, bytes per block)
BLOCKS = {
    F32: (1, 4),
    BF16: (1, 2),
    Q8_0: (32, 34),
    Q4_K: (256, 144),
    Q5_K: (256, 176),
    Q6_K: (256, 210),
}
NAMES = {F32: "f32", BF16: "bf16", Q8_0: "q8_0", Q4_K: "q4_k", Q5_K: "q5_k", Q6_K: "q6_k"}

HOST_LIB = Path(__file__).resolve().parent / "lib" / "libnfn_mi355_kquant_host.so"
_host = None


def row_stride_bytes(encoding: int, input_dim: int) -> int:
    elements, nbytes = BLOCKS[encoding]
    if input_dim % elements:
        raise ValueError(f"input_dim {input_dim} is not a multiple of {elements}")
    return input_dim // elements * nbytes


def packed_nbytes(encoding: int, output_dim: int, input_dim: int) -> int:
    return output_dim * row_stride_bytes(encoding, input_dim)


def _host_lib() -> ctypes.CDLL:
    global _host
    if _host is None:
        if not HOST_LIB.exists():
            raise RuntimeError(
                f"{HOST_LIB} is not built; run `python -m neuralfn_amd.build` first")
        lib = ctypes.CDLL(str(HOST_LIB))
        lib.nfn_mi355_quantize_rows.argtypes = [
            ctypes.c_uint32, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int64, ctypes.c_void_p,
            ctypes.c_int]
        lib.nfn_mi355_quantize_rows.restype = ctypes.c_int
        _host = lib
    return _host


def quantize(encoding: int, weights: np.ndarray, threads: int = 0) -> np.ndarray:
    """Quantize a float32 [output_dim, input_dim] matrix; returns the packed bytes."""
    weights = np.ascontiguousarray(weights, dtype=np.float32)
    rows, cols = weights.shape
    if encoding == F32:
        return weights.view(np.uint8).reshape(-1).copy()
    if encoding == BF16:
        return (round_to_bf16(weights).view(np.uint32) >> 16).astype(np.uint16).view(np.uint8).reshape(-1)
    packed = np.empty(packed_nbytes(encoding, rows, cols), dtype=np.uint8)
    status = _host_lib().nfn_mi355_quantize_rows(
        encoding, weights.ctypes.data, rows, cols, packed.ctypes.data, threads)
    if status != 0:
        raise ValueError(f"cannot quantize {weights.shape} as encoding {encoding}")
    return packed


def round_to_bf16(values: np.ndarray) -> np.ndarray:
    """Round float32 to the nearest-even bfloat16 value, returned as float32."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounded = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return rounded.astype(np.uint32).view(np.float32)


def synthetic_weights(seed: int, output_dim: int, input_dim: int, std: float = 0.02) -> np.ndarray:
    """Float32 N(0, std) weights from a seed (the benchmark's weight recipe)."""
    rng = np.random.Generator(np.random.PCG64(seed))
    return (rng.standard_normal((output_dim, input_dim), dtype=np.float32) * np.float32(std))


def synthetic_activations(seed: int, rows: int, input_dim: int, rms_normalize: bool = False) -> np.ndarray:
    """N(0,1) activations rounded to bf16 and stored as float32."""
    rng = np.random.Generator(np.random.PCG64(seed))
    x = rng.standard_normal((rows, input_dim), dtype=np.float32)
    if rms_normalize:
        x = x / np.sqrt(np.mean(x.astype(np.float64) ** 2, axis=1, keepdims=True)).astype(np.float32)
    return round_to_bf16(x)


def patterned_bytes(encoding: int, output_dim: int, input_dim: int, multiplier: int = 29,
                    offset: int = 17) -> np.ndarray:
    """The reference probe's byte pattern with fixed half-precision scales.

    bytes[i] = (i*multiplier + offset) & 0xff, then per block d = 2**-5 and
    dmin = 2**-6 with small scale bytes (Q4_K/Q5_K) or small signed sub-scales
    (Q6_K): tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:769-797.
    """
    elements, nbytes = BLOCKS[encoding]
    total = packed_nbytes(encoding, output_dim, input_dim)
    index = np.arange(total, dtype=np.uint64)
    packed = ((index * np.uint64(multiplier) + np.uint64(offset)) & np.uint64(0xFF)).astype(np.uint8)
    blocks = packed.reshape(-1, nbytes)
    if encoding in (Q4_K, Q5_K):
        blocks[:, 0] = 0x00
        blocks[:, 1] = 0x28
        blocks[:, 2] = 0x00
        blocks[:, 3] = 0x24
        for scale in range(12):
            blocks[:, 4 + scale] = 1 + (scale % 4)
    elif encoding == Q6_K:
        for scale in range(16):
            blocks[:, 192 + scale] = np.uint8((scale % 9 - 4) & 0xFF)
        blocks[:, 208] = 0x00
        blocks[:, 209] = 0x28
    elif encoding == Q8_0:
        blocks[:, 0] = 0x00
        blocks[:, 1] = 0x28
    return packed
