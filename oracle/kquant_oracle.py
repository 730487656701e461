"""ctypes front end of the CPU oracle (kquant_oracle.cpp) and of the compiled
reference harness (ref_harness.cpp -> _ref/), numpy in and out.

Test infrastructure only; see the header of kquant_oracle.cpp for which
reference lines each function follows and what pins it.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path
from typing import Optional

import numpy as np

HERE = Path(__file__).resolve().parent
ORACLE_LIB = HERE / "libnfn_kquant_oracle.so"
REF_LIB = HERE / "_ref" / "libnfn_kquant_ref.so"
REFERENCE_ROOT = Path("/root/reference")

_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_U32 = ctypes.c_uint32

_oracle: Optional[ctypes.CDLL] = None
_ref: Optional[ctypes.CDLL] = None


def build(with_reference: bool = True) -> None:
    """Compile the oracle, and the reference harness when the checkout is present."""
    subprocess.run(["make", "-C", str(HERE), "all"], check=True, capture_output=True)
    if with_reference and REFERENCE_ROOT.exists():
        subprocess.run(["make", "-C", str(HERE), "ref"], check=True, capture_output=True)


def lib() -> ctypes.CDLL:
    global _oracle
    if _oracle is None:
        if not ORACLE_LIB.exists():
            build(with_reference=False)
        o = ctypes.CDLL(str(ORACLE_LIB))
        o.nfo_fp16_to_float.argtypes = [ctypes.c_uint16]
        o.nfo_fp16_to_float.restype = ctypes.c_float
        o.nfo_k_scale_min.argtypes = [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_int),
                                      ctypes.POINTER(ctypes.c_int)]
        o.nfo_k_scale_min.restype = None
        o.nfo_worker_count.argtypes = [_I64, _I64, ctypes.c_int]
        o.nfo_worker_count.restype = ctypes.c_int
        o.nfo_dequantize.argtypes = [_U32, _P, _I64, _I64, _P, ctypes.c_int]
        o.nfo_dequantize.restype = ctypes.c_int
        for name in ("nfo_linear", "nfo_linear_as_written"):
            f = getattr(o, name)
            f.argtypes = [_U32, _P, _I64, _I64, _P, _I64, _P, _P, ctypes.c_int, ctypes.c_int]
            f.restype = ctypes.c_int
        o.nfo_argmax.argtypes = [_P, _I64]
        o.nfo_argmax.restype = _I64
        o.nfo_quantize_q8_1.argtypes = [_P, _I64, _I64, _P, _P, _P]
        o.nfo_quantize_q8_1.restype = ctypes.c_int
        o.nfo_round_through_fp16.argtypes = [ctypes.c_float]
        o.nfo_round_through_fp16.restype = ctypes.c_float
        o.nfo_linear_q8_1.argtypes = [_U32, _P, _I64, _I64, _P, _P, _I64, _P, _P]
        o.nfo_linear_q8_1.restype = ctypes.c_int
        o.nfo_sigmoid_gate.argtypes = [_P, _P, _P, _I64]
        o.nfo_sigmoid_gate.restype = None
        o.nfo_swiglu.argtypes = [_P, _P, _P, _I64]
        o.nfo_swiglu.restype = None
        o.nfo_rms_norm.argtypes = [_P, _P, ctypes.c_int, _I64, ctypes.c_double, _P]
        o.nfo_rms_norm.restype = None
        o.nfo_rms_norm_strict.argtypes = [_P, _P, ctypes.c_int, _P, _P, _I64, _I64, ctypes.c_float]
        o.nfo_rms_norm_strict.restype = None
        o.nfo_dual_rms_add_capture.argtypes = [_P, _P, ctypes.c_int, _P, _P, _P, ctypes.c_int, _P,
                                               _I64, _I64, ctypes.c_float, ctypes.c_float]
        o.nfo_dual_rms_add_capture.restype = None
        _oracle = o
    return _oracle


def reference_available() -> bool:
    return REF_LIB.exists()


def ref() -> ctypes.CDLL:
    """The reference engine's own compiled CPU code (built by `make ref`)."""
    global _ref
    if _ref is None:
        r = ctypes.CDLL(str(REF_LIB))
        r.nfr_fp16_to_float.argtypes = [ctypes.c_uint16]
        r.nfr_fp16_to_float.restype = ctypes.c_float
        r.nfr_k_scale_min.argtypes = [_P, ctypes.c_int, ctypes.POINTER(ctypes.c_int),
                                      ctypes.POINTER(ctypes.c_int)]
        r.nfr_k_scale_min.restype = None
        r.nfr_dequantize.argtypes = [_U32, _P, _I64, _I64, _P]
        r.nfr_dequantize.restype = ctypes.c_int
        r.nfr_linear.argtypes = [_U32, _P, _I64, _I64, _P, _I64, _P]
        r.nfr_linear.restype = ctypes.c_int
        r.nfr_rms_norm.argtypes = [_P, _P, ctypes.c_int, _I64, ctypes.c_double, _P]
        r.nfr_rms_norm.restype = ctypes.c_int
        r.nfr_argmax.argtypes = [_P, _I64]
        r.nfr_argmax.restype = _I64
        _ref = r
    return _ref


def _bytes(packed: np.ndarray) -> np.ndarray:
    return np.ascontiguousarray(packed, dtype=np.uint8)


def fp16_to_float(bits: int) -> float:
    return float(lib().nfo_fp16_to_float(bits))


def k_scale_min(scales: bytes, index: int) -> tuple[int, int]:
    buffer = (ctypes.c_uint8 * 12).from_buffer_copy(bytes(scales))
    scale, minimum = ctypes.c_int(), ctypes.c_int()
    lib().nfo_k_scale_min(ctypes.addressof(buffer), index, ctypes.byref(scale),
                          ctypes.byref(minimum))
    return scale.value, minimum.value


def dequantize(encoding: int, packed: np.ndarray, output_dim: int, input_dim: int,
               q6_as_written: bool = False) -> np.ndarray:
    packed = _bytes(packed)
    out = np.empty((output_dim, input_dim), dtype=np.float32)
    status = lib().nfo_dequantize(encoding, packed.ctypes.data, output_dim, input_dim,
                                  out.ctypes.data, int(q6_as_written))
    if status:
        raise ValueError(f"oracle dequantize status {status}")
    return out


def linear(encoding: int, packed: np.ndarray, output_dim: int, input_dim: int, x: np.ndarray,
           bias: Optional[np.ndarray] = None, threads: int = 0, q6_as_written: bool = False,
           as_written: bool = False) -> np.ndarray:
    """y[r, o] = float(sum_c double(x[r, c]) * w(o, c)) (+ bias[o] in float)."""
    packed = _bytes(packed)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, input_dim)
    rows = x.shape[0]
    out = np.empty((rows, output_dim), dtype=np.float32)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
    function = lib().nfo_linear_as_written if as_written else lib().nfo_linear
    status = function(encoding, packed.ctypes.data, output_dim, input_dim, x.ctypes.data, rows,
                      bias.ctypes.data if bias is not None else None, out.ctypes.data, threads,
                      int(q6_as_written))
    if status == 1:
        raise ValueError("oracle linear: bad geometry")
    if status == 2:
        raise FloatingPointError("oracle linear produced a non-finite value")
    return out


def worker_count(count: int, minimum_per_thread: int = 128, cap: int = 0) -> int:
    return int(lib().nfo_worker_count(count, minimum_per_thread, cap))


def argmax(values: np.ndarray) -> int:
    values = np.ascontiguousarray(values, dtype=np.float32)
    return int(lib().nfo_argmax(values.ctypes.data, values.size))


def quantize_q8_1(x: np.ndarray):
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, width = x.shape
    codes = np.empty((rows, width), dtype=np.int8)
    scales = np.empty((rows, width // 32), dtype=np.float32)
    sums = np.empty_like(scales)
    status = lib().nfo_quantize_q8_1(x.ctypes.data, rows, width, codes.ctypes.data,
                                     scales.ctypes.data, sums.ctypes.data)
    if status:
        raise ValueError("oracle quantize_q8_1: bad geometry")
    return codes, scales, sums


def round_through_fp16(value: float) -> float:
    return float(lib().nfo_round_through_fp16(value))


def linear_q8_1(encoding: int, packed: np.ndarray, output_dim: int, input_dim: int,
                codes: np.ndarray, scales: np.ndarray, bias: Optional[np.ndarray] = None):
    packed = _bytes(packed)
    codes = np.ascontiguousarray(codes, dtype=np.int8)
    scales = np.ascontiguousarray(scales, dtype=np.float32)
    rows = codes.shape[0]
    out = np.empty((rows, output_dim), dtype=np.float32)
    if bias is not None:
        bias = np.ascontiguousarray(bias, dtype=np.float32)
    status = lib().nfo_linear_q8_1(encoding, packed.ctypes.data, output_dim, input_dim,
                                   codes.ctypes.data, scales.ctypes.data, rows,
                                   bias.ctypes.data if bias is not None else None,
                                   out.ctypes.data)
    if status:
        raise ValueError("oracle linear_q8_1: bad geometry")
    return out


def sigmoid_gate(values: np.ndarray, gate: np.ndarray) -> np.ndarray:
    values = np.ascontiguousarray(values, dtype=np.float32)
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    out = np.empty_like(values)
    lib().nfo_sigmoid_gate(values.ctypes.data, gate.ctypes.data, out.ctypes.data, values.size)
    return out


def swiglu(gate: np.ndarray, up: np.ndarray) -> np.ndarray:
    gate = np.ascontiguousarray(gate, dtype=np.float32)
    up = np.ascontiguousarray(up, dtype=np.float32)
    out = np.empty_like(gate)
    lib().nfo_swiglu(gate.ctypes.data, up.ctypes.data, out.ctypes.data, gate.size)
    return out


def _optional(values):
    if values is None:
        return None, None
    array = np.ascontiguousarray(values, dtype=np.float32)
    return array, array.ctypes.data


def rms_norm(x: np.ndarray, weight=None, centered: bool = False, epsilon: float = 1e-6) -> np.ndarray:
    """One row through the CPU engine's RMSNorm (double accumulation)."""
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    _keep, pointer = _optional(weight)
    out = np.empty_like(x)
    lib().nfo_rms_norm(x.ctypes.data, pointer, int(centered), x.size, float(epsilon), out.ctypes.data)
    return out


def rms_norm_strict(x: np.ndarray, weight=None, centered: bool = False, eps: float = 1e-6,
                    residual=None) -> np.ndarray:
    """rms(x, weight, eps) (+ residual) in the strict float order of the device kernel."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    rows, width = x.shape
    _weight, weight_pointer = _optional(weight)
    _residual, residual_pointer = _optional(residual)
    out = np.empty_like(x)
    lib().nfo_rms_norm_strict(x.ctypes.data, weight_pointer, int(centered), residual_pointer,
                              out.ctypes.data, rows, width, eps)
    return out


def dual_rms_add_capture(x: np.ndarray, residual: np.ndarray, first_weight=None,
                         first_centered: bool = False, second_weight=None,
                         second_centered: bool = False, first_eps: float = 1e-6,
                         second_eps: float = 1e-6):
    """(hidden, normalized) in the strict float order of the device kernel."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    residual = np.ascontiguousarray(residual, dtype=np.float32)
    rows, width = x.shape
    _first, first_pointer = _optional(first_weight)
    _second, second_pointer = _optional(second_weight)
    hidden = np.empty_like(x)
    normalized = np.empty_like(x)
    lib().nfo_dual_rms_add_capture(x.ctypes.data, first_pointer, int(first_centered),
                                   residual.ctypes.data, hidden.ctypes.data, second_pointer,
                                   int(second_centered), normalized.ctypes.data, rows, width,
                                   first_eps, second_eps)
    return hidden, normalized


# ---- the compiled reference (only where `make ref` has been run) ----------

def ref_rms_norm(x: np.ndarray, weight=None, centered: bool = False, epsilon: float = 1e-6):
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    _keep, pointer = _optional(weight)
    out = np.empty_like(x)
    status = ref().nfr_rms_norm(x.ctypes.data, pointer, int(centered), x.size, float(epsilon),
                                out.ctypes.data)
    if status:
        raise ValueError(f"reference rms_norm status {status}")
    return out


def ref_dequantize(encoding: int, packed: np.ndarray, output_dim: int, input_dim: int):
    packed = _bytes(packed)
    out = np.empty((output_dim, input_dim), dtype=np.float32)
    status = ref().nfr_dequantize(encoding, packed.ctypes.data, output_dim, input_dim,
                                  out.ctypes.data)
    if status:
        raise ValueError(f"reference dequantize status {status}")
    return out


def ref_linear(encoding: int, packed: np.ndarray, output_dim: int, input_dim: int,
               x: np.ndarray) -> np.ndarray:
    packed = _bytes(packed)
    x = np.ascontiguousarray(x, dtype=np.float32).reshape(-1, input_dim)
    out = np.empty((x.shape[0], output_dim), dtype=np.float32)
    status = ref().nfr_linear(encoding, packed.ctypes.data, output_dim, input_dim,
                              x.ctypes.data, x.shape[0], out.ctypes.data)
    if status:
        raise ValueError(f"reference linear status {status}")
    return out
