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
SIDECAR_REF_LIB = HERE / "_ref" / "libnfn_cpu_sidecar_ref.so"
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
        o.nfo_rope.argtypes = [_P, _I64, _I64, _I64, ctypes.c_double, ctypes.c_int, ctypes.c_int]
        o.nfo_rope.restype = None
        o.nfo_to_bf16.argtypes = [ctypes.c_float]
        o.nfo_to_bf16.restype = ctypes.c_uint16
        o.nfo_block_attention.argtypes = [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I64, _I64,
                                          _I64, _I64, _I64, _I64, ctypes.c_float, ctypes.c_int]
        o.nfo_block_attention.restype = None
        o.nfo_logit_transform.argtypes = [_P, _I64, ctypes.c_double, ctypes.c_double]
        o.nfo_logit_transform.restype = None
        o.nfo_qk_norm.argtypes = [_P, _I64, _I64, _P, ctypes.c_double, ctypes.c_double]
        o.nfo_qk_norm.restype = None
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
        r.nfr_apply_rope.argtypes = [_P, _I64, _I64, _I64, ctypes.c_double, ctypes.c_int]
        r.nfr_apply_rope.restype = ctypes.c_int
        r.nfr_qk_norm.argtypes = [_P, _I64, _I64, _P, ctypes.c_double, ctypes.c_double]
        r.nfr_qk_norm.restype = ctypes.c_int
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


# ---- the decode loop's operators around the packed linears ----------------

def rope(values: np.ndarray, position: int, theta: float, interleaved: bool = False,
         inverse: bool = False) -> np.ndarray:
    """values [heads, head_dim] rotated at `position`; returns a new array."""
    out = np.array(values, dtype=np.float32, order="C", copy=True)
    heads, head_dim = out.shape
    lib().nfo_rope(out.ctypes.data, heads, head_dim, int(position), float(theta), int(interleaved),
                   int(inverse))
    return out


def qk_norm(values: np.ndarray, weight=None, epsilon: float = 1e-5, scalar: float = 1.0):
    """values [heads, head_dim], each head RMS-normalised, times the weight row and `scalar`."""
    out = np.array(values, dtype=np.float32, order="C", copy=True)
    heads, head_dim = out.shape
    _keep, pointer = _optional(weight)
    lib().nfo_qk_norm(out.ctypes.data, heads, head_dim, pointer, float(epsilon), float(scalar))
    return out


def to_bf16(values: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bits (uint16), round to nearest even, vectorised restatement of nfo_to_bf16."""
    bits = np.ascontiguousarray(values, dtype=np.float32).view(np.uint32)
    rounding = np.uint32(0x7FFF) + ((bits >> np.uint32(16)) & np.uint32(1))
    rounded = ((bits + rounding) >> np.uint32(16)).astype(np.uint16)
    nan = (bits & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    return np.where(nan, ((bits >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16), rounded)


def to_bf16_scalar(value: float) -> int:
    return int(lib().nfo_to_bf16(float(value)))


def bf16_to_float(bits: np.ndarray) -> np.ndarray:
    return (np.ascontiguousarray(bits, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(
        np.float32)


def block_attention(query, block_key, block_value, key_cache, value_cache, context_length: int,
                    sliding_window: int, scale: float, causal: bool, cache_row_stride=None):
    """query [rows, query_heads, head_dim]; block_key/value [block_rows, kv_heads, head_dim];
    caches uint16 [capacity, row_stride]."""
    query = np.ascontiguousarray(query, dtype=np.float32)
    block_key = np.ascontiguousarray(block_key, dtype=np.float32)
    block_value = np.ascontiguousarray(block_value, dtype=np.float32)
    key_cache = np.ascontiguousarray(key_cache, dtype=np.uint16)
    value_cache = np.ascontiguousarray(value_cache, dtype=np.uint16)
    rows, query_heads, head_dim = query.shape
    block_rows, kv_heads, _ = block_key.shape
    capacity, stride = key_cache.shape
    out = np.empty_like(query)
    lib().nfo_block_attention(query.ctypes.data, block_key.ctypes.data, block_value.ctypes.data,
                              key_cache.ctypes.data, value_cache.ctypes.data, out.ctypes.data,
                              rows, block_rows, query_heads, kv_heads, head_dim,
                              int(context_length), int(sliding_window), capacity,
                              stride if cache_row_stride is None else cache_row_stride,
                              float(scale), int(causal))
    return out


def gqa_decode(query, current_key, current_value, key_cache, value_cache, position: int,
               first_key_position: int, scale: float):
    """One-token attention: query [query_heads, head_dim], current_key/value [kv_heads, head_dim]."""
    out = block_attention(np.asarray(query)[None], np.asarray(current_key)[None],
                          np.asarray(current_value)[None], key_cache, value_cache, position,
                          position - first_key_position + 1, scale, True)
    return out[0]


def logit_transform(logits: np.ndarray, multiplier: float, softcap: float) -> np.ndarray:
    out = np.array(logits, dtype=np.float32, order="C", copy=True)
    lib().nfo_logit_transform(out.ctypes.data, out.size, float(multiplier), float(softcap))
    return out


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


def ref_qk_norm(values: np.ndarray, weight=None, epsilon: float = 1e-5, scalar: float = 1.0):
    out = np.array(values, dtype=np.float32, order="C", copy=True)
    heads, head_dim = out.shape
    _keep, pointer = _optional(weight)
    status = ref().nfr_qk_norm(out.ctypes.data, heads, head_dim, pointer, float(epsilon),
                               float(scalar))
    if status:
        raise ValueError(f"reference qk_norm status {status}")
    return out


def ref_apply_rope(values: np.ndarray, position: int, theta: float, interleaved: bool = False):
    out = np.array(values, dtype=np.float32, order="C", copy=True)
    heads, head_dim = out.shape
    status = ref().nfr_apply_rope(out.ctypes.data, heads, head_dim, int(position), float(theta),
                                  int(interleaved))
    if status:
        raise ValueError(f"reference apply_rope status {status}")
    return out


# The reference's CPU stand-in for its sidecar (tests/cpp/fake_glimmer_tile_ops.cpp),
# compiled by `make ref`: same C ABI as the GPU library, host pointers.

class GqaDecodeDescriptor(ctypes.Structure):
    _fields_ = [("struct_size", ctypes.c_uint32), ("version", ctypes.c_uint32),
                ("flags", ctypes.c_uint32), ("reserved0", ctypes.c_uint32),
                ("query", _P), ("current_key", _P), ("current_value", _P),
                ("key_cache_bf16", _P), ("value_cache_bf16", _P), ("output", _P),
                ("query_heads", _I64), ("kv_heads", _I64), ("head_dim", _I64),
                ("position", _I64), ("first_key_position", _I64), ("cache_capacity", _I64),
                ("cache_row_stride", _I64), ("scale", ctypes.c_float),
                ("reserved1", ctypes.c_uint32), ("cuda_stream", _P)]


class BlockAttentionDescriptor(ctypes.Structure):
    _fields_ = [("struct_size", ctypes.c_uint32), ("version", ctypes.c_uint32),
                ("flags", ctypes.c_uint32), ("reserved0", ctypes.c_uint32),
                ("query", _P), ("block_key", _P), ("block_value", _P),
                ("key_cache_bf16", _P), ("value_cache_bf16", _P), ("output", _P),
                ("query_rows", _I64), ("block_rows", _I64), ("query_heads", _I64),
                ("kv_heads", _I64), ("head_dim", _I64), ("context_length", _I64),
                ("sliding_window", _I64), ("cache_capacity", _I64), ("cache_row_stride", _I64),
                ("scale", ctypes.c_float), ("reserved1", ctypes.c_uint32), ("cuda_stream", _P)]


_sidecar_ref: Optional[ctypes.CDLL] = None


def sidecar_reference_available() -> bool:
    return SIDECAR_REF_LIB.exists()


def sidecar_ref() -> ctypes.CDLL:
    global _sidecar_ref
    if _sidecar_ref is None:
        s = ctypes.CDLL(str(SIDECAR_REF_LIB), mode=ctypes.RTLD_LOCAL)
        s.nfn_native_tile_glimmer_gqa_decode_float32_v1.argtypes = [_P]
        s.nfn_native_tile_dflash_block_attention_float32_v1.argtypes = [_P]
        s.nfn_native_tile_glimmer_positioned_rope_float32_v1.argtypes = [
            _P, _P, _I64, _I64, _I64, _I64, ctypes.c_float, _U32, _P]
        _sidecar_ref = s
    return _sidecar_ref


def ref_sidecar_block_attention(query, block_key, block_value, key_cache, value_cache,
                                context_length: int, sliding_window: int, scale: float,
                                causal: bool):
    query = np.ascontiguousarray(query, dtype=np.float32)
    block_key = np.ascontiguousarray(block_key, dtype=np.float32)
    block_value = np.ascontiguousarray(block_value, dtype=np.float32)
    key_cache = np.ascontiguousarray(key_cache, dtype=np.uint16)
    value_cache = np.ascontiguousarray(value_cache, dtype=np.uint16)
    out = np.empty_like(query)
    d = BlockAttentionDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.flags = 1 if causal else 0
    d.query, d.block_key, d.block_value = query.ctypes.data, block_key.ctypes.data, block_value.ctypes.data
    d.key_cache_bf16, d.value_cache_bf16, d.output = key_cache.ctypes.data, value_cache.ctypes.data, out.ctypes.data
    d.query_rows, d.query_heads, d.head_dim = query.shape
    d.block_rows, d.kv_heads = block_key.shape[0], block_key.shape[1]
    d.context_length, d.sliding_window = int(context_length), int(sliding_window)
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.scale = float(scale)
    status = sidecar_ref().nfn_native_tile_dflash_block_attention_float32_v1(ctypes.byref(d))
    if status:
        raise ValueError(f"reference sidecar block attention status {status}")
    return out


def ref_sidecar_gqa_decode(query, current_key, current_value, key_cache, value_cache,
                           position: int, first_key_position: int, scale: float):
    query = np.ascontiguousarray(query, dtype=np.float32)
    current_key = np.ascontiguousarray(current_key, dtype=np.float32)
    current_value = np.ascontiguousarray(current_value, dtype=np.float32)
    key_cache = np.ascontiguousarray(key_cache, dtype=np.uint16)
    value_cache = np.ascontiguousarray(value_cache, dtype=np.uint16)
    out = np.empty_like(query)
    d = GqaDecodeDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.query, d.current_key, d.current_value = query.ctypes.data, current_key.ctypes.data, current_value.ctypes.data
    d.key_cache_bf16, d.value_cache_bf16, d.output = key_cache.ctypes.data, value_cache.ctypes.data, out.ctypes.data
    d.query_heads, d.head_dim = query.shape
    d.kv_heads = current_key.shape[0]
    d.position, d.first_key_position = int(position), int(first_key_position)
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.scale = float(scale)
    status = sidecar_ref().nfn_native_tile_glimmer_gqa_decode_float32_v1(ctypes.byref(d))
    if status:
        raise ValueError(f"reference sidecar gqa decode status {status}")
    return out
