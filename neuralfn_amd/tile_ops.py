"""ctypes binding of libnfn_mi355_tile_ops.so and a small torch-tensor front end.

The descriptor struct and the calling pattern mirror the reference's own ctypes
harness for this ABI (tools/bench_muse_glimmer_packed_linear.py:28-43, 560-640):
device pointers as integers, a 72-byte descriptor per packed matrix, an int
status per call.  torch is used only to own device memory and streams.

There is no CPU fallback: if the library is missing, loading raises.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from pathlib import Path
from typing import Optional, Sequence

from . import kquant

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libnfn_mi355_tile_ops.so"
INVALID = 1

GEMM_F16 = 0
GEMM_INT8 = 1


class PackedWeightDescriptor(ctypes.Structure):
    """NfnNativeTilePackedWeightDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:293-307)."""

    _fields_ = [
        ("struct_size", ctypes.c_uint32),
        ("version", ctypes.c_uint32),
        ("encoding", ctypes.c_uint32),
        ("flags", ctypes.c_uint32),
        ("data", ctypes.c_void_p),
        ("data_nbytes", ctypes.c_int64),
        ("output_dim", ctypes.c_int64),
        ("input_dim", ctypes.c_int64),
        ("row_stride_bytes", ctypes.c_int64),
        ("reserved0", ctypes.c_uint32),
        ("reserved1", ctypes.c_uint32),
        ("cuda_stream", ctypes.c_void_p),
    ]


_P = ctypes.c_void_p
_I64 = ctypes.c_int64
_U32 = ctypes.c_uint32
_F32 = ctypes.c_float


class GqaDecodeDescriptor(ctypes.Structure):
    """NfnNativeTileGlimmerGqaDecodeDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:316-339)."""

    _fields_ = [
        ("struct_size", _U32), ("version", _U32), ("flags", _U32), ("reserved0", _U32),
        ("query", _P), ("current_key", _P), ("current_value", _P),
        ("key_cache_bf16", _P), ("value_cache_bf16", _P), ("output", _P),
        ("query_heads", _I64), ("kv_heads", _I64), ("head_dim", _I64), ("position", _I64),
        ("first_key_position", _I64), ("cache_capacity", _I64), ("cache_row_stride", _I64),
        ("scale", _F32), ("reserved1", _U32), ("cuda_stream", _P),
    ]


class CacheCommitDescriptor(ctypes.Structure):
    """NfnNativeTileGlimmerCacheCommitDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:341-359)."""

    _fields_ = [
        ("struct_size", _U32), ("version", _U32), ("flags", _U32), ("reserved0", _U32),
        ("current_key", _P), ("current_value", _P), ("key_cache_bf16", _P),
        ("value_cache_bf16", _P),
        ("kv_heads", _I64), ("head_dim", _I64), ("position", _I64), ("cache_capacity", _I64),
        ("cache_row_stride", _I64), ("reserved1", _U32), ("reserved2", _U32), ("cuda_stream", _P),
    ]


class BlockAttentionDescriptor(ctypes.Structure):
    """NfnNativeTileDFlashBlockAttentionDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:461-486)."""

    _fields_ = [
        ("struct_size", _U32), ("version", _U32), ("flags", _U32), ("reserved0", _U32),
        ("query", _P), ("block_key", _P), ("block_value", _P),
        ("key_cache_bf16", _P), ("value_cache_bf16", _P), ("output", _P),
        ("query_rows", _I64), ("block_rows", _I64), ("query_heads", _I64), ("kv_heads", _I64),
        ("head_dim", _I64), ("context_length", _I64), ("sliding_window", _I64),
        ("cache_capacity", _I64), ("cache_row_stride", _I64),
        ("scale", _F32), ("reserved1", _U32), ("cuda_stream", _P),
    ]


class FusedDecodeAttentionDescriptor(ctypes.Structure):
    """NfnNativeTileGlimmerFusedDecodeAttentionDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:373-405)."""

    _fields_ = [
        ("struct_size", _U32), ("version", _U32), ("flags", _U32), ("reserved0", _U32),
        ("query", _P), ("key", _P), ("current_value", _P),
        ("key_cache_bf16", _P), ("value_cache_bf16", _P), ("output", _P),
        ("query_norm_weight", PackedWeightDescriptor), ("key_norm_weight", PackedWeightDescriptor),
        ("query_heads", _I64), ("kv_heads", _I64), ("head_dim", _I64), ("position", _I64),
        ("first_key_position", _I64), ("cache_capacity", _I64), ("cache_row_stride", _I64),
        ("norm_eps", _F32), ("query_scale", _F32), ("rope_theta", _F32), ("attention_scale", _F32),
        ("rope_layout", _U32), ("has_query_norm_weight", _U32), ("has_key_norm_weight", _U32),
        ("query_norm_centered", _U32), ("key_norm_centered", _U32), ("apply_rope", _U32),
        ("reserved1", _U32), ("cuda_stream", _P),
    ]


class CacheLayer(ctypes.Structure):
    """NfnNativeTileGlimmerCacheLayerV1 (neuralfn/csrc/native_train/tile_ops.h:416-421)."""

    _fields_ = [("key_cache_bf16", _P), ("value_cache_bf16", _P), ("cache_capacity", _I64),
                ("cache_row_stride", _I64)]


class CacheCommitLayersDescriptor(ctypes.Structure):
    """NfnNativeTileGlimmerCacheCommitLayersDescriptorV1 (neuralfn/csrc/native_train/tile_ops.h:430-453)."""

    _fields_ = [
        ("struct_size", _U32), ("version", _U32), ("flags", _U32), ("reserved0", _U32),
        ("staged_keys", _P), ("staged_values", _P), ("layers", ctypes.POINTER(CacheLayer)),
        ("layer_count", _I64), ("source_rows", _I64), ("rows", _I64), ("kv_heads", _I64),
        ("head_dim", _I64), ("position", _I64), ("source_layer_stride", _I64),
        ("reserved1", _U32), ("reserved2", _U32), ("cuda_stream", _P),
    ]


_DESC = ctypes.POINTER(PackedWeightDescriptor)
_DESC_ARRAY = ctypes.POINTER(_DESC)
_PTR_ARRAY = ctypes.POINTER(ctypes.c_void_p)

#: every symbol include/nfn_mi355_tile_ops.h declares: name -> (restype, argtypes)
SIGNATURES = {
    "nfn_native_tile_ops_abi_version": (ctypes.c_int, []),
    "nfn_native_tile_strict_math_abi_version": (ctypes.c_int, []),
    "nfn_native_tile_packed_weight_abi_version": (ctypes.c_int, []),
    "nfn_native_tile_glimmer_inference_abi_version": (ctypes.c_int, []),
    "nfn_native_tile_k_quant_mmq_abi_version": (ctypes.c_int, []),
    "nfn_mi355_abi_version": (ctypes.c_int, []),
    "nfn_native_tile_ops_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "nfn_native_tile_packed_weight_validate_v1": (ctypes.c_int, [_DESC]),
    "nfn_native_tile_packed_weight_dequantize_float32_v1": (ctypes.c_int, [_DESC, _P]),
    "nfn_native_tile_linear_packed_weight_float32_v1": (
        ctypes.c_int, [_DESC, _P, _P, _P, _I64, ctypes.c_bool]),
    "nfn_native_tile_quantize_q8_1_float32_v1": (ctypes.c_int, [_P, _P, _P, _P, _I64, _I64, _P]),
    "nfn_native_tile_linear_packed_weight_q8_1_float32_v1": (
        ctypes.c_int, [_DESC, _P, _P, _P, _P, _P, _I64, ctypes.c_bool]),
    "nfn_native_tile_linear_packed_weight_q8_1_multi_decode_float32_v1": (
        ctypes.c_int, [_DESC, _DESC, _DESC, _DESC, _P, _P, _P, _P, _P, _P, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmq_workspace_bytes_v1": (_I64, [_I64, _I64]),
    "nfn_native_tile_k_quant_mmq_multi_linear_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmq_multi_linear_gated_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_mi355_k_quant_mmq_multi_linear_prequantized_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmvq_multi_linear_gated_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmvq_multi_linear_swiglu_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, _P]),
    "nfn_native_tile_k_quant_mmvq_linear_float32_v1": (
        ctypes.c_int, [_DESC, _P, _P, _P, _I64, _P]),
    "nfn_native_tile_glimmer_rms_norm_affine_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_rms_norm_affine_capture_residual_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_rms_norm_affine_capture_residual_q8_1_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _P, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_rms_norm_affine_add_residual_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_dual_rms_add_capture_cooperative_batch_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_dual_rms_add_capture_mmvq_q8_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _P, _I64, _P]),
    "nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _P, _I64, _P]),
    "nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _P, _I64, _P]),
    "nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1": (ctypes.c_int, [_DESC, _DESC, _P, _P, _P]),
    "nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1": (
        ctypes.c_int, [_DESC, _DESC, _P, _P, _I64, _P, _I64, _P]),
    "nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1": (
        ctypes.c_int, [_P, _DESC, _P, _P, _DESC, _P, _P, _I64, ctypes.c_float, ctypes.c_bool,
                       ctypes.c_float, ctypes.c_bool, _DESC_ARRAY, _PTR_ARRAY, _I64, _P]),
    "nfn_native_tile_argmax_rows_float32_v1": (ctypes.c_int, [_P, _P, _P, _I64, _I64, _P]),
    "nfn_native_tile_glimmer_sigmoid_gate_float32_v1": (ctypes.c_int, [_P, _P, _P, _I64, _P]),
    "nfn_native_tile_swiglu_float32": (ctypes.c_int, [_P, _P, _P, _I64, _P]),
    "nfn_mi355_lm_head_argmax_workspace_bytes_v1": (_I64, [_I64, _I64]),
    "nfn_mi355_lm_head_argmax_v1": (ctypes.c_int, [_DESC, _P, _P, _P, _I64, _P, _I64, _P]),
    "nfn_mi355_lm_head_argmax_no_alloc_v1": (ctypes.c_int, [_DESC, _P, _P, _P, _I64, _P]),
    "nfn_mi355_k_quant_gemm_workspace_bytes_v1": (_I64, [_I64, _I64, _I64, ctypes.c_int]),
    "nfn_mi355_k_quant_gemm_plan_v1": (
        ctypes.c_int, [ctypes.c_uint32, _I64, _I64, _I64, ctypes.c_int, _P, _P]),
    "nfn_mi355_k_quant_gemm_float32_v1": (
        ctypes.c_int, [_DESC, _P, _P, _I64, _P, _I64, ctypes.c_int, _P]),
    "nfn_mi355_k_quant_gemm_multi_float32_v1": (
        ctypes.c_int, [_DESC_ARRAY, _P, _PTR_ARRAY, _I64, _I64, _P, _I64, ctypes.c_int, _P]),
    "nfn_mi355_gqa_decode_split_workspace_bytes_v1": (_I64, [_I64, _I64]),
    "nfn_mi355_attention_workspace_v1": (ctypes.c_int, [_P, _I64, _P]),
    "nfn_mi355_dflash_block_attention_split_v1": (
        ctypes.c_int, [ctypes.POINTER(BlockAttentionDescriptor), _P, _I64]),
    "nfn_mi355_gqa_decode_split_v1": (ctypes.c_int, [ctypes.POINTER(GqaDecodeDescriptor), _P, _I64]),
    "nfn_mi355_fused_decode_attention_split_v1": (
        ctypes.c_int, [ctypes.POINTER(FusedDecodeAttentionDescriptor), _P, _I64]),
    "nfn_mi355_fused_decode_attention_split_device_position_v1": (
        ctypes.c_int, [ctypes.POINTER(FusedDecodeAttentionDescriptor), _P, _I64, _P, _I64]),
    "nfn_native_tile_glimmer_embedding_gather_float32_v1": (ctypes.c_int, [_DESC, _I64, _P]),
    "nfn_native_tile_glimmer_embedding_gather_device_i64_float32_v1": (ctypes.c_int, [_DESC, _P, _P]),
    "nfn_native_tile_glimmer_embedding_batch_i32_float32_v1": (ctypes.c_int, [_DESC, _P, _P, _I64]),
    "nfn_native_tile_glimmer_positioned_rope_float32_v1": (
        ctypes.c_int, [_P, _P, _I64, _I64, _I64, _I64, _F32, _U32, _P]),
    "nfn_native_tile_glimmer_positioned_rope_batch_float32_v1": (
        ctypes.c_int, [_P, _P, _I64, _I64, _I64, _I64, _I64, _F32, _U32, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_qk_norm_scale_rope_float32_v1": (
        ctypes.c_int, [_P, _P, _DESC, _DESC, _I64, _I64, _I64, _F32, ctypes.c_bool, ctypes.c_bool,
                       _F32, _I64, _F32, _U32, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1": (
        ctypes.c_int, [_P, _P, _DESC, _DESC, _I64, _I64, _I64, _I64, _F32, ctypes.c_bool,
                       ctypes.c_bool, _F32, _I64, _F32, _U32, ctypes.c_bool, _P]),
    "nfn_native_tile_glimmer_fused_decode_attention_float32_v1": (
        ctypes.c_int, [ctypes.POINTER(FusedDecodeAttentionDescriptor)]),
    "nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1": (
        ctypes.c_int, [ctypes.POINTER(FusedDecodeAttentionDescriptor), _P, _I64]),
    "nfn_native_tile_glimmer_cache_commit_layers_bf16_v1": (
        ctypes.c_int, [ctypes.POINTER(CacheCommitLayersDescriptor)]),
    "nfn_native_tile_glimmer_pack_target_taps_float32_v1": (
        ctypes.c_int, [_P, _P, _I64, _I64, _I64, _I64, _I64, _P]),
    "nfn_native_tile_dflash_block_attention_short_split_float32_v1": (
        ctypes.c_int, [ctypes.POINTER(BlockAttentionDescriptor), _P, _I64]),
    "nfn_native_tile_glimmer_gqa_decode_float32_v1": (
        ctypes.c_int, [ctypes.POINTER(GqaDecodeDescriptor)]),
    "nfn_native_tile_glimmer_cache_commit_bf16_v1": (
        ctypes.c_int, [ctypes.POINTER(CacheCommitDescriptor)]),
    "nfn_native_tile_glimmer_cache_commit_rows_bf16_v1": (
        ctypes.c_int, [ctypes.POINTER(CacheCommitDescriptor), _I64]),
    "nfn_native_tile_dflash_block_attention_float32_v1": (
        ctypes.c_int, [ctypes.POINTER(BlockAttentionDescriptor)]),
    "nfn_native_tile_glimmer_logit_transform_float32_v1": (ctypes.c_int, [_P, _I64, _F32, _F32, _P]),
    "nfn_native_tile_add_float32": (ctypes.c_int, [_P, _P, _P, _I64, _P]),
    "nfn_native_tile_scale_inplace_float32": (ctypes.c_int, [_P, _I64, _F32, _P]),
}

_lib: Optional[ctypes.CDLL] = None


def load(path: Optional[Path] = None) -> ctypes.CDLL:
    """dlopen the library and bind every declared symbol; raises if absent."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    target = Path(path) if path is not None else LIB_PATH
    if not target.exists():
        raise RuntimeError(
            f"{target} is not built; run `python -m neuralfn_amd.build` (there is no CPU fallback)")
    lib = ctypes.CDLL(str(target), mode=ctypes.RTLD_LOCAL)
    for name, (restype, argtypes) in SIGNATURES.items():
        function = getattr(lib, name)  # AttributeError if the symbol is missing
        function.restype = restype
        function.argtypes = argtypes
    if path is None:
        _lib = lib
    return lib


class TileOpsError(RuntimeError):
    def __init__(self, operation: str, status: int):
        text = load().nfn_native_tile_ops_error_string(status)
        super().__init__(f"{operation} failed with status {status}: {text.decode() if text else '?'}")
        self.status = status


def check(status: int, operation: str) -> None:
    if status != 0:
        raise TileOpsError(operation, status)


def make_descriptor(encoding: int, data_ptr: int, output_dim: int, input_dim: int,
                    stream: int = 0) -> PackedWeightDescriptor:
    stride = kquant.row_stride_bytes(encoding, input_dim)
    return PackedWeightDescriptor(
        struct_size=ctypes.sizeof(PackedWeightDescriptor), version=1, encoding=encoding, flags=0,
        data=data_ptr, data_nbytes=output_dim * stride, output_dim=output_dim,
        input_dim=input_dim, row_stride_bytes=stride, reserved0=0, reserved1=0,
        cuda_stream=stream or None)


def _stream_handle() -> int:
    import torch
    return int(torch.cuda.current_stream().cuda_stream)


@dataclass
class PackedWeight:
    """A packed [output_dim, input_dim] matrix resident in device memory."""

    encoding: int
    output_dim: int
    input_dim: int
    data: "object"  # torch.uint8 tensor on the GPU, kept alive here

    @classmethod
    def from_numpy(cls, encoding: int, packed, output_dim: int, input_dim: int,
                   device: str = "cuda:0") -> "PackedWeight":
        import torch
        expected = kquant.packed_nbytes(encoding, output_dim, input_dim)
        if packed.size != expected:
            raise ValueError(f"packed tensor has {packed.size} bytes, expected {expected}")
        return cls(encoding, output_dim, input_dim, torch.from_numpy(packed).to(device))

    @property
    def nbytes(self) -> int:
        return int(self.data.numel())

    def descriptor(self, stream: int = 0) -> PackedWeightDescriptor:
        return make_descriptor(self.encoding, self.data.data_ptr(), self.output_dim,
                               self.input_dim, stream)


def _descriptor_array(descriptors: Sequence[PackedWeightDescriptor]):
    array = (_DESC * len(descriptors))()
    for index, descriptor in enumerate(descriptors):
        array[index] = ctypes.pointer(descriptor)
    return array


def _pointer_array(tensors) -> "ctypes.Array":
    array = (ctypes.c_void_p * len(tensors))()
    for index, tensor in enumerate(tensors):
        array[index] = tensor.data_ptr()
    return array


def dequantize(weight: PackedWeight):
    import torch
    out = torch.empty((weight.output_dim, weight.input_dim), dtype=torch.float32,
                      device=weight.data.device)
    descriptor = weight.descriptor(_stream_handle())
    check(load().nfn_native_tile_packed_weight_dequantize_float32_v1(
        ctypes.byref(descriptor), out.data_ptr()), "dequantize")
    return out


def linear(weight: PackedWeight, x, bias=None):
    """nfn_native_tile_linear_packed_weight_float32_v1: any row count."""
    import torch
    rows = x.shape[0]
    out = torch.empty((rows, weight.output_dim), dtype=torch.float32, device=x.device)
    descriptor = weight.descriptor(_stream_handle())
    check(load().nfn_native_tile_linear_packed_weight_float32_v1(
        ctypes.byref(descriptor), x.data_ptr(), bias.data_ptr() if bias is not None else None,
        out.data_ptr(), rows, bias is not None), "linear_packed_weight")
    return out


def small_batch_workspace(rows: int, input_dim: int, device="cuda:0"):
    import torch
    nbytes = load().nfn_native_tile_k_quant_mmq_workspace_bytes_v1(rows, input_dim)
    if nbytes <= 0:
        raise ValueError(f"no small-batch workspace for rows={rows}, input_dim={input_dim}")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


_MULTI = {
    ("mmq", "plain"): "nfn_native_tile_k_quant_mmq_multi_linear_float32_v1",
    ("mmq", "gated"): "nfn_native_tile_k_quant_mmq_multi_linear_gated_float32_v1",
    ("mmq", "swiglu"): "nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1",
    ("mmvq", "plain"): "nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1",
    ("mmvq", "gated"): "nfn_native_tile_k_quant_mmvq_multi_linear_gated_float32_v1",
    ("mmvq", "swiglu"): "nfn_native_tile_k_quant_mmvq_multi_linear_swiglu_float32_v1",
}


def multi_linear(weights: Sequence[PackedWeight], x, workspace, second=None, family: str = "mmq",
                 prologue: str = "plain", outputs=None):
    """1..4 projections of one shared input, rows 1..16.

    prologue "gated": x / (1 + exp(-second));  "swiglu": x is gate, second is up.
    """
    import torch
    rows = x.shape[0]
    stream = _stream_handle()
    if outputs is None:
        outputs = [torch.empty((rows, w.output_dim), dtype=torch.float32, device=x.device)
                   for w in weights]
    descriptors = [w.descriptor(stream) for w in weights]
    function = getattr(load(), _MULTI[(family, prologue)])
    args = [_descriptor_array(descriptors), x.data_ptr()]
    if prologue != "plain":
        args.append(second.data_ptr() if second is not None else None)
    args += [_pointer_array(outputs), len(weights), rows, workspace.data_ptr(),
             workspace.numel(), stream]
    check(function(*args), _MULTI[(family, prologue)])
    return outputs


def multi_linear_prequantized(weights: Sequence[PackedWeight], rows: int, workspace, outputs=None,
                              family: str = "mmvq"):
    """Projections of the input whose quantized form an earlier call left in `workspace`:
    family "mmvq": the activation records of a verifier-family call or of the one-row dual-RMS
    handoff; family "mmq": the fp16 rows of the 5..16-row dual-RMS handoff."""
    import torch
    stream = _stream_handle()
    if outputs is None:
        outputs = [torch.empty((rows, w.output_dim), dtype=torch.float32, device=workspace.device)
                   for w in weights]
    descriptors = [w.descriptor(stream) for w in weights]
    name = ("nfn_native_tile_k_quant_mmvq_multi_linear_prequantized_float32_v1" if family == "mmvq"
            else "nfn_mi355_k_quant_mmq_multi_linear_prequantized_float32_v1")
    check(getattr(load(), name)(
        _descriptor_array(descriptors), _pointer_array(outputs), len(weights), rows,
        workspace.data_ptr(), workspace.numel(), stream), f"{family}_multi_linear_prequantized")
    return outputs


def rms_norm(x, weight: Optional[PackedWeight] = None, centered: bool = False, eps: float = 1e-6,
             residual=None, capture: bool = False, q8: bool = False):
    """rms(x, weight, eps) (+ residual).  Returns a dict: "output", and per request "captured"
    (a copy of x), "codes"/"scales"/"sums" (the public Q8_1 form of the output)."""
    import torch
    rows, width = x.shape
    stream = _stream_handle()
    descriptor = weight.descriptor(stream) if weight is not None else None
    pointer = ctypes.byref(descriptor) if descriptor is not None else None
    result = {"output": torch.empty_like(x)}
    lib = load()
    if residual is not None:
        check(lib.nfn_native_tile_glimmer_rms_norm_affine_add_residual_float32_v1(
            x.data_ptr(), pointer, residual.data_ptr(), result["output"].data_ptr(), rows, width,
            eps, centered, stream), "rms_norm_affine_add_residual")
    elif q8:
        result["captured"] = torch.empty_like(x)
        result["codes"] = torch.empty((rows, width), dtype=torch.int8, device=x.device)
        result["scales"] = torch.empty((rows, width // 32), dtype=torch.float32, device=x.device)
        result["sums"] = torch.empty_like(result["scales"])
        check(lib.nfn_native_tile_glimmer_rms_norm_affine_capture_residual_q8_1_float32_v1(
            x.data_ptr(), pointer, result["output"].data_ptr(), result["captured"].data_ptr(),
            result["codes"].data_ptr(), result["scales"].data_ptr(), result["sums"].data_ptr(),
            rows, width, eps, centered, stream), "rms_norm_affine_capture_residual_q8_1")
    elif capture:
        result["captured"] = torch.empty_like(x)
        check(lib.nfn_native_tile_glimmer_rms_norm_affine_capture_residual_float32_v1(
            x.data_ptr(), pointer, result["output"].data_ptr(), result["captured"].data_ptr(),
            rows, width, eps, centered, stream), "rms_norm_affine_capture_residual")
    else:
        check(lib.nfn_native_tile_glimmer_rms_norm_affine_float32_v1(
            x.data_ptr(), pointer, result["output"].data_ptr(), rows, width, eps, centered,
            stream), "rms_norm_affine")
    return result


def dual_rms_add_capture(x, residual, first_weight: Optional[PackedWeight] = None,
                         first_centered: bool = False,
                         second_weight: Optional[PackedWeight] = None,
                         second_centered: bool = False, first_eps: float = 1e-6,
                         second_eps: float = 1e-6, handoff_workspace=None,
                         handoff_family: str = "mmq"):
    """hidden = residual + rms(x, first); normalized = rms(hidden, second).

    Returns (hidden, normalized, residual_output).  With `handoff_workspace` the quantized form
    of `normalized` is left there for multi_linear_prequantized: one row, family "mmvq";
    5..16 rows, family "mmq" (`handoff_family`), or 4..16 rows, family "mmvq".
    """
    import torch
    rows, width = x.shape
    stream = _stream_handle()
    hidden = torch.empty_like(x)
    normalized = torch.empty_like(x)
    captured = torch.empty_like(x)
    first = first_weight.descriptor(stream) if first_weight is not None else None
    second = second_weight.descriptor(stream) if second_weight is not None else None
    arguments = [x.data_ptr(), ctypes.byref(first) if first is not None else None,
                 residual.data_ptr(), hidden.data_ptr(),
                 ctypes.byref(second) if second is not None else None, normalized.data_ptr(),
                 captured.data_ptr(), rows, width, first_eps, first_centered, second_eps,
                 second_centered]
    if handoff_workspace is None:
        check(load().nfn_native_tile_glimmer_dual_rms_add_capture_float32_v1(*arguments, stream),
              "dual_rms_add_capture")
    elif rows == 1:
        check(load().nfn_native_tile_glimmer_dual_rms_add_capture_mmvq_q8_float32_v1(
            *arguments, handoff_workspace.data_ptr(), handoff_workspace.numel(), stream),
            "dual_rms_add_capture_mmvq_q8")
    elif handoff_family == "mmvq":
        check(load().nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1(
            *arguments, handoff_workspace.data_ptr(), handoff_workspace.numel(), stream),
            "dual_rms_add_capture_mmvq_rows")
    else:
        check(load().nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1(
            *arguments, handoff_workspace.data_ptr(), handoff_workspace.numel(), stream),
            "dual_rms_add_capture_mmq_f16")
    return hidden, normalized, captured


def dual_rms_multi_linear(x, residual, weights: Sequence[PackedWeight],
                          first_weight: Optional[PackedWeight] = None, first_centered: bool = False,
                          second_weight: Optional[PackedWeight] = None,
                          second_centered: bool = False, first_eps: float = 1e-6,
                          second_eps: float = 1e-6, outputs=None):
    """nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1: one row through the two normalisations
    and the projections of their result in one launch.
    Returns (hidden, normalized, residual_output, outputs)."""
    import torch
    stream = _stream_handle()
    width = x.shape[1]
    hidden, normalized, captured = torch.empty_like(x), torch.empty_like(x), torch.empty_like(x)
    if outputs is None:
        outputs = [torch.empty((1, w.output_dim), dtype=torch.float32, device=x.device)
                   for w in weights]
    first = first_weight.descriptor(stream) if first_weight is not None else None
    second = second_weight.descriptor(stream) if second_weight is not None else None
    descriptors = [w.descriptor(stream) for w in weights]
    check(load().nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1(
        x.data_ptr(), ctypes.byref(first) if first is not None else None, residual.data_ptr(),
        hidden.data_ptr(), ctypes.byref(second) if second is not None else None,
        normalized.data_ptr(), captured.data_ptr(), width, first_eps, first_centered, second_eps,
        second_centered, _descriptor_array(descriptors), _pointer_array(outputs), len(weights),
        stream), "dual_rms_mmvq_multi_linear")
    return hidden, normalized, captured, outputs


def dual_rms_multi_linear_supported(weights: Sequence[PackedWeight], width: int) -> bool:
    """Whether dual_rms_multi_linear takes these projections (else: the two calls)."""
    return (1 <= len(weights) <= 4 and width % 256 == 0 and width <= 8192 and
            all(w.encoding == weights[0].encoding and w.input_dim == width for w in weights) and
            weights[0].encoding in (kquant.Q4_K, kquant.Q5_K))


def mmvq_linear(weight: PackedWeight, x, workspace, out=None):
    """nfn_native_tile_k_quant_mmvq_linear_float32_v1: the one-row decode GEMV."""
    import torch
    stream = _stream_handle()
    if out is None:
        out = torch.empty((1, weight.output_dim), dtype=torch.float32, device=x.device)
    descriptor = weight.descriptor(stream)
    check(load().nfn_native_tile_k_quant_mmvq_linear_float32_v1(
        ctypes.byref(descriptor), x.data_ptr(), out.data_ptr(), workspace.data_ptr(),
        workspace.numel(), stream), "mmvq_linear")
    return out


def gate_up_swiglu(gate: PackedWeight, up: PackedWeight, x, out=None):
    """nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1: one token through the gate and up
    projections with the SwiGLU activation at the row ends."""
    import torch
    stream = _stream_handle()
    if out is None:
        out = torch.empty((1, gate.output_dim), dtype=torch.float32, device=x.device)
    gate_descriptor, up_descriptor = gate.descriptor(stream), up.descriptor(stream)
    check(load().nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1(
        ctypes.byref(gate_descriptor), ctypes.byref(up_descriptor), x.data_ptr(), out.data_ptr(),
        stream), "gate_up_swiglu")
    return out


def gate_up_swiglu_supported(gate: PackedWeight, up: PackedWeight) -> bool:
    """Whether gate_up_swiglu takes this pair (else: multi_linear, then the swiglu prologue)."""
    return (gate.encoding == up.encoding and gate.encoding in (kquant.Q4_K, kquant.Q5_K) and
            gate.output_dim == up.output_dim and gate.input_dim == up.input_dim and
            gate.input_dim % 256 == 0 and gate.input_dim <= 8192)


def gate_up_swiglu_rows(gate: PackedWeight, up: PackedWeight, x, rows: int, workspace, out=None):
    """nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1: a block of 5..16 rows through the gate and
    up projections with the SwiGLU activation applied to the pair of results.  x None: the
    workspace holds the rows as dual_rms_add_capture(handoff_workspace=...) left them."""
    import torch
    stream = _stream_handle()
    if out is None:
        out = torch.empty((rows, gate.output_dim), dtype=torch.float32, device=workspace.device)
    gate_descriptor, up_descriptor = gate.descriptor(stream), up.descriptor(stream)
    check(load().nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1(
        ctypes.byref(gate_descriptor), ctypes.byref(up_descriptor),
        None if x is None else x.data_ptr(), out.data_ptr(), rows, workspace.data_ptr(),
        workspace.numel(), stream), "gate_up_swiglu_rows")
    return out


def gate_up_swiglu_rows_supported(gate: PackedWeight, up: PackedWeight, rows: int) -> bool:
    """Whether gate_up_swiglu_rows takes this pair and row count."""
    return (5 <= rows <= 16 and gate.encoding == up.encoding and
            gate.encoding in (kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0) and
            gate.output_dim == up.output_dim and gate.input_dim == up.input_dim and
            gate.input_dim % 256 == 0 and gate.input_dim <= 65536)


def quantize_q8_1(x):
    import torch
    rows, width = x.shape
    codes = torch.empty((rows, width), dtype=torch.int8, device=x.device)
    scales = torch.empty((rows, width // 32), dtype=torch.float32, device=x.device)
    sums = torch.empty_like(scales)
    check(load().nfn_native_tile_quantize_q8_1_float32_v1(
        x.data_ptr(), codes.data_ptr(), scales.data_ptr(), sums.data_ptr(), rows, width,
        _stream_handle()), "quantize_q8_1")
    return codes, scales, sums


def linear_q8_1(weight: PackedWeight, codes, scales, sums, bias=None):
    import torch
    rows = codes.shape[0]
    out = torch.empty((rows, weight.output_dim), dtype=torch.float32, device=codes.device)
    descriptor = weight.descriptor(_stream_handle())
    check(load().nfn_native_tile_linear_packed_weight_q8_1_float32_v1(
        ctypes.byref(descriptor), codes.data_ptr(), scales.data_ptr(), sums.data_ptr(),
        bias.data_ptr() if bias is not None else None, out.data_ptr(), rows, bias is not None),
        "linear_q8_1")
    return out


def linear_q8_1_multi_decode(weights: Sequence[PackedWeight], codes, scales, sums):
    import torch
    stream = _stream_handle()
    outputs = [torch.empty((1, w.output_dim), dtype=torch.float32, device=codes.device)
               for w in weights]
    descriptors = [w.descriptor() for w in weights]
    refs = [ctypes.byref(d) for d in descriptors] + [None] * (4 - len(weights))
    outs = [o.data_ptr() for o in outputs] + [None] * (4 - len(weights))
    check(load().nfn_native_tile_linear_packed_weight_q8_1_multi_decode_float32_v1(
        *refs, codes.data_ptr(), scales.data_ptr(), sums.data_ptr(), *outs, len(weights),
        stream), "q8_1_multi_decode")
    return outputs


def argmax_rows(values, indices=None, maxima=None):
    import torch
    rows, width = values.shape
    if indices is None:
        indices = torch.empty(rows, dtype=torch.int64, device=values.device)
    if maxima is None:
        maxima = torch.empty(rows, dtype=torch.float32, device=values.device)
    check(load().nfn_native_tile_argmax_rows_float32_v1(
        values.data_ptr(), indices.data_ptr(), maxima.data_ptr(), rows, width,
        _stream_handle()), "argmax_rows")
    return indices, maxima


def sigmoid_gate(values, gate):
    import torch
    out = torch.empty_like(values)
    check(load().nfn_native_tile_glimmer_sigmoid_gate_float32_v1(
        values.data_ptr(), gate.data_ptr(), out.data_ptr(), values.numel(), _stream_handle()),
        "sigmoid_gate")
    return out


def swiglu(gate, up):
    import torch
    out = torch.empty_like(gate)
    check(load().nfn_native_tile_swiglu_float32(
        gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), _stream_handle()), "swiglu")
    return out


def lm_head_argmax(weight: PackedWeight, x, workspace=None, indices=None, maxima=None):
    """nfn_mi355_lm_head_argmax_v1: GEMV + argmax, logits never stored."""
    import torch
    rows = x.shape[0]
    stream = _stream_handle()
    if workspace is None:
        nbytes = load().nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, weight.output_dim)
        if nbytes <= 0:
            raise ValueError("lm_head_argmax supports 1..16 rows")
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    if indices is None:
        indices = torch.empty(rows, dtype=torch.int64, device=x.device)
    if maxima is None:
        maxima = torch.empty(rows, dtype=torch.float32, device=x.device)
    descriptor = weight.descriptor(stream)
    check(load().nfn_mi355_lm_head_argmax_v1(
        ctypes.byref(descriptor), x.data_ptr(), indices.data_ptr(), maxima.data_ptr(), rows,
        workspace.data_ptr(), workspace.numel(), stream), "lm_head_argmax")
    return indices, maxima


STATIC_SCRATCH_EXCEEDED = 0x4e46  # NFN_MI355_STATUS_STATIC_SCRATCH_EXCEEDED
LM_HEAD_NO_ALLOC_SCRATCH_BYTES = 1 << 20


def lm_head_argmax_no_alloc(weight: PackedWeight, x, indices, maxima):
    """nfn_mi355_lm_head_argmax_no_alloc_v1: the fused lm_head argmax with the library's own
    scratch; the caller passes inputs and outputs only and nothing is allocated."""
    stream = _stream_handle()
    descriptor = weight.descriptor(stream)
    check(load().nfn_mi355_lm_head_argmax_no_alloc_v1(
        ctypes.byref(descriptor), x.data_ptr(), indices.data_ptr(), maxima.data_ptr(), x.shape[0],
        stream), "lm_head_argmax_no_alloc")
    return indices, maxima


def gemm(weight: PackedWeight, x, mode: int = GEMM_F16, workspace=None, out=None):
    """nfn_mi355_k_quant_gemm_float32_v1: prefill dequant-GEMM, any row count."""
    import torch
    rows = x.shape[0]
    stream = _stream_handle()
    if workspace is None:
        nbytes = load().nfn_mi355_k_quant_gemm_workspace_bytes_v1(
            rows, weight.input_dim, weight.output_dim, mode)
        if nbytes <= 0:
            raise ValueError("unsupported GEMM geometry or mode")
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    if out is None:
        out = torch.empty((rows, weight.output_dim), dtype=torch.float32, device=x.device)
    descriptor = weight.descriptor(stream)
    check(load().nfn_mi355_k_quant_gemm_float32_v1(
        ctypes.byref(descriptor), x.data_ptr(), out.data_ptr(), rows, workspace.data_ptr(),
        workspace.numel(), mode, stream), "k_quant_gemm")
    return out


def gemm_plan(encoding: int, rows: int, input_dim: int, output_dim: int, mode: int = GEMM_F16):
    """nfn_mi355_k_quant_gemm_plan_v1: (rows per workgroup tile, K shares) of a launch."""
    tile_rows, shares = ctypes.c_int(0), ctypes.c_int(0)
    check(load().nfn_mi355_k_quant_gemm_plan_v1(
        encoding, rows, input_dim, output_dim, mode, ctypes.addressof(tile_rows),
        ctypes.addressof(shares)), "k_quant_gemm_plan")
    return tile_rows.value, shares.value


def gemm_multi(weights: Sequence[PackedWeight], x, mode: int = GEMM_F16, workspace=None,
               outputs=None):
    """nfn_mi355_k_quant_gemm_multi_float32_v1: 1..4 projections of one input, converted once."""
    import torch
    rows = x.shape[0]
    stream = _stream_handle()
    if workspace is None:
        nbytes = max(load().nfn_mi355_k_quant_gemm_workspace_bytes_v1(
            rows, w.input_dim, w.output_dim, mode) for w in weights)
        if nbytes <= 0:
            raise ValueError("unsupported GEMM geometry or mode")
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    if outputs is None:
        outputs = [torch.empty((rows, w.output_dim), dtype=torch.float32, device=x.device)
                   for w in weights]
    descriptors = [w.descriptor(stream) for w in weights]
    check(load().nfn_mi355_k_quant_gemm_multi_float32_v1(
        _descriptor_array(descriptors), x.data_ptr(), _pointer_array(outputs), len(weights), rows,
        workspace.data_ptr(), workspace.numel(), mode, stream), "k_quant_gemm_multi")
    return outputs
