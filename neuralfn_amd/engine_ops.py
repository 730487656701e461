"""torch-tensor front end of the decode loop's operators around the packed linears.

Embedding, rotary position embedding, one-token and block attention over a bf16
cache, the cache commit, the logit transform, add and scale: the operators the
reference's resident engine requires from its sidecar besides the linears
(neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:431-495).  Everything goes
through the C ABI of libnfn_mi355_tile_ops.so; torch only owns the memory.
"""
from __future__ import annotations

import ctypes

from . import tile_ops
from .tile_ops import (BlockAttentionDescriptor, CacheCommitDescriptor,
                       FusedDecodeAttentionDescriptor, GqaDecodeDescriptor, PackedWeight, check,
                       load)

ROPE_HALF_SPLIT = 0
ROPE_INTERLEAVED = 1
BLOCK_ATTENTION_CAUSAL = 1


def _stream() -> int:
    return tile_ops._stream_handle()


def embedding(table: PackedWeight, tokens):
    """Rows of the table: `tokens` is an int (host), an int64 tensor of one element, or an int32 tensor."""
    import torch
    stream = _stream()
    descriptor = table.descriptor(stream)
    device = table.data.device
    if isinstance(tokens, int):
        out = torch.empty(table.input_dim, dtype=torch.float32, device=device)
        check(load().nfn_native_tile_glimmer_embedding_gather_float32_v1(
            ctypes.byref(descriptor), tokens, out.data_ptr()), "embedding_gather")
        return out
    if tokens.dtype == torch.int64:
        out = torch.empty(table.input_dim, dtype=torch.float32, device=device)
        check(load().nfn_native_tile_glimmer_embedding_gather_device_i64_float32_v1(
            ctypes.byref(descriptor), tokens.data_ptr(), out.data_ptr()),
            "embedding_gather_device_i64")
        return out
    rows = tokens.numel()
    out = torch.empty((rows, table.input_dim), dtype=torch.float32, device=device)
    check(load().nfn_native_tile_glimmer_embedding_batch_i32_float32_v1(
        ctypes.byref(descriptor), tokens.data_ptr(), out.data_ptr(), rows), "embedding_batch_i32")
    return out


def rope(query, key, position: int, theta: float, layout: int = ROPE_HALF_SPLIT,
         inverse: bool = False, batch: bool = False) -> None:
    """In place.  query [rows, query_heads, head_dim] / key [rows, kv_heads, head_dim] with
    `batch`, else [query_heads, head_dim] / [kv_heads, head_dim] at one position."""
    if batch:
        rows, query_heads, head_dim = query.shape
        check(load().nfn_native_tile_glimmer_positioned_rope_batch_float32_v1(
            query.data_ptr(), key.data_ptr(), rows, query_heads, key.shape[1], head_dim,
            position, theta, layout, inverse, _stream()), "positioned_rope_batch")
        return
    query_heads, head_dim = query.shape
    check(load().nfn_native_tile_glimmer_positioned_rope_float32_v1(
        query.data_ptr(), key.data_ptr(), query_heads, key.shape[0], head_dim, position, theta,
        layout, _stream()), "positioned_rope")


def qk_norm_scale_rope(query, key, query_weight=None, key_weight=None, eps: float = 1e-5,
                       query_scale: float = 1.0, position: int = 0, theta: float = 500000.0,
                       layout: int = ROPE_HALF_SPLIT, apply_rope: bool = True,
                       query_centered: bool = False, key_centered: bool = False) -> None:
    """In place: per-head RMS norm, query scale, rope.  query [heads, head_dim] or
    [rows, heads, head_dim] (then key [rows, kv_heads, head_dim], row r at position + r)."""
    stream = _stream()
    q_descriptor = query_weight.descriptor(stream) if query_weight is not None else None
    k_descriptor = key_weight.descriptor(stream) if key_weight is not None else None
    q_pointer = ctypes.byref(q_descriptor) if q_descriptor is not None else None
    k_pointer = ctypes.byref(k_descriptor) if k_descriptor is not None else None
    if query.dim() == 3:
        rows, query_heads, head_dim = query.shape
        check(load().nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1(
            query.data_ptr(), key.data_ptr(), q_pointer, k_pointer, rows, query_heads,
            key.shape[1], head_dim, eps, query_centered, key_centered, query_scale, position,
            theta, layout, apply_rope, stream), "qk_norm_scale_rope_batch")
        return
    query_heads, head_dim = query.shape
    check(load().nfn_native_tile_glimmer_qk_norm_scale_rope_float32_v1(
        query.data_ptr(), key.data_ptr(), q_pointer, k_pointer, query_heads, key.shape[0],
        head_dim, eps, query_centered, key_centered, query_scale, position, theta, layout,
        apply_rope, stream), "qk_norm_scale_rope")


def fused_decode_attention(query, key, value, key_cache, value_cache, position: int,
                           first_key_position: int, attention_scale: float, query_weight=None,
                           key_weight=None, eps: float = 1e-5, query_scale: float = 1.0,
                           theta: float = 500000.0, layout: int = ROPE_HALF_SPLIT,
                           apply_rope: bool = True, out=None, device_position=None,
                           sliding_window: int = 0, workspace=None):
    """qk_norm_scale_rope (in place on query/key), one-token attention, cache commit.

    With `device_position` (an int64 tensor of one element) the kernels read the position when
    they run and `position` / `first_key_position` are ignored; `sliding_window` then bounds a
    local layer's keys.  With `workspace` (gqa_decode_workspace) the attention is the split form."""
    import torch
    if out is None:
        out = torch.empty_like(query)
    stream = _stream()
    d = FusedDecodeAttentionDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.query, d.key, d.current_value = query.data_ptr(), key.data_ptr(), value.data_ptr()
    d.key_cache_bf16, d.value_cache_bf16 = key_cache.data_ptr(), value_cache.data_ptr()
    d.output = out.data_ptr()
    if query_weight is not None:
        d.query_norm_weight = query_weight.descriptor(stream)
        d.has_query_norm_weight = 1
    if key_weight is not None:
        d.key_norm_weight = key_weight.descriptor(stream)
        d.has_key_norm_weight = 1
    d.query_heads, d.head_dim = query.shape
    d.kv_heads = key.shape[0]
    d.position, d.first_key_position = position, first_key_position
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.norm_eps, d.query_scale, d.rope_theta = eps, query_scale, theta
    d.attention_scale = attention_scale
    d.rope_layout = layout
    d.apply_rope = 1 if apply_rope else 0
    d.cuda_stream = stream
    if workspace is not None and device_position is not None:
        check(load().nfn_mi355_fused_decode_attention_split_device_position_v1(
            ctypes.byref(d), device_position.data_ptr(), sliding_window, workspace.data_ptr(),
            workspace.numel()), "fused_decode_attention_split_device_position")
    elif workspace is not None:
        check(load().nfn_mi355_fused_decode_attention_split_v1(
            ctypes.byref(d), workspace.data_ptr(), workspace.numel()), "fused_decode_attention_split")
    elif device_position is not None:
        check(load().nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1(
            ctypes.byref(d), device_position.data_ptr(), sliding_window),
            "fused_decode_attention_device_position")
    else:
        check(load().nfn_native_tile_glimmer_fused_decode_attention_float32_v1(ctypes.byref(d)),
              "fused_decode_attention")
    return out


def lend_attention_workspace(workspace=None, stream=None) -> None:
    """Lends the reference-named attention calls issued on `stream` (a raw handle; default: torch's
    current stream) a split-form workspace (gqa_decode_workspace), or takes that stream's loan
    back with None.  The tensor must outlive the loan."""
    handle = _stream() if stream is None else stream
    if workspace is None:
        check(load().nfn_mi355_attention_workspace_v1(None, 0, handle), "attention_workspace")
    else:
        check(load().nfn_mi355_attention_workspace_v1(workspace.data_ptr(), workspace.numel(), handle),
              "attention_workspace")


def gqa_decode_workspace(query_heads: int, head_dim: int, device="cuda:0"):
    """Workspace of the split form of gqa_decode (nfn_mi355_gqa_decode_split_v1)."""
    import torch
    nbytes = load().nfn_mi355_gqa_decode_split_workspace_bytes_v1(query_heads, head_dim)
    if nbytes <= 0:
        raise ValueError("no split-attention workspace for this geometry")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def gqa_decode(query, current_key, current_value, key_cache, value_cache, position: int,
               first_key_position: int, scale: float, out=None, workspace=None):
    """query [query_heads, head_dim]; current_key/value [kv_heads, head_dim]; caches uint16
    (or bfloat16) [capacity, row_stride].  With `workspace` the split form runs."""
    import torch
    if out is None:
        out = torch.empty_like(query)
    d = GqaDecodeDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.query, d.current_key, d.current_value = (query.data_ptr(), current_key.data_ptr(),
                                               current_value.data_ptr())
    d.key_cache_bf16, d.value_cache_bf16 = key_cache.data_ptr(), value_cache.data_ptr()
    d.output = out.data_ptr()
    d.query_heads, d.head_dim = query.shape
    d.kv_heads = current_key.shape[0]
    d.position, d.first_key_position = position, first_key_position
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.scale = scale
    d.cuda_stream = _stream()
    if workspace is not None:
        check(load().nfn_mi355_gqa_decode_split_v1(ctypes.byref(d), workspace.data_ptr(),
                                                   workspace.numel()), "gqa_decode_split")
    else:
        check(load().nfn_native_tile_glimmer_gqa_decode_float32_v1(ctypes.byref(d)), "gqa_decode")
    return out


def cache_commit(keys, values, key_cache, value_cache, position: int, rows: int = 0) -> None:
    """keys/values [kv_heads, head_dim] (rows == 0) or [rows, kv_heads, head_dim]."""
    d = CacheCommitDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.current_key, d.current_value = keys.data_ptr(), values.data_ptr()
    d.key_cache_bf16, d.value_cache_bf16 = key_cache.data_ptr(), value_cache.data_ptr()
    d.kv_heads, d.head_dim = keys.shape[-2], keys.shape[-1]
    d.position = position
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.cuda_stream = _stream()
    if rows:
        check(load().nfn_native_tile_glimmer_cache_commit_rows_bf16_v1(ctypes.byref(d), rows),
              "cache_commit_rows")
    else:
        check(load().nfn_native_tile_glimmer_cache_commit_bf16_v1(ctypes.byref(d)), "cache_commit")


def block_attention(query, block_key, block_value, key_cache, value_cache, context_length: int,
                    sliding_window: int, scale: float, causal: bool, out=None, workspace=None):
    """query [query_rows, query_heads, head_dim]; block_key/value [block_rows, kv_heads, head_dim].
    With `workspace` (any 16-byte aligned uint8 tensor, e.g. gqa_decode_workspace) the split form."""
    import torch
    if out is None:
        out = torch.empty_like(query)
    d = BlockAttentionDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.flags = BLOCK_ATTENTION_CAUSAL if causal else 0
    d.query, d.block_key, d.block_value = (query.data_ptr(), block_key.data_ptr(),
                                           block_value.data_ptr())
    d.key_cache_bf16, d.value_cache_bf16 = key_cache.data_ptr(), value_cache.data_ptr()
    d.output = out.data_ptr()
    d.query_rows, d.query_heads, d.head_dim = query.shape
    d.block_rows, d.kv_heads = block_key.shape[0], block_key.shape[1]
    d.context_length, d.sliding_window = context_length, sliding_window
    d.cache_capacity, d.cache_row_stride = key_cache.shape
    d.scale = scale
    d.cuda_stream = _stream()
    if workspace is not None:
        check(load().nfn_mi355_dflash_block_attention_split_v1(
            ctypes.byref(d), workspace.data_ptr(), workspace.numel()), "block_attention_split")
    else:
        check(load().nfn_native_tile_dflash_block_attention_float32_v1(ctypes.byref(d)),
              "block_attention")
    return out


def logit_transform(logits, multiplier: float, softcap: float) -> None:
    check(load().nfn_native_tile_glimmer_logit_transform_float32_v1(
        logits.data_ptr(), logits.numel(), multiplier, softcap, _stream()), "logit_transform")


def add(lhs, rhs, out=None):
    import torch
    if out is None:
        out = torch.empty_like(lhs)
    check(load().nfn_native_tile_add_float32(lhs.data_ptr(), rhs.data_ptr(), out.data_ptr(),
                                             lhs.numel(), _stream()), "add")
    return out


def scale_inplace(values, scale: float) -> None:
    check(load().nfn_native_tile_scale_inplace_float32(values.data_ptr(), values.numel(), scale,
                                                       _stream()), "scale_inplace")


def cache_commit_layers(staged_keys, staged_values, caches, rows: int, position: int) -> None:
    """staged_keys/values [layers, source_rows, kv_heads, head_dim]; caches: a (key_cache,
    value_cache) pair per layer.  Rows 0..rows-1 go to positions position .. position+rows-1."""
    layers, source_rows, kv_heads, head_dim = staged_keys.shape
    table = (tile_ops.CacheLayer * layers)()
    for entry, (key_cache, value_cache) in zip(table, caches):
        entry.key_cache_bf16, entry.value_cache_bf16 = key_cache.data_ptr(), value_cache.data_ptr()
        entry.cache_capacity, entry.cache_row_stride = key_cache.shape
    d = tile_ops.CacheCommitLayersDescriptor()
    d.struct_size = ctypes.sizeof(d)
    d.version = 1
    d.staged_keys, d.staged_values = staged_keys.data_ptr(), staged_values.data_ptr()
    d.layers = table
    d.layer_count, d.source_rows, d.rows = layers, source_rows, rows
    d.kv_heads, d.head_dim, d.position = kv_heads, head_dim, position
    d.source_layer_stride = source_rows * kv_heads * head_dim
    d.cuda_stream = _stream()
    check(load().nfn_native_tile_glimmer_cache_commit_layers_bf16_v1(ctypes.byref(d)),
          "cache_commit_layers")


def pack_target_taps(tap_major, source_row_offset: int, rows: int):
    """[taps, source_rows, hidden] -> [rows, taps, hidden]."""
    import torch
    taps, source_rows, hidden = tap_major.shape
    out = torch.empty((rows, taps, hidden), dtype=torch.float32, device=tap_major.device)
    check(load().nfn_native_tile_glimmer_pack_target_taps_float32_v1(
        tap_major.data_ptr(), out.data_ptr(), source_rows, source_row_offset, rows, taps, hidden,
        _stream()), "pack_target_taps")
    return out
