"""One decode step of one transformer layer as the reference's resident engine sequences it,
every operator through the C ABI of libnfn_mi355_tile_ops.so.

The arithmetic of a layer is the CPU engine's
(neuralfn/csrc/native_gpt2/resident_glimmer.cpp:1719-1830): input norm; Q, K, V and attention-gate
projections; per-head Q/K norm; rope; attention over the bf16 cache; sigmoid gate; output
projection; post-attention norm + residual; pre-feed-forward norm; gate/up projections; SwiGLU;
down projection; post-feed-forward norm + residual.  The grouping into calls is the device
engine's: one grouped small-batch call per shared input, the sigmoid gate and SwiGLU as prologues
of the projection that consumes them, two adjacent norms in one dual-RMS call
(neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:2233-2585, 2913-2960), and the Q/K norms,
rope, attention and cache commit in its fused decode-attention call (two launches here).
Eight launches per layer and token.

This is host-side sequencing for tests and benchmarks, not an engine: no sampling, no prompt
handling, one token per step.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional

from . import engine_ops, tile_ops
from .tile_ops import PackedWeight


@dataclass
class LayerGeometry:
    model_dim: int
    query_heads: int
    kv_heads: int
    head_dim: int
    ffn_dim: int
    sliding_window: int      # keys a local layer attends to, cache capacity of the layer
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    post_norm_eps: float = 1e-5
    interleaved_rope: bool = True  # the GGUF container's layout (resident_glimmer.cpp:1736-1743)

    @property
    def attention_dim(self) -> int:
        return self.query_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.kv_heads * self.head_dim


@dataclass
class LayerWeights:
    """Packed projections and float norm rows (PackedWeight with encoding F32 or BF16, [1, width])."""
    q: PackedWeight
    k: PackedWeight
    v: PackedWeight
    attention_gate: PackedWeight
    output: PackedWeight
    mlp_gate: PackedWeight
    mlp_up: PackedWeight
    mlp_down: PackedWeight
    input_norm: Optional[PackedWeight] = None
    q_norm: Optional[PackedWeight] = None
    k_norm: Optional[PackedWeight] = None
    post_attention_norm: Optional[PackedWeight] = None
    pre_feedforward_norm: Optional[PackedWeight] = None
    post_feedforward_norm: Optional[PackedWeight] = None

    def packed_bytes(self) -> int:
        return sum(w.nbytes for w in (self.q, self.k, self.v, self.attention_gate, self.output,
                                      self.mlp_gate, self.mlp_up, self.mlp_down))


class LayerCache:
    """bf16 key/value ring of one layer: [capacity, kv_heads * head_dim] each."""

    def __init__(self, geometry: LayerGeometry, device):
        import torch
        shape = (geometry.sliding_window, geometry.kv_dim)
        self.keys = torch.zeros(shape, dtype=torch.int16, device=device)
        self.values = torch.zeros(shape, dtype=torch.int16, device=device)


def decode_layer(geometry: LayerGeometry, weights: LayerWeights, cache: LayerCache, pending, residual,
                 pending_norm: Optional[PackedWeight], position: int, workspace, local: bool = True,
                 attention_workspace=None, fused_gate_up: bool = False,
                 fused_input_norm: bool = False):
    """One token through one layer.

    `pending` is the previous layer's down-projection output whose post-feed-forward norm and
    residual add are still owed (for the first layer: the embedding row with `pending_norm` None
    and `residual` zeros gives hidden = rms(embedding), the engine's embedding norm,
    resident_glimmer.cpp:1700-1701).  Returns (down, hidden): this layer's owed pair.
    `attention_workspace` (engine_ops.gqa_decode_workspace) selects the split attention form.
    `fused_gate_up`: the gate and up projections in one call with the SwiGLU activation at the
    row ends (nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1) where the pair allows it, so
    that the down projection reads one plain vector; the same bits as the separate calls.
    `fused_input_norm`: the first dual norm inside the launch of the projections it feeds
    (nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1) where those allow it; the same bits.
    """
    g = geometry
    # hidden = residual + rms(pending); normalized = rms(hidden, input_norm)
    first_eps = g.post_norm_eps if pending_norm is not None else g.norm_eps
    attention_inputs = [weights.q, weights.k, weights.v, weights.attention_gate]
    if fused_input_norm and tile_ops.dual_rms_multi_linear_supported(attention_inputs, g.model_dim):
        hidden, normalized, _, (query, key, value, gate) = tile_ops.dual_rms_multi_linear(
            pending, residual, attention_inputs, pending_norm, False, weights.input_norm, False,
            first_eps, g.norm_eps)
    else:
        hidden, normalized, _ = tile_ops.dual_rms_add_capture(
            pending, residual, pending_norm, False, weights.input_norm, False, first_eps, g.norm_eps)
        query, key, value, gate = tile_ops.multi_linear(attention_inputs, normalized, workspace)
    # per-head norms and rope in one launch, attention, the cache commit
    query = query.view(g.query_heads, g.head_dim)
    key = key.view(g.kv_heads, g.head_dim)
    value = value.view(g.kv_heads, g.head_dim)
    first = max(0, position - g.sliding_window + 1) if local else 0
    layout = engine_ops.ROPE_INTERLEAVED if g.interleaved_rope else engine_ops.ROPE_HALF_SPLIT
    # the reference's fused call (one workgroup per query head), or with a workspace this
    # library's split form of it (the keys of a head over several workgroups)
    attention = engine_ops.fused_decode_attention(
        query, key, value, cache.keys, cache.values, position, first, g.head_dim ** -0.5,
        weights.q_norm, weights.k_norm, g.norm_eps, 1.0, g.rope_theta, layout, local,
        workspace=attention_workspace)
    # output projection of attention * sigmoid(gate), the gate as the call's prologue
    (projected,) = tile_ops.multi_linear([weights.output], attention.view(1, g.attention_dim),
                                         workspace, second=gate, prologue="gated")
    hidden, normalized, _ = tile_ops.dual_rms_add_capture(
        projected, hidden, weights.post_attention_norm, False, weights.pre_feedforward_norm, False,
        g.post_norm_eps, g.norm_eps)
    if fused_gate_up and tile_ops.gate_up_swiglu_supported(weights.mlp_gate, weights.mlp_up):
        activated = tile_ops.gate_up_swiglu(weights.mlp_gate, weights.mlp_up, normalized)
        (down,) = tile_ops.multi_linear([weights.mlp_down], activated, workspace)
        return down, hidden
    mlp_gate, mlp_up = tile_ops.multi_linear([weights.mlp_gate, weights.mlp_up], normalized,
                                             workspace)
    (down,) = tile_ops.multi_linear([weights.mlp_down], mlp_gate, workspace, second=mlp_up,
                                    prologue="swiglu")
    return down, hidden


def verify_layer(geometry: LayerGeometry, weights: LayerWeights, cache: LayerCache, pending, residual,
                 pending_norm: Optional[PackedWeight], position: int, workspace, local: bool = True,
                 attention_workspace=None, handoff: bool = False, fused_gate_up: bool = False,
                 family: str = "mmq"):
    """A block of tokens (rows of `pending`, at positions position, position + 1, ...) through
    one layer the way the verifier runs it (resident_glimmer_cuda.cpp:2913-2960, 3437-3520): the
    same operators in their batch forms, a causal block attention over the cache and the
    block's own rows, and no cache commit -- the block's key/value rows are returned for the
    commit of the accepted ones (cache_commit, cache_commit_layers).  Row r equals decode_layer
    at position + r after the commits of the rows before it, to rounding.

    handoff (5..16 rows, a model width of at most 8,192): the two dual norms also leave their
    output in `workspace` in the form the projections would convert it to
    (nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1) and the projections behind them
    multiply from it; the same bits, two launches less.

    fused_gate_up (5..16 rows): gate and up in one call that stores swiglu(gate, up)
    (nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1) where the pair allows it; the down
    projection then reads that one block of rows plainly; the same bits.

    family "mmvq": every projection through the exact verifier's entry points
    (nfn_native_tile_k_quant_mmvq_multi_linear*_float32_v1), as the engine's speculative decode
    calls them with exact_verifier_rows (resident_glimmer.cpp:2662-2666,
    resident_glimmer_cuda.cpp:3526-3532): row r then equals decode_layer's projections bit for
    bit.  With handoff (4..16 rows) the norms leave the rows' activation records and their
    matrix-operand copy (nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1) for the reference's
    prequantized consumer; the gate/up pair call belongs to the other family.

    Returns (down, hidden, key_rows, value_rows).
    """
    g = geometry
    rows = pending.shape[0]
    if family == "mmvq" and fused_gate_up:
        raise ValueError("the gate/up pair call is a form of the mmq family")
    hidden, normalized, _ = tile_ops.dual_rms_add_capture(
        pending, residual, pending_norm, False, weights.input_norm, False,
        g.post_norm_eps if pending_norm is not None else g.norm_eps, g.norm_eps,
        handoff_workspace=workspace if handoff else None, handoff_family=family)
    attention_inputs = [weights.q, weights.k, weights.v, weights.attention_gate]
    if handoff:
        query, key, value, gate = tile_ops.multi_linear_prequantized(
            attention_inputs, rows, workspace, family=family)
    else:
        query, key, value, gate = tile_ops.multi_linear(attention_inputs, normalized, workspace,
                                                        family=family)
    query = query.view(rows, g.query_heads, g.head_dim)
    key = key.view(rows, g.kv_heads, g.head_dim)
    value = value.view(rows, g.kv_heads, g.head_dim)
    layout = engine_ops.ROPE_INTERLEAVED if g.interleaved_rope else engine_ops.ROPE_HALF_SPLIT
    engine_ops.qk_norm_scale_rope(query, key, weights.q_norm, weights.k_norm, g.norm_eps, 1.0,
                                  position, g.rope_theta, layout, local)
    # a local layer's row sees its last sliding_window keys, a global one everything
    window = g.sliding_window if local else position + rows
    attention = engine_ops.block_attention(query, key, value, cache.keys, cache.values, position,
                                           window, g.head_dim ** -0.5, True,
                                           workspace=attention_workspace)
    (projected,) = tile_ops.multi_linear([weights.output], attention.view(rows, g.attention_dim),
                                         workspace, second=gate, family=family, prologue="gated")
    hidden, normalized, _ = tile_ops.dual_rms_add_capture(
        projected, hidden, weights.post_attention_norm, False, weights.pre_feedforward_norm, False,
        g.post_norm_eps, g.norm_eps, handoff_workspace=workspace if handoff else None,
        handoff_family=family)
    if fused_gate_up and tile_ops.gate_up_swiglu_rows_supported(weights.mlp_gate, weights.mlp_up, rows):
        activated = tile_ops.gate_up_swiglu_rows(weights.mlp_gate, weights.mlp_up,
                                                 None if handoff else normalized, rows, workspace)
        (down,) = tile_ops.multi_linear([weights.mlp_down], activated, workspace)
        return down, hidden, key, value
    if handoff:
        mlp_gate, mlp_up = tile_ops.multi_linear_prequantized(
            [weights.mlp_gate, weights.mlp_up], rows, workspace, family=family)
    else:
        mlp_gate, mlp_up = tile_ops.multi_linear([weights.mlp_gate, weights.mlp_up], normalized,
                                                 workspace, family=family)
    (down,) = tile_ops.multi_linear([weights.mlp_down], mlp_gate, workspace, second=mlp_up,
                                    family=family, prologue="swiglu")
    return down, hidden, key, value


LAUNCHES_PER_LAYER = 8           # with the reference's fused attention call
LAUNCHES_PER_LAYER_SPLIT = 9     # with the split attention form (one more: the merge)
LAUNCHES_PER_LAYER_FUSED = 8     # ... and the first dual norm inside the Q/K/V/gate launch
