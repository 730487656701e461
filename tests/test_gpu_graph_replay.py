"""The entry points under HIP graph capture: the engine replays its decode step from a graph
(resident_glimmer_cuda.cpp:2705-2760), and so does bench.py.  A captured sequence of calls is
replayed several times, with new inputs, eager work and synchronisations between the replays,
and every replay must give the bits of the same calls made eagerly on the same inputs: nothing
may depend on state that only the first execution sets up (no memset nodes, no host-side
decisions baked into the capture, outputs that a kernel adds onto refilled on every replay).
"""
import numpy as np
import pytest

from neuralfn_amd import kquant, tile_ops

pytestmark = pytest.mark.gpu


def random_packed(encoding, out_dim, in_dim, seed):
    rng = np.random.default_rng(seed)
    elements, nbytes = kquant.BLOCKS[encoding]
    blocks = rng.integers(0, 256, (out_dim * in_dim // elements, nbytes), dtype=np.uint8)
    offsets = {kquant.Q4_K: (0, 2), kquant.Q5_K: (0, 2), kquant.Q6_K: (208,), kquant.Q8_0: (0,)}
    for offset in offsets[encoding]:
        blocks[:, offset + 1] = (blocks[:, offset + 1] & 0x83) | 0x24
    return blocks.reshape(-1)


def test_small_batch_calls_replayed_from_a_graph(cuda):
    import torch
    in_dim, rows = 2304, 16
    specs = [(kquant.Q4_K, 2048), (kquant.Q6_K, 70), (kquant.Q8_0, 33), (kquant.Q5_K, 300)]
    weights = [tile_ops.PackedWeight.from_numpy(e, random_packed(e, n, in_dim, 11 + i), n, in_dim)
               for i, (e, n) in enumerate(specs)]
    lm_head = tile_ops.PackedWeight.from_numpy(kquant.Q6_K, random_packed(kquant.Q6_K, 5003, in_dim, 19),
                                               5003, in_dim)
    scale = tile_ops.PackedWeight.from_numpy(
        kquant.F32, kquant.quantize(kquant.F32, np.linspace(0.5, 1.5, in_dim, dtype=np.float32)[None, :]),
        1, in_dim)
    x = torch.empty((rows, in_dim), dtype=torch.float32, device=cuda)
    gate = torch.empty_like(x)
    block_workspace = tile_ops.small_batch_workspace(rows, in_dim)
    one_workspace = tile_ops.small_batch_workspace(1, in_dim)
    lm_workspace = torch.empty(tile_ops.load().nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, 5003),
                               dtype=torch.uint8, device=cuda)

    def sequence():
        results = []
        # one token: the decode call and its norm handoff
        results += tile_ops.multi_linear(weights, x[:1], one_workspace)
        hidden, normalized, _ = tile_ops.dual_rms_add_capture(
            x[:1], gate[:1], scale, False, scale, False, 1e-6, 1e-6, handoff_workspace=one_workspace)
        results += [hidden, normalized]
        results += tile_ops.multi_linear_prequantized(weights, 1, one_workspace, family="mmvq")
        # a block of 16: both families, a fused prologue, the exact family's split form
        # (2,048 rows of Q4_K are 64 tiles) and its handoff with a prequantized consumer
        results += tile_ops.multi_linear(weights, x, block_workspace, family="mmq")
        results += tile_ops.multi_linear(weights, x, block_workspace, second=gate, family="mmvq",
                                         prologue="gated")
        hidden, normalized, _ = tile_ops.dual_rms_add_capture(
            x, gate, scale, False, scale, False, 1e-6, 1e-6, handoff_workspace=block_workspace,
            handoff_family="mmvq")
        results += [hidden, normalized]
        results += tile_ops.multi_linear_prequantized(weights, rows, block_workspace, family="mmvq")
        indices, values = tile_ops.lm_head_argmax(lm_head, x, lm_workspace)
        results += [indices, values]
        return results

    def fill(seed):
        rng = np.random.default_rng(seed)
        x.copy_(torch.from_numpy(rng.standard_normal((rows, in_dim)).astype(np.float32)))
        gate.copy_(torch.from_numpy(rng.standard_normal((rows, in_dim)).astype(np.float32)))

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        fill(0)
        sequence()  # loads the code objects; nothing is allocated by the library itself
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            captured = sequence()
        for replay in range(4):
            fill(100 + replay)
            graph.replay()
            stream.synchronize()
            replayed = [tensor.clone() for tensor in captured]
            # eager work of the program's own between the replays
            eager = sequence()
            stream.synchronize()
            for index, (a, b) in enumerate(zip(replayed, eager)):
                assert torch.equal(a, b), f"replay {replay}, result {index}"


def test_decode_and_verifier_layers_replayed_from_a_graph(cuda, oracle):
    """A whole decode layer (split attention on a lent workspace, the fused gate/up call, the
    first dual norm inside the Q/K/V/gate launch, the cache commit) and a 16-row verifier block
    in both families, captured once and replayed on new inputs."""
    import torch
    from neuralfn_amd import decode_layer as dl, engine_ops
    rng = np.random.default_rng(31)
    g = dl.LayerGeometry(model_dim=768, query_heads=8, kv_heads=2, head_dim=128, ffn_dim=1280,
                         sliding_window=256)
    shapes = dict(q=(g.attention_dim, g.model_dim), k=(g.kv_dim, g.model_dim),
                  v=(g.kv_dim, g.model_dim), attention_gate=(g.attention_dim, g.model_dim),
                  output=(g.model_dim, g.attention_dim), mlp_gate=(g.ffn_dim, g.model_dim),
                  mlp_up=(g.ffn_dim, g.model_dim), mlp_down=(g.model_dim, g.ffn_dim))
    device = {}
    for index, (name, (out_dim, in_dim)) in enumerate(shapes.items()):
        packed = kquant.quantize(kquant.Q4_K, (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32))
        device[name] = tile_ops.PackedWeight.from_numpy(kquant.Q4_K, packed, out_dim, in_dim)
    for name, width in dict(input_norm=g.model_dim, q_norm=g.head_dim, k_norm=g.head_dim,
                            post_attention_norm=g.model_dim, pre_feedforward_norm=g.model_dim,
                            post_feedforward_norm=g.model_dim).items():
        row = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)
        device[name] = tile_ops.PackedWeight.from_numpy(kquant.F32, row.view(np.uint8).copy(), 1, width)
    weights = dl.LayerWeights(**device)
    keys = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    cache = dl.LayerCache(g, cuda)
    key_image = torch.from_numpy(np.ascontiguousarray(keys, dtype=np.uint16).view(np.int16)).to(cuda)
    value_image = torch.from_numpy(np.ascontiguousarray(values, dtype=np.uint16).view(np.int16)).to(cuda)
    rows, position = 16, 700
    block = torch.empty((rows, g.model_dim), dtype=torch.float32, device=cuda)
    zeros = torch.zeros_like(block)
    attention_workspace = engine_ops.gqa_decode_workspace(g.query_heads, g.head_dim)
    one = tile_ops.small_batch_workspace(1, max(g.model_dim, g.ffn_dim, g.attention_dim))
    many = tile_ops.small_batch_workspace(rows, max(g.model_dim, g.ffn_dim, g.attention_dim))

    def sequence():
        # the same cache before every run: the decode layer commits a row
        cache.keys.copy_(key_image)
        cache.values.copy_(value_image)
        results = list(dl.decode_layer(g, weights, cache, block[:1], zeros[:1], None, position, one, True,
                                       attention_workspace, fused_gate_up=True, fused_input_norm=True))
        results += [cache.keys, cache.values]
        for family, handoff, pair in (("mmq", True, True), ("mmvq", False, False), ("mmvq", True, False)):
            results += list(dl.verify_layer(g, weights, cache, block, zeros, None, position + 1, many, True,
                                            attention_workspace, handoff=handoff, fused_gate_up=pair,
                                            family=family))
        return results

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        block.copy_(torch.from_numpy(rng.standard_normal((rows, g.model_dim)).astype(np.float32)))
        sequence()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            captured = sequence()
        for replay in range(3):
            block.copy_(torch.from_numpy(
                np.random.default_rng(200 + replay).standard_normal((rows, g.model_dim)).astype(np.float32)))
            graph.replay()
            stream.synchronize()
            replayed = [tensor.clone() for tensor in captured]
            eager = sequence()
            stream.synchronize()
            for index, (a, b) in enumerate(zip(replayed, eager)):
                assert torch.equal(a, b), f"replay {replay}, result {index}"
