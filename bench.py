#!/usr/bin/env python3
"""Benchmark of the K-Quant packed-linear hot path on one MI355X.

Headline workload (the configuration the metric is quoted on): decode
attention projections of Glimmer-shaped layers with Q4_K weights — per layer one
grouped launch for Q (6656->4096), K and V (6656->256 each) and one launch for
O (4096->6656) — over 48 independently seeded layers so that no weight byte is
served from cache.  One "step" is one pass over all layers for one batch of
`--rows` tokens, replayed from a HIP graph as the reference's decode loop does.

Prints one JSON line.  `value` is whole-job algorithmic GB/s: packed weight
bytes + float activations in + float outputs, per step, over the step time,
with every input resident in HBM before the timed region.  `roofline` is the
same traffic per launch over the average launch duration measured with HIP
events on the launch stream.  `cpu_baseline` is the reference's CPU K-Quant
matmul timed on this host's cores on a bounded sample of the same workload.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
# HBM bytes per launch of the default workload (rows=1), from the FETCH_SIZE and
# WRITE_SIZE counters of a `--traffic-probe` run, each calibrated on a plain
# copy of known size; the figures and commands are in
# profiles/gemv_dot_kernel_decode_attention_projections_rows1_hbm_traffic.txt
MEASURED_TRAFFIC_BYTES_PER_LAUNCH = {1: 16_690_369}
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "int8": 5000.0, "f32": 157.3}
CU_COUNT = 256
F16_FLOP_PER_CYCLE_PER_CU = 4096   # 4 SIMDs x one 32x32x16 fp16 matrix instruction per 32 cycles
MODEL_DIM, ATTN_DIM, KV_DIM = 6656, 4096, 256
FFN_DIM = 16384
VOCAB = 202048


def parse_args() -> argparse.Namespace:
    parser = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    parser.add_argument("--gpus", type=int, default=1)
    parser.add_argument("--steps", type=int, default=20)
    parser.add_argument("--warmup", type=int, default=3)
    parser.add_argument("--rows", type=int, default=1, help="tokens per step (1, 4 or 8)")
    parser.add_argument("--layers", type=int, default=48)
    parser.add_argument("--no-cpu-baseline", action="store_true")
    parser.add_argument("--no-extras", action="store_true",
                        help="skip the lm_head and prefill side measurements")
    parser.add_argument("--no-graph", action="store_true", help="enqueue directly, no HIP graph")
    parser.add_argument("--traffic-probe", action="store_true",
                        help="for a counter run: one plain copy of 256 MiB, then one eager step; "
                             "no timing, no JSON")
    return parser.parse_args()


def layer_algorithmic_bytes(rows: int) -> int:
    """Packed weights + float inputs (once per distinct input) + float outputs."""
    from neuralfn_amd import kquant
    weights = (kquant.packed_nbytes(kquant.Q4_K, ATTN_DIM, MODEL_DIM)
               + 2 * kquant.packed_nbytes(kquant.Q4_K, KV_DIM, MODEL_DIM)
               + kquant.packed_nbytes(kquant.Q4_K, MODEL_DIM, ATTN_DIM))
    inputs = rows * (MODEL_DIM + ATTN_DIM) * 4
    outputs = rows * (ATTN_DIM + KV_DIM + KV_DIM + MODEL_DIM) * 4
    return weights + inputs + outputs


def make_layers(layers: int, device):
    """Seeded N(0, 0.02) weights, quantized to Q4_K on the host, resident on the GPU."""
    import torch
    from neuralfn_amd import kquant, tile_ops
    shapes = (("q", ATTN_DIM, MODEL_DIM), ("k", KV_DIM, MODEL_DIM), ("v", KV_DIM, MODEL_DIM),
              ("o", MODEL_DIM, ATTN_DIM))
    result = []
    host_copies = []
    for layer in range(layers):
        entry = {}
        host = {}
        for index, (name, out_dim, in_dim) in enumerate(shapes):
            generator = torch.Generator(device=device).manual_seed(1_000_003 * layer + index + 1)
            weights = (torch.randn((out_dim, in_dim), generator=generator, device=device,
                                   dtype=torch.float32) * 0.02).cpu().numpy()
            packed = kquant.quantize(kquant.Q4_K, weights)
            entry[name] = tile_ops.PackedWeight.from_numpy(kquant.Q4_K, packed, out_dim, in_dim,
                                                           str(device))
            host[name] = packed
        result.append(entry)
        host_copies.append(host)
    return result, host_copies


class DecodeStep:
    """Pre-built ctypes arguments for the two launches of every layer."""

    def __init__(self, layers, rows: int, device, family: str = "mmq"):
        import torch
        from neuralfn_amd import kquant, tile_ops
        self.lib = tile_ops.load()
        self.rows = rows
        # "mmvq": the verifier family, every row in the one-row arithmetic bit for bit
        self.function = (self.lib.nfn_native_tile_k_quant_mmq_multi_linear_float32_v1 if family == "mmq"
                         else self.lib.nfn_native_tile_k_quant_mmvq_multi_linear_float32_v1)
        self.layers = layers
        self.workspace = tile_ops.small_batch_workspace(16, MODEL_DIM, device)
        self.hidden = torch.from_numpy(
            kquant.synthetic_activations(11, rows * len(layers), MODEL_DIM)).to(device)
        self.attention = torch.from_numpy(
            kquant.synthetic_activations(12, rows * len(layers), ATTN_DIM)).to(device)
        self.outputs = []
        self.calls = []
        for index, layer in enumerate(layers):
            outs = {name: torch.empty((rows, weight.output_dim), dtype=torch.float32, device=device)
                    for name, weight in layer.items()}
            self.outputs.append(outs)
            self.calls.append((index, layer, outs))
        self._keep = []

    def enqueue(self, stream: int) -> None:
        from neuralfn_amd import tile_ops
        function = self.function
        rows = self.rows
        for index, layer, outs in self.calls:
            qkv = [layer[n].descriptor(stream) for n in ("q", "k", "v")]
            o = [layer["o"].descriptor(stream)]
            self._keep.append((qkv, o))
            hidden = self.hidden[index * rows:(index + 1) * rows]
            attention = self.attention[index * rows:(index + 1) * rows]
            tile_ops.check(function(
                tile_ops._descriptor_array(qkv), hidden.data_ptr(),
                tile_ops._pointer_array([outs["q"], outs["k"], outs["v"]]), 3, rows,
                self.workspace.data_ptr(), self.workspace.numel(), stream), "qkv projections")
            tile_ops.check(function(
                tile_ops._descriptor_array(o), attention.data_ptr(),
                tile_ops._pointer_array([outs["o"]]), 1, rows,
                self.workspace.data_ptr(), self.workspace.numel(), stream), "o projection")
        self._keep.clear()

    @property
    def launches_per_step(self) -> int:
        return 2 * len(self.calls)


SETTLE_SECONDS = 0.08


def settle(run) -> None:
    """Untimed calls of run() for SETTLE_SECONDS before a measurement's warm-up.

    The memory-side clocks take tens of milliseconds of load to reach their steady
    state after the idle time of a host-side set-up: the same lm_head launch measured
    249 us in the first 6 ms of load and 208 us from about 60 ms on.  A decode loop runs
    in that steady state; the figures here are meant to be its figures.
    """
    import torch
    torch.cuda.synchronize()
    start = time.perf_counter()
    while time.perf_counter() - start < SETTLE_SECONDS:
        for _ in range(8):
            run()
        torch.cuda.synchronize()


def time_replays(run, steps: int, warmup: int) -> float:
    """Milliseconds per call of run(), measured with events on the current stream
    (after settle(): untimed calls until the clocks are steady, then `warmup` more)."""
    import torch
    settle(run)
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        run()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def step_distribution(run, steps: int, warmup: int, per_step: int) -> dict:
    """Median and 5th / 95th percentile of run()'s duration, one event pair per call.

    Reported in microseconds per launch (`per_step` launches per call).
    """
    import torch
    for _ in range(warmup):
        run()
    torch.cuda.synchronize()
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True))
             for _ in range(steps)]
    for start, stop in pairs:
        start.record()
        run()
        stop.record()
    torch.cuda.synchronize()
    times = sorted(start.elapsed_time(stop) * 1e3 / per_step for start, stop in pairs)

    def at(fraction: float) -> float:
        return round(times[min(len(times) - 1, int(fraction * len(times)))], 3)

    return {"median": at(0.5), "p05": at(0.05), "p95": at(0.95), "samples": len(times)}


def time_graph(run, stream, steps: int, warmup: int) -> float:
    """Milliseconds per call of run(), captured once into a HIP graph and replayed.

    A call is a few dependent launches; replaying them from a graph takes the
    host's launch latency between them out of the measurement, as the decode
    loop's own graph replay does.
    """
    import torch
    run()  # eager: loads code objects, and nothing is allocated during capture
    stream.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=stream):
        run()
    return time_replays(graph.replay, steps, warmup)


def cpu_baseline(host_layers, rows: int, budget_seconds: float = 20.0) -> dict:
    """The reference's CPU matmul on this host, on as many layers as fit the budget."""
    from neuralfn_amd import kquant
    from oracle import kquant_oracle
    use_reference = kquant_oracle.reference_available()
    kind = "reference" if use_reference else "port"
    hidden = kquant.synthetic_activations(11, rows * len(host_layers), MODEL_DIM)
    attention = kquant.synthetic_activations(12, rows * len(host_layers), ATTN_DIM)
    shapes = {"q": (ATTN_DIM, MODEL_DIM), "k": (KV_DIM, MODEL_DIM), "v": (KV_DIM, MODEL_DIM),
              "o": (MODEL_DIM, ATTN_DIM)}

    def run(name, packed, x):
        out_dim, in_dim = shapes[name]
        if use_reference:
            return kquant_oracle.ref_linear(kquant.Q4_K, packed, out_dim, in_dim, x)
        return kquant_oracle.linear(kquant.Q4_K, packed, out_dim, in_dim, x, as_written=True)

    done = 0
    began = time.perf_counter()
    minimum_seconds = 10.0
    while True:
        for index, layer in enumerate(host_layers):
            x = hidden[index * rows:(index + 1) * rows]
            a = attention[index * rows:(index + 1) * rows]
            for name in ("q", "k", "v"):
                run(name, layer[name], x)
            run("o", layer["o"], a)
            done += 1
            if time.perf_counter() - began > budget_seconds:
                break
        if time.perf_counter() - began > minimum_seconds:
            break
    elapsed = time.perf_counter() - began
    cores = kquant_oracle.worker_count(ATTN_DIM, 128)
    return {
        "value": round(done * layer_algorithmic_bytes(rows) / elapsed / 1e9, 4),
        "unit": "GB/s",
        "cores": cores,
        "kind": kind,
        "sample": f"{done} layer passes (Q,K,V,O at rows={rows}) over the {len(host_layers)} "
                  f"layers of the workload in {elapsed:.2f} s; "
                  f"{done * rows / elapsed:.3f} layer-tokens/s",
    }


def launch_floor_extra(layers, device, stream, steps: int, warmup: int) -> dict:
    """What the headline's launches would cost with no arithmetic at all: the same number of
    back-to-back launches in a HIP graph, each one workgroup per compute unit that only reads
    the bytes a decode launch streams (nfn_mi355_read_probe_v1), and the same with an empty
    kernel.  The ceiling these two put over the headline is a property of 16 MB launches on
    this chip, not of the kernels."""
    import torch
    from neuralfn_amd import kquant, probes, tile_ops
    lib = probes.load()
    qkv = (kquant.packed_nbytes(kquant.Q4_K, ATTN_DIM, MODEL_DIM)
           + 2 * kquant.packed_nbytes(kquant.Q4_K, KV_DIM, MODEL_DIM))
    out = kquant.packed_nbytes(kquant.Q4_K, MODEL_DIM, ATTN_DIM)
    per_layer = qkv + out
    pool = torch.randint(0, 256, (len(layers) * per_layer,), dtype=torch.uint8, device=device)
    sink = torch.zeros(1024, dtype=torch.int32, device=device)

    def enqueue(read: bool):
        handle = int(torch.cuda.current_stream().cuda_stream)
        for layer in range(len(layers)):
            base = pool.data_ptr() + layer * per_layer
            for offset, nbytes in ((0, qkv), (qkv, out)):
                tile_ops.check(lib.nfn_mi355_read_probe_v1(
                    base + offset, nbytes if read else 0, sink.data_ptr(), handle), "read probe")

    launches = 2 * len(layers)
    read_ms = time_graph(lambda: enqueue(True), stream, steps, warmup)
    empty_ms = time_graph(lambda: enqueue(False), stream, steps, warmup)
    bytes_per_launch = per_layer / 2

    # Would a launch gain by pulling the next launch's first bytes into its XCD's L2 while it
    # streams its own (weights are static, so a decode loop could hand the next descriptor set
    # down as a hint)?  The same chain of launches over equal regions, each also requesting
    # `rounds` x 512 16-byte pieces per workgroup of the following region (8 rounds = all of it).
    region = (per_layer // 2) // (16 * CU_COUNT) * (16 * CU_COUNT)
    def enqueue_chained(rounds: int):
        handle = int(torch.cuda.current_stream().cuda_stream)
        for index in range(launches):
            base = pool.data_ptr() + index * region
            following = pool.data_ptr() + ((index + 1) % launches) * region
            tile_ops.check(lib.nfn_mi355_read_probe_chained_v1(
                base, region, following, rounds, sink.data_ptr(), handle), "chained read probe")
    chained = {f"prefetch_{rounds}_of_8_rounds": round(
        time_graph(lambda: enqueue_chained(rounds), stream, steps, warmup) * 1e3 / launches, 3)
        for rounds in (0, 1, 2, 4, 8)}
    return {
        "chained_read_only_us_per_launch": chained,
        "workload": f"{launches} launches a HIP-graph replay, one workgroup of 512 per compute unit: "
                    "read only the packed bytes of a decode launch / an empty kernel",
        "read_only_us_per_launch": round(read_ms * 1e3 / launches, 3),
        "empty_kernel_us_per_launch": round(empty_ms * 1e3 / launches, 3),
        "read_only_GB/s": round(bytes_per_launch / (read_ms * 1e3 / launches) / 1e3, 1),
        "read_only_frac_hbm": round(bytes_per_launch / (read_ms * 1e3 / launches) / 1e3 / HBM_PEAK_GBS, 4)}


def patterned_packed_on_device(encoding: int, out_dim: int, in_dim: int, device):
    """The reference benchmark's weights (tools/bench_muse_glimmer_packed_linear.py:161-177):
    byte i of the tensor is (29 i + 17) mod 256, then every block gets d = 0x2800 and (Q4_K,
    Q5_K) dmin = 0x2400."""
    import torch
    from neuralfn_amd import kquant, tile_ops
    elements, nbytes = kquant.BLOCKS[encoding]
    total = out_dim * in_dim // elements * nbytes
    data = ((torch.arange(total, dtype=torch.int64, device=device) * 29 + 17) & 0xFF).to(torch.uint8)
    blocks = data.view(-1, nbytes)
    if encoding == kquant.Q6_K:
        blocks[:, 208], blocks[:, 209] = 0x00, 0x28
    else:
        blocks[:, 0], blocks[:, 1], blocks[:, 2], blocks[:, 3] = 0x00, 0x28, 0x00, 0x24
    return tile_ops.PackedWeight(encoding, out_dim, in_dim, data)


# ms on an RTX 5090 as the reference publishes them (docs/glimmer-support-todo.md:730-739, 746-750)
PUBLISHED_SHAPES = (
    ("q4_k", 6656, 4096, {1: 0.018, 16: 0.106}),
    ("q4_k", 6656, 19968, {1: 0.055, 16: 0.376}),
    ("q6_k", 19968, 6656, {1: 0.083, 16: 0.454}),
    ("q5_k", 6656, VOCAB, {1: 0.626, 16: 4.198}),
    ("q4_k", 6656, 256, {1: 0.008, 16: 0.032}),
    ("q6_k", 6656, 256, {16: 0.038}),
)


def published_shapes_extra(device, stream, steps: int, warmup: int) -> dict:
    """The reference's own microbenchmark shapes with its patterned bytes and inputs, one and 16
    rows, through the same entry point (k_quant_mmq_multi_linear), timed the way it times them
    (back-to-back enqueues of one call, events around them), beside its published RTX 5090 times."""
    import torch
    from neuralfn_amd import kquant, tile_ops
    names = {"q4_k": kquant.Q4_K, "q5_k": kquant.Q5_K, "q6_k": kquant.Q6_K}
    result = {"workload": "patterned bytes (29 i + 17 mod 256, d 0x2800, dmin 0x2400), inputs "
                          "((37 r + 13 c) mod 257 - 128) / 257; ms: per call over 30 back-to-back eager "
                          "enqueues, as the reference times them (bound by the host for the small shapes: "
                          "an eager launch costs about 8 us here); ms_graph_replay: the same call eight "
                          "times in a HIP graph, per call; GB/s and frac_hbm from ms_graph_replay"}
    for name, in_dim, out_dim, published in PUBLISHED_SHAPES:
        weight = patterned_packed_on_device(names[name], out_dim, in_dim, device)
        workspace = tile_ops.small_batch_workspace(16, in_dim, device)
        for rows in (1, 16):
            if rows not in published:
                continue
            r = torch.arange(rows, dtype=torch.int64, device=device)[:, None]
            c = torch.arange(in_dim, dtype=torch.int64, device=device)[None, :]
            x = (((r * 37 + c * 13) % 257 - 128).to(torch.float32) / 257.0).contiguous()
            out = torch.empty((rows, out_dim), dtype=torch.float32, device=device)
            ms = time_replays(lambda: tile_ops.multi_linear([weight], x, workspace, outputs=[out]),
                              30, 5)

            def eight():
                for _ in range(8):
                    tile_ops.multi_linear([weight], x, workspace, outputs=[out])
            replayed = time_graph(eight, stream, max(5, steps // 2), max(2, warmup // 2)) / 8
            if not bool(torch.isfinite(out).all()):
                raise RuntimeError(f"{name} {in_dim}->{out_dim}: non-finite output")
            traffic = weight.nbytes + rows * (in_dim + out_dim) * 4
            result[f"{name}_{in_dim}_to_{out_dim}_rows{rows}"] = {
                "ms": round(ms, 4), "ms_graph_replay": round(replayed, 4),
                "GB/s": round(traffic / replayed / 1e6, 1),
                "frac_hbm": round(traffic / replayed / 1e6 / HBM_PEAK_GBS, 4),
                "reference_rtx5090_ms": published[rows]}
        del weight
    return result


def large_projection_extra(device, stream, steps: int, warmup: int) -> dict:
    """One-token GEMV of one projection large enough (65,536 rows of 6,656) that the launch's
    fixed costs vanish: what the decode kernels stream at per format."""
    import torch
    from neuralfn_amd import kquant, tile_ops
    out_dim = 65536
    x = torch.from_numpy(kquant.synthetic_activations(51, 1, MODEL_DIM)).to(device)
    workspace = tile_ops.small_batch_workspace(1, MODEL_DIM, device)
    out = torch.empty((1, out_dim), dtype=torch.float32, device=device)
    result = {"workload": f"one token, {MODEL_DIM}->{out_dim}, one projection per launch, HIP-graph replay"}
    for encoding in (kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0):
        # two tensors visited in turn, together beyond the 256 MB memory-side cache
        weights = [random_packed_on_device(encoding, out_dim, MODEL_DIM, device, 60 + k) for k in range(2)]

        def run():
            for weight in weights:
                tile_ops.multi_linear([weight], x, workspace, outputs=[out])

        ms = time_graph(run, stream, max(5, steps // 2), max(2, warmup // 2)) / len(weights)
        traffic = weights[0].nbytes + (MODEL_DIM + out_dim) * 4
        result[kquant.NAMES[encoding]] = {
            "MB": round(weights[0].nbytes / 1e6, 1), "us": round(ms * 1e3, 2),
            "GB/s": round(traffic / ms / 1e6, 1),
            "frac_hbm": round(traffic / ms / 1e6 / HBM_PEAK_GBS, 4)}
        del weights
    return result


def cpu_baselines_other_configs(host_layers) -> dict:
    """The CPU path on the other configurations: config 0 (one Q4_K GEMV 6656->4096) and config 2
    (the whole Q6_K lm_head, one row) in full with the reference's own linear() where it is
    built; config 3 as a stated slice of the reference's batched form (linear_rows,
    resident_glimmer_assistant.cpp:459-483: one flat loop over rows x outputs, every weight decoded
    again for every row), restated by the oracle, and extrapolated linearly in the rows."""
    from neuralfn_amd import kquant
    from oracle import kquant_oracle
    use_reference = kquant_oracle.reference_available()
    kind = "reference" if use_reference else "port"

    def single(encoding, packed, out_dim, in_dim, x):
        if use_reference:
            return kquant_oracle.ref_linear(encoding, packed, out_dim, in_dim, x)
        return kquant_oracle.linear(encoding, packed, out_dim, in_dim, x, as_written=True)

    result = {}
    # config 0
    x = kquant.synthetic_activations(11, 1, MODEL_DIM)
    packed = host_layers[0]["q"]
    single(kquant.Q4_K, packed, ATTN_DIM, MODEL_DIM, x)
    calls, began = 0, time.perf_counter()
    while time.perf_counter() - began < 3.0:
        single(kquant.Q4_K, packed, ATTN_DIM, MODEL_DIM, x)
        calls += 1
    seconds = (time.perf_counter() - began) / calls
    traffic = packed.size + (MODEL_DIM + ATTN_DIM) * 4
    result["config0_q4_k_gemv_6656_to_4096"] = {
        "value": round(traffic / seconds / 1e9, 4), "unit": "GB/s", "ms_per_call": round(seconds * 1e3, 3),
        "cores": kquant_oracle.worker_count(ATTN_DIM, 128), "kind": kind,
        "sample": f"{calls} full calls at one row"}
    # config 2: the byte values do not change what the CPU path costs
    rng = np.random.default_rng(7)
    stride = kquant.row_stride_bytes(kquant.Q6_K, MODEL_DIM)
    lm_head = rng.integers(0, 256, VOCAB * stride, dtype=np.uint8).reshape(-1, 210)
    lm_head[:, 208], lm_head[:, 209] = 0, 0x14
    lm_head = lm_head.reshape(-1)
    x = kquant.synthetic_activations(21, 1, MODEL_DIM, True)
    began = time.perf_counter()
    logits = single(kquant.Q6_K, lm_head, VOCAB, MODEL_DIM, x)
    kquant_oracle.argmax(logits[0])
    seconds = time.perf_counter() - began
    result["config2_q6_k_lm_head_argmax_one_row"] = {
        "value": round((lm_head.size + MODEL_DIM * 4 + 12) / seconds / 1e9, 4), "unit": "GB/s",
        "ms_per_call": round(seconds * 1e3, 1), "cores": kquant_oracle.worker_count(VOCAB, 128),
        "kind": kind, "sample": "one full call: 202,048 x 6,656 Q6_K rows and the argmax over the logits"}
    del lm_head, logits
    # config 3: 8 rows of the gate projection in the batched form, then times M / 8 and three projections
    rng = np.random.default_rng(8)
    stride = kquant.row_stride_bytes(kquant.Q4_K, MODEL_DIM)
    gate = rng.integers(0, 256, FFN_DIM * stride, dtype=np.uint8).reshape(-1, 144)
    gate[:, 0], gate[:, 1], gate[:, 2], gate[:, 3] = 0, 0x14, 0, 0x14
    gate = gate.reshape(-1)
    slice_rows = 8
    x = kquant.synthetic_activations(31, slice_rows, MODEL_DIM)
    began = time.perf_counter()
    kquant_oracle.linear(kquant.Q4_K, gate, FFN_DIM, MODEL_DIM, x, as_written=True)
    seconds = time.perf_counter() - began
    flops = 2.0 * slice_rows * MODEL_DIM * FFN_DIM
    result["config3_q4_k_ffn_prefill_slice"] = {
        "value": round(flops / seconds / 1e12, 6), "unit": "TFLOP/s",
        "cores": kquant_oracle.worker_count(slice_rows * FFN_DIM, 128), "kind": "port",
        "sample": f"{slice_rows} rows x 6656->16384 in the reference's batched CPU form (every weight "
                  f"decoded again per row) in {seconds:.2f} s",
        "extrapolated_seconds_for_one_ffn": {
            f"M={rows}": round(seconds / slice_rows * rows * 3, 1) for rows in (512, 2048)},
        "note": "extrapolation: cost is linear in rows and the three projections have the same size"}
    return result


def decode_batch_extra(layers, device, stream, steps: int, warmup: int, headline_rows: int) -> dict:
    """The headline workload at the other batch sizes of the same configuration."""
    import torch

    result = {"workload": "decode attention projections as the headline, other batch sizes, HIP-graph replay"}
    for rows in (1, 4, 8, 16):
        if rows == headline_rows:
            continue
        step = DecodeStep(layers, rows, device)
        ms = time_graph(lambda: step.enqueue(int(torch.cuda.current_stream().cuda_stream)),
                        stream, steps, warmup)
        traffic = len(layers) * layer_algorithmic_bytes(rows)
        result[f"rows{rows}"] = {
            "ms_per_step": round(ms, 5), "GB/s": round(traffic / ms / 1e6, 1),
            "frac_hbm": round(traffic / ms / 1e6 / HBM_PEAK_GBS, 4),
            "us_per_launch": round(ms * 1e3 / step.launches_per_step, 3),
            "tokens/s": round(rows / ms * 1e3, 1)}
    # the exact verifier's form of a block: the `mmvq` family, whose rows carry the one-row
    # arithmetic bit for bit (vector-ALU kernels, four rows a pass over the weights)
    for rows in (4, 16):
        step = DecodeStep(layers, rows, device, "mmvq")
        ms = time_graph(lambda: step.enqueue(int(torch.cuda.current_stream().cuda_stream)),
                        stream, max(5, steps // 2), max(2, warmup // 2))
        traffic = len(layers) * layer_algorithmic_bytes(rows)
        result[f"rows{rows}_exact_verifier_family"] = {
            "ms_per_step": round(ms, 5), "GB/s": round(traffic / ms / 1e6, 1),
            "frac_hbm": round(traffic / ms / 1e6 / HBM_PEAK_GBS, 4),
            "us_per_launch": round(ms * 1e3 / step.launches_per_step, 3),
            "tokens/s": round(rows / ms * 1e3, 1)}
    return result


def random_packed_on_device(encoding: int, out_dim: int, in_dim: int, device, seed: int):
    """Uniform random quant bytes with small finite scales, made on the GPU.

    Used only where throughput is measured on tensors too large to quantize on
    the host within the benchmark's time; parity for these paths is in tests/.
    """
    import torch
    from neuralfn_amd import kquant, tile_ops
    elements, nbytes = kquant.BLOCKS[encoding]
    generator = torch.Generator(device=device).manual_seed(seed)
    blocks = torch.randint(0, 256, (out_dim * in_dim // elements, nbytes), generator=generator,
                           device=device, dtype=torch.uint8)
    halves = {kquant.Q4_K: (0, 2), kquant.Q5_K: (0, 2), kquant.Q6_K: (208,), kquant.Q8_0: (0,)}
    for offset in halves[encoding]:
        blocks[:, offset + 1] = (blocks[:, offset + 1] & 0x03) | 0x14  # d in [2^-10, 2^-9)
    return tile_ops.PackedWeight(encoding, out_dim, in_dim, blocks.reshape(-1))


def lm_head_extra(device, stream, steps: int, warmup: int) -> dict:
    import torch
    from neuralfn_amd import kquant, tile_ops
    weight = random_packed_on_device(kquant.Q6_K, VOCAB, MODEL_DIM, device, 7)
    result = {}
    # one row: the streaming dot kernel; four, eight and sixteen (a verifier block): the fp16
    # matrix-core kernel behind its conversion launch
    for rows in (1, 4, 8, 16):
        x = torch.from_numpy(kquant.synthetic_activations(21, rows, MODEL_DIM, True)).to(device)
        nbytes = tile_ops.load().nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, VOCAB)
        workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
        indices = torch.empty(rows, dtype=torch.int64, device=device)
        values = torch.empty(rows, dtype=torch.float32, device=device)
        ms = time_graph(lambda: tile_ops.lm_head_argmax(weight, x, workspace, indices, values),
                        stream, steps, warmup)
        traffic = weight.nbytes + rows * MODEL_DIM * 4 + rows * 12
        result[f"rows{rows}"] = {"ms": round(ms, 4), "GB/s": round(traffic / ms / 1e6, 1),
                                 "frac_hbm": round(traffic / ms / 1e6 / HBM_PEAK_GBS, 4),
                                 "tokens/s": round(rows / ms * 1e3, 1)}
    # The same block of 16 rows through the reference's own pair of calls, the small-batch linear
    # (logits to memory) and the row argmax.
    rows = 16
    x = torch.from_numpy(kquant.synthetic_activations(21, rows, MODEL_DIM, True)).to(device)
    workspace = tile_ops.small_batch_workspace(rows, MODEL_DIM, device)
    logits = torch.empty((rows, VOCAB), dtype=torch.float32, device=device)
    indices = torch.empty(rows, dtype=torch.int64, device=device)
    values = torch.empty(rows, dtype=torch.float32, device=device)

    def block():
        tile_ops.multi_linear([weight], x, workspace, outputs=[logits])
        tile_ops.argmax_rows(logits, indices, values)

    ms = time_graph(block, stream, steps, warmup)
    traffic = weight.nbytes + rows * MODEL_DIM * 4 + 2 * rows * VOCAB * 4
    result["rows16_linear_then_argmax"] = {
        "ms": round(ms, 4), "GB/s": round(traffic / ms / 1e6, 1),
        "frac_hbm": round(traffic / ms / 1e6 / HBM_PEAK_GBS, 4),
        "tokens/s": round(rows / ms * 1e3, 1)}
    return {"workload": f"Q6_K lm_head {MODEL_DIM}->{VOCAB}, fused argmax", **result}


def prefill_extra(device, stream, steps: int, warmup: int) -> dict:
    import torch
    from neuralfn_amd import kquant, probes, tile_ops
    gate = random_packed_on_device(kquant.Q4_K, FFN_DIM, MODEL_DIM, device, 8)
    up = random_packed_on_device(kquant.Q4_K, FFN_DIM, MODEL_DIM, device, 10)
    down = random_packed_on_device(kquant.Q4_K, MODEL_DIM, FFN_DIM, device, 9)
    result = {}
    for mode, name in ((tile_ops.GEMM_F16, "f16"),):
        for rows in (512, 2048):
            x = torch.from_numpy(kquant.synthetic_activations(31, rows, MODEL_DIM)).to(device)
            h = torch.from_numpy(kquant.synthetic_activations(32, rows, FFN_DIM)).to(device)
            # gate_up: both projections of the block's input through the call that converts
            # the activations once (nfn_mi355_k_quant_gemm_multi_float32_v1), as a SwiGLU
            # feed-forward block runs them; gate_alone: one of them through the single call
            for label, weights, source in (("gate_up", [gate, up], x), ("gate_alone", [gate], x),
                                           ("down", [down], h)):
                outs = [torch.empty((rows, w.output_dim), dtype=torch.float32, device=device)
                        for w in weights]
                nbytes = max(tile_ops.load().nfn_mi355_k_quant_gemm_workspace_bytes_v1(
                    rows, w.input_dim, w.output_dim, mode) for w in weights)
                workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
                if len(weights) == 1:
                    call = lambda: tile_ops.gemm(weights[0], source, mode, workspace, outs[0])
                else:
                    call = lambda: tile_ops.gemm_multi(weights, source, mode, workspace, outs)
                ms = time_graph(call, stream, max(5, steps // 2), max(2, warmup // 2))
                flops = sum(2.0 * rows * w.input_dim * w.output_dim for w in weights)
                tflops = flops / ms / 1e9
                result[f"{name}_{label}_M{rows}"] = {
                    "ms": round(ms, 4), "TFLOP/s": round(tflops, 1),
                    "frac_mfma": round(tflops / MFMA_PEAK_TFLOPS[name], 4),
                    "tokens/s": round(rows / ms * 1e3, 1)}
    # The same gate projection at M = 512 through the generic v1 call, the only v1 call that
    # takes more than 16 rows.  It has no workspace argument, so it stays in the exact tier:
    # float activations against weights decoded to float, on the float matrix instruction
    # (256 flop per cycle and compute unit, a sixteenth of the fp16 one).
    rows = 512
    x = torch.from_numpy(kquant.synthetic_activations(31, rows, MODEL_DIM)).to(device)
    ms = time_replays(lambda: tile_ops.linear(gate, x), 5, 2)
    tflops = 2.0 * rows * MODEL_DIM * FFN_DIM / ms / 1e9
    result["generic_v1_linear_f32_matrix_cores_gate_M512"] = {
        "ms": round(ms, 4), "TFLOP/s": round(tflops, 2),
        "frac_mfma_f32": round(tflops / MFMA_PEAK_TFLOPS["f32"], 4),
        "x_workspace_gemm": round(ms / result["f16_gate_alone_M512"]["ms"], 1)}
    # The shader clock while the largest shape runs, and the matrix-core peak at
    # that clock: 256 CUs x 4096 fp16 flop per cycle per CU.
    rows = 2048
    x = torch.from_numpy(kquant.synthetic_activations(31, rows, MODEL_DIM)).to(device)
    out = torch.empty((rows, FFN_DIM), dtype=torch.float32, device=device)
    nbytes = tile_ops.load().nfn_mi355_k_quant_gemm_workspace_bytes_v1(
        rows, MODEL_DIM, FFN_DIM, tile_ops.GEMM_F16)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)
    probe = probes.ShaderClockProbe(device)
    for _ in range(10):  # the clock settles under load before the probe's window
        tile_ops.gemm(gate, x, tile_ops.GEMM_F16, workspace, out)
    probe.start(5000)
    for _ in range(16):
        tile_ops.gemm(gate, x, tile_ops.GEMM_F16, workspace, out)
    stream.synchronize()
    megahertz = probe.megahertz()
    peak_at_clock = megahertz * 1e6 * CU_COUNT * F16_FLOP_PER_CYCLE_PER_CU / 1e12
    result["shader_clock_under_gemm_MHz"] = round(megahertz, 1)
    result["f16_peak_at_that_clock_TFLOP/s"] = round(peak_at_clock, 1)
    result["f16_peak_published_TFLOP/s"] = MFMA_PEAK_TFLOPS["f16"]
    # The same shape as a plain fp16 GEMM through the vendor library (no packed
    # weights, no dequantization): what the matrix cores sustain on this box
    # with operands of the same statistics.
    a16 = x.to(torch.float16)
    w16 = (torch.randn(FFN_DIM, MODEL_DIM, device=device) * 0.02).to(torch.float16)
    ms = time_replays(lambda: torch.matmul(a16, w16.t()), max(5, steps // 2), max(2, warmup // 2))
    library = 2.0 * rows * MODEL_DIM * FFN_DIM / ms / 1e9
    result["library_f16_gemm_same_shape_M2048"] = {
        "ms": round(ms, 4), "TFLOP/s": round(library, 1),
        "frac_mfma": round(library / MFMA_PEAK_TFLOPS["f16"], 4)}
    # Config 3's int8 leg: what the int8 matrix cores would have to run, from registers
    # (nfn_mi355_mfma_rate_probe_v1), beside the fp16 instruction the GEMM uses.  One step =
    # one 32 x 32 x 32 product per wave = 65,536 flop.
    lib = probes.load()
    sink = torch.zeros(4096, dtype=torch.float32, device=device)
    probe_steps, groups = 20000, 2 * CU_COUNT
    legs = {}
    for mode, label in ((0, "f16_mfma"), (1, "int8_mfma_one_plane_no_rescale"),
                        (3, "int8_mfma_one_plane_rescaled_per_32"),
                        (2, "int8_mfma_two_planes_rescaled_per_32")):
        def run():
            tile_ops.check(lib.nfn_mi355_mfma_rate_probe_v1(
                mode, probe_steps, groups, sink.data_ptr(),
                int(torch.cuda.current_stream().cuda_stream)), "mfma rate probe")
        ms = time_replays(run, 5, 2)
        legs[label] = round(65536.0 * probe_steps * groups * 4 / ms / 1e9, 1)
    result["matrix_core_probe_TFLOP/s_equivalent"] = {
        **legs,
        "note": "useful 32x32x32 products per second x 65,536; one plane rescaled per 32 values is "
                "config 3's int8 leg as written (8-bit activations per 32-value group, judged "
                "against the Q8_1 oracle); the last row is the only int8 form whose results can "
                "meet the 2e-3 bound against the float oracle (16-bit activation codes); "
                "NFN_MI355_GEMM_INT8 stays reserved while both are below the fp16 row"}
    return {"workload": f"Q4_K SwiGLU FFN projections {MODEL_DIM}<->{FFN_DIM}, dequant-GEMM "
                        "incl. activation conversion", **result}


def decode_layer_extra(device, stream, steps: int, warmup: int) -> dict:
    """Whole decode layers at the workload's geometry, every operator through the C ABI in the
    engine's order (neuralfn_amd/decode_layer.py): what a token costs beyond the projections.
    Local layers (2048-key window) and global ones at a 32768-token context, each with the
    reference's fused attention call and with the split form."""
    import torch
    from neuralfn_amd import decode_layer as dl, engine_ops, kquant, tile_ops
    layers = 8
    ones = {width: tile_ops.PackedWeight(
        kquant.F32, 1, width, torch.ones(width, dtype=torch.float32, device=device).view(torch.uint8))
        for width in (MODEL_DIM, 128)}
    shapes = dict(q=(ATTN_DIM, MODEL_DIM), k=(KV_DIM, MODEL_DIM), v=(KV_DIM, MODEL_DIM),
                  attention_gate=(ATTN_DIM, MODEL_DIM), output=(MODEL_DIM, ATTN_DIM),
                  mlp_gate=(FFN_DIM, MODEL_DIM), mlp_up=(FFN_DIM, MODEL_DIM),
                  mlp_down=(MODEL_DIM, FFN_DIM))
    weights = []
    for layer in range(layers):
        packed = {name: random_packed_on_device(kquant.Q4_K, out_dim, in_dim, device,
                                                1000 + 10 * layer + index)
                  for index, (name, (out_dim, in_dim)) in enumerate(shapes.items())}
        weights.append(dl.LayerWeights(
            **packed, input_norm=ones[MODEL_DIM], q_norm=ones[128], k_norm=ones[128],
            post_attention_norm=ones[MODEL_DIM], pre_feedforward_norm=ones[MODEL_DIM],
            post_feedforward_norm=ones[MODEL_DIM]))
    weight_bytes = sum(w.packed_bytes() for w in weights)
    workspace = tile_ops.small_batch_workspace(1, FFN_DIM, device)
    embedding = torch.from_numpy(kquant.synthetic_activations(41, 1, MODEL_DIM)).to(device)
    zeros = torch.zeros_like(embedding)
    last = {}
    result = {
        "workload": f"{layers} whole decode layers (Q4_K projections incl. attention gate and FFN "
                    f"{MODEL_DIM}<->{FFN_DIM}), one token, HIP-graph replay; local = 2048-key "
                    "window, global = every key of a 32768-token context; "
                    "reference_fused_attention = the reference's entry points only, "
                    "split_attention = with this library's additions (split attention, gate and "
                    "up in one call with SwiGLU at the row ends, the first dual norm inside the "
                    "Q/K/V/gate launch)"}
    for kind, keys, local in (("local", 2048, True), ("global", 32768, False)):
        g = dl.LayerGeometry(model_dim=MODEL_DIM, query_heads=ATTN_DIM // 128,
                             kv_heads=KV_DIM // 128, head_dim=128, ffn_dim=FFN_DIM,
                             sliding_window=keys)
        position = 5000 if local else keys - 1
        caches = []
        for _ in range(layers):
            cache = dl.LayerCache(g, device)
            cache.keys.copy_(torch.randn(cache.keys.shape, device=device).to(torch.bfloat16).view(torch.int16))
            cache.values.copy_(torch.randn(cache.values.shape, device=device).to(torch.bfloat16).view(torch.int16))
            caches.append(cache)
        cache_bytes = layers * 2 * keys * g.kv_dim * 2
        forms = (("reference_fused_attention", None, dl.LAUNCHES_PER_LAYER),
                 ("split_attention", engine_ops.gqa_decode_workspace(g.query_heads, g.head_dim, device),
                  dl.LAUNCHES_PER_LAYER_FUSED))
        for name, attention_workspace, launches in forms:
            def token():
                pending, residual, pending_norm = embedding, zeros, None
                for layer_weights, cache in zip(weights, caches):
                    # (the reference form keeps to the reference's entry points; the other
                    # also takes gate and up with the activation folded into their row ends)
                    pending, residual = dl.decode_layer(g, layer_weights, cache, pending, residual,
                                                        pending_norm, position, workspace, local,
                                                        attention_workspace,
                                                        fused_gate_up=attention_workspace is not None,
                                                        fused_input_norm=attention_workspace is not None)
                    pending_norm = layer_weights.post_feedforward_norm
                last["hidden"] = residual

            ms = time_graph(token, stream, max(5, steps // 2), max(2, warmup // 2))
            if not bool(torch.isfinite(last["hidden"]).all()):
                raise RuntimeError("the decode-layer chain produced a non-finite hidden state")
            per_layer_us = ms * 1e3 / layers
            entry = {
                "us_per_layer": round(per_layer_us, 2),
                "launches_per_layer": launches,
                "weight_GB/s": round(weight_bytes / ms / 1e6, 1),
                "frac_hbm": round((weight_bytes + cache_bytes) / ms / 1e6 / HBM_PEAK_GBS, 4)}
            if local:
                entry["tokens/s_at_48_layers_without_lm_head"] = round(1e6 / (48 * per_layer_us), 1)
                result[name] = entry
            else:
                result.setdefault("global_32768_keys", {})[name] = entry
        if local:
            # the verifier's block of 16 tokens through the same layers (batch forms of the
            # operators, causal block attention, no commit)
            rows = 16
            block = torch.from_numpy(kquant.synthetic_activations(42, rows, MODEL_DIM)).to(device)
            block_zeros = torch.zeros_like(block)
            block_workspace = tile_ops.small_batch_workspace(rows, FFN_DIM, device)
            # (the last form: the dual norms also hand their output to the projections behind
            # them in the small-batch workspace, nfn_mi355_dual_rms_add_capture_mmq_f16_float32_v1)
            # (and the one after: gate and up in the call that stores swiglu(gate, up),
            # nfn_mi355_k_quant_mmq_gate_up_swiglu_float32_v1)
            # (and last the exact verifier's family, every row in the one-row arithmetic bit for
            # bit: what the engine's speculative decode calls with exact_verifier_rows; then with
            # the norms handing the rows' records over,
            # nfn_mi355_dual_rms_add_capture_mmvq_rows_float32_v1)
            block_forms = [(name, workspace, False, False, "mmq") for name, workspace, _ in forms]
            block_forms.append((forms[-1][0] + "_norm_handoff", forms[-1][1], True, False, "mmq"))
            block_forms.append((forms[-1][0] + "_norm_handoff_gate_up_swiglu", forms[-1][1], True, True, "mmq"))
            block_forms.append((forms[-1][0] + "_exact_verifier_family", forms[-1][1], False, False, "mmvq"))
            block_forms.append((forms[-1][0] + "_exact_verifier_family_norm_handoff", forms[-1][1], True, False, "mmvq"))
            for name, attention_workspace, handoff, fused_gate_up, family in block_forms:
                def verify():
                    pending, residual, pending_norm = block, block_zeros, None
                    for layer_weights, cache in zip(weights, caches):
                        pending, residual, _, _ = dl.verify_layer(
                            g, layer_weights, cache, pending, residual, pending_norm, position,
                            block_workspace, True, attention_workspace, handoff, fused_gate_up, family)
                        pending_norm = layer_weights.post_feedforward_norm
                    last["hidden"] = residual

                ms = time_graph(verify, stream, max(5, steps // 2), max(2, warmup // 2))
                if not bool(torch.isfinite(last["hidden"]).all()):
                    raise RuntimeError("the verifier chain produced a non-finite hidden state")
                result.setdefault("verify_block_16_rows", {})[name] = {
                    "us_per_layer": round(ms * 1e3 / layers, 2),
                    "weight_GB/s": round(weight_bytes / ms / 1e6, 1)}
        del caches
    return result


def memory_rate_extra(device, stream, steps: int, warmup: int) -> dict:
    """What the vendor library's own streaming kernels reach on this GPU: a float sum (read
    only) and a copy (read + write) over buffers below and far above the 256 MB the memory-side
    cache holds, and this library's read-only probe kernel over the same buffers.  The
    comparators for every HBM-bound figure here, next to the published 8 TB/s."""
    import torch
    from neuralfn_amd import probes, tile_ops
    result = {"workload": "torch.sum / Tensor.copy_ / this library's read-only probe kernel over a "
                          "float32 buffer, TB/s of bytes moved"}
    steps, warmup = max(5, steps // 2), max(2, warmup // 2)
    for mib in (256, 2048):
        source = torch.empty(mib * (1 << 20) // 4, dtype=torch.float32, device=device).normal_()
        target = torch.empty_like(source)
        nbytes = source.numel() * 4
        read_ms = time_replays(lambda: source.sum(), steps, warmup)
        copy_ms = time_replays(lambda: target.copy_(source), steps, warmup)
        # this library's own read-only kernel (nfn_mi355_read_probe_v1: one workgroup per
        # compute unit streams its share in 16-byte pieces and stores nothing): what a kernel
        # of the decode kernels' shape can read at best
        sink = torch.zeros(1024, dtype=torch.int32, device=device)
        handle = int(torch.cuda.current_stream().cuda_stream)
        probe_ms = time_replays(lambda: tile_ops.check(probes.load().nfn_mi355_read_probe_v1(
            source.data_ptr(), nbytes, sink.data_ptr(), handle), "read probe"), steps, warmup)
        result[f"{mib}_MiB"] = {"sum_read_TB/s": round(nbytes / read_ms / 1e9, 2),
                                "copy_read_plus_write_TB/s": round(2 * nbytes / copy_ms / 1e9, 2),
                                "read_probe_TB/s": round(nbytes / probe_ms / 1e9, 2)}
        del source, target
    return result


def attention_extra(device, stream, steps: int, warmup: int) -> dict:
    """Attention alone at the workload's head geometry: the one-token call in the reference's
    form (one workgroup per query head, no workspace) and in the split form, over a local
    window and a long context, and the verifier's 16-row causal block."""
    import torch
    from neuralfn_amd import engine_ops
    query_heads, kv_heads, head_dim = ATTN_DIM // 128, KV_DIM // 128, 128
    scale = head_dim ** -0.5
    steps, warmup = max(5, steps // 2), max(2, warmup // 2)
    calls = 16  # per graph: a replay's own cost is not the call's

    def time_calls(call) -> float:
        def run():
            for _ in range(calls):
                call()
        return time_graph(run, stream, steps, warmup) / calls

    result = {"workload": f"{query_heads} query heads over {kv_heads} key/value heads of "
                          f"{head_dim}, bf16 cache, {calls} calls a HIP-graph replay; GB/s = "
                          "cache bytes of the attended keys / time"}
    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim, device)
    for keys in (2048, 32768):
        query = torch.randn(query_heads, head_dim, device=device)
        key = torch.randn(kv_heads, head_dim, device=device)
        value = torch.randn(kv_heads, head_dim, device=device)
        key_cache = torch.randn(keys, kv_heads * head_dim, device=device).to(torch.bfloat16)
        value_cache = torch.randn(keys, kv_heads * head_dim, device=device).to(torch.bfloat16)
        out = torch.empty_like(query)
        position = 2 * keys - 1  # the ring is full and has wrapped once
        first = position - keys + 1
        cache_bytes = 2 * keys * kv_heads * head_dim * 2
        entry = {}
        for name, lent in (("reference_form", None), ("split_form", workspace)):
            ms = time_calls(lambda: engine_ops.gqa_decode(query, key, value, key_cache, value_cache,
                                                          position, first, scale, out=out,
                                                          workspace=lent))
            entry[name] = {"us": round(ms * 1e3, 2), "GB/s": round(cache_bytes / ms / 1e6, 1)}
        result[f"one_token_{keys}_keys"] = entry
    rows, window = 16, 2048
    query = torch.randn(rows, query_heads, head_dim, device=device)
    block_key = torch.randn(rows, kv_heads, head_dim, device=device)
    block_value = torch.randn(rows, kv_heads, head_dim, device=device)
    key_cache = torch.randn(window, kv_heads * head_dim, device=device).to(torch.bfloat16)
    value_cache = torch.randn(window, kv_heads * head_dim, device=device).to(torch.bfloat16)
    out = torch.empty_like(query)
    entry = {}
    for name, lent in (("reference_form", None), ("split_form", workspace)):
        ms = time_calls(lambda: engine_ops.block_attention(query, block_key, block_value, key_cache,
                                                           value_cache, 4000, window, scale, True,
                                                           out=out, workspace=lent))
        entry[name] = {"us": round(ms * 1e3, 2)}
    result[f"causal_block_{rows}_rows_{window}_window"] = entry
    return result


def mixed_profile_extra(device, stream, steps: int, warmup: int) -> dict:
    """Four layers of attention and FFN projections with per-tensor formats drawn by seed
    from {Q4_K, Q5_K, Q6_K, Q8_0} (V, O and down at least Q5_K), at one row (decode)
    and 1024 rows (prefill): per-format dispatch through the same entry points."""
    import random
    import torch
    from neuralfn_amd import kquant, tile_ops

    draw = random.Random(4)
    every = [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0]
    wide = [kquant.Q5_K, kquant.Q6_K, kquant.Q8_0]
    shapes = {"q": (ATTN_DIM, MODEL_DIM), "k": (KV_DIM, MODEL_DIM), "v": (KV_DIM, MODEL_DIM),
              "o": (MODEL_DIM, ATTN_DIM), "gate": (FFN_DIM, MODEL_DIM), "up": (FFN_DIM, MODEL_DIM),
              "down": (MODEL_DIM, FFN_DIM)}
    layers, formats = [], []
    for layer in range(4):
        chosen = {name: draw.choice(wide if name in ("v", "o", "down") else every) for name in shapes}
        formats.append("/".join(kquant.NAMES[chosen[name]] for name in shapes))
        layers.append({name: random_packed_on_device(chosen[name], *shapes[name], device,
                                                     100 + 10 * layer + index)
                       for index, name in enumerate(shapes)})
    weight_bytes = sum(weight.nbytes for layer in layers for weight in layer.values())
    flops_per_row = sum(2.0 * w.input_dim * w.output_dim for layer in layers for w in layer.values())
    inputs = {MODEL_DIM: kquant.synthetic_activations(41, 1024, MODEL_DIM),
              ATTN_DIM: kquant.synthetic_activations(42, 1024, ATTN_DIM),
              FFN_DIM: kquant.synthetic_activations(43, 1024, FFN_DIM)}
    result = {"workload": "4 layers of Q/K/V (grouped), O, gate+up (grouped), down with seeded per-tensor formats",
              "formats_q_k_v_o_gate_up_down": formats}

    # decode: one row, the small-batch entry point, grouped where the engine groups
    x = {dim: torch.from_numpy(values[:1].copy()).to(device) for dim, values in inputs.items()}
    outs = [{name: torch.empty((1, w.output_dim), dtype=torch.float32, device=device)
             for name, w in layer.items()} for layer in layers]
    workspace = tile_ops.small_batch_workspace(1, FFN_DIM)

    def decode():
        for layer, out in zip(layers, outs):
            tile_ops.multi_linear([layer["q"], layer["k"], layer["v"]], x[MODEL_DIM], workspace,
                                  outputs=[out["q"], out["k"], out["v"]])
            tile_ops.multi_linear([layer["o"]], x[ATTN_DIM], workspace, outputs=[out["o"]])
            tile_ops.multi_linear([layer["gate"], layer["up"]], x[MODEL_DIM], workspace,
                                  outputs=[out["gate"], out["up"]])
            tile_ops.multi_linear([layer["down"]], x[FFN_DIM], workspace, outputs=[out["down"]])

    ms = time_graph(decode, stream, steps, warmup)
    result["decode_rows1"] = {"ms": round(ms, 4), "GB/s": round(weight_bytes / ms / 1e6, 1),
                              "frac_hbm": round(weight_bytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                              "tokens/s": round(1e3 / ms, 1)}

    # a verifier block: 16 rows through the same calls, both small-batch families
    # (mmvq: every row carries the one-row call's bits)
    x16 = {dim: torch.from_numpy(values[:16].copy()).to(device) for dim, values in inputs.items()}
    outs16 = [{name: torch.empty((16, w.output_dim), dtype=torch.float32, device=device)
               for name, w in layer.items()} for layer in layers]
    workspace16 = tile_ops.small_batch_workspace(16, FFN_DIM)
    for family, key in (("mmq", "verifier_rows16"), ("mmvq", "verifier_rows16_exact_verifier_family")):
        def verify(family=family):
            for layer, out in zip(layers, outs16):
                tile_ops.multi_linear([layer["q"], layer["k"], layer["v"]], x16[MODEL_DIM], workspace16,
                                      outputs=[out["q"], out["k"], out["v"]], family=family)
                tile_ops.multi_linear([layer["o"]], x16[ATTN_DIM], workspace16, outputs=[out["o"]],
                                      family=family)
                tile_ops.multi_linear([layer["gate"], layer["up"]], x16[MODEL_DIM], workspace16,
                                      outputs=[out["gate"], out["up"]], family=family)
                tile_ops.multi_linear([layer["down"]], x16[FFN_DIM], workspace16, outputs=[out["down"]],
                                      family=family)
        ms = time_graph(verify, stream, steps, warmup)
        result[key] = {"ms": round(ms, 4), "GB/s": round(weight_bytes / ms / 1e6, 1),
                       "frac_hbm": round(weight_bytes / ms / 1e6 / HBM_PEAK_GBS, 4),
                       "tokens/s": round(16e3 / ms, 1)}

    # prefill: 1024 rows through the dequant-GEMM
    rows = 1024
    xs = {dim: torch.from_numpy(values).to(device) for dim, values in inputs.items()}
    big = {name: torch.empty((rows, shape[0]), dtype=torch.float32, device=device)
           for name, shape in shapes.items()}
    nbytes = max(tile_ops.load().nfn_mi355_k_quant_gemm_workspace_bytes_v1(
        rows, shape[1], shape[0], tile_ops.GEMM_F16) for shape in shapes.values())
    gemm_workspace = torch.empty(nbytes, dtype=torch.uint8, device=device)

    def prefill():
        # grouped where the engine groups: projections of one input convert it once
        for layer in layers:
            tile_ops.gemm_multi([layer["q"], layer["k"], layer["v"]], xs[MODEL_DIM], tile_ops.GEMM_F16,
                                gemm_workspace, [big["q"], big["k"], big["v"]])
            tile_ops.gemm(layer["o"], xs[ATTN_DIM], tile_ops.GEMM_F16, gemm_workspace, big["o"])
            tile_ops.gemm_multi([layer["gate"], layer["up"]], xs[MODEL_DIM], tile_ops.GEMM_F16,
                                gemm_workspace, [big["gate"], big["up"]])
            tile_ops.gemm(layer["down"], xs[FFN_DIM], tile_ops.GEMM_F16, gemm_workspace, big["down"])

    ms = time_graph(prefill, stream, max(5, steps // 2), max(2, warmup // 2))
    tflops = rows * flops_per_row / ms / 1e9
    result["prefill_rows1024"] = {"ms": round(ms, 4), "TFLOP/s": round(tflops, 1),
                                  "frac_mfma": round(tflops / MFMA_PEAK_TFLOPS["f16"], 4),
                                  "tokens/s": round(rows / ms * 1e3, 1)}
    return result


def main() -> int:
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path; run with --gpus 1",
              file=sys.stderr)
        return 2
    if args.rows not in (1, 2, 4, 8, 16):
        print("--rows must be one of 1, 2, 4, 8, 16", file=sys.stderr)
        return 2
    import torch
    from neuralfn_amd import tile_ops

    tile_ops.load()
    device = torch.device("cuda:0")
    torch.cuda.set_device(device)

    began = time.perf_counter()
    layers, host_layers = make_layers(args.layers, device)
    setup_seconds = time.perf_counter() - began
    step = DecodeStep(layers, args.rows, device)

    if args.traffic_probe:
        # a copy kernel of known size calibrates the byte counters, then the
        # launches of one step follow as separate dispatches
        source = torch.empty(256 << 20, dtype=torch.uint8, device=device)
        target = torch.empty_like(source)
        source.fill_(1)
        torch.cuda.synchronize()
        target.copy_(source)
        torch.cuda.synchronize()
        step.enqueue(int(torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        print(f"traffic probe: copy of {source.numel()} bytes, then {step.launches_per_step} "
              f"launches of {layer_algorithmic_bytes(args.rows) // 2} bytes on average",
              file=sys.stderr)
        return 0

    stream = torch.cuda.Stream()
    graph = None
    with torch.cuda.stream(stream):
        step.enqueue(int(stream.cuda_stream))  # eager warm-up, loads code objects
        stream.synchronize()
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                step.enqueue(int(torch.cuda.current_stream().cuda_stream))

        def run():
            if graph is not None:
                graph.replay()
            else:
                step.enqueue(int(stream.cuda_stream))

        ms_per_step = time_replays(run, args.steps, args.warmup)
        samples = max(30, args.steps)
        per_launch = {"unit": "us per launch"}
        if graph is not None:
            per_launch["graph_replay"] = step_distribution(run, samples, 5, step.launches_per_step)
        per_launch["eager"] = step_distribution(
            lambda: step.enqueue(int(stream.cuda_stream)), samples, 5, step.launches_per_step)

    bytes_per_step = args.layers * layer_algorithmic_bytes(args.rows)
    value = bytes_per_step / ms_per_step / 1e6  # GB/s
    launches = step.launches_per_step
    record = {
        "metric": "Q4_K decode GEMV GB/s",
        "value": round(value, 2),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic (seeded N(0,0.02) weights quantized to Q4_K; bf16-rounded N(0,1) activations)",
        "config": {
            "workload": f"decode attention projections Q/K/V (grouped) + O, Q4_K, "
                        f"{args.layers} layers, rows={args.rows}",
            "rows": args.rows,
            "layers": args.layers,
            "launches_per_step": launches,
            "hip_graph": graph is not None,
            "setup_seconds": round(setup_seconds, 1),
        },
        "tokens_per_s": round(args.rows / ms_per_step * 1e3, 2),
        "frac_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "roofline": {
            "bound": "hbm",
            "achieved": round(value, 2),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(value / HBM_PEAK_GBS, 4),
            "traffic": MEASURED_TRAFFIC_BYTES_PER_LAUNCH.get(args.rows),
            "traffic_source": "stored result of a counter run of this workload (FETCH_SIZE + "
                              "WRITE_SIZE, see profiles/); not measured in this run",
            "kernel": "decode GEMV (Q/K/V grouped launch and O launch, averaged)",
            "bytes_per_launch": bytes_per_step // launches,
            "us_per_launch": round(ms_per_step * 1e3 / launches, 3),
        },
    }
    record["per_launch_distribution"] = per_launch
    if not args.no_extras:
        try:
            with torch.cuda.stream(stream):
                record["decode_batches"] = decode_batch_extra(layers, device, stream, args.steps,
                                                              args.warmup, args.rows)
                record["lm_head"] = lm_head_extra(device, stream, args.steps, args.warmup)
                record["prefill"] = prefill_extra(device, stream, args.steps, args.warmup)
                record["mixed_profile"] = mixed_profile_extra(device, stream, args.steps, args.warmup)
                record["attention"] = attention_extra(device, stream, args.steps, args.warmup)
                record["library_memory_rate"] = memory_rate_extra(device, stream, args.steps,
                                                                  args.warmup)
                record["decode_layer"] = decode_layer_extra(device, stream, args.steps, args.warmup)
                record["launch_floor"] = launch_floor_extra(layers, device, stream, args.steps,
                                                            args.warmup)
                record["large_projection_rows1"] = large_projection_extra(device, stream, args.steps,
                                                                          args.warmup)
                record["published_shapes"] = published_shapes_extra(device, stream, args.steps,
                                                                    args.warmup)
        except Exception as error:  # the headline is still printed; the exit code says it failed
            record["extras_error"] = repr(error)
    if not args.no_cpu_baseline:
        record["cpu_baseline"] = cpu_baseline(host_layers, args.rows)
        record["cpu_baselines_other_configs"] = cpu_baselines_other_configs(host_layers)
    print(json.dumps(record))
    return 1 if "extras_error" in record else 0


if __name__ == "__main__":
    sys.exit(main())
