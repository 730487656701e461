"""Seeded sweep over the small-batch and GEMM entry points: shapes, formats, projection counts and
prologues drawn at random, each checked against the CPU oracle at the build's tolerance and against the
bit-level contracts between entry points (one row: `mmq` == `mmvq_linear`; verifier rows == row by row).

The fixed cases of test_gpu_parity.py follow the reference probe; this sweep is there for what a fixed list
misses: output widths that are not a multiple of any tile, K with fewer blocks than a workgroup has waves,
mixed formats in one call, every row count from 1 to 16.
"""
import numpy as np
import pytest

from neuralfn_amd import kquant, tile_ops

pytestmark = pytest.mark.gpu

TOLERANCE = 2e-3
FORMATS = [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0]


def to_device(array, device):
    import torch
    return torch.from_numpy(np.ascontiguousarray(array)).to(device)


def normalised_error(actual, expected):
    scale = max(float(np.max(np.abs(expected))), 1e-30)
    return float(np.max(np.abs(actual.astype(np.float64) - expected.astype(np.float64))) / scale)


def bits(tensor):
    return tensor.cpu().numpy().view(np.uint32)


def draw_case(seed):
    rng = np.random.default_rng(seed)
    in_dim = 256 * int(rng.choice([1, 2, 3, 4, 5, 8, 13, 16, 26]))
    rows = int(rng.integers(1, 17))
    count = int(rng.integers(1, 5))
    formats = [int(rng.choice(FORMATS)) for _ in range(count)]
    out_dims = [int(rng.choice([1, 7, 31, 32, 33, 64, 97, 129, 255, 300])) for _ in range(count)]
    prologue = str(rng.choice(["plain", "plain", "gated", "swiglu"]))
    family = str(rng.choice(["mmq", "mmvq"]))
    return rng, in_dim, rows, formats, out_dims, prologue, family


@pytest.mark.parametrize("seed", range(48))
def test_small_batch_random_case(cuda, oracle, seed):
    rng, in_dim, rows, formats, out_dims, prologue, family = draw_case(1000 + seed)
    packed = [kquant.quantize(f, (rng.standard_normal((n, in_dim)) * 0.05).astype(np.float32))
              for f, n in zip(formats, out_dims)]
    weights = [tile_ops.PackedWeight.from_numpy(f, p, n, in_dim)
               for f, p, n in zip(formats, packed, out_dims)]
    x = rng.standard_normal((rows, in_dim)).astype(np.float32)
    second = rng.standard_normal((rows, in_dim)).astype(np.float32)
    if prologue == "gated":
        effective = oracle.sigmoid_gate(x, second)
    elif prologue == "swiglu":
        effective = oracle.swiglu(x, second)
    else:
        effective = x
    workspace = tile_ops.small_batch_workspace(rows, in_dim)
    device_x, device_second = to_device(x, cuda), to_device(second, cuda)
    outputs = tile_ops.multi_linear(weights, device_x, workspace,
                                    second=None if prologue == "plain" else device_second,
                                    family=family, prologue=prologue)
    label = f"K {in_dim} rows {rows} {family}/{prologue} {list(zip(formats, out_dims))}"
    for f, p, n, y in zip(formats, packed, out_dims, outputs):
        expected = oracle.linear(f, p, n, in_dim, effective)
        assert normalised_error(y.cpu().numpy(), expected) <= TOLERANCE, label
    # a second call gives the same bits
    again = tile_ops.multi_linear(weights, device_x, workspace,
                                  second=None if prologue == "plain" else device_second,
                                  family=family, prologue=prologue)
    for a, b in zip(outputs, again):
        assert np.array_equal(bits(a), bits(b)), label
    if family == "mmvq":
        # every row of a verifier call is the one-row call on that row, bit for bit
        one = tile_ops.small_batch_workspace(1, in_dim)
        for row in sorted({0, rows - 1, rows // 2}):
            single = tile_ops.multi_linear(
                weights, device_x[row:row + 1], one,
                second=None if prologue == "plain" else device_second[row:row + 1],
                family="mmvq", prologue=prologue)
            for a, b in zip(outputs, single):
                assert np.array_equal(bits(a)[row], bits(b)[0]), f"{label} row {row}"
    if rows == 1 and prologue == "plain":
        direct = tile_ops.mmvq_linear(weights[0], device_x, workspace)
        assert np.array_equal(bits(direct), bits(outputs[0])), label


@pytest.mark.parametrize("seed", range(16))
def test_gemm_random_case(cuda, oracle, seed):
    rng = np.random.default_rng(2000 + seed)
    in_dim = 256 * int(rng.choice([1, 2, 3, 5, 8, 12, 16]))
    rows = int(rng.choice([17, 31, 64, 100, 129, 255, 256, 300, 513]))
    out_dim = int(rng.choice([1, 17, 127, 128, 129, 200, 384, 500]))
    encoding = int(rng.choice(FORMATS))
    packed = kquant.quantize(encoding, (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32))
    weight = tile_ops.PackedWeight.from_numpy(encoding, packed, out_dim, in_dim)
    x = (rng.standard_normal((rows, in_dim)) * 10.0 ** rng.integers(-3, 4)).astype(np.float32)
    y = tile_ops.gemm(weight, to_device(x, cuda)).cpu().numpy()
    expected = oracle.linear(encoding, packed, out_dim, in_dim, x)
    label = f"M {rows} N {out_dim} K {in_dim} format {encoding}"
    assert normalised_error(y, expected) <= TOLERANCE, label
    if out_dim >= 127:
        # every row has its own scale on the way into fp16: the bound holds row by row
        # (a row of a few outputs can cancel to nearly nothing, so only wide rows are asked)
        for row in range(rows):
            assert normalised_error(y[row], expected[row]) <= TOLERANCE, f"{label} row {row}"
    # the generic linear has no workspace and stays on the float kernel at any row count
    z = tile_ops.linear(weight, to_device(x, cuda)).cpu().numpy()
    for row in range(0, rows, 7):
        assert normalised_error(z[row], expected[row]) <= 1e-5, f"{label} row {row} (generic linear)"
