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


def random_bytes(rng, encoding, out_dim, in_dim):
    """Packed rows of random bytes with the fp16 scales kept finite and small."""
    elements, nbytes = kquant.BLOCKS[encoding]
    blocks = rng.integers(0, 256, (out_dim * in_dim // elements, nbytes), dtype=np.uint8)
    offsets = {kquant.Q4_K: (0, 2), kquant.Q5_K: (0, 2), kquant.Q6_K: (208,), kquant.Q8_0: (0,)}
    for offset in offsets[encoding]:
        blocks[:, offset + 1] = (blocks[:, offset + 1] & 0x83) | 0x24
    return blocks.reshape(-1)


@pytest.mark.parametrize("seed", range(16))
def test_small_batch_model_sized_case(cuda, oracle, seed):
    """The sweep above keeps its outputs narrow; a wave's or a workgroup's share of the rows, and
    with it where a row starts inside a kernel's pass, only changes with thousands of rows.
    Model-sized projections, random formats, row counts and grouping: against the oracle on a
    sample of the rows, verifier rows against the one-row call on every row, the one-row call
    of the group against the single-projection entry point, and the prequantized call."""
    rng = np.random.default_rng(5000 + seed)
    in_dim = int(rng.choice([4096, 6656, 8192, 13312, 16384]))
    rows = int(rng.integers(1, 17))
    count = int(rng.integers(1, 4))
    formats = [int(rng.choice(FORMATS)) for _ in range(count)]
    out_dims = [int(rng.choice([256, 2100, 3000, 4608, 6656, 9000])) for _ in range(count)]
    family = "mmvq" if seed % 4 else "mmq"
    packed = [random_bytes(rng, f, n, in_dim) for f, n in zip(formats, out_dims)]
    weights = [tile_ops.PackedWeight.from_numpy(f, p, n, in_dim) for f, p, n in zip(formats, packed, out_dims)]
    x = rng.standard_normal((rows, in_dim)).astype(np.float32)
    device_x = to_device(x, cuda)
    workspace = tile_ops.small_batch_workspace(rows, in_dim)
    outputs = tile_ops.multi_linear(weights, device_x, workspace, family=family)
    label = f"K {in_dim} rows {rows} {family} {list(zip(formats, out_dims))}"
    for f, p, n, y in zip(formats, packed, out_dims, outputs):
        picked = np.unique(np.concatenate([np.arange(0, n, 97), [n - 1]]))
        sample = p.reshape(n, -1)[picked].reshape(-1)
        expected = oracle.linear(f, sample, picked.size, in_dim, x)
        assert normalised_error(y.cpu().numpy()[:, picked], expected) <= TOLERANCE, label
    one = tile_ops.small_batch_workspace(1, in_dim)
    if family == "mmvq":
        for row in range(rows):
            single = tile_ops.multi_linear(weights, device_x[row:row + 1], one, family="mmvq")
            for a, b in zip(outputs, single):
                assert np.array_equal(bits(a)[row], bits(b)[0]), f"{label} row {row}"
        reused = tile_ops.multi_linear_prequantized(weights, rows, workspace)
        for a, b in zip(outputs, reused):
            assert np.array_equal(bits(a), bits(b)), f"{label} prequantized"
    first_row = tile_ops.multi_linear(weights, device_x[:1], one, family=family)
    for weight, grouped in zip(weights, first_row):
        direct = tile_ops.mmvq_linear(weight, device_x[:1], one)
        assert np.array_equal(bits(direct), bits(grouped)), f"{label} single projection"


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
    # the generic linear has no workspace: exact float arithmetic at any row count
    z = tile_ops.linear(weight, to_device(x, cuda)).cpu().numpy()
    for row in range(0, rows, 7):
        assert normalised_error(z[row], expected[row]) <= 1e-5, f"{label} row {row} (generic linear)"


# ---- attention ---------------------------------------------------------------------------------------

def _bf16(oracle, rng, shape):
    return oracle.to_bf16(rng.standard_normal(shape).astype(np.float32))


def _bf16_tensor(bits_, device):
    return to_device(np.ascontiguousarray(bits_, dtype=np.uint16).view(np.int16), device)


@pytest.mark.parametrize("seed", range(24))
def test_attention_random_case(cuda, oracle, seed):
    """One-token attention (both forms) and block attention (both modes) on drawn geometries: head sizes
    on and off the vector kernel, padded cache rows, rings smaller than a tile, windows that cut the
    context or exceed it, positions before and after the ring wraps."""
    from neuralfn_amd import engine_ops
    rng = np.random.default_rng(3000 + seed)
    head_dim = int(rng.choice([8, 32, 50, 64, 96, 128, 128, 256]))
    kv_heads = int(rng.choice([1, 2, 4]))
    query_heads = kv_heads * int(rng.choice([1, 2, 4, 16]))
    capacity = int(rng.choice([16, 63, 64, 100, 512, 2048]))
    padding = int(rng.choice([0, 0, 8, 6]))
    stride = kv_heads * head_dim + padding
    position = int(rng.integers(0, 3 * capacity))
    window = int(rng.integers(1, capacity + 1))
    first = max(0, position - window + 1)
    scale = float(head_dim ** -0.5)
    key_cache, value_cache = _bf16(oracle, rng, (capacity, stride)), _bf16(oracle, rng, (capacity, stride))
    device_keys, device_values = _bf16_tensor(key_cache, cuda), _bf16_tensor(value_cache, cuda)
    label = (f"heads {query_heads}/{kv_heads} x {head_dim}, ring {capacity} x {stride}, position {position}, "
             f"window {window}")

    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    expected = oracle.gqa_decode(query, key, value, key_cache, value_cache, position, first, scale)
    arguments = (to_device(query, cuda), to_device(key, cuda), to_device(value, cuda), device_keys,
                 device_values, position, first, scale)
    plain = engine_ops.gqa_decode(*arguments).cpu().numpy()
    assert np.abs(plain - expected).max() <= 4e-6, label
    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim)
    workspace.fill_(0xFF)
    split = engine_ops.gqa_decode(*arguments, workspace=workspace).cpu().numpy()
    assert np.abs(split - expected).max() <= 4e-6, label + " (split form)"
    # the fused call with the position on the device and the split form (no norm weights):
    # per-head norm and rope of query and key, then the same attention, then the commit
    device_position = to_device(np.array([position], dtype=np.int64), cuda)
    keys_copy, values_copy = device_keys.clone(), device_values.clone()
    fused = engine_ops.fused_decode_attention(
        to_device(query, cuda), to_device(key, cuda), to_device(value, cuda), keys_copy, values_copy,
        3, 1, scale, None, None, 1e-5, 1.0, 500000.0, engine_ops.ROPE_HALF_SPLIT, True,
        device_position=device_position, sliding_window=window, workspace=workspace).cpu().numpy()
    normalized_query = oracle.rope(np.stack([oracle.rms_norm(row, None, False, 1e-5) for row in query]),
                                   position, 500000.0, False)
    normalized_key = oracle.rope(np.stack([oracle.rms_norm(row, None, False, 1e-5) for row in key]),
                                 position, 500000.0, False)
    expected_fused = oracle.gqa_decode(normalized_query, normalized_key, value, key_cache, value_cache,
                                       position, first, scale)
    assert np.abs(fused - expected_fused).max() <= 6e-6, label + " (fused, device position, split)"
    # the committed key row: the normalised, rotated key, a bf16 rounding step apart at most
    committed = oracle.bf16_to_float(
        keys_copy.cpu().numpy().view(np.uint16)[position % capacity, :kv_heads * head_dim])
    assert np.abs(committed - normalized_key.reshape(-1)).max() <= \
        2.0 ** -7 * np.abs(normalized_key).max(), label

    rows = int(rng.integers(1, 9))
    block_rows = rows + int(rng.integers(0, 5))
    context = position
    block_query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    for causal in (True, False):
        expected = oracle.block_attention(block_query, block_key, block_value, key_cache, value_cache,
                                          context, window, scale, causal)
        actual = engine_ops.block_attention(
            to_device(block_query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
            device_keys, device_values, context, window, scale, causal).cpu().numpy()
        assert np.abs(actual - expected).max() <= 4e-6, f"{label}, block {rows}/{block_rows}, causal {causal}"


@pytest.mark.parametrize("seed", range(24))
def test_matrix_core_attention_random_case(cuda, oracle, seed):
    """Geometries of the matrix-core kernel (head size 128, four or more query heads per key/value
    head, also more than 16 and not a multiple of 16): the split one-token form with the position on
    the host and on the device, and blocks large enough to take that kernel, unsplit and split, in
    both modes.  Padded cache rows, rings that wrapped, windows that cut the context, short rings."""
    from neuralfn_amd import engine_ops
    rng = np.random.default_rng(5000 + seed)
    head_dim = 128
    kv_heads = int(rng.choice([1, 2, 3, 8]))
    per_kv = int(rng.choice([4, 5, 16, 17, 20, 32]))
    query_heads = kv_heads * per_kv
    capacity = int(rng.choice([64, 100, 130, 512, 2048, 5000]))
    padding = int(rng.choice([0, 0, 8, 24]))
    stride = kv_heads * head_dim + padding
    position = int(rng.integers(0, 3 * capacity))
    window = int(rng.integers(1, capacity + 1))
    first = max(0, position - window + 1)
    scale = float(head_dim ** -0.5)
    key_cache, value_cache = _bf16(oracle, rng, (capacity, stride)), _bf16(oracle, rng, (capacity, stride))
    device_keys, device_values = _bf16_tensor(key_cache, cuda), _bf16_tensor(value_cache, cuda)
    label = (f"heads {query_heads}/{kv_heads}, ring {capacity} x {stride}, position {position}, "
             f"window {window}")

    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    expected = oracle.gqa_decode(query, key, value, key_cache, value_cache, position, first, scale)
    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim)
    workspace.fill_(0xFF)
    split = engine_ops.gqa_decode(to_device(query, cuda), to_device(key, cuda), to_device(value, cuda),
                                  device_keys, device_values, position, first, scale,
                                  workspace=workspace).cpu().numpy()
    assert np.abs(split - expected).max() <= 4e-6, label + " (split form)"
    # position on the device, no norm weights and no rope: the fused call is attention + commit
    device_position = to_device(np.array([position], dtype=np.int64), cuda)
    keys_copy, values_copy = device_keys.clone(), device_values.clone()
    fused = engine_ops.fused_decode_attention(
        to_device(query, cuda), to_device(key, cuda), to_device(value, cuda), keys_copy, values_copy,
        3, 1, scale, None, None, 1e-5, 1.0, 500000.0, engine_ops.ROPE_INTERLEAVED, True,
        device_position=device_position, sliding_window=window, workspace=workspace)
    # that call normalises query and key per head first (no weights): compare with the oracle on those
    normalized_query = oracle.rope(np.stack([oracle.rms_norm(row, None, False, 1e-5) for row in query]),
                                   position, 500000.0, True)
    normalized_key = oracle.rope(np.stack([oracle.rms_norm(row, None, False, 1e-5) for row in key]),
                                 position, 500000.0, True)
    expected_fused = oracle.gqa_decode(normalized_query, normalized_key, value, key_cache, value_cache,
                                       position, first, scale)
    assert np.abs(fused.cpu().numpy() - expected_fused).max() <= 6e-6, label + " (fused, device position)"

    rows = int(rng.integers(1, 17))
    # more rows x heads than compute units where 64 block rows allow it: the matrix cores
    rows = min(max(rows, 256 // query_heads + 1), 62)
    block_rows = rows + int(rng.integers(0, 3))
    block_query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    for causal in (True, False):
        expected = oracle.block_attention(block_query, block_key, block_value, key_cache, value_cache,
                                          position, window, scale, causal)
        arguments = (to_device(block_query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
                     device_keys, device_values, position, window, scale, causal)
        for lent in (None, workspace):
            actual = engine_ops.block_attention(*arguments, workspace=lent).cpu().numpy()
            assert np.abs(actual - expected).max() <= 4e-6, \
                f"{label}, block {rows}/{block_rows}, causal {causal}, split {lent is not None}"


@pytest.mark.parametrize("seed", range(24))
def test_lm_head_block_random_case(cuda, seed):
    """The fused lm_head argmax at 5..16 rows against the logits of the small-batch call, which runs
    the same kernel and stores them: the value must be the row's largest logit bit for bit and the
    index the first column that holds it.  Widths off the 16-row tile, K from one block up, ties
    planted across tiles and workgroups, a NaN logit, one all-NaN row."""
    import torch
    rng = np.random.default_rng(7000 + seed)
    encoding = int(rng.choice(FORMATS))
    in_dim = 256 * int(rng.choice([1, 2, 5, 8, 26]))
    out_dim = int(rng.choice([1, 15, 16, 17, 255, 1000, 4097, 8200, 20011]))
    rows = int(rng.integers(5, 17))
    w = (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32)
    if out_dim > 40:  # equal rows of weights give equal logits: the first of them must win
        source = int(rng.integers(0, out_dim))
        for twin in rng.integers(0, out_dim, size=3):
            w[int(twin)] = w[source]
    weight = tile_ops.PackedWeight.from_numpy(encoding, kquant.quantize(encoding, w), out_dim, in_dim)
    x = rng.standard_normal((rows, in_dim)).astype(np.float32)
    x[0] *= 1e-4
    x[rows - 1] *= 3e3
    if seed % 4 == 0:
        x[1, 3] = np.nan   # every logit of this row is NaN
    device_x = to_device(x, cuda)
    workspace = tile_ops.small_batch_workspace(rows, in_dim)
    (logits,) = tile_ops.multi_linear([weight], device_x, workspace)
    indices, maxima = tile_ops.lm_head_argmax(weight, device_x)
    logits = logits.cpu().numpy()
    for row in range(rows):
        values = logits[row]
        if np.all(np.isnan(values)):
            assert int(indices[row]) == 0 and float(maxima[row]) == -np.inf
            continue
        best = np.nanmax(values)
        assert np.float32(maxima[row].item()).view(np.uint32) == np.float32(best).view(np.uint32), (row, seed)
        assert int(indices[row]) == int(np.flatnonzero(values == best)[0]), (row, seed)
