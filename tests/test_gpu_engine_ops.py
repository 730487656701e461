"""The decode loop's operators around the packed linears, through the C ABI, against the oracle.

Cases and tolerances follow the reference's device probe
(tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:114-175 embedding, 417-458 rope,
2366-2512 one-token attention and cache commit, 2515-2745 block attention):
rope within 2e-4, one-token attention within 4e-4, block attention within 5e-4
of the double-precision formula; bf16 cache rows exact; a causal block equal
bit for bit to token-at-a-time decode.  This build's results sit well inside
those bounds and the assertions below say by how much.
"""
import ctypes

import numpy as np
import pytest

from neuralfn_amd import engine_ops, kquant, tile_ops

pytestmark = pytest.mark.gpu


def torch_():
    import torch
    return torch


def to_device(array, device):
    return torch_().from_numpy(np.ascontiguousarray(array)).to(device)


def bf16_tensor(bits, device):
    """uint16 bit patterns as an int16 device tensor (torch has no uint16 arithmetic; only the bytes matter)."""
    return to_device(np.ascontiguousarray(bits, dtype=np.uint16).view(np.int16), device)


def bits_of(tensor):
    return tensor.cpu().numpy().view(np.uint16)


def patterned(first, second, modulus, divisor):
    """patterned_value of the reference probe (:622-626); all operands are non-negative."""
    first, second = np.asarray(first, dtype=np.int64), np.asarray(second, dtype=np.int64)
    return ((first * 17 + second * 13) % modulus - modulus // 2).astype(np.float32) / np.float32(divisor)


def assert_bits_equal(a, b, label=""):
    a = a.detach().cpu().numpy() if hasattr(a, "detach") else a
    b = b.detach().cpu().numpy() if hasattr(b, "detach") else b
    assert a.shape == b.shape, label
    mismatch = np.flatnonzero(a.reshape(-1).view(np.uint32) != b.reshape(-1).view(np.uint32))
    assert mismatch.size == 0, f"{label}: {mismatch.size} values differ, first at {mismatch[:4]}"


def random_packed(encoding, out_dim, in_dim, seed):
    rng = np.random.default_rng(seed)
    elements, nbytes = kquant.BLOCKS[encoding]
    blocks = rng.integers(0, 256, (out_dim * in_dim // elements, nbytes), dtype=np.uint8)
    offsets = {kquant.Q4_K: (0, 2), kquant.Q5_K: (0, 2), kquant.Q6_K: (208,), kquant.Q8_0: (0,)}
    for offset in offsets[encoding]:
        blocks[:, offset + 1] = (blocks[:, offset + 1] & 0x83) | 0x24
    return blocks.reshape(-1)


# ---- embedding -------------------------------------------------------------------

@pytest.mark.parametrize("encoding", [kquant.Q4_K, kquant.Q5_K, kquant.Q6_K, kquant.Q8_0,
                                      kquant.BF16, kquant.F32])
def test_embedding_rows_are_the_dequantized_rows(cuda, oracle, encoding):
    vocabulary, width = 53, 1024
    if encoding in (kquant.F32, kquant.BF16):
        packed = kquant.quantize(encoding, kquant.synthetic_weights(5, vocabulary, width))
    else:
        packed = random_packed(encoding, vocabulary, width, 40 + encoding)
    table = tile_ops.PackedWeight.from_numpy(encoding, packed, vocabulary, width)
    expected = oracle.dequantize(encoding, packed, vocabulary, width)
    assert_bits_equal(engine_ops.embedding(table, 17), expected[17], "host token")
    token = to_device(np.array([52], dtype=np.int64), cuda)
    assert_bits_equal(engine_ops.embedding(table, token), expected[52], "device token")
    tokens = np.array([3, 52, 0, 3, 29], dtype=np.int32)
    assert_bits_equal(engine_ops.embedding(table, to_device(tokens, cuda)), expected[tokens], "batch")


def test_embedding_refuses_or_zeroes_unknown_tokens(cuda):
    vocabulary, width = 8, 256
    packed = random_packed(kquant.Q4_K, vocabulary, width, 3)
    table = tile_ops.PackedWeight.from_numpy(kquant.Q4_K, packed, vocabulary, width)
    lib = tile_ops.load()
    descriptor = table.descriptor(0)
    out = torch_().full((2, width), 7.0, dtype=torch_().float32, device=cuda)
    for token in (-1, vocabulary):
        assert lib.nfn_native_tile_glimmer_embedding_gather_float32_v1(
            ctypes.byref(descriptor), token, out.data_ptr()) == 1
    assert lib.nfn_native_tile_glimmer_embedding_gather_float32_v1(
        ctypes.byref(descriptor), 0, None) == 1
    assert lib.nfn_native_tile_glimmer_embedding_batch_i32_float32_v1(
        ctypes.byref(descriptor), None, out.data_ptr(), 2) == 1
    assert lib.nfn_native_tile_glimmer_embedding_batch_i32_float32_v1(
        ctypes.byref(descriptor), out.data_ptr(), out.data_ptr(), 0) == 1
    # tokens that live in device memory cannot be checked on the host: zeros, no fault
    tokens = to_device(np.array([vocabulary, -5], dtype=np.int32), cuda)
    rows = engine_ops.embedding(table, tokens)
    assert torch_().count_nonzero(rows).item() == 0


# ---- rotary position embedding -------------------------------------------------------

def test_rope_probe_case(cuda, oracle):
    # probe :417-458
    query_heads, kv_heads, head_dim, position, theta = 32, 2, 128, 2051, 500000.0
    query = ((np.arange(query_heads * head_dim) % 29 - 14) / np.float32(17.0)).astype(np.float32)
    key = ((np.arange(kv_heads * head_dim) % 19 - 9) / np.float32(13.0)).astype(np.float32)
    query, key = query.reshape(query_heads, head_dim), key.reshape(kv_heads, head_dim)
    q, k = to_device(query, cuda), to_device(key, cuda)
    engine_ops.rope(q, k, position, theta)
    # the engine's double-precision formula to the last bit or the one beside it
    assert np.abs(q.cpu().numpy() - oracle.rope(query, position, theta)).max() <= 1.2e-7
    assert np.abs(k.cpu().numpy() - oracle.rope(key, position, theta)).max() <= 1.2e-7


@pytest.mark.parametrize("layout", [engine_ops.ROPE_HALF_SPLIT, engine_ops.ROPE_INTERLEAVED])
@pytest.mark.parametrize("inverse", [False, True])
def test_rope_batch_against_oracle(cuda, oracle, layout, inverse):
    rng = np.random.default_rng(11)
    rows, query_heads, kv_heads, head_dim, start, theta = 7, 6, 3, 64, 130000, 10000.0
    query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    q, k = to_device(query, cuda), to_device(key, cuda)
    engine_ops.rope(q, k, start, theta, layout, inverse, batch=True)
    for row in range(rows):
        for actual, source in ((q, query), (k, key)):
            expected = oracle.rope(source[row], start + row, theta, layout == 1, inverse)
            assert np.abs(actual[row].cpu().numpy() - expected).max() <= 5e-7
    # rows == 1 of the batch form is the one-position form
    q1, k1 = to_device(query[0], cuda), to_device(key[0], cuda)
    if not inverse:
        engine_ops.rope(q1, k1, start, theta, layout)
        assert_bits_equal(q1, q[0])
        assert_bits_equal(k1, k[0])


def test_rope_fails_closed(cuda):
    lib = tile_ops.load()
    x = torch_().zeros(64, dtype=torch_().float32, device=cuda)
    good = (x.data_ptr(), x.data_ptr(), 1, 1, 64, 5, 10000.0, 0, None)
    assert lib.nfn_native_tile_glimmer_positioned_rope_float32_v1(*good) == 0
    for index, bad in ((0, None), (1, None), (2, 0), (3, 0), (4, 63), (4, 258), (4, 0), (5, -1),
                       (6, 0.0), (6, float("inf")), (6, float("nan")), (7, 2)):
        arguments = list(good)
        arguments[index] = bad
        assert lib.nfn_native_tile_glimmer_positioned_rope_float32_v1(*arguments) == 1, (index, bad)
    assert lib.nfn_native_tile_glimmer_positioned_rope_float32_v1(
        x.data_ptr(), x.data_ptr(), 3, 2, 8, 5, 10000.0, 0, None) == 1  # 3 heads over 2
    assert lib.nfn_native_tile_glimmer_positioned_rope_batch_float32_v1(
        x.data_ptr(), x.data_ptr(), 0, 1, 1, 64, 5, 10000.0, 0, False, None) == 1
    torch_().cuda.synchronize()


# ---- cache commit ---------------------------------------------------------------------

def test_cache_commit_rounds_to_bf16_in_the_ring(cuda, oracle):
    rng = np.random.default_rng(12)
    kv_heads, head_dim, capacity, stride = 2, 128, 16, 2 * 128 + 8
    keys = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    values = (rng.standard_normal((kv_heads, head_dim)) * 1e-3).astype(np.float32)
    keys[0, :4] = [1.0 + 2.0 ** -8, 1.0 + 3.0 * 2.0 ** -8, -0.0, 65504.0]  # ties and edge values
    before = rng.integers(0, 65536, (capacity, stride), dtype=np.uint16)
    key_cache, value_cache = bf16_tensor(before, cuda), bf16_tensor(before, cuda)
    position = 3 * capacity + 5
    engine_ops.cache_commit(to_device(keys, cuda), to_device(values, cuda), key_cache, value_cache,
                            position)
    expected_keys, expected_values = before.copy(), before.copy()
    expected_keys[5, :kv_heads * head_dim] = oracle.to_bf16(keys.reshape(-1))
    expected_values[5, :kv_heads * head_dim] = oracle.to_bf16(values.reshape(-1))
    assert np.array_equal(bits_of(key_cache), expected_keys)      # nothing else touched,
    assert np.array_equal(bits_of(value_cache), expected_values)  # not even the row's padding
    # rows form: rows wrap around the ring
    rows = 4
    block_keys = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    block_values = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    engine_ops.cache_commit(to_device(block_keys, cuda), to_device(block_values, cuda), key_cache,
                            value_cache, capacity - 2, rows=rows)
    for row in range(rows):
        slot = (capacity - 2 + row) % capacity
        expected_keys[slot, :kv_heads * head_dim] = oracle.to_bf16(block_keys[row].reshape(-1))
        expected_values[slot, :kv_heads * head_dim] = oracle.to_bf16(block_values[row].reshape(-1))
    assert np.array_equal(bits_of(key_cache), expected_keys)
    assert np.array_equal(bits_of(value_cache), expected_values)
    lib = tile_ops.load()
    d = tile_ops.CacheCommitDescriptor()
    assert lib.nfn_native_tile_glimmer_cache_commit_bf16_v1(ctypes.byref(d)) == 1
    assert lib.nfn_native_tile_glimmer_cache_commit_bf16_v1(None) == 1


# ---- one-token attention -----------------------------------------------------------------

def test_gqa_probe_case_local_window_2048(cuda, oracle):
    # probe :2366-2482
    query_heads, kv_heads, head_dim, position, first, capacity = 32, 2, 128, 2048, 1, 2048
    stride, scale = kv_heads * head_dim, 0.08838834764831845
    dims = np.arange(head_dim)
    query = patterned(np.arange(query_heads)[:, None], dims[None, :], 31, 29.0)
    heads = np.arange(kv_heads)
    current_key = patterned((position + heads)[:, None], dims[None, :], 37, 41.0)
    current_value = patterned((position + heads * 3)[:, None], dims[None, :], 43, 47.0)
    key_cache = np.zeros((capacity, stride), dtype=np.uint16)
    value_cache = np.zeros((capacity, stride), dtype=np.uint16)
    positions = np.arange(first, position)
    for head in range(kv_heads):
        rows = positions % capacity
        key_cache[rows, head * head_dim:(head + 1) * head_dim] = oracle.to_bf16(
            patterned((positions + head)[:, None], dims[None, :], 37, 41.0))
        value_cache[rows, head * head_dim:(head + 1) * head_dim] = oracle.to_bf16(
            patterned((positions + head * 3)[:, None], dims[None, :], 43, 47.0))
    out = engine_ops.gqa_decode(to_device(query, cuda), to_device(current_key, cuda),
                                to_device(current_value, cuda), bf16_tensor(key_cache, cuda),
                                bf16_tensor(value_cache, cuda), position, first, scale)
    expected = oracle.gqa_decode(query, current_key, current_value, key_cache, value_cache, position,
                                 first, scale)
    assert np.abs(out.cpu().numpy() - expected).max() <= 2e-6  # the probe allows 4e-4


@pytest.mark.parametrize("query_heads,kv_heads,head_dim,position,first,capacity,padding", [
    (32, 2, 128, 5000, 0, 8192, 0),      # global layer: whole context, 79 tiles over 16 waves
    (32, 2, 128, 70, 7, 2048, 0),        # two tiles
    (8, 8, 64, 0, 0, 16, 0),             # first token: only its own key
    (6, 3, 50, 300, 100, 256, 6),        # head_dim not a multiple of 8: element-wise loads
    (4, 1, 256, 130, 0, 2048, 8),        # the widest head, padded cache rows
    (16, 4, 8, 1000, 0, 1024, 0),        # the narrowest vector head
])
def test_gqa_against_oracle(cuda, oracle, query_heads, kv_heads, head_dim, position, first, capacity,
                            padding):
    rng = np.random.default_rng(position + head_dim)
    stride = kv_heads * head_dim + padding
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    key_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    value_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    scale = 1.0 / np.sqrt(head_dim)
    out = engine_ops.gqa_decode(to_device(query, cuda), to_device(key, cuda), to_device(value, cuda),
                                bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda),
                                position, first, scale)
    expected = oracle.gqa_decode(query, key, value, key_cache, value_cache, position, first, scale)
    assert np.abs(out.cpu().numpy() - expected).max() <= 4e-6


@pytest.mark.parametrize("query_heads,kv_heads,head_dim,position,first,capacity", [
    (32, 2, 128, 5000, 2953, 2048),   # a full local window: 32 tiles in eight shares
    (32, 2, 128, 9000, 0, 16384),     # 141 tiles, shares of 18
    (8, 8, 64, 200, 0, 256),          # four tiles in four shares, the last one holds the current key
    (4, 1, 256, 130, 2, 2048),        # three tiles
    (6, 3, 128, 70, 7, 64),           # one tile: nothing to split
    (6, 3, 50, 300, 100, 256),        # no vector form: the ordinary kernel
    # head_dim 128 with four or more query heads per key/value head: the matrix-core kernel
    (32, 2, 128, 2047, 0, 2048),      # 2048 keys: 32 full tiles, the current key closes the last
    (32, 2, 128, 2048, 1, 2048),      # the current key alone in its tile; the ring is full and wraps
    (8, 2, 128, 64, 0, 128),          # one cached tile and the current key
    (20, 1, 128, 333, 40, 512),       # two groups of query heads (16 + 4), a window, ragged last tile
    (48, 3, 128, 40000, 0, 65536),    # 626 tiles: 85 shares, more than one tile a wave
    (4, 1, 128, 700, 130, 640),       # the fewest grouped heads; window wraps the ring
])
def test_gqa_split_form_against_oracle(cuda, oracle, query_heads, kv_heads, head_dim, position, first,
                                       capacity):
    rng = np.random.default_rng(position + head_dim + 1)
    stride = kv_heads * head_dim + (6 if head_dim == 50 else 0)
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    key_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    value_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    scale = 1.0 / np.sqrt(head_dim)
    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim)
    workspace.fill_(0xFF)  # the workspace comes uninitialised: NaN patterns must not leak
    arguments = (to_device(query, cuda), to_device(key, cuda), to_device(value, cuda),
                 bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda), position, first, scale)
    out = engine_ops.gqa_decode(*arguments, workspace=workspace)
    expected = oracle.gqa_decode(query, key, value, key_cache, value_cache, position, first, scale)
    assert np.abs(out.cpu().numpy() - expected).max() <= 4e-6
    again = engine_ops.gqa_decode(*arguments, workspace=workspace)
    assert_bits_equal(out, again, "repeatable")
    lib = tile_ops.load()
    assert lib.nfn_mi355_gqa_decode_split_workspace_bytes_v1(0, 128) == 0
    assert lib.nfn_mi355_gqa_decode_split_workspace_bytes_v1(32, 257) == 0
    assert lib.nfn_mi355_gqa_decode_split_v1(None, workspace.data_ptr(), workspace.numel()) == 1


def test_gqa_fails_closed(cuda):
    lib = tile_ops.load()
    x = torch_().zeros(4096, dtype=torch_().float32, device=cuda)

    def descriptor(**changes):
        d = tile_ops.GqaDecodeDescriptor()
        d.struct_size, d.version = ctypes.sizeof(d), 1
        for name in ("query", "current_key", "current_value", "key_cache_bf16", "value_cache_bf16",
                     "output"):
            setattr(d, name, x.data_ptr())
        d.query_heads, d.kv_heads, d.head_dim = 4, 2, 64
        d.position, d.first_key_position, d.cache_capacity, d.cache_row_stride = 3, 0, 16, 128
        d.scale = 0.125
        for name, value in changes.items():
            setattr(d, name, value)
        return d

    call = lib.nfn_native_tile_glimmer_gqa_decode_float32_v1
    assert call(ctypes.byref(descriptor())) == 0
    for changes in ({"version": 2}, {"flags": 1}, {"reserved0": 1}, {"reserved1": 1}, {"query": None},
                    {"output": None}, {"key_cache_bf16": None}, {"query_heads": 3}, {"kv_heads": 0},
                    {"head_dim": 0}, {"head_dim": 257}, {"position": -1}, {"first_key_position": 4},
                    {"first_key_position": -1}, {"cache_capacity": 0}, {"cache_row_stride": 127},
                    {"scale": 0.0}, {"scale": float("nan")}, {"struct_size": 8}):
        assert call(ctypes.byref(descriptor(**changes))) == 1, changes
    assert call(None) == 1
    torch_().cuda.synchronize()


# ---- block attention -------------------------------------------------------------------------

def _probe_block_case(oracle):
    # probe :2515-2575
    rows, query_heads, kv_heads, head_dim, context, capacity = 16, 32, 8, 128, 32, 64
    stride = kv_heads * head_dim
    dims = np.arange(head_dim)
    query = patterned(np.arange(rows * query_heads)[:, None], dims[None, :], 29, 37.0).reshape(
        rows, query_heads, head_dim)
    row_index, head_index = np.arange(rows)[:, None, None], np.arange(kv_heads)[None, :, None]
    block_key = patterned(context + row_index + head_index, dims[None, None, :], 31, 43.0)
    block_value = patterned(context + row_index + head_index * 2, dims[None, None, :], 41, 53.0)
    key_cache = np.zeros((capacity, stride), dtype=np.uint16)
    value_cache = np.zeros((capacity, stride), dtype=np.uint16)
    cached = np.arange(context)[:, None, None]
    key_cache[:context] = oracle.to_bf16(
        patterned(cached + head_index, dims[None, None, :], 31, 43.0)).reshape(context, stride)
    value_cache[:context] = oracle.to_bf16(
        patterned(cached + head_index * 2, dims[None, None, :], 41, 53.0)).reshape(context, stride)
    return query, block_key, block_value, key_cache, value_cache, context, 64, 0.08838834764831845


@pytest.mark.parametrize("causal", [False, True])
def test_block_attention_probe_case(cuda, oracle, causal):
    query, block_key, block_value, key_cache, value_cache, context, window, scale = \
        _probe_block_case(oracle)
    out = engine_ops.block_attention(
        to_device(query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
        bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda), context, window, scale, causal)
    expected = oracle.block_attention(query, block_key, block_value, key_cache, value_cache, context,
                                      window, scale, causal)
    assert np.abs(out.cpu().numpy() - expected).max() <= 2e-6  # the probe allows 5e-4


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("rows,block_rows,context,window,capacity,head_dim", [
    (5, 7, 150, 60, 96, 64),     # the window cuts the context; the ring has wrapped
    (64, 64, 3000, 2048, 2048, 128),  # the largest block over a full local window
    (1, 1, 0, 4, 4, 32),         # nothing cached yet
    (3, 9, 20, 90, 128, 50),     # the window is wider than everything; element-wise loads
])
def test_block_attention_against_oracle(cuda, oracle, causal, rows, block_rows, context, window,
                                        capacity, head_dim):
    rng = np.random.default_rng(rows * 1000 + context)
    query_heads, kv_heads = 8, 2
    stride = kv_heads * head_dim
    query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    key_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    value_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    scale = 1.0 / np.sqrt(head_dim)
    out = engine_ops.block_attention(
        to_device(query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
        bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda), context, window, scale, causal)
    expected = oracle.block_attention(query, block_key, block_value, key_cache, value_cache, context,
                                      window, scale, causal)
    assert np.abs(out.cpu().numpy() - expected).max() <= 4e-6


@pytest.mark.parametrize("query_heads,kv_heads,context,capacity,rows", [
    (8, 2, 32, 64, 16), (8, 2, 1000, 2048, 24), (8, 8, 2040, 4096, 12),
    (32, 8, 32, 64, 16), (32, 8, 1000, 2048, 24), (32, 2, 2040, 4096, 12),
])
def test_causal_block_is_token_at_a_time_decode(cuda, oracle, query_heads, kv_heads, context,
                                                capacity, rows):
    """The verifier's rule (probe :2683-2745): a causal block sees earlier block rows as the
    bf16 cache would hold them, and each row equals one-token attention followed by the commit.
    Bit for bit while the block runs on the kernel of the one-token call (its rows x heads fit
    the chip at once); a larger block with head_dim 128 runs on the matrix cores and agrees to
    rounding -- unrounded earlier rows would differ in the third digit."""
    rng = np.random.default_rng(context)
    head_dim = 128
    stride = kv_heads * head_dim
    query = to_device(rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32), cuda)
    block_key = to_device(rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32), cuda)
    block_value = to_device(rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32), cuda)
    key_cache = bf16_tensor(oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32)), cuda)
    value_cache = bf16_tensor(oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32)), cuda)
    scale = 0.08838834764831845
    block = engine_ops.block_attention(query, block_key, block_value, key_cache, value_cache, context,
                                       capacity, scale, True)
    serial = torch_().empty_like(block)
    for row in range(rows):
        engine_ops.gqa_decode(query[row], block_key[row], block_value[row], key_cache, value_cache,
                              context + row, 0, scale, out=serial[row])
        engine_ops.cache_commit(block_key[row], block_value[row], key_cache, value_cache, context + row)
    if query_heads == 8:
        assert_bits_equal(block, serial)
    else:
        assert np.abs(block.cpu().numpy() - serial.cpu().numpy()).max() <= 4e-6


@pytest.mark.parametrize("causal", [False, True])
@pytest.mark.parametrize("rows,block_rows,query_heads,kv_heads,context,window,capacity,head_dim", [
    (16, 16, 32, 2, 3000, 2048, 2048, 128),  # the verifier's block: matrix-core kernel, eight shares
    (5, 7, 8, 2, 150, 60, 96, 64),           # vector kernel, shares of one tile; the ring has wrapped
    (64, 64, 8, 2, 3000, 2048, 2048, 128),   # more rows than the workspace has room to split well
    (3, 9, 6, 3, 20, 90, 128, 50),           # no vector form: the ordinary kernel, workspace untouched
    (2, 2, 16, 1, 40, 64, 64, 128),          # one tile: nothing to split
])
def test_block_attention_split_form(cuda, oracle, causal, rows, block_rows, query_heads, kv_heads,
                                    context, window, capacity, head_dim):
    rng = np.random.default_rng(rows * 100 + context + head_dim)
    stride = kv_heads * head_dim
    query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    key_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    value_cache = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    scale = 1.0 / np.sqrt(head_dim)
    arguments = (to_device(query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
                 bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda), context, window, scale,
                 causal)
    workspace = engine_ops.gqa_decode_workspace(32, 128)  # what an engine would have at hand
    workspace.fill_(0xFF)
    out = engine_ops.block_attention(*arguments, workspace=workspace)
    expected = oracle.block_attention(query, block_key, block_value, key_cache, value_cache, context,
                                      window, scale, causal)
    assert np.abs(out.cpu().numpy() - expected).max() <= 4e-6
    # the reference-named call takes the same form while the workspace is lent
    engine_ops.lend_attention_workspace(workspace)
    try:
        lent = engine_ops.block_attention(*arguments)
    finally:
        engine_ops.lend_attention_workspace(None)
    assert_bits_equal(lent, out, "lent = explicit split form")
    lib = tile_ops.load()
    assert lib.nfn_mi355_dflash_block_attention_split_v1(None, workspace.data_ptr(), 1 << 20) == 1


def test_block_attention_fails_closed(cuda):
    lib = tile_ops.load()
    x = torch_().zeros(1 << 16, dtype=torch_().float32, device=cuda)

    def descriptor(**changes):
        d = tile_ops.BlockAttentionDescriptor()
        d.struct_size, d.version = ctypes.sizeof(d), 1
        for name in ("query", "block_key", "block_value", "key_cache_bf16", "value_cache_bf16",
                     "output"):
            setattr(d, name, x.data_ptr())
        d.query_rows, d.block_rows, d.query_heads, d.kv_heads, d.head_dim = 2, 4, 4, 2, 64
        d.context_length, d.sliding_window, d.cache_capacity, d.cache_row_stride = 5, 16, 16, 128
        d.scale = 0.125
        for name, value in changes.items():
            setattr(d, name, value)
        return d

    call = lib.nfn_native_tile_dflash_block_attention_float32_v1
    assert call(ctypes.byref(descriptor())) == 0
    assert call(ctypes.byref(descriptor(flags=1))) == 0
    for changes in ({"version": 0}, {"flags": 2}, {"reserved0": 1}, {"block_key": None},
                    {"query_rows": 0}, {"query_rows": 5}, {"block_rows": 65}, {"query_heads": 3},
                    {"head_dim": 300}, {"context_length": -1}, {"sliding_window": 0},
                    {"cache_capacity": 15}, {"cache_row_stride": 100}, {"scale": -1.0}):
        assert call(ctypes.byref(descriptor(**changes))) == 1, changes
    assert call(None) == 1
    torch_().cuda.synchronize()


# ---- logit transform, add, scale -------------------------------------------------------------------

def test_logit_transform_add_scale(cuda, oracle):
    rng = np.random.default_rng(13)
    logits = (rng.standard_normal(202048) * 25).astype(np.float32)
    device_logits = to_device(logits, cuda)
    engine_ops.logit_transform(device_logits, 1.5, 20.0)
    expected = oracle.logit_transform(logits, 1.5, 20.0)
    difference = np.abs(device_logits.cpu().numpy().astype(np.float64) - expected)
    assert difference.max() <= 2e-6  # one float rounding of a value up to 20
    a = rng.standard_normal(6656 * 3 + 1).astype(np.float32)
    b = rng.standard_normal(6656 * 3 + 1).astype(np.float32)
    assert_bits_equal(engine_ops.add(to_device(a, cuda), to_device(b, cuda)), a + b)
    values = to_device(a, cuda)
    engine_ops.scale_inplace(values, 0.3)
    assert_bits_equal(values, a * np.float32(0.3))
    lib = tile_ops.load()
    assert lib.nfn_native_tile_glimmer_logit_transform_float32_v1(None, 4, 1.0, 1.0, None) == 1
    assert lib.nfn_native_tile_glimmer_logit_transform_float32_v1(values.data_ptr(), 0, 1.0, 1.0, None) == 1
    assert lib.nfn_native_tile_glimmer_logit_transform_float32_v1(values.data_ptr(), 4, 0.0, 1.0, None) == 1
    assert lib.nfn_native_tile_glimmer_logit_transform_float32_v1(values.data_ptr(), 4, 1.0, float("inf"), None) == 1
    assert lib.nfn_native_tile_add_float32(values.data_ptr(), values.data_ptr(), values.data_ptr(), 0, None) == 1
    assert lib.nfn_native_tile_scale_inplace_float32(None, 4, 1.0, None) == 1


# ---- fused per-head norm + scale + rope, fused decode attention ---------------------------------------

def _norm_row(values):
    return tile_ops.PackedWeight.from_numpy(kquant.F32, values.view(np.uint8).copy(), 1, values.size)


@pytest.mark.parametrize("apply_rope", [False, True])
@pytest.mark.parametrize("weights", ["none", "f32", "f32_centered"])
def test_qk_norm_scale_rope_equals_the_three_separate_calls(cuda, oracle, weights, apply_rope):
    # probe :461-610: the fused result is the unfused composition bit for bit
    query_heads, kv_heads, head_dim = 32, 2, 128
    eps, query_scale, position, theta = 1e-5, 3.87, 2051, 500000.0
    query = (((np.arange(query_heads * head_dim) * 31 + 11) % 257 - 128) / np.float32(73.0)).astype(np.float32)
    key = (((np.arange(kv_heads * head_dim) * 23 + 5) % 193 - 96) / np.float32(61.0)).astype(np.float32)
    query, key = query.reshape(query_heads, head_dim), key.reshape(kv_heads, head_dim)
    rng = np.random.default_rng(31)
    q_row = (0.1 * rng.standard_normal(head_dim)).astype(np.float32) + (0 if weights == "f32_centered" else 1)
    k_row = (0.1 * rng.standard_normal(head_dim)).astype(np.float32) + (0 if weights == "f32_centered" else 1)
    q_weight = None if weights == "none" else _norm_row(q_row.astype(np.float32))
    k_weight = None if weights == "none" else _norm_row(k_row.astype(np.float32))
    centered = weights == "f32_centered"

    baseline_q = tile_ops.rms_norm(to_device(query, cuda), q_weight, centered, eps)["output"]
    baseline_k = tile_ops.rms_norm(to_device(key, cuda), k_weight, centered, eps)["output"]
    engine_ops.scale_inplace(baseline_q, query_scale)
    if apply_rope:
        engine_ops.rope(baseline_q, baseline_k, position, theta)
    fused_q, fused_k = to_device(query, cuda), to_device(key, cuda)
    engine_ops.qk_norm_scale_rope(fused_q, fused_k, q_weight, k_weight, eps, query_scale, position,
                                  theta, engine_ops.ROPE_HALF_SPLIT, apply_rope, centered, centered)
    assert_bits_equal(fused_q, baseline_q, "query")
    assert_bits_equal(fused_k, baseline_k, "key")

    # and the CPU engine's double-precision statement of the same thing
    scale_q = None if weights == "none" else (q_row + 1 if centered else q_row).astype(np.float32)
    scale_k = None if weights == "none" else (k_row + 1 if centered else k_row).astype(np.float32)
    expected_q = oracle.qk_norm(query, scale_q, eps, query_scale)
    expected_k = oracle.qk_norm(key, scale_k, eps, 1.0)
    if apply_rope:
        expected_q = oracle.rope(expected_q, position, theta)
        expected_k = oracle.rope(expected_k, position, theta)
    assert np.abs(fused_q.cpu().numpy() - expected_q).max() <= 4e-6 * np.abs(expected_q).max()
    assert np.abs(fused_k.cpu().numpy() - expected_k).max() <= 4e-6 * np.abs(expected_k).max()


def test_qk_norm_scale_rope_batch_rows_and_fail_closed(cuda):
    rng = np.random.default_rng(32)
    rows, query_heads, kv_heads, head_dim = 5, 6, 3, 64
    query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    q, k = to_device(query, cuda), to_device(key, cuda)
    engine_ops.qk_norm_scale_rope(q, k, None, None, 1e-6, 0.5, 700, 10000.0,
                                  engine_ops.ROPE_INTERLEAVED, True)
    for row in range(rows):
        q1, k1 = to_device(query[row], cuda), to_device(key[row], cuda)
        engine_ops.qk_norm_scale_rope(q1, k1, None, None, 1e-6, 0.5, 700 + row, 10000.0,
                                      engine_ops.ROPE_INTERLEAVED, True)
        assert_bits_equal(q[row], q1, f"query row {row}")
        assert_bits_equal(k[row], k1, f"key row {row}")
    lib = tile_ops.load()
    good = [q.data_ptr(), k.data_ptr(), None, None, rows, query_heads, kv_heads, head_dim, 1e-6, False,
            False, 0.5, 700, 10000.0, 0, True, None]
    call = lib.nfn_native_tile_glimmer_qk_norm_scale_rope_batch_float32_v1
    assert call(*good) == 0
    for index, bad in ((0, None), (1, None), (4, 0), (4, 65), (5, 4), (7, 63), (7, 258), (8, 0.0),
                       (11, 0.0), (11, float("inf")), (12, -1), (13, float("nan")), (14, 2)):
        arguments = list(good)
        arguments[index] = bad
        assert call(*arguments) == 1, (index, bad)
    wrong_width = _norm_row(np.ones(32, dtype=np.float32)).descriptor(0)
    arguments = list(good)
    arguments[2] = ctypes.byref(wrong_width)
    assert call(*arguments) == 1
    torch_().cuda.synchronize()


@pytest.mark.parametrize("apply_rope,first", [(False, 2500), (True, 4100 - 2048 + 1), (True, 4100 - 2048)])
def test_fused_decode_attention_equals_the_separate_calls(cuda, oracle, apply_rope, first):
    # the last case reads as many keys as the ring has rows: the oldest one sits in the row
    # the commit overwrites, so the commit has to come after the attention, as in the separate calls
    rng = np.random.default_rng(33)
    query_heads, kv_heads, head_dim, capacity, position = 32, 2, 128, 2048, 4100
    stride = kv_heads * head_dim
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    keys = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    q_weight = _norm_row((1.0 + 0.1 * rng.standard_normal(head_dim)).astype(np.float32))
    k_weight = _norm_row((1.0 + 0.1 * rng.standard_normal(head_dim)).astype(np.float32))
    scale = head_dim ** -0.5

    q1, k1, v1 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc1, vc1 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    engine_ops.qk_norm_scale_rope(q1, k1, q_weight, k_weight, 1e-5, 1.0, position, 500000.0,
                                  engine_ops.ROPE_INTERLEAVED, apply_rope)
    separate = engine_ops.gqa_decode(q1, k1, v1, kc1, vc1, position, first, scale)
    engine_ops.cache_commit(k1, v1, kc1, vc1, position)

    q2, k2, v2 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc2, vc2 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    fused = engine_ops.fused_decode_attention(q2, k2, v2, kc2, vc2, position, first, scale, q_weight,
                                              k_weight, 1e-5, 1.0, 500000.0,
                                              engine_ops.ROPE_INTERLEAVED, apply_rope)
    assert_bits_equal(fused, separate, "attention output")
    assert_bits_equal(q2, q1, "query in place")
    assert_bits_equal(k2, k1, "key in place")
    assert np.array_equal(bits_of(kc2), bits_of(kc1)) and np.array_equal(bits_of(vc2), bits_of(vc1))
    assert np.array_equal(bits_of(kc2)[position % capacity], oracle.to_bf16(k1.cpu().numpy().reshape(-1)))
    # the split form of the fused call: same in-place results and cache, attention within tolerance
    q3, k3, v3 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc3, vc3 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    split = engine_ops.fused_decode_attention(q3, k3, v3, kc3, vc3, position, first, scale, q_weight,
                                              k_weight, 1e-5, 1.0, 500000.0,
                                              engine_ops.ROPE_INTERLEAVED, apply_rope,
                                              workspace=engine_ops.gqa_decode_workspace(query_heads, head_dim))
    assert_bits_equal(q3, q1, "query, split form")
    assert np.array_equal(bits_of(kc3), bits_of(kc1)) and np.array_equal(bits_of(vc3), bits_of(vc1))
    assert np.abs(split.cpu().numpy() - separate.cpu().numpy()).max() <= 4e-6
    lib = tile_ops.load()
    assert lib.nfn_native_tile_glimmer_fused_decode_attention_float32_v1(None) == 1
    empty = tile_ops.FusedDecodeAttentionDescriptor()
    assert lib.nfn_native_tile_glimmer_fused_decode_attention_float32_v1(ctypes.byref(empty)) == 1


@pytest.mark.parametrize("apply_rope,position", [(True, 4100), (True, 70), (False, 1500), (False, 0)])
def test_fused_decode_attention_with_the_position_on_the_device(cuda, oracle, apply_rope, position):
    """The graph form reads the position when the kernels run: same bits as the host form at
    that position, with the window rule of the reference (kernels.cu:2604-2611): a layer with
    rope sees its last `sliding_window` keys, one without sees everything."""
    rng = np.random.default_rng(34 + position)
    query_heads, kv_heads, head_dim, window = 32, 2, 128, 2048
    capacity = window if apply_rope else 4096
    stride = kv_heads * head_dim
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    keys = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    weight = _norm_row((1.0 + 0.1 * rng.standard_normal(head_dim)).astype(np.float32))
    first = max(0, position - window + 1) if apply_rope else 0
    common = dict(query_weight=weight, key_weight=weight, eps=1e-5, query_scale=1.0, theta=500000.0,
                  layout=engine_ops.ROPE_INTERLEAVED, apply_rope=apply_rope)

    q1, k1, v1 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc1, vc1 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    host = engine_ops.fused_decode_attention(q1, k1, v1, kc1, vc1, position, first,
                                             head_dim ** -0.5, **common)
    q2, k2, v2 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc2, vc2 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    device_position = to_device(np.array([position], dtype=np.int64), cuda)
    # the descriptor's own position fields are ignored in this form: give it other ones
    device = engine_ops.fused_decode_attention(q2, k2, v2, kc2, vc2, 7, 3, head_dim ** -0.5,
                                               device_position=device_position,
                                               sliding_window=window, **common)
    assert_bits_equal(device, host, "attention output")
    assert_bits_equal(q2, q1, "query")
    assert_bits_equal(k2, k1, "key")
    assert np.array_equal(bits_of(kc2), bits_of(kc1)) and np.array_equal(bits_of(vc2), bits_of(vc1))
    # the split form with the position on the device: one workspace and one launch geometry
    # for every position (shares are cut on the device; those past the row's keys stay empty)
    q3, k3, v3 = to_device(query, cuda), to_device(key, cuda), to_device(value, cuda)
    kc3, vc3 = bf16_tensor(keys, cuda), bf16_tensor(values, cuda)
    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim)
    workspace.fill_(0xFF)
    split = engine_ops.fused_decode_attention(q3, k3, v3, kc3, vc3, 7, 3, head_dim ** -0.5,
                                              device_position=device_position,
                                              sliding_window=window, workspace=workspace, **common)
    assert np.abs(split.cpu().numpy() - host.cpu().numpy()).max() <= 4e-6
    assert_bits_equal(q3, q1, "query, split form")
    assert np.array_equal(bits_of(kc3), bits_of(kc1)) and np.array_equal(bits_of(vc3), bits_of(vc1))
    lib = tile_ops.load()
    call = lib.nfn_native_tile_glimmer_fused_decode_attention_device_position_float32_v1
    assert call(None, device_position.data_ptr(), window) == 1
    split_call = lib.nfn_mi355_fused_decode_attention_split_device_position_v1
    assert split_call(None, device_position.data_ptr(), window, workspace.data_ptr(),
                      workspace.numel()) == 1


def test_lent_workspace_turns_the_reference_named_calls_into_their_split_forms(cuda, oracle):
    rng = np.random.default_rng(41)
    query_heads, kv_heads, head_dim, capacity, position = 32, 2, 128, 2048, 3000
    first = position - capacity + 1
    stride = kv_heads * head_dim
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    keys = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((capacity, stride)).astype(np.float32))
    scale = head_dim ** -0.5
    device_position = to_device(np.array([position], dtype=np.int64), cuda)
    fused = dict(eps=1e-5, query_scale=1.0, theta=500000.0, layout=engine_ops.ROPE_INTERLEAVED,
                 apply_rope=True)

    def run(lent, explicit):
        """(gqa_decode, fused host position, fused device position) outputs"""
        outputs = []
        engine_ops.lend_attention_workspace(lent)
        try:
            tensors = lambda: (to_device(query, cuda), to_device(key, cuda), to_device(value, cuda),
                               bf16_tensor(keys, cuda), bf16_tensor(values, cuda))
            outputs.append(engine_ops.gqa_decode(*tensors(), position, first, scale,
                                                 workspace=explicit))
            outputs.append(engine_ops.fused_decode_attention(*tensors(), position, first, scale,
                                                             workspace=explicit, **fused))
            outputs.append(engine_ops.fused_decode_attention(
                *tensors(), 5, 2, scale, device_position=device_position, sliding_window=capacity,
                workspace=explicit, **fused))
        finally:
            engine_ops.lend_attention_workspace(None)
        return outputs

    workspace = engine_ops.gqa_decode_workspace(query_heads, head_dim)
    plain = run(None, None)
    split = run(None, workspace)
    lent = run(workspace, None)
    after = run(None, None)
    for index, name in enumerate(("gqa_decode", "fused", "fused, device position")):
        assert_bits_equal(lent[index], split[index], name + ": lent = explicit split form")
        assert_bits_equal(after[index], plain[index], name + ": taken back")
        assert not np.array_equal(bits_of(split[index]), bits_of(plain[index])), name
        assert np.abs(split[index].cpu().numpy() - plain[index].cpu().numpy()).max() <= 4e-6
    # too small for the geometry: the ordinary form; bad arguments are refused
    small = torch_().empty(1024, dtype=torch_().uint8, device=cuda)
    assert_bits_equal(run(small, None)[0], plain[0], "a workspace too small is not used")
    lib = tile_ops.load()
    assert lib.nfn_mi355_attention_workspace_v1(workspace.data_ptr() + 4, 1 << 20, None) == 1
    assert lib.nfn_mi355_attention_workspace_v1(None, 16, None) == 1
    assert lib.nfn_mi355_attention_workspace_v1(workspace.data_ptr(), 0, None) == 1
    assert lib.nfn_mi355_attention_workspace_v1(None, 0, None) == 0
    # a loan serves the stream it was made for and no other: a call on a second stream keeps
    # the ordinary form (and its bits) while the first stream's loan stands
    torch = torch_()
    side = torch.cuda.Stream(device=cuda)
    engine_ops.lend_attention_workspace(workspace)           # for the current (default) stream
    try:
        tensors = (to_device(query, cuda), to_device(key, cuda), to_device(value, cuda),
                   bf16_tensor(keys, cuda), bf16_tensor(values, cuda))
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            elsewhere = engine_ops.gqa_decode(*tensors, position, first, scale)
        side.synchronize()
        assert_bits_equal(elsewhere, plain[0], "another stream does not see the loan")
        here = engine_ops.gqa_decode(*tensors, position, first, scale)
        assert_bits_equal(here, split[0], "the loan's stream does")
        # the side stream can hold a loan of its own; taking it back leaves the first in place
        own = engine_ops.gqa_decode_workspace(query_heads, head_dim)
        engine_ops.lend_attention_workspace(own, side.cuda_stream)
        with torch.cuda.stream(side):
            elsewhere = engine_ops.gqa_decode(*tensors, position, first, scale)
        side.synchronize()
        assert_bits_equal(elsewhere, split[0], "the side stream's own loan")
        engine_ops.lend_attention_workspace(None, side.cuda_stream)
        assert_bits_equal(engine_ops.gqa_decode(*tensors, position, first, scale), split[0])
    finally:
        engine_ops.lend_attention_workspace(None, side.cuda_stream)
        engine_ops.lend_attention_workspace(None)
    # the table is bounded: a 33rd stream's loan is refused, the 32 others stand until taken back
    for handle in range(1, 33):
        assert lib.nfn_mi355_attention_workspace_v1(workspace.data_ptr(), 1 << 20, handle << 8) == 0
    assert lib.nfn_mi355_attention_workspace_v1(workspace.data_ptr(), 1 << 20, 33 << 8) == 1
    for handle in range(1, 33):
        assert lib.nfn_mi355_attention_workspace_v1(None, 0, handle << 8) == 0
    assert lib.nfn_mi355_attention_workspace_v1(workspace.data_ptr(), 1 << 20, 33 << 8) == 0
    assert lib.nfn_mi355_attention_workspace_v1(None, 0, 33 << 8) == 0


def test_cache_commit_layers_and_pack_target_taps(cuda, oracle):
    rng = np.random.default_rng(35)
    layers, source_rows, rows, kv_heads, head_dim, position = 5, 9, 6, 2, 64, 1021
    width = kv_heads * head_dim
    capacities = [1024, 2048, 64, 1024, 4096]  # rows wrap in some rings and not in others
    staged_keys = rng.standard_normal((layers, source_rows, kv_heads, head_dim)).astype(np.float32)
    staged_values = rng.standard_normal((layers, source_rows, kv_heads, head_dim)).astype(np.float32)
    before = [rng.integers(0, 65536, (capacity, width + 8), dtype=np.uint16) for capacity in capacities]
    caches = [(bf16_tensor(b, cuda), bf16_tensor(b, cuda)) for b in before]
    engine_ops.cache_commit_layers(to_device(staged_keys, cuda), to_device(staged_values, cuda), caches,
                                   rows, position)
    for layer, (capacity, start) in enumerate(zip(capacities, before)):
        expected_keys, expected_values = start.copy(), start.copy()
        for row in range(rows):
            slot = (position + row) % capacity
            expected_keys[slot, :width] = oracle.to_bf16(staged_keys[layer, row].reshape(-1))
            expected_values[slot, :width] = oracle.to_bf16(staged_values[layer, row].reshape(-1))
        assert np.array_equal(bits_of(caches[layer][0]), expected_keys), f"layer {layer} keys"
        assert np.array_equal(bits_of(caches[layer][1]), expected_values), f"layer {layer} values"
    lib = tile_ops.load()
    assert lib.nfn_native_tile_glimmer_cache_commit_layers_bf16_v1(None) == 1
    empty = tile_ops.CacheCommitLayersDescriptor()
    assert lib.nfn_native_tile_glimmer_cache_commit_layers_bf16_v1(ctypes.byref(empty)) == 1

    taps, hidden = 4, 6656
    tap_major = rng.standard_normal((taps, source_rows, hidden)).astype(np.float32)
    packed = engine_ops.pack_target_taps(to_device(tap_major, cuda), 2, 5).cpu().numpy()
    assert np.array_equal(packed, np.transpose(tap_major[:, 2:7], (1, 0, 2)))
    x = to_device(tap_major, cuda)
    call = lib.nfn_native_tile_glimmer_pack_target_taps_float32_v1
    assert call(x.data_ptr(), x.data_ptr(), source_rows, 5, 5, taps, hidden, None) == 1  # 5 + 5 > 9
    assert call(None, x.data_ptr(), source_rows, 0, 5, taps, hidden, None) == 1
    assert call(x.data_ptr(), x.data_ptr(), 65, 0, 5, taps, hidden, None) == 1
    assert call(x.data_ptr(), x.data_ptr(), source_rows, 0, 5, taps, 65537, None) == 1


def test_short_split_block_attention_is_the_general_one_inside_its_geometry(cuda, oracle):
    # probe :2666-2682: the short-split output within 5e-4 of the general one; here the same bits
    query, block_key, block_value, key_cache, value_cache, context, window, scale = \
        _probe_block_case(oracle)
    import torch
    arguments = (to_device(query, cuda), to_device(block_key, cuda), to_device(block_value, cuda),
                 bf16_tensor(key_cache, cuda), bf16_tensor(value_cache, cuda))
    general = engine_ops.block_attention(*arguments, context, window, scale, False)
    lib = tile_ops.load()
    call = lib.nfn_native_tile_dflash_block_attention_short_split_float32_v1
    stream = torch.cuda.Stream()

    def descriptor(out, **changes):
        d = tile_ops.BlockAttentionDescriptor()
        d.struct_size, d.version = ctypes.sizeof(d), 1
        d.query, d.block_key, d.block_value = (t.data_ptr() for t in arguments[:3])
        d.key_cache_bf16, d.value_cache_bf16, d.output = (arguments[3].data_ptr(),
                                                          arguments[4].data_ptr(), out.data_ptr())
        d.query_rows, d.query_heads, d.head_dim = query.shape
        d.block_rows, d.kv_heads = block_key.shape[0], block_key.shape[1]
        d.context_length, d.sliding_window = context, window
        d.cache_capacity, d.cache_row_stride = key_cache.shape
        d.scale = scale
        d.cuda_stream = int(stream.cuda_stream)
        for name, value in changes.items():
            setattr(d, name, value)
        return d

    score_count = 16 * 32 * 6 * 8  # rows x heads x ceil(48 keys / 8) x 8, the probe's workspace
    scores = torch.empty(score_count, dtype=torch.float32, device=cuda)
    out = torch.zeros_like(general)
    torch.cuda.synchronize()
    assert call(ctypes.byref(descriptor(out)), scores.data_ptr(), score_count * 4) == 0
    stream.synchronize()
    assert_bits_equal(out, general)
    # outside the geometry, or with too small a workspace, it fails closed
    assert call(ctypes.byref(descriptor(out)), scores.data_ptr(), score_count * 4 - 1) == 1
    assert call(ctypes.byref(descriptor(out)), None, score_count * 4) == 1
    assert call(ctypes.byref(descriptor(out, cuda_stream=None)), scores.data_ptr(), score_count * 4) == 1
    assert call(ctypes.byref(descriptor(out, sliding_window=4096, context_length=500)),
                scores.data_ptr(), 1 << 30) == 1  # more than 128 keys
    assert call(ctypes.byref(descriptor(out, query_heads=16)), scores.data_ptr(), score_count * 4) == 1


# ---- a whole decode layer ---------------------------------------------------------------------------

def test_two_decode_layers_against_the_cpu_engine_arithmetic(cuda, oracle):
    """neuralfn_amd/decode_layer.py sequences every operator of a layer through the C ABI; the
    same layer in the oracle's double-precision operators (resident_glimmer.cpp:1719-1830) must
    agree at the linear path's tolerance."""
    from neuralfn_amd import decode_layer as dl
    rng = np.random.default_rng(21)
    g = dl.LayerGeometry(model_dim=512, query_heads=4, kv_heads=2, head_dim=64, ffn_dim=768,
                         sliding_window=128)
    position = 200  # the ring has wrapped
    formats = dict(q=kquant.Q4_K, k=kquant.Q5_K, v=kquant.Q6_K, attention_gate=kquant.Q4_K,
                   output=kquant.Q5_K, mlp_gate=kquant.Q4_K, mlp_up=kquant.Q8_0, mlp_down=kquant.Q6_K)
    shapes = dict(q=(g.attention_dim, g.model_dim), k=(g.kv_dim, g.model_dim),
                  v=(g.kv_dim, g.model_dim), attention_gate=(g.attention_dim, g.model_dim),
                  output=(g.model_dim, g.attention_dim), mlp_gate=(g.ffn_dim, g.model_dim),
                  mlp_up=(g.ffn_dim, g.model_dim), mlp_down=(g.model_dim, g.ffn_dim))
    norms = dict(input_norm=g.model_dim, q_norm=g.head_dim, k_norm=g.head_dim,
                 post_attention_norm=g.model_dim, pre_feedforward_norm=g.model_dim,
                 post_feedforward_norm=g.model_dim)

    host_layers, device_layers, host_caches, device_caches = [], [], [], []
    for _ in range(2):
        host, device = {}, {}
        for name, (out_dim, in_dim) in shapes.items():
            packed = kquant.quantize(formats[name],
                                     (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32))
            host[name] = (formats[name], packed, out_dim, in_dim)
            device[name] = tile_ops.PackedWeight.from_numpy(formats[name], packed, out_dim, in_dim)
        for name, width in norms.items():
            row = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)
            host[name] = row
            device[name] = tile_ops.PackedWeight.from_numpy(kquant.F32, row.view(np.uint8).copy(), 1, width)
        host_layers.append(host)
        device_layers.append(dl.LayerWeights(**device))
        keys = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
        values = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
        host_caches.append((keys.copy(), values.copy()))
        cache = dl.LayerCache(g, cuda)
        cache.keys.copy_(bf16_tensor(keys, cuda))
        cache.values.copy_(bf16_tensor(values, cuda))
        device_caches.append(cache)

    embedding = rng.standard_normal((1, g.model_dim)).astype(np.float32)

    # ---- the library ----
    workspace = tile_ops.small_batch_workspace(1, max(g.model_dim, g.ffn_dim))
    pending, residual, pending_norm = to_device(embedding, cuda), to_device(np.zeros_like(embedding), cuda), None
    for weights, cache in zip(device_layers, device_caches):
        pending, residual = dl.decode_layer(g, weights, cache, pending, residual, pending_norm,
                                            position, workspace)
        pending_norm = weights.post_feedforward_norm
    actual_down, actual_hidden = pending.cpu().numpy(), residual.cpu().numpy()

    # ---- the oracle ----
    def linear(entry, x):
        encoding, packed, out_dim, in_dim = entry
        return oracle.linear(encoding, packed, out_dim, in_dim, x.reshape(1, in_dim))[0]

    owed, hidden_before, owed_norm = embedding[0], np.zeros(g.model_dim, dtype=np.float32), None
    for host, (keys, values) in zip(host_layers, host_caches):
        eps = g.post_norm_eps if owed_norm is not None else g.norm_eps
        hidden = hidden_before + oracle.rms_norm(owed, owed_norm, False, eps)
        normalized = oracle.rms_norm(hidden, host["input_norm"], False, g.norm_eps)
        query = linear(host["q"], normalized).reshape(g.query_heads, g.head_dim)
        key = linear(host["k"], normalized).reshape(g.kv_heads, g.head_dim)
        value = linear(host["v"], normalized).reshape(g.kv_heads, g.head_dim)
        gate = linear(host["attention_gate"], normalized)
        query = np.stack([oracle.rms_norm(row, host["q_norm"], False, g.norm_eps) for row in query])
        key = np.stack([oracle.rms_norm(row, host["k_norm"], False, g.norm_eps) for row in key])
        query = oracle.rope(query, position, g.rope_theta, True)
        key = oracle.rope(key, position, g.rope_theta, True)
        attention = oracle.gqa_decode(query, key, value, keys, values, position,
                                      position - g.sliding_window + 1, g.head_dim ** -0.5)
        gated = oracle.sigmoid_gate(attention.reshape(-1), gate)
        projected = linear(host["output"], gated)
        hidden = hidden + oracle.rms_norm(projected, host["post_attention_norm"], False, g.post_norm_eps)
        normalized = oracle.rms_norm(hidden, host["pre_feedforward_norm"], False, g.norm_eps)
        activated = oracle.swiglu(linear(host["mlp_gate"], normalized), linear(host["mlp_up"], normalized))
        owed, hidden_before, owed_norm = linear(host["mlp_down"], activated), hidden, host["post_feedforward_norm"]
        # what the commit must have left in the ring
        keys[position % g.sliding_window] = oracle.to_bf16(key.reshape(-1))
        values[position % g.sliding_window] = oracle.to_bf16(value.reshape(-1))

    def error(actual, expected):
        return float(np.max(np.abs(actual.reshape(-1) - expected)) / np.max(np.abs(expected)))

    assert error(actual_hidden, hidden_before) <= 2e-3
    assert error(actual_down, owed) <= 4e-3  # two layers of 2e-3 operators in sequence
    # The committed rows: bf16 of values that carry the projections' error, so a rounding step
    # (2^-8 relative) apart at most, and exact for most entries.
    for cache, (keys, values) in zip(device_caches, host_caches):
        slot = position % g.sliding_window
        for device_rows, host_rows in ((cache.keys, keys), (cache.values, values)):
            committed = oracle.bf16_to_float(bits_of(device_rows)[slot])
            expected = oracle.bf16_to_float(host_rows[slot])
            assert np.max(np.abs(committed - expected)) <= 2e-3 * np.max(np.abs(expected)) + 2.0 ** -8 * np.max(np.abs(expected))
        untouched = np.delete(np.arange(g.sliding_window), slot)
        assert np.array_equal(bits_of(cache.keys)[untouched], keys[untouched])


def test_decode_layer_with_the_fused_calls_gives_the_same_bits(cuda, oracle):
    """decode_layer(fused_gate_up=True, fused_input_norm=True) takes gate and up through
    nfn_mi355_k_quant_mmvq_gate_up_swiglu_float32_v1 (the down projection on its plain output)
    and the first dual norm inside the Q/K/V/gate launch
    (nfn_mi355_dual_rms_mmvq_multi_linear_float32_v1): the layer's two results and the
    committed cache rows equal the separate calls' bit for bit."""
    from neuralfn_amd import decode_layer as dl
    rng = np.random.default_rng(23)
    g = dl.LayerGeometry(model_dim=768, query_heads=4, kv_heads=2, head_dim=64, ffn_dim=1280,
                         sliding_window=128)
    shapes = dict(q=(g.attention_dim, g.model_dim), k=(g.kv_dim, g.model_dim),
                  v=(g.kv_dim, g.model_dim), attention_gate=(g.attention_dim, g.model_dim),
                  output=(g.model_dim, g.attention_dim), mlp_gate=(g.ffn_dim, g.model_dim),
                  mlp_up=(g.ffn_dim, g.model_dim), mlp_down=(g.model_dim, g.ffn_dim))
    device = {}
    for name, (out_dim, in_dim) in shapes.items():
        encoding = kquant.Q5_K if name in ("mlp_gate", "mlp_up") else kquant.Q4_K
        packed = kquant.quantize(encoding, (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32))
        device[name] = tile_ops.PackedWeight.from_numpy(encoding, packed, out_dim, in_dim)
    for name, width in dict(input_norm=g.model_dim, q_norm=g.head_dim, k_norm=g.head_dim,
                            post_attention_norm=g.model_dim, pre_feedforward_norm=g.model_dim,
                            post_feedforward_norm=g.model_dim).items():
        row = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)
        device[name] = tile_ops.PackedWeight.from_numpy(kquant.F32, row.view(np.uint8).copy(), 1, width)
    weights = dl.LayerWeights(**device)
    assert tile_ops.gate_up_swiglu_supported(weights.mlp_gate, weights.mlp_up)
    keys = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    embedding = to_device(rng.standard_normal((1, g.model_dim)).astype(np.float32), cuda)
    workspace = tile_ops.small_batch_workspace(1, max(g.model_dim, g.ffn_dim))
    results = []
    assert tile_ops.dual_rms_multi_linear_supported(
        [weights.q, weights.k, weights.v, weights.attention_gate], g.model_dim)
    for fused in (False, True):
        cache = dl.LayerCache(g, cuda)
        cache.keys.copy_(bf16_tensor(keys, cuda))
        cache.values.copy_(bf16_tensor(values, cuda))
        results.append(dl.decode_layer(g, weights, cache, embedding, torch_().zeros_like(embedding),
                                       None, 150, workspace, fused_gate_up=fused,
                                       fused_input_norm=fused))
        results[-1] += (cache.keys.clone(), cache.values.clone())
    for separate, together in zip(results[0], results[1]):
        assert torch_().equal(separate, together)
    assert bool(torch_().isfinite(results[1][0]).all())


def test_model_sized_layer_fused_calls_and_verifier_families(cuda, oracle):
    """The fused forms and the two small-batch families on a layer of the benchmark's geometry
    (6,656 wide, 32 query heads over 2 key/value heads of 128, FFN 16,384, a 2,048-key ring;
    random packed bytes): launch grids, tiles per workgroup and rows per wave are those of the
    model, not of the small layers above.  One token: the fused gate/up call and the dual norm
    inside the Q/K/V/gate launch against the separate calls, bit for bit.  A block of 16: the
    `mmq` family with and without the norm handoff and the gate/up call, bit for bit; the exact
    verifier family against the token-at-a-time chain (projections bit-equal, attention to
    its summation order)."""
    from neuralfn_amd import decode_layer as dl
    rng = np.random.default_rng(29)
    g = dl.LayerGeometry(model_dim=6656, query_heads=32, kv_heads=2, head_dim=128, ffn_dim=16384,
                         sliding_window=2048)
    shapes = dict(q=(g.attention_dim, g.model_dim), k=(g.kv_dim, g.model_dim),
                  v=(g.kv_dim, g.model_dim), attention_gate=(g.attention_dim, g.model_dim),
                  output=(g.model_dim, g.attention_dim), mlp_gate=(g.ffn_dim, g.model_dim),
                  mlp_up=(g.ffn_dim, g.model_dim), mlp_down=(g.model_dim, g.ffn_dim))
    device = {}
    for index, (name, (out_dim, in_dim)) in enumerate(shapes.items()):
        device[name] = tile_ops.PackedWeight.from_numpy(
            kquant.Q4_K, random_packed(kquant.Q4_K, out_dim, in_dim, 300 + index), out_dim, in_dim)
    for name, width in dict(input_norm=g.model_dim, q_norm=g.head_dim, k_norm=g.head_dim,
                            post_attention_norm=g.model_dim, pre_feedforward_norm=g.model_dim,
                            post_feedforward_norm=g.model_dim).items():
        row = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)
        device[name] = tile_ops.PackedWeight.from_numpy(kquant.F32, row.view(np.uint8).copy(), 1, width)
    weights = dl.LayerWeights(**device)
    keys = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    values = oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))
    attention_workspace = engine_ops.gqa_decode_workspace(g.query_heads, g.head_dim)

    def cache():
        made = dl.LayerCache(g, cuda)
        made.keys.copy_(bf16_tensor(keys, cuda))
        made.values.copy_(bf16_tensor(values, cuda))
        return made

    rows, position = 16, 5000
    embeddings = to_device(rng.standard_normal((rows, g.model_dim)).astype(np.float32), cuda)
    one = tile_ops.small_batch_workspace(1, g.ffn_dim)
    serial_cache, serial = cache(), []
    for row in range(rows):
        results = []
        for fused in ((False, True) if row == 0 else (False,)):
            used = cache() if row == 0 else serial_cache
            results.append(dl.decode_layer(g, weights, used, embeddings[row:row + 1],
                                           torch_().zeros_like(embeddings[row:row + 1]), None,
                                           position + row, one, True, attention_workspace,
                                           fused_gate_up=fused, fused_input_norm=fused))
            if row == 0:
                results[-1] += (used.keys.clone(), used.values.clone())
        if row == 0:
            for separate, together in zip(results[0], results[1]):
                assert torch_().equal(separate, together), "one token: fused calls"
            serial_cache.keys.copy_(results[0][2])
            serial_cache.values.copy_(results[0][3])
        serial.append(results[0][0].cpu().numpy()[0])
    serial = np.stack(serial)

    block = tile_ops.small_batch_workspace(rows, g.ffn_dim)
    zero = torch_().zeros_like(embeddings)
    plain = dl.verify_layer(g, weights, cache(), embeddings, zero, None, position, block, True,
                            attention_workspace)
    fused = dl.verify_layer(g, weights, cache(), embeddings, zero, None, position, block, True,
                            attention_workspace, handoff=True, fused_gate_up=True)
    for a, b in zip(plain, fused):
        assert torch_().equal(a, b), "block of 16: handoff and gate/up call"
    exact = dl.verify_layer(g, weights, cache(), embeddings, zero, None, position, block, True,
                            attention_workspace, family="mmvq")
    handed = dl.verify_layer(g, weights, cache(), embeddings, zero, None, position, block, True,
                             attention_workspace, family="mmvq", handoff=True)
    for a, b in zip(exact, handed):
        assert torch_().equal(a, b), "block of 16, exact family: norm handoff"
    scale = float(np.max(np.abs(serial)))
    assert scale > 0 and np.isfinite(scale)
    assert float(np.max(np.abs(exact[0].cpu().numpy() - serial))) <= 1e-4 * scale
    assert float(np.max(np.abs(plain[0].cpu().numpy() - serial))) <= 2e-2 * scale


@pytest.mark.parametrize("split", [False, True])
def test_verifier_block_through_two_layers_equals_token_at_a_time_decode(cuda, oracle, split):
    """decode_layer.verify_layer runs a block of tokens through a layer in the batch forms of the
    operators with a causal block attention and no commit; every row must come out as the
    token-at-a-time chain (decode_layer, which commits) leaves it."""
    from neuralfn_amd import decode_layer as dl
    rng = np.random.default_rng(22)
    g = dl.LayerGeometry(model_dim=512, query_heads=8, kv_heads=2, head_dim=128, ffn_dim=768,
                         sliding_window=256)
    rows, position, layers = 5, 700, 2  # the ring has wrapped
    formats = dict(q=kquant.Q4_K, k=kquant.Q5_K, v=kquant.Q6_K, attention_gate=kquant.Q4_K,
                   output=kquant.Q5_K, mlp_gate=kquant.Q4_K, mlp_up=kquant.Q8_0, mlp_down=kquant.Q6_K)
    shapes = dict(q=(g.attention_dim, g.model_dim), k=(g.kv_dim, g.model_dim),
                  v=(g.kv_dim, g.model_dim), attention_gate=(g.attention_dim, g.model_dim),
                  output=(g.model_dim, g.attention_dim), mlp_gate=(g.ffn_dim, g.model_dim),
                  mlp_up=(g.ffn_dim, g.model_dim), mlp_down=(g.model_dim, g.ffn_dim))
    norms = dict(input_norm=g.model_dim, q_norm=g.head_dim, k_norm=g.head_dim,
                 post_attention_norm=g.model_dim, pre_feedforward_norm=g.model_dim,
                 post_feedforward_norm=g.model_dim)
    stack, rings = [], []
    for _ in range(layers):
        device = {}
        for name, (out_dim, in_dim) in shapes.items():
            packed = kquant.quantize(formats[name],
                                     (rng.standard_normal((out_dim, in_dim)) * 0.05).astype(np.float32))
            device[name] = tile_ops.PackedWeight.from_numpy(formats[name], packed, out_dim, in_dim)
        for name, width in norms.items():
            row = (1.0 + 0.1 * rng.standard_normal(width)).astype(np.float32)
            device[name] = tile_ops.PackedWeight.from_numpy(kquant.F32, row.view(np.uint8).copy(), 1, width)
        stack.append(dl.LayerWeights(**device))
        rings.append((oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32)),
                      oracle.to_bf16(rng.standard_normal((g.sliding_window, g.kv_dim)).astype(np.float32))))

    def caches():
        made = []
        for keys, values in rings:
            cache = dl.LayerCache(g, cuda)
            cache.keys.copy_(bf16_tensor(keys, cuda))
            cache.values.copy_(bf16_tensor(values, cuda))
            made.append(cache)
        return made

    embeddings = rng.standard_normal((rows, g.model_dim)).astype(np.float32)
    attention_workspace = engine_ops.gqa_decode_workspace(g.query_heads, g.head_dim) if split else None

    # token at a time, committing
    serial_caches = caches()
    workspace = tile_ops.small_batch_workspace(1, max(g.model_dim, g.ffn_dim, g.attention_dim))
    serial_down, serial_hidden = [], []
    for row in range(rows):
        pending = to_device(embeddings[row:row + 1], cuda)
        residual, pending_norm = torch_().zeros_like(pending), None
        for weights, cache in zip(stack, serial_caches):
            pending, residual = dl.decode_layer(g, weights, cache, pending, residual, pending_norm,
                                                position + row, workspace, True, attention_workspace)
            pending_norm = weights.post_feedforward_norm
        serial_down.append(pending.cpu().numpy()[0])
        serial_hidden.append(residual.cpu().numpy()[0])

    # the block, then the commit of all its rows
    block_caches = caches()
    workspace = tile_ops.small_batch_workspace(rows, max(g.model_dim, g.ffn_dim, g.attention_dim))
    pending = to_device(embeddings, cuda)
    residual, pending_norm = torch_().zeros_like(pending), None
    staged = []
    for weights, cache in zip(stack, block_caches):
        pending, residual, key_rows, value_rows = dl.verify_layer(
            g, weights, cache, pending, residual, pending_norm, position, workspace, True,
            attention_workspace)
        pending_norm = weights.post_feedforward_norm
        staged.append((key_rows, value_rows))

    # the same block with the dual norms handing their output to the projections in the
    # small-batch workspace: two launches less per layer, the same bits
    handed_pending = to_device(embeddings, cuda)
    handed_residual, pending_norm = torch_().zeros_like(handed_pending), None
    for weights, cache, (key_rows, value_rows) in zip(stack, caches(), staged):
        handed_pending, handed_residual, handed_keys, handed_values = dl.verify_layer(
            g, weights, cache, handed_pending, handed_residual, pending_norm, position, workspace,
            True, attention_workspace, handoff=True)
        pending_norm = weights.post_feedforward_norm
        assert torch_().equal(handed_keys, key_rows) and torch_().equal(handed_values, value_rows)
    assert torch_().equal(handed_pending, pending) and torch_().equal(handed_residual, residual)

    # ... and with gate and up in the one call that stores swiglu(gate, up), with and without
    # the handoff: the same bits again
    for handoff in (False, True):
        fused_pending = to_device(embeddings, cuda)
        fused_residual, pending_norm = torch_().zeros_like(fused_pending), None
        for weights, cache in zip(stack, caches()):
            fused_pending, fused_residual, _, _ = dl.verify_layer(
                g, weights, cache, fused_pending, fused_residual, pending_norm, position, workspace,
                True, attention_workspace, handoff=handoff, fused_gate_up=True)
            pending_norm = weights.post_feedforward_norm
        assert torch_().equal(fused_pending, pending) and torch_().equal(fused_residual, residual)

    def error(actual, expected):
        return float(np.max(np.abs(actual - expected)) / np.max(np.abs(expected)))

    # the exact verifier's family: every projection of the block carries the one-row kernel's
    # bits, so what is left between the block and the serial chain is the summation order of
    # the attention kernels (none while both run on the vector kernel)
    exact_pending = to_device(embeddings, cuda)
    exact_residual, pending_norm = torch_().zeros_like(exact_pending), None
    for weights, cache in zip(stack, caches()):
        exact_pending, exact_residual, _, _ = dl.verify_layer(
            g, weights, cache, exact_pending, exact_residual, pending_norm, position, workspace,
            True, attention_workspace, family="mmvq")
        pending_norm = weights.post_feedforward_norm
    # (the two attention forms cut the keys into shares differently, so their partial sums meet
    # in another order; where such a last-bit difference moves an activation across a
    # quantization step of the next projection (16-bit codes: 3e-5 of a block's largest value)
    # it grows to that size, and two layers leave about 1e-4)
    assert error(exact_residual.cpu().numpy(), np.stack(serial_hidden)) <= 3e-4
    assert error(exact_pending.cpu().numpy(), np.stack(serial_down)) <= 3e-4

    # the projections of a block (fp16 weights and activations on the matrix cores, 11
    # significant bits each) and of one token (integer codes against 16-bit activation codes)
    # run in different kernels: each within 2e-3 of the float formula, and after two layers
    # about 1e-3 apart
    assert error(residual.cpu().numpy(), np.stack(serial_hidden)) <= 2e-3
    assert error(pending.cpu().numpy(), np.stack(serial_down)) <= 2e-3
    for cache, serial_cache, (key_rows, value_rows) in zip(block_caches, serial_caches, staged):
        engine_ops.cache_commit(key_rows, value_rows, cache.keys, cache.values, position, rows=rows)
        # committed rows carry the upstream rounding differences: a bf16 step apart at most
        for ours, theirs in ((cache.keys, serial_cache.keys), (cache.values, serial_cache.values)):
            ours = oracle.bf16_to_float(bits_of(ours)).astype(np.float64)
            theirs = oracle.bf16_to_float(bits_of(theirs)).astype(np.float64)
            assert np.max(np.abs(ours - theirs)) <= 2.0 ** -7 * np.max(np.abs(theirs))
