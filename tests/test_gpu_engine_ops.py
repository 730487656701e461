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


@pytest.mark.parametrize("context,capacity,rows", [(32, 64, 16), (1000, 2048, 24), (2040, 4096, 12)])
def test_causal_block_is_token_at_a_time_decode_bit_for_bit(cuda, oracle, context, capacity, rows):
    """The verifier's rule (probe :2683-2745): a causal block sees earlier block rows as the
    bf16 cache would hold them, and each row equals one-token attention followed by the commit."""
    rng = np.random.default_rng(context)
    query_heads, kv_heads, head_dim = 32, 8, 128
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
    assert_bits_equal(block, serial)


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
