"""What pins the oracle's restatement of the decode loop's operators around the linears.

Rotary embedding, bf16 rounding, attention over a bf16 cache, the logit
transform: each against the compiled reference where it builds (the CPU
engine's apply_rope; the reference's CPU stand-in for its sidecar,
tests/cpp/fake_glimmer_tile_ops.cpp) and against what the mathematics fixes.
"""
import numpy as np
import pytest

needs_ref = pytest.mark.skipif(
    not __import__("oracle.kquant_oracle", fromlist=["x"]).reference_available(),
    reason="reference harness not built (no reference checkout here)")
needs_sidecar_ref = pytest.mark.skipif(
    not __import__("oracle.kquant_oracle", fromlist=["x"]).sidecar_reference_available(),
    reason="reference CPU sidecar not built (no reference checkout here)")


def _cache(rng, capacity, width, oracle):
    return oracle.to_bf16(rng.standard_normal((capacity, width)).astype(np.float32))


# ---- rotary position embedding -------------------------------------------------

@needs_ref
@pytest.mark.parametrize("interleaved", [False, True])
def test_rope_equals_the_compiled_reference(oracle, interleaved):
    rng = np.random.default_rng(3)
    for heads, head_dim, position, theta in ((32, 128, 2051, 500000.0), (2, 128, 0, 500000.0),
                                             (5, 64, 131071, 10000.0), (3, 6, 17, 100.0)):
        x = rng.standard_normal((heads, head_dim)).astype(np.float32)
        assert np.array_equal(oracle.rope(x, position, theta, interleaved),
                              oracle.ref_apply_rope(x, position, theta, interleaved))


@needs_ref
def test_qk_norm_equals_the_compiled_reference(oracle):
    rng = np.random.default_rng(10)
    for heads, head_dim in ((32, 128), (2, 128), (5, 64), (3, 6)):
        x = (rng.standard_normal((heads, head_dim)) * 3.0).astype(np.float32)
        weight = (1.0 + 0.2 * rng.standard_normal(head_dim)).astype(np.float32)
        assert np.array_equal(oracle.qk_norm(x, None, 1e-5, 1.0), oracle.ref_qk_norm(x, None, 1e-5, 1.0))
        assert np.array_equal(oracle.qk_norm(x, weight, 1e-6, 3.87),
                              oracle.ref_qk_norm(x, weight, 1e-6, 3.87))


def test_qk_norm_closed_forms(oracle):
    # a head of equal values v normalises to sign(v) / sqrt(1 + eps / v^2); scaling the input changes nothing
    x = np.full((2, 64), 3.0, dtype=np.float32)
    x[1] = -0.5
    y = oracle.qk_norm(x, None, 1e-5, 2.0)
    assert np.allclose(y[0], 2.0 / np.sqrt(1.0 + 1e-5 / 9.0), rtol=1e-7)
    assert np.allclose(y[1], -2.0 / np.sqrt(1.0 + 1e-5 / 0.25), rtol=1e-7)
    rng = np.random.default_rng(11)
    z = rng.standard_normal((3, 128)).astype(np.float32)
    unit = oracle.qk_norm(z, None, 1e-12, 1.0)
    assert np.allclose((unit.astype(np.float64) ** 2).mean(axis=1), 1.0, rtol=1e-6)
    assert np.allclose(oracle.qk_norm(z * 8.0, None, 1e-12, 1.0), unit, rtol=1e-6)


def test_rope_is_a_rotation(oracle):
    rng = np.random.default_rng(4)
    x = rng.standard_normal((4, 128)).astype(np.float32)
    assert np.array_equal(oracle.rope(x, 0, 500000.0), x)  # angle 0
    y = oracle.rope(x, 977, 500000.0)
    # each pair keeps its length
    assert np.allclose(y[:, :64] ** 2 + y[:, 64:] ** 2, x[:, :64] ** 2 + x[:, 64:] ** 2, rtol=1e-5)
    assert np.allclose(oracle.rope(y, 977, 500000.0, inverse=True), x, atol=1e-6)
    # pair 0 turns by exactly `position` radians: (1, 0) -> (cos p, sin p)
    unit = np.zeros((1, 128), dtype=np.float32)
    unit[0, 0] = 1.0
    turned = oracle.rope(unit, 3, 500000.0)
    assert turned[0, 0] == np.float32(np.cos(3.0)) and turned[0, 64] == np.float32(np.sin(3.0))
    # the last pair turns by position / theta^((d-2)/d)
    unit[:] = 0.0
    unit[0, 63] = 1.0
    turned = oracle.rope(unit, 1000, 500000.0)
    angle = 1000.0 / 500000.0 ** (126.0 / 128.0)
    assert turned[0, 63] == np.float32(np.cos(angle)) and turned[0, 127] == np.float32(np.sin(angle))
    # the interleaved layout is the same rotation on pairs (2i, 2i+1)
    shuffled = np.empty_like(x)
    shuffled[:, 0::2], shuffled[:, 1::2] = x[:, :64], x[:, 64:]
    z = oracle.rope(shuffled, 977, 500000.0, interleaved=True)
    assert np.array_equal(z[:, 0::2], y[:, :64]) and np.array_equal(z[:, 1::2], y[:, 64:])


# ---- bf16 ---------------------------------------------------------------------

def test_bf16_rounds_to_nearest_even(oracle):
    cases = {
        1.0: 0x3F80,
        1.0 + 2.0 ** -8: 0x3F80,        # tie, even mantissa below
        1.0 + 3.0 * 2.0 ** -8: 0x3F82,  # tie, even mantissa above
        1.0 + 2.0 ** -8 + 2.0 ** -20: 0x3F81,
        -2.5: 0xC020,
        0.0: 0x0000,
        float("inf"): 0x7F80,
        3.3895313892515355e38: 0x7F7F,  # the largest bf16 stays
        3.4028234663852886e38: 0x7F80,  # the largest float rounds up to infinity
    }
    for value, bits in cases.items():
        assert oracle.to_bf16_scalar(value) == bits, value
    assert oracle.to_bf16_scalar(float("nan")) & 0x7FC0 == 0x7FC0
    # every bf16 value is a fixed point; the vector form equals the scalar one
    patterns = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    finite = (patterns & 0x7F80) != 0x7F80
    assert np.array_equal(oracle.to_bf16(oracle.bf16_to_float(patterns))[finite], patterns[finite])
    rng = np.random.default_rng(5)
    x = (rng.standard_normal(4096) * 10.0 ** rng.integers(-20, 20, 4096)).astype(np.float32)
    assert np.array_equal(oracle.to_bf16(x),
                          np.array([oracle.to_bf16_scalar(v) for v in x], dtype=np.uint16))


# ---- attention -----------------------------------------------------------------

@needs_sidecar_ref
def test_attention_equals_the_reference_cpu_sidecar(oracle):
    rng = np.random.default_rng(6)
    query_heads, kv_heads, head_dim, capacity = 8, 2, 64, 96
    width = kv_heads * head_dim
    key_cache, value_cache = _cache(rng, capacity, width, oracle), _cache(rng, capacity, width, oracle)
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    for position, first in ((150, 70), (40, 0), (95, 95)):
        ours = oracle.gqa_decode(query, key, value, key_cache, value_cache, position, first, 0.125)
        theirs = oracle.ref_sidecar_gqa_decode(query, key, value, key_cache, value_cache, position,
                                               first, 0.125)
        assert np.abs(ours - theirs).max() < 2e-7
    rows, block_rows = 5, 7
    block_query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((block_rows, kv_heads, head_dim)).astype(np.float32)
    for context, window in ((150, 60), (20, 90), (0, 4)):
        ours = oracle.block_attention(block_query, block_key, block_value, key_cache, value_cache,
                                      context, window, 0.125, False)
        theirs = oracle.ref_sidecar_block_attention(block_query, block_key, block_value, key_cache,
                                                    value_cache, context, window, 0.125, False)
        assert np.abs(ours - theirs).max() < 2e-7
        # The stand-in keeps earlier block rows in float where the device kernel
        # (kernels.cu:2983-2990) rounds them to bf16; on bf16-valued rows the two agree.
        rounded_key = oracle.bf16_to_float(oracle.to_bf16(block_key))
        rounded_value = oracle.bf16_to_float(oracle.to_bf16(block_value))
        ours = oracle.block_attention(block_query, rounded_key, rounded_value, key_cache,
                                      value_cache, context, window, 0.125, True)
        theirs = oracle.ref_sidecar_block_attention(block_query, rounded_key, rounded_value,
                                                    key_cache, value_cache, context, window, 0.125,
                                                    True)
        assert np.abs(ours - theirs).max() < 2e-7


def test_attention_closed_forms(oracle):
    rng = np.random.default_rng(7)
    query_heads, kv_heads, head_dim, capacity = 4, 2, 32, 16
    width = kv_heads * head_dim
    key_cache, value_cache = _cache(rng, capacity, width, oracle), _cache(rng, capacity, width, oracle)
    query = rng.standard_normal((query_heads, head_dim)).astype(np.float32)
    key = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    value = rng.standard_normal((kv_heads, head_dim)).astype(np.float32)
    # one key: the output is its value, whatever the score (heads 0,1 -> kv 0; 2,3 -> kv 1)
    out = oracle.gqa_decode(query, key, value, key_cache, value_cache, 9, 9, 0.3)
    assert np.array_equal(out, value[[0, 0, 1, 1]])
    # a zero query scores every key alike: the output is the mean of the values
    out = oracle.gqa_decode(np.zeros_like(query), key, value, key_cache, value_cache, 5, 2, 0.3)
    cached = oracle.bf16_to_float(value_cache).reshape(capacity, kv_heads, head_dim)
    mean = (cached[2:5].astype(np.float64).sum(0) + value) / 4.0
    assert np.allclose(out, mean[[0, 0, 1, 1]], rtol=0, atol=1e-7)
    # a key that dominates takes everything: current key = 100 * query of head 0
    big = key.copy()
    big[0] = 100.0 * query[0]
    out = oracle.gqa_decode(query, big, value, key_cache, value_cache, 5, 0, 1.0)
    assert np.allclose(out[0], value[0], atol=1e-6)
    # the ring: position p lives in row p % capacity
    out_a = oracle.gqa_decode(query, key, value, key_cache, value_cache, 3 + capacity, 1 + capacity, 0.3)
    out_b = oracle.gqa_decode(query, key, value, key_cache, value_cache, 3, 1, 0.3)
    assert np.array_equal(out_a, out_b)


def test_causal_block_equals_token_at_a_time_decode(oracle):
    """The rule of the reference's probe (muse_glimmer_cuda_kernel_probe.cpp:2683-2745)."""
    rng = np.random.default_rng(8)
    rows, query_heads, kv_heads, head_dim, capacity, context = 6, 8, 2, 32, 64, 20
    width = kv_heads * head_dim
    key_cache, value_cache = _cache(rng, capacity, width, oracle), _cache(rng, capacity, width, oracle)
    query = rng.standard_normal((rows, query_heads, head_dim)).astype(np.float32)
    block_key = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    block_value = rng.standard_normal((rows, kv_heads, head_dim)).astype(np.float32)
    block = oracle.block_attention(query, block_key, block_value, key_cache, value_cache, context,
                                   capacity, 0.2, True)
    for row in range(rows):
        serial = oracle.gqa_decode(query[row], block_key[row], block_value[row], key_cache,
                                   value_cache, context + row, 0, 0.2)
        assert np.array_equal(serial, block[row])
        key_cache[(context + row) % capacity] = oracle.to_bf16(block_key[row].reshape(-1))
        value_cache[(context + row) % capacity] = oracle.to_bf16(block_value[row].reshape(-1))
    # not causal: row r also sees later block rows, in float
    full = oracle.block_attention(query, block_key, block_value, key_cache[:capacity],
                                  value_cache[:capacity], context, capacity, 0.2, False)
    assert not np.array_equal(full[0], block[0])


# ---- logit transform -------------------------------------------------------------

def test_logit_transform_closed_forms(oracle):
    x = np.array([0.0, 1.0, -1.0, 20.0 / 1.5, 1e6, -1e6, 1e-4], dtype=np.float32)
    y = oracle.logit_transform(x, 1.5, 20.0)
    assert y[0] == 0.0 and y[1] == -y[2]
    assert y[3] == np.float32(20.0 * np.tanh(np.float64(1.5) * np.float64(x[3]) / 20.0))
    assert y[4] == np.float32(20.0) and y[5] == np.float32(-20.0)
    assert abs(y[6] / x[6] - 1.5) < 1e-6  # slope `multiplier` at 0
    rng = np.random.default_rng(9)
    z = (rng.standard_normal(1000) * 30).astype(np.float32)
    expected = (20.0 * np.tanh(1.5 * z.astype(np.float64) / 20.0)).astype(np.float32)
    assert np.array_equal(oracle.logit_transform(z, 1.5, 20.0), expected)
