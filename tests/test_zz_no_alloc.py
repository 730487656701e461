"""nfn_mi355_lm_head_argmax_no_alloc_v1: the fused lm_head argmax without a workspace argument,
for callers that cannot allocate.  Through the C ABI, against nfn_mi355_lm_head_argmax_v1 (same
kernels: the bits must be equal) and against the oracle, on two calls in a row of which the second
is smaller, so that what the first left in the library's scratch must not matter."""
import ctypes

import numpy as np
import pytest

from neuralfn_amd import kquant, tile_ops

pytestmark = pytest.mark.gpu


def _case(cuda, oracle, encoding, rows, out_dim, in_dim, seed):
    import torch
    packed = kquant.quantize(encoding, kquant.synthetic_weights(seed, out_dim, in_dim))
    x = kquant.synthetic_activations(seed + 1, rows, in_dim)
    weight = tile_ops.PackedWeight.from_numpy(encoding, packed, out_dim, in_dim)
    device_x = torch.from_numpy(x).to(cuda)
    indices = torch.full((rows,), -7, dtype=torch.int64, device=cuda)
    maxima = torch.full((rows,), float("nan"), dtype=torch.float32, device=cuda)
    # a first call, so that what a kernel's first launch loads (code objects) is resident; the
    # measured call then must neither move torch's allocator nor the device's free memory (a
    # hipMalloc inside the library would not show in the former)
    tile_ops.lm_head_argmax_no_alloc(weight, device_x, indices, maxima)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated(cuda)
    free_before, _ = torch.cuda.mem_get_info(cuda)
    indices.fill_(-7)
    tile_ops.lm_head_argmax_no_alloc(weight, device_x, indices, maxima)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info(cuda)
    assert torch.cuda.memory_allocated(cuda) == before
    assert free_after == free_before, "device memory was allocated or freed during the call"
    expected_indices, expected_maxima = tile_ops.lm_head_argmax(weight, device_x)
    assert torch.equal(indices, expected_indices)
    assert np.array_equal(maxima.cpu().numpy().view(np.uint32),
                          expected_maxima.cpu().numpy().view(np.uint32))
    logits = oracle.linear(encoding, packed, out_dim, in_dim, x)
    for row in range(rows):
        ordered = np.sort(logits[row])
        if ordered[-1] - ordered[-2] > 4e-3 * np.max(np.abs(logits[row])):  # not a near tie
            assert int(indices[row]) == oracle.argmax(logits[row])
        assert abs(float(maxima[row]) - logits[row].max()) <= 2e-3 * np.max(np.abs(logits[row]))


@pytest.mark.parametrize("encoding", [kquant.Q6_K, kquant.Q4_K])
def test_two_calls_in_a_row_second_smaller(cuda, oracle, encoding):
    _case(cuda, oracle, encoding, 4, 4160, 1024, 900 + encoding)   # many workgroups, four rows
    _case(cuda, oracle, encoding, 1, 520, 1024, 950 + encoding)    # fewer candidates, one row
    _case(cuda, oracle, encoding, 8, 96, 512, 970 + encoding)      # eight rows, a few tiles
    _case(cuda, oracle, encoding, 16, 4160, 1024, 980 + encoding)  # sixteen rows, a tile per workgroup
    _case(cuda, oracle, encoding, 5, 40, 256, 990 + encoding)      # five rows, three tiles


def test_full_vocabulary_fits_and_larger_is_refused(cuda):
    import torch
    lib = tile_ops.load()
    assert lib.nfn_mi355_lm_head_argmax_workspace_bytes_v1(8, 202048) <= tile_ops.LM_HEAD_NO_ALLOC_SCRATCH_BYTES
    assert lib.nfn_mi355_lm_head_argmax_workspace_bytes_v1(16, 202048) <= tile_ops.LM_HEAD_NO_ALLOC_SCRATCH_BYTES
    # a vocabulary whose candidates do not fit: refused before anything is launched or read
    out_dim, in_dim = 300_000, 256
    assert lib.nfn_mi355_lm_head_argmax_workspace_bytes_v1(8, out_dim) > tile_ops.LM_HEAD_NO_ALLOC_SCRATCH_BYTES
    descriptor = tile_ops.make_descriptor(kquant.Q4_K, 0x1000, out_dim, in_dim)
    indices = torch.full((8,), -7, dtype=torch.int64, device=cuda)
    maxima = torch.zeros(8, dtype=torch.float32, device=cuda)
    x = torch.zeros((8, in_dim), dtype=torch.float32, device=cuda)
    status = lib.nfn_mi355_lm_head_argmax_no_alloc_v1(
        ctypes.byref(descriptor), x.data_ptr(), indices.data_ptr(), maxima.data_ptr(), 8, None)
    assert status == tile_ops.STATIC_SCRATCH_EXCEEDED
    assert b"scratch" in lib.nfn_native_tile_ops_error_string(status)
    assert lib.nfn_mi355_lm_head_argmax_no_alloc_v1(
        ctypes.byref(descriptor), x.data_ptr(), indices.data_ptr(), maxima.data_ptr(), 17, None) == 1
    assert lib.nfn_mi355_lm_head_argmax_no_alloc_v1(
        None, x.data_ptr(), indices.data_ptr(), maxima.data_ptr(), 1, None) == 1
    torch.cuda.synchronize()
    assert int(indices[0]) == -7
