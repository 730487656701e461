"""The GGUF tensor-table reader (include/nfn_mi355_gguf.h) without a GPU.

The files are written here from the format's definition (GGUF version 3, as the
reference reads it: neuralfn/csrc/native_gpt2/resident_glimmer.cpp:976-1160,
neuralfn/native_gguf.py:60-99), not by the code under test.
"""
import ctypes
import re
import struct
from pathlib import Path

import numpy as np
import pytest

from neuralfn_amd import gguf, kquant

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "nfn_mi355_gguf.h"

# metadata value types
U8, I8, U16, I16, U32, I32, F32V, BOOL, STRING, ARRAY, U64, I64, F64 = range(13)


def _string(text: str) -> bytes:
    raw = text.encode()
    return struct.pack("<Q", len(raw)) + raw


def _value(kind: int, value) -> bytes:
    formats = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32V: "<f",
               BOOL: "<B", U64: "<Q", I64: "<q", F64: "<d"}
    if kind == STRING:
        return _string(value)
    if kind == ARRAY:
        element, items = value
        return struct.pack("<IQ", element, len(items)) + b"".join(_value(element, i) for i in items)
    return struct.pack(formats[kind], value)


def write_gguf(path, tensors, metadata=(), version=3, padding_byte=0, tail=b"",
               offsets=None, magic=b"GGUF"):
    """tensors: (name, encoding, dims (ne order), bytes).  Returns the data offset."""
    header = magic + struct.pack("<IQQ", version, len(tensors), len(metadata))
    for key, kind, value in metadata:
        header += _string(key) + struct.pack("<I", kind) + _value(kind, value)
    data = b""
    placed = []
    for index, (name, encoding, dims, raw) in enumerate(tensors):
        offset = len(data) if offsets is None else offsets[index]
        placed.append(offset)
        data += bytes(raw)
        data += b"\0" * (-len(data) % 32)
    for (name, encoding, dims, raw), offset in zip(tensors, placed):
        header += _string(name) + struct.pack("<I", len(dims))
        header += b"".join(struct.pack("<Q", d) for d in dims)
        header += struct.pack("<IQ", encoding, offset)
    data_offset = (len(header) + 31) // 32 * 32
    header += bytes([padding_byte]) * (data_offset - len(header))
    # no bytes after the last tensor: its alignment padding is not written
    last = tensors[-1][3]
    data = data[:len(data) - (-len(bytes(last)) % 32)] if offsets is None else data
    Path(path).write_bytes(header + data + tail)
    return data_offset


def sample_tensors(seed=3):
    rng = np.random.default_rng(seed)
    tensors = []
    for name, encoding, rows, cols in (
            ("blk.0.attn_q.weight", kquant.Q4_K, 6, 512), ("blk.0.attn_k.weight", kquant.Q5_K, 3, 256),
            ("output.weight", kquant.Q6_K, 5, 768), ("blk.0.ffn_down.weight", kquant.Q8_0, 4, 96),
            ("blk.0.attn_norm.weight", kquant.F32, 1, 40), ("token_embd.weight", kquant.BF16, 7, 24)):
        nbytes = kquant.packed_nbytes(encoding, rows, cols)
        raw = rng.integers(0, 256, nbytes, dtype=np.uint8)
        dims = (cols,) if rows == 1 else (cols, rows)
        tensors.append((name, encoding, dims, raw))
    return tensors


METADATA = [
    ("general.architecture", STRING, "muse-glimmer"), ("muse-glimmer.block_count", U32, 52),
    ("muse-glimmer.rope.freq_base", F32V, 500000.0), ("tokenizer.ggml.add_bos_token", BOOL, 1),
    ("tokenizer.ggml.tokens", ARRAY, (STRING, ["a", "bc", ""])),
    ("muse-glimmer.attention.sliding_window_pattern", ARRAY, (BOOL, [1, 1, 1, 0])),
    ("general.file_type", U64, 15), ("x.i8", I8, -3), ("x.u16", U16, 65535), ("x.i16", I16, -2),
    ("x.i32", I32, -7), ("x.i64", I64, -9), ("x.f64", F64, 0.25), ("x.u8", U8, 200),
    ("x.nested", ARRAY, (ARRAY, [(U32, [1, 2]), (U32, [])])),
]


def test_header_symbols_are_exported():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    names = sorted(set(re.findall(r"\b(nfn_mi355_gguf_[a-z0-9_]+)\s*\(", text)))
    assert len(names) == 8
    lib = gguf._load()
    for name in names:
        assert hasattr(lib, name), f"{name} is declared but not exported"
    assert ctypes.sizeof(gguf._Tensor) == 56


def test_tensor_table_and_bytes(tmp_path):
    tensors = sample_tensors()
    path = tmp_path / "model.gguf"
    data_offset = write_gguf(path, tensors, METADATA)
    with gguf.GgufFile(path) as file:
        assert len(file) == len(tensors) and file.metadata_count == len(METADATA)
        expected_offset = data_offset
        for found, (name, encoding, dims, raw) in zip(file, tensors):
            rows = dims[1] if len(dims) == 2 else 1
            elements, block_bytes = kquant.BLOCKS[encoding]
            assert (found.name, found.encoding, found.rank) == (name, encoding, len(dims))
            assert (found.rows, found.cols) == (rows, dims[0])
            assert found.row_stride_bytes == dims[0] // elements * block_bytes
            assert found.nbytes == raw.size and found.file_offset == expected_offset
            assert np.array_equal(file.bytes_of(found), raw)
            assert file.find(name) == found
            expected_offset += (raw.size + 31) // 32 * 32
        with pytest.raises(gguf.GgufError) as error:
            file.find("missing.weight")
        assert error.value.code == 15


def test_file_order_need_not_be_offset_order(tmp_path):
    tensors = sample_tensors()[:3]
    sizes = [(t[3].size + 31) // 32 * 32 for t in tensors]
    # second tensor's bytes first in the data section
    offsets = [sizes[1], 0, sizes[0] + sizes[1]]
    path = tmp_path / "reordered.gguf"
    header_only = write_gguf(path, tensors, offsets=offsets)
    blob = bytearray(path.read_bytes()[:header_only])
    blob += bytes(tensors[1][3]) + b"\0" * (sizes[1] - tensors[1][3].size)
    blob += bytes(tensors[0][3]) + b"\0" * (sizes[0] - tensors[0][3].size)
    blob += bytes(tensors[2][3])
    path.write_bytes(blob)
    with gguf.GgufFile(path) as file:
        for found, (name, _, _, raw) in zip(file, tensors):
            assert np.array_equal(file.bytes_of(found), raw), name


def _expect(path, code):
    with pytest.raises(gguf.GgufError) as error:
        gguf.GgufFile(path)
    assert error.value.code == code, error.value


def test_malformed_files_are_refused(tmp_path):
    tensors = sample_tensors()
    path = tmp_path / "bad.gguf"
    write_gguf(path, tensors, magic=b"GGUX")
    _expect(path, 4)
    write_gguf(path, tensors, version=2)
    _expect(path, 5)
    write_gguf(path, tensors, METADATA, padding_byte=1)
    _expect(path, 12)
    write_gguf(path, tensors, tail=b"\0")
    _expect(path, 14)
    good = tmp_path / "good.gguf"
    write_gguf(good, tensors, METADATA)
    blob = good.read_bytes()
    path.write_bytes(blob[:-1])              # last tensor cut short
    _expect(path, 13)
    path.write_bytes(blob[:40])              # ends inside the header
    _expect(path, 3)
    write_gguf(path, [tensors[0], tensors[0]])
    _expect(path, 11)
    name, encoding, dims, raw = tensors[0]
    write_gguf(path, [(name, 2, dims, raw)])                     # Q4_0: no layout here
    _expect(path, 9)
    write_gguf(path, [(name, encoding, (dims[0], dims[1], 1), raw)])
    _expect(path, 7)
    write_gguf(path, [(name, encoding, (500, 6), raw)])          # not a multiple of 256
    _expect(path, 8)
    write_gguf(path, [(name, encoding, (0, 6), raw)])
    _expect(path, 8)
    write_gguf(path, tensors[:2], offsets=[0, 8])
    _expect(path, 10)
    sizes = [(t[3].size + 31) // 32 * 32 for t in tensors[:2]]
    write_gguf(path, tensors[:2], offsets=[0, sizes[0] + 32])    # a hole between the tensors
    _expect(path, 13)
    write_gguf(path, tensors[:1], [("bad", U32, 0)])
    blob = bytearray(path.read_bytes())
    blob[24 + 8 + 3:24 + 8 + 3 + 4] = struct.pack("<I", 13)      # metadata type out of range
    path.write_bytes(blob)
    _expect(path, 6)
    _expect(tmp_path / "absent.gguf", 2)
    # a header that claims more tensors (or metadata entries) than the file has bytes for is
    # refused before anything is reserved for them
    write_gguf(good, tensors, METADATA)
    for field_offset in (8, 16):
        blob = bytearray(good.read_bytes())
        blob[field_offset:field_offset + 8] = struct.pack("<Q", len(blob) // 32 + 1)
        path.write_bytes(blob)
        _expect(path, 3)
        blob[field_offset:field_offset + 8] = struct.pack("<Q", (1 << 63) - 1)
        path.write_bytes(blob)
        _expect(path, 3)


@pytest.mark.gpu
def test_weights_loaded_from_a_file_match_the_oracle(tmp_path, oracle):
    import torch
    from neuralfn_amd import tile_ops
    in_dim = 512
    specs = [("blk.0.attn_q.weight", kquant.Q4_K, 64), ("blk.0.attn_v.weight", kquant.Q6_K, 24),
             ("blk.0.ffn_down.weight", kquant.Q8_0, 40)]
    tensors = []
    for index, (name, encoding, rows) in enumerate(specs):
        packed = kquant.quantize(encoding, kquant.synthetic_weights(300 + index, rows, in_dim))
        tensors.append((name, encoding, (in_dim, rows), packed))
    path = tmp_path / "weights.gguf"
    write_gguf(path, tensors, METADATA)
    x = kquant.synthetic_activations(301, 1, in_dim)
    device = torch.device("cuda:0")
    with gguf.GgufFile(path) as file:
        weights = [file.packed_weight(name, device) for name, _, _ in specs]
    workspace = tile_ops.small_batch_workspace(1, in_dim)
    outputs = tile_ops.multi_linear(weights, torch.from_numpy(x).to(device), workspace)
    for (name, encoding, rows), (_, _, _, packed), y in zip(specs, tensors, outputs):
        expected = oracle.linear(encoding, packed, rows, in_dim, x)
        error = np.max(np.abs(y.cpu().numpy() - expected)) / np.max(np.abs(expected))
        assert error <= 2e-3, name
