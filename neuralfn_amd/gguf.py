"""GGUF tensor tables as packed weights (host side, ctypes over include/nfn_mi355_gguf.h).

The reader is the structural part of the reference's loaders
(neuralfn/csrc/native_gpt2/resident_glimmer.cpp:976-1160, neuralfn/native_gguf.py);
a tensor's bytes are used as they lie in the file, `row r` at `offset + r * row_stride_bytes`.
"""
from __future__ import annotations

import ctypes
from dataclasses import dataclass
from pathlib import Path
from typing import Iterator, Optional

import numpy as np

from .build import HOST_LIB


class _Tensor(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char_p), ("encoding", ctypes.c_uint32), ("rank", ctypes.c_uint32),
                ("rows", ctypes.c_int64), ("cols", ctypes.c_int64),
                ("row_stride_bytes", ctypes.c_int64), ("nbytes", ctypes.c_int64),
                ("file_offset", ctypes.c_uint64)]


_lib: Optional[ctypes.CDLL] = None


def _load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not HOST_LIB.exists():
            raise FileNotFoundError(f"{HOST_LIB} is not built: run python -m neuralfn_amd.build")
        lib = ctypes.CDLL(str(HOST_LIB))
        lib.nfn_mi355_gguf_open_v1.argtypes = [ctypes.c_char_p, ctypes.POINTER(ctypes.c_void_p)]
        lib.nfn_mi355_gguf_open_v1.restype = ctypes.c_int
        lib.nfn_mi355_gguf_close_v1.argtypes = [ctypes.c_void_p]
        lib.nfn_mi355_gguf_close_v1.restype = None
        lib.nfn_mi355_gguf_tensor_count_v1.argtypes = [ctypes.c_void_p]
        lib.nfn_mi355_gguf_tensor_count_v1.restype = ctypes.c_int64
        lib.nfn_mi355_gguf_metadata_count_v1.argtypes = [ctypes.c_void_p]
        lib.nfn_mi355_gguf_metadata_count_v1.restype = ctypes.c_int64
        lib.nfn_mi355_gguf_tensor_v1.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.POINTER(_Tensor)]
        lib.nfn_mi355_gguf_tensor_v1.restype = ctypes.c_int
        lib.nfn_mi355_gguf_find_v1.argtypes = [ctypes.c_void_p, ctypes.c_char_p, ctypes.POINTER(_Tensor)]
        lib.nfn_mi355_gguf_find_v1.restype = ctypes.c_int
        lib.nfn_mi355_gguf_data_v1.argtypes = [ctypes.c_void_p, ctypes.POINTER(ctypes.c_uint64)]
        lib.nfn_mi355_gguf_data_v1.restype = ctypes.c_void_p
        lib.nfn_mi355_gguf_error_string.argtypes = [ctypes.c_int]
        lib.nfn_mi355_gguf_error_string.restype = ctypes.c_char_p
        _lib = lib
    return _lib


class GgufError(ValueError):
    def __init__(self, code: int):
        self.code = code
        super().__init__(f"GGUF error {code}: {_load().nfn_mi355_gguf_error_string(code).decode()}")


@dataclass(frozen=True)
class GgufTensor:
    name: str
    encoding: int
    rank: int
    rows: int
    cols: int
    row_stride_bytes: int
    nbytes: int
    file_offset: int


def _convert(raw: _Tensor) -> GgufTensor:
    return GgufTensor(raw.name.decode(), raw.encoding, raw.rank, raw.rows, raw.cols,
                      raw.row_stride_bytes, raw.nbytes, raw.file_offset)


class GgufFile:
    """An open GGUF file: its tensor table and the mapped bytes."""

    def __init__(self, path):
        self._handle = ctypes.c_void_p()
        code = _load().nfn_mi355_gguf_open_v1(str(Path(path)).encode(), ctypes.byref(self._handle))
        if code:
            raise GgufError(code)

    def close(self) -> None:
        if self._handle:
            _load().nfn_mi355_gguf_close_v1(self._handle)
            self._handle = ctypes.c_void_p()

    def __enter__(self) -> "GgufFile":
        return self

    def __exit__(self, *unused) -> None:
        self.close()

    def __len__(self) -> int:
        return int(_load().nfn_mi355_gguf_tensor_count_v1(self._handle))

    @property
    def metadata_count(self) -> int:
        return int(_load().nfn_mi355_gguf_metadata_count_v1(self._handle))

    def __iter__(self) -> Iterator[GgufTensor]:
        raw = _Tensor()
        for index in range(len(self)):
            code = _load().nfn_mi355_gguf_tensor_v1(self._handle, index, ctypes.byref(raw))
            if code:
                raise GgufError(code)
            yield _convert(raw)

    def find(self, name: str) -> GgufTensor:
        raw = _Tensor()
        code = _load().nfn_mi355_gguf_find_v1(self._handle, name.encode(), ctypes.byref(raw))
        if code:
            raise GgufError(code)
        return _convert(raw)

    def bytes_of(self, tensor: GgufTensor) -> np.ndarray:
        """A copy of the tensor's packed bytes."""
        size = ctypes.c_uint64()
        base = _load().nfn_mi355_gguf_data_v1(self._handle, ctypes.byref(size))
        view = (ctypes.c_uint8 * tensor.nbytes).from_address(base + tensor.file_offset)
        return np.frombuffer(view, dtype=np.uint8).copy()

    def packed_weight(self, name: str, device="cuda:0"):
        """The tensor on the device as a tile_ops.PackedWeight ([rows, cols], bytes as in the file)."""
        import torch
        from . import tile_ops
        tensor = self.find(name)
        data = torch.from_numpy(self.bytes_of(tensor)).to(device)
        return tile_ops.PackedWeight(tensor.encoding, tensor.rows, tensor.cols, data)
