"""MI355X-native K-Quant packed-linear operators behind NeuralFn's tile-ops C ABI.

The product is `lib/libnfn_mi355_tile_ops.so` (HIP, gfx950).  This package is
the thin host layer over it: `tile_ops` binds the C ABI with ctypes, `kquant`
describes the packed formats and makes synthetic packed tensors.
"""
from . import kquant, tile_ops  # noqa: F401

__all__ = ["kquant", "tile_ops"]
