"""ctypes binding of libnfn_mi355_probes.so: the benchmark's measurement aids
(include/nfn_mi355_probes.h).  Not part of the path; only bench.py and the probes' test load it."""
from __future__ import annotations

import ctypes
from pathlib import Path
from typing import Optional

from .tile_ops import check

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libnfn_mi355_probes.so"
_P = ctypes.c_void_p
_I64 = ctypes.c_int64

SIGNATURES = {
    "nfn_mi355_probes_abi_version": (ctypes.c_int, []),
    "nfn_mi355_shader_clock_probe_v1": (ctypes.c_int, [_P, _I64, _P]),
    "nfn_mi355_read_probe_v1": (ctypes.c_int, [_P, _I64, _P, _P]),
    "nfn_mi355_read_probe_chained_v1": (ctypes.c_int, [_P, _I64, _P, ctypes.c_int, _P, _P]),
    "nfn_mi355_mfma_rate_probe_v1": (ctypes.c_int, [ctypes.c_int, ctypes.c_int, ctypes.c_int, _P, _P]),
}

_lib: Optional[ctypes.CDLL] = None


def load() -> ctypes.CDLL:
    """dlopen the probes library and bind every declared symbol; raises if absent."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(f"{LIB_PATH} is not built; run `python -m neuralfn_amd.build`")
    lib = ctypes.CDLL(str(LIB_PATH), mode=ctypes.RTLD_LOCAL)
    for name, (restype, argtypes) in SIGNATURES.items():
        function = getattr(lib, name)
        function.restype = restype
        function.argtypes = argtypes
    _lib = lib
    return lib


class ShaderClockProbe:
    """nfn_mi355_shader_clock_probe_v1 on a side stream: the shader clock while other work runs.

    start() enqueues the wait, the caller then runs the work under test on its
    own stream and synchronizes it, megahertz() waits for the probe and returns
    shader cycles per second / 1e6 over the probe's window.
    """

    def __init__(self, device):
        import torch
        self._torch = torch
        self.stream = torch.cuda.Stream(device=device)
        self.result = torch.zeros(3, dtype=torch.int64, device=device)

    def start(self, microseconds: int) -> None:
        self.result.zero_()
        self._torch.cuda.current_stream().synchronize()
        check(load().nfn_mi355_shader_clock_probe_v1(
            self.result.data_ptr(), microseconds, int(self.stream.cuda_stream)), "clock probe")

    def megahertz(self) -> float:
        self.stream.synchronize()
        cycles, ticks, ticks_per_second = (int(v) for v in self.result.tolist())
        if ticks <= 0:
            raise RuntimeError("the clock probe reported no elapsed ticks")
        return cycles / ticks * ticks_per_second / 1e6
