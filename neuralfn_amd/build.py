"""Build recipe for the HIP library and the host-side library (quantizer, GGUF tensor table).

`build_all()` compiles every source for gfx950 with hipcc and links
`neuralfn_amd/lib/libnfn_mi355_tile_ops.so` (and the benchmark's measurement aids into
`libnfn_mi355_probes.so`); hipcc cross-compiles, so this runs
on a machine without a GPU.  Nothing is built at import time: tests, the smoke
check and the benchmark load what is already built.
"""
from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PACKAGE = Path(__file__).resolve().parent
CSRC = PACKAGE / "csrc"
LIB_DIR = PACKAGE / "lib"
OBJ_DIR = PACKAGE / "build"
TILE_OPS_LIB = LIB_DIR / "libnfn_mi355_tile_ops.so"
PROBES_LIB = LIB_DIR / "libnfn_mi355_probes.so"
HOST_LIB = LIB_DIR / "libnfn_mi355_kquant_host.so"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
ARCH = "gfx950"

# -ffp-contract=off: the weight decode is two roundings and a subtraction, as
#   the reference's CPU engine computes it; FMAs are written explicitly.
# packed-fp32-ops off: the compiler must not form packed float instructions.
DEVICE_FLAGS = [
    f"--offload-arch={ARCH}",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-ffp-contract=off",
    "-fno-fast-math",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # leading scalar and pointer arguments arrive in registers at wave start
    # instead of through a first load from the argument block
    "-mllvm", "-amdgpu-kernarg-preload-count=14",
    "-Wall",
    "-Wno-unused-function",
]


def _run(command: list[str]) -> None:
    result = subprocess.run(command, capture_output=True, text=True)
    if result.returncode != 0:
        sys.stderr.write(" ".join(command) + "\n" + result.stdout + result.stderr)
        raise RuntimeError(f"build step failed: {command[0]} ... {command[-1]}")
    noise = "unknown target feature"
    text = "\n".join(
        line for line in (result.stdout + result.stderr).splitlines()
        if line.strip() and noise not in line and "packed-fp32-ops" not in line
    )
    if text:
        sys.stderr.write(text + "\n")


def device_sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip")) + sorted(CSRC.glob("*.cpp"))


def build_tile_ops(jobs: int = 8) -> Path:
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    sources = device_sources()
    objects = [OBJ_DIR / (source.name + ".o") for source in sources]

    def compile_one(pair: tuple[Path, Path]) -> None:
        source, target = pair
        command = [HIPCC, *DEVICE_FLAGS]
        if source.suffix == ".cpp":
            command += ["-x", "hip"]
        command += ["-c", str(source), "-o", str(target)]
        _run(command)

    with ThreadPoolExecutor(max_workers=jobs) as pool:
        list(pool.map(compile_one, zip(sources, objects)))
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(TILE_OPS_LIB),
          *map(str, objects)])
    return TILE_OPS_LIB


def build_probes() -> Path:
    """The benchmark's measurement aids: a library of their own, not part of the product."""
    LIB_DIR.mkdir(exist_ok=True)
    OBJ_DIR.mkdir(exist_ok=True)
    target = OBJ_DIR / "probes.hip.o"
    _run([HIPCC, *DEVICE_FLAGS, "-c", str(CSRC / "probes" / "probes.hip"), "-o", str(target)])
    _run([HIPCC, f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", str(PROBES_LIB), str(target)])
    return PROBES_LIB


def build_host() -> Path:
    LIB_DIR.mkdir(exist_ok=True)
    sources = sorted((CSRC / "host").glob("*.cpp"))
    _run(["g++", "-std=c++17", "-O2", "-pthread", "-fPIC", "-shared", "-Wall", "-o", str(HOST_LIB),
          *map(str, sources)])
    return HOST_LIB


def build_all() -> None:
    build_tile_ops()
    build_probes()
    build_host()


if __name__ == "__main__":
    build_all()
    print(TILE_OPS_LIB)
    print(PROBES_LIB)
    print(HOST_LIB)
