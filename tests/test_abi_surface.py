"""The C ABI without a GPU: the library loads, exports every symbol the header
declares, and fails closed on bad arguments before touching the device.

Negative cases follow the reference probe
(tests/cpp/muse_glimmer_cuda_kernel_probe.cpp:1429-1433, 1740-1762, 1834-1866).
"""
import ctypes
import re
from pathlib import Path

import pytest

from neuralfn_amd import kquant, tile_ops

ROOT = Path(__file__).resolve().parents[1]
HEADER = ROOT / "include" / "nfn_mi355_tile_ops.h"


@pytest.fixture(scope="module")
def lib():
    return tile_ops.load()


def declared_symbols():
    text = re.sub(r"/\*.*?\*/", "", HEADER.read_text(), flags=re.S)
    return sorted(set(re.findall(r"\b(nfn_(?:native_tile|mi355)_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    names = declared_symbols()
    assert len(names) >= 28
    for name in names:
        assert hasattr(lib, name), f"{name} is declared but not exported"
    assert set(names) == set(tile_ops.SIGNATURES), "binding and header disagree"


def test_the_probes_library_exports_what_its_header_declares():
    from neuralfn_amd import probes
    header = ROOT / "include" / "nfn_mi355_probes.h"
    text = re.sub(r"/\*.*?\*/", "", header.read_text(), flags=re.S)
    names = sorted(set(re.findall(r"\b(nfn_mi355_[a-z0-9_]+)\s*\(", text)))
    assert set(names) == set(probes.SIGNATURES)
    loaded = probes.load()
    for name in names:
        assert hasattr(loaded, name), f"{name} is declared but not exported"
    # and the product library exports none of them
    product = tile_ops.load()
    for name in names:
        assert not hasattr(product, name), f"{name} is a measurement aid inside the product library"


def test_versions(lib):
    for name in ("nfn_native_tile_ops_abi_version", "nfn_native_tile_strict_math_abi_version",
                 "nfn_native_tile_packed_weight_abi_version",
                 "nfn_native_tile_glimmer_inference_abi_version",
                 "nfn_native_tile_k_quant_mmq_abi_version"):
        assert getattr(lib, name)() == 1


def test_descriptor_is_72_bytes():
    assert ctypes.sizeof(tile_ops.PackedWeightDescriptor) == 72
    assert tile_ops.PackedWeightDescriptor.data.offset == 16
    assert tile_ops.PackedWeightDescriptor.row_stride_bytes.offset == 48
    assert tile_ops.PackedWeightDescriptor.cuda_stream.offset == 64


def test_attention_and_cache_descriptors_have_the_reference_layout():
    # sizeof / offsetof of the structs in the reference's tile_ops.h:316-339, 341-359, 373-405, 461-486,
    # as its own header compiles with g++ on x86-64
    for struct, size, field, offset, stream in (
            (tile_ops.GqaDecodeDescriptor, 136, "scale", 120, 128),
            (tile_ops.CacheCommitDescriptor, 104, "cache_row_stride", 80, 96),
            (tile_ops.BlockAttentionDescriptor, 152, "scale", 136, 144),
            (tile_ops.FusedDecodeAttentionDescriptor, 320, "query_heads", 208, 312)):
        assert ctypes.sizeof(struct) == size
        assert getattr(struct, field).offset == offset
        assert struct.cuda_stream.offset == stream


def test_every_symbol_the_reference_engine_requires_is_exported(lib):
    """tests/golden/engine_sidecar_symbols.json lists what the reference's resident engine
    binds from its sidecar (resident_glimmer_cuda.cpp:336-495): everything it requires for
    text decoding must be here, and optional groups must be whole where the engine insists
    (resident_glimmer_cuda.cpp:356-359, 385-428, 453-461)."""
    import json
    symbols = json.loads((ROOT / "tests" / "golden" / "engine_sidecar_symbols.json").read_text())
    assert len(symbols["required"]) == 20
    missing = [name for name in symbols["required"] if not hasattr(lib, name)]
    assert not missing, missing
    exported = {name for name in symbols["optional"] if hasattr(lib, name)}
    assert set(symbols["optional"]) == exported, "an optional symbol of the engine is missing"

    def together(*names):
        present = [("nfn_native_tile_" + name) in exported for name in names]
        assert all(present) or not any(present), names

    together("quantize_q8_1_float32_v1", "linear_packed_weight_q8_1_float32_v1")
    together("k_quant_mmq_abi_version", "k_quant_mmq_workspace_bytes_v1",
             "k_quant_mmq_multi_linear_float32_v1")
    together("k_quant_mmvq_multi_linear_float32_v1", "k_quant_mmvq_multi_linear_gated_float32_v1",
             "k_quant_mmvq_multi_linear_swiglu_float32_v1")
    together("glimmer_rms_norm_affine_capture_residual_float32_v1",
             "glimmer_rms_norm_affine_add_residual_float32_v1")
    together("glimmer_dual_rms_add_capture_mmvq_q8_float32_v1",
             "k_quant_mmvq_multi_linear_prequantized_float32_v1")


def _descriptor(encoding=kquant.Q4_K, out_dim=5, in_dim=512):
    return tile_ops.make_descriptor(encoding, 0x1000, out_dim, in_dim)


def test_validate_accepts_canonical_layouts(lib):
    for encoding in (kquant.F32, kquant.BF16, kquant.Q8_0, kquant.Q4_K, kquant.Q5_K, kquant.Q6_K):
        d = _descriptor(encoding)
        assert lib.nfn_native_tile_packed_weight_validate_v1(ctypes.byref(d)) == 0


@pytest.mark.parametrize("mutate", [
    lambda d: setattr(d, "data_nbytes", d.data_nbytes - 1),
    lambda d: setattr(d, "row_stride_bytes", d.row_stride_bytes - 1),
    lambda d: setattr(d, "encoding", 0xFFFF),
    lambda d: setattr(d, "encoding", 31),
    lambda d: setattr(d, "version", 2),
    lambda d: setattr(d, "flags", 1),
    lambda d: setattr(d, "reserved0", 1),
    lambda d: setattr(d, "reserved1", 1),
    lambda d: setattr(d, "struct_size", 64),
    lambda d: setattr(d, "data", None),
    lambda d: setattr(d, "output_dim", 0),
    lambda d: setattr(d, "input_dim", 511),
])
def test_validate_fails_closed(lib, mutate):
    d = _descriptor()
    mutate(d)
    assert lib.nfn_native_tile_packed_weight_validate_v1(ctypes.byref(d)) == tile_ops.INVALID
    assert lib.nfn_native_tile_packed_weight_validate_v1(None) == tile_ops.INVALID


def test_workspace_contract(lib):
    query = lib.nfn_native_tile_k_quant_mmq_workspace_bytes_v1
    assert query(5, 512) > 0 and query(1, 512) > 0
    assert query(17, 512) == 0
    assert query(0, 512) == 0
    assert query(5, 511) == 0
    assert query(16, 6656) >= query(1, 6656)
    assert query(1, 512) >= 512 // 32 * 36  # at least the reference's one-row need


def test_small_batch_entry_points_fail_closed_without_launching(lib):
    d = _descriptor()
    descriptors = (ctypes.POINTER(tile_ops.PackedWeightDescriptor) * 1)(ctypes.pointer(d))
    outputs = (ctypes.c_void_p * 1)(0x2000)
    need = lib.nfn_native_tile_k_quant_mmq_workspace_bytes_v1(5, 512)
    mmq = lib.nfn_native_tile_k_quant_mmq_multi_linear_float32_v1
    good = dict(x=0x3000, count=1, rows=5, ws=0x4000, ws_bytes=need)

    def call(desc=descriptors, **kw):
        a = {**good, **kw}
        return mmq(desc, a["x"], outputs, a["count"], a["rows"], a["ws"], a["ws_bytes"], None)

    assert call(ws_bytes=need - 1) == tile_ops.INVALID      # short workspace
    assert call(rows=17) == tile_ops.INVALID                # unsupported row count
    assert call(rows=0) == tile_ops.INVALID
    assert call(count=0) == tile_ops.INVALID
    assert call(count=5) == tile_ops.INVALID
    assert call(x=None) == tile_ops.INVALID
    assert call(ws=None) == tile_ops.INVALID
    for mutate in (lambda v: setattr(v, "data_nbytes", v.data_nbytes - 1),
                   lambda v: setattr(v, "encoding", 0xFFFF),
                   lambda v: setattr(v, "encoding", kquant.F32),
                   lambda v: setattr(v, "row_stride_bytes", v.row_stride_bytes - 1),
                   lambda v: setattr(v, "cuda_stream", 0x1234)):
        bad = _descriptor()
        mutate(bad)
        array = (ctypes.POINTER(tile_ops.PackedWeightDescriptor) * 1)(ctypes.pointer(bad))
        assert call(desc=array) == tile_ops.INVALID
    gated = lib.nfn_native_tile_k_quant_mmq_multi_linear_gated_float32_v1
    assert gated(descriptors, 0x3000, None, outputs, 1, 5, 0x4000, need, None) == tile_ops.INVALID
    swiglu = lib.nfn_native_tile_k_quant_mmq_multi_linear_swiglu_float32_v1
    assert swiglu(descriptors, 0x3000, None, outputs, 1, 5, 0x4000, need, None) == tile_ops.INVALID
    mmvq = lib.nfn_native_tile_k_quant_mmvq_linear_float32_v1
    one = lib.nfn_native_tile_k_quant_mmq_workspace_bytes_v1(1, 512)
    assert mmvq(ctypes.byref(d), 0x3000, 0x2000, 0x4000, one - 1, None) == tile_ops.INVALID
    assert mmvq(None, 0x3000, 0x2000, 0x4000, one, None) == tile_ops.INVALID


def test_other_entry_points_fail_closed(lib):
    d = _descriptor()
    assert lib.nfn_native_tile_linear_packed_weight_float32_v1(
        ctypes.byref(d), 0x3000, None, 0x2000, 0, False) == tile_ops.INVALID
    assert lib.nfn_native_tile_linear_packed_weight_float32_v1(
        ctypes.byref(d), 0x3000, None, 0x2000, 1, True) == tile_ops.INVALID  # bias promised, absent
    assert lib.nfn_native_tile_packed_weight_dequantize_float32_v1(
        ctypes.byref(d), None) == tile_ops.INVALID
    assert lib.nfn_native_tile_quantize_q8_1_float32_v1(
        0x1, 0x2, 0x3, 0x4, 1, 33, None) == tile_ops.INVALID
    f32 = _descriptor(kquant.F32)
    assert lib.nfn_native_tile_linear_packed_weight_q8_1_float32_v1(
        ctypes.byref(f32), 0x1, 0x2, 0x3, None, 0x4, 1, False) == tile_ops.INVALID
    multi = lib.nfn_native_tile_linear_packed_weight_q8_1_multi_decode_float32_v1
    assert multi(ctypes.byref(d), ctypes.byref(d), None, None, 0x1, 0x2, 0x3, 0x4, 0x5, None,
                 None, 1, None) == tile_ops.INVALID                      # fewer than two
    assert multi(ctypes.byref(d), ctypes.byref(d), ctypes.byref(d), None, 0x1, 0x2, 0x3, 0x4,
                 0x5, None, None, 2, None) == tile_ops.INVALID           # unused slot not null
    assert lib.nfn_native_tile_argmax_rows_float32_v1(0x1, 0x2, 0x3, 0, 8, None) == tile_ops.INVALID
    assert lib.nfn_mi355_lm_head_argmax_workspace_bytes_v1(17, 1000) == 0
    assert lib.nfn_mi355_lm_head_argmax_workspace_bytes_v1(16, 1000) > 0
    assert lib.nfn_mi355_k_quant_gemm_workspace_bytes_v1(512, 6656, 16384, 7) == 0
    assert lib.nfn_mi355_k_quant_gemm_workspace_bytes_v1(512, 100, 16384, 0) == 0


def test_error_string_never_null(lib):
    for code in (0, 1, 2, 98, 719, 12345):
        assert lib.nfn_native_tile_ops_error_string(code)


def test_the_reference_engines_own_loader_opens_the_library():
    """Runtime::Runtime of the reference engine (resident_glimmer_cuda.cpp:329-630), compiled
    from the reference checkout where it lies (oracle/loader_harness.cpp, `make -C oracle ref`),
    constructs itself on this library: every required symbol resolves, no optional group is
    only partly present, the four ABI versions are the ones it insists on.  Its runtime library
    is the reference's own CPU double (tests/cpp/fake_cuda_runtime.cpp), so no GPU is touched;
    that double has no graph functions, hence decode_graphs stays off."""
    loader = ROOT / "oracle" / "_ref" / "libnfn_engine_loader_ref.so"
    runtime = ROOT / "oracle" / "_ref" / "libnfn_fake_cuda_runtime_ref.so"
    if not loader.exists() or not runtime.exists():
        pytest.skip("oracle/_ref is not built: the reference checkout is absent on this machine")
    harness = ctypes.CDLL(str(loader))
    harness.nfn_ref_loader_probe.argtypes = [ctypes.c_char_p, ctypes.c_char_p, ctypes.c_char_p,
                                             ctypes.c_int]
    harness.nfn_ref_loader_probe.restype = ctypes.c_int
    report = ctypes.create_string_buffer(4096)
    status = harness.nfn_ref_loader_probe(str(tile_ops.LIB_PATH.resolve()).encode(),
                                          str(runtime.resolve()).encode(), report, len(report))
    text = report.value.decode()
    assert status == 0, f"the engine's loader refused the library: {text}"
    bound = dict(line.split("=", 1) for line in text.splitlines() if "=" in line)
    for group in ("q8_linear", "k_quant_mmq", "k_quant_mmq_gated", "k_quant_mmq_swiglu",
                  "k_quant_mmvq", "k_quant_mmvq_rows", "k_quant_mmvq_prequantized",
                  "rms_to_mmvq_handoff", "fused_residual_norm", "short_attention_split",
                  "cooperative_batch_rms"):
        assert bound.get(group) == "1", f"the engine did not bind {group}: {text}"
    assert bound["tile_path"] == str(tile_ops.LIB_PATH.resolve())
    # a relative path is refused by the engine before it loads anything
    status = harness.nfn_ref_loader_probe(b"libnfn_mi355_tile_ops.so", str(runtime).encode(),
                                          report, len(report))
    assert status == 1 and "absolute" in report.value.decode()
