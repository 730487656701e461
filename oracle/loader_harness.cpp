// Lets the reference engine's own loader open a sidecar library.  TEST INFRASTRUCTURE ONLY.
//
// The engine binds its sidecar in Runtime::Runtime
// (neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp:329-630): it canonicalises the path,
// dlopens the library, resolves the required and optional symbols, refuses feature groups
// that are only partly present and checks four ABI versions, then opens a runtime library
// and creates its streams.  Runtime sits in an anonymous namespace, so the only way to run
// that code is a translation unit that textually includes resident_glimmer_cuda.cpp; the
// Makefile passes that file with -include from the reference checkout where it lies.  The
// runtime library handed to it is the reference's own CPU test double
// (tests/cpp/fake_cuda_runtime.cpp, compiled by the same Makefile), so no GPU is touched:
// what is exercised is the engine's binding code against this repository's exports.
#include <cstdio>
#include <cstring>
#include <exception>
#include <memory>
#include <string>

#ifndef NFN_REF_LOADER_INCLUDED
#error "build with -include <reference>/neuralfn/csrc/native_gpt2/resident_glimmer_cuda.cpp -DNFN_REF_LOADER_INCLUDED"
#endif

extern "C" {

// Constructs the engine's Runtime on `tile_ops_lib` (absolute path) and `runtime_lib`.
// Returns 0 and writes "name=0|1" lines (the engine's own capability queries) into `report`,
// or returns 1 and writes the engine's exception text.
int nfn_ref_loader_probe(const char* tile_ops_lib, const char* runtime_lib, char* report,
                         int report_size) {
    using namespace neuralfn::resident_glimmer_cuda;
    std::string text;
    int status = 0;
    try {
        Config config;
        config.tile_ops_lib = tile_ops_lib;
        config.cuda_runtime_lib = runtime_lib;
        config.cuda_device = 0;
        const auto runtime = std::make_shared<Runtime>(config);
        const auto line = [&text](const char* name, bool value) {
            text += name;
            text += value ? "=1\n" : "=0\n";
        };
        line("q8_linear", runtime->has_q8_linear());
        line("k_quant_mmq", runtime->has_k_quant_mmq());
        line("k_quant_mmq_gated", runtime->has_k_quant_mmq_gated());
        line("k_quant_mmq_swiglu", runtime->has_k_quant_mmq_swiglu());
        line("k_quant_mmvq", runtime->has_k_quant_mmvq());
        line("k_quant_mmvq_rows", runtime->has_k_quant_mmvq_rows());
        line("k_quant_mmvq_prequantized", runtime->has_k_quant_mmvq_prequantized());
        line("rms_to_mmvq_handoff", runtime->has_rms_to_mmvq_handoff());
        line("fused_residual_norm", runtime->has_fused_residual_norm());
        line("decode_graphs", runtime->has_decode_graphs());
        line("short_attention_split", runtime->short_attention_split_enabled());
        line("cooperative_batch_rms", runtime->cooperative_batch_rms_enabled());
        text += "tile_path=" + runtime->tile_path() + "\n";
    } catch (const std::exception& error) {
        text = error.what();
        status = 1;
    }
    if (report != nullptr && report_size > 0) {
        std::snprintf(report, static_cast<std::size_t>(report_size), "%s", text.c_str());
    }
    return status;
}

}  // extern "C"
