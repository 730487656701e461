// The fused lm_head argmax for callers that cannot allocate device memory
// (code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc): nfn_mi355_lm_head_argmax_no_alloc_v1 is
// nfn_mi355_lm_head_argmax_v1 without the workspace arguments.  The candidate
// records that the first pass leaves for the second live in a file-scope device
// array of a fixed size instead; the kernels are the same and receive the
// array's address the way they receive a caller's workspace.
//
// `scratch` below is a host-side stand-in for the device array: its name is
// never passed to a kernel or a runtime call.  Every GPU holds its own copy at
// its own address, which hipGetSymbolAddress returns for the current device;
// that address is looked up once per device and kept.
#include "common.hpp"

#include "../../include/nfn_mi355_tile_ops.h"

#include <atomic>

namespace {

constexpr std::int64_t kScratchBytes = NFN_MI355_LM_HEAD_NO_ALLOC_SCRATCH_BYTES;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Device address of `scratch` on each device, null until first asked for.
std::atomic<void*> scratch_address[nfn::kMaxDevices];

// The current device's copy of the array.  The first call on a device asks the
// runtime (a lookup: nothing is allocated); two threads that race here store
// the same address.
int scratch_on_current_device(void** address) {
    int device = 0;
    const hipError_t found = hipGetDevice(&device);
    if (found != hipSuccess) return static_cast<int>(found);
    if (device < 0 || device >= nfn::kMaxDevices) return static_cast<int>(hipErrorInvalidDevice);
    void* known = scratch_address[device].load(std::memory_order_acquire);
    if (known == nullptr) {
        const hipError_t status =
            hipGetSymbolAddress(reinterpret_cast<void**>(&known), HIP_SYMBOL(scratch));
        if (status != hipSuccess) return static_cast<int>(status);
        if (known == nullptr) return static_cast<int>(hipErrorInvalidSymbol);
        scratch_address[device].store(known, std::memory_order_release);
    }
    *address = known;
    return 0;
}

}  // namespace

extern "C" int nfn_mi355_lm_head_argmax_no_alloc_v1(
    const NfnNativeTilePackedWeightDescriptorV1* descriptor, const float* input,
    std::int64_t* output_indices, float* output_values, std::int64_t rows, void* cuda_stream) {
    if (descriptor == nullptr) return nfn::kInvalid;
    // The workspace the ordinary entry point would ask for; 0 = rows or width it refuses.
    const std::int64_t required =
        nfn_mi355_lm_head_argmax_workspace_bytes_v1(rows, descriptor->output_dim);
    if (required == 0) return nfn::kInvalid;
    if (required > kScratchBytes) return NFN_MI355_STATUS_STATIC_SCRATCH_EXCEEDED;
    void* candidates = nullptr;
    const int status = scratch_on_current_device(&candidates);
    if (status != 0) return status;
    // Both passes write every record they later read (one per workgroup or tile and
    // input row), so what an earlier call left in the array needs no clearing.
    return nfn_mi355_lm_head_argmax_v1(descriptor, input, output_indices, output_values, rows,
                                       candidates, kScratchBytes, cuda_stream);
}
