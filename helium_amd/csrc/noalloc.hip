// The entry point that allocates nothing. Kernels whose reductions span several workgroups park per-workgroup partial
// results (and arrival counters) in device scratch; he_tile_kernel_execute takes that scratch from a buffer the kernel
// object allocates on its first launch on a stream. Callers that cannot allocate - code under HIP graph capture,
// tight serving loops - get the same launches here with the scratch in a device array that is part of this library's
// code object, so the call makes no hipMalloc / hipFree and loads no module.
//
// The array is shared by every call on a device and keeps the last call's contents: what must start at zero (the
// arrival counters) is cleared by a fill kernel at the head of each call, and calls that overlap on one device (two
// streams, two host threads) race on it.
#include <hip/hip_runtime.h>

#include "capi_types.h"

namespace {

constexpr size_t kScratchBytes = HE_NOALLOC_SCRATCH_BYTES;
constexpr int kMaxDevices = 64;

static __device__ __align__(256) unsigned char scratch[kScratchBytes];

// Address of `scratch` on each device (every device holds its own copy of the array at its own address). In host code
// the array's name is only a handle for hipGetSymbolAddress, never an address to pass on.
void* g_scratch_ptr[kMaxDevices] = {};

}  // namespace

namespace he {

// Called by he_init with `device` current.
void noalloc_init_device(int device) {
    HE_REQUIRE(device >= 0 && device < kMaxDevices, HE_ERR_INVALID, "device %d beyond the %d this library tracks", device, kMaxDevices);
    if (g_scratch_ptr[device]) return;
    void* ptr = nullptr;
    hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !ptr)
        fail(HE_ERR_HIP, strfmt("hipGetSymbolAddress of the library's scratch array failed on device %d: %s", device, hipGetErrorString(e)));
    g_scratch_ptr[device] = ptr;
}

}  // namespace he

extern "C" int he_tile_kernel_execute_noalloc(he_tile_kernel_t kernel, void* const* arg_ptrs, int num_args, he_stream_t stream) {
    return he::guard([&] {
        HE_REQUIRE(kernel && arg_ptrs, HE_ERR_INVALID, "bad argument");
        HE_REQUIRE(num_args == (int)kernel->k->args().size(), HE_ERR_INVALID, "kernel takes %zu arguments, got %d",
                   kernel->k->args().size(), num_args);
        int device = -1;
        HE_HIP(hipGetDevice(&device));
        HE_REQUIRE(device >= 0 && device < kMaxDevices && g_scratch_ptr[device], HE_ERR_INVALID,
                   "he_init has not run for device %d", device);
        const size_t need = kernel->k->scratch_bytes_needed();
        HE_REQUIRE(need <= kScratchBytes, HE_ERR_INVALID,
                   "this kernel parks %zu bytes of partial results; the allocation-free entry point holds %zu - use he_tile_kernel_execute",
                   need, kScratchBytes);
        kernel->k->execute_in_scratch(arg_ptrs, stream ? stream->s : nullptr, g_scratch_ptr[device], kScratchBytes);
    });
}
