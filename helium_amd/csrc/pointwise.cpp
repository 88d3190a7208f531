// Pointwise / reduction instruction: helium/src/cuda/instr/pointwise.rs + pointwise/jit.rs (kernels K2/K3).
#include "kernels.h"

namespace he {

TileKernel::TileKernel(tp::Program prog, const std::string& entry) : prog_(std::move(prog)) {
    launch_ = tp::emit_pointwise(prog_, entry);
    if (launch_.grid > 0) kernel_.reset(new JitKernel(launch_.source, launch_.entry, launch_.options));
}

void TileKernel::execute(void* const* ptrs, hipStream_t stream) {
    const size_t nargs = prog_.args.size();
    for (size_t i = 0; i < nargs; i++)
        HE_REQUIRE(ptrs[i] != nullptr || prog_.args[i].numel == 0, HE_ERR_INVALID, "kernel argument %zu is null", i);
    for (auto& f : launch_.fills) {
        const tp::Arg& a = prog_.args[f.first];
        size_t words = storage_bytes(a.dtype, (size_t)a.numel) / 4;
        // Reduction outputs start from the operator's identity and bitset outputs from zero
        // (helium/src/cuda/instr/pointwise.rs:62-74).
        if (words) HE_HIP(hipMemsetD32Async((hipDeviceptr_t)ptrs[f.first], (int)f.second, words, stream));
    }
    if (launch_.grid == 0) return;
    for (size_t i = 0; i < nargs; i++)
        HE_REQUIRE(((uintptr_t)ptrs[i] & 15) == 0, HE_ERR_INVALID, "kernel argument %zu is not 16-byte aligned", i);
    std::vector<void*> holders(ptrs, ptrs + nargs);
    std::vector<void*> argv(nargs);
    for (size_t i = 0; i < nargs; i++) argv[i] = &holders[i];
    const uint32_t grid[3] = {launch_.grid, 1, 1}, block[3] = {launch_.threads, 1, 1};
    kernel_->launch(grid, block, 0, stream, argv.data());
}

}  // namespace he
