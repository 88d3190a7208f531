// hiprtc compilation with a memory + disk cache, and a loaded-kernel wrapper
// (the counterpart of KernelBuilder::build_ptx / JitKernel in helium/src/cuda/kernel_jit.rs).
#pragma once
#include <atomic>
#include <memory>
#include <string>
#include <vector>

#include "common.h"

namespace he {

// Compiles HIP source for gfx950. Cached by (source, options, hiprtc / HIP / library version): in memory, and as a
// checksummed code-object file under the cache directory (HELIUM_HIP_CACHE_DIR, default <library dir>/_kcache) when
// that directory is usable. `bypass_caches` compiles regardless and replaces both entries.
std::shared_ptr<const std::vector<char>> rtc_compile(const std::string& source, const std::string& name,
                                                     const std::vector<std::string>& extra_options, bool bypass_caches = false);
void rtc_stats(uint64_t stats[3]);

// Flags every generated kernel is compiled with.
std::vector<std::string> default_kernel_options();

// A compiled kernel: code object + entry name. The module is loaded lazily on first launch (so that
// generation and compilation work on a machine without a GPU) and kept for the life of the object.
// An event the next instruction-closing launch of this thread should signal on completion. The executor sets it ahead
// of the last instruction of an execution that used one stream only; whoever set it takes it back afterwards and
// records it the ordinary way if no launch took it.
void set_pending_stop_event(hipEvent_t event);
hipEvent_t take_pending_stop_event();

class JitKernel {
public:
    JitKernel(std::string source, std::string entry, std::vector<std::string> options = {});
    ~JitKernel();
    JitKernel(const JitKernel&) = delete;
    JitKernel& operator=(const JitKernel&) = delete;

    const std::string& source() const { return source_; }
    const std::string& entry() const { return entry_; }
    // `closes_instruction`: this is the last launch an instruction makes. If the calling thread has an event pending
    // (set_pending_stop_event), the launch carries it as its completion event, which saves the separate record (a
    // record occupies the device for about as long as a small kernel does).
    void launch(const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes, hipStream_t stream,
                void** args, bool closes_instruction = false);
    // Number of scratch bytes per lane the compiler reported (0 == no spills); -1 before the module is loaded.
    int private_bytes();
    int vgprs();
    // Loads the code object onto the current device (allocates device memory for the code); launch does it on demand.
    void load() { ensure_loaded(); }
    bool loaded() const { return func_.load(std::memory_order_acquire) != nullptr; }

private:
    void ensure_loaded();
    std::string source_, entry_;
    std::vector<std::string> options_;
    std::shared_ptr<const std::vector<char>> code_;
    hipModule_t module_ = nullptr;
    std::atomic<hipFunction_t> func_{nullptr};  // written under the load mutex, read without it
};

}  // namespace he
