// Executable kernels built from tile programs: the pointwise/reduction instruction and fused fusion-IR kernels.
#pragma once
#include <memory>

#include "rtc.h"
#include "tp.h"

namespace he {

// A tile program compiled into one kernel launch (plus the fills its reduction / bitset outputs need).
class TileKernel {
public:
    TileKernel(tp::Program prog, const std::string& entry);
    const tp::Program& program() const { return prog_; }
    const tp::PointwiseLaunch& launch_info() const { return launch_; }
    const std::string& source() const { return launch_.source; }
    // `ptrs[i]` is the device address of program argument i.
    void execute(void* const* ptrs, hipStream_t stream);

private:
    tp::Program prog_;
    tp::PointwiseLaunch launch_;
    std::unique_ptr<JitKernel> kernel_;
};

}  // namespace he
