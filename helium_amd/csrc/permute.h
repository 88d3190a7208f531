// Permute instruction: LDS-staged tiled transposition of an N-d tensor for gfx950.
// Replaces helium/src/cuda/instr/permute_dims.rs and permute_dims/jit.rs.
#pragma once
#include <memory>
#include <string>
#include <vector>

#include "common.h"
#include "rtc.h"

namespace he {

struct PermutePlan {
    enum Variant { Copy, Rows, Tile };
    Variant variant = Copy;
    int elem_bytes = 2;
    int64_t numel = 0;
    // Collapsed problem, indexed by collapsed *input* dimension.
    std::vector<int64_t> dims, in_stride, out_stride;
    std::vector<int> out_order;  // collapsed input dims listed in output order (slowest first)
    int ax_a = -1;               // innermost input dim
    int ax_b = -1;               // innermost output dim
    int va = 1, vb = 1;          // elements per global load / store
    int ta = 64, tb = 64;        // tile extents along A / B
    int threads = 256;
    int unroll = 1;              // vectors per thread (Rows / Copy)
    uint32_t grid = 0;
    uint32_t lds_bytes = 0;
};

// Drops extent-1 dims and merges dims that stay adjacent, then picks the kernel variant and tile.
// `perm` follows numpy.transpose. Tunables may be overridden through the environment variables
// HELIUM_HIP_PERMUTE_TA / _TB (tile extents), used for tuning runs only.
PermutePlan plan_permute(const std::vector<int64_t>& shape, const std::vector<int>& perm, int elem_bytes);
std::string emit_permute_source(const PermutePlan& plan);

// Sequential SwapDims → numpy-style permutation (helium-ir/src/opgraph/op.rs:102-110 applied in order).
std::vector<int> perm_from_swaps(int rank, const std::vector<std::pair<int, int>>& swaps);

class Permute {
public:
    Permute(const std::vector<int64_t>& shape, const std::vector<int>& perm, int dtype);
    void execute(const void* in, void* out, hipStream_t stream);
    const std::string& source() const { return kernel_->source(); }
    const std::string& describe() const { return desc_; }
    const PermutePlan& plan() const { return plan_; }

private:
    PermutePlan plan_;
    std::unique_ptr<JitKernel> kernel_;
    std::string desc_;
};

}  // namespace he
