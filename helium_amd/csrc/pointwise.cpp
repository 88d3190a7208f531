// Pointwise / reduction instruction: helium/src/cuda/instr/pointwise.rs + pointwise/jit.rs (kernels K2/K3).
#include "kernels.h"

namespace he {

// One launch that fills up to 8 buffers with 32-bit patterns (reduction identities, cleared bitsets): a single
// small kernel instead of one memset per output.
namespace {
struct FillArgs {
    uint32_t* ptr[8];
    uint32_t words[8];
    uint32_t value[8];
    int32_t count;
};
const char* kFillSource = R"HIP(
struct FillArgs { unsigned* ptr[8]; unsigned words[8]; unsigned value[8]; int count; };
extern "C" __global__ __launch_bounds__(256) void fill_many(FillArgs a) {
    for (int k = 0; k < a.count; k++)
        for (unsigned i = blockIdx.x * 256u + threadIdx.x; i < a.words[k]; i += gridDim.x * 256u) a.ptr[k][i] = a.value[k];
}
)HIP";
JitKernel& fill_kernel() {
    static JitKernel k(kFillSource, "fill_many");
    return k;
}
}  // namespace

void load_fill_kernel() { fill_kernel().load(); }
bool fill_kernel_loaded() { return fill_kernel().loaded(); }

void fill_buffers(const std::vector<std::pair<void*, std::pair<uint32_t, uint32_t>>>& fills, hipStream_t stream) {
    for (size_t base = 0; base < fills.size(); base += 8) {
        FillArgs a{};
        uint32_t max_words = 0;
        a.count = (int)std::min<size_t>(8, fills.size() - base);
        for (int k = 0; k < a.count; k++) {
            a.ptr[k] = (uint32_t*)fills[base + k].first;
            a.words[k] = fills[base + k].second.first;
            a.value[k] = fills[base + k].second.second;
            max_words = std::max(max_words, a.words[k]);
        }
        if (!max_words) continue;
        const uint32_t grid[3] = {std::min<uint32_t>((max_words + 1023) / 1024, 1024), 1, 1}, block[3] = {256, 1, 1};
        void* argv[] = {&a};
        fill_kernel().launch(grid, block, 0, stream, argv);
    }
}

namespace {
uint64_t aligned_float_bytes(uint64_t n_floats) { return (n_floats * 4 + 255) & ~255ull; }
}  // namespace

ReduceScratch::Buf ReduceScratch::get(uint64_t n_floats, uint64_t n_counters, hipStream_t stream) {
    const uint64_t float_bytes = aligned_float_bytes(n_floats);
    std::lock_guard<std::mutex> lk(mu_);
    auto it = per_stream_.find(stream);
    if (it == per_stream_.end()) {
        void* p = nullptr;
        HE_HIP(hipMalloc(&p, float_bytes + std::max<uint64_t>(n_counters, 1) * 4));
        it = per_stream_.emplace(stream, p).first;
        if (n_counters) fill_buffers({{(char*)p + float_bytes, {(uint32_t)n_counters, 0u}}}, stream);
    }
    return {(float*)it->second, (uint32_t*)((char*)it->second + float_bytes)};
}

void ReduceScratch::release() {
    std::lock_guard<std::mutex> lk(mu_);
    for (auto& kv : per_stream_) (void)hipFree(kv.second);
    per_stream_.clear();
}

TileKernel::~TileKernel() { scratch_.release(); }

TileKernel::TileKernel(tp::Program prog, const std::string& entry) : prog_(std::move(prog)) {
    launch_ = tp::emit_pointwise(prog_, entry);
    HE_REQUIRE(!prog_.post || launch_.post_carried, HE_ERR_INTERNAL, "the program's carried part has no fold launch to ride on");
    if (launch_.grid > 0) kernel_.reset(new JitKernel(launch_.source, launch_.entry, launch_.options));
    if (launch_.grid > 0 && launch_.finalize_grid > 0)
        finalize_.reset(new JitKernel(launch_.source, launch_.finalize_entry, launch_.options));
}

void TileKernel::execute(void* const* ptrs, hipStream_t stream) {
    ReduceScratch::Buf ws{nullptr, nullptr};
    if (launch_.grid && launch_.ws_floats) ws = scratch_.get(launch_.ws_floats, launch_.ws_counters, stream);
    run(ptrs, stream, ws);
}

size_t TileKernel::scratch_bytes_needed() const {
    if (!launch_.grid || !launch_.ws_floats) return 0;
    return (size_t)(aligned_float_bytes(launch_.ws_floats) + launch_.ws_counters * 4);
}

void TileKernel::load() {
    if (kernel_) kernel_->load();
    if (finalize_) finalize_->load();
    if (!launch_.fills.empty() || launch_.ws_counters) load_fill_kernel();
}

bool TileKernel::loaded() const {
    return (!kernel_ || kernel_->loaded()) && (!finalize_ || finalize_->loaded()) &&
           ((launch_.fills.empty() && !launch_.ws_counters) || fill_kernel_loaded());
}

void TileKernel::execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) {
    HE_REQUIRE(loaded(), HE_ERR_INVALID, "the kernel's code objects are not loaded on this device yet");
    const size_t need = scratch_bytes_needed();
    HE_REQUIRE(need <= scratch_bytes, HE_ERR_INVALID,
               "the kernel needs %zu bytes of scratch for its partial results, the buffer holds %zu", need, scratch_bytes);
    ReduceScratch::Buf ws{nullptr, nullptr};
    if (need) {
        HE_REQUIRE(scratch && ((uintptr_t)scratch & 255) == 0, HE_ERR_INVALID, "scratch buffer missing or not 256-byte aligned");
        ws.floats = (float*)scratch;
        ws.counters = (uint32_t*)((char*)scratch + aligned_float_bytes(launch_.ws_floats));
        // the buffer is shared with whatever ran before: arrival counters must start at zero
        if (launch_.ws_counters) fill_buffers({{ws.counters, {(uint32_t)launch_.ws_counters, 0u}}}, stream);
    }
    run(ptrs, stream, ws);
}

void TileKernel::run(void* const* ptrs, hipStream_t stream, ReduceScratch::Buf ws) {
    const size_t nargs = prog_.args.size();
    for (size_t i = 0; i < nargs; i++)
        HE_REQUIRE(ptrs[i] != nullptr || prog_.args[i].numel == 0, HE_ERR_INVALID, "kernel argument %zu is null", i);
    // Reduction outputs start from the operator's identity and bitset outputs from zero
    // (helium/src/cuda/instr/pointwise.rs:62-74).
    std::vector<std::pair<void*, std::pair<uint32_t, uint32_t>>> fills;
    for (auto& f : launch_.fills) {
        const tp::Arg& a = prog_.args[f.first];
        size_t words = storage_bytes(a.dtype, (size_t)a.numel) / 4;
        if (words) fills.push_back({ptrs[f.first], {(uint32_t)words, f.second}});
    }
    if (!fills.empty()) fill_buffers(fills, stream);
    if (launch_.grid == 0) return;
    for (size_t i = 0; i < nargs; i++)
        HE_REQUIRE(((uintptr_t)ptrs[i] & 15) == 0, HE_ERR_INVALID, "kernel argument %zu is not 16-byte aligned", i);
    std::vector<void*> holders(ptrs, ptrs + nargs);
    if (launch_.ws_floats) {
        holders.push_back(ws.floats);
        holders.push_back(ws.counters);
    }
    std::vector<void*> argv(holders.size());
    for (size_t i = 0; i < holders.size(); i++) argv[i] = &holders[i];
    const uint32_t grid[3] = {launch_.grid, 1, 1}, block[3] = {launch_.threads, 1, 1};
    kernel_->launch(grid, block, 0, stream, argv.data(), !finalize_);
    if (finalize_) {
        // same arguments, then the float scratch
        argv.resize(nargs + 1);
        const uint32_t fgrid[3] = {launch_.finalize_grid, 1, 1};
        finalize_->launch(fgrid, block, 0, stream, argv.data(), true);
    }
}

}  // namespace he
