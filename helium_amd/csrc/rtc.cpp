#include "rtc.h"

#include <hip/hip_ext.h>

#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cstdlib>
#include <fstream>
#include <mutex>
#include <unordered_map>

namespace he {

namespace {

std::mutex g_mu;
std::unordered_map<std::string, std::shared_ptr<const std::vector<char>>> g_cache;
std::atomic<uint64_t> g_compiles{0}, g_mem_hits{0}, g_disk_hits{0};

std::string cache_dir() {
    static std::string dir = [] {
        std::string d;
        if (const char* env = getenv("HELIUM_HIP_CACHE_DIR")) {
            d = env;
        } else {
            Dl_info info;
            if (dladdr((void*)&rtc_stats, &info) && info.dli_fname) {
                std::string p = info.dli_fname;
                size_t slash = p.rfind('/');
                d = (slash == std::string::npos ? std::string(".") : p.substr(0, slash)) + "/_kcache";
            }
        }
        if (d.empty() || d == "off") return std::string();
        mkdir(d.c_str(), 0755);
        if (access(d.c_str(), W_OK) != 0) return std::string();
        return d;
    }();
    return dir;
}

std::string key_of(const std::string& source, const std::vector<std::string>& opts) {
    std::string k = source;
    for (auto& o : opts) {
        k.push_back('\0');
        k += o;
    }
    return k;
}

}  // namespace

std::vector<std::string> default_kernel_options() {
    return {
        "--offload-arch=gfx950",
        "-O3",
        "-std=c++17",
        // Packed-f32 VALU forms are kept out of every kernel.
        "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    };
}

void rtc_stats(uint64_t stats[3]) {
    stats[0] = g_compiles.load();
    stats[1] = g_mem_hits.load();
    stats[2] = g_disk_hits.load();
}

std::shared_ptr<const std::vector<char>> rtc_compile(const std::string& source, const std::string& name,
                                                     const std::vector<std::string>& extra_options) {
    std::vector<std::string> opts = default_kernel_options();
    for (auto& o : extra_options) opts.push_back(o);
    std::string key = key_of(source, opts);
    {
        std::lock_guard<std::mutex> lk(g_mu);
        auto it = g_cache.find(key);
        if (it != g_cache.end()) {
            g_mem_hits++;
            return it->second;
        }
    }

    // Disk cache: the file name is two independent 64-bit hashes of the key.
    std::string path;
    std::string dir = cache_dir();
    if (!dir.empty()) {
        uint64_t h1 = fnv1a(key.data(), key.size());
        uint64_t h2 = fnv1a(key.data(), key.size(), 0x9e3779b97f4a7c15ull);
        path = strfmt("%s/%016llx%016llx.hsaco", dir.c_str(), (unsigned long long)h1, (unsigned long long)h2);
        std::ifstream f(path, std::ios::binary);
        if (f) {
            std::vector<char> blob((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
            if (blob.size() > 64) {
                g_disk_hits++;
                auto sp = std::make_shared<const std::vector<char>>(std::move(blob));
                std::lock_guard<std::mutex> lk(g_mu);
                g_cache[key] = sp;
                return sp;
            }
        }
    }

    if (const char* dump = getenv("HELIUM_HIP_DUMP_DIR")) {
        // Written before compiling, so that a source that crashes the compiler is still on disk. The counterpart
        // of the reference's `cuda-debug` feature, which writes every JIT source to kernel/
        // (helium/src/cuda/kernel_jit.rs:145-151).
        static std::atomic<int> id{0};
        mkdir(dump, 0755);
        std::ofstream f(strfmt("%s/jit_%s_%d.hip", dump, name.c_str(), id++));
        f << source;
    }
    hiprtcProgram prog;
    hiprtcResult r = hiprtcCreateProgram(&prog, source.c_str(), (name + ".hip").c_str(), 0, nullptr, nullptr);
    HE_REQUIRE(r == HIPRTC_SUCCESS, HE_ERR_RTC, "hiprtcCreateProgram: %s", hiprtcGetErrorString(r));
    std::vector<const char*> copts;
    for (auto& o : opts) copts.push_back(o.c_str());
    r = hiprtcCompileProgram(prog, (int)copts.size(), copts.data());
    if (r != HIPRTC_SUCCESS) {
        size_t n = 0;
        hiprtcGetProgramLogSize(prog, &n);
        std::string log(n, '\0');
        if (n) hiprtcGetProgramLog(prog, &log[0]);
        hiprtcDestroyProgram(&prog);
        if (getenv("HELIUM_HIP_DUMP_FAILED")) {
            std::ofstream f(std::string(getenv("HELIUM_HIP_DUMP_FAILED")) + "/" + name + ".failed.hip");
            f << source;
        }
        fail(HE_ERR_RTC, strfmt("hiprtc failed to compile %s: %s\n%s", name.c_str(), hiprtcGetErrorString(r),
                                log.c_str()));
    }
    size_t sz = 0;
    r = hiprtcGetCodeSize(prog, &sz);
    HE_REQUIRE(r == HIPRTC_SUCCESS && sz > 0, HE_ERR_RTC, "hiprtcGetCodeSize: %s", hiprtcGetErrorString(r));
    std::vector<char> blob(sz);
    r = hiprtcGetCode(prog, blob.data());
    hiprtcDestroyProgram(&prog);
    HE_REQUIRE(r == HIPRTC_SUCCESS, HE_ERR_RTC, "hiprtcGetCode: %s", hiprtcGetErrorString(r));
    g_compiles++;

    if (!path.empty()) {
        std::string tmp = path + strfmt(".tmp%d", (int)getpid());
        {
            std::ofstream f(tmp, std::ios::binary);
            f.write(blob.data(), (std::streamsize)blob.size());
        }
        rename(tmp.c_str(), path.c_str());
    }
    auto sp = std::make_shared<const std::vector<char>>(std::move(blob));
    std::lock_guard<std::mutex> lk(g_mu);
    g_cache[key] = sp;
    return sp;
}

JitKernel::JitKernel(std::string source, std::string entry, std::vector<std::string> options)
    : source_(std::move(source)), entry_(std::move(entry)) {
    code_ = rtc_compile(source_, entry_, options);
}

JitKernel::~JitKernel() {
    if (module_) (void)hipModuleUnload(module_);
}

void JitKernel::ensure_loaded() {
    if (func_) return;
    static std::mutex mu;
    std::lock_guard<std::mutex> lk(mu);
    if (func_) return;
    hipModule_t m;
    HE_HIP(hipModuleLoadData(&m, code_->data()));
    hipFunction_t f;
    hipError_t e = hipModuleGetFunction(&f, m, entry_.c_str());
    if (e != hipSuccess) {
        (void)hipModuleUnload(m);
        fail(HE_ERR_HIP, strfmt("kernel entry %s not found: %s", entry_.c_str(), hipGetErrorString(e)));
    }
    module_ = m;
    func_ = f;
}

namespace {
thread_local hipEvent_t t_pending_stop = nullptr;
}
void set_pending_stop_event(hipEvent_t event) { t_pending_stop = event; }
hipEvent_t take_pending_stop_event() {
    hipEvent_t e = t_pending_stop;
    t_pending_stop = nullptr;
    return e;
}

void JitKernel::launch(const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes, hipStream_t stream,
                       void** args, bool closes_instruction) {
    ensure_loaded();
    HE_REQUIRE(grid[0] && grid[1] && grid[2], HE_ERR_INVALID, "kernel %s: empty grid", entry_.c_str());
    if (closes_instruction && t_pending_stop) {
        // this entry point takes the global work size, in 32 bits per dim
        const uint64_t gx = (uint64_t)grid[0] * block[0], gy = (uint64_t)grid[1] * block[1], gz = (uint64_t)grid[2] * block[2];
        if (gx < (1ull << 32) && gy < (1ull << 32) && gz < (1ull << 32)) {
            hipEvent_t stop = take_pending_stop_event();
            HE_HIP(hipExtModuleLaunchKernel(func_, (uint32_t)gx, (uint32_t)gy, (uint32_t)gz, block[0], block[1], block[2], lds_bytes, stream,
                                            args, nullptr, nullptr, stop, 0));
            return;
        }
    }
    HE_HIP(hipModuleLaunchKernel(func_, grid[0], grid[1], grid[2], block[0], block[1], block[2], lds_bytes,
                                 stream, args, nullptr));
}

int JitKernel::private_bytes() {
    ensure_loaded();
    int v = 0;
    HE_HIP(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_LOCAL_SIZE_BYTES, func_));
    return v;
}

int JitKernel::vgprs() {
    ensure_loaded();
    int v = 0;
    HE_HIP(hipFuncGetAttribute(&v, HIP_FUNC_ATTRIBUTE_NUM_REGS, func_));
    return v;
}

}  // namespace he
