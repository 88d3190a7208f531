#include "rtc.h"

#include <hip/hip_ext.h>

#include <dlfcn.h>
#include <hip/hiprtc.h>
#include <sys/stat.h>
#include <unistd.h>

#include <atomic>
#include <cstdlib>
#include <cstring>
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

// What a cached code object depends on besides the source and the options: the compiler that made it.
const std::string& toolchain_tag() {
    static const std::string tag = [] {
        int major = 0, minor = 0;
        if (hiprtcVersion(&major, &minor) != HIPRTC_SUCCESS) major = minor = -1;
        return strfmt("hiprtc %d.%d|hip %d|%s", major, minor, (int)HIP_VERSION, he_version());
    }();
    return tag;
}

std::string key_of(const std::string& source, const std::vector<std::string>& opts) {
    std::string k = source;
    for (auto& o : opts) {
        k.push_back('\0');
        k += o;
    }
    k.push_back('\0');
    k += toolchain_tag();
    return k;
}

// A cache file is a header followed by the code object. A file that is short, was written by another format version,
// fails its checksum or does not hold an ELF image is ignored (and overwritten by the compile that follows).
struct CacheHeader {
    char magic[8];       // "HEKCACHE"
    uint32_t format;     // kCacheFormat
    uint32_t reserved;
    uint64_t payload_bytes;
    uint64_t payload_hash;  // fnv1a
};
constexpr uint32_t kCacheFormat = 2;

bool read_cache_file(const std::string& path, std::vector<char>* blob) {
    std::ifstream f(path, std::ios::binary);
    if (!f) return false;
    CacheHeader h;
    if (!f.read((char*)&h, sizeof h)) return false;
    if (memcmp(h.magic, "HEKCACHE", 8) != 0 || h.format != kCacheFormat || h.payload_bytes < 64 || h.payload_bytes > (1ull << 31)) return false;
    blob->resize(h.payload_bytes);
    if (!f.read(blob->data(), (std::streamsize)h.payload_bytes)) return false;
    if (f.peek() != std::ifstream::traits_type::eof()) return false;
    if (memcmp(blob->data(), "\x7f" "ELF", 4) != 0) return false;
    return fnv1a(blob->data(), blob->size()) == h.payload_hash;
}

void write_cache_file(const std::string& path, const std::vector<char>& blob) {
    // written under a private name and renamed: a reader never sees half a file
    const std::string tmp = path + strfmt(".tmp%d", (int)getpid());
    {
        std::ofstream f(tmp, std::ios::binary);
        CacheHeader h{};
        memcpy(h.magic, "HEKCACHE", 8);
        h.format = kCacheFormat;
        h.payload_bytes = blob.size();
        h.payload_hash = fnv1a(blob.data(), blob.size());
        f.write((const char*)&h, sizeof h);
        f.write(blob.data(), (std::streamsize)blob.size());
        if (!f) {
            f.close();
            unlink(tmp.c_str());
            return;
        }
    }
    if (rename(tmp.c_str(), path.c_str()) != 0) unlink(tmp.c_str());
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
                                                     const std::vector<std::string>& extra_options, bool bypass_caches) {
    std::vector<std::string> opts = default_kernel_options();
    for (auto& o : extra_options) opts.push_back(o);
    std::string key = key_of(source, opts);
    if (!bypass_caches) {
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
        path = strfmt("%s/%016llx%016llx.hekc", dir.c_str(), (unsigned long long)h1, (unsigned long long)h2);
        std::vector<char> blob;
        if (!bypass_caches && read_cache_file(path, &blob)) {
            g_disk_hits++;
            auto sp = std::make_shared<const std::vector<char>>(std::move(blob));
            std::lock_guard<std::mutex> lk(g_mu);
            g_cache[key] = sp;
            return sp;
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

    if (!path.empty()) write_cache_file(path, blob);
    auto sp = std::make_shared<const std::vector<char>>(std::move(blob));
    std::lock_guard<std::mutex> lk(g_mu);
    g_cache[key] = sp;
    return sp;
}

JitKernel::JitKernel(std::string source, std::string entry, std::vector<std::string> options)
    : source_(std::move(source)), entry_(std::move(entry)), options_(std::move(options)) {
    code_ = rtc_compile(source_, entry_, options_);
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
    if (hipModuleLoadData(&m, code_->data()) != hipSuccess) {
        // a code object this device does not take (a cache directory carried over from another machine): compile
        // afresh, past the caches, and load that
        (void)hipGetLastError();
        code_ = rtc_compile(source_, entry_, options_, true);
        HE_HIP(hipModuleLoadData(&m, code_->data()));
    }
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
