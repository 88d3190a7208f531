// Device shim: the HIP equivalents of the driver-API wrappers in helium/src/cuda/context.rs
// (streams, events, modules, launches, memory), exported through the C ABI.
#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>

#include "common.h"
#include "exec.h"
#include "rtc.h"

namespace he {

static thread_local std::string g_last_error;
void set_error(const std::string& msg) { g_last_error = msg; }
const char* last_error() { return g_last_error.c_str(); }

std::string strfmt(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    va_list ap2;
    va_copy(ap2, ap);
    int n = vsnprintf(nullptr, 0, fmt, ap);
    va_end(ap);
    std::string s(n > 0 ? n : 0, '\0');
    if (n > 0) vsnprintf(&s[0], n + 1, fmt, ap2);
    va_end(ap2);
    return s;
}

const char* dtype_name(int dt) {
    switch (dt) {
        case HE_F16: return "f16";
        case HE_BF16: return "bf16";
        case HE_F32: return "f32";
        case HE_U32: return "u32";
        case HE_BOOL: return "bool";
    }
    return "?";
}

uint64_t fnv1a(const void* data, size_t n, uint64_t h) {
    const unsigned char* p = static_cast<const unsigned char*>(data);
    for (size_t i = 0; i < n; i++) {
        h ^= p[i];
        h *= 1099511628211ull;
    }
    return h;
}

}  // namespace he

struct he_event_s {
    hipEvent_t e;
};
struct he_module_s {
    hipModule_t m;
};
// he_function_t is the hipFunction_t itself, cast.

static hipStream_t raw(he_stream_t s) { return s ? s->s : nullptr; }

static std::atomic<bool> g_initialised{false};

extern char** environ;

namespace he::tuning {
namespace {
int mode() {
    static const int m = [] {
        const char* v = getenv("HELIUM_HIP_TUNING");
        if (!v || !*v || !strcmp(v, "0")) return 0;
        return !strcmp(v, "measure") ? 2 : 1;
    }();
    return m;
}
// what a generated kernel or plan never depends on
bool is_override(const char* entry) {
    if (strncmp(entry, "HELIUM_HIP_", 11) != 0) return false;
    for (const char* other : {"HELIUM_HIP_TUNING=", "HELIUM_HIP_CACHE_DIR=", "HELIUM_HIP_DUMP_DIR=", "HELIUM_HIP_DUMP_FAILED=",
                              "HELIUM_HIP_EXEC_TIMING=", "HELIUM_HIP_NO_LAUNCH_EVENTS=", "HELIUM_HIP_STREAMS=",
                              "HELIUM_HIP_INSTR_TIMING=", "HELIUM_HIP_PLAN_DEBUG="})
        if (strncmp(entry, other, strlen(other)) == 0) return false;
    return true;
}
}  // namespace
bool enabled() { return mode() != 0; }
bool measuring() { return mode() == 2; }
const char* get(const char* name) { return enabled() ? getenv(name) : nullptr; }
int get_int(const char* name, int dflt) {
    const char* v = get(name);
    return v ? atoi(v) : dflt;
}
std::string key() {
    if (!enabled()) return std::string();
    std::vector<std::string> all;
    for (char** e = environ; e && *e; e++)
        if (is_override(*e)) all.push_back(*e);
    std::sort(all.begin(), all.end());
    std::string k = measuring() ? "measure;" : "tuning;";
    for (auto& v : all) k += v + ";";
    return k;
}
uint32_t hash() {
    if (!enabled()) return 0;
    const std::string k = key();
    return (uint32_t)fnv1a(k.data(), k.size()) | 1u;
}
}  // namespace he::tuning
namespace he {
void noalloc_init_device(int device);  // noalloc.hip
bool device_initialised() { return g_initialised.load(std::memory_order_acquire); }
}  // namespace he

extern "C" {

const char* he_last_error(void) { return he::last_error(); }
const char* he_version(void) { return "helium-hip 0.1 (gfx950)"; }
const char* he_target_arch(void) { return "gfx950"; }

int he_init(int device) {
    return he::guard([&] {
        HE_HIP(hipInit(0));
        int n = 0;
        HE_HIP(hipGetDeviceCount(&n));
        HE_REQUIRE(device >= 0 && device < n, HE_ERR_INVALID, "device %d out of range (%d devices)", device, n);
        HE_HIP(hipSetDevice(device));
        HE_HIP(hipFree(nullptr));  // forces creation of the primary context
        he::noalloc_init_device(device);
        g_initialised.store(true, std::memory_order_release);
    });
}

int he_device_count(int* count) {
    return he::guard([&] { HE_HIP(hipGetDeviceCount(count)); });
}

int he_device_attr(int device, int attr, int64_t* value) {
    return he::guard([&] {
        int v = 0;
        switch (attr) {
            case HE_ATTR_CU_COUNT:
                HE_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeMultiprocessorCount, device));
                *value = v;
                break;
            case HE_ATTR_L2_BYTES:
                HE_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeL2CacheSize, device));
                *value = v;
                break;
            case HE_ATTR_LDS_BYTES_PER_BLOCK:
                HE_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeMaxSharedMemoryPerBlock, device));
                *value = v;
                break;
            case HE_ATTR_CLOCK_KHZ:
                HE_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeClockRate, device));
                *value = v;
                break;
            case HE_ATTR_WAVEFRONT:
                HE_HIP(hipDeviceGetAttribute(&v, hipDeviceAttributeWarpSize, device));
                *value = v;
                break;
            case HE_ATTR_TOTAL_MEM_BYTES: {
                size_t bytes = 0;
                HE_HIP(hipDeviceTotalMem(&bytes, device));
                *value = (int64_t)bytes;
                break;
            }
            default: he::fail(HE_ERR_INVALID, he::strfmt("unknown device attribute %d", attr));
        }
    });
}

int he_device_arch(int device, char* buf, size_t buf_len) {
    return he::guard([&] {
        hipDeviceProp_t prop;
        HE_HIP(hipGetDeviceProperties(&prop, device));
        HE_REQUIRE(buf && buf_len > 0, HE_ERR_INVALID, "null buffer");
        strncpy(buf, prop.gcnArchName, buf_len - 1);
        buf[buf_len - 1] = 0;
    });
}

int he_device_synchronize(void) {
    return he::guard([&] {
        HE_HIP(hipDeviceSynchronize());
        he::exec::DevicePool::poll_if_created();
    });
}

int he_stream_create(he_stream_t* stream) {
    return he::guard([&] {
        hipStream_t s;
        HE_HIP(hipStreamCreateWithFlags(&s, hipStreamNonBlocking));
        *stream = new he_stream_s{s};
    });
}
int he_stream_destroy(he_stream_t stream) {
    return he::guard([&] {
        if (!stream) return;
        HE_HIP(hipStreamDestroy(stream->s));
        delete stream;
    });
}
int he_stream_synchronize(he_stream_t stream) {
    return he::guard([&] {
        HE_HIP(hipStreamSynchronize(raw(stream)));
        he::exec::DevicePool::poll_if_created();
    });
}
namespace {
struct HostCb {
    void (*fn)(void*);
    void* user;
};
void host_cb_trampoline(void* p) {
    HostCb* cb = static_cast<HostCb*>(p);
    cb->fn(cb->user);
    delete cb;
}
}  // namespace
int he_stream_host_callback(he_stream_t stream, void (*fn)(void*), void* user) {
    return he::guard([&] {
        HE_REQUIRE(fn, HE_ERR_INVALID, "null callback");
        HostCb* cb = new HostCb{fn, user};
        hipError_t e = hipLaunchHostFunc(raw(stream), host_cb_trampoline, cb);
        if (e != hipSuccess) {
            delete cb;
            he::fail(HE_ERR_HIP, he::strfmt("hipLaunchHostFunc failed: %s", hipGetErrorString(e)));
        }
    });
}
void* he_stream_raw(he_stream_t stream) { return raw(stream); }

int he_event_create(he_event_t* event) {
    return he::guard([&] {
        hipEvent_t e;
        HE_HIP(hipEventCreateWithFlags(&e, hipEventBlockingSync));
        *event = new he_event_s{e};
    });
}
int he_event_destroy(he_event_t event) {
    return he::guard([&] {
        if (!event) return;
        HE_HIP(hipEventDestroy(event->e));
        delete event;
    });
}
int he_event_record(he_event_t event, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipEventRecord(event->e, raw(stream))); });
}
int he_event_wait(he_event_t event, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipStreamWaitEvent(raw(stream), event->e, 0)); });
}
int he_event_synchronize(he_event_t event) {
    return he::guard([&] {
        HE_HIP(hipEventSynchronize(event->e));
        he::exec::DevicePool::poll_if_created();
    });
}
int he_event_elapsed_ms(he_event_t start, he_event_t stop, float* ms) {
    return he::guard([&] { HE_HIP(hipEventElapsedTime(ms, start->e, stop->e)); });
}

int he_malloc(void** dptr, size_t bytes) {
    return he::guard([&] { HE_HIP(hipMalloc(dptr, bytes ? bytes : 1)); });
}
int he_free(void* dptr) {
    return he::guard([&] { HE_HIP(hipFree(dptr)); });
}
int he_host_alloc(void** hptr, size_t bytes) {
    return he::guard([&] { HE_HIP(hipHostMalloc(hptr, bytes ? bytes : 1, hipHostMallocDefault)); });
}
int he_host_free(void* hptr) {
    return he::guard([&] { HE_HIP(hipHostFree(hptr)); });
}
int he_memcpy_h2d_async(void* dst, const void* src, size_t bytes, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, raw(stream))); });
}
int he_memcpy_d2h_async(void* dst, const void* src, size_t bytes, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, raw(stream))); });
}
int he_memcpy_d2d_async(void* dst, const void* src, size_t bytes, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, raw(stream))); });
}
int he_memset_d8_async(void* dst, uint8_t value, size_t count, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemsetD8Async((hipDeviceptr_t)dst, value, count, raw(stream))); });
}
int he_memset_d16_async(void* dst, uint16_t value, size_t count, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemsetD16Async((hipDeviceptr_t)dst, value, count, raw(stream))); });
}
int he_memset_d32_async(void* dst, uint32_t value, size_t count, he_stream_t stream) {
    return he::guard([&] { HE_HIP(hipMemsetD32Async((hipDeviceptr_t)dst, (int)value, count, raw(stream))); });
}

int he_rtc_compile(const char* source, const char* name, const char* const* options, int num_options,
                   void** code, size_t* code_size) {
    return he::guard([&] {
        HE_REQUIRE(source && code && code_size, HE_ERR_INVALID, "null argument");
        std::vector<std::string> opts;
        for (int i = 0; i < num_options; i++) opts.push_back(options[i]);
        std::shared_ptr<const std::vector<char>> blob = he::rtc_compile(source, name ? name : "kernel", opts);
        void* p = malloc(blob->size());
        HE_REQUIRE(p, HE_ERR_INTERNAL, "out of host memory");
        memcpy(p, blob->data(), blob->size());
        *code = p;
        *code_size = blob->size();
    });
}
int he_rtc_free(void* code) {
    free(code);
    return HE_OK;
}
int he_rtc_stats(uint64_t stats[3]) {
    he::rtc_stats(stats);
    return HE_OK;
}

int he_module_load(he_module_t* module, const void* code, size_t code_size) {
    (void)code_size;
    return he::guard([&] {
        hipModule_t m;
        HE_HIP(hipModuleLoadData(&m, code));
        *module = new he_module_s{m};
    });
}
int he_module_unload(he_module_t module) {
    return he::guard([&] {
        if (!module) return;
        HE_HIP(hipModuleUnload(module->m));
        delete module;
    });
}
int he_module_get_function(he_module_t module, const char* name, he_function_t* function) {
    return he::guard([&] {
        hipFunction_t f;
        HE_HIP(hipModuleGetFunction(&f, module->m, name));
        *function = reinterpret_cast<he_function_t>(f);
    });
}
int he_launch(he_function_t function, const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes,
              he_stream_t stream, void** args) {
    return he::guard([&] {
        HE_REQUIRE(grid[0] && grid[1] && grid[2] && block[0] && block[1] && block[2], HE_ERR_INVALID,
                   "empty launch");
        HE_HIP(hipModuleLaunchKernel(reinterpret_cast<hipFunction_t>(function), grid[0], grid[1], grid[2],
                                     block[0], block[1], block[2], lds_bytes, raw(stream), args, nullptr));
    });
}

}  // extern "C"
