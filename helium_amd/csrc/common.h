// Shared declarations for the helium HIP backend library (host side).
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

#include "../../include/helium_hip.h"

// Opaque stream handle of the C ABI.
struct he_stream_s {
    hipStream_t s;
};

namespace he {

// Thread-local last-error text, read through he_last_error().
void set_error(const std::string& msg);
const char* last_error();

std::string strfmt(const char* fmt, ...) __attribute__((format(printf, 1, 2)));

struct Error : std::runtime_error {
    int code;
    Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

[[noreturn]] inline void fail(int code, const std::string& msg) { throw Error(code, msg); }

#define HE_HIP(expr)                                                                         \
    do {                                                                                     \
        hipError_t _e = (expr);                                                              \
        if (_e != hipSuccess)                                                                \
            ::he::fail(HE_ERR_HIP, ::he::strfmt("%s failed: %s (%s:%d)", #expr,              \
                                                hipGetErrorString(_e), __FILE__, __LINE__)); \
    } while (0)

#define HE_REQUIRE(cond, code, ...)                                   \
    do {                                                              \
        if (!(cond)) ::he::fail((code), ::he::strfmt(__VA_ARGS__));   \
    } while (0)

// Wraps the body of every extern "C" entry point: exceptions become a status code plus the
// thread-local error text, so nothing unwinds across the C boundary.
template <class F>
int guard(F&& f) noexcept {
    try {
        f();
        return HE_OK;
    } catch (const Error& e) {
        set_error(e.what());
        return e.code;
    } catch (const std::exception& e) {
        set_error(e.what());
        return HE_ERR_INTERNAL;
    } catch (...) {
        set_error("unknown exception");
        return HE_ERR_INTERNAL;
    }
}

inline size_t dtype_bits(int dt) {
    switch (dt) {
        case HE_F16:
        case HE_BF16: return 16;
        case HE_F32:
        case HE_U32: return 32;
        case HE_BOOL: return 1;
    }
    fail(HE_ERR_INVALID, strfmt("bad dtype %d", dt));
}

enum class DataClass { Float, Int, Bool };
inline DataClass dtype_class(int dt) {
    switch (dt) {
        case HE_F16:
        case HE_BF16:
        case HE_F32: return DataClass::Float;
        case HE_U32: return DataClass::Int;
        case HE_BOOL: return DataClass::Bool;
    }
    fail(HE_ERR_INVALID, strfmt("bad dtype %d", dt));
}

// Bytes of device storage for `len` elements; Bool is a bitset rounded up to whole 32-bit words
// (helium/src/cuda/tensor_storage.rs:53-60).
inline size_t storage_bytes(int dt, size_t len) {
    if (dt == HE_BOOL) return (len + 31) / 32 * 4;
    return len * dtype_bits(dt) / 8;
}

const char* dtype_name(int dt);

// he_init has run in this process: code objects can be loaded.
bool device_initialised();

uint64_t fnv1a(const void* data, size_t n, uint64_t seed = 1469598103934665603ull);

// Overrides of the kernel generators' choices (HELIUM_HIP_GEMM_TILE, HELIUM_HIP_POINTWISE_RPT, ...). They exist for
// tuning and measurement and are dead unless the process starts with HELIUM_HIP_TUNING set: then every generator reads
// them through get(), and key() - all of them, sorted, as text - is part of every kernel-cache key and of the plan
// cache's, so a changed override never meets a kernel built under another. HELIUM_HIP_TUNING=measure also admits the
// switches that take a component out of a kernel (its results are then wrong on purpose).
namespace tuning {
bool enabled();
bool measuring();
const char* get(const char* name);  // nullptr when tuning is off or the variable is unset
int get_int(const char* name, int dflt);
std::string key();                  // empty when tuning is off
uint32_t hash();                    // 0 when tuning is off
}  // namespace tuning

}  // namespace he
