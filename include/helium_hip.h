/*
 * helium_hip.h — C ABI of libhelium_hip.so, the MI355X (gfx950) execution backend for helium.
 *
 * Every function returns an int status (HE_OK == 0 on success). On failure the text of the error is kept
 * per thread and read with he_last_error(); the Rust shim panics with it, which preserves the reference's
 * behaviour (its backend methods are infallible in signature and `expect`/`panic!` on any driver failure,
 * helium/src/cuda.rs:67-76, helium/src/cuda/kernel_jit.rs:170-175).
 *
 * Handles are opaque pointers owned by the library until the matching *_destroy/_free call.
 * Each declaration cites the reference interface it replaces (paths relative to the reference tree).
 */
#ifndef HELIUM_HIP_H
#define HELIUM_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ---- status codes -------------------------------------------------------------------------------- */
enum {
    HE_OK = 0,
    HE_ERR_INVALID = 1,     /* bad argument / unsupported shape */
    HE_ERR_HIP = 2,         /* a HIP runtime call failed */
    HE_ERR_RTC = 3,         /* hiprtc compilation failed (log in he_last_error) */
    HE_ERR_UNSUPPORTED = 4, /* UnsupportedFusion (helium-kernel-generator/src/generators/matmul.rs:81-82) */
    HE_ERR_INTERNAL = 5
};

/* DataType, same order as helium-ir/src/data_type.rs:8-17. Bool is a bitset packed in 32-bit words. */
enum { HE_F16 = 0, HE_BF16 = 1, HE_F32 = 2, HE_U32 = 3, HE_BOOL = 4 };

const char* he_last_error(void);
/* Library version string and the GPU architecture every kernel is generated for ("gfx950"). */
const char* he_version(void);
const char* he_target_arch(void);

/* ==================================================================================================
 * 1. Device shim — replaces the cudarc driver-API call sites of helium/src/cuda/context.rs.
 * ================================================================================================== */
typedef struct he_stream_s* he_stream_t;
typedef struct he_event_s* he_event_t;
typedef struct he_module_s* he_module_t;
typedef struct he_function_s* he_function_t;

/* cuInit + cuDeviceGet + cuCtxCreate (context.rs:72-110). Uses the device's primary context. */
int he_init(int device);
int he_device_count(int* count);
/* cuDeviceGetAttribute (context.rs:83-94; helium-kernel-generator/src/architecture.rs:29-32,80). */
enum {
    HE_ATTR_CU_COUNT = 0,
    HE_ATTR_L2_BYTES = 1,
    HE_ATTR_LDS_BYTES_PER_BLOCK = 2,
    HE_ATTR_CLOCK_KHZ = 3,
    HE_ATTR_WAVEFRONT = 4,
    HE_ATTR_TOTAL_MEM_BYTES = 5
};
int he_device_attr(int device, int attr, int64_t* value);
/* Writes the gcnArchName of the device ("gfx950:sramecc+:xnack-") into buf. */
int he_device_arch(int device, char* buf, size_t buf_len);
int he_device_synchronize(void);

/* cuStreamCreate(NON_BLOCKING) / cuStreamDestroy (context.rs:205-212). Default priority only. */
int he_stream_create(he_stream_t* stream);
int he_stream_destroy(he_stream_t stream);
int he_stream_synchronize(he_stream_t stream);
/* cuLaunchHostFunc (context.rs:214-228): fn(user) runs on a runtime thread once prior work is done. */
int he_stream_host_callback(he_stream_t stream, void (*fn)(void*), void* user);
/* The raw hipStream_t, for callers that share the stream with other HIP code. */
void* he_stream_raw(he_stream_t stream);

/* cuEventCreate(BLOCKING_SYNC) / record / cuStreamWaitEvent / synchronize / elapsed (context.rs:247-295). */
int he_event_create(he_event_t* event);
int he_event_destroy(he_event_t event);
int he_event_record(he_event_t event, he_stream_t stream);
int he_event_wait(he_event_t event, he_stream_t stream);
int he_event_synchronize(he_event_t event);
int he_event_elapsed_ms(he_event_t start, he_event_t stop, float* ms);

/* cuMemAlloc / cuMemFree (allocator/device.rs:109,148,196), cuMemHostAlloc (allocator/host_pinned.rs:5). */
int he_malloc(void** dptr, size_t bytes);
int he_free(void* dptr);
int he_host_alloc(void** hptr, size_t bytes);
int he_host_free(void* hptr);
/* cuMemcpyHtoDAsync / DtoHAsync (tensor_storage.rs:101-105,125). stream may be NULL (null stream). */
int he_memcpy_h2d_async(void* dst, const void* src, size_t bytes, he_stream_t stream);
int he_memcpy_d2h_async(void* dst, const void* src, size_t bytes, he_stream_t stream);
int he_memcpy_d2d_async(void* dst, const void* src, size_t bytes, he_stream_t stream);
/* cuMemsetD8/D16/D32Async (tensor_storage.rs:176-207); count is in units of the element width. */
int he_memset_d8_async(void* dst, uint8_t value, size_t count, he_stream_t stream);
int he_memset_d16_async(void* dst, uint16_t value, size_t count, he_stream_t stream);
int he_memset_d32_async(void* dst, uint32_t value, size_t count, he_stream_t stream);

/* NVRTC compile (kernel_jit.rs:153-177; helium-kernel-generator/src/builder.rs:83-121) → hiprtc.
 * Compiles `source` for gfx950 and returns a malloc'd code object (free with he_rtc_free). `options` may add
 * compiler flags. Works without a GPU. Results are cached in memory by (source, options) like the
 * reference's PTX cache (kernel_jit.rs:128-134) and, when HELIUM_HIP_CACHE_DIR is set or the default cache
 * directory is writable, on disk. */
int he_rtc_compile(const char* source, const char* name, const char* const* options, int num_options,
                   void** code, size_t* code_size);
int he_rtc_free(void* code);
/* Counters of the compile cache: [0] hiprtc compilations, [1] memory hits, [2] disk hits. */
int he_rtc_stats(uint64_t stats[3]);

/* cuModuleLoadData / cuModuleGetFunction / cuModuleUnload (context.rs:150-170,310-327). */
int he_module_load(he_module_t* module, const void* code, size_t code_size);
int he_module_unload(he_module_t module);
int he_module_get_function(he_module_t module, const char* name, he_function_t* function);
/* cuLaunchKernel (kernel_jit.rs:267-280). args is an array of pointers to the argument values. */
int he_launch(he_function_t function, const uint32_t grid[3], const uint32_t block[3], uint32_t lds_bytes,
              he_stream_t stream, void** args);

/* ==================================================================================================
 * 2. Permute instruction — replaces helium/src/cuda/instr/permute_dims.rs + permute_dims/jit.rs (kernel K1).
 * ================================================================================================== */
typedef struct he_permute_s* he_permute_t;

/* PermuteDims::new + build_kernel (permute_dims.rs:31-33,66-87). `perm` follows numpy.transpose:
 * out.shape[i] = shape[perm[i]]. dtype is any 16- or 32-bit DataType. Compiles the kernel (precompile). */
int he_permute_create(he_permute_t* permute, const int64_t* shape, const int32_t* perm, int rank, int dtype);
/* Same, from a chain of SwapDims applied in order — what enumerate_swaps yields (permute_dims.rs:112-142). */
int he_permute_create_from_swaps(he_permute_t* permute, const int64_t* shape, int rank, const int32_t* swaps,
                                 int num_swaps, int dtype);
int he_permute_destroy(he_permute_t permute);
/* PermuteDims::execute (permute_dims.rs:35-58): one kernel launch on `stream`. */
int he_permute_execute(he_permute_t permute, const void* in, void* out, he_stream_t stream);
/* The generated HIP source, and a one-line description of the launch (variant, tile, grid). */
const char* he_permute_source(he_permute_t permute);
const char* he_permute_describe(he_permute_t permute);
/* compute_output_strides exactly as written in permute_dims.rs:159-171, kept for its unit test's known
 * answers (:180-187). For compositions of swaps that are not involutions it yields the strides of the
 * inverse permutation; the kernels above do not use it. */
int he_permute_reference_output_strides(const int64_t* shape, int rank, const int32_t* swaps, int num_swaps,
                                        int64_t* strides_out);

#ifdef __cplusplus
}
#endif
#endif /* HELIUM_HIP_H */
