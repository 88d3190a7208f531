"""Runs a generated HIP kernel on the CPU for bounds and index checking (host AddressSanitizer).

The kernel text is compiled as host C++ behind a small shim: every GPU thread of a block is an OS thread,
__syncthreads() is a pthread barrier, __shared__ variables are function-static, blocks run one after another.
Operand buffers are heap allocations of exactly the tensor's size, so any out-of-bounds access of the kernel's
index arithmetic aborts the run. Only kernels without wave intrinsics can run this way.
"""
import os
import subprocess
import tempfile

import numpy as np

CLANG = "/opt/rocm/lib/llvm/bin/clang++"

SHIM = r"""
#include <pthread.h>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>
struct Dim3 { unsigned x = 0, y = 0, z = 0; };
static thread_local Dim3 threadIdx, blockIdx;
static Dim3 blockDim, gridDim;
static pthread_barrier_t g_bar;
// wave-level stand-ins (shuffles, matrix-core and transposing loads) meet on their own wave's barrier, so the waves of a
// block need not run the same instruction stream (two groups of waves half a k-tile apart)
static pthread_barrier_t g_wbar[16];
#define WAVE_BAR() pthread_barrier_wait(&g_wbar[threadIdx.x >> 6])
#define __global__
#define __device__
#define __forceinline__ inline
#define __launch_bounds__(...)
#define __shared__ static
#define __restrict__
#define __syncthreads() pthread_barrier_wait(&g_bar)
#define __builtin_nontemporal_load(p) (*(p))
#define __builtin_nontemporal_store(v, p) (*(p) = (v))
#include <cmath>
// wave shuffles: every thread of a wave calls in lockstep, so an exchange through memory between wave barriers works
static float g_shfl[1024];
static inline float __shfl_xor(float v, int mask, int width) {
    unsigned tid = threadIdx.x;
    g_shfl[tid] = v;
    WAVE_BAR();
    float r = g_shfl[(tid & ~63u) | ((tid & 63u) ^ (unsigned)mask)];
    WAVE_BAR();
    return r;
}
static inline int __float_as_int(float f) { int i; memcpy(&i, &f, 4); return i; }
static inline unsigned __float_as_uint(float f) { unsigned i; memcpy(&i, &f, 4); return i; }
static inline float atomicAdd(float* a, float v) {
    unsigned* ua = (unsigned*)a; unsigned old = __atomic_load_n(ua, __ATOMIC_RELAXED), nw;
    float f;
    do { memcpy(&f, &old, 4); f += v; memcpy(&nw, &f, 4); } while (!__atomic_compare_exchange_n(ua, &old, nw, false, __ATOMIC_SEQ_CST, __ATOMIC_RELAXED));
    return f;
}
template <class T> static inline T atomicMax(T* a, T v) {
    T old = __atomic_load_n(a, __ATOMIC_RELAXED);
    while (old < v && !__atomic_compare_exchange_n(a, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_RELAXED)) {}
    return old;
}
template <class T> static inline T atomicMin(T* a, T v) {
    T old = __atomic_load_n(a, __ATOMIC_RELAXED);
    while (old > v && !__atomic_compare_exchange_n(a, &old, v, false, __ATOMIC_SEQ_CST, __ATOMIC_RELAXED)) {}
    return old;
}
static inline unsigned atomicAdd(unsigned* a, unsigned v) { return __atomic_fetch_add(a, v, __ATOMIC_SEQ_CST); }
// blocks run one after another here, so the scratch exchange needs no atomicity
#define HE_WS_STORE(p, v) (*(p) = (v))
#define HE_WS_LOAD(p) (*(p))
#define HE_WS_TICKET(p) __atomic_fetch_add((p), 1u, __ATOMIC_RELAXED)
#define HE_WS_DRAIN()
static inline unsigned atomicOr(unsigned* a, unsigned v) { return __atomic_fetch_or(a, v, __ATOMIC_SEQ_CST); }
// matrix-core and transposing-LDS-load stand-ins: whole waves call them in lockstep, lanes meet in memory
typedef short emu_s16x8 __attribute__((ext_vector_type(8)));
typedef short emu_s16x4 __attribute__((ext_vector_type(4)));
typedef float emu_f32x16 __attribute__((ext_vector_type(16)));
static emu_s16x8 g_mfa[1024], g_mfb[1024];
static inline float emu_bf16(short h) { unsigned u = ((unsigned)(unsigned short)h) << 16; float f; memcpy(&f, &u, 4); return f; }
static inline float emu_f16(short h) { _Float16 x; memcpy(&x, &h, 2); return (float)x; }
template <class V, bool BF> static inline emu_f32x16 emu_mfma(V a, V b, emu_f32x16 c) {
    // v_mfma_f32_32x32x16: lane l holds A[l%32][(l/32)*8+j] and B[(l/32)*8+j][l%32]; c[i] is row (i/4)*8+(l/32)*4+i%4
    unsigned tid = threadIdx.x, base = tid & ~63u, lane = tid & 63u;
    g_mfa[tid] = __builtin_bit_cast(emu_s16x8, a);
    g_mfb[tid] = __builtin_bit_cast(emu_s16x8, b);
    WAVE_BAR();
    for (int i = 0; i < 16; i++) {
        unsigned row = (i / 4) * 8 + (lane / 32) * 4 + i % 4, col = lane % 32;
        float sum = 0;
        for (int k = 0; k < 16; k++) {
            short av = g_mfa[base + row + 32 * (k / 8)][k % 8], bv = g_mfb[base + col + 32 * (k / 8)][k % 8];
            sum += BF ? emu_bf16(av) * emu_bf16(bv) : emu_f16(av) * emu_f16(bv);
        }
        c[i] += sum;
    }
    WAVE_BAR();
    return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, x, y, z) emu_mfma<decltype(a), true>(a, b, c)
#define __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, x, y, z) emu_mfma<decltype(a), false>(a, b, c)
static float g_mfa32[1024], g_mfb32[1024];
static inline emu_f32x16 emu_mfma_f32(float a, float b, emu_f32x16 c) {
    // v_mfma_f32_32x32x2_f32: lane l holds A[l%32][l/32] and B[l/32][l%32]
    unsigned tid = threadIdx.x, base = tid & ~63u, lane = tid & 63u;
    g_mfa32[tid] = a; g_mfb32[tid] = b;
    WAVE_BAR();
    for (int i = 0; i < 16; i++) {
        unsigned row = (i / 4) * 8 + (lane / 32) * 4 + i % 4, col = lane % 32;
        c[i] += g_mfa32[base + row] * g_mfb32[base + col] + g_mfa32[base + 32 + row] * g_mfb32[base + 32 + col];
    }
    WAVE_BAR();
    return c;
}
#define __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, c, x, y, z) emu_mfma_f32(a, b, c)
static const short* g_traddr[1024];
static inline emu_s16x4 emu_tr16(const emu_s16x4* p) {
    // ds_read_b64_tr_b16, as measured on gfx950: within each group of 16 lanes, lane L gets element L%4 of the
    // four source lanes 4e + L/4 (e = 0..3)
    unsigned tid = threadIdx.x, gbase = tid & ~15u, L = tid & 15u;
    g_traddr[tid] = (const short*)p;
    WAVE_BAR();
    emu_s16x4 r;
    for (int e = 0; e < 4; e++) r[e] = g_traddr[gbase + 4 * e + L / 4][L % 4];
    WAVE_BAR();
    return r;
}
#define __builtin_amdgcn_ds_read_tr16_b64_v4i16(p) emu_tr16(p)
#define LDS_AS
#define GLOBAL_AS
// global_load_lds_dwordx4: lane L of the wave writes its 16 bytes at lds_base + L * 16
#define __builtin_amdgcn_global_load_lds(g, l, size, off, aux) memcpy((char*)(l) + (threadIdx.x & 63u) * (size), (const void*)(g), (size))
#define __builtin_amdgcn_s_waitcnt(x)
#define __builtin_amdgcn_s_barrier() pthread_barrier_wait(&g_bar)
#define KERNEL_ATTRS
#define __builtin_amdgcn_fence(...)
#define __builtin_amdgcn_sched_barrier(x)
#define __builtin_amdgcn_sched_group_barrier(a, b, c)
#define __builtin_amdgcn_s_setprio(x)
#define __builtin_amdgcn_wave_barrier() WAVE_BAR()
#define __builtin_amdgcn_readfirstlane(x) (x)
#define __expf expf
#define HE_FAST_RCP(x) (1.0f / (x))
#define HE_OPAQUE(x) (x)
#define __logf logf
#define __sinf sinf
#define __cosf cosf
#define __tanf tanf
#define __powf powf
static inline float he_fdividef(float x, float y) { return x / y; }
#define __fdividef he_fdividef
#define __fsqrt_rn sqrtf
"""

MAIN = r"""
template <class... A, size_t... I>
static void call_impl(void (*f)(A...), void** b, std::index_sequence<I...>) { f((A)b[I]...); }
template <class... A>
static void call(void (*f)(A...), void** b) { call_impl(f, b, std::index_sequence_for<A...>{}); }
static void** g_bufs;
static void* worker(void* arg) {
    unsigned tid = (unsigned)(size_t)arg;
    threadIdx.x = tid;
    for (unsigned b = 0; b < gridDim.x * gridDim.y; b++) {
        blockIdx.x = b % gridDim.x; blockIdx.y = b / gridDim.x;
        call(&ENTRY, g_bufs);
        pthread_barrier_wait(&g_bar);
    }
    return nullptr;
}
int main(int argc, char** argv) {
    // argv: grid threads (path bytes is_output)...
    gridDim.x = atoi(argv[1]); blockDim.x = atoi(argv[2]);
    gridDim.y = 1;
    if (const char* gy = getenv("EMUL_GRID_Y")) gridDim.y = atoi(gy);
    int nb = (argc - 3) / 3;
    std::vector<void*> bufs(nb); std::vector<size_t> sizes(nb); std::vector<int> isout(nb);
    for (int i = 0; i < nb; i++) {
        sizes[i] = strtoull(argv[4 + 3 * i], nullptr, 10); isout[i] = atoi(argv[5 + 3 * i]);
        bufs[i] = malloc(sizes[i] ? sizes[i] : 1);
        if (isout[i] != 1) { FILE* f = fopen(argv[3 + 3 * i], "rb"); if (fread(bufs[i], 1, sizes[i], f) != sizes[i]) return 3; fclose(f); }
        else memset(bufs[i], 0xEE, sizes[i]);
    }
    g_bufs = bufs.data();
    pthread_barrier_init(&g_bar, nullptr, blockDim.x);
    for (unsigned w = 0; w < (blockDim.x + 63) / 64; w++) pthread_barrier_init(&g_wbar[w], nullptr, blockDim.x - w * 64 < 64 ? blockDim.x - w * 64 : 64);
    std::vector<pthread_t> th(blockDim.x);
    for (unsigned t = 0; t < blockDim.x; t++) pthread_create(&th[t], nullptr, worker, (void*)(size_t)t);
    for (auto& t : th) pthread_join(t, nullptr);
    for (int i = 0; i < nb; i++) if (isout[i]) { FILE* f = fopen(argv[3 + 3 * i], "wb"); fwrite(bufs[i], 1, sizes[i], f); fclose(f); }
    for (auto p : bufs) free(p);
    return 0;
}
"""


def run_kernel(source, entry, grid, threads, buffers, flags=(), grid_y=1):
    """buffers: list of (numpy array, mode) with mode False/0 = input, True/1 = output (starts as 0xEE bytes),
    2 = in-out (starts from the array's contents). Returns the output arrays (same dtype/shape as given)."""
    with tempfile.TemporaryDirectory() as d:
        src = os.path.join(d, "k.cpp")
        with open(src, "w") as f:
            f.write(SHIM + source + f"\n#define ENTRY {entry}\n" + MAIN)
        exe = os.path.join(d, "k")
        subprocess.check_call([CLANG, "-O1", "-g", "-std=c++17", "-fsanitize=address", "-fno-omit-frame-pointer",
                               "-pthread", *flags, src, "-o", exe])
        argv = [exe, str(grid), str(threads)]
        paths = []
        for i, (a, is_out) in enumerate(buffers):
            p = os.path.join(d, f"b{i}.bin")
            paths.append(p)
            if int(is_out) != 1:
                np.ascontiguousarray(a).tofile(p)
            argv += [p, str(a.nbytes), str(int(is_out))]
        res = subprocess.run(argv, capture_output=True, text=True, env={**os.environ, "ASAN_OPTIONS": "detect_leaks=0", "EMUL_GRID_Y": str(grid_y)})
        if res.returncode != 0:
            raise AssertionError(f"CPU emulation of {entry} failed (exit {res.returncode}):\n{res.stderr[-4000:]}")
        outs = []
        for p, (a, is_out) in zip(paths, buffers):
            if is_out:
                outs.append(np.fromfile(p, dtype=a.dtype).reshape(a.shape))
        return outs
