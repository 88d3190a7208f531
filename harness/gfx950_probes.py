"""Microbenchmarks of the gfx950 resources the fused GEMM's mainloop shares: the matrix pipe, LDS fragment reads, the
issue cost of direct global->LDS loads, and the L2 -> LDS operand stream. Measurement harness, not product: the
figures it prints are the denominators the design of `helium_amd/csrc/gemm.cpp` is argued from.

    python3 -m harness.gfx950_probes

Every probe is one workgroup of 8 waves per CU (256 workgroups), the GEMM's own launch shape. Times come from HIP
events around one launch of a fixed number of loop iterations; "clk" figures use the wave's own clock counter
(s_memtime) of workgroup 0.
"""
import sys

import numpy as np

import helium_amd as ha
from helium_amd import device

COMMON = r'''
typedef unsigned int u32;
typedef unsigned long long u64;
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
#define WAITCNT_VM(n) ((((n) & 15) | (((n) >> 4) << 14)))
#define MFMA(c, a, b) asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b))
#define RD128(dst, addr, off) asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
#define RDTR(dst, addr, off) asm volatile("ds_read_b64_tr_b16 %0, %1 offset:%2" : "=v"(dst) : "v"(addr), "n"(off))
'''

# One k-tile of the 256x256x64 GEMM per iteration and wave: 32 MFMAs (64 per SIMD with two waves on it), optionally the
# fragment reads of the A tile (16 ds_read_b128 = 16 KB per wave) and of the B tile (16 ds_read_b64_tr_b16 = 8 KB).
MFMA_LDS = COMMON + r'''
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void probe(u64* __restrict__ out, float* __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[131072];
    const u32 tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    for (u32 i = tid; i < 131072 / 4; i += 512) ((u32*)lds)[i] = 0u;
    __syncthreads();
    f32x16 acc[8];
    for (int i = 0; i < 8; i++) for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
    u32x4 fa[2][4]; u32x2 fb[2][4];
    for (int s = 0; s < 2; s++) for (int i = 0; i < 4; i++) { fa[s][i] = u32x4{0u, 0u, 0u, 0u}; fb[s][i] = u32x2{0u, 0u}; }
    const u32 a_addr = wave * 8192 + lane * 16, b_addr = 65536 + wave * 4096 + lane * 8;
    const u64 t0 = __builtin_amdgcn_s_memtime();
#pragma unroll 1
    for (int it = 0; it < ITERS; it++) {
#define STEP(cur, nxt) \
        if (NA > 0) { RD128(fa[nxt][0], a_addr, 0); RD128(fa[nxt][1], a_addr, 4096); } \
        MFMA(acc[0], fa[cur][0], fa[cur][1]); \
        if (NA > 0) { RD128(fa[nxt][2], a_addr, 8192); RD128(fa[nxt][3], a_addr, 12288); } \
        MFMA(acc[1], fa[cur][0], fa[cur][2]); \
        if (NTR > 0) { RDTR(fb[nxt][0], b_addr, 0); RDTR(fb[nxt][1], b_addr, 2048); } \
        MFMA(acc[2], fa[cur][1], fa[cur][1]); \
        if (NTR > 0) { RDTR(fb[nxt][2], b_addr, 1024); RDTR(fb[nxt][3], b_addr, 3072); } \
        MFMA(acc[3], fa[cur][1], fa[cur][2]); \
        MFMA(acc[4], fa[cur][2], fa[cur][3]); \
        MFMA(acc[5], fa[cur][2], fa[cur][0]); \
        MFMA(acc[6], fa[cur][3], fa[cur][3]); \
        MFMA(acc[7], fa[cur][3], fa[cur][0]); \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); \
        asm volatile("" :: "v"(fb[nxt][0]), "v"(fb[nxt][1]), "v"(fb[nxt][2]), "v"(fb[nxt][3]));
        STEP(0, 1)
        STEP(1, 0)
        STEP(0, 1)
        STEP(1, 0)
        if (BARRIER) __builtin_amdgcn_s_barrier();
    }
    const u64 t1 = __builtin_amdgcn_s_memtime();
    float s = 0.0f;
    for (int i = 0; i < 8; i++) for (int e = 0; e < 16; e++) s += acc[i][e];
    if (s == 12345.0f) sink[tid] = s;
    if (blockIdx.x == 0 && lane == 0) out[wave] = t1 - t0;
}
'''

# 8 MFMAs per iteration and wave with NL direct 1 KB global->LDS loads spread between them; every workgroup re-reads
# its own 64 KB (L2 hits), so the loads cost issue slots and LDS writes, not memory time.
LOAD_COST = COMMON + r'''
extern "C" __global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2)))
void probe(const unsigned char* __restrict__ g, u64* __restrict__ out, float* __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[131072];
    const u32 tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    f32x16 acc[8];
    for (int i = 0; i < 8; i++) for (int e = 0; e < 16; e++) acc[i][e] = 0.0f;
    u32x4 fa = {lane, 0u, 0u, 0u}, fb = {0u, 0u, 0u, 0u};
    const unsigned char* base = g + (size_t)blockIdx.x * (64u << 10);
    u32 goff = wave * 1024;
    const u64 t0 = __builtin_amdgcn_s_memtime();
#pragma unroll 1
    for (int it = 0; it < ITERS; it++) {
#pragma unroll
        for (int m = 0; m < 8; m++) {
            if (NL > 0 && (m % (8 / (NL > 0 ? NL : 1))) == 0) {
                __builtin_amdgcn_global_load_lds((GLOBAL_AS const void*)(base + goff + (u32)(lane * 16)),
                                                 (LDS_AS void*)(lds + wave * 16384 + (m & 7) * 1024), 16, 0, 0);
                goff = (goff + 8192) & ((64u << 10) - 1);
            }
            MFMA(acc[m], fa, fb);
        }
        __builtin_amdgcn_s_waitcnt(0x0F70 | WAITCNT_VM(2 * NL));
    }
    const u64 t1 = __builtin_amdgcn_s_memtime();
    __builtin_amdgcn_s_waitcnt(0x0F70);
    float s = 0.0f;
    for (int i = 0; i < 8; i++) for (int e = 0; e < 16; e++) s += acc[i][e];
    if (s == 12345.0f) sink[tid] = s;
    if (blockIdx.x == 0 && lane == 0) out[wave] = t1 - t0;
}
'''

# The operand stream of the 4096^3 bf16 GEMM and nothing else: 256 workgroups in the kernel's XCD-aware tile order each
# pull the 64 k-tiles (32 KB of A rows + 32 KB of B rows) of their 256x256 tile into a two-stage LDS ring with direct
# loads, waiting for a stage (and optionally meeting at a barrier) before they ask for the next but one.
STREAM = COMMON + r'''
extern "C" __global__ __launch_bounds__(512) void probe(const unsigned short* __restrict__ A, const unsigned short* __restrict__ B, u32* __restrict__ sink) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[2 * 65536];
    const u32 tid = threadIdx.x, lane = tid & 63, wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    u32 b = blockIdx.x;
    b = (b % 8u) * 32u + b / 8u;
    const u32 group = b / 64u, first = group * 4u;
    const u32 tile_m = first + (b % 64u) % 4u, tile_n = (b % 64u) / 4u;
    const u32 m0 = tile_m * 256u, n0 = tile_n * 256u;
    const u32 K = 4096u, N = 4096u;
    auto issue = [&](u32 kt, int slot) {
        const u32 k0 = kt * 64u;
#pragma unroll
        for (int i = 0; i < 8; i++) {
            const unsigned short* gp;
            u32 ldsoff;
            const u32 blk = wave * 4u + (i % 4);
            if (i < 4) {
                const u32 rr = lane / 8u, kc = lane % 8u;
                gp = (const unsigned short*)((const char*)(A + (size_t)(m0 + blk * 8u) * K + k0) + (u32)((rr * K + kc * 8u) * 2u));
                ldsoff = blk * 1024u;
            } else {
                const u32 kr = lane / 32u, nc = lane % 32u;
                gp = (const unsigned short*)((const char*)(B + (size_t)(k0 + blk * 2u) * N + n0) + (u32)((kr * N + nc * 8u) * 2u));
                ldsoff = 32768u + blk * 1024u;
            }
            __builtin_amdgcn_global_load_lds((GLOBAL_AS const void*)gp, (LDS_AS void*)(lds + (slot & 1) * 65536 + ldsoff), 16, 0, 0);
        }
    };
    issue(0, 0);
#pragma unroll 1
    for (u32 kt0 = 0; kt0 < 64u; kt0 += 2) {
#pragma unroll
        for (int d = 0; d < 2; d++) {
            const u32 kt = kt0 + d;
            if (kt + 1 < 64u) issue(kt + 1, (d + 1) % 2);
            if (kt + 1 < 64u && !DRAIN) __builtin_amdgcn_s_waitcnt(0x0F70 | WAITCNT_VM(8));
            else __builtin_amdgcn_s_waitcnt(0x0F70);
            if (BARRIER) __builtin_amdgcn_s_barrier();
        }
    }
    __syncthreads();
    const u32x4 acc = *(u32x4*)(lds + tid * 16);
    if (acc[0] == 0x12345u && acc[1] == 77u) sink[tid] = acc[2] + acc[3];
}
'''


def _build(src, defines):
    head = "".join(f"#define {k} {v}\n" for k, v in defines.items())
    mod = device.Module(device.rtc_compile(head + src, "probe", ["-O3"]))
    return mod, mod.function("probe")


def _time(mod, f, args, stream, warm=2, reps=1):
    for _ in range(warm):
        mod.launch(f, [256, 1, 1], [512, 1, 1], args, stream=stream)
    stream.synchronize()
    s, e = ha.Event(), ha.Event()
    s.record(stream)
    for _ in range(reps):
        mod.launch(f, [256, 1, 1], [512, 1, 1], args, stream=stream)
    e.record(stream)
    e.synchronize()
    return s.elapsed_ms(e) * 1e6 / reps  # ns per launch


def main():
    ha.device.init(0)
    stream = ha.Stream()
    out = ha.DeviceBuffer(8 * 16 * 2)
    sink = ha.DeviceBuffer(4096)
    print(f"device: {ha.device.device_arch(0)}, {ha.device.device_attr(0)} CUs; 256 workgroups x 8 waves in every probe")

    iters = 2000
    print("\n1. matrix pipe and LDS fragment reads, per k-tile of the 256x256x64 GEMM (64 v_mfma_f32_32x32x16_bf16 per SIMD):")
    base = None
    for na, ntr, bar, what in [(0, 0, 0, "MFMAs alone"), (1, 0, 0, "+ A fragment reads (128 KB per CU as ds_read_b128)"),
                               (1, 1, 0, "+ B fragment reads too (64 KB per CU as ds_read_b64_tr_b16)"),
                               (1, 1, 1, "+ one s_barrier per k-tile")]:
        mod, f = _build(MFMA_LDS, dict(NA=na, NTR=ntr, BARRIER=bar, ITERS=iters))
        ns = _time(mod, f, [out.ptr, sink.ptr], stream) / iters
        clk = int(out.to_numpy(np.uint64)[:8].max() / iters)
        base = base or ns
        lds_kb = 128 * na + 64 * ntr
        print(f"   {what:62s} {ns:7.0f} ns, {clk:5d} clk per k-tile ({clk / 64:.1f} clk per MFMA and SIMD"
              + (f"; {lds_kb * 1024 / clk:.0f} B/clk/CU read from LDS beside them" if lds_kb else "") + f"; clock {clk / ns:.2f} GHz)")

    print("\n2. what a direct global->LDS load (global_load_lds_dwordx4, 1 KB per wave) costs the MFMA stream of its SIMD"
          "\n   (16 MFMAs per SIMD and iteration, the loads hit L2):")
    g = ha.DeviceBuffer(256 * (64 << 10))
    g.fill_u8(0)
    iters = 4000
    first = None
    for nl in (0, 1, 2, 4):
        mod, f = _build(LOAD_COST, dict(NL=nl, ITERS=iters))
        ns = _time(mod, f, [g.ptr, out.ptr, sink.ptr], stream) / iters
        clk = out.to_numpy(np.uint64)[:8].max() / iters
        first = first or clk
        extra = (clk - first) / (2 * nl) if nl else 0.0
        print(f"   {nl} loads per 8 MFMAs and wave: {ns:6.0f} ns, {clk:6.0f} clk per iteration"
              + (f"  (+{extra:.1f} clk per load; the GEMM issues 16 per 64 MFMAs and SIMD: +{16 * extra / (64 * first / 16) * 100:.0f}%)" if nl else ""))

    print("\n3. the L2 -> LDS operand stream of the 4096^3 bf16 GEMM alone (1.07 GB per launch: every workgroup pulls 64 k-tiles"
          "\n   of 64 KB; operands rotate through 4 sets of 64 MB):")
    n = 4096
    rng = np.random.default_rng(1)
    sets = [(ha.DeviceBuffer.from_numpy(rng.integers(0, 65535, size=(n, n), dtype=np.uint16)),
             ha.DeviceBuffer.from_numpy(rng.integers(0, 65535, size=(n, n), dtype=np.uint16))) for _ in range(4)]
    for drain, bar, what in [(0, 0, "wait for the older stage only"), (0, 1, "+ a barrier per k-tile (the GEMM's own schedule)"),
                             (1, 1, "+ every load drained before the barrier")]:
        mod, f = _build(STREAM, dict(DRAIN=drain, BARRIER=bar))
        for i in range(200):
            mod.launch(f, [256, 1, 1], [512, 1, 1], [sets[i % 4][0].ptr, sets[i % 4][1].ptr, sink.ptr], stream=stream)
        stream.synchronize()
        s, e = ha.Event(), ha.Event()
        s.record(stream)
        for i in range(100):
            mod.launch(f, [256, 1, 1], [512, 1, 1], [sets[i % 4][0].ptr, sets[i % 4][1].ptr, sink.ptr], stream=stream)
        e.record(stream)
        e.synchronize()
        us = s.elapsed_ms(e) * 10
        print(f"   {what:50s} {us:6.1f} us per launch, {256 * 64 * 65536 / us / 1e6:5.1f} TB/s into LDS")
    return 0


if __name__ == "__main__":
    sys.exit(main())
