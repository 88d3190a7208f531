// Fused GEMM generator for gfx950: bf16/f16 MFMA (v_mfma_f32_32x32x16) with f32 accumulators.
//
//   * Raw operands travel by direct global -> LDS loads (global_load_lds_dwordx4) into a ring of LDS stages; an
//     operand with mainloop ops (e.g. Relu, Mul by a tensor) is staged global -> registers -> LDS instead: its source
//     vectors are requested ahead of a k-tile's MFMAs, evaluated in f32 after them and rounded to the multiplicand
//     type on the way to LDS, so every element is computed once per workgroup and the MFMA loop reads finished
//     operands.
//   * A tiles sit in LDS as [m][k] (k contiguous, 16-byte chunks XOR-swizzled by m), read with one 128-bit LDS
//     load per MFMA operand. B tiles sit as [k][n] exactly as they are in memory and are read with the
//     transposing LDS load of gfx950 (ds_read_b64_tr_b16), which hands every lane the 4 consecutive k it needs.
//   * The epilogue program runs on the f32 accumulators: each wave passes its accumulators through a private LDS
//     strip to get row-major vectors of NV consecutive columns, so auxiliary tensors are read and outputs written
//     with coalesced 16-byte accesses. Column / row / scalar reductions are folded per lane, combined with wave
//     shuffles and through LDS per workgroup, parked as one partial per workgroup in a workspace, and folded in a
//     fixed order by a second small launch (no atomics: results are the same from run to run).
#include <cmath>
#include <cstring>
#include <sstream>

#include "kernels.h"

namespace he {

namespace {

struct Tile {
    int bm = 256, bn = 256, bk = 64;  // workgroup tile
    int wm = 2, wn = 4;               // waves along m / n (wm * wn * 64 threads)
    int stages = 2;                   // LDS stages (direct global->LDS loads use a deeper ring)
};

const char* kGemmPrelude = R"HIP(
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
#ifndef LDS_AS
#define LDS_AS __attribute__((address_space(3)))
#define GLOBAL_AS __attribute__((address_space(1)))
#endif
)HIP";

// Helpers that depend on the problem constants.
const char* kGemmHelpers = R"HIP(
#if MMA_F32
__device__ __forceinline__ u32x4 pack_chunk(const float (&v)[4]) {
    return u32x4{__builtin_bit_cast(u32, v[0]), __builtin_bit_cast(u32, v[1]), __builtin_bit_cast(u32, v[2]),
                 __builtin_bit_cast(u32, v[3])};
}
#else
__device__ __forceinline__ u32x4 pack_chunk(const float (&v)[8]) {
#if MMA_BF16
    bf16x8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = (__bf16)v[j];
#else
    f16x8 r;
#pragma unroll
    for (int j = 0; j < 8; j++) r[j] = (_Float16)v[j];
#endif
    return __builtin_bit_cast(u32x4, r);
}
#endif
)HIP";

// Kernel body; problem and tile constants are #defines in front of it.
const char* kGemmBody = R"HIP(
#define NWAVES (WAVES_M * WAVES_N)
#define NTHREADS (NWAVES * 64)
#define WTM (BM / WAVES_M)        /* wave tile */
#define WTN (BN / WAVES_N)
#define MB (WTM / 32)             /* 32x32 MFMA blocks per wave tile */
#define NB (WTN / 32)
#define ESZ (MMA_F32 ? 4 : 2)     /* bytes per multiplicand */
#define EPC (16 / ESZ)            /* multiplicands per 16-byte chunk */
#define KK (BK / (2 * EPC))       /* k-steps per tile: one 16-byte chunk per lane half */
#define A_CHUNKS (BK / EPC)       /* 16-byte chunks per A row */
#define B_CHUNKS (BN / EPC)
#define A_TILE_BYTES (BM * BK * ESZ)
#define B_TILE_BYTES (BK * BN * ESZ)
#define STAGE_BYTES (A_TILE_BYTES + B_TILE_BYTES)
#define A_PER_THREAD (BM * A_CHUNKS / NTHREADS)
#define B_PER_THREAD (BK * B_CHUNKS / NTHREADS)
#define EP (WTN + 4)              /* float pitch of the epilogue strip */
#define EPI_STEPS ((32 * WTN) / (64 * NVE))  /* NVE-wide steps a lane takes through one 32-row block */
#if NSTAGES * STAGE_BYTES < NWAVES * 32 * EP * 4
#error "the epilogue strip does not fit in the operand stages"
#endif
#define KT_ALL ((GK + BK - 1) / BK)
#define KT_PER_SPLIT ((KT_ALL + SPLIT_K - 1) / SPLIT_K)

__device__ __forceinline__ u32 a_off(u32 m, u32 kc) { return m * (BK * ESZ) + ((kc ^ ((m >> A_SWZ_SHIFT) & (A_CHUNKS - 1))) << 4); }
// B rows keep their memory order; the chunk index is XORed with 4 * (k % 4) for the transposing 16-bit reads
// (f32 operands are read one word per lane along n and need no swizzle).
#define B_SWZ(k) (MMA_F32 ? 0u : (((k) & 3) << 2) & (B_CHUNKS - 1))
__device__ __forceinline__ u32 b_chunk_off(u32 k, u32 nc) { return k * (BN * ESZ) + ((nc ^ B_SWZ(k)) << 4); }
__device__ __forceinline__ u32 b_off(u32 k, u32 n) { return b_chunk_off(k, (n * ESZ) >> 4) + ((n * ESZ) & 15); }
// A_KM: A arrives with m contiguous ([k][m] in memory, a transposed matrix). Its tile is then [k][m] in LDS, staged and
// read like a [k][n] B tile: 16-byte chunks along m, transposing reads for the 16-bit fragments.
#define AKM_CHUNKS (BM / EPC)
#define AKM_SWZ(k) (MMA_F32 ? 0u : (((k) & 3) << 2) & (AKM_CHUNKS - 1))
__device__ __forceinline__ u32 akm_chunk_off(u32 k, u32 mc) { return k * (BM * ESZ) + ((mc ^ AKM_SWZ(k)) << 4); }
__device__ __forceinline__ u32 akm_off(u32 k, u32 m) { return akm_chunk_off(k, (m * ESZ) >> 4) + ((m * ESZ) & 15); }
// B_NK: B arrives with k contiguous ([n][k] in memory). Its tile is then [n][k] in LDS too, staged and read like
// A's: the MFMA wants 8 consecutive k of one n per lane, which is one 16-byte chunk of row n.

#if MMA_F32
typedef f32x4 afrag_t;
typedef f32x4 bfrag_t;
#else
typedef s16x8 afrag_t;
typedef s16x8 bfrag_t;
#endif
struct WavePos {
    u32 lane, wave, wave_m, wave_n;
    u32 m0, n0;       /* first row / column of the workgroup's tile (gathers need absolute coordinates) */
    const void* img;  /* CONV_A: the image the A operand is gathered from */
    const void* bsrc; /* B_ROW_GATHER: the tensor B's rows are picked from */
#if CONV_A_FAST
    /* CONV_A with direct loads: the rows a lane fetches are the same in every k-tile, so their pixel coordinates are
       worked out once. Per direct-load instruction of the wave: image offset of the pixel's image, the pixel's
       coordinate terms that do not depend on the tap, and whether the row exists at all. */
    u32 cbase[A_DPW_MAX];
    int ch0[A_DPW_MAX], cw0[A_DPW_MAX];
#endif
};
#if CONV_A || CONV_B
// Where the taps that fall outside the image (or the matrix) are read from by the direct global->LDS loads.
__device__ __attribute__((aligned(16))) const u32 conv_zeros[4] = {0u, 0u, 0u, 0u};
#endif
#if MMA_F32
typedef float mul_t;   /* multiplicand as stored in global memory */
#else
typedef bf16_t mul_t;  /* any two-byte multiplicand: only the element size matters to the address arithmetic */
#endif

// Operand fragments of k-step kk from one LDS stage. `st` is __restrict__ on purpose: after inlining, every LDS
// read carries alias-scope information that separates it from the direct global->LDS writes into the *other*
// stage, so the compiler does not make the reads wait for those writes (vmcnt) before the MFMAs can start.
__device__ __forceinline__ void load_frags(const unsigned char* __restrict__ st, int kk, const WavePos& w,
                                           afrag_t (&af)[MB], bfrag_t (&bf)[NB]) {
    const unsigned char* la = st;
    const unsigned char* lb = st + A_TILE_BYTES;
    const u32 lane = w.lane;
#if MMA_F32
    // v_mfma_f32_32x32x2_f32: lane l supplies A[l % 32][l / 32] and B[l / 32][l % 32]. One k-step covers 8 k: each
    // lane half owns 4 consecutive k (one 16-byte chunk of its A row) and issues 4 MFMAs per output block.
#pragma unroll
    for (int i = 0; i < MB; i++) {
        const u32 row = w.wave_m * WTM + i * 32 + (lane & 31);
#if A_KM
#pragma unroll
        for (int e = 0; e < 4; e++) af[i][e] = *(const float*)(la + akm_off(kk * 8 + (lane >> 5) * 4 + e, row));
#else
        af[i] = *(const f32x4*)(la + a_off(row, kk * 2 + (lane >> 5)));
#endif
    }
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const u32 n = w.wave_n * WTN + j * 32 + (lane & 31);
#if B_NK
        bf[j] = *(const f32x4*)(lb + a_off(n, kk * 2 + (lane >> 5)));
#else
#pragma unroll
        for (int e = 0; e < 4; e++) bf[j][e] = *(const float*)(lb + b_off(kk * 8 + (lane >> 5) * 4 + e, n));
#endif
    }
#else
    const u32 grp = lane >> 4, sub = lane & 15;
#if A_KM
#pragma unroll
    for (int i = 0; i < MB; i++) {
        const u32 k = kk * 16 + (grp >> 1) * 8 + (sub >> 2);
        const u32 m = w.wave_m * WTM + i * 32 + (grp & 1) * 16 + (sub & 3) * 4;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(la + akm_off(k, m)));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(la + akm_off(k + 4, m)));
        af[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#else
#pragma unroll
    for (int i = 0; i < MB; i++) {
        const u32 row = w.wave_m * WTM + i * 32 + (lane & 31);
        af[i] = *(const s16x8*)(la + a_off(row, kk * 2 + (lane >> 5)));
    }
#endif
#if B_NK
    (void)grp; (void)sub;
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const u32 n = w.wave_n * WTN + j * 32 + (lane & 31);
        bf[j] = *(const s16x8*)(lb + a_off(n, kk * 2 + (lane >> 5)));
    }
#else
#pragma unroll
    for (int j = 0; j < NB; j++) {
        const u32 k = kk * 16 + (grp >> 1) * 8 + (sub >> 2);
        const u32 n = w.wave_n * WTN + j * 32 + (grp & 1) * 16 + (sub & 3) * 4;
        s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(lb + b_off(k, n)));
        s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LDS_AS s16x4*)(lb + b_off(k + 4, n)));
        bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
    }
#endif
#endif
}

__device__ __forceinline__ void mma_step(f32x16 (&acc)[MB][NB], const afrag_t (&af)[MB], const bfrag_t (&bf)[NB]) {
#if MMA_F32
#pragma unroll
    for (int e = 0; e < 4; e++)
#pragma unroll
        for (int i = 0; i < MB; i++)
#pragma unroll
            for (int j = 0; j < NB; j++)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i][e], bf[j][e], acc[i][j], 0, 0, 0);
#else
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NB; j++) {
#if MMA_BF16
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, af[i]),
                                                               __builtin_bit_cast(bf16x8, bf[j]), acc[i][j], 0, 0, 0);
#else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, af[i]),
                                                              __builtin_bit_cast(f16x8, bf[j]), acc[i][j], 0, 0, 0);
#endif
        }
#endif
}

// Fragment registers: double-buffered over the k-steps and carried from one k-tile to the next.
struct Frags {
    afrag_t a[2][MB];
    bfrag_t b[2][NB];
};
__device__ __forceinline__ void mma_or_skip(f32x16 (&acc)[MB][NB], const afrag_t (&af)[MB], const bfrag_t (&bf)[NB]) {
#if !(GEMM_SKIP & 4)
    mma_step(acc, af, bf);
#else
    acc[0][0][0] += (float)af[0][0] + (float)bf[0][0];
#endif
}
// One k-tile, rotated by one k-step: the MFMAs of the previous tile's last step run right after this tile's first
// fragment reads have been issued, so the LDS latency that follows the workgroup barrier hides behind them; this
// tile's own last step is left in `fr` for the next call (or for finish_tiles after the last tile).
template <class PerStep>
__device__ __forceinline__ void compute_tile(const unsigned char* __restrict__ st, f32x16 (&acc)[MB][NB], const WavePos& w,
                                             Frags& fr, PerStep&& per_step) {
    static_assert(KK % 2 == 0, "the fragment double buffer assumes an even number of k-steps per tile");
#if !(GEMM_SKIP & 2)
    load_frags(st, 0, w, fr.a[0], fr.b[0]);
#endif
    // A slice (or all) of the next tile's global->LDS traffic. Issuing a direct load takes tens of cycles; the MFMAs
    // of the previous tile's step KK-1 (zero fragments before the first tile) need nothing from memory and are
    // scheduled between the loads, so the matrix pipes work while the address unit does.
    per_step(0);
    mma_or_skip(acc, fr.a[1], fr.b[1]);
#pragma unroll
    for (int kk = 0; kk + 1 < KK; kk++) {
        per_step(kk + 1);
#if GEMM_SKIP & 2
        for (int i = 0; i < MB; i++) fr.a[(kk + 1) & 1][i] = fr.a[kk & 1][i];
        for (int j = 0; j < NB; j++) fr.b[(kk + 1) & 1][j] = fr.b[kk & 1][j];
#else
        load_frags(st, kk + 1, w, fr.a[(kk + 1) & 1], fr.b[(kk + 1) & 1]);
#endif
        mma_or_skip(acc, fr.a[kk & 1], fr.b[kk & 1]);
        SCHED_HINT
    }
    SCHED_PLAN
}
__device__ __forceinline__ void init_frags(Frags& fr) {
#pragma unroll
    for (int i = 0; i < MB; i++) fr.a[0][i] = fr.a[1][i] = afrag_t{};
#pragma unroll
    for (int j = 0; j < NB; j++) fr.b[0][j] = fr.b[1][j] = bfrag_t{};
}
__device__ __forceinline__ void finish_tiles(f32x16 (&acc)[MB][NB], const Frags& fr) { mma_or_skip(acc, fr.a[1], fr.b[1]); }

#if DIRECT_LOADS
// Operand tiles go from global memory straight into LDS (global_load_lds_dwordx4): a wave instruction fills
// 1 KB of LDS in lane order, so each lane fetches the global chunk whose swizzled LDS slot is lane * 16.
// `ga` / `gb` point at the tile's first A row / first B k-row (at this workgroup's columns).
#define A_DPW (DIRECT_A ? A_TILE_BYTES / 1024 / NWAVES : 0)  /* direct-load instructions per wave and tile */
#define B_DPW (DIRECT_B ? B_TILE_BYTES / 1024 / NWAVES : 0)
__device__ __forceinline__ void direct_issue(unsigned char* __restrict__ st, const mul_t* __restrict__ ga,
                                             const mul_t* __restrict__ gb, const WavePos& w, int i) {
#if GEMM_SKIP & 1
    return;
#endif
    const u32 lane = w.lane, wave = w.wave;
    if (i < A_DPW) {
        const u32 blk = wave * A_DPW + i;
#if A_KM
        const u32 krow = blk * (64 / AKM_CHUNKS) + lane / AKM_CHUNKS, pcm = lane % AKM_CHUNKS;
        const u32 mc = pcm ^ AKM_SWZ(krow);
        const mul_t* gpm = ga + (size_t)krow * GM + mc * EPC;
        __builtin_amdgcn_global_load_lds((GLOBAL_AS const void*)gpm, (LDS_AS void*)(st + blk * 1024), 16, 0, 0);
        return;
#endif
        const u32 row = blk * (64 / A_CHUNKS) + lane / A_CHUNKS, pc = lane % A_CHUNKS;
        const u32 kc = pc ^ ((row >> A_SWZ_SHIFT) & (A_CHUNKS - 1));
#if CONV_A_FAST
        // `ga` carries the tile's first k as an element offset from null. The channel count is a multiple of the
        // k-tile, so the whole tile lies in one filter tap: the tap is worked out once per wave (scalar), and the
        // lane adds it to the pixel terms it keeps from before the k-loop.
        size_t at;
        const bool inside = conv_tap_fast((u32)(ga - (const mul_t*)nullptr), kc * EPC, w.cbase[i], w.ch0[i], w.cw0[i], at);
        const mul_t* gp = inside ? (const mul_t*)w.img + at : (const mul_t*)conv_zeros;
#elif CONV_A
        // `ga` carries the tile's first k as an element offset from null: every lane computes the address of its
        // own chunk of 8 (4) channels of one filter tap, or points at zeros when the tap is outside the image
        size_t at;
        const bool inside = conv_tap(w.m0 + row, (u32)(ga - (const mul_t*)nullptr) + kc * EPC, at);
        const mul_t* gp = inside ? (const mul_t*)w.img + at : (const mul_t*)conv_zeros;
#else
        const mul_t* gp = ga + (size_t)row * GK + kc * EPC;
#endif
        __builtin_amdgcn_global_load_lds((GLOBAL_AS const void*)gp, (LDS_AS void*)(st + blk * 1024), 16, 0, 0);
    } else {
        const u32 blk = wave * B_DPW + (i - A_DPW);
#if B_NK
        const u32 row = blk * (64 / A_CHUNKS) + lane / A_CHUNKS, pc = lane % A_CHUNKS;
        const u32 kc = pc ^ ((row >> A_SWZ_SHIFT) & (A_CHUNKS - 1));
        const mul_t* gp = gb + (size_t)row * GK + kc * EPC;
#else
        const u32 krow = blk * (64 / B_CHUNKS) + lane / B_CHUNKS, pc = lane % B_CHUNKS;
        const u32 nc = pc ^ B_SWZ(krow);
#if CONV_B
        // `gb` carries the tile's first k (an output pixel index) as an element offset from null; the lane's chunk is
        // 8 (4) channels of tap n of that pixel, or zeros when the tap is outside the image
        size_t bat;
        const bool binside = conv_tap((u32)(gb - (const mul_t*)nullptr) + krow, w.n0 + nc * EPC, bat);
        const mul_t* gp = binside ? (const mul_t*)w.bsrc + bat : (const mul_t*)conv_zeros;
#elif B_ROW_GATHER
        // `gb` carries the tile's first k as an element offset from null; row k of B starts at b_row_addr(k)
        const mul_t* gp = (const mul_t*)w.bsrc + b_row_addr((u32)(gb - (const mul_t*)nullptr) + krow) + w.n0 + nc * EPC;
#else
        const mul_t* gp = gb + (size_t)krow * GN + nc * EPC;
#endif
#endif
        __builtin_amdgcn_global_load_lds((GLOBAL_AS const void*)gp, (LDS_AS void*)(st + A_TILE_BYTES + blk * 1024), 16, 0, 0);
    }
}
// Multiplies the tile in stage `rd` while requesting the tile that goes into stage `wr`.
__device__ __forceinline__ void direct_tile(const unsigned char* __restrict__ rd, unsigned char* __restrict__ wr,
                                            const mul_t* __restrict__ ga, const mul_t* __restrict__ gb, bool more,
                                            f32x16 (&acc)[MB][NB], const WavePos& w, Frags& fr) {
    compute_tile(rd, acc, w, fr, [&](int kk) {
        constexpr int per = ISSUE_FRONT ? (A_DPW + B_DPW) : (A_DPW + B_DPW + KK - 1) / KK;
        if (more) {
#pragma unroll
            for (int i = kk * per; i < (kk + 1) * per && i < A_DPW + B_DPW; i++) direct_issue(wr, ga, gb, w, i);
        }
    });
}
#endif

#ifndef KERNEL_ATTRS
/* NWAVES / 4 waves per SIMD and workgroup: with four waves each one owns the full 512-register budget; WGS_PER_CU
   workgroups are meant to share a CU */
#define KERNEL_ATTRS __attribute__((amdgpu_waves_per_eu(NWAVES / 4 * WGS_PER_CU, NWAVES / 4 * WGS_PER_CU)))
#endif
extern "C" __global__ __launch_bounds__(NTHREADS) KERNEL_ATTRS
void fused_matmul(KERNEL_PARAMS) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[NSTAGES * STAGE_BYTES];
    const u32 tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const u32 wave_m = wave / WAVES_N, wave_n = wave % WAVES_N;
    u32 tile_m, tile_n;
    TILE_ORDER
#if SPLIT_K > 1
    // blockIdx.y is the k-range index, not a batch index: this workgroup multiplies k-tiles [kt0, kt0 + KT)
    const u32 bz = 0, split = blockIdx.y, kt0 = split * KT_PER_SPLIT;
    const u32 KT = kt0 >= KT_ALL ? 0u : (KT_ALL - kt0 < KT_PER_SPLIT ? KT_ALL - kt0 : KT_PER_SPLIT);
#else
    const u32 bz = blockIdx.y, kt0 = 0;
    constexpr u32 KT = KT_ALL;
#endif
    const u32 m0 = tile_m * BM, n0 = tile_n * BN;
    EPILOGUE_EARLY
    // Optional rotation of the k loop per workgroup (tuning knob, off by default: workgroups that share an A or B
    // panel read the same k range at the same time, which is what lets them share it through L2).
    const u32 k_shift = KT ? (STAGGER_EXPR) % KT : 0u;
    auto k_tile = [&](u32 kt) { u32 x = kt + k_shift; return kt0 + (x >= KT ? x - KT : x); };

    f32x16 acc[MB][NB];
#pragma unroll
    for (int i = 0; i < MB; i++)
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) acc[i][j][e] = 0.0f;

    // Register staging of the operands that do not travel by direct global->LDS loads. A raw operand waits in
    // registers as the 16-byte chunk it was loaded as; a mainloop-fused one as its undecoded source vectors, which
    // stage_store turns into multiplicands after the tile's MFMAs.
#if !DIRECT_A
#if RAW_A
    u32x4 sa[A_PER_THREAD];
#else
    raw_a_t sa[A_PER_THREAD][SPLIT_A];
#endif
#endif
#if !DIRECT_B
#if RAW_B
    u32x4 sb[B_PER_THREAD];
#else
    raw_b_t sb[B_PER_THREAD][SPLIT_B];
#endif
#endif
    auto stage_load = [&](u32 kt) {
        const u32 k0 = k_tile(kt) * BK; (void)k0;
#if !DIRECT_A
#pragma unroll
        for (int i = 0; i < A_PER_THREAD; i++) {
            const u32 idx = tid + i * NTHREADS;
#if A_KM
            const u32 arow = k0 + idx / AKM_CHUNKS, acol = m0 + (idx % AKM_CHUNKS) * EPC;
#else
            const u32 arow = m0 + idx / A_CHUNKS, acol = k0 + (idx % A_CHUNKS) * EPC;
#endif
#if RAW_A
            sa[i] = fetch_a(FETCH_A_ARGS bz, arow, acol);
#else
            fetch_a_load(FETCH_A_ARGS bz, arow, acol, sa[i]);
#endif
        }
#endif
#if !DIRECT_B
#pragma unroll
        for (int i = 0; i < B_PER_THREAD; i++) {
            const u32 idx = tid + i * NTHREADS;
#if B_NK
            const u32 brow = n0 + idx / A_CHUNKS, bcol = k0 + (idx % A_CHUNKS) * EPC;
#else
            const u32 brow = k0 + idx / B_CHUNKS, bcol = n0 + (idx % B_CHUNKS) * EPC;
#endif
#if RAW_B
            sb[i] = fetch_b(FETCH_B_ARGS bz, brow, bcol);
#else
            fetch_b_load(FETCH_B_ARGS bz, brow, bcol, sb[i]);
#endif
        }
#endif
    };
    auto stage_store = [&](u32 kt, u32 buf) {
        const u32 k0 = k_tile(kt) * BK; (void)k0;
        unsigned char* la = lds + buf * STAGE_BYTES;
        unsigned char* lb = la + A_TILE_BYTES;
        (void)la; (void)lb;
#if !DIRECT_A
#pragma unroll
        for (int i = 0; i < A_PER_THREAD; i++) {
            const u32 idx = tid + i * NTHREADS;
#if A_KM
            const u32 aslot = akm_chunk_off(idx / AKM_CHUNKS, idx % AKM_CHUNKS);
            const u32 arow = k0 + idx / AKM_CHUNKS, acol = m0 + (idx % AKM_CHUNKS) * EPC;
#else
            const u32 aslot = a_off(idx / A_CHUNKS, idx % A_CHUNKS);
            const u32 arow = m0 + idx / A_CHUNKS, acol = k0 + (idx % A_CHUNKS) * EPC;
#endif
            (void)arow; (void)acol;
#if RAW_A
            *(u32x4*)(la + aslot) = sa[i];
#else
            *(u32x4*)(la + aslot) = fetch_a_eval(FETCH_A_ARGS bz, arow, acol, sa[i]);
#endif
        }
#endif
#if !DIRECT_B
#pragma unroll
        for (int i = 0; i < B_PER_THREAD; i++) {
            const u32 idx = tid + i * NTHREADS;
#if B_NK
            const u32 slot = a_off(idx / A_CHUNKS, idx % A_CHUNKS);
            const u32 brow = n0 + idx / A_CHUNKS, bcol = k0 + (idx % A_CHUNKS) * EPC;
#else
            const u32 slot = b_chunk_off(idx / B_CHUNKS, idx % B_CHUNKS);
            const u32 brow = k0 + idx / B_CHUNKS, bcol = n0 + (idx % B_CHUNKS) * EPC;
#endif
            (void)brow; (void)bcol;
#if RAW_B
            *(u32x4*)(lb + slot) = sb[i];
#else
            *(u32x4*)(lb + slot) = fetch_b_eval(FETCH_B_ARGS bz, brow, bcol, sb[i]);
#endif
        }
#endif
    };
#if CONV_A_FAST
    WavePos wpos = {lane, wave, wave_m, wave_n, m0, n0, (const void*)CONV_IMG_OR_NULL, (const void*)B_SRC_OR_NULL, {}, {}, {}};
#pragma unroll
    for (int i = 0; i < A_DPW_MAX; i++) conv_row_terms(m0 + (wave * A_DPW_MAX + i) * (64 / A_CHUNKS) + lane / A_CHUNKS, wpos.cbase[i], wpos.ch0[i], wpos.cw0[i]);
#else
    const WavePos wpos = {lane, wave, wave_m, wave_n, m0, n0, (const void*)CONV_IMG_OR_NULL, (const void*)B_SRC_OR_NULL};
#endif

/* s_waitcnt immediate: vmcnt lives in bits [3:0] and [15:14] */
#define WAITCNT_VM(n) ((((n) & 15) | (((n) >> 4) << 14)))
#if DIRECT_LOADS
#if CONV_A
    const mul_t* const ga0 = (const mul_t*)nullptr;  // direct_issue reads the k offset back from it
#define A_TILE_AT(k) (ga0 + (k))
#elif A_KM
    const mul_t* const ga0 = (const mul_t*)DIRECT_A_PTR + (size_t)bz * GK * GM + m0;
#define A_TILE_AT(k) (ga0 + (size_t)(k) * GM)
#else
    const mul_t* const ga0 = (const mul_t*)DIRECT_A_PTR + ((size_t)bz * GM + m0) * GK;
#define A_TILE_AT(k) (ga0 + (k))
#endif
#if B_NK
    const mul_t* const gb0 = (const mul_t*)DIRECT_B_PTR + ((size_t)bz * GN + n0) * GK;
#define B_TILE_AT(k) (gb0 + (k))
#elif B_ROW_GATHER || CONV_B
    const mul_t* const gb0 = (const mul_t*)nullptr;  // direct_issue reads the k offset back from it
#define B_TILE_AT(k) (gb0 + (k))
#else
    const mul_t* const gb0 = (const mul_t*)DIRECT_B_PTR + (size_t)bz * GK * GN + n0;
#define B_TILE_AT(k) (gb0 + (size_t)(k) * GN)
#endif
    // NSTAGES-deep ring of LDS stages: tile kt + NSTAGES - 1 is requested while tile kt is multiplied, so a
    // wave only ever waits for loads issued NSTAGES - 2 tiles earlier.
#pragma unroll
    for (int st = 0; st < NSTAGES - 1; st++)
        if (st < KT) {
#pragma unroll
            for (int i = 0; i < A_DPW + B_DPW; i++)
                direct_issue(lds + st * STAGE_BYTES, A_TILE_AT(k_tile(st) * BK), B_TILE_AT(k_tile(st) * BK), wpos, i);
        }
#endif
#if STAGED
    stage_load(0);
    stage_store(0, 0);
#endif
    Frags frags;
    init_frags(frags);
    for (u32 kt = 0; kt < KT; kt++) {
#if DIRECT_LOADS
        // tile kt must have landed; up to NSTAGES - 2 younger tiles may still be in flight
        const u32 younger = KT - 1 - kt < NSTAGES - 2 ? KT - 1 - kt : NSTAGES - 2;
        // (0x0070: no wait on the export counter, lgkmcnt(0) so that this wave's LDS reads and staged LDS stores are done)
        if (younger >= 3) __builtin_amdgcn_s_waitcnt(0x0070 | WAITCNT_VM(3 * (A_DPW + B_DPW)));
        else if (younger == 2) __builtin_amdgcn_s_waitcnt(0x0070 | WAITCNT_VM(2 * (A_DPW + B_DPW)));
        else if (younger == 1) __builtin_amdgcn_s_waitcnt(0x0070 | WAITCNT_VM(A_DPW + B_DPW));
        else __builtin_amdgcn_s_waitcnt(0x0070);
#endif
        // every wave's share of tile kt is in LDS (direct loads waited for above, staged stores made before the
        // barrier) and nobody still reads the stage that this iteration refills
#if DIRECT_LOADS
        // The bare barrier: __syncthreads() carries a fence for which the compiler drains every outstanding load,
        // the ones for younger stages included, and a ring deeper than two stages would gain nothing.
        __builtin_amdgcn_s_barrier();
#else
        __syncthreads();
#endif
        const u32 next = kt + NSTAGES - 1;
        const bool more = next < KT;
#if STAGED
        // The next tile's global loads are issued before any MFMA of this tile and consumed after the last one.
        if (more) stage_load(next);
        STAGE_SCHED_BARRIER
#endif
#if DIRECT_LOADS
        const u32 knext = more ? k_tile(next) * BK : 0u;
        direct_tile(lds + (kt % NSTAGES) * STAGE_BYTES, lds + (next % NSTAGES) * STAGE_BYTES, A_TILE_AT(knext),
                    B_TILE_AT(knext), more, acc, wpos, frags);
#else
        compute_tile(lds + (kt % NSTAGES) * STAGE_BYTES, acc, wpos, frags, [](int) {});
#endif
#if STAGED
        STAGE_SCHED_BARRIER
        if (more) stage_store(next, next % NSTAGES);
#endif
        __builtin_amdgcn_sched_barrier(0);
    }
    finish_tiles(acc, frags);
    __syncthreads();

    // ---- epilogue: accumulators -> wave-private LDS strip -> row-major NV-wide vectors -----------------------
    float* strip = (float*)lds + wave * (32 * EP);
    EPILOGUE_SETUP
#pragma unroll
    for (int i = 0; i < MB; i++) {
#pragma unroll
        for (int j = 0; j < NB; j++)
#pragma unroll
            for (int e = 0; e < 16; e++) {
                const u32 row = (e >> 2) * 8 + (lane >> 5) * 4 + (e & 3), col = j * 32 + (lane & 31);
                strip[row * EP + col] = acc[i][j][e];
            }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
        for (int step = 0; step < (32 * WTN) / (64 * NVE); step++) {
            EPILOGUE_PREFETCH
            const u32 idx = (step * 64 + lane) * NVE;
            const u32 row = idx / WTN, col = idx % WTN;
            const u32 m = m0 + wave_m * WTM + i * 32 + row;
            const u32 nn = n0 + wave_n * WTN + col;
            float acc_v[NVE];
#pragma unroll
            for (int k = 0; k < NVE; k++) acc_v[k] = strip[row * EP + col + k];
            const bool ok = m < GM && nn < GN;  // kept a run-time test even when every tile is full: with it folded away the
            // compiler merges the unrolled steps, hoists every step's loads and spills (2.3x slower on the 40-op epilogue)
            EPILOGUE_BODY
        }
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
    EPILOGUE_FINISH
}
)HIP";

bool is_raw_copy(const tp::Program& p, int root, int mma_dtype) {
    const tp::Expr& e = p.exprs[root];
    if (e.kind != tp::Expr::Load || !e.access.chain.empty() || e.access.dtype != mma_dtype) return false;
    const ir::Shape packed = ir::packed_strides(p.dims);
    for (size_t d = 0; d < p.dims.size(); d++)
        if (p.dims[d] > 1 && e.access.stride[d] != packed[d]) return false;  // the stride of an extent-1 dim is never used
    return true;
}

// The same program in two halves: `<name>_load` issues the full-vector loads into a Raw struct, `<name>_eval`
// turns them into the operand's NV values. A kernel calls the first before a tile's MFMAs and the second after.
std::string emit_operand_split(const tp::Program& p, int root, const std::string& name, int nv) {
    std::ostringstream s;
    std::string sig;
    for (size_t a = 0; a < p.args.size(); a++) sig += std::string("const ") + tp::c_type(p.args[a].dtype) + "* __restrict__ a" + std::to_string(a) + ", ";
    s << "struct Raw_" << name << " {\n" << tp::emit_raw_members(p, nv) << "};\n";
    tp::EmitCtx cx;
    cx.nv = nv;
    cx.phase = 1;
    s << "__device__ __forceinline__ void " << name << "_load(" << sig << "u32 cB0, u32 m, u32 n0, Raw_" << name << "& R) {\n(void)cB0; (void)m; (void)n0; (void)R;\n"
      << tp::emit_exprs(p, cx) << "}\n";
    cx.phase = 2;
    s << "__device__ __forceinline__ void " << name << "_eval(" << sig << "u32 cB0, u32 m, u32 n0, const Raw_" << name << "& R, float* out) {\n(void)cB0; (void)R;\n"
      << tp::emit_exprs(p, cx) << "#pragma unroll\nfor (int k = 0; k < " << nv << "; k++) out[k] = e" << root << "[k];\n}\n";
    return s.str();
}

}  // namespace

GemmProblem gemm_problem_from_fusion(const fir::OpGraph& g) {
    GemmProblem pr;
    fir::OpNode anchor = g.anchor();
    HE_REQUIRE(anchor != fir::kNoOpNode, HE_ERR_UNSUPPORTED, "fusion has no Matmul anchor");
    int anchors = 0;
    for (fir::OpNode n : g.nodes()) anchors += g.get(n).is_anchor();
    HE_REQUIRE(anchors == 1, HE_ERR_UNSUPPORTED, "a Core fusion holds exactly one Matmul");
    const fir::Op& mm = g.get(anchor);
    const fir::Shape3 &sa = g.shape(mm.a), &sc = g.shape(anchor);
    pr.batch = sc[0];
    pr.M = sc[1];
    pr.N = sc[2];
    pr.K = sa[2];
    pr.op_a = tp::lower_operand(g, mm.a, &pr.root_a);
    if (operand_b_prefers_nk(pr.op_a) && !tuning::get("HELIUM_HIP_GEMM_NO_KM")) {
        // the same test on A's [batch, M, K] program asks whether A's source is contiguous along m
        pr.op_a = tp::lower_operand(g, mm.a, &pr.root_a, true);
        pr.a_km = true;
    }
    pr.op_b = tp::lower_operand(g, mm.b, &pr.root_b);
    if (operand_b_prefers_nk(pr.op_b) && !tuning::get("HELIUM_HIP_GEMM_NO_NK")) {
        pr.op_b = tp::lower_operand(g, mm.b, &pr.root_b, true);
        pr.b_nk = true;
    }
    pr.epi = tp::lower_epilogue(g, anchor);
    // Multiplicand type (the fusion IR carries no Precision): f16 when every operand source is f16, f32 when every
    // one is f32, bf16 otherwise (mixed sources are rounded to bf16, the reference's MulBf16AccumF32).
    bool all_f16 = true, all_f32 = true;
    for (auto* p : {&pr.op_a, &pr.op_b})
        for (auto& a : p->args) {
            all_f16 = all_f16 && a.dtype == HE_F16;
            all_f32 = all_f32 && a.dtype == HE_F32;
        }
    pr.mma_dtype = all_f16 ? HE_F16 : all_f32 ? HE_F32 : HE_BF16;

    assemble_gemm_args(pr);
    return pr;
}

int choose_split_k(int64_t M, int64_t N, int64_t K, int64_t batch) {
    if (tuning::get("HELIUM_HIP_GEMM_NO_SPLIT_K") || batch != 1) return 1;
    if (const char* env = tuning::get("HELIUM_HIP_GEMM_SPLIT_K")) return std::max(1, atoi(env));
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128), k_tiles = (K + 63) / 64;
    if (tiles >= 128) return 1;
    // 64x64 tiles fill the chip before a split k range has to: the partial tiles of a split cost a second pass over
    // the output (a 3136 x 512 x 4608 convolution: 51 us with 128x128 tiles and four k ranges, 34 us with 64x64 tiles)
    if (((M + 63) / 64) * ((N + 63) / 64) >= 192) return 1;
    return (int)std::max<int64_t>(1, std::min<int64_t>({(384 + tiles - 1) / tiles, k_tiles / 8, 1024}));
}

bool operand_b_prefers_nk(const tp::Program& op_b) {
    const tp::Expr* big = nullptr;
    for (auto& e : op_b.exprs) {
        if (e.kind != tp::Expr::Load) continue;
        if (!e.access.chain.empty() || e.access.stride.size() != 3) return false;
        if (!big || op_b.args[e.access.arg].numel > op_b.args[big->access.arg].numel) big = &e;
    }
    // dims are [batch, K, N]: stride[1] walks k, stride[2] walks n
    return big && big->access.stride[1] == 1 && big->access.stride[2] > 1;
}

void assemble_gemm_args(GemmProblem& pr) {
    // Kernel arguments: every distinct input in id order, then every output in leaf order.
    std::vector<tp::Arg> inputs, outputs;
    auto add_input = [&](const tp::Arg& a) {
        for (auto& x : inputs)
            if (x.node == a.node) return;
        inputs.push_back(a);
    };
    for (auto* p : {&pr.op_a, &pr.op_b, &pr.epi})
        for (auto& a : p->args) {
            if (a.is_output) outputs.push_back(a);
            else add_input(a);
        }
    std::sort(inputs.begin(), inputs.end(), [](const tp::Arg& x, const tp::Arg& y) { return x.node < y.node; });
    pr.args = inputs;
    pr.args.insert(pr.args.end(), outputs.begin(), outputs.end());
    auto map_of = [&](const tp::Program& p) {
        std::vector<int> m;
        for (auto& a : p.args)
            for (size_t k = 0; k < pr.args.size(); k++)
                if (pr.args[k].node == a.node && pr.args[k].is_output == a.is_output) {
                    m.push_back((int)k);
                    break;
                }
        HE_REQUIRE(m.size() == p.args.size(), HE_ERR_INTERNAL, "argument mapping failed");
        return m;
    };
    pr.map_a = map_of(pr.op_a);
    pr.map_b = map_of(pr.op_b);
    pr.map_e = map_of(pr.epi);
}

void validate_gemm_epilogue(const tp::Program& epi) {
    HE_REQUIRE(epi.dims.size() <= 3, HE_ERR_UNSUPPORTED, "GEMM epilogues run over [batch, rows, cols]");
    HE_REQUIRE(!epi.outs.empty(), HE_ERR_UNSUPPORTED, "GEMM fusion without an output");
    for (auto& o : epi.outs) {
        HE_REQUIRE(epi.exprs[o.expr].cls == tp::Cls::F, HE_ERR_UNSUPPORTED, "GEMM epilogues store float values");
        if (o.reduce) HE_REQUIRE((o.rop == tp::ROp::Sum || o.rop == tp::ROp::Mean) && o.dtype == HE_F32, HE_ERR_UNSUPPORTED, "GEMM epilogues reduce with Sum or Mean, into f32");
        else HE_REQUIRE(o.dtype == HE_F32 || o.dtype == HE_BF16 || o.dtype == HE_F16, HE_ERR_UNSUPPORTED, "GEMM epilogues store float tensors");
    }
}

GemmKernel::GemmKernel(GemmProblem prob) : prob_(std::move(prob)) {
    const GemmProblem& pr = prob_;
    HE_REQUIRE(pr.M > 0 && pr.N > 0 && pr.K > 0 && pr.batch > 0, HE_ERR_INVALID, "empty GEMM");
    HE_REQUIRE(pr.M < (1ll << 31) && pr.N < (1ll << 31) && pr.K < (1ll << 31) &&
                   pr.batch * pr.M * std::max(pr.N, pr.K) < (1ll << 40),
               HE_ERR_INVALID, "GEMM too large");
    HE_REQUIRE(pr.mma_dtype == HE_BF16 || pr.mma_dtype == HE_F16 || pr.mma_dtype == HE_F32, HE_ERR_UNSUPPORTED,
               "unsupported multiplicand type");
    validate_gemm_epilogue(pr.epi);
    const bool f32 = pr.mma_dtype == HE_F32;
    const int epc = f32 ? 4 : 8;  // multiplicands per 16-byte chunk
    Tile t;
    bool small = false;
    const bool raw_a0 = pr.conv_a.on || (is_raw_copy(pr.op_a, pr.root_a, pr.mma_dtype) && (pr.a_km ? pr.M : pr.K) % epc == 0);
    const bool raw_b0 = pr.conv_b.on ? true : pr.b_rows.on ? pr.N % epc == 0 : is_raw_copy(pr.op_b, pr.root_b, pr.mma_dtype) && (pr.b_nk ? pr.K : pr.N) % epc == 0;
    const bool want_direct = !tuning::get("HELIUM_HIP_GEMM_NO_DIRECT");
    const int esz = 16 / epc;  // bytes per multiplicand
    if (const char* env = tuning::get("HELIUM_HIP_GEMM_TILE")) {
        int v[6] = {256, 256, 64, 2, 4, 2};
        int n = sscanf(env, "%d,%d,%d,%d,%d,%d", &v[0], &v[1], &v[2], &v[3], &v[4], &v[5]);
        HE_REQUIRE(n >= 5, HE_ERR_INVALID, "HELIUM_HIP_GEMM_TILE wants bm,bn,bk,wm,wn[,stages]");
        t = {v[0], v[1], v[2], v[3], v[4], v[5]};
    } else {
        if (f32) t.bk = 32;  // same bytes per tile row as 64 two-byte multiplicands
        // A skinny product (few output columns, many rows: a convolution with 64 output channels) takes tiles as
        // narrow as N, so that no matrix-core work is spent on columns that do not exist; eight waves of 64x32
        // (measured on [200704 x 576] x [576 x 64]: 71 us with 128x128 tiles, 44 us with 256x64).
        const bool skinny = !f32 && pr.N <= 64 && pr.N > 32 && pr.M >= 256 * 256;
        // Half as wide again (a convolution into 32 channels, the data gradient of one out of 32): four waves of 64x32.
        // Measured at batch 128 on the 112x112x32 layer of the resnet-train model: data gradient of the 3x3 stride-2
        // layer 469 -> 131 us, of the 1x1 shortcut 121 -> 34 us. When the operand is gathered element by element (a
        // 3-channel image) the gather is what takes the time, and twice the threads per row of pixels gather faster
        // than the unused half of a 256x64 tile costs (7x7 stem: 885 us with 128x128 tiles, 408 with 256x32, 276 with 256x64).
        const bool narrow = !f32 && pr.N <= 32 && pr.N > 16 && pr.M >= 256 * 256;
        const bool gathered_by_element = pr.conv_a.on && pr.conv_a.C % epc != 0;
        if (skinny || (narrow && gathered_by_element)) {
            t.bm = 256;
            t.bn = 64;
            t.wm = 4;
            t.wn = 2;
        } else if (narrow) {
            t.bm = 256;
            t.bn = 32;
            t.wm = 4;
            t.wn = 1;
        } else if (!f32 && pr.M <= 32 && pr.M > 16 && pr.N >= 128 && pr.conv_b.on && pr.conv_b.C % epc != 0) {
            // ... and a B operand gathered element by element (the filter gradient of the 7x7 stem on a 3-channel
            // image): the gather is bound by the loads it keeps in flight, so small workgroups, six of which share a
            // CU's LDS, and as many k ranges as fill the chip once (plan.cpp); 664 -> 439 us at batch 128
            t.bm = 32;
            t.bn = 64;
            t.wm = 1;
            t.wn = 2;
            small = true;
        } else if (!f32 && pr.M <= 32 && pr.M > 16 && pr.N >= 128) {
            // few output rows (a filter gradient with 32 output channels): four waves side by side
            // (the 7x7x3 stem's: 1095 us with 128x128 tiles, 668 us)
            t.bm = 32;
            t.bn = 128;
            t.wm = 1;
            t.wn = 4;
            small = true;
        } else if (!f32 && pr.M <= 64 && pr.M > 32 && pr.N >= 128) {
            // few output rows (a filter gradient with 64 output channels): tiles as low as M, of eight waves when the k
            // range is split (the 56x56x64 layer: 107 us with four waves, 103-105 with eight on 64x128 or 64x256 at batch
            // 128; at batch 64 48 us on 64x128 against 57 on 64x256)
            t.bm = 64;
            t.bn = 128;
            t.wm = t.wn = 2;
            if (pr.split_k > 1 && pr.N >= 256) t.wn = 4;
            small = true;
        } else if (!f32 && pr.M <= 128 && pr.M > 64 && pr.N >= 512 && pr.conv_b.on && pr.conv_b.C % epc == 0 && pr.split_k > 1 &&
                   !tuning::get("HELIUM_HIP_GEMM_NO_WIDE_CONV_TILES")) {
            // a filter gradient with 128 output channels: tiles as tall as M and 256 wide, so that the image's pixels
            // travel to half as many workgroups (plan.cpp deals the k range to one workgroup per CU)
            t.bm = 128;
            t.bn = 256;
            t.wm = 2;
            t.wn = 4;
            small = true;
        } else if (!f32 && pr.conv_a.on && pr.conv_a.C % epc == 0 && pr.N >= 256 && pr.N % 256 == 0 && pr.split_k == 1 &&
                   ((pr.M + 255) / 256) * (pr.N / 256) * pr.batch < 128 && ((pr.M + 127) / 128) * (pr.N / 256) * pr.batch >= 192 &&
                   !tuning::get("HELIUM_HIP_GEMM_NO_WIDE_CONV_TILES")) {
            // a convolution (or data gradient) into a multiple of 256 channels whose 256x256 tiles would leave half the chip
            // idle while 128x256 tiles fill three quarters of it or more: the filter travels to half as many workgroups
            // as with 128x128 tiles (the 14x14x256 layer at batch 128: forward 45.4 -> 41.4 us, data gradient 46.1 -> 42.5;
            // the 7x7x512 layer has 98 such tiles and loses: 47.8 -> 65.2)
            t.bm = 128;
            t.bn = 256;
            t.wm = 2;
            t.wn = 4;
            small = true;
        } else
        // Smaller problems take smaller tiles so that every CU gets work.
        // (a split k range multiplies the workgroups: the filter gradients of 256 and 512 channels keep the large tile,
        // 81 -> 70 us and 93 -> 78 us)
        // (... of 512; with 256 output channels eight waves on the small tile do better: 46.8 -> 41.5 and 71.1 -> 67.1 us)
        if (pr.M <= 128 || pr.N <= 128 || ((pr.M + 255) / 256) * ((pr.N + 255) / 256) * pr.batch * pr.split_k < 128 ||
            (pr.conv_b.on && !f32 && pr.conv_b.C % epc == 0 && pr.M <= 256)) {
            t.bm = t.bn = 128;
            t.wm = t.wn = 2;
            // (a convolution's gather on direct loads: eight waves of 64x32 - twice as many waves issue the per-lane
            // addressed loads and cover each other's waits; at batch 128 the 28x28x128 layer 59.6 -> 42.5 us forward and
            // 60.1 -> 50.3 us data gradient, 14x14x256 54.8 -> 45.7 and 57.3 -> 47.3, 7x7x512 54.7 -> 51.0 and 62.2 -> 49.6)
            // (the same for a filter gradient's gather: 128 output channels 82.4 -> 77.9 us, 54.5 -> 51.3 at stride 2)
            if (!f32 && ((pr.conv_a.on && pr.conv_a.C % epc == 0) || (pr.conv_b.on && pr.conv_b.C % epc == 0))) t.wn = 4;
            small = true;
            // still fewer workgroups than half the CUs: 64x64 tiles (one MFMA block per wave) spread the work
            // (a split k range multiplies the workgroups instead and keeps the tile's arithmetic intensity)
            if (pr.M > 64 && pr.N > 64 && ((pr.M + 127) / 128) * ((pr.N + 127) / 128) * pr.batch * pr.split_k < 128) {
                t.bm = t.bn = 64;
                t.wn = 2;
            }
        }
    }
    HE_REQUIRE(!pr.out_rows.on || (pr.split_k == 1 && pr.batch == 1 && pr.epi.outs.size() == 1 && !pr.epi.outs[0].reduce), HE_ERR_INVALID,
               "scattered output rows need a plain epilogue and a whole k range");
    HE_REQUIRE(t.bm % (t.wm * 32) == 0 && t.bn % (t.wn * 32) == 0 && (t.bk == 64 || t.bk == 32) && (!f32 || t.bk == 32), HE_ERR_INVALID, "bad GEMM tile");
    const int threads = t.wm * t.wn * 64;
    HE_REQUIRE(threads == 64 || threads == 128 || threads == 256 || threads == 512, HE_ERR_INVALID, "GEMM workgroups have 1, 2, 4 or 8 waves");
    HE_REQUIRE((t.bm * t.bk / epc) % threads == 0 && (t.bk * t.bn / epc) % threads == 0, HE_ERR_INVALID, "bad GEMM tile");
    HE_REQUIRE(t.stages >= 2 && t.stages <= 5 && t.stages * (t.bm + t.bn) * t.bk * (16 / epc) <= 160 * 1024, HE_ERR_INVALID,
               "GEMM tile exceeds LDS");
    const int wtn = t.bn / t.wn;
    // Reductions of the epilogue never meet in memory: every workgroup (for row sums: every wave) parks its partial
    // result in a workspace (plain stores) and a second small launch folds the partials of each output element in a
    // fixed order. Float atomics on
    // the outputs were the alternative: the 2048 waves of a 4096^2 product adding into one scalar cost 12 us of its
    // launch, and the per-channel sums of a convolution (784 workgroups, 64 columns = two cache lines) 680 us, since
    // atomics on one line are served one after another.
    struct RedOut {
        size_t out;         // index into epi.outs
        uint64_t off;       // first float of this output's partials
        int64_t elems;      // output elements
        int64_t parts;      // partials per element
        int64_t inner;      // partials of one element lie `inner` floats apart (GN for column sums, else 1)
    };
    std::vector<RedOut> reds;
    const int64_t tiles_m = (pr.M + t.bm - 1) / t.bm, tiles_n = (pr.N + t.bn - 1) / t.bn;
    uint64_t red_floats = 0;
    for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
        const tp::Out& o = pr.epi.outs[oi];
        if (!o.reduce) continue;
        HE_REQUIRE(pr.split_k == 1, HE_ERR_UNSUPPORTED, "a split k range has no epilogue reductions");
        RedOut r{oi, red_floats, 0, 0, 1};
        if (o.fold_m && !o.fold_n) {
            r.elems = pr.batch * pr.N;
            r.parts = tiles_m;
            r.inner = pr.N;
        } else if (o.fold_m && o.fold_n) {
            HE_REQUIRE(o.b_div >= 1 && pr.batch % o.b_div == 0, HE_ERR_INVALID, "bad batch fold of a reduction");
            r.elems = pr.batch / o.b_div;
            r.parts = o.b_div * tiles_m * tiles_n;
        } else {
            r.elems = pr.batch * pr.M;
            r.parts = tiles_n * t.wn;
        }
        HE_REQUIRE(r.elems < (1ll << 31) && r.parts < (1ll << 31), HE_ERR_UNSUPPORTED, "reduction too large");
        red_floats += (uint64_t)r.elems * r.parts;
        reds.push_back(r);
    }
    // Reductions of a small product fold inside the kernel: the last workgroup of a tile column adds that column's
    // partials (one per tile row), the last workgroup of all the scalar's. That saves the second launch where launches
    // are what a graph's time consists of (a 256 x 512 x 512 linear layer with bias, relu and column sums: 15.8 -> 13.7 us
    // per graph). A large product is better off with the second launch: its workgroups all end together, the tickets and
    // the loads of the partials are three dependent round trips at the very end of the kernel, and a 4096^3 product with
    // the README's epilogue took 155 us this way against 141. Row sums keep the second launch as well.
    // (a program that rides on the fold launch needs that launch)
    bool fold_in_kernel = !reds.empty() && pr.split_k == 1 && tiles_m * tiles_n * pr.batch <= 64 && !pr.epi.post &&
                          !tuning::get("HELIUM_HIP_GEMM_NO_TICKET_FOLD");
    for (auto& r : reds) {
        const tp::Out& o = pr.epi.outs[r.out];
        fold_in_kernel = fold_in_kernel && o.fold_m && (!o.fold_n || r.parts <= 4096);
    }
    // arrival counters: one per (batch index, tile column), then one per scalar output element group
    uint64_t ticket_cols = 0, ticket_all = 0;
    if (fold_in_kernel) {
        ticket_cols = (uint64_t)pr.batch * tiles_n;
        for (auto& r : reds)
            if (pr.epi.outs[r.out].fold_n) ticket_all = std::max<uint64_t>(ticket_all, (uint64_t)r.elems);
    }
    reduce_counters_ = ticket_cols + ticket_all;
    auto red_of = [&](size_t oi) -> const RedOut& {
        for (auto& r : reds)
            if (r.out == oi) return r;
        fail(HE_ERR_INTERNAL, "output is not a reduction");
    };

    const bool raw_a = raw_a0, raw_b = raw_b0;
    const int nva = std::min(epc, tp::pick_nv(pr.op_a, 16)), nvb = std::min(epc, tp::pick_nv(pr.op_b, 16));
    // Direct global->LDS loads need unpredicated, unmodified 16-byte chunks: raw operands and full tiles everywhere.
    // Each operand qualifies on its own; the other one then goes through registers.
    const bool direct_a = want_direct && raw_a && (pr.conv_a.on ? pr.conv_a.C % epc == 0 : pr.M % t.bm == 0 && pr.K % t.bk == 0) &&
                          (!pr.a_km || 64 % (t.bm / epc) == 0) && (t.bm * t.bk * esz / 1024) % (threads / 64) == 0 &&
                          !tuning::get("HELIUM_HIP_GEMM_NO_DIRECT_A");
    const bool direct_b = want_direct && raw_b && (pr.conv_b.on ? pr.conv_b.C % epc == 0 : pr.N % t.bn == 0 && pr.K % t.bk == 0) && (t.bk * t.bn * esz / 1024) % (threads / 64) == 0 &&
                          (pr.b_nk || 64 % (t.bn / epc) == 0) && !tuning::get("HELIUM_HIP_GEMM_NO_DIRECT_B");
    // A convolution's gather with direct loads, a channel count that is a multiple of the k-tile (every tile then lies in
    // one filter tap) and a wave that issues a whole number of loads: the per-lane address arithmetic of a load
    // shrinks from a full (pixel, tap) decomposition to a few adds.
    // (the image offset a lane carries across the k-loop is 32 bits wide: larger images take the general gather)
    const bool conv_a_fast = pr.conv_a.on && direct_a && pr.conv_a.C % t.bk == 0 && (t.bm * t.bk * esz / 1024) % (threads / 64) == 0 &&
                             (int64_t)pr.conv_a.N * pr.conv_a.H * pr.conv_a.W * pr.conv_a.C < (int64_t(1) << 32) &&
                             !tuning::get("HELIUM_HIP_GEMM_NO_CONV_FAST");
    if (!(direct_a && direct_b)) t.stages = 2;  // register staging is double-buffered only
    else if (!tuning::get("HELIUM_HIP_GEMM_TILE") && small) {
        // A grid that leaves CUs idle is bound by the latency of its k-loop: keep as many tiles in flight as LDS holds.
        // With more than one workgroup per CU (a split k range) the LDS is better spent on a second and third
        // workgroup, whose loads hide each other's waits (filter gradient of a 64-channel layer: 66 -> 56 us).
        const int64_t workgroups = ((pr.M + t.bm - 1) / t.bm) * ((pr.N + t.bn - 1) / t.bn) * pr.batch * pr.split_k;
        // (not for a data gradient's gather: at batch 128 the 7x7x512 layer takes 54.2 us with four stages, 49.7 with three,
        // 48.9 with two, the 14x14x256 layer at batch 64 29.3 / 27.5 / 27.8; the forward gather does not care)
        const bool deeper = !(pr.conv_a.on && pr.conv_a.bwd);
        while (deeper && workgroups <= 256 && t.stages < 4 && (t.stages + 1) * (t.bm + t.bn) * t.bk * esz <= 128 * 1024) t.stages++;
    }
    // All direct loads of the next tile are issued at the start of a tile's MFMAs (the round trip needs the whole
    // tile to hide); HELIUM_HIP_GEMM_ISSUE=0 spreads them over the k-steps instead.
    const bool issue_front = tuning::get("HELIUM_HIP_GEMM_ISSUE") ? atoi(tuning::get("HELIUM_HIP_GEMM_ISSUE")) != 0 : true;
    int nve = tp::pick_nv(pr.epi, 32);
    while (nve > 1 && ((32 * wtn) % (64 * nve) != 0)) nve /= 2;
    nve = std::min(nve, 8);
    const int lanes_per_row = wtn / nve;           // lanes that share one row of the strip in one step
    const int colsets = std::max(1, lanes_per_row / 64);  // distinct column sets a lane visits

    std::ostringstream s;
    s << "// fused_matmul generated for gfx950: [" << pr.batch << "," << pr.M << "," << pr.K << "] x [" << pr.batch << ","
      << pr.K << "," << pr.N << "], tile " << t.bm << "x" << t.bn << "x" << t.bk << "\n";
    s << tp::emit_prelude(pr.epi) << kGemmPrelude;
    s << "#define GM " << pr.M << "u\n#define GN " << pr.N << "u\n#define GK " << pr.K << "u\n";
    // Two workgroups share a CU when the LDS ring of one takes at most half of it: the second one's mainloop then runs
    // under the first one's epilogue, and a launch of a few workgroups per CU ends in a shorter tail. For that the
    // waves of both must fit the register file, so the allocation is held to the budget of twice the waves.
    std::string wgs_per_cu_attr;
    {
        const int lds_bytes = t.stages * (t.bm + t.bn) * t.bk * esz;
        const int acc_regs = t.bm * t.bn / threads;
        int wgs = tuning::get("HELIUM_HIP_GEMM_WGS_PER_CU") ? atoi(tuning::get("HELIUM_HIP_GEMM_WGS_PER_CU")) : (lds_bytes * 2 <= 160 * 1024 && acc_regs <= 32 ? 2 : 1);
        if (threads < 256) wgs = 1;
        wgs_per_cu_attr = "\n#define WGS_PER_CU " + std::to_string(std::max(1, wgs));
    }
    s << "#define BM " << t.bm << "\n#define BN " << t.bn << "\n#define BK " << t.bk << "\n#define WAVES_M " << t.wm
      << "\n#define WAVES_N " << t.wn << wgs_per_cu_attr << "\n#define NSTAGES " << t.stages << "\n#define NVE " << nve << "\n#define MMA_BF16 " << (pr.mma_dtype == HE_BF16 ? 1 : 0) << "\n#define MMA_F32 " << (f32 ? 1 : 0)
      << "\n#define STAGGER_EXPR " << (tuning::measuring() && tuning::get("HELIUM_HIP_GEMM_STAGGER") ? tuning::get("HELIUM_HIP_GEMM_STAGGER") : "0u")
      << "\n#define ISSUE_FRONT " << (issue_front ? 1 : 0)
      // measurement only (HELIUM_HIP_TUNING=measure): bit 0 drops the direct loads, bit 1 the fragment reads, bit 2 the
      // MFMAs - the kernel's results are then wrong, its timing tells what the rest costs
      << "\n#define GEMM_SKIP " << (tuning::measuring() ? tuning::get_int("HELIUM_HIP_GEMM_SKIP", 0) : 0)
      << "\n#define DIRECT_A " << (direct_a ? 1 : 0) << "\n#define DIRECT_B " << (direct_b ? 1 : 0)
      << "\n#define CONV_A_FAST " << (conv_a_fast ? 1 : 0) << "\n#define A_DPW_MAX " << std::max(1, t.bm * t.bk * esz / 1024 / (threads / 64))
      << "\n#define A_KM " << (pr.a_km ? 1 : 0) << "\n#define B_NK " << (pr.b_nk ? 1 : 0) << "\n#define CONV_A " << (pr.conv_a.on ? 1 : 0) << "\n#define CONV_IMG p" << (pr.conv_a.on ? pr.map_a[0] : 0)
      << "\n#define CONV_IMG_OR_NULL " << (pr.conv_a.on ? "p" + std::to_string(pr.map_a[0]) : std::string("nullptr"))
      << "\n#define B_ROW_GATHER " << (pr.b_rows.on ? 1 : 0) << "\n#define CONV_B " << (pr.conv_b.on ? 1 : 0) << "\n#define SPLIT_K " << pr.split_k
      << "\n#define B_SRC_OR_NULL " << (pr.b_rows.on || pr.conv_b.on ? "p" + std::to_string(pr.map_b[0]) : std::string("nullptr")) << "\n#define DIRECT_LOADS (DIRECT_A || DIRECT_B)\n#define STAGED (!DIRECT_A || !DIRECT_B)"
      << "\n#define DIRECT_A_PTR p" << (direct_a ? pr.map_a[0] : 0)
      << "\n#define DIRECT_B_PTR p" << (direct_b ? pr.map_b[0] : 0) << "\n#define STAGE_SCHED_BARRIER "
      << ((tuning::get("HELIUM_HIP_GEMM_PIN") ? atoi(tuning::get("HELIUM_HIP_GEMM_PIN")) != 0 : true) ? "__builtin_amdgcn_sched_barrier(0);" : "") << "\n#define A_SWZ_SHIFT " << (tuning::get("HELIUM_HIP_GEMM_ASWZ") ? atoi(tuning::get("HELIUM_HIP_GEMM_ASWZ")) : (t.bk == 64 ? 1 : 2)) << "\n";

    s << kGemmHelpers;
    // kernel parameters
    {
        std::ostringstream ps;
        for (size_t a = 0; a < pr.args.size(); a++)
            ps << (a ? ", " : "") << (pr.args[a].is_output ? "" : "const ") << tp::c_type(pr.args[a].dtype) << "* __restrict__ p" << a;
        if (pr.split_k > 1) ps << ", float* __restrict__ splitk_ws";
        if (!reds.empty()) ps << ", float* __restrict__ red_ws";
        if (fold_in_kernel) ps << ", u32* __restrict__ red_cnt";
        s << "#define KERNEL_PARAMS " << ps.str() << "\n";
    }
    // operand fetchers
    auto emit_fetch = [&](const char* which, const tp::Program& p, int root, const std::vector<int>& map, bool raw, int nv,
                          const char* rows, const char* cols, bool aligned) {
        // rows/cols: extents of the operand matrix ("GM","GK" for A; "GK","GN" for B)
        std::ostringstream args, params;
        for (size_t a = 0; a < p.args.size(); a++) {
            args << "p" << map[a] << ", ";
            params << "const " << tp::c_type(p.args[a].dtype) << "* __restrict__ q" << a << ", ";
        }
        std::string W = which;
        s << "#define FETCH_" << (W == "a" ? "A" : "B") << "_ARGS " << args.str() << "\n";
        const std::string X = (W == "a" ? "A" : "B");
        s << "#define RAW_" << X << " " << (raw ? 1 : 0) << "\n#define SPLIT_" << X << " " << epc / nv << "\n";
        if (raw) {
            s << "__device__ __forceinline__ u32x4 fetch_" << W << "(" << params.str() << "u32 b, u32 row, u32 col) {\n";
            if (aligned)  // every tile is full: no predication on the operand loads
                s << "return *(const u32x4*)(q0 + ((size_t)b * " << rows << " + row) * " << cols << " + col);\n}\n";
            else
                s << "u32x4 v = {0u, 0u, 0u, 0u};\nif (row < " << rows << " && col < " << cols << ") v = *(const u32x4*)(q0 + ((size_t)b * "
                  << rows << " + row) * " << cols << " + col);\nreturn v;\n}\n";
            return;
        }
        // Mainloop-fused operand: loads first (fetch_x_load), arithmetic and rounding to the multiplicand type later
        // (fetch_x_eval), so that the memory latency is covered by the MFMAs in between.
        s << emit_operand_split(p, root, "operand_" + W, nv);
        std::string pass;
        for (size_t a = 0; a < p.args.size(); a++) pass += "q" + std::to_string(a) + ", ";
        const std::string guard = aligned ? "" : "if (row < " + std::string(rows) + " && col + j < " + cols + ") ";
        s << "typedef Raw_operand_" << W << " raw_" << W << "_t;\n";
        s << "__device__ __forceinline__ void fetch_" << W << "_load(" << params.str() << "u32 b, u32 row, u32 col, raw_" << W << "_t (&R)[" << epc / nv << "]) {\n"
          << "#pragma unroll\nfor (int j = 0; j < " << epc << "; j += " << nv << ") " << guard << "operand_" << W << "_load(" << pass << "b, row, col + j, R[j / " << nv << "]);\n}\n";
        s << "__device__ __forceinline__ u32x4 fetch_" << W << "_eval(" << params.str() << "u32 b, u32 row, u32 col, const raw_" << W << "_t (&R)[" << epc / nv << "]) {\n"
          << "float v[" << epc << "];\n#pragma unroll\nfor (int j = 0; j < " << epc << "; j += " << nv << ") {\n";
        if (aligned) s << "operand_" << W << "_eval(" << pass << "b, row, col + j, R[j / " << nv << "], v + j);\n}\n";
        else s << guard << "operand_" << W << "_eval(" << pass << "b, row, col + j, R[j / " << nv << "], v + j);\nelse {\n#pragma unroll\nfor (int k = 0; k < " << nv << "; k++) v[j + k] = 0.0f; }\n}\n";
        s << "return pack_chunk(v);\n}\n";
    };
    auto emit_conv_tap = [&](const GemmProblem::ConvGather& cv) {
        // (row, col) = (pixel (n, p, q), tap (r, s, c)) -> element offset in the gathered NHWC tensor; false when the
        // tap lies outside it (or outside the matrix)
        s << "__device__ __forceinline__ bool conv_tap(u32 row, u32 col, size_t& at) {\n"
          << "const u32 n = row / " << cv.P * cv.Q << "u, pq = row % " << cv.P * cv.Q << "u, p = pq / " << cv.Q << "u, q = pq % " << cv.Q << "u;\n"
          << "const u32 rs = col / " << cv.C << "u, c = col % " << cv.C << "u, r = rs / " << cv.S << "u, sx = rs % " << cv.S << "u;\n";
        if (!cv.bwd)
            s << "const int ih = (int)(p * " << cv.sh << "u + r * " << cv.dh << "u) - " << cv.ph << ", iw = (int)(q * " << cv.sw << "u + sx * " << cv.dw << "u) - " << cv.pw << ";\n"
              << "const bool hit = true;\n";
        else
            s << "const int th = (int)p + " << cv.ph << " - (int)(r * " << cv.dh << "u), tw = (int)q + " << cv.pw << " - (int)(sx * " << cv.dw << "u);\n"
              << "const bool hit = th >= 0 && tw >= 0 && th % " << cv.sh << " == 0 && tw % " << cv.sw << " == 0;\n"
              << "const int ih = th / " << cv.sh << ", iw = tw / " << cv.sw << ";\n";
        s << "at = (((size_t)n * " << cv.H << "u + (u32)ih) * " << cv.W << "u + (u32)iw) * " << cv.C << "u + c;\n"
          << "return row < " << cv.N * cv.P * cv.Q << "u && col < " << cv.R * cv.S * cv.C << "u && hit && ih >= 0 && ih < " << cv.H << " && iw >= 0 && iw < " << cv.W << ";\n}\n";
    };
    if (conv_a_fast) {
        const auto& cv = pr.conv_a;
        // row -> (image offset, tap-independent coordinate terms); a row beyond the matrix gets coordinates that no tap
        // brings inside the image
        s << "__device__ __forceinline__ void conv_row_terms(u32 row, u32& base, int& h0, int& w0) {\n"
          << "const u32 n = row / " << cv.P * cv.Q << "u, pq = row % " << cv.P * cv.Q << "u, p = pq / " << cv.Q << "u, q = pq % " << cv.Q << "u;\n"
          << "base = n * " << cv.H * cv.W * cv.C << "u;\n";
        if (!cv.bwd) s << "h0 = (int)(p * " << cv.sh << "u) - " << cv.ph << "; w0 = (int)(q * " << cv.sw << "u) - " << cv.pw << ";\n";
        else s << "h0 = (int)p + " << cv.ph << "; w0 = (int)q + " << cv.pw << ";\n";
        s << "if (row >= " << cv.N * cv.P * cv.Q << "u) { base = 0u; h0 = -(1 << 24); w0 = -(1 << 24); }\n}\n";
        // k0: first k of the tile (uniform), kc: the lane's channel offset inside the tile
        s << "__device__ __forceinline__ bool conv_tap_fast(u32 k0, u32 kc, u32 base, int h0, int w0, size_t& at) {\n"
          << "const u32 rs = k0 / " << cv.C << "u, c = k0 % " << cv.C << "u + kc, r = rs / " << cv.S << "u, sx = rs % " << cv.S << "u;\n";
        if (!cv.bwd)
            s << "const int ih = h0 + (int)(r * " << cv.dh << "u), iw = w0 + (int)(sx * " << cv.dw << "u);\nconst bool hit = true;\n";
        else
            s << "const int th = h0 - (int)(r * " << cv.dh << "u), tw = w0 - (int)(sx * " << cv.dw << "u);\n"
              << "const bool hit = th >= 0 && tw >= 0 && th % " << cv.sh << " == 0 && tw % " << cv.sw << " == 0;\n"
              << "const int ih = th / " << cv.sh << ", iw = tw / " << cv.sw << ";\n";
        s << "at = (size_t)base + (size_t)(((u32)ih * " << cv.W << "u + (u32)iw) * " << cv.C << "u + c);\n"
          << "return k0 < " << cv.R * cv.S * cv.C << "u && hit && ih >= 0 && ih < " << cv.H << " && iw >= 0 && iw < " << cv.W << ";\n}\n";
    }
    // Body of a gather that fetches EPC consecutive taps (columns) of one pixel (row) element by element, for images whose
    // channel count does not fill 16-byte chunks (a 3-channel image: 8 elements span 3 taps): the pixel is decomposed
    // once, and the tap walks on by one channel per element instead of being decomposed 8 times.
    auto emit_elementwise_gather = [&](const GemmProblem::ConvGather& cv) {
            s << "float v[" << epc << "];\n"
              << "const u32 n = row / " << cv.P * cv.Q << "u, pq = row % " << cv.P * cv.Q << "u, p = pq / " << cv.Q << "u, q = pq % " << cv.Q << "u;\n"
              << "u32 rs = col / " << cv.C << "u, c = col % " << cv.C << "u, r = rs / " << cv.S << "u, sx = rs % " << cv.S << "u;\n"
              << "const bool row_ok = row < " << cv.N * cv.P * cv.Q << "u;\n"
              << "#pragma unroll\nfor (int j = 0; j < " << epc << "; j++) {\n";
            if (!cv.bwd)
                s << "const int ih = (int)(p * " << cv.sh << "u + r * " << cv.dh << "u) - " << cv.ph << ", iw = (int)(q * " << cv.sw << "u + sx * " << cv.dw << "u) - " << cv.pw << ";\n"
                  << "const bool hit = true;\n";
            else
                s << "const int th = (int)p + " << cv.ph << " - (int)(r * " << cv.dh << "u), tw = (int)q + " << cv.pw << " - (int)(sx * " << cv.dw << "u);\n"
                  << "const bool hit = th >= 0 && tw >= 0 && th % " << cv.sh << " == 0 && tw % " << cv.sw << " == 0;\n"
                  << "const int ih = th / " << cv.sh << ", iw = tw / " << cv.sw << ";\n";
            s << "const bool inside = row_ok && r < " << cv.R << "u && hit && ih >= 0 && ih < " << cv.H << " && iw >= 0 && iw < " << cv.W << ";\n"
              << "v[j] = inside ? ld_one(q0 + (((size_t)n * " << cv.H << "u + (u32)ih) * " << cv.W << "u + (u32)iw) * " << cv.C << "u + c) : 0.0f;\n"
              << "if (++c == " << cv.C << "u) { c = 0u; if (++sx == " << cv.S << "u) { sx = 0u; ++r; } }\n}\n"
              << "return pack_chunk(v);\n}\n";
    };
    if (pr.conv_a.on) {
        // The gather of an implicit-GEMM convolution in place of A's loads: one 16-byte chunk is EPC consecutive
        // channels of one filter tap when the channel count allows, EPC separate taps otherwise.
        const auto& cv = pr.conv_a;
        const tp::Arg& img = pr.op_a.args[0];
        s << "#define FETCH_A_ARGS p" << pr.map_a[0] << ", \n#define RAW_A 1\n#define SPLIT_A 1\n";
        emit_conv_tap(cv);
        s << "__device__ __forceinline__ u32x4 fetch_a(const " << tp::c_type(img.dtype) << "* __restrict__ q0, u32 b, u32 row, u32 col) {\n(void)b;\n";
        if (cv.C % epc == 0) {
            s << "u32x4 v = {0u, 0u, 0u, 0u};\nsize_t at;\nif (conv_tap(row, col, at)) v = *(const u32x4*)(q0 + at);\nreturn v;\n}\n";
        } else {
            emit_elementwise_gather(cv);
        }
    } else if (pr.a_km) {
        emit_fetch("a", pr.op_a, pr.root_a, pr.map_a, raw_a, nva, "GK", "GM", pr.M % t.bm == 0 && pr.K % t.bk == 0);
    } else {
        emit_fetch("a", pr.op_a, pr.root_a, pr.map_a, raw_a, nva, "GM", "GK", pr.M % t.bm == 0 && pr.K % t.bk == 0);
    }
    if (pr.conv_b.on) {
        emit_conv_tap(pr.conv_b);
        s << "#define FETCH_B_ARGS p" << pr.map_b[0] << ", \n#define RAW_B 1\n#define SPLIT_B 1\n";
        s << "__device__ __forceinline__ u32x4 fetch_b(const " << tp::c_type(pr.op_b.args[0].dtype) << "* __restrict__ q0, u32 b, u32 row, u32 col) {\n(void)b;\n";
        if (pr.conv_b.C % epc == 0) s << "u32x4 v = {0u, 0u, 0u, 0u};\nsize_t at;\nif (conv_tap(row, col, at)) v = *(const u32x4*)(q0 + at);\nreturn v;\n}\n";
        else emit_elementwise_gather(pr.conv_b);  // the filter gradient of a 3-channel image: B[pixel][(r, s, c)]
    } else if (pr.b_rows.on) {
        const auto& br = pr.b_rows;
        if (br.s_count > 0)
            s << "__device__ __forceinline__ size_t b_row_addr(u32 k) { const u32 rs = k / " << br.group << "u; return (size_t)(k % " << br.group << "u) * "
              << br.o_stride << "ull + " << br.base << "ull + (size_t)(rs / " << br.s_count << "u) * " << br.r_stride << "ull + (size_t)(rs % " << br.s_count
              << "u) * " << br.s_stride << "ull; }\n";
        else
        s << "__device__ __forceinline__ size_t b_row_addr(u32 k) { return (size_t)(k % " << br.group << "u) * " << br.o_stride << "ull + (size_t)(k / "
          << br.group << "u) * " << br.rs_stride << "ull; }\n";
        s << "#define FETCH_B_ARGS p" << pr.map_b[0] << ", \n#define RAW_B 1\n#define SPLIT_B 1\n";
        s << "__device__ __forceinline__ u32x4 fetch_b(const " << tp::c_type(pr.op_b.args[0].dtype) << "* __restrict__ q0, u32 b, u32 row, u32 col) {\n(void)b;\n"
          << "u32x4 v = {0u, 0u, 0u, 0u};\nif (row < GK && col < GN) v = *(const u32x4*)(q0 + b_row_addr(row) + col);\nreturn v;\n}\n";
    } else if (pr.b_nk) emit_fetch("b", pr.op_b, pr.root_b, pr.map_b, raw_b, nvb, "GN", "GK", pr.K % t.bk == 0 && pr.N % t.bn == 0);
    else emit_fetch("b", pr.op_b, pr.root_b, pr.map_b, raw_b, nvb, "GK", "GN", pr.K % t.bk == 0 && pr.N % t.bn == 0);

    // epilogue pieces
    std::ostringstream setup, body, finish, prefetch, early;
    // The tensors an epilogue reads row by row (full-size operands, per-row vectors) are requested EPI_DEPTH steps ahead
    // of the step that uses them, into registers; what does not depend on the row (per-column vectors, constants and
    // what is computed from those alone) is loaded and computed once per wave, ahead of the strips. Left to itself
    // the compiler requests a step's operands inside the step, in two dependent groups, so that a wave's sixteen steps
    // were thirty-two memory round trips one after the other (the 40-op epilogue: 30 us on top of the product). A load
    // left inside the step would also be younger than the requests for the next step, and waiting for it waits for
    // them: hence everything row-varying is requested ahead, and everything else hoisted.
    const std::string raw_members = tp::emit_raw_members(pr.epi, nve, true);
    const int epi_depth = std::max(0, std::min(3, tuning::get_int("HELIUM_HIP_GEMM_EPIPIPE", 1)));
    const bool pipelined = !raw_members.empty() && epi_depth > 0 && pr.split_k == 1;
    // hoisting needs a lane's columns to be the same in every step: steps that cover whole rows of the strip
    bool hoisted = pipelined && colsets == 1 && (64 * nve) % wtn == 0 && !tuning::get("HELIUM_HIP_GEMM_NO_EPI_HOIST");
    for (size_t i = 0; i < pr.epi.exprs.size(); i++) hoisted = hoisted && !tp::is_uniform_pow(pr.epi, (int)i);
    if (pipelined) {
        tp::EmitCtx lx;
        lx.nv = nve;
        lx.phase = 1;
        lx.defer_row_varying_only = true;
        s << "#define EPI_DEPTH " << epi_depth << "\nstruct RawE {\n" << raw_members << "};\n__device__ __forceinline__ void epi_load(";
        for (size_t a = 0; a < pr.epi.args.size(); a++)
            s << (pr.epi.args[a].is_output ? "" : "const ") << tp::c_type(pr.epi.args[a].dtype) << "* __restrict__ a" << a << ", ";
        s << "u32 cB0, u32 m, u32 n0, RawE& R) {\n(void)cB0; (void)m; (void)n0;\n" << tp::emit_exprs(pr.epi, lx) << "}\n";
        std::string pass;
        for (size_t a = 0; a < pr.epi.args.size(); a++) pass += "a" + std::to_string(a) + ", ";
        prefetch << "{ const int q1 = i * EPI_STEPS + step + EPI_DEPTH;\nif (q1 < MB * EPI_STEPS) {\nconst int i1 = q1 / EPI_STEPS, s1 = q1 % EPI_STEPS;\n"
                 << "const u32 idx1 = (s1 * 64 + lane) * NVE;\nconst u32 m1 = m0 + wave_m * WTM + i1 * 32 + idx1 / WTN, nn1 = n0 + wave_n * WTN + idx1 % WTN;\n"
                 << "if (m1 < GM && nn1 < GN) epi_load(" << pass << "bz, m1, nn1, Rb[q1 % (EPI_DEPTH + 1)]);\n} }\n";
    }
    for (size_t a = 0; a < pr.epi.args.size(); a++)
        setup << "auto* a" << a << " = p" << pr.map_e[a] << "; (void)a" << a << ";\n";
    setup << "const u32 cB0 = bz; (void)cB0;\n";
    if (pipelined) {
        std::string pass;
        for (size_t a = 0; a < pr.epi.args.size(); a++) pass += "a" + std::to_string(a) + ", ";
        setup << "RawE Rb[EPI_DEPTH + 1];\n#pragma unroll\nfor (int q1 = 0; q1 < EPI_DEPTH && q1 < MB * EPI_STEPS; q1++) {\nconst int i1 = q1 / EPI_STEPS, s1 = q1 % EPI_STEPS;\n"
              << "const u32 idx1 = (s1 * 64 + lane) * NVE;\nconst u32 m1 = m0 + wave_m * WTM + i1 * 32 + idx1 / WTN, nn1 = n0 + wave_n * WTN + idx1 % WTN;\n"
              << "if (m1 < GM && nn1 < GN) epi_load(" << pass << "bz, m1, nn1, Rb[q1]);\n}\n";
    }
    if (hoisted) {
        // the emitter names the first of a lane's columns `n0`, which is the tile's origin out here
        tp::EmitCtx hx;
        hx.nv = nve;
        hx.row_part = 1;
        std::string text = tp::emit_exprs(pr.epi, hx), renamed;
        for (size_t i = 0; i < text.size();) {
            const bool word_start = i == 0 || !(isalnum((unsigned char)text[i - 1]) || text[i - 1] == '_');
            if (word_start && text.compare(i, 2, "n0") == 0 && (i + 2 == text.size() || !(isalnum((unsigned char)text[i + 2]) || text[i + 2] == '_'))) {
                renamed += "n0_lane";
                i += 2;
            } else {
                renamed += text[i++];
            }
        }
        setup << "const u32 n0_lane = n0 + wave_n * WTN + (lane * NVE) % WTN; const bool col_ok = n0_lane < GN; (void)col_ok;\n" << renamed;
    }
    for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
        const tp::Out& o = pr.epi.outs[oi];
        if (!o.reduce) continue;
        if (o.fold_m && !o.fold_n)
            setup << "float rc" << oi << "[" << colsets << "][NVE];\n#pragma unroll\nfor (int c = 0; c < " << colsets
                  << "; c++)\n#pragma unroll\nfor (int k = 0; k < NVE; k++) rc" << oi << "[c][k] = 0.0f;\n";
        else if (o.fold_m && o.fold_n)
            setup << "float rs" << oi << " = 0.0f;\n";
    }
    {
        // body: runs once per (row, NVE columns) of the strip
        for (size_t oi = 0; oi < pr.epi.outs.size(); oi++)
            if (pr.epi.outs[oi].reduce && pr.epi.outs[oi].fold_n && !pr.epi.outs[oi].fold_m) body << "float rr" << oi << " = 0.0f;\n";
        if (pr.split_k > 1) {
            // the partial tile of this k range, as f32, for the second launch to add up
            body << "if (ok) {\nfloat* dst = splitk_ws + ((size_t)split * GM + m) * GN + nn;\n#pragma unroll\nfor (int k = 0; k < NVE; k++) if (nn + k < GN) dst[k] = acc_v[k];\n}\n";
        } else {
        // `x.pow_scalar(2.0)` reaches the kernel as Pow with a broadcast 1-element operand (the square in BatchNorm2d's
        // statistics). The exponents are read once per workgroup; when all of them are 2 the copy of the body that
        // squares runs, and the general routine stays out of the common case's instruction stream.
        std::vector<int> exps;
        for (size_t i = 0; i < pr.epi.exprs.size(); i++)
            if (tp::is_uniform_pow(pr.epi, (int)i)) exps.push_back(pr.epi.exprs[pr.epi.exprs[i].b].access.arg);
        std::sort(exps.begin(), exps.end());
        exps.erase(std::unique(exps.begin(), exps.end()), exps.end());
        // (read ahead of the k-loop: at the head of the epilogue the load's round trip, a microsecond, would stand between
        // the last k-tile and the first strip of every workgroup)
        if (!exps.empty()) {
            early << "bool all_squares = true;\n";
            for (int a : exps) early << "all_squares = all_squares && ld_one(p" << pr.map_e[a] << ") == 2.0f;\n";
        }
        auto element_body = [&](bool squares) {
            std::ostringstream b;
            tp::EmitCtx cx;
            cx.nv = nve;
            cx.uniform_pow_is_square = squares;
            if (pipelined) {
                cx.phase = 2;
                cx.defer_row_varying_only = true;
                b << "const RawE& R = Rb[(i * EPI_STEPS + step) % (EPI_DEPTH + 1)]; (void)R;\n";
            }
            if (hoisted) cx.row_part = 2;
            // the emitter names the first of the NV columns `n0`; the tile origin of the same name is shadowed here
            b << tp::emit_exprs(pr.epi, cx);
            for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
                const tp::Out& o = pr.epi.outs[oi];
                const std::string v = "e" + std::to_string(o.expr);
                if (!o.reduce) {
                    if (pr.out_rows.on) {
                        const auto& orow = pr.out_rows;
                        b << "{ const u32 on_ = m / " << orow.P * orow.Q << "u, opq = m % " << orow.P * orow.Q << "u, op_ = opq / " << orow.Q << "u, oq = opq % " << orow.Q
                          << "u;\nst_vec<NVE, " << (tp::streams_out(pr.epi.args[o.arg]) ? "true" : "false") << ">(a" << o.arg << " + (((size_t)on_ * " << orow.H << "u + op_ * " << orow.sh << "u + " << orow.a << "u) * " << orow.W << "u + oq * "
                          << orow.sw << "u + " << orow.b << "u) * GN + nn, " << v << "); }\n";
                    } else
                    b << "st_vec<NVE, " << (tp::streams_out(pr.epi.args[o.arg]) ? "true" : "false") << ">(a" << o.arg << " + ((size_t)bz * GM + m) * GN + nn, " << v << ");\n";
                } else if (o.fold_m && !o.fold_n) {
                    b << "#pragma unroll\nfor (int k = 0; k < NVE; k++) rc" << oi << "[step % " << colsets << "][k] += " << v << "[k];\n";
                } else if (o.fold_m && o.fold_n) {
                    b << "#pragma unroll\nfor (int k = 0; k < NVE; k++) rs" << oi << " += " << v << "[k];\n";
                } else {
                    b << "#pragma unroll\nfor (int k = 0; k < NVE; k++) rr" << oi << " += " << v << "[k];\n";
                }
            }
            return b.str();
        };
        body << "if (ok) {\nconst u32 n0 = nn; (void)n0;\nfloat (&acc)[NVE] = acc_v;\n";
        if (exps.empty()) body << element_body(false);
        else body << "if (all_squares) {\n" << element_body(true) << "} else {\n" << element_body(false) << "}\n";
        body << "}\n";
        // per-row sums: combine the lanes that share the row; every wave that holds a piece of the row parks its
        // partial (zero where its columns lie beyond the matrix)
        for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
            const tp::Out& o = pr.epi.outs[oi];
            if (!(o.reduce && o.fold_n && !o.fold_m)) continue;
            const int width = std::min(lanes_per_row, 64);
            const RedOut& ro = red_of(oi);
            body << "{ float r = wave_reduce<0, " << width << ">(rr" << oi << ");\nif ((lane % " << width << ") == 0 && m < GM) red_ws[" << ro.off
                 << "ull + ((size_t)bz * GM + m) * " << ro.parts << "u + tile_n * WAVES_N + wave_n] = r; }\n";
        }
        }
    }
    {
        // Column and scalar sums: the waves of the workgroup meet in LDS (free once every wave has left its strip), so
        // the workgroup parks one partial per column, or one in all, instead of one per wave.
        int ncol = 0, nsc = 0;
        for (auto& o : pr.epi.outs) {
            if (o.reduce && o.fold_m && !o.fold_n) ncol++;
            if (o.reduce && o.fold_m && o.fold_n) nsc++;
        }
        if (ncol + nsc) {
            HE_REQUIRE((size_t)(ncol * t.wm * t.bn + nsc * t.wm * t.wn) * 4 <= (size_t)t.stages * (t.bm + t.bn) * t.bk * esz, HE_ERR_INTERNAL,
                       "reduction exchange exceeds the tile's LDS");
            finish << "__syncthreads();\nfloat* red = (float*)lds;\n";
            int ci = 0, si = 0;
            for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
                const tp::Out& o = pr.epi.outs[oi];
                if (!o.reduce || !o.fold_m) continue;
                if (!o.fold_n) {
                    // lanes that hold the same columns differ by multiples of lanes_per_row
                    finish << "#pragma unroll\nfor (int c = 0; c < " << colsets << "; c++) {\n#pragma unroll\nfor (int k = 0; k < NVE; k++) {\nfloat r = rc"
                           << oi << "[c][k];\n";
                    for (int off = lanes_per_row; off < 64; off *= 2) finish << "r += __shfl_xor(r, " << off << ", 64);\n";
                    finish << "const u32 col = ((c * 64 + lane) * NVE) % WTN + k;\n";
                    finish << "if (lane < " << std::min(lanes_per_row, 64) << ") red[" << ci * t.wm * t.bn << " + wave_m * BN + wave_n * WTN + col] = r;\n}\n}\n";
                    ci++;
                } else {
                    finish << "{ float r = wave_reduce<0, 64>(rs" << oi << ");\nif (lane == 0) red[" << ncol * t.wm * t.bn + si * t.wm * t.wn << " + wave] = r; }\n";
                    si++;
                }
            }
            finish << "__syncthreads();\n";
            ci = si = 0;
            for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
                const tp::Out& o = pr.epi.outs[oi];
                if (!o.reduce || !o.fold_m) continue;
                const RedOut& ro = red_of(oi);
                if (!o.fold_n) {
                    finish << "for (u32 c = tid; c < BN; c += NTHREADS) {\nfloat r = 0.0f;\n#pragma unroll\nfor (int w = 0; w < WAVES_M; w++) r += red["
                           << ci * t.wm * t.bn << " + w * BN + c];\nif (n0 + c < GN) " << (fold_in_kernel ? "HE_WS_STORE(red_ws + " : "red_ws[") << ro.off
                           << "ull + ((size_t)bz * " << ro.parts << "u + tile_m) * GN + n0 + c" << (fold_in_kernel ? ", r);" : "] = r;") << "\n}\n";
                    ci++;
                } else {
                    const int64_t per_b = ro.parts / o.b_div;  // partials per batch index: one per tile
                    finish << "if (tid == 0) {\nfloat r = 0.0f;\n#pragma unroll\nfor (int w = 0; w < WAVES_M * WAVES_N; w++) r += red["
                           << ncol * t.wm * t.bn + si * t.wm * t.wn << " + w];\n" << (fold_in_kernel ? "HE_WS_STORE(red_ws + " : "red_ws[") << ro.off
                           << "ull + (size_t)(bz / " << o.b_div << "u) * " << ro.parts << "u + (size_t)(bz % " << o.b_div << "u) * " << per_b << "u + tile_m * "
                           << tiles_n << "u + tile_n" << (fold_in_kernel ? ", r);" : "] = r;") << "\n}\n";
                    si++;
                }
            }
            if (fold_in_kernel) {
                // every partial of this workgroup has left the CU before its tickets are taken; whoever takes the last
                // ticket of a counter finds all partials in memory, adds them in tile order, and leaves the counter at
                // zero for the next launch
                finish << "HE_WS_DRAIN();\n__syncthreads();\n__shared__ u32 red_last[2];\nif (tid == 0) {\n"
                       << "u32* c0 = red_cnt + (size_t)bz * " << tiles_n << "u + tile_n;\nconst bool l0 = HE_WS_TICKET(c0) == " << tiles_m - 1 << "u;\nif (l0) HE_WS_STORE(c0, 0u);\nred_last[0] = l0;\n";
                if (nsc) {
                    // (scalar outputs of one kernel share b_div: one counter per element group)
                    uint32_t b_div = 1;
                    for (auto& o : pr.epi.outs)
                        if (o.reduce && o.fold_m && o.fold_n) b_div = (uint32_t)o.b_div;
                    finish << "u32* c1 = red_cnt + " << ticket_cols << "ull + bz / " << b_div << "u;\nconst bool l1 = HE_WS_TICKET(c1) == "
                           << (uint64_t)b_div * tiles_m * tiles_n - 1 << "u;\nif (l1) HE_WS_STORE(c1, 0u);\nred_last[1] = l1;\n";
                } else {
                    finish << "red_last[1] = 0u;\n";
                }
                finish << "}\n__syncthreads();\n";
                for (size_t oi = 0; oi < pr.epi.outs.size(); oi++) {
                    const tp::Out& o = pr.epi.outs[oi];
                    if (!o.reduce || !o.fold_m) continue;
                    const RedOut& ro = red_of(oi);
                    char scale[64];
                    snprintf(scale, sizeof scale, "%.9ef", o.rop == tp::ROp::Mean ? (float)o.mean_scale : 1.0f);
                    if (!o.fold_n) {
                        finish << "if (red_last[0]) {\nfor (u32 c = tid; c < BN; c += NTHREADS) {\nif (n0 + c < GN) {\nfloat r = 0.0f;\n#pragma unroll 8\nfor (u32 p = 0; p < "
                               << ro.parts << "u; p++) r += HE_WS_LOAD(red_ws + " << ro.off << "ull + ((size_t)bz * " << ro.parts << "u + p) * GN + n0 + c);\na"
                               << o.arg << "[(size_t)bz * GN + n0 + c] = r * " << scale << ";\n}\n}\n}\n";
                    } else {
                        // one thread per partial (at most 4096), then the waves' sums in order
                        finish << "if (red_last[1]) {\nfloat r = 0.0f;\nfor (u32 p = tid; p < " << ro.parts << "u; p += NTHREADS) r += HE_WS_LOAD(red_ws + " << ro.off
                               << "ull + (size_t)(bz / " << o.b_div << "u) * " << ro.parts << "u + p);\nr = wave_reduce<0, 64>(r);\n__syncthreads();\nif (lane == 0) red[wave] = r;\n__syncthreads();\n"
                               << "if (tid == 0) {\nfloat total = 0.0f;\nfor (int w = 0; w < WAVES_M * WAVES_N; w++) total += red[w];\na" << o.arg << "[bz / " << o.b_div
                               << "u] = total * " << scale << ";\n}\n}\n";
                    }
                }
            }
        }
    }
    // splice the generated pieces into the body
    std::string body_text = kGemmBody;
    auto splice = [&](const std::string& marker, const std::string& text) {
        size_t pos = body_text.find(marker);
        HE_REQUIRE(pos != std::string::npos, HE_ERR_INTERNAL, "kernel template lacks %s", marker.c_str());
        body_text.replace(pos, marker.size(), text);
    };
    {
        // Tile order. Workgroups are dealt round-robin to the 8 XCDs, each with its own L2: when the tile count
        // allows, XCD x takes the x-th eighth of a sequence in which groups of 4 tile rows are walked column by
        // column, so the tiles resident on one XCD form a compact block sharing few A and B panels.
        const int64_t tm = (pr.M + t.bm - 1) / t.bm, tn = (pr.N + t.bn - 1) / t.bn;
        std::ostringstream o;
        const bool xcd = (tm * tn) % 8 == 0 && !tuning::get("HELIUM_HIP_GEMM_NO_XCD");
        o << "{ u32 b = blockIdx.x;\n";
        if (xcd) o << "b = (b % 8u) * " << (tm * tn / 8) << "u + b / 8u;\n";
        const int G = tuning::get("HELIUM_HIP_GEMM_GROUP") ? atoi(tuning::get("HELIUM_HIP_GEMM_GROUP")) : 4;
        o << "const u32 gsize = " << G * tn << "u, group = b / gsize, first = group * " << G << "u;\n";
        o << "const u32 rows = (" << tm << "u - first) < " << G << "u ? (" << tm << "u - first) : " << G << "u;\n";
        o << "tile_m = first + (b % gsize) % rows; tile_n = (b % gsize) / rows; }\n";
        splice("TILE_ORDER", o.str());
        std::ostringstream h;
        if (tuning::get("HELIUM_HIP_GEMM_SCHED")) {
            // ask the scheduler to alternate LDS reads with MFMAs instead of batching either
            h << "_Pragma(\"unroll\") for (int q = 0; q < MB + 2 * NB; q++) { __builtin_amdgcn_sched_group_barrier(0x100, 1, 0); "
                 "__builtin_amdgcn_sched_group_barrier(0x008, 1, 0); }\n";
            h << "__builtin_amdgcn_sched_group_barrier(0x008, MB * NB - (MB + 2 * NB) > 0 ? MB * NB - (MB + 2 * NB) : 0, 0);\n";
        }
        splice("SCHED_HINT", h.str());
        std::ostringstream plan;
        // The instruction-order plan is written for tiles whose operands both arrive by direct loads; with an operand
        // staged through registers the compiler's own order, fenced off from the staging code, measured 1.9x faster.
        const int mode = tuning::get("HELIUM_HIP_GEMM_PLAN") ? atoi(tuning::get("HELIUM_HIP_GEMM_PLAN")) : (direct_a && direct_b) ? 3 : 0;
        const int mb = t.bm / t.wm / 32, nb = t.bn / t.wn / 32, kk_steps = t.bk / (2 * epc);
        const int nr = f32 ? mb + 4 * nb : mb + 2 * nb, nm = f32 ? 4 * mb * nb : mb * nb;
        if (mode == 1) {
            // all operand reads of step kk+1 are issued ahead of the MFMAs of step kk
            plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << nr << ", 0);\n";
            for (int kk = 0; kk < kk_steps; kk++) {
                if (kk + 1 < kk_steps) plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << nr << ", 0);\n";
                plan << "__builtin_amdgcn_sched_group_barrier(0x008, " << nm << ", 0);\n";
            }
        } else if (mode == 3 || mode == 4) {
            // Rotated tile: direct loads, the first k-step's reads, the MFMAs left over from the previous tile, then
            // per k-step the next step's reads between the first MFMAs (two per MFMA in mode 3, all before the
            // second MFMA in mode 4) so that they have landed when the step ends: while direct loads are in flight
            // the compiler can only wait for *all* outstanding LDS reads at once.
            const int waves = threads / 64;
            const int dl = ((direct_a ? t.bm * t.bk * esz / 1024 : 0) + (direct_b ? t.bk * t.bn * esz / 1024 : 0)) / waves;
            const int per = issue_front ? dl : (dl + kk_steps - 1) / kk_steps;
            const int rate = mode == 3 ? 2 : nr;
            for (int g = 0; g < kk_steps; g++) {
                int issue = std::max(0, std::min(per, dl - g * per));
                if (g == 0) {
                    plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << nr << ", 0);\n";
                    int done = 0;
                    for (int m = 0; m < nm; m++) {  // direct loads spread evenly between the carried MFMAs
                        const int upto = issue * (m + 1) / nm;
                        if (upto > done) plan << "__builtin_amdgcn_sched_group_barrier(0x020, " << (upto - done) << ", 0);\n";
                        done = upto;
                        plan << "__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);\n";
                    }
                } else if (issue) {
                    plan << "__builtin_amdgcn_sched_group_barrier(0x020, " << issue << ", 0);\n";
                }
                if (g + 1 == kk_steps) break;
                // MFMAs of step g with the reads of step g + 1
                int left = nr;
                for (int m = 0; m < nm; m++) {
                    plan << "__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);\n";
                    const int r = std::min(left, rate);
                    if (r) plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << r << ", 0);\n";
                    left -= r;
                }
            }
        } else if (mode == 2) {
            // reads of step kk+1 are spread between the MFMAs of step kk
            plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << nr << ", 0);\n";
            const int waves = threads / 64;
            const int dl = ((direct_a ? t.bm * t.bk * esz / 1024 : 0) + (direct_b ? t.bk * t.bn * esz / 1024 : 0)) / waves;
            const int per = issue_front ? dl : (dl + kk_steps - 1) / kk_steps;
            for (int kk = 0; kk < kk_steps; kk++) {
                int issue = std::max(0, std::min(per, dl - kk * per));
                if (issue) plan << "__builtin_amdgcn_sched_group_barrier(0x020, " << issue << ", 0);\n";
                int reads = kk + 1 < kk_steps ? nr : 0, done_r = 0;
                for (int m = 0; m < nm; m++) {
                    int want_r = reads * (m + 1) / nm;
                    if (want_r > done_r) plan << "__builtin_amdgcn_sched_group_barrier(0x100, " << (want_r - done_r) << ", 0);\n";
                    done_r = want_r;
                    plan << "__builtin_amdgcn_sched_group_barrier(0x008, 1, 0);\n";
                }
            }
        }
        splice("SCHED_PLAN", plan.str());
    }
    splice("EPILOGUE_SETUP", setup.str());
    splice("EPILOGUE_PREFETCH", prefetch.str());
    splice("EPILOGUE_BODY", body.str());
    splice("EPILOGUE_FINISH", finish.str());
    splice("EPILOGUE_EARLY", early.str());
    s << body_text;
    if (pr.split_k > 1) {
        // second launch of a split-k product: the output element is the sum of its partials, rounded once
        HE_REQUIRE(pr.batch == 1 && pr.epi.outs.size() == 1 && !pr.epi.outs[0].reduce && pr.epi.exprs.size() == 1, HE_ERR_UNSUPPORTED,
                   "split-k needs an unbatched product with a plain epilogue");
        const tp::Out& o = pr.epi.outs[0];
        // 32 consecutive output elements per workgroup. With 16 partial tiles or more and an element count that is a
        // multiple of 4: 8 threads take 4 elements
        // each (one 16-byte load per partial tile), 32 such groups share the partials (group q adds partials q, q + 32,
        // ...), then one thread per element adds the 32 sums in order. Otherwise 8 threads per element, one element each.
        if ((pr.M * pr.N) % 4 == 0 && pr.split_k >= 16)
            s << "extern \"C\" __global__ __launch_bounds__(256) void fused_matmul_finalize(const float* __restrict__ ws, " << tp::c_type(o.dtype)
              << "* __restrict__ out) {\n__shared__ float part[1024];\nconst size_t total = (size_t)GM * GN;\nconst u32 e4 = threadIdx.x % 8u, pg = threadIdx.x / 8u;\n"
              << "const size_t i = (size_t)blockIdx.x * 32 + e4 * 4u;\nf32x4 acc = {0.0f, 0.0f, 0.0f, 0.0f};\nif (i < total) {\n#pragma unroll 4\nfor (u32 sp = pg; sp < " << pr.split_k
              << "u; sp += 32u) acc += *(const f32x4*)(ws + (size_t)sp * total + i);\n}\n#pragma unroll\nfor (int k = 0; k < 4; k++) part[pg * 32u + e4 * 4u + k] = acc[k];\n__syncthreads();\n"
              << "const size_t j = (size_t)blockIdx.x * 32 + threadIdx.x;\nif (threadIdx.x < 32u && j < total) {\nfloat r = 0.0f;\n#pragma unroll\nfor (int q = 0; q < 32; q++) r += part[q * 32 + threadIdx.x];\n"
              << "float one[1] = {r};\nst_vec<1>(out + j, one);\n}\n}\n";
        else
            s << "extern \"C\" __global__ __launch_bounds__(256) void fused_matmul_finalize(const float* __restrict__ ws, " << tp::c_type(o.dtype)
              << "* __restrict__ out) {\n__shared__ float part[256];\nconst size_t total = (size_t)GM * GN;\nconst u32 e = threadIdx.x % 32u, pg = threadIdx.x / 32u;\n"
              << "const size_t i = (size_t)blockIdx.x * 32 + e;\nfloat acc = 0.0f;\nif (i < total) {\n#pragma unroll 4\nfor (u32 sp = pg; sp < " << pr.split_k
              << "u; sp += 8u) acc += ws[(size_t)sp * total + i];\n}\npart[pg * 32u + e] = acc;\n__syncthreads();\n"
              << "if (pg == 0 && i < total) {\nfloat r = 0.0f;\n#pragma unroll\nfor (int q = 0; q < 8; q++) r += part[q * 32 + e];\nfloat one[1] = {r};\nst_vec<1>(out + i, one);\n}\n}\n";
    }
    if (!reds.empty() && !fold_in_kernel) {
        // Second launch: one workgroup folds EB output elements, PG = 256 / EB threads share the partials of each
        // (thread q takes partials q, q + PG, ...), then one thread adds the PG sums in order: the same order every run.
        s << "template <int EB, bool CONTIG>\n__device__ __forceinline__ void fold_partials(const float* __restrict__ ws, float* __restrict__ out, u32 n, u32 parts, "
             "u32 inner, float scale, u32 blk, float* part) {\n"
             "constexpr int PG = 256 / EB;\nconst u32 tid = threadIdx.x;\n"
             "const u32 e = CONTIG ? tid / PG : tid % EB, pg = CONTIG ? tid % PG : tid / EB;\nconst u32 j = blk * EB + e;\nfloat acc = 0.0f;\n"
             "if (j < n) {\nconst float* src = ws + (size_t)(j / inner) * parts * inner + (j % inner);\n#pragma unroll 8\n"
             "for (u32 p = pg; p < parts; p += PG) acc += src[(size_t)p * inner];\n}\n"
             "part[e * PG + pg] = acc;\n__syncthreads();\n"
             "if (pg == 0 && j < n) {\nfloat r = 0.0f;\nfor (int q = 0; q < PG; q++) r += part[e * PG + q];\nout[j] = r * scale;\n}\n}\n";
        // The column sums that a carried program reads (tp::Program::post: the per-channel arithmetic behind a batch norm's
        // statistics) are folded by the same blocks, EB columns each, and the threads that end up with a column's sums
        // evaluate the program for that column. The kernel then takes every argument of the epilogue program.
        std::vector<size_t> carried;  // indices into reds
        if (pr.epi.post) {
            std::vector<char> read(pr.epi.args.size(), 0);
            for (const tp::Expr& e : pr.epi.post->exprs)
                if (e.kind == tp::Expr::Load) read[e.access.arg] = 1;
            for (size_t i = 0; i < reds.size(); i++) {
                const tp::Out& o = pr.epi.outs[reds[i].out];
                if (!read[o.arg]) continue;
                HE_REQUIRE(o.fold_m && !o.fold_n && pr.batch == 1, HE_ERR_INTERNAL, "a carried program reads column sums of an unbatched product");
                carried.push_back(i);
            }
            HE_REQUIRE(!carried.empty(), HE_ERR_INTERNAL, "the carried program reads no reduction of this product");
            reduce_all_args_ = true;
        }
        s << "extern \"C\" __global__ __launch_bounds__(256) void fused_matmul_reduce(const float* __restrict__ ws";
        if (reduce_all_args_) {
            for (size_t a = 0; a < pr.epi.args.size(); a++)
                s << ", " << (pr.epi.args[a].is_output ? "" : "const ") << tp::c_type(pr.epi.args[a].dtype) << "* __restrict__ a" << a;
        } else {
            for (size_t i = 0; i < reds.size(); i++) s << ", float* __restrict__ o" << i;
        }
        s << ") {\n__shared__ float part[256];\nu32 blk = blockIdx.x;\n";
        if (!carried.empty()) {
            const RedOut& r0 = reds[carried[0]];
            int eb = 16;
            while (eb > 1 && (r0.elems < eb || (r0.elems / eb < 64 && r0.parts > 256 / eb))) eb /= 2;
            const int pg = 256 / eb;
            const uint32_t blocks = (uint32_t)((r0.elems + eb - 1) / eb);
            s << "if (blk < " << blocks << "u) {\nconst u32 tid = threadIdx.x, e = tid % " << eb << "u, pg = tid / " << eb << "u, j = blk * " << eb << "u + e;\n";
            std::map<int, std::string> values;
            for (size_t i : carried) s << "float red" << i << " = 0.0f, acc" << i << " = 0.0f;\n";
            s << "if (j < " << r0.elems << "u) {\n#pragma unroll 8\nfor (u32 p = pg; p < " << r0.parts << "u; p += " << pg << "u) {\n";
            for (size_t i : carried) s << "acc" << i << " += ws[" << reds[i].off << "ull + (size_t)p * " << reds[i].inner << "u + j];\n";
            s << "}\n}\n";
            for (size_t i : carried) {
                const tp::Out& o = pr.epi.outs[reds[i].out];
                char scale[64];
                snprintf(scale, sizeof scale, "%.9ef", o.rop == tp::ROp::Mean ? (float)o.mean_scale : 1.0f);
                s << "__syncthreads();\npart[pg * " << eb << "u + e] = acc" << i << ";\n__syncthreads();\nif (pg == 0 && j < " << r0.elems << "u) {\nfloat r = 0.0f;\nfor (int q = 0; q < "
                  << pg << "; q++) r += part[q * " << eb << " + e];\nred" << i << " = store_and_keep(a" << o.arg << " + j, r * " << scale << ");\n}\n";
                values[o.arg] = "red" + std::to_string(i);
            }
            tp::EmitCtx cx;
            cx.nv = 1;
            cx.arg_values = &values;
            s << "if (pg == 0 && j < " << r0.elems << "u) {\nconst u32 n0 = j, m = 0u; (void)m;\n" << tp::emit_exprs(*pr.epi.post, cx);
            for (const tp::Out& o : pr.epi.post->outs) s << "st_one(a" << o.arg << " + n0, e" << o.expr << "[0]);\n";
            s << "}\nreturn;\n}\nblk -= " << blocks << "u;\n";
            reduce_grid_ += blocks;
        }
        for (size_t i = 0; i < reds.size(); i++) {
            if (std::find(carried.begin(), carried.end(), i) != carried.end()) continue;
            const RedOut& r = reds[i];
            const tp::Out& o = pr.epi.outs[r.out];
            // elements per workgroup: 16 where there are many elements with few partials each, fewer (more threads per
            // element, more workgroups) where a few elements have thousands of partials
            int eb = 16;
            while (eb > 1 && (r.elems < eb || (r.elems / eb < 64 && r.parts > 256 / eb))) eb /= 2;
            const uint32_t blocks = (uint32_t)((r.elems + eb - 1) / eb);
            char scale[64];
            snprintf(scale, sizeof scale, "%.9ef", o.rop == tp::ROp::Mean ? (float)o.mean_scale : 1.0f);
            s << "if (blk < " << blocks << "u) { fold_partials<" << eb << ", " << (r.inner == 1 ? "true" : "false") << ">(ws + " << r.off << "ull, " << (reduce_all_args_ ? "(float*)a" + std::to_string(o.arg) : "o" + std::to_string(i)) << ", "
              << r.elems << "u, " << r.parts << "u, " << r.inner << "u, " << scale << ", blk, part); return; }\nblk -= " << blocks << "u;\n";
            reduce_grid_ += blocks;
        }
        s << "}\n";
    }
    source_ = s.str();

    const int64_t tiles = ((pr.M + t.bm - 1) / t.bm) * ((pr.N + t.bn - 1) / t.bn);
    HE_REQUIRE(tiles < (1ll << 31) && pr.batch < 65536, HE_ERR_INVALID, "GEMM grid too large");
    grid_[0] = (uint32_t)tiles;
    grid_[1] = (uint32_t)(pr.split_k > 1 ? pr.split_k : pr.batch);
    threads_ = (uint32_t)threads;
    for (auto& r : reds) reduce_outs_.push_back(pr.map_e[pr.epi.outs[r.out].arg]);
    reduce_floats_ = red_floats;
    std::string reduce_args;
    for (int a : reduce_all_args_ ? pr.map_e : reduce_outs_) reduce_args += (reduce_args.empty() ? "" : ",") + std::to_string(a);
    describe_ = strfmt("gemm [%lld,%lld,%lld]x[%lld] tile=%dx%dx%d stages=%d waves=%dx%d threads=%d grid=%ux%u rawA=%d rawB=%d NVA=%d NVB=%d NVE=%d "
                       "direct=%d%d mma=%s epilogue_exprs=%zu outs=%zu split_k=%d reduce_ws=%llu reduce_grid=%u reduce_args=[%s] reduce_counters=%llu",
                       (long long)pr.batch, (long long)pr.M, (long long)pr.K, (long long)pr.N, t.bm, t.bn, t.bk, t.stages, t.wm, t.wn, threads,
                       grid_[0], grid_[1], (int)raw_a, (int)raw_b, nva, nvb, nve, (int)direct_a, (int)direct_b, dtype_name(pr.mma_dtype), pr.epi.exprs.size(),
                       pr.epi.outs.size(), pr.split_k, (unsigned long long)reduce_floats_, reduce_grid_, reduce_args.c_str(), (unsigned long long)reduce_counters_);
    kernel_.reset(new JitKernel(source_, "fused_matmul", {"-ffp-contract=fast", "-munsafe-fp-atomics"}));
    if (pr.split_k > 1) finalize_.reset(new JitKernel(source_, "fused_matmul_finalize", {"-ffp-contract=fast", "-munsafe-fp-atomics"}));
    if (pr.epi.post) describe_ += strfmt(" carries=%zuexprs/%zuouts", pr.epi.post->exprs.size(), pr.epi.post->outs.size());
    // (a carried program is a pointwise instruction's: no contraction into fused multiply-adds, as when it runs alone)
    if (reduce_grid_) reduce_.reset(new JitKernel(source_, "fused_matmul_reduce", {reduce_all_args_ ? "-ffp-contract=off" : "-ffp-contract=fast"}));
}

GemmKernel::~GemmKernel() { scratch_.release(); }

static uint64_t counters_offset(uint64_t n_floats) { return (n_floats * 4 + 255) & ~255ull; }  // as ReduceScratch lays them out

size_t GemmKernel::scratch_bytes_needed() const {
    if (prob_.split_k > 1) return (size_t)prob_.split_k * prob_.M * prob_.N * 4;
    if (reduce_counters_) return (size_t)(counters_offset(reduce_floats_) + reduce_counters_ * 4);
    return (size_t)reduce_floats_ * 4;
}

void GemmKernel::load() {
    kernel_->load();
    if (finalize_) finalize_->load();
    if (reduce_) reduce_->load();
    if (reduce_counters_) load_fill_kernel();  // execute_in_scratch clears the arrival counters with it
}

bool GemmKernel::loaded() const {
    return kernel_->loaded() && (!finalize_ || finalize_->loaded()) && (!reduce_ || reduce_->loaded()) &&
           (!reduce_counters_ || fill_kernel_loaded());
}

void GemmKernel::execute(void* const* ptrs, hipStream_t stream) {
    ReduceScratch::Buf ws{nullptr, nullptr};
    if (reduce_counters_) ws = scratch_.get(reduce_floats_, reduce_counters_, stream);  // (counters start at zero and are left there)
    else if (const size_t need = scratch_bytes_needed()) ws = scratch_.get(need / 4, 0, stream);
    run(ptrs, stream, ws.floats, reduce_counters_ ? ws.counters : nullptr);
}

void GemmKernel::execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) {
    HE_REQUIRE(loaded(), HE_ERR_INVALID, "the kernel's code objects are not loaded on this device yet");
    const size_t need = scratch_bytes_needed();
    HE_REQUIRE(need <= scratch_bytes, HE_ERR_INVALID,
               "the kernel needs %zu bytes of scratch for its partial results, the buffer holds %zu", need, scratch_bytes);
    HE_REQUIRE(!need || (scratch && ((uintptr_t)scratch & 255) == 0), HE_ERR_INVALID, "scratch buffer missing or not 256-byte aligned");
    // every partial that is read is written by the same call first: only arrival counters have to be cleared (the buffer
    // is shared with whatever ran before)
    uint32_t* counters = nullptr;
    if (reduce_counters_) {
        counters = (uint32_t*)((char*)scratch + counters_offset(reduce_floats_));
        fill_buffers({{counters, {(uint32_t)reduce_counters_, 0u}}}, stream);
    }
    run(ptrs, stream, need ? (float*)scratch : nullptr, counters);
}

void GemmKernel::run(void* const* ptrs, hipStream_t stream, float* ws, uint32_t* counters) {
    const size_t nargs = prob_.args.size();
    for (size_t i = 0; i < nargs; i++) {
        HE_REQUIRE(ptrs[i] != nullptr, HE_ERR_INVALID, "kernel argument %zu is null", i);
        HE_REQUIRE(((uintptr_t)ptrs[i] & 15) == 0, HE_ERR_INVALID, "kernel argument %zu is not 16-byte aligned", i);
    }
    std::vector<void*> holders(ptrs, ptrs + nargs);
    if (ws) holders.push_back(ws);
    if (counters) holders.push_back(counters);
    std::vector<void*> argv(holders.size());
    for (size_t i = 0; i < holders.size(); i++) argv[i] = &holders[i];
    const uint32_t block[3] = {threads_, 1, 1};
    kernel_->launch(grid_, block, 0, stream, argv.data(), !finalize_ && !reduce_);
    if (finalize_) {
        void* out = ptrs[prob_.map_e[prob_.epi.outs[0].arg]];
        void* fargv[] = {&ws, &out};
        const uint64_t total = (uint64_t)prob_.M * prob_.N;
        const uint32_t fgrid[3] = {(uint32_t)((total + 31) / 32), 1, 1}, fblock[3] = {256, 1, 1};
        finalize_->launch(fgrid, fblock, 0, stream, fargv, !reduce_);
    }
    if (reduce_) {
        std::vector<void*> rh{ws};
        if (reduce_all_args_)
            for (int a : prob_.map_e) rh.push_back(ptrs[a]);
        else
            for (int a : reduce_outs_) rh.push_back(ptrs[a]);
        std::vector<void*> rargv(rh.size());
        for (size_t i = 0; i < rh.size(); i++) rargv[i] = &rh[i];
        const uint32_t rgrid[3] = {reduce_grid_, 1, 1}, rblock[3] = {256, 1, 1};
        reduce_->launch(rgrid, rblock, 0, stream, rargv.data(), true);
    }
}

CompositeKernel::CompositeKernel(std::vector<std::unique_ptr<KernelBase>> parts, bool zero_outputs_first)
    : parts_(std::move(parts)), zero_first_(zero_outputs_first) {
    HE_REQUIRE(!parts_.empty(), HE_ERR_INTERNAL, "a composite kernel needs a part");
    for (auto& p : parts_) {
        HE_REQUIRE(p->args().size() == parts_[0]->args().size(), HE_ERR_INTERNAL, "the parts of a composite kernel take different arguments");
        // (sources and descriptions one after the other, each introduced by a line that names the part)
        source_ += "// ---- part " + std::to_string(&p - &parts_[0]) + " of " + std::to_string(parts_.size()) + "\n" + p->source() + "\n";
        describe_ += (describe_.empty() ? "" : "\n") + p->describe();
    }
    describe_ = "composite parts=" + std::to_string(parts_.size()) + " zero_first=" + (zero_first_ ? "1" : "0") + "\n" + describe_;
}

void CompositeKernel::zero_outputs(void* const* ptrs, hipStream_t stream) const {
    std::vector<std::pair<void*, std::pair<uint32_t, uint32_t>>> fills;
    const auto& a = args();
    for (size_t i = 0; i < a.size(); i++)
        // (whole words, rounded up: an odd count of 16-bit elements ends in half a word, and blocks are 256-byte granules)
        if (a[i].is_output) fills.push_back({ptrs[i], {(uint32_t)((storage_bytes(a[i].dtype, (size_t)a[i].numel) + 3) / 4), 0u}});
    if (!fills.empty()) fill_buffers(fills, stream);
}

// Only the last part's last launch closes the instruction: an event that is pending for it is held back until then.
namespace {
struct HeldStopEvent {
    hipEvent_t e = take_pending_stop_event();
    void give_back() {
        if (e) set_pending_stop_event(e);
        e = nullptr;
    }
    ~HeldStopEvent() { give_back(); }
};
}  // namespace

void CompositeKernel::execute(void* const* ptrs, hipStream_t stream) {
    HeldStopEvent held;
    if (zero_first_) zero_outputs(ptrs, stream);
    for (auto& p : parts_) {
        if (&p == &parts_.back()) held.give_back();
        p->execute(ptrs, stream);
    }
}

void CompositeKernel::execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) {
    HeldStopEvent held;
    if (zero_first_) zero_outputs(ptrs, stream);
    for (auto& p : parts_) {
        if (&p == &parts_.back()) held.give_back();
        p->execute_in_scratch(ptrs, stream, scratch, scratch_bytes);  // (one after the other: they may share it)
    }
}

size_t CompositeKernel::scratch_bytes_needed() const {
    size_t need = 0;
    for (auto& p : parts_) need = std::max(need, p->scratch_bytes_needed());
    return need;
}

void CompositeKernel::load() {
    for (auto& p : parts_) p->load();
    if (zero_first_) load_fill_kernel();
}

bool CompositeKernel::loaded() const {
    for (auto& p : parts_)
        if (!p->loaded()) return false;
    return !zero_first_ || fill_kernel_loaded();
}

// ---------------------------------------------------------------------------------------------------------
// Convolutions over a repacked few-channel image
// ---------------------------------------------------------------------------------------------------------
RepackedConvKernel::RepackedConvKernel(std::vector<tp::Arg> args, ConvRepack geometry, std::unique_ptr<KernelBase> inner)
    : args_(std::move(args)), geo_(geometry), inner_(std::move(inner)) {
    const ConvRepack& c = geo_;
    HE_REQUIRE(inner_->args().size() == args_.size(), HE_ERR_INTERNAL, "the product over repacked operands takes other arguments");
    HE_REQUIRE(c.C >= 1 && c.C <= 4 && c.image_arg >= 0 && c.filter_arg >= 0, HE_ERR_INTERNAL, "bad repacking geometry");
    const uint64_t pixels = (uint64_t)c.N * c.Hp * c.Wp, taps = (uint64_t)c.O * c.R * c.Sp;
    HE_REQUIRE(pixels + taps < (1ull << 31), HE_ERR_UNSUPPORTED, "image too large to repack");
    image_bytes_ = (size_t)((pixels * 8 + 255) & ~255ull);
    filter_bytes_ = (size_t)((taps * (c.filter_gradient ? 4 * c.elem_bytes : 8) + 255) & ~255ull);
    std::ostringstream s;
    s << "// repacks a " << c.C << "-channel 16-bit image [" << c.N << "," << c.H << "," << c.W << "," << c.C << "] as [" << c.N << "," << c.Hp << "," << c.Wp
      << ",4] with the padding (" << c.ph << "," << c.pw << ") written out" << (c.filter_gradient ? "" : ", and the filter alike") << "\n"
      << "typedef unsigned short u16;\ntypedef unsigned int u32;\ntypedef unsigned long long u64;\n"
      << "#define PIXELS " << pixels << "u\n#define TAPS " << taps << "u\n";
    // one thread per pixel of the copy: up to 4 two-byte loads, one 8-byte store
    s << "static __device__ __forceinline__ u64 pixel_of(const u16* __restrict__ src) {\nu64 v = 0;\n";
    for (int ch = 0; ch < c.C; ch++) s << "v |= (u64)src[" << ch << "] << " << 16 * ch << ";\n";
    s << "return v;\n}\n";
    s << "extern \"C\" __global__ __launch_bounds__(256) void repack_conv_operands(const u16* __restrict__ image, "
      << (c.filter_gradient ? "" : "const u16* __restrict__ filter, ") << "u64* __restrict__ image_p" << (c.filter_gradient ? "" : ", u64* __restrict__ filter_p") << ") {\n"
      << "u32 t = blockIdx.x * 256u + threadIdx.x;\n"
      << "if (t < PIXELS) {\n"
      << "u32 w = t % " << c.Wp << "u, rest = t / " << c.Wp << "u, h = rest % " << c.Hp << "u, n = rest / " << c.Hp << "u;\n"
      << "int hs = (int)h - " << c.ph << ", ws = (int)w - " << c.pw << ";\n"
      << "u64 v = 0;\n"
      << "if (hs >= 0 && hs < " << c.H << " && ws >= 0 && ws < " << c.W << ") v = pixel_of(image + ((u64)(n * " << c.H << "u + (u32)hs) * " << c.W << "u + (u32)ws) * " << c.C << "u);\n"
      << "image_p[t] = v;\nreturn;\n}\n";
    if (!c.filter_gradient)
        s << "t -= PIXELS;\nif (t < TAPS) {\n"
          << "u32 sp = t % " << c.Sp << "u, row = t / " << c.Sp << "u;\n"  // row = o * R + r
          << "u64 v = 0;\nif (sp < " << c.S << "u) v = pixel_of(filter + ((u64)row * " << c.S << "u + sp) * " << c.C << "u);\n"
          << "filter_p[t] = v;\n}\n";
    s << "}\n";
    pack_grid_ = (uint32_t)((pixels + (c.filter_gradient ? 0 : taps) + 255) / 256);
    if (c.filter_gradient) {
        const uint64_t elems = (uint64_t)c.O * c.R * c.S * c.C;
        const char* et = c.elem_bytes == 4 ? "u32" : "u16";
        s << "extern \"C\" __global__ __launch_bounds__(256) void unpack_filter_gradient(const " << et << "* __restrict__ packed, " << et << "* __restrict__ out) {\n"
          << "u32 t = blockIdx.x * 256u + threadIdx.x;\nif (t >= " << elems << "u) return;\n"
          << "u32 ch = t % " << c.C << "u, rest = t / " << c.C << "u, sx = rest % " << c.S << "u, row = rest / " << c.S << "u;\n"
          << "out[t] = packed[((u64)row * " << c.Sp << "u + sx) * 4u + ch];\n}\n";
        unpack_grid_ = (uint32_t)((elems + 255) / 256);
    }
    pack_source_ = s.str();
    source_ = "// ---- repack\n" + pack_source_ + "// ---- product\n" + inner_->source();
    describe_ = strfmt("repacked image_arg=%d filter_arg=%d filter_gradient=%d image=[%lld,%lld,%lld,%lld] packed=[%lld,%lld,%lld,4] pad=[%lld,%lld] filter=[%lld,%lld,%lld->%lld] "
                       "pack_grid=%u unpack_grid=%u image_bytes=%zu filter_bytes=%zu\n",
                       c.image_arg, c.filter_arg, (int)c.filter_gradient, (long long)c.N, (long long)c.H, (long long)c.W, (long long)c.C, (long long)c.N,
                       (long long)c.Hp, (long long)c.Wp, (long long)c.ph, (long long)c.pw, (long long)c.O, (long long)c.R, (long long)c.S, (long long)c.Sp, pack_grid_,
                       unpack_grid_, image_bytes_, filter_bytes_) +
                inner_->describe();
    pack_.reset(new JitKernel(pack_source_, "repack_conv_operands"));
    if (c.filter_gradient) unpack_.reset(new JitKernel(pack_source_, "unpack_filter_gradient"));
}

RepackedConvKernel::~RepackedConvKernel() { scratch_.release(); }

size_t RepackedConvKernel::scratch_bytes_needed() const { return own_bytes() + inner_->scratch_bytes_needed(); }

void RepackedConvKernel::load() {
    pack_->load();
    if (unpack_) unpack_->load();
    inner_->load();
}

bool RepackedConvKernel::loaded() const { return pack_->loaded() && (!unpack_ || unpack_->loaded()) && inner_->loaded(); }

void RepackedConvKernel::execute(void* const* ptrs, hipStream_t stream) {
    run(ptrs, stream, (char*)scratch_.get(own_bytes() / 4, 0, stream).floats, nullptr, 0);
}

void RepackedConvKernel::execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) {
    HE_REQUIRE(loaded(), HE_ERR_INVALID, "the kernel's code objects are not loaded on this device yet");
    HE_REQUIRE(scratch_bytes_needed() <= scratch_bytes, HE_ERR_INVALID,
               "the kernel needs %zu bytes of scratch for its repacked operands and partial results, the buffer holds %zu", scratch_bytes_needed(), scratch_bytes);
    HE_REQUIRE(scratch && ((uintptr_t)scratch & 255) == 0, HE_ERR_INVALID, "scratch buffer missing or not 256-byte aligned");
    run(ptrs, stream, (char*)scratch, (char*)scratch + own_bytes(), scratch_bytes - own_bytes());
}

void RepackedConvKernel::run(void* const* ptrs, hipStream_t stream, char* own, void* inner_scratch, size_t inner_scratch_bytes) {
    for (size_t i = 0; i < args_.size(); i++) HE_REQUIRE(ptrs[i] != nullptr, HE_ERR_INVALID, "kernel argument %zu is null", i);
    void* image = ptrs[geo_.image_arg];
    void* filter = ptrs[geo_.filter_arg];
    void* image_p = own;
    void* filter_p = own + image_bytes_;
    const uint32_t block[3] = {256, 1, 1};
    {
        void* fwd[] = {&image, &filter, &image_p, &filter_p};
        void* grad[] = {&image, &image_p};
        const uint32_t grid[3] = {pack_grid_, 1, 1};
        pack_->launch(grid, block, 0, stream, geo_.filter_gradient ? grad : fwd, false);
    }
    std::vector<void*> inner_ptrs(ptrs, ptrs + args_.size());
    inner_ptrs[geo_.image_arg] = image_p;
    inner_ptrs[geo_.filter_arg] = filter_p;
    // (a forward convolution's last launch is the product's: it closes the instruction; a filter gradient's is the unpacking)
    HeldStopEvent held;
    if (!geo_.filter_gradient) held.give_back();
    if (inner_scratch) inner_->execute_in_scratch(inner_ptrs.data(), stream, inner_scratch, inner_scratch_bytes);
    else inner_->execute(inner_ptrs.data(), stream);
    if (geo_.filter_gradient) {
        held.give_back();
        void* argv[] = {&filter_p, &filter};
        const uint32_t grid[3] = {unpack_grid_, 1, 1};
        unpack_->launch(grid, block, 0, stream, argv, true);
    }
}

}  // namespace he
