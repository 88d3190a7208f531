#include "permute.h"

#include <algorithm>
#include <cstdlib>
#include <numeric>
#include <sstream>

namespace he {

std::vector<int> perm_from_swaps(int rank, const std::vector<std::pair<int, int>>& swaps) {
    // out.shape[i] = in.shape[perm[i]]; every SwapDims exchanges two positions of the current view.
    std::vector<int> perm(rank);
    std::iota(perm.begin(), perm.end(), 0);
    for (auto& s : swaps) {
        HE_REQUIRE(s.first >= 0 && s.first < rank && s.second >= 0 && s.second < rank, HE_ERR_INVALID,
                   "swap axis out of range");
        std::swap(perm[s.first], perm[s.second]);
    }
    return perm;
}

static int pow2_floor(int64_t x) {
    int p = 1;
    while ((int64_t)p * 2 <= x) p *= 2;
    return p;
}
static int pow2_ceil(int64_t x) {
    int p = 1;
    while (p < x) p *= 2;
    return p;
}
static int env_int(const char* name, int dflt) {
    const char* v = tuning::get(name);
    return v ? atoi(v) : dflt;
}

PermutePlan plan_permute(const std::vector<int64_t>& shape, const std::vector<int>& perm, int elem_bytes) {
    const int rank = (int)shape.size();
    HE_REQUIRE(rank >= 1 && rank <= 12, HE_ERR_INVALID, "permute rank %d not in 1..12", rank);
    HE_REQUIRE((int)perm.size() == rank, HE_ERR_INVALID, "perm has %zu entries for rank %d", perm.size(), rank);
    HE_REQUIRE(elem_bytes == 2 || elem_bytes == 4, HE_ERR_INVALID, "permute supports 16- and 32-bit elements");
    std::vector<char> seen(rank, 0);
    for (int p : perm) {
        HE_REQUIRE(p >= 0 && p < rank && !seen[p], HE_ERR_INVALID, "perm is not a permutation");
        seen[p] = 1;
    }
    PermutePlan plan;
    plan.elem_bytes = elem_bytes;
    plan.numel = 1;
    for (int64_t d : shape) {
        HE_REQUIRE(d >= 0, HE_ERR_INVALID, "negative extent");
        plan.numel *= d;
    }

    // 1. Drop extent-1 dims and renumber the rest.
    std::vector<int> relabel(rank, -1);
    std::vector<int64_t> kept;
    for (int i = 0; i < rank; i++)
        if (shape[i] != 1) {
            relabel[i] = (int)kept.size();
            kept.push_back(shape[i]);
        }
    std::vector<int> out_seq;
    for (int i = 0; i < rank; i++)
        if (relabel[perm[i]] >= 0) out_seq.push_back(relabel[perm[i]]);

    // 2. Merge runs of dims that are adjacent and in the same order on both sides.
    struct Group {
        int first_in;
        int64_t extent;
    };
    std::vector<Group> groups;  // in output order
    for (size_t i = 0; i < out_seq.size(); i++) {
        if (i > 0 && out_seq[i] == out_seq[i - 1] + 1)
            groups.back().extent *= kept[out_seq[i]];
        else
            groups.push_back({out_seq[i], kept[out_seq[i]]});
    }
    if (groups.empty()) groups.push_back({0, plan.numel == 0 ? 0 : 1});
    const int n = (int)groups.size();
    std::vector<int> by_in(n);
    std::iota(by_in.begin(), by_in.end(), 0);
    std::sort(by_in.begin(), by_in.end(), [&](int x, int y) { return groups[x].first_in < groups[y].first_in; });
    std::vector<int> in_index_of_group(n);
    for (int k = 0; k < n; k++) in_index_of_group[by_in[k]] = k;
    plan.dims.resize(n);
    for (int k = 0; k < n; k++) plan.dims[k] = groups[by_in[k]].extent;
    plan.out_order.resize(n);
    for (int g = 0; g < n; g++) plan.out_order[g] = in_index_of_group[g];
    plan.in_stride.assign(n, 1);
    for (int k = n - 2; k >= 0; k--) plan.in_stride[k] = plan.in_stride[k + 1] * plan.dims[k + 1];
    plan.out_stride.assign(n, 1);
    {
        int64_t s = 1;
        for (int g = n - 1; g >= 0; g--) {
            plan.out_stride[plan.out_order[g]] = s;
            s *= plan.dims[plan.out_order[g]];
        }
    }
    plan.ax_a = n - 1;
    plan.ax_b = plan.out_order[n - 1];

    const int vmax = 16 / elem_bytes;
    auto vec_for = [&](int64_t extent) {
        int v = vmax;
        while (v > 1 && extent % v != 0) v /= 2;
        return v;
    };
    plan.threads = 256;

    if (plan.ax_a == plan.ax_b) {
        // Innermost dim untouched: whole rows move. n == 1 is a plain copy.
        plan.variant = (n == 1) ? PermutePlan::Copy : PermutePlan::Rows;
        plan.va = plan.vb = vec_for(plan.dims[plan.ax_a]);
        plan.unroll = 4;
        int64_t vecs = plan.numel / plan.va;
        int64_t per_block = (int64_t)plan.threads * plan.unroll;
        int64_t grid = (vecs + per_block - 1) / per_block;
        HE_REQUIRE(grid < (1ll << 31), HE_ERR_INVALID, "tensor too large for permute grid");
        plan.grid = (uint32_t)std::max<int64_t>(grid, 1);
        plan.lds_bytes = 0;
        return plan;
    }

    plan.variant = PermutePlan::Tile;
    const int64_t da = plan.dims[plan.ax_a], db = plan.dims[plan.ax_b];
    plan.va = vec_for(da);
    plan.vb = vec_for(db);
    // 64x64 tiles; rows of the input that are at least 4 KB long take 128-element (256-byte) load segments, which
    // measured 17% faster on the 4096^2 transpose and slower on short-row shapes.
    const int ta_default = da * elem_bytes >= 4096 && db >= 64 ? 128 : 64;
    int ta = env_int("HELIUM_HIP_PERMUTE_TA", ta_default), tb = env_int("HELIUM_HIP_PERMUTE_TB", 64);
    const int area = ta * tb;
    const int min_ta = std::max(16 / elem_bytes, plan.va);  // a row of the tile is at least one 16-byte chunk
    // Shrink a tile side that overhangs a short dim and give the area to the other side.
    ta = std::max(min_ta, std::min(ta, pow2_ceil(da)));
    tb = std::max(plan.vb, std::min(area / ta, pow2_ceil(db)));
    tb = std::min(tb, 256);
    ta = std::max(min_ta, std::min({area / tb, pow2_ceil(da), 256}));
    HE_REQUIRE((ta & (ta - 1)) == 0 && (tb & (tb - 1)) == 0, HE_ERR_INVALID, "tile extents must be powers of two");
    (void)pow2_floor;
    plan.ta = ta;
    plan.tb = tb;
    plan.lds_bytes = (uint32_t)(ta * tb * elem_bytes);
    int64_t nta = (da + ta - 1) / ta, ntb = (db + tb - 1) / tb;
    int64_t rest = 1;
    for (int k = 0; k < n; k++)
        if (k != plan.ax_a && k != plan.ax_b) rest *= plan.dims[k];
    int64_t grid = nta * ntb * rest;
    HE_REQUIRE(grid < (1ll << 31), HE_ERR_INVALID, "tensor too large for permute grid");
    plan.grid = (uint32_t)std::max<int64_t>(grid, 1);
    return plan;
}

// ---------------------------------------------------------------------------------------------------------
// Kernel text. The problem constants are #defines placed in front of one of two fixed bodies.
// ---------------------------------------------------------------------------------------------------------

static const char* kPrelude = R"HIP(
typedef unsigned short u16;
typedef unsigned int u32;
typedef unsigned long long u64;
typedef u32 u32x2 __attribute__((ext_vector_type(2)));
typedef u32 u32x4 __attribute__((ext_vector_type(4)));
template <int B> struct VT;
template <> struct VT<2> { typedef u16 T; };
template <> struct VT<4> { typedef u32 T; };
template <> struct VT<8> { typedef u32x2 T; };
template <> struct VT<16> { typedef u32x4 T; };
)HIP";

// Tile variant. A is the input's contiguous axis, B the output's. One block moves a TB x TA tile:
//   phase 1: 16-byte (VA-element) loads along A, coalesced, written to LDS rows of TA elements;
//   phase 2: each lane gathers VB elements along B from LDS and issues one 16-byte store along B.
// LDS rows are split in 16-byte chunks and the chunk index is XORed with (b / VB), so the column gathers of
// phase 2 spread over all banks while the 16-byte row writes of phase 1 stay aligned.
static const char* kTileBody = R"HIP(
#define RP (TA * ELEM)            /* bytes per LDS row */
#define NCH (RP / 16)             /* 16-byte chunks per row */
#define LB (VA * ELEM)            /* bytes per global load */
#define SB (VB * ELEM)            /* bytes per global store */

__device__ __forceinline__ u32 lds_off(u32 b, u32 a) {
    u32 byte = a * ELEM;
    return b * RP + ((((byte >> 4) ^ (b / VB)) & (NCH - 1)) << 4) + (byte & 15);
}

extern "C" __global__ __launch_bounds__(NT) void permute_dims(const unsigned char* __restrict__ in,
                                                              unsigned char* __restrict__ out) {
    __shared__ __attribute__((aligned(16))) unsigned char lds[TB * RP];
    u32 t = blockIdx.x;
    XCD_ORDER
    TILE_DECOMP
    u64 base_in = 0, base_out = 0;
    REST_DECOMP
    const u32 a0 = ta_i * TA, b0 = tb_i * TB;
    base_in += (u64)b0 * ISB + a0;
    base_out += (u64)a0 * OSA + b0;
    const unsigned char* src = in + base_in * ELEM;
    unsigned char* dst = out + base_out * ELEM;

    typedef typename VT<LB>::T LT;
    constexpr u32 LV = TA / VA;  // load vectors per tile row
#pragma unroll
    for (u32 v = threadIdx.x; v < TB * LV; v += NT) {
        u32 b = v / LV, a = (v % LV) * VA;
        if (a0 + a < DA && b0 + b < DB) {
            LT val = LOAD_VEC((const LT*)(src + ((u64)b * ISB + a) * ELEM));
            *(LT*)(lds + lds_off(b, a)) = val;
        }
    }
    __syncthreads();

    typedef typename VT<SB>::T ST;
    constexpr u32 SV = TB / VB;  // store vectors per output row of the tile
#if ELEM == 2 && VB >= 2
    // Two output rows (a, a+1) per item: each LDS read fetches the 32-bit word holding both.
    for (u32 v = threadIdx.x; v < (TA / 2) * SV; v += NT) {
        u32 cb = v % SV, a = (v / SV) * 2, b = cb * VB;
        u32 w[VB];
#pragma unroll
        for (u32 i = 0; i < VB; i++) w[i] = *(const u32*)(lds + lds_off(b + i, a));
        __attribute__((aligned(16))) u32 lo[VB / 2], hi[VB / 2];
#pragma unroll
        for (u32 j = 0; j < VB / 2; j++) {
            lo[j] = (w[2 * j] & 0xffffu) | (w[2 * j + 1] << 16);
            hi[j] = (w[2 * j] >> 16) | (w[2 * j + 1] & 0xffff0000u);
        }
        if (b0 + b < DB) {
            if (a0 + a < DA)
                __builtin_nontemporal_store(*(const ST*)lo, (ST*)(dst + ((u64)a * OSA + b) * ELEM));
            if (a0 + a + 1 < DA)
                __builtin_nontemporal_store(*(const ST*)hi, (ST*)(dst + ((u64)(a + 1) * OSA + b) * ELEM));
        }
    }
#else
    typedef typename VT<ELEM>::T ET;
    for (u32 v = threadIdx.x; v < TA * SV; v += NT) {
        u32 cb = v % SV, a = v / SV, b = cb * VB;
        __attribute__((aligned(16))) ET e[VB];
#pragma unroll
        for (u32 i = 0; i < VB; i++) e[i] = *(const ET*)(lds + lds_off(b + i, a));
        if (a0 + a < DA && b0 + b < DB)
            __builtin_nontemporal_store(*(const ST*)e, (ST*)(dst + ((u64)a * OSA + b) * ELEM));
    }
#endif
}
)HIP";

// Rows variant: the innermost dim keeps its place, so whole rows of DA elements move; one lane moves
// UNROLL vectors of V elements, consecutive lanes take consecutive output vectors.
static const char* kRowsBody = R"HIP(
#define VBYTES (V * ELEM)
extern "C" __global__ __launch_bounds__(NT) void permute_dims(const unsigned char* __restrict__ in,
                                                              unsigned char* __restrict__ out) {
    typedef typename VT<VBYTES>::T T;
    constexpr u64 RV = DA / V;  // vectors per row
    u64 first = ((u64)blockIdx.x * UNROLL) * NT + threadIdx.x;
    T vals[UNROLL];
    u64 oidx[UNROLL];
#pragma unroll
    for (int u = 0; u < UNROLL; u++) {
        u64 ov = first + (u64)u * NT;
        oidx[u] = ov;
        if (ov < NVEC) {
            u64 row = ov / RV;
            u64 cv = ov - row * RV;
            u64 in_off = cv * V;
            ROW_DECOMP
            vals[u] = __builtin_nontemporal_load((const T*)(in + in_off * ELEM));
        }
    }
#pragma unroll
    for (int u = 0; u < UNROLL; u++)
        if (oidx[u] < NVEC) __builtin_nontemporal_store(vals[u], (T*)(out + oidx[u] * VBYTES));
}
)HIP";

std::string emit_permute_source(const PermutePlan& p) {
    std::ostringstream s;
    s << "// permute_dims: generated for gfx950\n";
    s << kPrelude;
    s << "#define ELEM " << p.elem_bytes << "\n#define NT " << p.threads << "\n";
    const int n = (int)p.dims.size();
    if (p.variant == PermutePlan::Tile) {
        const int64_t da = p.dims[p.ax_a], db = p.dims[p.ax_b];
        const int64_t nta = (da + p.ta - 1) / p.ta, ntb = (db + p.tb - 1) / p.tb;
        s << "#define VA " << p.va << "\n#define VB " << p.vb << "\n#define TA " << p.ta << "\n#define TB "
          << p.tb << "\n";
        s << "#define DA " << da << "u\n#define DB " << db << "u\n";
        s << "#define ISB " << p.in_stride[p.ax_b] << "ull\n#define OSA " << p.out_stride[p.ax_a] << "ull\n";
        // Consecutive blocks walk the B tiles first: neighbouring blocks then write neighbouring segments of
        // the same output rows.
        // Workgroups are dealt round-robin to the 8 XCDs, each with its own L2. When the tile segments of an input row
        // do not start on cache-line boundaries (a row pitch that is no multiple of 128 bytes), neighbouring tiles
        // share lines: XCD x then takes the x-th eighth of the tile sequence, so that the tiles which share a line
        // meet in one L2 instead of fetching it once per XCD, and the loads are ordinary ones that leave the line
        // there ([32,128,28,28] -> (0,2,3,1): 11.2 MB fetched for 6.4 MB of input before).
        const bool shared_lines = (p.in_stride[p.ax_b] * p.elem_bytes) % 128 != 0 || (p.ta * p.elem_bytes) % 128 != 0;
        const bool xcd = env_int("HELIUM_HIP_PERMUTE_XCD", shared_lines ? 1 : 0) != 0 && p.grid >= 16;
        const bool nt = env_int("HELIUM_HIP_PERMUTE_NT", shared_lines ? 0 : 1) != 0;
        s << "#define LOAD_VEC(p) " << (nt ? "__builtin_nontemporal_load(p)" : "(*(p))") << "\n";
        if (xcd) {
            const uint32_t q = p.grid / 8, r = p.grid % 8;
            s << "#define XCD_ORDER { const u32 x = t % 8u; t = x * " << q << "u + (x < " << r << "u ? x : " << r << "u) + t / 8u; }\n";
        } else {
            s << "#define XCD_ORDER\n";
        }
        s << "#define TILE_DECOMP u32 tb_i = t % " << ntb << "u; t /= " << ntb << "u; u32 ta_i = t % " << nta
          << "u; t /= " << nta << "u;\n";
        s << "#define REST_DECOMP";
        for (int g = n - 1; g >= 0; g--) {
            int k = p.out_order[g];
            if (k == p.ax_a || k == p.ax_b) continue;
            s << " { u32 c = t % " << p.dims[k] << "u; t /= " << p.dims[k] << "u; base_in += (u64)c * "
              << p.in_stride[k] << "ull; base_out += (u64)c * " << p.out_stride[k] << "ull; }";
        }
        s << "\n" << kTileBody;
    } else {
        const int64_t da = p.dims[p.ax_a];
        s << "#define V " << p.va << "\n#define UNROLL " << p.unroll << "\n#define DA " << da << "ull\n";
        s << "#define NVEC " << (p.numel / p.va) << "ull\n";
        s << "#define ROW_DECOMP";
        for (int g = n - 2; g >= 0; g--) {  // output dims above the row, fastest first
            int k = p.out_order[g];
            s << " { u64 c = row % " << p.dims[k] << "ull; row /= " << p.dims[k] << "ull; in_off += c * "
              << p.in_stride[k] << "ull; }";
        }
        s << "\n" << kRowsBody;
    }
    return s.str();
}

Permute::Permute(const std::vector<int64_t>& shape, const std::vector<int>& perm, int dtype) {
    HE_REQUIRE(dtype == HE_F16 || dtype == HE_BF16 || dtype == HE_F32 || dtype == HE_U32, HE_ERR_INVALID,
               "permute does not take dtype %s", dtype_name(dtype));
    plan_ = plan_permute(shape, perm, (int)dtype_bits(dtype) / 8);
    kernel_.reset(new JitKernel(emit_permute_source(plan_), "permute_dims"));
    const char* vname = plan_.variant == PermutePlan::Tile ? "tile" : plan_.variant == PermutePlan::Rows ? "rows" : "copy";
    std::string dims;
    for (size_t i = 0; i < plan_.dims.size(); i++) dims += (i ? "x" : "") + std::to_string(plan_.dims[i]);
    desc_ = strfmt("variant=%s elem=%dB collapsed=[%s] axA=%d axB=%d VA=%d VB=%d TA=%d TB=%d grid=%u threads=%d lds=%uB",
                   vname, plan_.elem_bytes, dims.c_str(), plan_.ax_a, plan_.ax_b, plan_.va, plan_.vb, plan_.ta,
                   plan_.tb, plan_.grid, plan_.threads, plan_.lds_bytes);
}

void Permute::execute(const void* in, void* out, hipStream_t stream) {
    if (plan_.numel == 0) return;
    HE_REQUIRE(in && out, HE_ERR_INVALID, "null tensor pointer");
    const uintptr_t amask = (uintptr_t)(std::max(plan_.va, plan_.vb) * plan_.elem_bytes - 1);
    HE_REQUIRE((((uintptr_t)in | (uintptr_t)out) & amask) == 0, HE_ERR_INVALID,
               "permute operands must be aligned to %d bytes", (int)amask + 1);
    const uint32_t grid[3] = {plan_.grid, 1, 1}, block[3] = {(uint32_t)plan_.threads, 1, 1};
    void* args[] = {(void*)&in, (void*)&out};
    kernel_->launch(grid, block, 0, stream, args, true);
}

}  // namespace he

// ---- C ABI ------------------------------------------------------------------------------------------------
struct he_permute_s {
    he::Permute impl;
    he_permute_s(const std::vector<int64_t>& s, const std::vector<int>& p, int dt) : impl(s, p, dt) {}
};

extern "C" {

int he_permute_create(he_permute_t* permute, const int64_t* shape, const int32_t* perm, int rank, int dtype) {
    return he::guard([&] {
        HE_REQUIRE(permute && shape && perm && rank >= 1, HE_ERR_INVALID, "bad argument");
        *permute = new he_permute_s(std::vector<int64_t>(shape, shape + rank), std::vector<int>(perm, perm + rank),
                                    dtype);
    });
}

int he_permute_create_from_swaps(he_permute_t* permute, const int64_t* shape, int rank, const int32_t* swaps,
                                 int num_swaps, int dtype) {
    return he::guard([&] {
        HE_REQUIRE(permute && shape && rank >= 1 && (swaps || num_swaps == 0), HE_ERR_INVALID, "bad argument");
        std::vector<std::pair<int, int>> sw;
        for (int i = 0; i < num_swaps; i++) sw.emplace_back(swaps[2 * i], swaps[2 * i + 1]);
        *permute = new he_permute_s(std::vector<int64_t>(shape, shape + rank), he::perm_from_swaps(rank, sw), dtype);
    });
}

int he_permute_destroy(he_permute_t permute) {
    delete permute;
    return HE_OK;
}

int he_permute_execute(he_permute_t permute, const void* in, void* out, he_stream_t stream) {
    return he::guard([&] {
        HE_REQUIRE(permute, HE_ERR_INVALID, "null permute");
        permute->impl.execute(in, out, stream ? stream->s : nullptr);
    });
}

const char* he_permute_source(he_permute_t permute) { return permute ? permute->impl.source().c_str() : ""; }
const char* he_permute_describe(he_permute_t permute) { return permute ? permute->impl.describe().c_str() : ""; }

int he_permute_reference_output_strides(const int64_t* shape, int rank, const int32_t* swaps, int num_swaps,
                                        int64_t* strides_out) {
    return he::guard([&] {
        HE_REQUIRE(shape && strides_out && rank >= 1, HE_ERR_INVALID, "bad argument");
        std::vector<int> permutation(rank);
        std::iota(permutation.begin(), permutation.end(), 0);
        for (int i = 0; i < num_swaps; i++) std::swap(permutation[swaps[2 * i]], permutation[swaps[2 * i + 1]]);
        int64_t stride = 1;
        for (int i = rank - 1; i >= 0; i--) {
            int j = (int)(std::find(permutation.begin(), permutation.end(), i) - permutation.begin());
            strides_out[j] = stride;
            stride *= shape[j];
        }
    });
}

}  // extern "C"
