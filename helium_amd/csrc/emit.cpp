// HIP source emission for tile programs: the shared expression emitter and the pointwise/reduction kernel.
#include <algorithm>
#include <cmath>
#include <cstring>
#include <sstream>

#include "tp.h"

namespace he::tp {

const char* c_type(int dtype) {
    switch (dtype) {
        case HE_F16: return "f16_t";
        case HE_BF16: return "bf16_t";
        case HE_F32: return "float";
        case HE_U32: return "u32";
        case HE_BOOL: return "u32";
    }
    return "?";
}

static const char* cls_type(Cls c) { return c == Cls::F ? "float" : c == Cls::I ? "u32" : "bool"; }

// Types, vector loads/stores with conversion, wave/block reductions, float atomics.
static const char* kPrelude = R"HIP(
typedef unsigned short u16;
typedef unsigned int u32;
typedef unsigned long long u64;
typedef __bf16 bf16_t;
typedef _Float16 f16_t;
#ifndef HE_OPAQUE
// Hides where a value came from. Negating a just-widened bf16 and narrowing it again makes this compiler (with
// packed FP32 off) build an integer xor it then cannot select; the barrier keeps the three steps apart.
__device__ __forceinline__ float he_opaque(float x) { asm volatile("" : "+v"(x)); return x; }
#define HE_OPAQUE(x) he_opaque(x)
#endif
#ifndef HE_FAST_RCP
#define HE_FAST_RCP(x) __builtin_amdgcn_rcpf(x)
#endif
#ifndef HE_WS_STORE
// Cross-block exchange through scratch memory. Device-scope atomic accesses go past the per-XCD L2 caches, so a
// partial result written this way and waited for (HE_WS_DRAIN: all of the wave's memory operations have completed)
// before the block takes its ticket is in memory by the time any other block can see that ticket. A device-scope
// fence would give the same guarantee by writing back and invalidating the whole L2, once per wave.
#define HE_WS_STORE(p, v) __hip_atomic_store((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define HE_WS_LOAD(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define HE_WS_TICKET(p) __hip_atomic_fetch_add((p), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define HE_WS_DRAIN() __builtin_amdgcn_s_waitcnt(0)
#endif
template <class T, int N> struct Vec { typedef T type __attribute__((ext_vector_type(N))); };
template <class T> struct Vec<T, 1> { typedef T type; };

template <int NV> __device__ __forceinline__ void ld_vec(const float* p, float (&e)[NV]) {
    typedef typename Vec<float, NV>::type V;
    V v = *(const V*)p;
    if constexpr (NV == 1) e[0] = v; else
#pragma unroll
    for (int k = 0; k < NV; k++) e[k] = v[k];
}
template <int NV> __device__ __forceinline__ void ld_vec(const u32* p, u32 (&e)[NV]) {
    typedef typename Vec<u32, NV>::type V;
    V v = *(const V*)p;
    if constexpr (NV == 1) e[0] = v; else
#pragma unroll
    for (int k = 0; k < NV; k++) e[k] = v[k];
}
template <int NV> __device__ __forceinline__ void ld_vec(const bf16_t* p, float (&e)[NV]) {
    typedef typename Vec<u16, NV>::type V;
    V v = *(const V*)p;
    if constexpr (NV == 1) e[0] = __builtin_bit_cast(float, (u32)v << 16); else
#pragma unroll
    for (int k = 0; k < NV; k++) e[k] = __builtin_bit_cast(float, (u32)v[k] << 16);
}
template <int NV> __device__ __forceinline__ void ld_vec(const f16_t* p, float (&e)[NV]) {
    typedef typename Vec<f16_t, NV>::type V;
    V v = *(const V*)p;
    if constexpr (NV == 1) e[0] = (float)v; else
#pragma unroll
    for (int k = 0; k < NV; k++) e[k] = (float)v[k];
}
__device__ __forceinline__ float ld_one(const float* p) { return *p; }
__device__ __forceinline__ u32 ld_one(const u32* p) { return *p; }
__device__ __forceinline__ float ld_one(const bf16_t* p) { return __builtin_bit_cast(float, (u32)(*(const u16*)p) << 16); }
__device__ __forceinline__ float ld_one(const f16_t* p) { return (float)*p; }

// STREAM: the store bypasses the caches' write allocation (a large output that nobody reads back before it has left L2
// anyway: with plain stores the 32 MB output of a 4096^2 product cost 5 us more, and up to 26 us when the launch had
// streamed its operands through L2 just before)
template <int NV, bool STREAM = false> __device__ __forceinline__ void st_vec(float* p, const float (&e)[NV]) {
    typedef typename Vec<float, NV>::type V;
    V v;
    if constexpr (NV == 1) v = e[0]; else
#pragma unroll
    for (int k = 0; k < NV; k++) v[k] = e[k];
    if constexpr (STREAM) __builtin_nontemporal_store(v, (V*)p); else *(V*)p = v;
}
template <int NV, bool STREAM = false> __device__ __forceinline__ void st_vec(u32* p, const u32 (&e)[NV]) {
    typedef typename Vec<u32, NV>::type V;
    V v;
    if constexpr (NV == 1) v = e[0]; else
#pragma unroll
    for (int k = 0; k < NV; k++) v[k] = e[k];
    if constexpr (STREAM) __builtin_nontemporal_store(v, (V*)p); else *(V*)p = v;
}
template <int NV, bool STREAM = false> __device__ __forceinline__ void st_vec(bf16_t* p, const float (&e)[NV]) {
    typedef typename Vec<bf16_t, NV>::type V;
    V v;
    if constexpr (NV == 1) v = (bf16_t)e[0]; else
#pragma unroll
    for (int k = 0; k < NV; k++) v[k] = (bf16_t)e[k];   // round to nearest even
    if constexpr (STREAM) __builtin_nontemporal_store(v, (V*)p); else *(V*)p = v;
}
template <int NV, bool STREAM = false> __device__ __forceinline__ void st_vec(f16_t* p, const float (&e)[NV]) {
    typedef typename Vec<f16_t, NV>::type V;
    V v;
    if constexpr (NV == 1) v = (f16_t)e[0]; else
#pragma unroll
    for (int k = 0; k < NV; k++) v[k] = (f16_t)e[k];
    if constexpr (STREAM) __builtin_nontemporal_store(v, (V*)p); else *(V*)p = v;
}
__device__ __forceinline__ void st_one(float* p, float v) { *p = v; }
__device__ __forceinline__ void st_one(u32* p, u32 v) { *p = v; }
__device__ __forceinline__ void st_one(bf16_t* p, float v) { *p = (bf16_t)v; }
__device__ __forceinline__ void st_one(f16_t* p, float v) { *p = (f16_t)v; }
// stores v and returns what a load of that element would give back (the value rounded to the element type)
template <class T> __device__ __forceinline__ float store_and_keep(T* p, float v) {
    T t;
    st_one(&t, v);
    st_one(p, v);
    return ld_one((const T*)&t);
}

// Reduction operators: 0 Sum, 1 Mean (terms are pre-scaled), 2 Max, 3 Min.
template <int OP> __device__ __forceinline__ float red_op(float a, float b) {
    if constexpr (OP == 2) return fmaxf(a, b);
    else if constexpr (OP == 3) return fminf(a, b);
    else return a + b;
}
template <int OP> __device__ __forceinline__ float red_identity() {
    if constexpr (OP == 2) return -__builtin_huge_valf();
    else if constexpr (OP == 3) return __builtin_huge_valf();
    else return 0.0f;
}
// Butterfly over the `WIDTH` consecutive lanes a value's group occupies (WIDTH a power of two <= 64).
template <int OP, int WIDTH> __device__ __forceinline__ float wave_reduce(float v) {
#pragma unroll
    for (int off = WIDTH / 2; off > 0; off /= 2) v = red_op<OP>(v, __shfl_xor(v, off, 64));
    return v;
}
template <int OP> __device__ __forceinline__ void atomic_red(float* addr, float v) {
    if constexpr (OP == 2) {
        // float max through integer atomics, split by sign (helium/src/cuda/instr/pointwise/jit.rs:40-56)
        if (v >= 0) atomicMax((int*)addr, __float_as_int(v)); else atomicMin((unsigned int*)addr, __float_as_uint(v));
    } else if constexpr (OP == 3) {
        if (v >= 0) atomicMin((int*)addr, __float_as_int(v)); else atomicMax((unsigned int*)addr, __float_as_uint(v));
    } else {
        atomicAdd(addr, v);
    }
}
// tanh to within 2 ulp without branches (lanes of a wave rarely agree on which side of a branch they are):
// x + x^3 P(x^2) below 1, 1 - 2 / (exp(2|x|) + 1) from there on; measured against double tanh over every float in
// (0, 10] with exp off by one ulp either way the worst error is 1.21 ulp.
__device__ __forceinline__ float tanh_2ulp(float x) {
    const float ax = __builtin_fabsf(x);
    const float u = ax * ax;
    float p = __builtin_fmaf(u, -0.0003552270936779678f, 0.002289985306560993f);
    p = __builtin_fmaf(u, p, -0.007930326275527477f);
    p = __builtin_fmaf(u, p, 0.021475814282894135f);
    p = __builtin_fmaf(u, p, -0.05387599393725395f);
    p = __builtin_fmaf(u, p, 0.1333228200674057f);
    p = __builtin_fmaf(u, p, -0.33333292603492737f);
    const float small = __builtin_fmaf(ax * u, p, ax);
    const float d = expf(2.0f * ax) + 1.0f;            // +inf for large |x|: the quotient is 0 and tanh is 1
    float r = HE_FAST_RCP(d);
    r = __builtin_isinf(d) ? 0.0f : __builtin_fmaf(__builtin_fmaf(-d, r, 1.0f), r, r);  // one Newton step
    const float big = __builtin_fmaf(-2.0f, r, 1.0f);
    const float t = ax < 1.0f ? small : big;           // NaN falls through to `big`, which is NaN
    return __builtin_copysignf(t, x);
}
// a / b as a * rcp(b): about 1 ulp, one quarter-rate instruction instead of the ten of an IEEE division
__device__ __forceinline__ float fast_div(float a, float b) { return a * HE_FAST_RCP(b); }
// powf, one copy per kernel: inlined at every use (a kernel of per-channel arithmetic has twenty, each in the interior
// and the ragged form of the loop body) the routine makes a kernel of a few hundred elements spend its time fetching
// code. Squares and first powers (`x.pow_scalar(2.0)`) skip the general routine when every lane of the wave has one.
__device__ __attribute__((noinline)) float he_powf(float x, float y) {
    if (y == 2.0f) return x * x;
    if (y == 1.0f) return x;
    return powf(x, y);
}
// powf whose exponent is one value for the whole launch (a broadcast 1-element operand): the tests are the same in
// every lane.
__device__ __forceinline__ float pow_uniform(float x, float y) {
    if (y == 2.0f) return x * x;
    if (y == 1.0f) return x;
    return he_powf(x, y);
}
__device__ __forceinline__ float fast_tanh(float x) {
    float t = __expf(2.0f * x);
    return 1.0f - fast_div(2.0f, t + 1.0f);
}
)HIP";

std::string emit_prelude(const Program&) { return kPrelude; }

static std::string f32_literal(uint32_t bits) {
    // Bit-exact constants, as the reference prints them (jit.rs:697-702).
    return strfmt("__builtin_bit_cast(float, 0x%08xu)", bits);
}

static std::string unary_expr(const Expr& e, const std::string& x, bool fast) {
    float cf;
    memcpy(&cf, &e.bits, 4);
    std::string c = f32_literal(e.bits);
    switch ((UOp)e.op) {
        case UOp::Recip: return fast ? "HE_FAST_RCP(" + x + ")" : "1.0f / " + x;
        case UOp::Neg: return "-HE_OPAQUE(" + x + ")";
        case UOp::Exp: return (fast ? "__expf(" : "expf(") + x + ")";
        case UOp::Sin: return (fast ? "__sinf(" : "sinf(") + x + ")";
        case UOp::Cos: return (fast ? "__cosf(" : "cosf(") + x + ")";
        case UOp::Tan: return (fast ? "__tanf(" : "tanf(") + x + ")";
        case UOp::Sigmoid:
            return fast ? "HE_FAST_RCP(1.0f + __expf(-" + x + "))" : "1.0f / (1.0f + expf(-" + x + "))";
        case UOp::Tanh: return (fast ? "fast_tanh(" : "tanh_2ulp(") + x + ")";
        case UOp::Relu: return "fmaxf(" + x + ", 0.0f)";
        case UOp::Sqrt: return (fast ? "__fsqrt_rn(" : "sqrtf(") + x + ")";
        case UOp::Log: return (fast ? "__logf(" : "logf(") + x + ")";
        case UOp::Gelu: return "0.5f * " + x + " * (1.0f + erff(" + x + " * 0.70710678118654752f))";
        case UOp::AddC: return x + " + " + c;
        case UOp::MulC: return x + " * " + c;
        case UOp::PowC:
            // x*x for an exponent of exactly 2, as the reference's generator special-cases
            // (helium-playground/src/kernel_generator.rs:383-391); x**c otherwise (torch_synthesizer.rs:55).
            if (cf == 2.0f) return x + " * " + x;
            return "he_powf(" + x + ", " + c + ")";
    }
    fail(HE_ERR_INTERNAL, "bad unary op");
}

static std::string binary_expr(const Expr& e, Cls cls, const std::string& a, const std::string& b, bool fast) {
    switch ((BOp)e.op) {
        case BOp::Add: return cls == Cls::B ? a + " != " + b : a + " + " + b;
        case BOp::Sub: return a + " - " + b;
        case BOp::Mul: return cls == Cls::B ? a + " && " + b : a + " * " + b;
        case BOp::Div: return fast ? "fast_div(" + a + ", " + b + ")" : a + " / " + b;
        case BOp::Pow: return "he_powf(" + a + ", " + b + ")";
        case BOp::Min: return cls == Cls::F ? "fminf(" + a + ", " + b + ")" : "(" + a + " < " + b + " ? " + a + " : " + b + ")";
        case BOp::Max: return cls == Cls::F ? "fmaxf(" + a + ", " + b + ")" : "(" + a + " > " + b + " ? " + a + " : " + b + ")";
        case BOp::And: return cls == Cls::B ? a + " && " + b : a + " & " + b;
        case BOp::Or: return cls == Cls::B ? a + " || " + b : a + " | " + b;
        case BOp::Xor: return cls == Cls::B ? a + " != " + b : a + " ^ " + b;
        case BOp::Drelu: return "(" + b + " > 0.0f) ? " + a + " : 0.0f";
    }
    fail(HE_ERR_INTERNAL, "bad binary op");
}

static const char* compare_sym(int op) {
    static const char* s[] = {"==", "!=", "<", "<=", ">", ">="};
    HE_REQUIRE(op >= 0 && op < 6, HE_ERR_INVALID, "bad compare op");
    return s[op];
}

// One generic index map applied to the u32 variable `lin` (jit.rs:807-906).
static void emit_generic_map(std::ostringstream& s, const GenericMap& g) {
    if (g.kind == GenericMap::Swap) {
        Shape out = g.in_shape;
        std::swap(out[g.axis_a], out[g.axis_b]);
        const int n = (int)out.size();
        s << "{ u32 in_index = 0;";
        int64_t ostride = 1;
        for (int i = n - 1; i >= 0; i--) {
            s << " u32 c" << i << " = (lin / " << ostride << "u) % " << out[i] << "u;";
            ostride *= out[i];
        }
        int64_t istride = 1;
        for (int j = n - 1; j >= 0; j--) {
            int k = j == g.axis_a ? (int)g.axis_b : j == g.axis_b ? (int)g.axis_a : j;
            s << " in_index += c" << k << " * " << istride << "u;";
            istride *= g.in_shape[j];
        }
        s << " lin = in_index; }";
    } else {
        const int n = (int)g.out_shape.size(), r = (int)g.in_shape.size();
        s << "{ u32 in_index = 0;";
        int64_t ostride = 1, istride = 1;
        for (int i = 0; i < n; i++) {  // i counts dims from the last
            int od = n - 1 - i, id = r - 1 - i;
            s << " u32 co" << i << " = (lin / " << ostride << "u) % " << g.out_shape[od] << "u;";
            ostride *= g.out_shape[od];
            bool zero = id < 0 || g.bcast[od];
            if (!zero) s << " in_index += co" << i << " * " << istride << "u;";
            istride *= id >= 0 ? g.in_shape[id] : 1;
        }
        s << " lin = in_index; }";
    }
}

bool streams_out(const Arg& a) {
    if (tuning::get("HELIUM_HIP_NO_STREAM_STORES")) return false;
    return a.is_output && storage_bytes(a.dtype, (size_t)a.numel) >= (size_t(4) << 20);
}

int pick_nv(const Program& p, int max_bytes) {
    const int n = (int)p.dims.size();
    const int64_t N = p.N();
    int widest = 1;  // bytes of the widest element moved along full rows
    auto consider = [&](int dtype) {
        if (dtype != HE_BOOL) widest = std::max(widest, (int)dtype_bits(dtype) / 8);
    };
    for (auto& e : p.exprs)
        if (e.kind == Expr::Load && e.access.chain.empty() && e.access.stride[n - 1] == 1) consider(e.access.dtype);
    for (auto& o : p.outs)
        if (!o.reduce) consider(o.dtype);
    if (p.acc_expr >= 0) widest = std::max(widest, 4);
    int nv = std::max(1, max_bytes / widest);
    auto ok = [&](int v) {
        if (N % v) return false;
        for (auto& e : p.exprs) {
            if (e.kind != Expr::Load || !e.access.chain.empty()) continue;
            if (e.access.stride[n - 1] != 1) continue;
            if (e.access.dtype == HE_BOOL) return false;
            for (int d = 0; d + 1 < n; d++)
                if (e.access.stride[d] % v) return false;
        }
        for (auto& o : p.outs) {
            if (!o.reduce && o.dtype == HE_BOOL) return false;
            if (!o.reduce && !o.stride.empty() && o.stride[n - 1] == 1)
                for (int d = 0; d + 1 < n; d++)
                    if (o.stride[d] % v) return false;
        }
        return true;
    };
    while (nv > 1 && !ok(nv)) nv /= 2;
    return nv;
}

bool attach_post(Program* main, const Program& post) {
    if (main->post || post.acc_expr >= 0 || post.post || post.dims.empty()) return false;
    // one thread per column evaluates it: a program over [columns] and nothing else
    const int64_t cols = post.N();
    if (ir::num_elements(post.dims) != cols || cols != main->N() || post.exprs.empty() || post.outs.empty()) return false;
    for (const Out& o : post.outs)
        if (o.reduce || o.dtype == HE_BOOL || !o.stride.empty()) return false;
    for (const Expr& e : post.exprs)
        if (e.kind == Expr::Load && (!e.access.chain.empty() || e.access.dtype == HE_BOOL)) return false;
    // its arguments among main's: a column reduction that yields one row of `cols` values, or a tensor both only read
    std::vector<int> to_main(post.args.size(), -1);
    std::vector<Arg> args = main->args;
    bool reads_a_reduction = false;
    for (size_t a = 0; a < post.args.size(); a++) {
        const Arg& pa = post.args[a];
        for (size_t m = 0; m < main->args.size() && to_main[a] < 0; m++)
            if (main->args[m].node == pa.node) to_main[a] = (int)m;
        if (to_main[a] < 0) {
            to_main[a] = (int)args.size();
            args.push_back(pa);
            continue;
        }
        const Arg& ma = main->args[to_main[a]];
        if (pa.is_output) return false;  // writes what main reads or writes
        if (!ma.is_output) continue;
        const Out* out = nullptr;
        for (const Out& o : main->outs)
            if (o.arg == to_main[a]) out = &o;
        if (!out || !out->reduce || !out->fold_m || out->fold_n || main->B() / out->b_div != 1) return false;
        reads_a_reduction = true;
    }
    if (!reads_a_reduction) return false;
    Program carried = post;
    carried.args.clear();  // indices refer to main's list
    for (Expr& e : carried.exprs)
        if (e.kind == Expr::Load) e.access.arg = to_main[e.access.arg];
    for (Out& o : carried.outs) o.arg = to_main[o.arg];
    main->args = std::move(args);
    main->post = std::make_shared<const Program>(std::move(carried));
    return true;
}

// A load whose value is one element per row (a [.., M, 1] operand broadcast along the columns): deferred as a scalar
// when only row-varying loads are (the GEMM epilogue's pipelined form, where a load left inline would be younger than
// the next step's requests and make the step wait for them).
static bool is_deferred_row_scalar(const Program& p, const Expr& e, bool row_varying_only) {
    if (!row_varying_only || e.kind != Expr::Load || !e.access.chain.empty() || e.access.dtype == HE_BOOL) return false;
    const int n = (int)p.dims.size();
    if (n < 2 || p.dims[n - 2] <= 1 || e.access.stride[n - 2] == 0) return false;
    return p.dims[n - 1] <= 1 || e.access.stride[n - 1] == 0;
}
static bool is_deferred_load(const Program& p, const Expr& e, int nv, bool row_varying_only = false) {
    if (e.kind != Expr::Load || nv < 2 || !e.access.chain.empty() || e.access.dtype == HE_BOOL) return false;
    const int n = (int)p.dims.size();
    if (row_varying_only && (n < 2 || p.dims[n - 2] <= 1 || e.access.stride[n - 2] == 0)) return false;
    return p.dims[n - 1] > 1 && e.access.stride[n - 1] == 1;
}
static std::string raw_type(int dtype, int nv) {
    const char* elem = dtype == HE_BF16 ? "u16" : dtype == HE_F16 ? "f16_t" : dtype == HE_U32 ? "u32" : "float";
    return strfmt("typename Vec<%s, %d>::type", elem, nv);
}
std::string emit_raw_members(const Program& p, int nv, bool row_varying_only) {
    std::ostringstream s;
    for (size_t i = 0; i < p.exprs.size(); i++)
        if (is_deferred_load(p, p.exprs[i], nv, row_varying_only)) s << raw_type(p.exprs[i].access.dtype, nv) << " raw" << i << ";\n";
        else if (is_deferred_row_scalar(p, p.exprs[i], row_varying_only)) s << cls_type(p.exprs[i].cls) << " raw" << i << ";\n";
    return s.str();
}

bool is_uniform_pow(const Program& p, int id) {
    const Expr& e = p.exprs[id];
    if (e.kind != Expr::Binary || (BOp)e.op != BOp::Pow) return false;
    const Expr& rhs = p.exprs[e.b];
    return rhs.kind == Expr::Load && rhs.cls == Cls::F && rhs.access.chain.empty() &&
           std::all_of(rhs.access.stride.begin(), rhs.access.stride.end(), [](int64_t w) { return w == 0; });
}

std::vector<char> row_invariant_exprs(const Program& p) {
    const int n = (int)p.dims.size();
    std::vector<char> inv(p.exprs.size(), 0);
    if (n < 2) return inv;
    for (size_t i = 0; i < p.exprs.size(); i++) {
        const Expr& e = p.exprs[i];
        switch (e.kind) {
            case Expr::Load: inv[i] = e.access.chain.empty() && (p.dims[n - 2] <= 1 || e.access.stride[n - 2] == 0); break;
            case Expr::Acc: inv[i] = 0; break;
            case Expr::Const: inv[i] = 1; break;
            case Expr::Unary:
            case Expr::Cast: inv[i] = inv[e.a]; break;
            case Expr::Binary:
            case Expr::Compare: inv[i] = inv[e.a] && inv[e.b]; break;
            case Expr::Select: inv[i] = inv[e.a] && inv[e.b] && inv[e.c]; break;
        }
    }
    return inv;
}

std::string emit_exprs(const Program& p, const EmitCtx& cx) {
    const int n = (int)p.dims.size();
    const int NV = cx.nv;
    std::ostringstream s;
    const std::vector<char> invariant = cx.row_part ? row_invariant_exprs(p) : std::vector<char>();
    auto coord_sum = [&](const std::vector<int64_t>& stride) {
        // Linear index of the first of the NV columns.
        std::ostringstream o;
        o << "(size_t)0";
        for (int d = 0; d < n; d++) {
            if (stride[d] == 0 || p.dims[d] <= 1) continue;
            std::string c = d == n - 1 ? "n0" : d == n - 2 ? "m" : "cB" + std::to_string(d);
            o << " + (size_t)" << c << " * " << stride[d] << "ull";
        }
        return o.str();
    };
    for (size_t i = 0; i < p.exprs.size(); i++) {
        const Expr& e = p.exprs[i];
        const std::string v = "e" + std::to_string(i);
        const char* T = cls_type(e.cls);
        if (cx.row_part == 1 && !invariant[i]) continue;
        if (cx.row_part == 2 && invariant[i]) continue;
        if (cx.phase != 0 && is_deferred_row_scalar(p, e, cx.defer_row_varying_only)) {
            if (cx.phase == 1) s << "R.raw" << i << " = ld_one(a" << e.access.arg << " + " << coord_sum(e.access.stride) << ");\n";
            else s << T << " " << v << "[" << NV << "];\n#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) " << v << "[k] = R.raw" << i << ";\n";
            continue;
        }
        if (cx.phase != 0) {
            const bool deferred = is_deferred_load(p, e, NV, cx.defer_row_varying_only);
            if (cx.phase == 1) {
                if (deferred)
                    s << "{ const size_t o = " << coord_sum(e.access.stride) << ";\nR.raw" << i << " = *(const " << raw_type(e.access.dtype, NV)
                      << "*)(a" << e.access.arg << " + o); }\n";
                continue;
            }
            if (deferred) {
                s << T << " " << v << "[" << NV << "];\n#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) " << v << "[k] = ";
                if (e.access.dtype == HE_BF16) s << "__builtin_bit_cast(float, (u32)R.raw" << i << "[k] << 16);\n";
                else if (e.access.dtype == HE_F16) s << "(float)R.raw" << i << "[k];\n";
                else s << "R.raw" << i << "[k];\n";
                continue;
            }
        }
        auto each = [&](const std::string& rhs_k) {
            s << T << " " << v << "[" << NV << "];\n#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) " << v
              << "[k] = " << rhs_k << ";\n";
        };
        auto ref = [&](int id) { return "e" + std::to_string(id) + "[k]"; };
        switch (e.kind) {
            case Expr::Load: {
                const Access& a = e.access;
                if (cx.arg_values && cx.arg_values->count(a.arg)) {
                    each(cx.arg_values->at(a.arg));
                    break;
                }
                const int64_t sn = p.dims[n - 1] > 1 ? a.stride[n - 1] : 0;
                const std::string ptr = "a" + std::to_string(a.arg);
                if (cx.row_part == 1) s << T << " " << v << "[" << NV << "] = {};\nif (col_ok) { const size_t o = " << coord_sum(a.stride) << ";\n";
                else s << T << " " << v << "[" << NV << "];\n{ const size_t o = " << coord_sum(a.stride) << ";\n";
                if (!a.chain.empty()) {
                    s << "#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) { u32 lin = (u32)(o + (size_t)k * " << sn
                      << "ull);\n";
                    for (auto& g : a.chain) emit_generic_map(s, g);
                    if (a.dtype == HE_BOOL)
                        s << "\n" << v << "[k] = ((" << ptr << "[lin >> 5] >> (lin & 31u)) & 1u) != 0; }\n";
                    else
                        s << "\n" << v << "[k] = ld_one(" << ptr << " + lin); }\n";
                } else if (a.dtype == HE_BOOL) {
                    s << "#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) { const size_t l = o + (size_t)k * " << sn
                      << "ull; " << v << "[k] = ((" << ptr << "[l >> 5] >> (l & 31)) & 1u) != 0; }\n";
                } else if (sn == 1 && NV > 1) {
                    s << "ld_vec<" << NV << ">(" << ptr << " + o, " << v << ");\n";
                } else if (sn == 0) {
                    s << "const " << T << " t = ld_one(" << ptr << " + o);\n#pragma unroll\nfor (int k = 0; k < " << NV
                      << "; k++) " << v << "[k] = t;\n";
                } else {
                    s << "#pragma unroll\nfor (int k = 0; k < " << NV << "; k++) " << v << "[k] = ld_one(" << ptr
                      << " + o + (size_t)k * " << sn << "ull);\n";
                }
                s << "}\n";
                break;
            }
            case Expr::Acc: each("acc[k]"); break;
            case Expr::Const:
                if (e.cls == Cls::F) each(f32_literal(e.bits));
                else if (e.cls == Cls::I) each(strfmt("0x%xu", e.bits));
                else each(e.bits ? "true" : "false");
                break;
            case Expr::Unary: each(unary_expr(e, ref(e.a), p.fast_math)); break;
            case Expr::Binary: {
                const Expr& rhs = p.exprs[e.b];
                if ((BOp)e.op == BOp::Pow && rhs.kind == Expr::Const && rhs.cls == Cls::F) {
                    // x ** 1 and x ** 2 are exact products; any other exponent takes the precise powf (the fast
                    // exp2(y * log2(x)) form is undefined for negative bases).
                    float y;
                    memcpy(&y, &rhs.bits, 4);
                    if (y == 1.0f) { each(ref(e.a)); break; }
                    if (y == 2.0f) { each(ref(e.a) + " * " + ref(e.a)); break; }
                }
                if (is_uniform_pow(p, (int)i)) {
                    if (cx.uniform_pow_is_square) each(ref(e.a) + " * " + ref(e.a));
                    else each("pow_uniform(" + ref(e.a) + ", " + ref(e.b) + ")");
                    break;
                }
                each(binary_expr(e, e.cls, ref(e.a), ref(e.b), p.fast_math));
                break;
            }
            case Expr::Compare: each(ref(e.a) + " " + compare_sym(e.op) + " " + ref(e.b)); break;
            case Expr::Select: each(ref(e.c) + " ? " + ref(e.b) + " : " + ref(e.a)); break;  // rhs when true (jit.rs:583-586)
            case Expr::Cast: {
                Cls from = p.exprs[e.a].cls;
                std::string x = ref(e.a);
                if (from == Cls::F && e.cls == Cls::B) each(x + " != 0.0f");
                else if (from == Cls::B && e.cls == Cls::F) each(x + " ? 1.0f : 0.0f");
                else if (from == Cls::F && e.cls == Cls::I) each("(u32)" + x);
                else if (from == Cls::I && e.cls == Cls::F) each("(float)" + x);
                else if (from == Cls::B && e.cls == Cls::I) each(x + " ? 1u : 0u");
                else if (from == Cls::I && e.cls == Cls::B) each(x + " != 0u");
                else fail(HE_ERR_INTERNAL, "cast within one data class");
                break;
            }
        }
    }
    return s.str();
}

// ---------------------------------------------------------------------------------------------------------
// Pointwise / reduction kernel.
//
// The iteration space is viewed as [B][M][N]. A block of 256 threads owns one b, TR = TY*RPT rows and
// TC = TX*NV columns; a thread owns NV consecutive columns (one 16-byte access per operand) and walks RPT rows.
//   * reductions that keep the row (fold N only) finish per row: butterfly over the row's TX lanes, then one
//     store or atomic per row segment;
//   * reductions that keep the column (fold M only) accumulate NV partial sums per thread over its rows, are
//     combined across the block's TY row-groups through LDS and issue one atomic per column per block;
//   * reductions that fold both accumulate one scalar per thread, reduced per wave (shuffles), per block (LDS)
//     and finished with one atomic per block.
// ---------------------------------------------------------------------------------------------------------
static int pow2_ceil(int64_t x) {
    int p = 1;
    while (p < x) p *= 2;
    return p;
}

PointwiseLaunch emit_pointwise(const Program& p, const std::string& entry) {
    HE_REQUIRE(p.acc_expr < 0, HE_ERR_INVALID, "program reads a GEMM accumulator");
    const int n = (int)p.dims.size();
    const int64_t N = p.N(), M = p.M(), B = p.B();
    HE_REQUIRE(ir::num_elements(p.dims) < (1ll << 32), HE_ERR_INVALID, "pointwise kernels index with 32 bits");
    PointwiseLaunch L;
    L.entry = entry;
    if (ir::num_elements(p.dims) == 0) {
        L.grid = 0;
        L.source = "";
        return L;
    }
    const int NV = pick_nv(p, 16);
    const int threads = 256;
    // A Mean is the sum scaled by 1/group. The reference scales every term (float * double literal,
    // pointwise/jit.rs:413-418); scaling the finished sum once, also in double, differs from that by rounding only
    // and takes three double-rate instructions per element out of the inner loop.
    auto scaled = [](const Out& o, const std::string& x) {
        return o.rop == ROp::Mean ? strfmt("(float)((double)(%s) * %.17g)", x.c_str(), o.mean_scale) : x;
    };
    bool any_col = false, any_scalar = false;
    for (auto& o : p.outs) {
        if (!o.reduce) continue;
        if (o.fold_m && !o.fold_n) any_col = true;
        if (o.fold_m && o.fold_n) any_scalar = true;
    }
    // Threads along a row. With a column reduction a block should be tall rather than wide: its TY row groups are
    // combined in LDS, so every block leaves one partial per column it spans, not one per column per row group.
    int tx_cap = any_col ? 64 : threads;
    if (const char* env = tuning::get("HELIUM_HIP_POINTWISE_TX")) tx_cap = std::max(1, atoi(env));
    int TX = (int)std::min<int64_t>(tx_cap, pow2_ceil((N + NV - 1) / NV));
    int TY = threads / TX;
    const int64_t gx = (N + (int64_t)TX * NV - 1) / ((int64_t)TX * NV);
    const int64_t gy1 = (M + TY - 1) / TY;
    int64_t blocks1 = gx * gy1 * B;
    int RPT = 1;
    if (const char* env = tuning::get("HELIUM_HIP_POINTWISE_RPT")) {
        RPT = std::max(1, atoi(env));
    } else {
        // Blocks that end in a column or scalar reduction pay for it once per block (LDS exchange, partials) and are
        // worth making tall, up to about 256 KB of operands per block and no fewer than two blocks per CU
        // (measured: [1,4096,4096] f32 chain with four operands best at 16 rows per thread, a [200704,256] bf16
        // column reduction at 32).
        const bool tall = any_col || any_scalar;
        int64_t row_bytes = 0;  // bytes one row of a block moves
        for (auto& e : p.exprs)
            if (e.kind == Expr::Load && n >= 2 && e.access.chain.empty() && e.access.stride[n - 2] != 0 && e.access.stride[n - 1] != 0)
                row_bytes += (int64_t)TX * NV * (int64_t)storage_bytes(e.access.dtype, 1);
        for (auto& o : p.outs)
            if (!o.reduce) row_bytes += (int64_t)TX * NV * (int64_t)storage_bytes(o.dtype == HE_BOOL ? HE_U32 : o.dtype, 1);
        while (RPT < (tall ? 32 : 16) && blocks1 / (RPT * 2) >= (tall ? 512 : 2048) &&
               (!tall || row_bytes * TY * RPT * 2 <= (256 << 10)))
            RPT *= 2;
        // A column reduction over few rows (a mean over the 7x7 pixels of a pooled image): when one more doubling or two
        // let a block span all of them and a block per CU is still left, no partial results are written and no second
        // launch folds them.
        if (any_col && !any_scalar)
            for (int r = RPT * 2; r <= 32; r *= 2)
                if ((int64_t)TY * r >= M) {
                    if ((int64_t)TY * RPT < M && gx * B >= 256 && row_bytes * TY * r <= (256 << 10)) RPT = r;
                    break;
                }
    }
    RPT = (int)std::min<int64_t>(RPT, std::max<int64_t>(1, gy1));
    const int TR = TY * RPT;
    const int64_t gy = (M + TR - 1) / TR;
    const int64_t grid = gx * gy * B;
    HE_REQUIRE(grid < (1ll << 31), HE_ERR_INVALID, "pointwise grid too large");
    L.grid = (uint32_t)grid;
    L.threads = threads;
    L.nv = NV;
    L.tx = TX;
    L.ty = TY;
    L.rpt = RPT;
    L.options = {p.fast_math ? "-ffp-contract=fast" : "-ffp-contract=off", "-munsafe-fp-atomics"};

    std::ostringstream s;
    s << "// pointwise kernel generated for gfx950: dims=[";
    for (int d = 0; d < n; d++) s << (d ? "," : "") << p.dims[d];
    s << "] NV=" << NV << " TX=" << TX << " TY=" << TY << " RPT=" << RPT << "\n";
    s << kPrelude;
    s << "#define NV " << NV << "\n#define TX " << TX << "\n#define TY " << TY << "\n#define RPT " << RPT
      << "\n#define TR " << TR << "\n#define DIM_N " << N << "u\n#define DIM_M " << M << "u\n";
    s << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void " << entry << "(";
    for (size_t a = 0; a < p.args.size(); a++)
        s << (a ? ", " : "") << (p.args[a].is_output ? "" : "const ") << c_type(p.args[a].dtype) << "* __restrict__ a" << a;
    // Reductions whose terms come from several blocks: each block parks its partial result in scratch, and the
    // partials are folded in block order (the same result on every run) into an output that needs no initial value:
    //  - short launches: by the block that arrives last, which every block finds out from a ticket (one launch);
    //  - long launches: by a second, small launch of `<entry>_finalize` (two launches, as many as fill + kernel).
    // One float atomic per block and column onto a pre-filled output is only left for rows wider than a block:
    // atomics on one address, or on neighbours within a cache line, are served one after another (about 20 ns
    // each), which for a [200704 x 256] column sum is 25,000 per line and took 200 us.
    struct WsUse {
        bool on = false, ticket = false;
        uint64_t foff = 0, coff = 0, coff1 = 0;
        int64_t group = 0, ngroups = 0;  // scalar reductions with many blocks: tickets in two levels
    };
    // Every ticket counter gets a cache line of its own, and a scalar reduction over many blocks counts arrivals in
    // groups of about sqrt(blocks), the last arrival of a group carrying the group's ticket to the second level.
    //
    // The last block's way out is a chain of memory round trips (partials land, ticket, partials back, result), a few
    // microseconds that nothing overlaps when all blocks end together. A short launch still gains, because a second
    // dependent launch costs more than that (measured: [1,4096,4096] f32 with two reductions 54 us with tickets,
    // 50 us with two launches; a [256,512] f32 column sum inside a graph 29 us -> 26 us with tickets).
    const uint64_t CS = 32;  // counter stride in u32
    bool tickets = B * M * N <= (int64_t)1 << 21;
    if (const char* env = tuning::get("HELIUM_HIP_REDUCE")) tickets = std::string(env) == "ticket";
    std::vector<WsUse> ws(p.outs.size());
    bool any_finalize = false;
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!o.reduce) continue;
        if (o.fold_m && !o.fold_n && gy * o.b_div > 1) {
            ws[oi].on = true;
            // a column's counter is one address: beyond a few dozen arrivals the tickets would queue up
            ws[oi].ticket = tickets && gy * o.b_div <= 64;
            ws[oi].foff = L.ws_floats;
            L.ws_floats += (uint64_t)grid * TX * NV;
            if (ws[oi].ticket) {
                ws[oi].coff = L.ws_counters;
                L.ws_counters += (uint64_t)(B / o.b_div) * gx * CS;
            }
        } else if (o.fold_m && o.fold_n && gx * gy * o.b_div > 1) {
            const int64_t per = gx * gy * o.b_div, outs_n = B / o.b_div;
            ws[oi].on = true;
            ws[oi].ticket = tickets;
            ws[oi].foff = L.ws_floats;
            L.ws_floats += (uint64_t)grid;
            if (ws[oi].ticket) {
                ws[oi].coff = L.ws_counters;
                L.ws_counters += (uint64_t)outs_n * CS;
                if (per > 64) {
                    int64_t G = 8;
                    while (G * G < per) G *= 2;
                    ws[oi].group = G;
                    ws[oi].ngroups = (per + G - 1) / G;
                    ws[oi].coff1 = L.ws_counters;
                    L.ws_counters += (uint64_t)outs_n * ws[oi].ngroups * CS;
                }
            }
        }
        if (ws[oi].on && !ws[oi].ticket) any_finalize = true;
    }
    const bool any_ws = L.ws_floats > 0;
    const bool any_ticket = L.ws_counters > 0;
    if (any_ws) s << ", float* wsf, u32* wsc";
    s << ") {\n";
    if (any_col && TY > 1) s << "__shared__ float col_red[TY * TX * NV];\n";
    if (any_scalar) s << "__shared__ float blk_red[" << threads / 64 << "];\n";
    // rows that one block spans with two or four waves: the waves' parts of a row meet in LDS (two sets taking turns, so
    // one barrier per row is enough), and no atomics - and no fill launch ahead of the kernel - are needed
    const bool rows_meet_in_lds = gx == 1 && TX > 64 && !tuning::get("HELIUM_HIP_NO_ROW_LDS");
    if (rows_meet_in_lds) {
        size_t row_outs = 0;
        for (auto& o : p.outs) row_outs += o.reduce && o.fold_n && !o.fold_m;
        if (row_outs) s << "__shared__ float row_red[" << row_outs << "][2][" << threads / 64 << "];\n";
    }
    if (any_ticket) s << "__shared__ u32 ticket_s[" << p.outs.size() << "];\n";
    s << "u32 t = blockIdx.x;\nconst u32 tile_x = t % " << gx << "u; t /= " << gx << "u;\nconst u32 tile_y = t % " << gy
      << "u; t /= " << gy << "u;\nconst u32 b = t;\n";
    {
        // coordinates of the dims that flatten into b
        s << "u32 brem = b; (void)brem;\n";
        for (int d = n - 3; d >= 0; d--)
            s << "const u32 cB" << d << " = brem % " << p.dims[d] << "u; brem /= " << p.dims[d] << "u; (void)cB" << d << ";\n";
    }
    s << "const u32 tx = threadIdx.x % TX, ty = threadIdx.x / TX;\n";
    s << "const u32 n0 = (tile_x * TX + tx) * NV;\nconst bool col_ok = n0 < DIM_N;\n";
    // reduction partials
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!o.reduce) continue;
        if (o.fold_m && !o.fold_n)
            s << "float rc" << oi << "[NV];\n#pragma unroll\nfor (int k = 0; k < NV; k++) rc" << oi << "[k] = red_identity<"
              << (int)o.rop << ">();\n";
        else if (o.fold_m && o.fold_n)
            s << "float rs" << oi << " = red_identity<" << (int)o.rop << ">();\n";
    }
    // The rows of a block whose tile lies wholly inside the tensor carry no bounds test: a load under a per-row
    // predicate cannot be issued ahead of the previous row's work, and a streaming kernel then waits out one memory
    // round trip per row.
    // What is the same in every row a thread walks (per-channel operands of an NHWC activation seen as [rows, channels],
    // and what is computed from them alone) is loaded and computed once, ahead of the rows: under the rows' predicate
    // the compiler may not move those loads itself.
    bool hoist_rows = false;
    {
        const std::vector<char> inv = row_invariant_exprs(p);
        for (size_t i = 0; i < p.exprs.size(); i++) hoist_rows = hoist_rows || (inv[i] && p.exprs[i].kind == Expr::Load);
        hoist_rows = hoist_rows && RPT > 1;
        if (hoist_rows) {
            EmitCtx cx;
            cx.nv = NV;
            cx.row_part = 1;
            s << emit_exprs(p, cx);
        }
    }
    std::ostringstream& main_stream = s;
    auto row_body = [&](bool squares, bool from_raw) {
    std::ostringstream s;
    for (size_t oi = 0; oi < p.outs.size(); oi++)
        if (p.outs[oi].reduce && p.outs[oi].fold_n && !p.outs[oi].fold_m)
            s << "float rr" << oi << " = red_identity<" << (int)p.outs[oi].rop << ">();\n";
    s << "if (ok) {\n";
    EmitCtx cx;
    cx.nv = NV;
    cx.uniform_pow_is_square = squares;
    cx.row_part = hoist_rows ? 2 : 0;
    cx.phase = from_raw ? 2 : 0;
    cx.defer_row_varying_only = from_raw;
    s << emit_exprs(p, cx);
    // outputs
    Shape pst = ir::packed_strides(p.dims);
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        const std::string v = "e" + std::to_string(o.expr);
        if (!o.reduce) {
            if (o.stride.empty()) {
                s << "{ const size_t o = (size_t)b * " << (M * N) << "ull + (size_t)m * " << N << "ull + n0;\n";
            } else {
                // stored by its own strides: vectors where its innermost coordinate is the iteration's
                s << "{ const size_t o = (size_t)0";
                for (int d = 0; d < n; d++) {
                    if (o.stride[d] == 0 || p.dims[d] <= 1) continue;
                    s << " + (size_t)" << (d == n - 1 ? std::string("n0") : d == n - 2 ? std::string("m") : "cB" + std::to_string(d)) << " * " << o.stride[d] << "ull";
                }
                s << ";\n";
                if (!(p.dims[n - 1] <= 1 || o.stride[n - 1] == 1)) {
                    s << "#pragma unroll\nfor (int k = 0; k < NV; k++) st_one(a" << o.arg << " + o + (size_t)k * " << o.stride[n - 1] << "ull, " << v << "[k]);\n}\n";
                    continue;
                }
            }
            if (o.dtype == HE_BOOL) {
                // bit k of word o/32; the buffer is cleared before the launch (jit.rs:293-301)
                s << "#pragma unroll\nfor (int k = 0; k < NV; k++) { const size_t l = o + k; if (" << v
                  << "[k]) atomicOr(a" << o.arg << " + (l >> 5), 1u << (l & 31)); }\n";
            } else {
                s << "st_vec<NV, " << (streams_out(p.args[o.arg]) ? "true" : "false") << ">(a" << o.arg << " + o, " << v << ");\n";
            }
            s << "}\n";
            continue;
        }
        std::string term = v + "[k]";
        if (o.fold_m && !o.fold_n)
            s << "#pragma unroll\nfor (int k = 0; k < NV; k++) rc" << oi << "[k] = red_op<" << (int)o.rop << ">(rc" << oi
              << "[k], " << term << ");\n";
        else if (o.fold_m && o.fold_n)
            s << "#pragma unroll\nfor (int k = 0; k < NV; k++) rs" << oi << " = red_op<" << (int)o.rop << ">(rs" << oi << ", "
              << term << ");\n";
        else
            s << "#pragma unroll\nfor (int k = 0; k < NV; k++) rr" << oi << " = red_op<" << (int)o.rop << ">(rr" << oi << ", "
              << term << ");\n";
    }
    s << "}\n";  // if (ok)
    // per-row reductions: every lane takes part in the butterfly
    size_t row_out = 0;
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!(o.reduce && o.fold_n && !o.fold_m)) continue;
        const int width = std::min(TX, 64);
        s << "{ float r = wave_reduce<" << (int)o.rop << ", " << width << ">(rr" << oi << ");\n";
        if (gx == 1 && TX <= 64)  // one wave segment holds the whole row
            s << "if ((threadIdx.x % " << width << ") == 0 && m < DIM_M && col_ok) a" << o.arg << "[(size_t)b * " << M << "ull + m] = " << scaled(o, "r") << "; }\n";
        else if (rows_meet_in_lds) {
            // (lanes past the row's end hold the identity; the row's first lane is in range whenever the row is)
            s << "if ((threadIdx.x & 63u) == 0) row_red[" << row_out << "][i & 1u][threadIdx.x >> 6] = r;\n__syncthreads();\n"
              << "if ((threadIdx.x % " << TX << "u) == 0 && m < DIM_M) {\nfloat acc = r;\nfor (u32 w = 1; w < " << TX / 64
              << "u; w++) acc = red_op<" << (int)o.rop << ">(acc, row_red[" << row_out << "][i & 1u][(threadIdx.x >> 6) + w]);\na" << o.arg << "[(size_t)b * "
              << M << "ull + m] = " << scaled(o, "acc") << ";\n} }\n";
            row_out++;
        } else
            s << "if ((threadIdx.x % " << width << ") == 0 && m < DIM_M && col_ok) atomic_red<" << (int)o.rop << ">(a" << o.arg
              << " + (size_t)b * " << M << "ull + m, " << scaled(o, "r") << "); }\n";
    }
    return s.str();
    };
    {
        std::ostringstream& s = main_stream;
        const int64_t TRv = (int64_t)TY * RPT;
        const bool ragged = M % TRv != 0 || N % ((int64_t)TX * NV) != 0;
        // UNROLL rows are in flight at a time: all RPT at once would keep every row's operands in registers
        // (one row where the expression count is large: two rows of a 75-expression kernel keep twice the registers and
        // gain nothing; training step with the limit at none / 64 / 40 / 24 expressions: 5.34 / 5.31 / 5.30 / 5.28 ms)
        int unroll = std::min(RPT, p.exprs.size() > 24 ? 1 : 2);
        if (const char* env = tuning::get("HELIUM_HIP_POINTWISE_UNROLL")) unroll = std::max(1, std::min(RPT, atoi(env)));
        while (RPT % unroll) unroll--;
        const std::string head = "#pragma unroll 1\nfor (u32 i0 = 0; i0 < RPT; i0 += " + std::to_string(unroll) + ") {\n#pragma unroll\nfor (u32 iu = 0; iu < " +
                                 std::to_string(unroll) + "; iu++) {\nconst u32 i = i0 + iu;\nconst u32 m = tile_y * TR + i * TY + ty;\n";
        // (a launch of a few workgroups runs its code once or twice: a second form of the body without the bounds tests
        // costs more in instruction fetch than the tests do)
        const bool few_blocks = grid <= 16;
        // One row in flight per thread leaves a streaming kernel short of outstanding loads (three 8-byte loads per
        // lane, four waves per SIMD: 24 KB per CU). The next row's operands are therefore requested before the current
        // row is computed: they cost a few registers, where a second whole row in flight would double all of them.
        bool any_deferred = false;
        for (const Expr& e : p.exprs) any_deferred = any_deferred || is_deferred_load(p, e, NV, true);
        bool pipelined = unroll == 1 && RPT >= 2 && any_deferred && !few_blocks;
        int ahead = 1;  // rows requested ahead of the one being computed
        if (const char* env = tuning::get("HELIUM_HIP_POINTWISE_PIPELINE")) ahead = atoi(env);
        ahead = std::min(ahead, RPT - 1);
        pipelined = pipelined && ahead >= 1;
        std::string ahead_head, ahead_tail;
        if (pipelined) {
            EmitCtx lx;
            lx.nv = NV;
            lx.row_part = hoist_rows ? 2 : 0;
            lx.phase = 1;
            lx.defer_row_varying_only = true;
            const std::string issue = emit_exprs(p, lx);
            s << "struct RowRaw {\n" << emit_raw_members(p, NV, true) << "};\n";
            auto name = [](int d) { return d == 0 ? std::string("R") : "R" + std::to_string(d); };
            for (int d = 0; d < ahead; d++)
                ahead_head += "RowRaw " + name(d) + ";\n{ const u32 m = tile_y * TR + " + std::to_string(d) + " * TY + ty;\n" +
                              (d ? "RowRaw& R = " + name(d) + ";\n" : std::string()) + issue + "}\n";
            ahead_head += "#pragma unroll 1\nfor (u32 i = 0; i < RPT; i++) {\nconst u32 m = tile_y * TR + i * TY + ty;\nRowRaw Rn;\n{ const u32 i1 = i + " +
                          std::to_string(ahead) + " < RPT ? i + " + std::to_string(ahead) + " : RPT - 1;\nconst u32 m = tile_y * TR + i1 * TY + ty;\nRowRaw& R = Rn;\n" +
                          issue + "}\n{\n";
            for (int d = 0; d + 1 < ahead; d++) ahead_tail += name(d) + " = " + name(d + 1) + ";\n";
            ahead_tail += name(ahead - 1) + " = Rn;\n";
        }
        auto loops = [&](const std::string& body, const std::string& body_from_raw) {
            if (ragged && few_blocks) {
                s << head << "const bool ok = col_ok && m < DIM_M;\n" << body << "}\n}\n";
                return;
            }
            if (ragged) s << "if ((tile_y + 1) * TR <= DIM_M && (tile_x + 1) * (TX * NV) <= DIM_N) {\n";
            if (pipelined) s << ahead_head << "const bool ok = true;\n" << body_from_raw << "}\n" << ahead_tail << "}\n";
            else s << head << "const bool ok = true;\n" << body << "}\n}\n";
            if (ragged) s << "} else {\n" << head << "const bool ok = col_ok && m < DIM_M;\n" << body << "}\n}\n}\n";
        };
        // `x.pow_scalar(2.0)` reaches the kernel as Pow with a broadcast 1-element operand. The exponents are read
        // once; when all of them are 2 the loop that squares runs, and the general routine (a few hundred
        // instructions per call site) stays out of the instruction stream of the common case.
        std::vector<int> exps;
        for (size_t i = 0; i < p.exprs.size(); i++)
            if (is_uniform_pow(p, (int)i)) exps.push_back(p.exprs[p.exprs[i].b].access.arg);
        std::sort(exps.begin(), exps.end());
        exps.erase(std::unique(exps.begin(), exps.end()), exps.end());
        if (exps.empty()) {
            loops(row_body(false, false), pipelined ? row_body(false, true) : std::string());
        } else {
            s << "bool all_squares = true;\n";
            for (int a : exps) s << "all_squares = all_squares && ld_one(a" << a << ") == 2.0f;\n";
            s << "if (all_squares) {\n";
            loops(row_body(true, false), pipelined ? row_body(true, true) : std::string());
            s << "} else {\n";
            loops(row_body(false, false), pipelined ? row_body(false, true) : std::string());
            s << "}\n";
        }
    }
    // Phase 1: every block finishes its own partial of each reduction. What no other block contributes to is stored
    // straight to the output; the rest is parked in scratch.
    int n_tickets = 0;
    std::vector<int> ticket_of(p.outs.size(), -1);
    for (size_t oi = 0; oi < p.outs.size(); oi++)
        if (ws[oi].ticket) ticket_of[oi] = n_tickets++;
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!(o.reduce && o.fold_m && !o.fold_n)) continue;
        if (TY > 1) {
            s << "__syncthreads();\n#pragma unroll\nfor (int k = 0; k < NV; k++) col_red[(ty * TX + tx) * NV + k] = rc" << oi
              << "[k];\n__syncthreads();\nif (ty == 0) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) { float r = rc" << oi
              << "[k];\nfor (u32 y = 1; y < TY; y++) r = red_op<" << (int)o.rop << ">(r, col_red[(y * TX + tx) * NV + k]);\nrc"
              << oi << "[k] = r; } }\n";
        }
        if (!ws[oi].on)
            s << "if (ty == 0 && col_ok) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) if (n0 + k < DIM_N) a" << o.arg << "[(size_t)b * " << N
              << "ull + n0 + k] = " << scaled(o, "rc" + std::to_string(oi) + "[k]") << "; }\n";
        else if (ws[oi].ticket)
            s << "if (ty == 0) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) HE_WS_STORE(wsf + " << ws[oi].foff
              << "ull + (size_t)blockIdx.x * (TX * NV) + tx * NV + k, rc" << oi << "[k]); }\n";
        else
            s << "if (ty == 0) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) wsf[" << ws[oi].foff
              << "ull + (size_t)blockIdx.x * (TX * NV) + tx * NV + k] = rc" << oi << "[k]; }\n";
    }
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!(o.reduce && o.fold_m && o.fold_n)) continue;
        s << "{ float r = wave_reduce<" << (int)o.rop << ", 64>(rs" << oi << ");\n__syncthreads();\nif ((threadIdx.x & 63) == 0) blk_red[threadIdx.x >> 6] = r;\n__syncthreads();\n";
        s << "if (threadIdx.x == 0) { r = blk_red[0];\nfor (int w = 1; w < " << threads / 64 << "; w++) r = red_op<"
          << (int)o.rop << ">(r, blk_red[w]);\n";
        if (!ws[oi].on)
            s << "a" << o.arg << "[b / " << o.b_div << "u] = " << scaled(o, "r") << "; } }\n";
        else if (ws[oi].ticket)
            s << "HE_WS_STORE(wsf + " << ws[oi].foff << "ull + blockIdx.x, r); } }\n";
        else
            s << "wsf[" << ws[oi].foff << "ull + blockIdx.x] = r; } }\n";
    }
    if (n_tickets) {
        // Phase 2: once every wave's partials have landed, one thread takes the block's ticket of each reduction.
        s << "HE_WS_DRAIN();\n__syncthreads();\nif (threadIdx.x == 0) {\n";
        for (size_t oi = 0; oi < p.outs.size(); oi++) {
            if (!ws[oi].ticket) continue;
            const Out& o = p.outs[oi];
            const int j = ticket_of[oi];
            if (!o.fold_n) {
                s << "const u32 tk" << j << " = HE_WS_TICKET(wsc + " << ws[oi].coff << "ull + (size_t)((b / " << o.b_div << "u) * " << gx << "u + tile_x) * " << CS << "u) == "
                  << gy * o.b_div - 1 << "u;\n";
                continue;
            }
            const int64_t per = gx * gy * o.b_div;
            if (!ws[oi].group) {
                s << "const u32 tk" << j << " = HE_WS_TICKET(wsc + " << ws[oi].coff << "ull + (size_t)(b / " << o.b_div << "u) * " << CS << "u) == "
                  << per - 1 << "u;\n";
                continue;
            }
            s << "u32 tk" << j << " = 0u;\n{ const u32 q = b / " << o.b_div << "u, lb = blockIdx.x - q * " << per << "u, grp = lb / " << ws[oi].group
              << "u;\nconst u32 rest = " << per << "u - grp * " << ws[oi].group << "u, members = rest < " << ws[oi].group << "u ? rest : " << ws[oi].group << "u;\nu32* c1 = wsc + " << ws[oi].coff1
              << "ull + (size_t)(q * " << ws[oi].ngroups << "u + grp) * " << CS << "u;\nif (HE_WS_TICKET(c1) == members - 1u) {\nHE_WS_STORE(c1, 0u);\n"
              << "tk" << j << " = HE_WS_TICKET(wsc + " << ws[oi].coff << "ull + (size_t)q * " << CS << "u) == " << ws[oi].ngroups - 1 << "u; } }\n";
        }
        for (int j = 0; j < n_tickets; j++) s << "ticket_s[" << j << "] = tk" << j << ";\n";
        s << "}\n__syncthreads();\n";
    }
    // Phase 3: the block that drew the last ticket of a reduction folds all partials, always in the same order. The
    // loads are issued in batches of independent registers: one at a time they would cost a memory round trip each.
    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (!ws[oi].ticket) continue;
        const int rop = (int)o.rop;
        if (!o.fold_n) {
            const int64_t arrivals = gy * o.b_div;  // blocks (b, tile_y) that feed one (output row, tile_x): consecutive b * gy + tile_y
            s << "if (ticket_s[" << ticket_of[oi] << "]) {\nconst u32 q = b / " << o.b_div << "u;\nfloat r[NV];\n#pragma unroll\nfor (int k = 0; k < NV; k++) r[k] = red_identity<"
              << rop << ">();\nif (col_ok) {\nfor (u32 y0 = ty; y0 < " << arrivals << "u; y0 += TY * 8) {\nfloat pv[8][NV];\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\n"
              << "const u32 y = y0 + c * TY;\nconst float* part = wsf + " << ws[oi].foff << "ull + (size_t)((q * " << arrivals << "u + (y < " << arrivals
              << "u ? y : 0u)) * " << gx << "u + tile_x) * (TX * NV) + tx * NV;\n#pragma unroll\nfor (int k = 0; k < NV; k++) pv[c][k] = y < " << arrivals
              << "u ? HE_WS_LOAD(part + k) : red_identity<" << rop << ">();\n}\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\n#pragma unroll\n"
              << "for (int k = 0; k < NV; k++) r[k] = red_op<" << rop << ">(r[k], pv[c][k]);\n}\n}\n}\n";
            if (TY > 1)
                s << "__syncthreads();\n#pragma unroll\nfor (int k = 0; k < NV; k++) col_red[(ty * TX + tx) * NV + k] = r[k];\n__syncthreads();\n"
                  << "if (ty == 0) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) {\nfor (u32 y = 1; y < TY; y++) r[k] = red_op<" << rop
                  << ">(r[k], col_red[(y * TX + tx) * NV + k]);\n} }\n";
            s << "if (ty == 0 && col_ok) {\n#pragma unroll\nfor (int k = 0; k < NV; k++) if (n0 + k < DIM_N) a" << o.arg << "[(size_t)q * " << N
              << "ull + n0 + k] = " << scaled(o, "r[k]") << ";\n}\nif (threadIdx.x == 0) HE_WS_STORE(wsc + " << ws[oi].coff << "ull + (size_t)(q * " << gx << "u + tile_x) * " << CS << "u, 0u);\n}\n";
        } else {
            const int64_t per = gx * gy * o.b_div;  // blocks that feed one output element: consecutive block indices
            s << "if (ticket_s[" << ticket_of[oi] << "]) {\nconst u32 q = b / " << o.b_div << "u;\nfloat acc = red_identity<" << rop
              << ">();\nfor (u32 i0 = threadIdx.x; i0 < " << per << "u; i0 += " << threads * 8 << "u) {\nfloat pv[8];\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\n"
              << "const u32 i = i0 + c * " << threads << "u;\npv[c] = i < " << per << "u ? HE_WS_LOAD(wsf + " << ws[oi].foff << "ull + (size_t)q * " << per
              << "ull + i) : red_identity<" << rop << ">();\n}\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) acc = red_op<" << rop << ">(acc, pv[c]);\n}\n"
              << "acc = wave_reduce<" << rop << ", 64>(acc);\n__syncthreads();\nif ((threadIdx.x & 63) == 0) blk_red[threadIdx.x >> 6] = acc;\n"
              << "__syncthreads();\nif (threadIdx.x == 0) { acc = blk_red[0];\nfor (int w = 1; w < " << threads / 64 << "; w++) acc = red_op<"
              << rop << ">(acc, blk_red[w]);\na" << o.arg << "[q] = " << scaled(o, "acc") << ";\nHE_WS_STORE(wsc + " << ws[oi].coff << "ull + (size_t)q * " << CS << "u, 0u); }\n}\n";
        }
    }
    s << "}\n";
    if (any_finalize) {
        // The second launch: one block per 16 output columns (or per scalar output) folds that slice of the
        // partials, 16 thread groups sharing the blocks of the first launch between them, always in the same order.
        // (fewer columns and more groups where a column has many partials: a thread then adds a few dozen of them, eight
        // loads at a time, instead of a hundred one batch after the other - the launch is all latency)
        auto fold_width = [&](const Out& o) {
            const int64_t arrivals = gy * o.b_div;
            return arrivals >= 512 ? 4 : arrivals >= 128 ? 8 : 16;
        };
        struct Job {
            size_t oi;
            uint32_t first, blocks;
        };
        std::vector<Job> jobs;
        uint32_t total = 0;
        // The column reductions a carried program reads are folded by the same blocks, FW columns each: the threads that
        // end up with a column's sums go on to evaluate that program for the column.
        std::vector<size_t> carried;  // outs
        int64_t carried_arrivals = 0;
        if (p.post) {
            bool ok = true;
            std::vector<char> read(p.args.size(), 0);
            for (const Expr& e : p.post->exprs)
                if (e.kind == Expr::Load) read[e.access.arg] = 1;
            for (size_t oi = 0; oi < p.outs.size() && ok; oi++) {
                const Out& o = p.outs[oi];
                if (!o.reduce || !read[o.arg]) continue;
                ok = ws[oi].on && !ws[oi].ticket && o.fold_m && !o.fold_n && B / o.b_div == 1 &&
                     (carried.empty() || carried_arrivals == gy * o.b_div);
                carried_arrivals = gy * o.b_div;
                carried.push_back(oi);
            }
            if (!ok || carried.empty()) carried.clear();
            L.post_carried = !carried.empty();
        }
        auto is_carried = [&](size_t oi) { return std::find(carried.begin(), carried.end(), oi) != carried.end(); };
        const int CFW = carried.empty() ? 0 : fold_width(p.outs[carried[0]]);
        if (!carried.empty()) total = (uint32_t)((N + CFW - 1) / CFW);
        for (size_t oi = 0; oi < p.outs.size(); oi++) {
            if (!ws[oi].on || ws[oi].ticket || is_carried(oi)) continue;
            const Out& o = p.outs[oi];
            const int FW = fold_width(o);
            const uint32_t nb = o.fold_n ? (uint32_t)(B / o.b_div) : (uint32_t)((B / o.b_div) * ((N + FW - 1) / FW));
            jobs.push_back({oi, total, nb});
            total += nb;
        }
        L.finalize_entry = entry + "_finalize";
        L.finalize_grid = total;
        s << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void " << L.finalize_entry << "(";
        for (size_t a = 0; a < p.args.size(); a++)
            s << (a ? ", " : "") << (p.args[a].is_output ? "" : "const ") << c_type(p.args[a].dtype) << "* __restrict__ a" << a;
        s << ", const float* __restrict__ wsf) {\n__shared__ float fin_red[" << threads << "];\n";
        if (!carried.empty()) {
            const int FW = CFW, FG = threads / FW;
            const int64_t arrivals = carried_arrivals, slices = (N + FW - 1) / FW;
            s << "if (blockIdx.x < " << slices << "u) {\nconst u32 n = blockIdx.x * " << FW << "u + threadIdx.x % " << FW
              << "u, grp = threadIdx.x / " << FW << "u;\nconst u32 tile_x = n / (TX * NV), within = n % (TX * NV);\n";
            std::map<int, std::string> values;
            // every reduction's partials are requested before any is added up: the launch is all latency
            for (size_t oi : carried)
                s << "float red" << oi << " = 0.0f, acc" << oi << " = red_identity<" << (int)p.outs[oi].rop << ">();\n";
            s << "if (n < DIM_N) {\nfor (u32 j0 = grp; j0 < " << arrivals << "u; j0 += " << FG * 8 << "u) {\n";
            for (size_t oi : carried) {
                const int rop = (int)p.outs[oi].rop;
                s << "float pv" << oi << "[8];\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\nconst u32 j = j0 + c * " << FG << "u;\npv" << oi << "[c] = j < "
                  << arrivals << "u ? wsf[" << ws[oi].foff << "ull + (size_t)(j * " << gx << "u + tile_x) * (TX * NV) + within] : red_identity<" << rop << ">();\n}\n";
            }
            for (size_t oi : carried)
                s << "#pragma unroll\nfor (u32 c = 0; c < 8; c++) acc" << oi << " = red_op<" << (int)p.outs[oi].rop << ">(acc" << oi << ", pv" << oi << "[c]);\n";
            s << "}\n}\n";
            for (size_t oi : carried) {
                const Out& o = p.outs[oi];
                const int rop = (int)o.rop;
                s << "__syncthreads();\nfin_red[threadIdx.x] = acc" << oi << ";\n__syncthreads();\nif (grp == 0 && n < DIM_N) {\nfloat acc = acc" << oi
                  << ";\nfor (u32 g = 1; g < " << FG << "u; g++) acc = red_op<" << rop << ">(acc, fin_red[g * " << FW << "u + threadIdx.x]);\nred" << oi
                  << " = store_and_keep(a" << o.arg << " + n, " << scaled(o, "acc") << ");\n}\n";
                values[o.arg] = "red" + std::to_string(oi);
            }
            // the carried program, one column per thread
            const Program& q = *p.post;
            EmitCtx cx;
            cx.nv = 1;
            cx.arg_values = &values;
            s << "if (grp == 0 && n < DIM_N) {\nconst u32 n0 = n, m = 0u; (void)m;\n" << emit_exprs(q, cx);
            for (const Out& o : q.outs) s << "st_one(a" << o.arg << " + n0, e" << o.expr << "[0]);\n";
            s << "}\nreturn;\n}\n";
        }
        for (auto& jb : jobs) {
            const Out& o = p.outs[jb.oi];
            const int rop = (int)o.rop;
            s << "if (blockIdx.x >= " << jb.first << "u && blockIdx.x < " << jb.first + jb.blocks << "u) {\nconst u32 job = blockIdx.x - " << jb.first
              << "u;\nfloat acc = red_identity<" << rop << ">();\n";
            if (!o.fold_n) {
                const int FW = fold_width(o), FG = threads / FW;
                const int64_t arrivals = gy * o.b_div, slices = (N + FW - 1) / FW;
                s << "const u32 q = job / " << slices << "u, n = (job % " << slices << "u) * " << FW << "u + threadIdx.x % " << FW
                  << "u, grp = threadIdx.x / " << FW << "u;\nconst u32 tile_x = n / (TX * NV), within = n % (TX * NV);\nif (n < DIM_N) {\n"
                  << "for (u32 j0 = grp; j0 < " << arrivals << "u; j0 += " << FG * 8 << "u) {\nfloat pv[8];\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\n"
                  << "const u32 j = j0 + c * " << FG << "u;\npv[c] = j < " << arrivals << "u ? wsf[" << ws[jb.oi].foff << "ull + (size_t)((q * " << arrivals
                  << "u + j) * " << gx << "u + tile_x) * (TX * NV) + within] : red_identity<" << rop << ">();\n}\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) acc = red_op<"
                  << rop << ">(acc, pv[c]);\n}\n}\nfin_red[threadIdx.x] = acc;\n__syncthreads();\nif (grp == 0 && n < DIM_N) {\nfor (u32 g = 1; g < " << FG
                  << "u; g++) acc = red_op<" << rop << ">(acc, fin_red[g * " << FW << "u + threadIdx.x]);\na" << o.arg << "[(size_t)q * " << N << "ull + n] = " << scaled(o, "acc") << ";\n}\n";
            } else {
                const int64_t per = gx * gy * o.b_div;
                s << "for (u32 i0 = threadIdx.x; i0 < " << per << "u; i0 += " << threads * 8 << "u) {\nfloat pv[8];\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) {\n"
                  << "const u32 i = i0 + c * " << threads << "u;\npv[c] = i < " << per << "u ? wsf[" << ws[jb.oi].foff << "ull + (size_t)job * " << per
                  << "ull + i] : red_identity<" << rop << ">();\n}\n#pragma unroll\nfor (u32 c = 0; c < 8; c++) acc = red_op<" << rop << ">(acc, pv[c]);\n}\n"
                  << "fin_red[threadIdx.x] = acc;\n__syncthreads();\nif (threadIdx.x == 0) {\nfor (u32 t = 1; t < " << threads << "u; t++) acc = red_op<" << rop
                  << ">(acc, fin_red[t]);\na" << o.arg << "[job] = " << scaled(o, "acc") << ";\n}\n";
            }
            s << "return;\n}\n";
        }
        s << "}\n";
    }
    L.source = s.str();

    for (size_t oi = 0; oi < p.outs.size(); oi++) {
        const Out& o = p.outs[oi];
        if (o.reduce) {
            // rows wider than a block accumulate with atomics, from the operator's identity
            if (!(o.fold_n && !o.fold_m) || (gx == 1 && TX <= 64) || rows_meet_in_lds) continue;
            uint32_t bits = 0;
            float f = o.rop == ROp::Max ? -INFINITY : o.rop == ROp::Min ? INFINITY : 0.0f;
            memcpy(&bits, &f, 4);
            L.fills.push_back({o.arg, bits});
        } else if (o.dtype == HE_BOOL) {
            L.fills.push_back({o.arg, 0u});
        }
    }
    std::ostringstream d;
    d << "dims=[";
    for (int i = 0; i < n; i++) d << (i ? "x" : "") << p.dims[i];
    d << "] NV=" << NV << " TX=" << TX << " TY=" << TY << " RPT=" << RPT << " grid=" << L.grid << " threads=" << threads
      << " exprs=" << p.exprs.size() << " outs=" << p.outs.size() << " ws_floats=" << L.ws_floats << " ws_counters=" << L.ws_counters << " finalize_grid=" << L.finalize_grid;
    if (L.post_carried) d << " carries=" << p.post->exprs.size() << "exprs/" << p.post->outs.size() << "outs";
    d << " fills=[";
    for (size_t i = 0; i < L.fills.size(); i++) d << (i ? "," : "") << L.fills[i].first << ":" << L.fills[i].second;
    d << "]";
    L.describe = d.str();
    return L;
}

}  // namespace he::tp
