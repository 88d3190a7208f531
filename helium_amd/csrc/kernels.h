// Executable kernels built from tile programs: the pointwise/reduction instruction, anchor-less fusion-IR kernels
// and the fused GEMM.
#pragma once
#include <map>
#include <mutex>
#include <memory>

#include "rtc.h"
#include "tp.h"

namespace he {

// Fills each (pointer, (32-bit words, pattern)) buffer on `stream` with one kernel launch per 8 buffers.
void fill_buffers(const std::vector<std::pair<void*, std::pair<uint32_t, uint32_t>>>& fills, hipStream_t stream);

// What every generated kernel offers the C ABI: an ordered argument list, its source and a launch.
class KernelBase {
public:
    virtual ~KernelBase() = default;
    virtual const std::vector<tp::Arg>& args() const = 0;
    virtual const std::string& source() const = 0;
    virtual const std::string& describe() const = 0;
    // `ptrs[i]` is the device address of argument i.
    virtual void execute(void* const* ptrs, hipStream_t stream) = 0;
    // The same launches with the kernels' scratch (partial results, arrival counters) taken from `scratch`, a device
    // buffer of `scratch_bytes` bytes that the caller owns, instead of a buffer the kernel object allocates on its
    // first launch on a stream. Allocates no device memory; fails with HE_ERR_INVALID when the buffer is too small
    // or a code object is not loaded yet. Whatever must start at zero is cleared by a fill kernel ahead of the launch.
    virtual void execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) = 0;
    virtual size_t scratch_bytes_needed() const = 0;
    // Loads every code object of the kernel onto the current device.
    virtual void load() = 0;
    virtual bool loaded() const = 0;
};

// Loads the fill kernel's code object (fill_buffers otherwise loads it on its first use).
void load_fill_kernel();
bool fill_kernel_loaded();

// Device scratch of a kernel whose reductions span several blocks: per-block partials (floats) followed by arrival
// counters (u32). One buffer per stream the kernel has run on, because launches on one stream run in order and
// launches on different streams may overlap. The counters are cleared once, by a fill kernel ahead of the first
// launch on that stream; every launch leaves them at zero again.
class ReduceScratch {
public:
    struct Buf {
        float* floats;
        uint32_t* counters;
    };
    Buf get(uint64_t n_floats, uint64_t n_counters, hipStream_t stream);
    void release();

private:
    std::mutex mu_;
    std::map<hipStream_t, void*> per_stream_;
};

// A tile program compiled into one kernel launch, plus the fills its bitset outputs (and rows wider than a block)
// need and, for reductions of long launches, the small second launch that folds the blocks' partial results.
class TileKernel : public KernelBase {
public:
    TileKernel(tp::Program prog, const std::string& entry);
    const tp::Program& program() const { return prog_; }
    const tp::PointwiseLaunch& launch_info() const { return launch_; }
    const std::vector<tp::Arg>& args() const override { return prog_.args; }
    const std::string& source() const override { return launch_.source; }
    const std::string& describe() const override { return launch_.describe; }
    void execute(void* const* ptrs, hipStream_t stream) override;
    void execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) override;
    size_t scratch_bytes_needed() const override;
    void load() override;
    bool loaded() const override;
    ~TileKernel() override;

private:
    void run(void* const* ptrs, hipStream_t stream, ReduceScratch::Buf ws);
    tp::Program prog_;
    tp::PointwiseLaunch launch_;
    std::unique_ptr<JitKernel> kernel_, finalize_;
    ReduceScratch scratch_;
};

// Fused GEMM: C = f(A) g(B) with mainloop op chains applied while tiles are staged into LDS and the epilogue
// program applied to the f32 accumulators (helium-kernel-generator/src/generators/matmul.rs,
// helium-playground/src/kernel_generator.rs + templates/matmul.cu).
struct GemmProblem {
    int64_t batch = 1, M = 0, N = 0, K = 0;
    int mma_dtype = HE_BF16;       // multiplicand type: HE_BF16, HE_F16 or HE_F32
    tp::Program op_a, op_b, epi;   // dims [batch,M,K], [batch,K,N] ([batch,N,K] when b_nk), [batch,M,N]
    // B's source is contiguous along k (a transposed matrix, a convolution filter): its program iterates [batch,N,K],
    // its tile is staged and read like A's, with 16-byte chunks along k.
    bool b_nk = false;
    // A's source is contiguous along m (a transposed matrix): its program iterates [batch,K,M], its tile is staged
    // and read like a [k][n] B tile, with 16-byte chunks along m.
    bool a_km = false;
    // Implicit-GEMM convolution: the A operand is never materialised. Row m of A is output pixel (n, p, q), column k
    // is filter tap (r, s, c); the element is image[n][p*sh + r*dh - ph][q*sw + s*dw - pw][c], or zero outside the
    // image. op_a then only names the image argument.
    // `bwd` (ConvBackwardData): rows are input pixels (n, p, q) of the gradient being computed, the gathered tensor
    // is the incoming flow [N, H, W, C] (C = output channels of the forward op), and tap (r, s) of row (p, q) reads
    // flow[n][(p + ph - r*dh) / sh][(q + pw - s*dw) / sw][c] where both divisions are exact and in range.
    struct ConvGather {
        bool on = false, bwd = false;
        int64_t N = 0, H = 0, W = 0, C = 0, R = 0, S = 0, P = 0, Q = 0, sh = 1, sw = 1, dh = 1, dw = 1, ph = 0, pw = 0;
    } conv_a;
    // ConvBackwardFilter: B[k = output pixel (n, p, q)][n = tap (r, s, c)] is gathered from the image with the same
    // map as a forward convolution's A operand, transposed in role.
    ConvGather conv_b;
    // The k range is dealt to `split_k` workgroups per output tile (blockIdx.y); each writes its f32 partial tile to
    // scratch and a second launch adds them up. For products with few output tiles and a long k (a filter gradient:
    // 64 x 576 outputs, k = 200704). Needs batch == 1 and a plain epilogue (one full-size output, no reduction).
    int split_k = 1;
    // B rows that are not consecutive in memory: row k = rs * group + o lives at element o * o_stride + rs * rs_stride
    // (the filter [o][r][s][c] seen as the [(r, s, o)][c] matrix of ConvBackwardData). Columns stay contiguous.
    // With s_count > 0 only every few taps are used (one class of a strided data gradient): tap index rs = k / group
    // stands for tap (rs / s_count, rs % s_count) of the classes's own grid and the row lives at
    // o * o_stride + base + (rs / s_count) * r_stride + (rs % s_count) * s_stride.
    struct RowGather {
        bool on = false;
        int64_t group = 1, o_stride = 0, rs_stride = 0;
        int64_t s_count = 0, r_stride = 0, s_stride = 0, base = 0;
    } b_rows;
    // Output rows that are not consecutive in memory: row m = (n, p, q) over a P x Q grid is pixel (p * sh + a, q * sw + b)
    // of an H x W image of N-element pixels (one class of a strided data gradient writes every sh-th row and sw-th
    // column of the gradient). Needs a plain epilogue (one full-size output) and no split k range.
    struct OutRows {
        bool on = false;
        int64_t P = 0, Q = 0, H = 0, W = 0, sh = 1, sw = 1, a = 0, b = 0;
    } out_rows;
    int root_a = -1, root_b = -1;  // expression ids of the operand values in op_a / op_b
    std::vector<tp::Arg> args;     // the kernel's arguments: inputs in node order, then outputs in node order
    std::vector<int> map_a, map_b, map_e;  // program argument -> kernel argument
};
GemmProblem gemm_problem_from_fusion(const fir::OpGraph& g);
// Fills args / map_a / map_b / map_e from the three programs: distinct inputs in node order, then outputs.
void assemble_gemm_args(GemmProblem& pr);
// True when the B operand program (over [batch,K,N]) reads its largest source with unit stride along k and a
// larger one along n: lowering it over [batch,N,K] instead makes its accesses vectors.
bool operand_b_prefers_nk(const tp::Program& op_b);
// How many workgroups should share one output tile's k range: 1 unless 128x128 tiles leave most CUs idle and k is
// long enough to give every share at least eight 64-wide k-tiles. Only products with a plain epilogue may split.
int choose_split_k(int64_t M, int64_t N, int64_t K, int64_t batch);
// Throws HE_ERR_UNSUPPORTED for an epilogue program the GEMM kernel cannot run.
void validate_gemm_epilogue(const tp::Program& epi);

class GemmKernel : public KernelBase {
public:
    explicit GemmKernel(GemmProblem prob);
    const std::vector<tp::Arg>& args() const override { return prob_.args; }
    const std::string& source() const override { return source_; }
    const std::string& describe() const override { return describe_; }
    void execute(void* const* ptrs, hipStream_t stream) override;
    void execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) override;
    size_t scratch_bytes_needed() const override;
    void load() override;
    bool loaded() const override;
    const GemmProblem& problem() const { return prob_; }
    ~GemmKernel() override;

private:
    void run(void* const* ptrs, hipStream_t stream, float* ws, uint32_t* counters);
    GemmProblem prob_;
    std::string source_, describe_;
    // finalize_: adds up the partial tiles of a split-k product; reduce_: folds the partials of the epilogue's reductions
    std::unique_ptr<JitKernel> kernel_, finalize_, reduce_;
    uint32_t grid_[3] = {1, 1, 1};
    uint32_t threads_ = 256;
    uint32_t reduce_grid_ = 0;
    uint64_t reduce_floats_ = 0;
    uint64_t reduce_counters_ = 0;  // arrival counters of reductions that fold inside the kernel (no reduce_ launch then)
    std::vector<int> reduce_outs_;  // kernel arguments the reduce launch writes, in its parameter order
    bool reduce_all_args_ = false;  // the reduce launch carries a program and takes every epilogue argument instead
    ReduceScratch scratch_;
};

// Several kernels with one argument list, launched one after the other on the same stream (the classes of a strided
// data gradient). `zero_outputs_first`: the kernels do not write every element of the outputs; the rest is zero.
class CompositeKernel : public KernelBase {
public:
    CompositeKernel(std::vector<std::unique_ptr<KernelBase>> parts, bool zero_outputs_first);
    const std::vector<tp::Arg>& args() const override { return parts_[0]->args(); }
    const std::string& source() const override { return source_; }
    const std::string& describe() const override { return describe_; }
    void execute(void* const* ptrs, hipStream_t stream) override;
    void execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) override;
    size_t scratch_bytes_needed() const override;
    void load() override;
    bool loaded() const override;
    const std::vector<std::unique_ptr<KernelBase>>& parts() const { return parts_; }

private:
    void zero_outputs(void* const* ptrs, hipStream_t stream) const;
    std::vector<std::unique_ptr<KernelBase>> parts_;
    bool zero_first_;
    std::string source_, describe_;
};

// A convolution (or its filter gradient) over a 16-bit image of 3 or 4 channels, run over a repacked copy of the
// image. A chunk of 16 bytes is what one lane loads straight into LDS, and an image of 3 channels has no such chunk
// that lies in one filter tap, so its gather would go element by element through registers. The copy has 4 channels
// per pixel (the added ones zero) and the padding written out, which makes two neighbouring pixels one 8-channel
// "pixel" of an image of half the width: with an even stride along w the convolution is an ordinary one over that
// image, with ceil(S / 2) taps per filter row, no padding, and every chunk aligned. The filter is repacked the same
// way ([O, R, 2 * ceil(S / 2), 4], zero where the source has nothing); a filter gradient comes out in that layout and
// is unpacked. One launch repacks, the product runs, one launch unpacks (filter gradient only).
struct ConvRepack {
    bool filter_gradient = false;
    int64_t N = 0, H = 0, W = 0, C = 0;     // the image as the caller holds it
    int64_t Hp = 0, Wp = 0, ph = 0, pw = 0; // the copy: [N, Hp, Wp, 4]; pixel (h, w) of the image is pixel (h + ph, w + pw) of it
    int64_t O = 0, R = 0, S = 0, Sp = 0;    // filter [O, R, S, C] and its packed row length Sp (pixels)
    int image_arg = -1, filter_arg = -1;    // positions in the argument list (the filter gradient is the output)
    int elem_bytes = 2;                     // of the filter gradient (2 or 4); images and filters are 16-bit
};
class RepackedConvKernel : public KernelBase {
public:
    // `args`: the instruction's arguments; `inner`: the product over the repacked operands, same argument positions.
    RepackedConvKernel(std::vector<tp::Arg> args, ConvRepack geometry, std::unique_ptr<KernelBase> inner);
    const std::vector<tp::Arg>& args() const override { return args_; }
    const std::string& source() const override { return source_; }
    const std::string& describe() const override { return describe_; }
    void execute(void* const* ptrs, hipStream_t stream) override;
    void execute_in_scratch(void* const* ptrs, hipStream_t stream, void* scratch, size_t scratch_bytes) override;
    size_t scratch_bytes_needed() const override;
    void load() override;
    bool loaded() const override;
    ~RepackedConvKernel() override;

private:
    size_t own_bytes() const { return image_bytes_ + filter_bytes_; }
    void run(void* const* ptrs, hipStream_t stream, char* own, void* inner_scratch, size_t inner_scratch_bytes);
    std::vector<tp::Arg> args_;
    ConvRepack geo_;
    std::unique_ptr<KernelBase> inner_;
    std::string pack_source_, source_, describe_;
    std::unique_ptr<JitKernel> pack_, unpack_;
    size_t image_bytes_ = 0, filter_bytes_ = 0;  // of the packed copies (256-byte multiples)
    uint32_t pack_grid_ = 0, unpack_grid_ = 0;
    ReduceScratch scratch_;
};

}  // namespace he
