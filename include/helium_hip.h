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


/* ==================================================================================================
 * 3. helium-ir operation graph — the structure helium/src/raw_tensor.rs records and hands to the backend
 *    (helium-ir/src/opgraph.rs, opgraph/op.rs, opgraph/subgraph.rs). Node ids are indices in creation order.
 * ================================================================================================== */
typedef struct he_graph_s* he_graph_t;

/* OpKind, same order as helium-ir/src/opgraph/op.rs:15-30. */
enum {
    HE_OP_MATMUL = 0, HE_OP_UNARY, HE_OP_BINARY, HE_OP_CHANGE_DTYPE, HE_OP_REDUCE, HE_OP_BROADCAST, HE_OP_RESHAPE,
    HE_OP_SWAP_DIMS, HE_OP_COMPARE, HE_OP_SELECT, HE_OP_CONV, HE_OP_CONV_BWD_DATA, HE_OP_CONV_BWD_FILTER,
    HE_OP_CONSTANT
};
/* UnaryPointwiseOp (op.rs:291-304) */
enum { HE_UN_RECIP = 0, HE_UN_NEG, HE_UN_EXP, HE_UN_SIN, HE_UN_COS, HE_UN_TAN, HE_UN_SIGMOID, HE_UN_TANH,
       HE_UN_RELU, HE_UN_SQRT, HE_UN_LOG };
/* BinaryPointwiseOp (op.rs:315-328) */
enum { HE_BIN_ADD = 0, HE_BIN_MUL, HE_BIN_POW, HE_BIN_MIN, HE_BIN_MAX, HE_BIN_AND, HE_BIN_OR, HE_BIN_XOR };
/* ReduceOp (op.rs:360-367) */
enum { HE_RED_SUM = 0, HE_RED_MEAN, HE_RED_MAX, HE_RED_MIN };
/* CompareOp (op.rs:429-437) */
enum { HE_CMP_EQ = 0, HE_CMP_NE, HE_CMP_LT, HE_CMP_LE, HE_CMP_GT, HE_CMP_GE };
/* Precision (op/precision.rs:36-81) */
enum { HE_PREC_F32_F32 = 0, HE_PREC_TF32_F32, HE_PREC_BF16_F32, HE_PREC_F16_F32, HE_PREC_F16_F16,
       HE_PREC_F8_F32, HE_PREC_F8_F16 };

/* One `Op` value (op.rs:15-30 and the structs below it). Only the fields of the given kind are read.
 *   inputs: Matmul a,b | Unary x | Binary/Compare lhs,rhs | Select lhs,rhs,selector | others x          */
typedef struct he_op_desc {
    int32_t kind;
    uint32_t inputs[3];
    int32_t num_inputs;
    int32_t sub_op;         /* HE_UN_* / HE_BIN_* / HE_RED_* / HE_CMP_* */
    int32_t precision;      /* Matmul: HE_PREC_* */
    int32_t target_type;    /* ChangeDataType */
    uint32_t depth;         /* Reduce: number of trailing dims folded */
    int64_t new_dim_count;  /* Broadcast */
    const int64_t* broadcast_axes; /* Broadcast: (axis, new_size) pairs */
    int32_t num_broadcast_axes;
    const int64_t* shape;   /* Reshape target shape / Constant shape */
    int32_t shape_rank;
    int64_t axis_a, axis_b; /* SwapDims */
    uint32_t const_bits;    /* Constant: the scalar's bit pattern in const_dtype */
    int32_t const_dtype;
    /* Conv (inputs image, filter), ConvBackwardData (flow, filter), ConvBackwardFilter (flow, image): Conv2dParams
     * (opgraph/op/conv.rs:5-12); images are NHWC, filters [out_channels, kh, kw, in_channels] (op.rs:123-173) */
    int64_t conv_in_channels, conv_out_channels;
    int64_t conv_kernel[2], conv_stride[2], conv_dilation[2];
    int32_t conv_padding_mode;     /* HE_PAD_* */
    int64_t conv_input_size[2];    /* ConvBackwardData::input_size */
} he_op_desc;
/* PaddingMode (conv.rs:76-81) */
enum { HE_PAD_SAME = 0, HE_PAD_VALID = 1, HE_PAD_FULL = 2 };

int he_graph_create(he_graph_t* graph);                                       /* OpGraph::new (opgraph.rs:21-23) */
int he_graph_destroy(he_graph_t graph);
int he_graph_new_input(he_graph_t graph, const int64_t* shape, int rank, int dtype, uint32_t* node); /* :66-70 */
int he_graph_new_op(he_graph_t graph, const he_op_desc* op, uint32_t* node);  /* new_op + shape inference :73-86 */
int he_graph_new_output(he_graph_t graph, uint32_t from_node, uint32_t* node); /* :89-100 */
int he_graph_optimize(he_graph_t graph);                                      /* prune_unused :165-191 */
int he_graph_num_nodes(he_graph_t graph, uint32_t* count);
/* Descriptor of a node (opgraph.rs:240-246). shape_out must hold 16 entries. kind: 0 input, 1 intermediate, 2 output. */
int he_graph_node_info(he_graph_t graph, uint32_t node, int32_t* kind, int32_t* dtype, int32_t* rank, int64_t* shape_out);
/* Reads a node back: the counterpart of he_graph_new_op. `op->kind` is -1 for an Input or Output node (an Output's
 * source is inputs[0]); `op->broadcast_axes` and `op->shape` point into axes_out (32 entries) and shape_out (16).
 * `origin`: for a graph that he_plan_graph returned, the node of the planned graph this node stands for; the node itself
 * otherwise. he_graph_capacity: one more than the largest node id ever given out (ids of pruned nodes stay unused). */
int he_graph_node_op(he_graph_t graph, uint32_t node, he_op_desc* op, int64_t* axes_out, int64_t* shape_out, uint32_t* origin);
int he_graph_capacity(he_graph_t graph, uint32_t* capacity);

/* ==================================================================================================
 * 4. Pointwise / reduction instruction — helium/src/cuda/instr/pointwise.rs + pointwise/jit.rs (kernels K2, K3).
 * ================================================================================================== */
typedef struct he_tile_kernel_s* he_tile_kernel_t;

/* supports_subgraph (pointwise.rs:121-186) for the subgraph made of `nodes`. */
int he_pointwise_supports(he_graph_t graph, const uint32_t* nodes, int num_nodes, int* supported);
/* PointwiseGraph::new + precompile (pointwise.rs:35-54): lowers the subgraph, generates and compiles its kernel. */
int he_pointwise_create(he_tile_kernel_t* kernel, he_graph_t graph, const uint32_t* nodes, int num_nodes);
/* Kernel arguments: the subgraph's inputs in id order, then its leafs in id order. */
int he_tile_kernel_num_args(he_tile_kernel_t kernel, int* count);
int he_tile_kernel_arg_info(he_tile_kernel_t kernel, int index, uint64_t* node, int32_t* is_output, int32_t* dtype,
                            int64_t* numel);
/* PointwiseGraph::execute (pointwise.rs:57-86): fills reduction / bitset outputs, then one launch. */
int he_tile_kernel_execute(he_tile_kernel_t kernel, void* const* arg_ptrs, int num_args, he_stream_t stream);
/* The same launches without any allocation. No counterpart in the reference; for callers that cannot allocate:
 * code under HIP graph capture, tight serving loops, harnesses that forbid it. The kernels' scratch (per-workgroup
 * partial results and arrival counters of reductions, partial tiles of a split product) lies in a device array of
 * HE_NOALLOC_SCRATCH_BYTES that is part of the library and is resolved per device by he_init; a kernel that needs more
 * is refused with HE_ERR_INVALID. The call makes no hipMalloc / hipFree and loads no code object: the kernel must
 * have been created after he_init (creation then loads its code) or have run once through he_tile_kernel_execute.
 * All calls on a device share the one array: calls that overlap on a device (other streams, other threads) race. */
#define HE_NOALLOC_SCRATCH_BYTES (8u << 20)
int he_tile_kernel_execute_noalloc(he_tile_kernel_t kernel, void* const* arg_ptrs, int num_args, he_stream_t stream);
const char* he_tile_kernel_source(he_tile_kernel_t kernel);
const char* he_tile_kernel_describe(he_tile_kernel_t kernel);
int he_tile_kernel_destroy(he_tile_kernel_t kernel);

/* ==================================================================================================
 * 5. Fusion IR — helium-playground/src/opgraph.rs: 3-d [batch, rows, cols] shapes, Core = Matmul with Mainloop
 *    and Epilogue op lists, or anchor-less auxiliary fusions.
 * ================================================================================================== */
typedef struct he_fgraph_s* he_fgraph_t;

/* Op variants (opgraph.rs:264-301) */
enum { HE_FOP_PRODUCER = 0, HE_FOP_CONSTANT, HE_FOP_MATMUL, HE_FOP_UNARY, HE_FOP_REDUCTION, HE_FOP_BINARY,
       HE_FOP_BROADCAST, HE_FOP_TRANSPOSE, HE_FOP_CONSUMER };
/* UnaryPointwiseOp (opgraph.rs:317-328) */
enum { HE_FUN_NEG = 0, HE_FUN_RELU, HE_FUN_GELU, HE_FUN_TANH, HE_FUN_EXP, HE_FUN_LN, HE_FUN_SQRT, HE_FUN_ADD_CONSTANT,
       HE_FUN_MUL_CONSTANT, HE_FUN_POW_CONSTANT };
/* BinaryPointwiseOp (opgraph.rs:330-338) */
enum { HE_FBIN_ADD = 0, HE_FBIN_SUB, HE_FBIN_MUL, HE_FBIN_DIV, HE_FBIN_POW, HE_FBIN_DRELU };
/* ReductionDepth (opgraph.rs:309-314) */
enum { HE_FRED_ROWS = 0, HE_FRED_COLUMNS, HE_FRED_ITEM, HE_FRED_BATCH };

typedef struct he_fop_desc {
    int32_t kind;          /* HE_FOP_* */
    uint32_t shape[3];     /* Producer / Constant */
    float value;           /* Constant */
    uint64_t a, b;         /* Matmul a,b | Binary lhs,rhs | Unary/Reduction/Broadcast/Transpose/Consumer x in a */
    int32_t sub_op;        /* HE_FUN_* / HE_FBIN_* */
    float constant;        /* AddConstant / MulConstant / PowConstant */
    int32_t depth;         /* Reduction: HE_FRED_* (the op is always Sum, opgraph.rs:303-306) */
    uint32_t axis, amount; /* Broadcast */
    int32_t dtype;         /* Producer / Consumer storage type (the reference's kernels assume bf16) */
} he_fop_desc;

int he_fgraph_create(he_fgraph_t* graph);                                  /* OpGraph::new (opgraph.rs:29-31) */
int he_fgraph_destroy(he_fgraph_t graph);
/* OpGraph::insert (opgraph.rs:33-57). With *node == UINT64_MAX on entry the id is assigned in insertion order,
 * otherwise the given id is used (to rebuild a printed fusion with its own numbering). */
int he_fgraph_insert(he_fgraph_t graph, const he_fop_desc* op, uint64_t* node);
int he_fgraph_shape(he_fgraph_t graph, uint64_t node, uint32_t shape_out[3]);

/* KernelGenerator::new + generate for an anchor-less fusion (kernel_generator.rs:22-49,98-115; template
 * templates/auxiliary.cu). Arguments: producers in id order, then leaves in id order (:52-63,138-148). */
int he_aux_kernel_create(he_tile_kernel_t* kernel, he_fgraph_t graph);
/* KernelGenerator::new + generate for any fusion (kernel_generator.rs:22-117): with a Matmul anchor the fused
 * GEMM (templates/matmul.cu's role: mainloop ops while tiles are staged, epilogue ops and reductions on the
 * accumulators), otherwise the auxiliary kernel. Arguments: producers in id order, then leaves in id order. */
int he_fused_kernel_create(he_tile_kernel_t* kernel, he_fgraph_t graph);


/* MatmulGenerator::new + generate (helium-kernel-generator/src/generators/matmul.rs:88-153) for the Matmul-anchored
 * subgraph made of `nodes` of a helium-ir graph; HE_ERR_UNSUPPORTED stands for Err(UnsupportedFusion). The kernel's
 * arguments are A, B, then the output, the order CompiledKernel::execute passes them (:181-219). */
int he_matmul_kernel_create(he_tile_kernel_t* kernel, he_graph_t graph, const uint32_t* nodes, int num_nodes);

/* ==================================================================================================
 * 6. Backend: tensors, plan generation and graph execution — helium/src/backend.rs, backend/plan_generation.rs,
 *    helium/src/cuda.rs, cuda/tensor_storage.rs, cuda/allocator/.
 * ================================================================================================== */
typedef struct he_tensor_s* he_tensor_t;
typedef struct he_plan_s* he_plan_t;

/* Backend::create_tensor_with_data (backend.rs:21-22, cuda.rs:62-79): asynchronous upload through pinned memory on
 * a dedicated stream; the tensor's ready event is recorded behind it. `len` counts elements (bits for Bool). */
int he_tensor_create_with_data(he_tensor_t* tensor, const void* data, int dtype, size_t len);
/* Backend::download_tensor (backend.rs:24-29, cuda.rs:81-96), blocking form: waits for the ready event, copies
 * the tensor's storage to `dst` and returns when the copy is done. */
int he_tensor_download(he_tensor_t tensor, void* dst);
int he_tensor_info(he_tensor_t tensor, int32_t* dtype, uint64_t* len, uint64_t* bytes, void** device_ptr);
/* Drops one reference (TensorStorage is reference counted, tensor_storage.rs:30-42). */
int he_tensor_free(he_tensor_t tensor);

/* generate_plan (plan_generation.rs:22-26) for the graph as it stands; the graph must outlive the plan. */
int he_plan_generate(he_graph_t graph, he_plan_t* plan);
/* The graph the plan's instructions are made of, as a new graph the caller destroys: the planned graph itself, or the
 * form the backend's rewrites gave it (HE_OPT_CANCEL_TRANSPOSES, HE_OPT_REMATERIALIZE). Instructions and
 * he_plan_describe name nodes of the planned graph (he_graph_node_op's `origin`). */
int he_plan_graph(he_plan_t plan, he_graph_t* graph);
int he_plan_num_steps(he_plan_t plan, int* steps);
/* One line per step: "step i: kind{node,node,...} ... | release node ...". */
const char* he_plan_describe(he_plan_t plan);
/* The same text with the node ids of the graph he_plan_graph returns. */
const char* he_plan_describe_planned(he_plan_t plan);
/* The compiled kernel of instruction `index` of the plan (instructions counted in the order he_plan_describe lists them),
 * for inspection and tests: its arguments name nodes of the graph he_plan_graph returns. An instruction whose kernel also
 * does the work of a later, small one (the per-channel arithmetic behind a batch norm's sums rides on the launch that
 * folds them) lists that one's tensors among its arguments; the later one, like a permute instruction, has no kernel of
 * this kind and gives HE_ERR_INVALID. The handle shares the kernel with the plan; destroy it like any other. No
 * counterpart in the reference (its instructions are not inspectable). */
int he_plan_instruction_kernel(he_plan_t plan, int index, he_tile_kernel_t* kernel);
/* Compiles the kernels of every instruction of the plan, in parallel, into the kernel caches: what begin_execute does
 * on first sight of a plan (cuda.rs:98-139, parallel_compile_kernels :262-270). Needs no device. */
int he_plan_precompile(he_plan_t plan);
int he_plan_destroy(he_plan_t plan);

/* BackendExt::execute_graph (backend.rs:40-80): prunes a copy of the graph, takes the cached plan, compiles its
 * kernels, and runs the steps over a pool of streams. input_tensors[i] is the storage of Input node input_nodes[i].
 * On return output_nodes / output_tensors hold one (Output node, tensor) pair per Output node of the graph; each
 * tensor is a new reference the caller frees. */
int he_execute_graph(he_graph_t graph, const uint32_t* input_nodes, const he_tensor_t* input_tensors, int num_inputs,
                     uint32_t* output_nodes, he_tensor_t* output_tensors, int max_outputs, int* num_outputs);
/* ---- 7. Fusion search over a fusion-IR graph ------------------------------------------------------------
 * helium-playground/src/fused_graph.rs (FusedGraph: identity, enumerate_possible_actions, apply_action,
 * produce_maximal_fusions, clean, topo_sort), cost_model.rs (naive_cost_function, analytical_cost_function,
 * minimize_cost_function) and subdivision.rs (subdivide). The plan holds the chosen Core(mainloop, anchor, epilogue)
 * and Aux fusions; each becomes one kernel (he_fused_kernel_create's generators) and he_fusion_plan_execute runs
 * them in dependency order with pooled temporaries. */
typedef struct he_fusion_plan_s* he_fusion_plan_t;
/* HE_FUSE_MIN_ANALYTICAL_COST is analytical_cost_function with the coefficients its authors fitted on their hardware
 * (cost_model.rs:200-207); HE_FUSE_MIN_MI355X_COST is the model of the same purpose fitted to this backend's kernels on
 * MI355X (terms: launches, matrix-core FLOP, L2->CU bytes of operands a mainloop fusion adds, HBM bytes, vector ops). */
enum { HE_FUSE_MAXIMAL = 0, HE_FUSE_MIN_NAIVE_COST = 1, HE_FUSE_MIN_ANALYTICAL_COST = 2, HE_FUSE_MIN_MI355X_COST = 3 };
enum { HE_FUSION_ROLE_MAINLOOP = 0, HE_FUSION_ROLE_EPILOGUE = 1, HE_FUSION_ROLE_ANCHOR = 2, HE_FUSION_ROLE_AUX = 3 };
/* objective HE_FUSE_MAXIMAL: produce_maximal_fusions only (fused_graph.rs:113-223); otherwise minimize_cost_function
 * (cost_model.rs:256-343) with the naive model on MI355X rates or the analytical model. */
int he_fusion_search(he_fgraph_t graph, int objective, he_fusion_plan_t* plan);
/* minimize_cost_function_with_subdivision (cost_model.rs:241-259): subdivide, search each subdivision's subgraph
 * (OpGraph::subgraph, opgraph.rs:96-178) on its own, then FusedGraph::merge_from_subdivisions
 * (fused_graph.rs:910-1058). The plan is used like he_fusion_search's. */
int he_fusion_search_subdivided(he_fgraph_t graph, int objective, he_fusion_plan_t* plan);
int he_fusion_plan_num_fusions(he_fusion_plan_t plan, int* count);   /* kernels, in execution order */
int he_fusion_plan_fusion_info(he_fusion_plan_t plan, int index, int32_t* is_core, uint64_t* anchor, uint64_t* nodes,
                               int32_t* roles, int capacity, int* count);
const char* he_fusion_plan_describe(he_fusion_plan_t plan);           /* FusedGraph::print (fused_graph.rs:1060-1068) */
/* objective 1: naive model (reference_constants != 0: the constants of cost_model.rs:10-12), 2: analytical model, 3: the
 * MI355X model (seconds) */
int he_fusion_plan_cost(he_fusion_plan_t plan, int objective, int reference_constants, double* cost, uint64_t* states_visited);
/* The MI355X model's terms for the plan, in the order: launches, matrix-core FLOP, L2->CU bytes of extra mainloop
 * operands, weighted mainloop ops, HBM bytes, weighted epilogue ops, weighted ops of anchor-less kernels. The model is
 * linear in them, which is what its fit uses. No counterpart in the reference (its coefficients are constants in
 * cost_model.rs:200-207 with no code that derived them). */
int he_fusion_plan_cost_terms(he_fusion_plan_t plan, double* terms, int capacity, int* count);
int he_fusion_plan_precompile(he_fusion_plan_t plan);
/* Producers and Consumers of the whole graph are bound by node id; values between kernels are bf16 (f32 for
 * reductions) in pooled device memory. */
int he_fusion_plan_execute(he_fusion_plan_t plan, const uint64_t* producer_nodes, void* const* producer_ptrs, int num_producers,
                           const uint64_t* consumer_nodes, void* const* consumer_ptrs, int num_consumers, he_stream_t stream);
int he_fusion_plan_destroy(he_fusion_plan_t plan);
/* subdivide (subdivision.rs:24-113): entry k is node nodes[k] as portion portions[k] (0 mainloop, 1 epilogue, 2 full)
 * of subdivision subdivision_of[k]. */
int he_fgraph_subdivide(he_fgraph_t graph, uint64_t* nodes, int32_t* portions, int32_t* subdivision_of, int capacity, int* count);

/* Backend options. HE_OPT_FUSE_MATMUL_EPILOGUE (default 1): pointwise / reduce ops that follow a Matmul join its
 * instruction and run as the fused GEMM's epilogue (the MatmulGenerator path, matmul.rs:88-130), and a SwapDims of the
 * two matrix dims that feeds only a Matmul joins it as a transposed operand; the same holds for a Conv, and a
 * SwapDims + Reduce that folds all rows of the product (column sums, BatchNorm2d statistics of a convolution's output)
 * joins as a column reduction of the epilogue; 0 restores the grouping of
 * helium/src/cuda/instr/cudnn_graph.rs:319-321, where a matmul or convolution instruction never fuses.
 * HE_OPT_FOLD_SWAP_INTO_REDUCE (default 1): a SwapDims above the 1M-element threshold of cuda.rs:38-41 whose values
 * all end in Reduce ops (BatchNorm2d statistics, column sums) stays in the pointwise instruction, which then folds the
 * leading dims of the untransposed tensor in one pass; 0 makes it a permute instruction as the reference does.
 * HE_OPT_REMATERIALIZE (default 1): pointwise / shape ops whose value depends on at most one tensor of their own size
 * (the rest being broadcasts of small tensors) are planned once per consumer, so that every copy fuses into the kernel
 * that uses it and the value never travels through memory - a batch norm's forward pass as the reference records it
 * (modules/batch_norm.rs:53-71) otherwise leaves eight full-size intermediates for the backward pass. The rewritten
 * graph is used only when its plan moves fewer bytes; he_plan_describe names copies by the nodes they stand for. 0 plans
 * the graph as recorded, like plan_generation.rs.
 * HE_OPT_CANCEL_TRANSPOSES (default 1): a SwapDims is moved towards the producers of its operand (through pointwise ops,
 * into broadcasts and constants) and dropped where on every path it meets the SwapDims it undoes, so the pointwise ops
 * between the two run in the layout the tensors have in memory; the chain of SwapDims in front of a Reduce becomes the
 * shortest chain that reduces the same dims. The backward pass of a reduction over leading dims (tensor.rs answers a
 * SwapDims with a SwapDims) otherwise transposes a full-size tensor twice. Applied before HE_OPT_REMATERIALIZE, under
 * the same condition (no more bytes moved by the plan); 0 keeps every SwapDims as recorded.
 * HE_OPT_HOIST_BROADCASTS (default 1): a pointwise op whose operands all are the same Broadcast of small tensors (or
 * Constants) is applied to the small tensors and its result broadcast - `(variance.broadcast_to(x.shape) + 1e-3).sqrt()`
 * (modules/batch_norm.rs:56) costs one square root per channel instead of one per element. 0 keeps the ops where they
 * were recorded.
 * HE_OPT_STREAM_FAN_OUT (default 1): how the independent instructions of a plan step are spread over the calling
 * thread's streams. 2: every step with several instructions fans out and the next step waits for all of its streams
 * (helium/src/cuda.rs:190-221). 1: only steps whose instructions are too small to fill the device and numerous enough to
 * outweigh the joins (each costs the host 15-20 us here); all others run on the first stream in plan order. 0: one
 * stream. Takes effect from the next he_execute_graph; results do not depend on it. */
enum { HE_OPT_FUSE_MATMUL_EPILOGUE = 0, HE_OPT_FOLD_SWAP_INTO_REDUCE = 1, HE_OPT_REMATERIALIZE = 2, HE_OPT_CANCEL_TRANSPOSES = 3,
       HE_OPT_HOIST_BROADCASTS = 4, HE_OPT_STREAM_FAN_OUT = 5 };
int he_backend_set_option(int option, int64_t value);

/* Counters of the last he_execute_graph on this thread: [0] steps run, [1] instructions, [2] streams used,
 * [3] event waits; and of the process: [4] plan-cache hits, [5] misses, [6] bytes held from the driver,
 * [7] driver allocations, [8] pooled reuses. */
int he_backend_stats(uint64_t stats[9]);

/* ---- device memory pool ------------------------------------------------------------------------------------------
 * helium/src/cuda/allocator/block.rs (BlockAllocator: best-fit free blocks, coalescing, logical allocation streams)
 * and allocator/device.rs (DeviceAllocator: pages from the driver, never returned). The block allocator is pure host
 * logic over address ranges and needs no device. */
typedef struct he_block_allocator_s* he_block_allocator_t;
typedef struct he_block {
    uint32_t page;
    uint64_t start, size;
    uint64_t streams[8]; /* streams whose device work may still touch the block (Block::in_use_by_streams) */
    int32_t num_streams;
} he_block;
int he_block_allocator_create(he_block_allocator_t* allocator);            /* BlockAllocator::new, block.rs:17-19 */
int he_block_allocator_destroy(he_block_allocator_t allocator);
int he_block_allocator_add_page(he_block_allocator_t allocator, uint64_t size, uint32_t* page); /* add_page :22-34 */
/* allocate (block.rs:37-118); stream 0 = None. *found = 0 when no free block fits (the Rust None). */
int he_block_allocator_allocate(he_block_allocator_t allocator, uint64_t size, uint64_t align, uint64_t stream,
                                he_block* block, int* found);
int he_block_allocator_deallocate(he_block_allocator_t allocator, const he_block* block);       /* :124-127 */
int he_block_allocator_begin_stream(he_block_allocator_t allocator, uint64_t parent, uint64_t* stream); /* :216-231 */
int he_block_allocator_end_stream(he_block_allocator_t allocator, uint64_t stream);                    /* :233-244 */
/* [0] free blocks, [1] free bytes, [2] largest free block, [3] live streams; also checks the allocator's indices
 * against each other and fails with HE_ERR_INTERNAL if they disagree. */
int he_block_allocator_stats(he_block_allocator_t allocator, uint64_t stats[4]);

/* DeviceAllocator (allocator/device.rs): begin_stream / end_stream (:78-89), allocate_in_stream (:66-73; scope 0 =
 * allocate, :57-59) and the drop of a DeviceMemory (:181-185). `thread` is any non-zero token of the calling host
 * thread whose scopes run one after the other on the device (0: none); he_pool_end_scope is for a caller that knows
 * the scope's device work has finished. */
int he_pool_begin_scope(uint64_t thread, uint64_t* scope);
int he_pool_end_scope(uint64_t scope);
int he_pool_allocate(size_t bytes, uint64_t scope, void** ptr, he_block* block);
int he_pool_release(void* ptr, const he_block* block, uint64_t scope);

#ifdef __cplusplus
}
#endif
#endif /* HELIUM_HIP_H */
