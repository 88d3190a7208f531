// C ABI for the two graph IRs and the tile-program kernels built from them.
#include <memory>

#include "fusion_ir.h"
#include "ir.h"
#include "kernels.h"

#include "capi_types.h"

namespace he {
ir::Op op_from_desc(const he_op_desc& d) {
    ir::Op op;
    HE_REQUIRE(d.kind >= 0 && d.kind <= HE_OP_CONSTANT, HE_ERR_INVALID, "bad op kind %d", d.kind);
    op.kind = (ir::OpKind)d.kind;
    HE_REQUIRE(d.num_inputs >= 0 && d.num_inputs <= 3, HE_ERR_INVALID, "bad input count");
    op.inputs.assign(d.inputs, d.inputs + d.num_inputs);
    static const int want_inputs[] = {2, 1, 2, 1, 1, 1, 1, 1, 2, 3, 2, 2, 2, 0};
    HE_REQUIRE(d.num_inputs == want_inputs[d.kind], HE_ERR_INVALID, "op kind %d takes %d inputs", d.kind,
               want_inputs[d.kind]);
    op.sub_op = d.sub_op;
    HE_REQUIRE(d.precision >= 0 && d.precision <= HE_PREC_F8_F16, HE_ERR_INVALID, "bad precision");
    op.precision = (ir::Precision)d.precision;
    op.target_type = d.target_type;
    op.depth = d.depth;
    op.new_dim_count = d.new_dim_count;
    for (int i = 0; i < d.num_broadcast_axes; i++)
        op.broadcast_axes.push_back({d.broadcast_axes[2 * i], d.broadcast_axes[2 * i + 1]});
    if (d.shape && d.shape_rank > 0) op.shape.assign(d.shape, d.shape + d.shape_rank);
    op.axis_a = d.axis_a;
    op.axis_b = d.axis_b;
    op.const_bits = d.const_bits;
    op.const_dtype = d.const_dtype;
    if (op.kind == ir::OpKind::Conv || op.kind == ir::OpKind::ConvBackwardData || op.kind == ir::OpKind::ConvBackwardFilter) {
        op.conv.in_channels = d.conv_in_channels;
        op.conv.out_channels = d.conv_out_channels;
        for (int i = 0; i < 2; i++) {
            op.conv.kernel[i] = d.conv_kernel[i];
            op.conv.stride[i] = d.conv_stride[i];
            op.conv.dilation[i] = d.conv_dilation[i];
            op.conv.input_size[i] = d.conv_input_size[i];
        }
        HE_REQUIRE(d.conv_padding_mode >= HE_PAD_SAME && d.conv_padding_mode <= HE_PAD_FULL, HE_ERR_INVALID, "bad padding mode");
        op.conv.padding_mode = d.conv_padding_mode;
    }
    if (op.kind == ir::OpKind::ChangeDataType || op.kind == ir::OpKind::Constant)
        (void)dtype_bits(op.kind == ir::OpKind::Constant ? op.const_dtype : op.target_type);
    return op;
}
}  // namespace he

extern "C" {

int he_graph_create(he_graph_t* graph) {
    return he::guard([&] { *graph = new he_graph_s(); });
}
int he_graph_destroy(he_graph_t graph) {
    delete graph;
    return HE_OK;
}
int he_graph_new_input(he_graph_t graph, const int64_t* shape, int rank, int dtype, uint32_t* node) {
    return he::guard([&] {
        HE_REQUIRE(graph && node && rank >= 0 && rank <= 16, HE_ERR_INVALID, "bad argument");
        (void)he::dtype_bits(dtype);
        *node = graph->g->new_input({he::ir::Shape(shape, shape + rank), dtype});
    });
}
int he_graph_new_op(he_graph_t graph, const he_op_desc* op, uint32_t* node) {
    return he::guard([&] {
        HE_REQUIRE(graph && op && node, HE_ERR_INVALID, "bad argument");
        *node = graph->g->new_op(he::op_from_desc(*op));
    });
}
int he_graph_new_output(he_graph_t graph, uint32_t from_node, uint32_t* node) {
    return he::guard([&] {
        HE_REQUIRE(graph && node, HE_ERR_INVALID, "bad argument");
        *node = graph->g->new_output(from_node);
    });
}
int he_graph_optimize(he_graph_t graph) {
    return he::guard([&] {
        std::lock_guard<std::mutex> lk(graph->mu);
        graph->prepared.reset();
        graph->g->optimize();
    });
}
int he_graph_num_nodes(he_graph_t graph, uint32_t* count) {
    return he::guard([&] { *count = (uint32_t)graph->g->num_nodes(); });
}
int he_graph_node_info(he_graph_t graph, uint32_t node, int32_t* kind, int32_t* dtype, int32_t* rank, int64_t* shape_out) {
    return he::guard([&] {
        const he::ir::Node& n = graph->g->get(node);
        HE_REQUIRE(n.desc.shape.size() <= 16, HE_ERR_INVALID, "rank too large");
        *kind = (int)n.kind;
        *dtype = n.desc.dtype;
        *rank = (int)n.desc.shape.size();
        for (size_t i = 0; i < n.desc.shape.size(); i++) shape_out[i] = n.desc.shape[i];
    });
}

int he_graph_node_op(he_graph_t graph, uint32_t node, he_op_desc* op, int64_t* axes_out, int64_t* shape_out, uint32_t* origin) {
    return he::guard([&] {
        HE_REQUIRE(graph && op && axes_out && shape_out && origin, HE_ERR_INVALID, "bad argument");
        const he::ir::Node& n = graph->g->get(node);
        *origin = graph->g->origin(node);
        *op = he_op_desc{};
        op->kind = -1;
        if (n.kind == he::ir::Node::Output) {
            op->inputs[0] = graph->g->inbound(node)[0];
            op->num_inputs = 1;
        }
        if (n.kind != he::ir::Node::Intermediate) return;
        const he::ir::Op& o = n.op;
        HE_REQUIRE(o.broadcast_axes.size() <= 16 && o.shape.size() <= 16, HE_ERR_INVALID, "rank too large");
        op->kind = (int)o.kind;
        op->num_inputs = (int)o.inputs.size();
        for (size_t i = 0; i < o.inputs.size(); i++) op->inputs[i] = o.inputs[i];
        op->sub_op = o.sub_op;
        op->precision = (int)o.precision;
        op->target_type = o.target_type;
        op->depth = o.depth;
        op->new_dim_count = o.new_dim_count;
        op->num_broadcast_axes = (int)o.broadcast_axes.size();
        for (size_t i = 0; i < o.broadcast_axes.size(); i++) {
            axes_out[2 * i] = o.broadcast_axes[i].axis;
            axes_out[2 * i + 1] = o.broadcast_axes[i].new_size;
        }
        op->broadcast_axes = axes_out;
        op->shape_rank = (int)o.shape.size();
        for (size_t i = 0; i < o.shape.size(); i++) shape_out[i] = o.shape[i];
        op->shape = shape_out;
        op->axis_a = o.axis_a;
        op->axis_b = o.axis_b;
        op->const_bits = o.const_bits;
        op->const_dtype = o.const_dtype;
        op->conv_in_channels = o.conv.in_channels;
        op->conv_out_channels = o.conv.out_channels;
        for (int i = 0; i < 2; i++) {
            op->conv_kernel[i] = o.conv.kernel[i];
            op->conv_stride[i] = o.conv.stride[i];
            op->conv_dilation[i] = o.conv.dilation[i];
            op->conv_input_size[i] = o.conv.input_size[i];
        }
        op->conv_padding_mode = o.conv.padding_mode;
    });
}
int he_graph_capacity(he_graph_t graph, uint32_t* capacity) {
    return he::guard([&] { *capacity = (uint32_t)graph->g->capacity(); });
}

int he_pointwise_supports(he_graph_t graph, const uint32_t* nodes, int num_nodes, int* supported) {
    return he::guard([&] {
        he::ir::OpSubgraph sg(graph->g, std::vector<he::ir::NodeId>(nodes, nodes + num_nodes));
        *supported = he::tp::pointwise_supports(sg) ? 1 : 0;
    });
}
int he_pointwise_create(he_tile_kernel_t* kernel, he_graph_t graph, const uint32_t* nodes, int num_nodes) {
    return he::guard([&] {
        HE_REQUIRE(kernel && graph && nodes && num_nodes > 0, HE_ERR_INVALID, "bad argument");
        he::ir::OpSubgraph sg(graph->g, std::vector<he::ir::NodeId>(nodes, nodes + num_nodes));
        auto k = std::make_unique<he_tile_kernel_s>();
        k->k.reset(new he::TileKernel(he::tp::lower_pointwise(sg), "pointwise_kernel"));
        if (he::device_initialised()) k->k->load();  // so that later launches need not
        *kernel = k.release();
    });
}
int he_aux_kernel_create(he_tile_kernel_t* kernel, he_fgraph_t graph) {
    return he::guard([&] {
        HE_REQUIRE(kernel && graph, HE_ERR_INVALID, "bad argument");
        auto k = std::make_unique<he_tile_kernel_s>();
        k->k.reset(new he::TileKernel(he::tp::lower_aux(graph->g), "fused_auxiliary"));
        if (he::device_initialised()) k->k->load();  // so that later launches need not
        *kernel = k.release();
    });
}
int he_fused_kernel_create(he_tile_kernel_t* kernel, he_fgraph_t graph) {
    return he::guard([&] {
        HE_REQUIRE(kernel && graph, HE_ERR_INVALID, "bad argument");
        auto k = std::make_unique<he_tile_kernel_s>();
        if (graph->g.anchor() == he::fir::kNoOpNode)
            k->k.reset(new he::TileKernel(he::tp::lower_aux(graph->g), "fused_auxiliary"));
        else
            k->k.reset(new he::GemmKernel(he::gemm_problem_from_fusion(graph->g)));
        if (he::device_initialised()) k->k->load();  // so that later launches need not
        *kernel = k.release();
    });
}
int he_tile_kernel_num_args(he_tile_kernel_t kernel, int* count) {
    return he::guard([&] { *count = (int)kernel->k->args().size(); });
}
int he_tile_kernel_arg_info(he_tile_kernel_t kernel, int index, uint64_t* node, int32_t* is_output, int32_t* dtype,
                            int64_t* numel) {
    return he::guard([&] {
        const auto& args = kernel->k->args();
        HE_REQUIRE(index >= 0 && index < (int)args.size(), HE_ERR_INVALID, "argument index out of range");
        *node = args[index].node;
        *is_output = args[index].is_output;
        *dtype = args[index].dtype;
        *numel = args[index].numel;
    });
}
int he_tile_kernel_execute(he_tile_kernel_t kernel, void* const* arg_ptrs, int num_args, he_stream_t stream) {
    return he::guard([&] {
        HE_REQUIRE(kernel && arg_ptrs, HE_ERR_INVALID, "bad argument");
        HE_REQUIRE(num_args == (int)kernel->k->args().size(), HE_ERR_INVALID, "kernel takes %zu arguments, got %d",
                   kernel->k->args().size(), num_args);
        kernel->k->execute(arg_ptrs, stream ? stream->s : nullptr);
    });
}
const char* he_tile_kernel_source(he_tile_kernel_t kernel) { return kernel ? kernel->k->source().c_str() : ""; }
const char* he_tile_kernel_describe(he_tile_kernel_t kernel) {
    return kernel ? kernel->k->describe().c_str() : "";
}
int he_tile_kernel_destroy(he_tile_kernel_t kernel) {
    delete kernel;
    return HE_OK;
}

int he_fgraph_create(he_fgraph_t* graph) {
    return he::guard([&] { *graph = new he_fgraph_s(); });
}
int he_fgraph_destroy(he_fgraph_t graph) {
    delete graph;
    return HE_OK;
}
int he_fgraph_insert(he_fgraph_t graph, const he_fop_desc* d, uint64_t* node) {
    return he::guard([&] {
        HE_REQUIRE(graph && d && node, HE_ERR_INVALID, "bad argument");
        HE_REQUIRE(d->kind >= 0 && d->kind <= HE_FOP_CONSUMER, HE_ERR_INVALID, "bad fusion-IR op kind %d", d->kind);
        he::fir::Op op;
        op.kind = (he::fir::OpKind)d->kind;
        op.shape = {d->shape[0], d->shape[1], d->shape[2]};
        op.value = d->value;
        op.a = d->a;
        op.b = d->b;
        op.sub_op = d->sub_op;
        op.constant = d->constant;
        HE_REQUIRE(d->depth >= 0 && d->depth <= HE_FRED_BATCH, HE_ERR_INVALID, "bad reduction depth");
        op.depth = (he::fir::ReductionDepth)d->depth;
        op.axis = d->axis;
        op.amount = d->amount;
        op.dtype = d->dtype;
        if (op.kind == he::fir::OpKind::Producer || op.kind == he::fir::OpKind::Consumer) (void)he::dtype_bits(op.dtype);
        *node = (*node == UINT64_MAX) ? graph->g.insert(op) : graph->g.insert_with_id(*node, op);
    });
}
int he_fgraph_shape(he_fgraph_t graph, uint64_t node, uint32_t shape_out[3]) {
    return he::guard([&] {
        const he::fir::Shape3& s = graph->g.shape(node);
        shape_out[0] = s[0];
        shape_out[1] = s[1];
        shape_out[2] = s[2];
    });
}

}  // extern "C"
