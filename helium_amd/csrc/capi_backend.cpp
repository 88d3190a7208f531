// C ABI of the backend layer: tensors, plans, execute_graph.
#include <future>
#include "exec.h"

#include "capi_types.h"

struct he_tensor_s {
    he::exec::TensorRef t;
};
struct he_plan_s {
    std::shared_ptr<const he::plan::Plan> plan;
    std::shared_ptr<const he::ir::OpGraph> graph;
    std::string text, text_planned;
};

static thread_local he::exec::ExecStats g_last_stats;

extern "C" {

int he_matmul_kernel_create(he_tile_kernel_t* kernel, he_graph_t graph, const uint32_t* nodes, int num_nodes) {
    return he::guard([&] {
        HE_REQUIRE(kernel && graph && nodes && num_nodes > 0, HE_ERR_INVALID, "bad argument");
        he::ir::OpSubgraph sg(graph->g, std::vector<he::ir::NodeId>(nodes, nodes + num_nodes));
        auto k = std::make_unique<he_tile_kernel_s>();
        k->k = he::plan::make_gemm_kernel(sg);
        if (he::device_initialised()) k->k->load();  // so that later launches need not
        *kernel = k.release();
    });
}

int he_tensor_create_with_data(he_tensor_t* tensor, const void* data, int dtype, size_t len) {
    return he::guard([&] {
        HE_REQUIRE(tensor && (data || len == 0), HE_ERR_INVALID, "bad argument");
        (void)he::dtype_bits(dtype);
        *tensor = new he_tensor_s{he::exec::create_tensor_with_data(data, dtype, len)};
    });
}
int he_tensor_download(he_tensor_t tensor, void* dst) {
    return he::guard([&] {
        HE_REQUIRE(tensor && dst, HE_ERR_INVALID, "bad argument");
        he::exec::download_tensor(tensor->t, dst);
    });
}
int he_tensor_info(he_tensor_t tensor, int32_t* dtype, uint64_t* len, uint64_t* bytes, void** device_ptr) {
    return he::guard([&] {
        HE_REQUIRE(tensor, HE_ERR_INVALID, "null tensor");
        if (dtype) *dtype = tensor->t->dtype;
        if (len) *len = tensor->t->len;
        if (bytes) *bytes = tensor->t->bytes;
        if (device_ptr) *device_ptr = tensor->t->ptr;
    });
}
int he_tensor_free(he_tensor_t tensor) {
    delete tensor;
    return HE_OK;
}

int he_plan_generate(he_graph_t graph, he_plan_t* plan) {
    return he::guard([&] {
        HE_REQUIRE(graph && plan, HE_ERR_INVALID, "bad argument");
        // a snapshot of the graph: later edits do not disturb the plan's subgraphs
        std::shared_ptr<const he::ir::OpGraph> snapshot = std::make_shared<he::ir::OpGraph>(*graph->g);
        snapshot = he::plan::graph_for_execution(snapshot);
        auto p = std::make_unique<he_plan_s>();
        p->graph = snapshot;
        p->plan = he::plan::generate_plan(snapshot);
        p->text = p->plan->describe();
        p->text_planned = p->plan->describe(false);
        *plan = p.release();
    });
}
int he_plan_graph(he_plan_t plan, he_graph_t* graph) {
    return he::guard([&] {
        HE_REQUIRE(plan && graph, HE_ERR_INVALID, "bad argument");
        auto g = std::make_unique<he_graph_s>();
        g->g = std::make_shared<he::ir::OpGraph>(*plan->graph);
        *graph = g.release();
    });
}
int he_plan_num_steps(he_plan_t plan, int* steps) {
    return he::guard([&] { *steps = (int)plan->plan->steps.size(); });
}
const char* he_plan_describe(he_plan_t plan) { return plan ? plan->text.c_str() : ""; }
const char* he_plan_describe_planned(he_plan_t plan) { return plan ? plan->text_planned.c_str() : ""; }
int he_plan_instruction_kernel(he_plan_t plan, int index, he_tile_kernel_t* kernel) {
    return he::guard([&] {
        HE_REQUIRE(plan && kernel && index >= 0, HE_ERR_INVALID, "bad argument");
        int at = 0;
        for (auto& step : plan->plan->steps)
            for (auto& instr : step.instrs)
                if (at++ == index) {
                    HE_REQUIRE(!instr->absorbed(), HE_ERR_INVALID, "instruction %d launches nothing: the kernel of an earlier instruction does its work", index);
                    auto k = std::make_unique<he_tile_kernel_s>();
                    k->k = instr->kernel();
                    HE_REQUIRE(k->k, HE_ERR_INVALID, "instruction %d is a permute instruction", index);
                    *kernel = k.release();
                    return;
                }
        he::fail(HE_ERR_INVALID, "the plan has " + std::to_string(at) + " instructions");
    });
}
int he_plan_precompile(he_plan_t plan) {
    return he::guard([&] {
        HE_REQUIRE(plan, HE_ERR_INVALID, "bad argument");
        {
            // the kernels the executor would run: its assignment of instructions to streams shapes some of them
            he::exec::Prepared as_executed;
            as_executed.graph = plan->graph;
            as_executed.plan = plan->plan;
            he::exec::assign_streams(&as_executed);
        }
        std::vector<std::future<void>> jobs;
        for (auto& step : plan->plan->steps)
            for (auto& instr : step.instrs)
                if (!instr->compiled())
                    jobs.push_back(std::async(std::launch::async, [instr] {
                        try {
                            instr->precompile();
                        } catch (const he::Error& e) {
                            he::fail(e.code, std::string(e.what()) + " (instruction " + instr->describe() + ")");
                        }
                    }));
        for (auto& j : jobs) j.get();
    });
}
int he_plan_destroy(he_plan_t plan) {
    delete plan;
    return HE_OK;
}

int he_execute_graph(he_graph_t graph, const uint32_t* input_nodes, const he_tensor_t* input_tensors, int num_inputs,
                     uint32_t* output_nodes, he_tensor_t* output_tensors, int max_outputs, int* num_outputs) {
    return he::guard([&] {
        HE_REQUIRE(graph && num_outputs && (num_inputs == 0 || (input_nodes && input_tensors)), HE_ERR_INVALID, "bad argument");
        std::map<he::ir::NodeId, he::exec::TensorRef> inputs;
        for (int i = 0; i < num_inputs; i++) {
            HE_REQUIRE(input_tensors[i], HE_ERR_INVALID, "null input tensor %d", i);
            const he::ir::Node& n = graph->g->get(input_nodes[i]);
            HE_REQUIRE(n.kind == he::ir::Node::Input, HE_ERR_INVALID, "node %u is not an input", input_nodes[i]);
            const he::exec::Tensor& t = *input_tensors[i]->t;
            HE_REQUIRE(t.dtype == n.desc.dtype && (int64_t)t.len == he::ir::num_elements(n.desc.shape), HE_ERR_INVALID,
                       "tensor for input node %u does not match its descriptor", input_nodes[i]);
            inputs[input_nodes[i]] = input_tensors[i]->t;
        }
        // the optimised copy of the graph and its plan are made on the first call and kept with the handle
        std::shared_ptr<const he::exec::Prepared> prepared;
        {
            std::lock_guard<std::mutex> lk(graph->mu);
            const uint64_t options = he::plan::option_mask();
            if (!graph->prepared || graph->prepared_nodes != graph->g->num_nodes() || graph->prepared_options != options) {
                graph->prepared = he::exec::prepare(*graph->g);
                graph->prepared_nodes = graph->g->num_nodes();
                graph->prepared_options = options;
            }
            prepared = graph->prepared;
        }
        auto outs = he::exec::execute_prepared(*prepared, inputs, &g_last_stats);
        HE_REQUIRE((int)outs.size() <= max_outputs, HE_ERR_INVALID, "graph has %zu outputs, room for %d", outs.size(), max_outputs);
        int k = 0;
        for (auto& kv : outs) {
            output_nodes[k] = kv.first;
            output_tensors[k] = new he_tensor_s{kv.second};
            k++;
        }
        *num_outputs = k;
    });
}

int he_backend_set_option(int option, int64_t value) {
    return he::guard([&] {
        switch (option) {
            case HE_OPT_FUSE_MATMUL_EPILOGUE: he::plan::set_fuse_matmul_epilogue(value != 0); break;
            case HE_OPT_FOLD_SWAP_INTO_REDUCE: he::plan::set_fold_swap_into_reduce(value != 0); break;
            case HE_OPT_REMATERIALIZE: he::plan::set_rematerialize(value != 0); break;
            case HE_OPT_CANCEL_TRANSPOSES: he::plan::set_cancel_transposes(value != 0); break;
            case HE_OPT_HOIST_BROADCASTS: he::plan::set_hoist_broadcasts(value != 0); break;
            case HE_OPT_STREAM_FAN_OUT: he::exec::set_stream_fan_out((int)value); break;
            default: he::fail(HE_ERR_INVALID, "unknown backend option");
        }
    });
}

int he_backend_stats(uint64_t stats[9]) {
    return he::guard([&] {
        stats[0] = g_last_stats.steps;
        stats[1] = g_last_stats.instrs;
        stats[2] = g_last_stats.streams_used;
        stats[3] = g_last_stats.event_waits;
        he::plan::plan_cache_stats(&stats[4], &stats[5]);
        he::exec::DevicePool::global().stats(&stats[6], &stats[7], &stats[8]);
    });
}

}  // extern "C"
