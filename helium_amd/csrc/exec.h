// Graph executor for the HIP backend: tensor storage, pooled device memory with execution scopes, and the step
// loop of helium/src/backend.rs:40-80 driven over a pool of HIP streams (helium/src/cuda.rs:98-260).
#pragma once
#include <atomic>
#include <deque>
#include <set>
#include <map>
#include <memory>
#include <mutex>
#include <vector>

#include "alloc.h"
#include "plan.h"

namespace he::exec {

using ir::NodeId;

// A device event with shared ownership: an execution records one at its end and hands it to every tensor it
// returns, to the pool (which ends the execution's scope once it has passed) and to the thread's next execution.
// When the last holder lets go the event returns to the pool's spare list.
struct SharedEvent {
    hipEvent_t e = nullptr;
    ~SharedEvent();
};
using EventRef = std::shared_ptr<SharedEvent>;

// A piece of device memory handed out by the pool: its address and the block of the page it was cut from.
struct Allocation {
    void* ptr = nullptr;
    alloc::Block block;
};

// Pooling device allocator (helium/src/cuda/allocator/device.rs): pages of at least 1 GiB (a power of two) come from
// the driver and are never returned; inside them a best-fit block allocator with coalescing hands out 256-byte
// aligned blocks. An execution is a logical allocation stream ("scope"): a block freed inside a scope is reusable by
// that scope and by later scopes of the same host thread at once (their device work is ordered after it), and by
// everyone else when the scope has ended on the device (device.rs:60-89, block.rs:216-244).
class DevicePool {
public:
    static constexpr uint64_t kAlign = 256;             // alignment of every block (device.rs:33)
    static constexpr uint64_t kMinPage = 1ull << 30;    // device.rs:35
    static DevicePool& global();
    // `thread`: a token of the calling host thread (0: none). The executions of one thread are ordered on the device
    // (each waits for the end of the one before), so the thread's previous scope is the new scope's parent.
    uint64_t begin_scope(uint64_t thread = 0);
    void end_scope(uint64_t scope);  // called once the scope's device work has finished
    // Ends the scope once `done` (recorded after all of its device work) has completed; polled from begin_scope and
    // from allocate, so no host callback sits in any stream.
    void end_scope_after(uint64_t scope, EventRef done);
    void poll();
    // The same, for callers that have just waited for the device (stream / event / device synchronize): retiring the
    // executions that finished meanwhile is then part of the wait and not of the next execution's set-up (a host that
    // ran 200 executions ahead found all of them to retire, 2.5 us each, at the head of its next call). No-op before
    // the pool exists.
    static void poll_if_created();
    Allocation allocate(size_t bytes, uint64_t scope);
    // `owner`: the scope the block was allocated in (0: none); `used`: every scope whose device work touches it. The
    // block is free again for whoever comes after all of those that are still live.
    void release(const Allocation& a, uint64_t owner, const std::vector<uint64_t>& used);
    void note_use(struct Tensor& t, uint64_t scope);
    void note_uses(const std::map<ir::NodeId, std::shared_ptr<struct Tensor>>& tensors, uint64_t scope);
    EventRef take_event();          // an event nobody holds any more, or a new one
    void recycle(hipEvent_t event);  // called when an event's last holder lets go
    void stats(uint64_t* driver_bytes, uint64_t* driver_allocs, uint64_t* reuses);
    size_t live_scopes();

private:
    std::mutex mu_;
    alloc::BlockAllocator blocks_;
    std::vector<char*> page_base_;                   // by page id
    std::map<uint64_t, uint64_t> thread_last_scope_;  // thread token -> its latest scope
    std::deque<std::pair<uint64_t, EventRef>> pending_;  // scopes whose device work may still be running, oldest first
    std::vector<hipEvent_t> spare_events_;
    void note_locked(struct Tensor& t, uint64_t scope);
    uint64_t driver_bytes_ = 0, driver_allocs_ = 0, reuses_ = 0;
};

// TensorStorage (helium/src/cuda/tensor_storage.rs:31-42): device buffer + ready event; shared by reference count.
struct Tensor {
    void* ptr = nullptr;
    alloc::Block block;  // where `ptr` lies in the pool's pages
    size_t bytes = 0, len = 0;
    int dtype = HE_F32;
    uint64_t scope = 0;
    // Live execution scopes that read or wrote the tensor (guarded by the pool's mutex); scopes that have ended on
    // the device are dropped whenever another one is noted, so a long-lived tensor's list stays short.
    std::vector<uint64_t> used;
    bool uploaded = false;       // filled by an asynchronous host-to-device copy
    std::atomic<bool> ready_seen{false};  // `ready` has been observed complete (it is recorded once per tensor)
    // Recorded after the work that fills the tensor: the upload's own event, or the one event its execution records
    // at its end (a record costs the device about as much as a small kernel, so an execution records one, not one
    // per output). Null while the producing execution is still being queued.
    EventRef ready;
    ~Tensor();
};
using TensorRef = std::shared_ptr<Tensor>;

TensorRef allocate_tensor(int dtype, size_t len, uint64_t scope);            // TensorStorage::new (:45-73)
TensorRef create_tensor_with_data(const void* data, int dtype, size_t len);  // Backend::create_tensor_with_data (cuda.rs:62-79)
void download_tensor(const TensorRef& t, void* dst);                         // Backend::download_tensor (cuda.rs:81-96), blocking

struct ExecStats {
    int steps = 0, instrs = 0, streams_used = 0, event_waits = 0;
};

// Everything about an execution that depends on the graph alone: the optimised copy, its plan and the tensors that
// outlive the plan. Built once per graph by `prepare` and shared by every later execution.
struct Prepared {
    std::shared_ptr<const ir::OpGraph> graph;
    std::shared_ptr<const plan::Plan> plan;
    std::set<NodeId> alive;  // enumerate_output_tensors (cuda.rs:142-153)
    // When the graph that runs is a rewritten form of the caller's (plan::graph_for_execution): its Input node for each
    // of the caller's, and the caller's Output node for each of its own. Empty when the ids are the caller's.
    std::map<NodeId, NodeId> input_of, caller_output;
    std::vector<uint8_t> fan_out;  // per step of the plan: whether its instructions are worth a stream each
    // The side stream (see side_stream_split in exec.cpp): the instructions that launch something, in plan order, which of
    // them run beside the main chain, and who reads whose results. `side` is empty when nothing runs on the side.
    struct Side {
        std::vector<const plan::Instr*> order;
        std::map<const plan::Instr*, size_t> index;
        std::vector<uint8_t> side;
        std::vector<std::vector<uint32_t>> deps, dependents;
    } side;
};
// 0: every instruction runs on one stream; 1 (default): the instructions of a step fan out over the thread's streams
// where the work that can overlap outweighs the joins; 2: every step with several instructions fans out, as
// cuda.rs:190-221 does.
void set_stream_fan_out(int mode);
// Which instructions of pr->plan (a plan of pr->graph) run on which stream of an execution; the products that will run
// beside the main chain are told so (plan::Instr::runs_beside_main_chain), which has to happen before their kernels are made.
void assign_streams(Prepared* pr);
std::shared_ptr<const Prepared> prepare(const ir::OpGraph& graph);
std::map<NodeId, TensorRef> execute_prepared(const Prepared& prepared, const std::map<NodeId, TensorRef>& inputs,
                                             ExecStats* stats = nullptr);

// BackendExt::execute_graph (backend.rs:40-80). `inputs`: storage for every Input node. Returns the storage of
// every node that feeds an Output node, keyed by the Output node's id.
std::map<NodeId, TensorRef> execute_graph(const ir::OpGraph& graph, const std::map<NodeId, TensorRef>& inputs,
                                          ExecStats* stats = nullptr);

}  // namespace he::exec
