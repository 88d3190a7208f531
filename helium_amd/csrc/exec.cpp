#include <chrono>
#include "exec.h"

#include <algorithm>
#include <atomic>
#include <cstring>
#include <functional>
#include <future>
#include <set>

namespace he::exec {

// ---------------------------------------------------------------------------------------------------------
// Device pool
// ---------------------------------------------------------------------------------------------------------
static std::atomic<DevicePool*> g_pool{nullptr};

DevicePool& DevicePool::global() {
    static DevicePool* pool = [] {
        DevicePool* p = new DevicePool();  // never destroyed: tensors may outlive static destruction order
        g_pool.store(p, std::memory_order_release);
        return p;
    }();
    return *pool;
}

void DevicePool::poll_if_created() {
    if (DevicePool* p = g_pool.load(std::memory_order_acquire)) p->poll();
}

SharedEvent::~SharedEvent() {
    if (e) DevicePool::global().recycle(e);
}

void DevicePool::end_scope_after(uint64_t scope, EventRef done) {
    std::lock_guard<std::mutex> lk(mu_);
    pending_.push_back({scope, std::move(done)});
}

void DevicePool::recycle(hipEvent_t event) {
    std::lock_guard<std::mutex> lk(mu_);
    spare_events_.push_back(event);
}

void DevicePool::poll() {
    // Oldest first, and no further than the first execution that is still running: a host that runs many
    // executions ahead of the device would otherwise query every one of them on every allocation. Executions of
    // one thread finish in order; another thread's younger ones wait for the next poll at worst.
    std::vector<EventRef> passed;  // let go of outside the lock: the last holder's release takes it again
    {
        std::lock_guard<std::mutex> lk(mu_);
        while (!pending_.empty() && hipEventQuery(pending_.front().second->e) == hipSuccess) {
            if (blocks_.stream_is_live(pending_.front().first)) blocks_.end_stream(pending_.front().first);
            passed.push_back(std::move(pending_.front().second));
            pending_.pop_front();
        }
    }
}

EventRef DevicePool::take_event() {
    auto ev = std::make_shared<SharedEvent>();
    {
        std::lock_guard<std::mutex> lk(mu_);
        if (!spare_events_.empty()) {
            ev->e = spare_events_.back();
            spare_events_.pop_back();
            return ev;
        }
    }
    HE_HIP(hipEventCreateWithFlags(&ev->e, hipEventDisableTiming));
    return ev;
}

uint64_t DevicePool::begin_scope(uint64_t thread) {
    poll();
    std::lock_guard<std::mutex> lk(mu_);
    uint64_t parent = 0;
    if (thread) {
        auto it = thread_last_scope_.find(thread);
        if (it != thread_last_scope_.end() && blocks_.stream_is_live(it->second)) parent = it->second;
    }
    const uint64_t s = blocks_.begin_stream(parent);
    if (thread) thread_last_scope_[thread] = s;
    return s;
}

void DevicePool::end_scope(uint64_t scope) {
    std::lock_guard<std::mutex> lk(mu_);
    if (blocks_.stream_is_live(scope)) blocks_.end_stream(scope);
}

size_t DevicePool::live_scopes() {
    std::lock_guard<std::mutex> lk(mu_);
    return blocks_.num_streams();
}

void DevicePool::note_locked(Tensor& t, uint64_t scope) {
    size_t kept = 0;
    bool present = false;
    for (uint64_t s : t.used)
        if (blocks_.stream_is_live(s)) {
            t.used[kept++] = s;
            present = present || s == scope;
        }
    t.used.resize(kept);
    if (!present) t.used.push_back(scope);
}

void DevicePool::note_use(Tensor& t, uint64_t scope) {
    std::lock_guard<std::mutex> lk(mu_);
    note_locked(t, scope);
}

void DevicePool::note_uses(const std::map<ir::NodeId, TensorRef>& tensors, uint64_t scope) {
    std::lock_guard<std::mutex> lk(mu_);
    for (auto& kv : tensors) note_locked(*kv.second, scope);
}

Allocation DevicePool::allocate(size_t bytes, uint64_t scope) {
    // sizes are rounded up to the alignment so that small requests do not fragment the pages (device.rs:104-108)
    const uint64_t size = std::max<uint64_t>((bytes + kAlign - 1) / kAlign * kAlign, kAlign);
    Allocation a;
    for (int attempt = 0; attempt < 2; attempt++) {
        if (attempt == 1) poll();  // blocks of executions that have finished since become available
        std::lock_guard<std::mutex> lk(mu_);
        if (blocks_.allocate(size, kAlign, scope, &a.block)) {
            a.ptr = page_base_[a.block.page] + a.block.start;
            reuses_++;
            return a;
        }
    }
    // a new page: at least 1 GiB, a power of two (device.rs:144-154)
    uint64_t page = kMinPage;
    while (page < size) page *= 2;
    void* base = nullptr;
    HE_HIP(hipMalloc(&base, page));
    std::lock_guard<std::mutex> lk(mu_);
    const alloc::PageId id = blocks_.add_page(page);
    if (page_base_.size() <= id) page_base_.resize(id + 1);
    page_base_[id] = (char*)base;
    driver_bytes_ += page;
    driver_allocs_++;
    HE_REQUIRE(blocks_.allocate(size, kAlign, scope, &a.block), HE_ERR_INTERNAL, "a new page does not hold the allocation");
    a.ptr = page_base_[a.block.page] + a.block.start;
    return a;
}

void DevicePool::release(const Allocation& a, uint64_t owner, const std::vector<uint64_t>& used) {
    if (!a.ptr) return;
    std::lock_guard<std::mutex> lk(mu_);
    alloc::Block b = a.block;
    b.in_use.clear();
    if (owner && blocks_.stream_is_live(owner)) b.in_use.insert(owner);
    for (uint64_t s : used)
        if (blocks_.stream_is_live(s)) b.in_use.insert(s);
    blocks_.deallocate(std::move(b));
}

void DevicePool::stats(uint64_t* driver_bytes, uint64_t* driver_allocs, uint64_t* reuses) {
    std::lock_guard<std::mutex> lk(mu_);
    *driver_bytes = driver_bytes_;
    *driver_allocs = driver_allocs_;
    *reuses = reuses_;
}

// ---------------------------------------------------------------------------------------------------------
// Tensors
// ---------------------------------------------------------------------------------------------------------
Tensor::~Tensor() {
    if (ready && uploaded) (void)hipEventSynchronize(ready->e);  // the copy that fills the block may still be queued
    Allocation a;
    a.ptr = ptr;
    a.block = block;
    DevicePool::global().release(a, scope, used);
}

TensorRef allocate_tensor(int dtype, size_t len, uint64_t scope) {
    auto t = std::make_shared<Tensor>();
    t->dtype = dtype;
    t->len = len;
    t->bytes = storage_bytes(dtype, len);
    t->scope = scope;
    Allocation a = DevicePool::global().allocate(t->bytes, scope);
    t->ptr = a.ptr;
    t->block = std::move(a.block);
    return t;
}

namespace {
struct Staging {
    void* host = nullptr;
    size_t capacity = 0;
    hipEvent_t done = nullptr;
};
struct Streams {
    std::vector<hipStream_t> s;
    EventRef exec_end;  // end of this thread's latest execution (recorded on s[0] after it joined the others)
    bool has_run = false;
    hipStream_t h2d = nullptr, d2h = nullptr;
    std::vector<Staging> staging;  // pinned upload buffers, reused once their copy has finished
};
// A pinned buffer of at least `bytes` whose previous copy (if any) has completed.
Staging& staging_buffer(Streams& st, size_t bytes) {
    for (Staging& b : st.staging)
        if (b.capacity >= bytes && hipEventQuery(b.done) == hipSuccess) return b;
    // drop finished buffers that are too small before growing: keeps at most a few per thread
    for (size_t i = 0; i < st.staging.size();) {
        if (hipEventQuery(st.staging[i].done) == hipSuccess) {
            (void)hipHostFree(st.staging[i].host);
            (void)hipEventDestroy(st.staging[i].done);
            st.staging[i] = st.staging.back();
            st.staging.pop_back();
        } else {
            i++;
        }
    }
    Staging b;
    b.capacity = std::max<size_t>(bytes, 1u << 20);
    HE_HIP(hipHostMalloc(&b.host, b.capacity, hipHostMallocDefault));
    HE_HIP(hipEventCreateWithFlags(&b.done, hipEventDisableTiming));
    st.staging.push_back(b);
    return st.staging.back();
}
Streams& thread_streams() {
    // a small pool of non-blocking streams per host thread (helium/src/cuda/context.rs:112-125)
    static thread_local Streams st;
    if (st.s.empty()) {
        // HELIUM_HIP_STREAMS=<1..4>: how many streams the independent instructions of a step fan out over
        const char* env = getenv("HELIUM_HIP_STREAMS");
        const int n = env ? std::max(1, std::min(4, atoi(env))) : 4;
        for (int i = 0; i < n; i++) {
            hipStream_t x;
            HE_HIP(hipStreamCreateWithFlags(&x, hipStreamNonBlocking));
            st.s.push_back(x);
        }
        HE_HIP(hipStreamCreateWithFlags(&st.h2d, hipStreamNonBlocking));
        HE_HIP(hipStreamCreateWithFlags(&st.d2h, hipStreamNonBlocking));
    }
    return st;
}
}  // namespace

TensorRef create_tensor_with_data(const void* data, int dtype, size_t len) {
    TensorRef t = allocate_tensor(dtype, len, 0);
    Streams& st = thread_streams();
    if (t->bytes) {
        // staged through pinned memory so that the copy is asynchronous (tensor_storage.rs:83-110)
        Staging& b = staging_buffer(st, t->bytes);
        memcpy(b.host, data, t->bytes);
        HE_HIP(hipMemcpyAsync(t->ptr, b.host, t->bytes, hipMemcpyHostToDevice, st.h2d));
        HE_HIP(hipEventRecord(b.done, st.h2d));
    }
    t->uploaded = true;
    t->ready = DevicePool::global().take_event();
    HE_HIP(hipEventRecord(t->ready->e, st.h2d));
    return t;
}

void download_tensor(const TensorRef& t, void* dst) {
    Streams& st = thread_streams();
    if (t->ready) HE_HIP(hipStreamWaitEvent(st.d2h, t->ready->e, 0));
    if (t->bytes) HE_HIP(hipMemcpyAsync(dst, t->ptr, t->bytes, hipMemcpyDeviceToHost, st.d2h));
    HE_HIP(hipStreamSynchronize(st.d2h));
}

// ---------------------------------------------------------------------------------------------------------
// execute_graph
// ---------------------------------------------------------------------------------------------------------
namespace {
// HELIUM_HIP_EXEC_TIMING=1: host time per section of execute_graph, averaged and printed every 100 calls.
struct HostTimer {
    static bool on() {
        static const bool v = getenv("HELIUM_HIP_EXEC_TIMING") != nullptr;
        return v;
    }
    std::chrono::steady_clock::time_point t = std::chrono::steady_clock::now();
    double acc[8] = {0};
    void lap(int i) {
        if (!on()) return;
        auto n = std::chrono::steady_clock::now();
        acc[i] += std::chrono::duration<double, std::micro>(n - t).count();
        t = n;
    }
    void restart() {
        if (on()) t = std::chrono::steady_clock::now();
    }
};
// Join events of an execution are destroyed one execution later on the same thread: by then they were recorded and
// waited on long ago.
void retire_join_events(const std::vector<hipEvent_t>& events) {
    static thread_local std::vector<hipEvent_t> garbage;
    for (hipEvent_t e : garbage) (void)hipEventDestroy(e);
    garbage = events;
}
thread_local double g_host_acc[8] = {0};
thread_local int g_host_calls = 0;
std::atomic<int> g_fan_out{1};

// Whether the independent instructions of a step are worth a stream each. Putting work on a second stream costs a
// join before and after it: on this runtime a hipStreamWaitEvent takes the host 15-20 us for the first stream that
// waits on an event and about 7 us for each further one, and the device a few microseconds per dependent queue. What
// it can gain is the time of instructions too small to fill the chip, which then run beside each other (or under an
// instruction that does fill it): an instruction that moves more than a few MiB already uses every CU or all of the
// memory bandwidth, and two of those side by side finish when they would have finished one after the other.
bool fan_out_pays(const plan::Step& step, const ir::OpGraph& g) {
    if (step.instrs.size() < 2) return false;
    constexpr double kLaunchUs = 4, kBytesPerUs = 2e6, kNarrowBytes = 4 << 20, kJoinUs = 20;
    double narrow_sum = 0, narrow_max = 0;
    bool wide = false;
    for (auto& instr : step.instrs) {
        double bytes = 0;
        for (NodeId n : instr->inputs()) bytes += (double)storage_bytes(g.get(n).desc.dtype, (size_t)ir::num_elements(g.get(n).desc.shape));
        for (NodeId n : instr->outputs()) bytes += (double)storage_bytes(g.get(n).desc.dtype, (size_t)ir::num_elements(g.get(n).desc.shape));
        if (bytes > kNarrowBytes) {
            wide = true;
            continue;
        }
        const double us = kLaunchUs + bytes / kBytesPerUs;
        narrow_sum += us;
        narrow_max = std::max(narrow_max, us);
    }
    const double gain = wide ? narrow_sum : narrow_sum - narrow_max;
    return gain > 2 * kJoinUs;
}

// The side stream. A training step ends in many chains that nothing else waits for: a filter gradient, the launch that
// adds up its partial tiles, the optimizer's update of that filter. On one stream each of them holds up the chain
// that everything else hangs on (the data gradients); on a second stream they run beside it - matrix-core work under
// the memory-bound kernels of the next layers, and the other way round. The split: the instruction that nothing reads
// and that the most work leads up to ends the main chain; every instruction it does not depend on, directly or
// indirectly, runs on the side (no main instruction reads what a side instruction writes, by construction) - the small
// ones too: keeping those of less than 10 us that read main results only on the main stream measured 0.5% slower.
// HELIUM_HIP_SIDE_STREAM=0 switches the side stream off, =1 on for plans of any size.
void side_stream_split(Prepared* pr) {
    const char* env = tuning::get("HELIUM_HIP_SIDE_STREAM");
    if (env && atoi(env) == 0) return;
    const bool forced = env && atoi(env) != 0;
    for (uint8_t f : pr->fan_out)
        if (f) return;  // a plan whose steps fan out keeps to that scheme
    Prepared::Side S;
    for (auto& step : pr->plan->steps)
        for (auto& instr : step.instrs)
            if (!instr->absorbed()) {
                S.index[instr.get()] = S.order.size();
                S.order.push_back(instr.get());
            }
    const size_t n = S.order.size();
    if (n < 3) return;
    const ir::OpGraph& g = *pr->graph;
    auto bytes_of = [&](NodeId id) { return (double)storage_bytes(g.get(id).desc.dtype, (size_t)ir::num_elements(g.get(id).desc.shape)); };
    constexpr double kLaunchUs = 4, kBytesPerUs = 2e6, kWorthUs = 200, kDeviceBoundUs = 10;
    std::map<NodeId, uint32_t> made_by;
    std::vector<double> cost(n);
    S.deps.resize(n);
    S.dependents.resize(n);
    for (size_t i = 0; i < n; i++) {
        double bytes = 0;
        std::set<uint32_t> from;
        for (NodeId in : S.order[i]->all_inputs()) {
            bytes += bytes_of(in);
            auto it = made_by.find(in);
            if (it != made_by.end() && it->second != i) from.insert(it->second);
        }
        for (uint32_t d : from) {
            S.deps[i].push_back(d);
            S.dependents[d].push_back((uint32_t)i);
        }
        for (NodeId out : S.order[i]->all_outputs()) {
            bytes += bytes_of(out);
            made_by[out] = (uint32_t)i;
        }
        cost[i] = kLaunchUs + bytes / kBytesPerUs;
    }
    auto ancestors = [&](size_t of) {
        std::vector<uint8_t> in(n, 0);
        std::vector<uint32_t> stack{(uint32_t)of};
        in[of] = 1;
        while (!stack.empty()) {
            const uint32_t cur = stack.back();
            stack.pop_back();
            for (uint32_t d : S.deps[cur])
                if (!in[d]) {
                    in[d] = 1;
                    stack.push_back(d);
                }
        }
        return in;
    };
    std::vector<uint8_t> main_set;
    double main_cost = -1;
    for (size_t s = 0; s < n; s++) {
        if (!S.dependents[s].empty()) continue;
        std::vector<uint8_t> in = ancestors(s);
        double c = 0;
        for (size_t i = 0; i < n; i++)
            if (in[i]) c += cost[i];
        if (c >= main_cost) {
            main_cost = c;
            main_set.swap(in);
        }
    }
    S.side.assign(n, 0);
    double side_cost = 0;
    for (size_t i = 0; i < n; i++) {
        if (main_set[i]) continue;
        S.side[i] = 1;
        side_cost += cost[i];
    }
    // Early instructions (side value 2): small main-chain instructions that read nothing but the graph's inputs (or each
    // other) - a filter converted to the multiplicands' type ahead of its convolution - and whose first reader comes
    // well into the execution. Each would hold the main stream for a launch's latency; the side stream runs them all at
    // the start instead, and the main stream waits for them once, ahead of the first instruction that reads one.
    size_t early = 0;
    if (!tuning::get("HELIUM_HIP_NO_EARLY_INSTRS")) {
        constexpr double kEarlyUs = 20, kLeadUs = 100;
        std::vector<double> before(n + 1, 0);  // main-stream work ahead of each position
        for (size_t i = 0; i < n; i++) before[i + 1] = before[i] + (S.side[i] ? 0 : cost[i]);
        for (size_t i = 0; i < n; i++) {
            if (S.side[i] || cost[i] >= kEarlyUs || S.dependents[i].empty()) continue;
            bool sources_only = true;
            for (uint32_t d : S.deps[i]) sources_only = sources_only && S.side[d] == 2;
            uint32_t first_reader = (uint32_t)n;
            for (uint32_t d : S.dependents[i]) first_reader = std::min(first_reader, d);
            if (!sources_only || (!forced && before[first_reader] < kLeadUs)) continue;
            S.side[i] = 2;
            early++;
        }
    }
    if (getenv("HELIUM_HIP_PLAN_DEBUG")) {
        size_t count = 0;
        for (uint8_t f : S.side) count += f == 1;
        fprintf(stderr, "[plan] side stream: %zu of %zu launching instructions, about %.0f us beside %.0f us; %zu early instructions\n", count, n, side_cost,
                main_cost, early);
    }
    if (side_cost == 0 || (!forced && side_cost < kWorthUs)) return;
    // An execution that the host cannot keep ahead of (it needs 8-10 us per launch, and 15-20 more per wait between
    // streams) gains nothing from a second stream and loses the waits: the training step at batch 4 to 16, where the
    // estimate is 6 to 8 us of device time per launch, ran up to 1.5x slower with it; at 11 us (batch 32) and above it
    // gains 7-12%.
    if (!forced && (main_cost + side_cost) / (double)n < kDeviceBoundUs) return;
    pr->side = std::move(S);
}
}  // namespace

void assign_streams(Prepared* pr) {
    for (auto& step : pr->plan->steps) pr->fan_out.push_back(fan_out_pays(step, *pr->graph));
    side_stream_split(pr);
    for (size_t i = 0; i < pr->side.order.size(); i++)
        if (pr->side.side[i] == 1 && pr->side.order[i]->kind() == plan::InstrKind::Gemm) pr->side.order[i]->runs_beside_main_chain();
}

void set_stream_fan_out(int mode) {
    HE_REQUIRE(mode >= 0 && mode <= 2, HE_ERR_INVALID, "stream fan-out is 0 (never), 1 (where it pays) or 2 (always)");
    g_fan_out.store(mode);
}

std::shared_ptr<const Prepared> prepare(const ir::OpGraph& graph_in) {
    auto pr = std::make_shared<Prepared>();
    auto graph = std::make_shared<ir::OpGraph>(graph_in);
    graph->optimize();
    pr->graph = plan::graph_for_execution(graph);
    if (pr->graph->has_origins()) {
        for (NodeId in : pr->graph->inputs()) pr->input_of[pr->graph->origin(in)] = in;
        for (NodeId out : pr->graph->outputs()) pr->caller_output[out] = pr->graph->origin(out);
    }
    pr->plan = plan::generate_cached_plan(pr->graph);
    // tensors that survive the plan get their ready event recorded (enumerate_output_tensors, cuda.rs:142-153)
    for (auto& step : pr->plan->steps) {
        for (auto& instr : step.instrs)
            for (NodeId o : instr->outputs()) pr->alive.insert(o);
        for (NodeId r : step.tensors_to_release) pr->alive.erase(r);
    }
    // (ahead of the kernels: a product that will run beside the main chain is built for that)
    assign_streams(pr.get());
    // begin_execute (cuda.rs:98-139): compile every kernel of the plan up front, in parallel (cuda.rs:262-270)
    std::vector<std::future<void>> jobs;
    for (auto& step : pr->plan->steps)
        for (auto& instr : step.instrs)
            if (!instr->compiled()) jobs.push_back(std::async(std::launch::async, [instr] { instr->precompile(); }));
    for (auto& j : jobs) j.get();
    if (getenv("HELIUM_HIP_PLAN_DEBUG")) {
        size_t fanned = 0, multi = 0;
        for (size_t k = 0; k < pr->plan->steps.size(); k++) {
            fanned += pr->fan_out[k];
            multi += pr->plan->steps[k].instrs.size() > 1;
        }
        fprintf(stderr, "[plan] %zu steps, %zu with several instructions, %zu of them fan out over streams\n", pr->plan->steps.size(), multi, fanned);
    }
    return pr;
}

std::map<NodeId, TensorRef> execute_graph(const ir::OpGraph& graph_in, const std::map<NodeId, TensorRef>& inputs,
                                          ExecStats* stats) {
    return execute_prepared(*prepare(graph_in), inputs, stats);
}

std::map<NodeId, TensorRef> execute_prepared(const Prepared& prepared, const std::map<NodeId, TensorRef>& caller_inputs,
                                             ExecStats* stats) {
    HostTimer ht;
    // the ids of a rewritten graph differ from the caller's: inputs are renamed on the way in, outputs on the way out
    std::map<NodeId, TensorRef> renamed;
    if (!prepared.input_of.empty())
        for (auto& kv : caller_inputs) {
            auto it = prepared.input_of.find(kv.first);
            if (it != prepared.input_of.end()) renamed[it->second] = kv.second;
        }
    const std::map<NodeId, TensorRef>& inputs = prepared.input_of.empty() ? caller_inputs : renamed;
    const std::shared_ptr<const ir::OpGraph>& graph = prepared.graph;
    const std::shared_ptr<const plan::Plan>& plan = prepared.plan;
    const std::set<NodeId>& alive = prepared.alive;
    DevicePool& pool = DevicePool::global();
    Streams& st = thread_streams();
    for (NodeId in : graph->inputs())
        HE_REQUIRE(inputs.count(in), HE_ERR_INVALID, "missing storage for input node %u", in);
    const uint64_t scope = pool.begin_scope((uint64_t)(uintptr_t)&st);
    std::map<NodeId, TensorRef> tensors = inputs;
    pool.note_uses(tensors, scope);
    ht.lap(2);
    ExecStats local;
    std::set<const Tensor*> synced;        // input tensors whose ready event a stream already waited on
    std::vector<size_t> prev_streams;      // streams the previous step ran on
    std::vector<hipEvent_t> events;        // join events of this execution
    std::map<size_t, std::set<hipEvent_t>> waited_for;  // per stream: the events it has been made to wait for
    std::set<size_t> used_streams;
    // Every stream in `cur` waits for the end of the previous step on every other stream it ran on. The events are
    // recorded here, before the new step enqueues anything, so they mark exactly the end of that step.
    auto join = [&](const std::vector<size_t>& cur) {
        for (size_t p : prev_streams) {
            bool needed = false;
            for (size_t w : cur) needed = needed || w != p;
            if (!needed) continue;
            hipEvent_t e;
            HE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
            events.push_back(e);
            HE_HIP(hipEventRecord(e, st.s[p]));
            for (size_t w : cur)
                if (w != p) {
                    HE_HIP(hipStreamWaitEvent(st.s[w], e, 0));
                    local.event_waits++;
                }
        }
    };
    // An execution whose steps hold one instruction each runs on stream 0 alone: its last launch can carry the
    // execution's event itself.
    const int fan_mode = g_fan_out.load();
    auto step_width = [&](size_t k) {
        const plan::Step& step = plan->steps[k];
        const bool fan = !step.in_order && (fan_mode == 2 || (fan_mode == 1 && prepared.fan_out[k]));
        return fan ? std::min(step.instrs.size(), st.s.size()) : std::min<size_t>(step.instrs.size(), 1);
    };
    const plan::Instr* closing = nullptr;
    {
        bool one_stream = true;
        for (size_t k = 0; k < plan->steps.size(); k++) {
            auto& step = plan->steps[k];
            one_stream = one_stream && step_width(k) <= 1;
            for (auto& instr : step.instrs)
                if (!instr->absorbed()) closing = instr.get();  // (an absorbed instruction launches nothing)
        }
        if (!one_stream || getenv("HELIUM_HIP_NO_LAUNCH_EVENTS")) closing = nullptr;
    }
    // The side stream (side_stream_split): stream 1 runs the chains that nothing on the main stream waits for.
    const Prepared::Side& S = prepared.side;
    const bool side_mode = fan_mode == 1 && !S.side.empty() && st.s.size() >= 2;
    // (the end event follows the join of the two streams: the last launch carries it only if it runs on the main stream)
    if (side_mode && (getenv("HELIUM_HIP_NO_LAUNCH_EVENTS") || S.side.back())) closing = nullptr;
    if (side_mode && !getenv("HELIUM_HIP_NO_LAUNCH_EVENTS") && !S.side.back()) closing = S.order.back();
    std::vector<uint8_t> issued(side_mode ? S.order.size() : 0, 0);
    std::vector<TensorRef> held;           // what side instructions touch stays allocated until the streams have joined
    std::set<const Tensor*> synced_side;   // input tensors whose ready event the side stream waited on
    bool main_dirty = false;               // the main stream has taken work since the side stream last waited for it
    bool side_joined = false;              // the main stream has waited for the end of the side stream's work
    std::vector<EventRef> launch_events;   // completion events of main-stream launches that a side instruction follows
    bool main_end_known = false;           // ... and whether the last of them marks the main stream's latest launch
    EventRef done = pool.take_event();
    bool done_recorded = false;
    struct InstrTime {
        double us;
        int64_t bytes;
        const plan::Instr* instr;
        size_t order;  // position in the execution
    };
    std::vector<InstrTime> instr_times;
    static const int instr_timing = getenv("HELIUM_HIP_INSTR_TIMING") ? atoi(getenv("HELIUM_HIP_INSTR_TIMING")) : 0;
    // One instruction on stream `w` of the thread's pool: storage for what it writes, waits for inputs made outside
    // this execution, its launches.
    auto run_instr = [&](const plan::Instr& instr, size_t w, bool on_side, std::vector<const Tensor*>& waited) {
        hipStream_t stream = st.s[w];
        // a stream's first work of this execution comes after the end of the thread's previous execution
        // (stream 0 carried that end itself)
        if (used_streams.insert(w).second && w != 0 && st.has_run) {
            HE_HIP(hipStreamWaitEvent(stream, st.exec_end->e, 0));
            waited_for[w].insert(st.exec_end->e);
        }
        for (NodeId out : instr.all_outputs()) {
            const ir::Descriptor& d = graph->get(out).desc;
            tensors[out] = allocate_tensor(d.dtype, (size_t)ir::num_elements(d.shape), scope);
        }
        for (NodeId in : instr.all_inputs()) {
            auto it = tensors.find(in);
            HE_REQUIRE(it != tensors.end(), HE_ERR_INTERNAL, "missing storage for node %u", in);
            // tensors made outside this execution carry a ready event (uploads, earlier graphs); a wait of the main
            // stream also covers the side stream, which waits for the main stream before every instruction it takes
            if (inputs.count(in) && !synced.count(it->second.get()) && !(on_side && synced_side.count(it->second.get()))) {
                Tensor& t = *it->second;
                // a producer seen finished once stays finished: no wait is queued for it again
                if (t.ready && !t.ready_seen.load(std::memory_order_acquire)) {
                    if (hipEventQuery(t.ready->e) == hipSuccess) {
                        t.ready_seen.store(true, std::memory_order_release);
                    } else if (waited_for[w].insert(t.ready->e).second) {
                        // (one wait per event and stream: the tensors a previous execution returned share its end event,
                        // and a wait costs the host 15-20 us on a stream other than the one that recorded the event)
                        HE_HIP(hipStreamWaitEvent(stream, t.ready->e, 0));
                        local.event_waits++;
                    }
                }
                waited.push_back(it->second.get());
            }
        }
        ht.lap(3);
        if (&instr == closing) set_pending_stop_event(done->e);
        // HELIUM_HIP_INSTR_TIMING=<n>: every instruction is timed on its own (the device is drained before and after
        // it), and the n slowest of the execution are listed with the bytes they read and write. A debugging aid:
        // the execution is serialised while it is on.
        std::chrono::steady_clock::time_point t_instr;
        if (instr_timing) {
            HE_HIP(hipDeviceSynchronize());
            t_instr = std::chrono::steady_clock::now();
        }
        try {
            instr.execute([&](NodeId n) -> void* { return tensors.at(n)->ptr; }, stream);
        } catch (...) {
            (void)take_pending_stop_event();
            throw;
        }
        if (instr_timing) {
            HE_HIP(hipDeviceSynchronize());
            const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t_instr).count();
            int64_t bytes = 0;
            for (NodeId n : instr.all_inputs()) bytes += (int64_t)tensors.at(n)->bytes;
            for (NodeId n : instr.all_outputs()) bytes += (int64_t)tensors.at(n)->bytes;
            instr_times.push_back({us, bytes, &instr, instr_times.size()});
        }
        // taken by the instruction's last launch, or still pending (a launch too large for that entry point)
        if (&instr == closing) done_recorded = take_pending_stop_event() == nullptr;
        ht.lap(4);
        local.instrs++;
    };
    // A side instruction waits for everything the main stream has taken so far: for the results it reads, and because
    // the blocks it is given may have been freed by the main stream just now. What it touches is held until the
    // streams join, so the main stream is never handed a block the side stream still uses. The side instructions that
    // read its results alone follow at once (a filter gradient's update), which saves them a wait of their own.
    std::function<void(size_t)> issue_side = [&](size_t idx) {
        const plan::Instr& instr = *S.order[idx];
        if (main_dirty) {
            hipEvent_t e;
            if (main_end_known) {
                e = launch_events.back()->e;
            } else {
                HE_HIP(hipEventCreateWithFlags(&e, hipEventDisableTiming));
                events.push_back(e);
                HE_HIP(hipEventRecord(e, st.s[0]));
            }
            HE_HIP(hipStreamWaitEvent(st.s[1], e, 0));
            local.event_waits++;
            main_dirty = false;
        }
        std::vector<const Tensor*> waited_side;
        run_instr(instr, 1, true, waited_side);
        synced_side.insert(waited_side.begin(), waited_side.end());
        for (NodeId n : instr.all_inputs()) held.push_back(tensors.at(n));
        for (NodeId n : instr.all_outputs()) held.push_back(tensors.at(n));
        issued[idx] = 1;
        for (uint32_t d : S.dependents[idx]) {
            if (issued[d] || S.side[d] != 1) continue;
            bool ready = true;
            for (uint32_t dep : S.deps[d]) ready = ready && issued[dep];
            if (ready) issue_side(d);
        }
    };
    // Whatever happens below, the scope must end, and only after the work already queued: a failing instruction leaves
    // earlier launches running on up to four streams. On failure stream 0 is ordered after every stream this execution
    // used, the end event is recorded there as usual, and the error goes on to the caller.
    EventRef early_done;  // the early instructions' end on the side stream, until the main stream has waited for it
    try {
    if (side_mode && !instr_timing) {
        for (size_t idx = 0; idx < S.order.size(); idx++) {
            if (S.side[idx] != 2) continue;
            std::vector<const Tensor*> waited_side;
            run_instr(*S.order[idx], 1, true, waited_side);
            synced_side.insert(waited_side.begin(), waited_side.end());
            for (NodeId n : S.order[idx]->all_inputs()) held.push_back(tensors.at(n));
            for (NodeId n : S.order[idx]->all_outputs()) held.push_back(tensors.at(n));
            issued[idx] = 1;
            if (!early_done) early_done = pool.take_event();
        }
        if (early_done) HE_HIP(hipEventRecord(early_done->e, st.s[1]));
    }
    for (size_t step_no = 0; step_no < plan->steps.size(); step_no++) {
        auto& step = plan->steps[step_no];
        for (NodeId r : step.tensors_to_release) tensors.erase(r);
        if (step.instrs.empty()) continue;
        local.steps++;
        std::vector<const Tensor*> waited;
        // Instructions of one step are independent: they fan out over the stream pool where that pays.
        const size_t width = step_width(step_no);
        std::vector<size_t> cur(width);
        for (size_t w = 0; w < width; w++) cur[w] = w;
        ht.lap(3);
        join(cur);
        ht.lap(6);
        for (size_t i = 0; i < step.instrs.size(); i++) {
            const plan::Instr& instr = *step.instrs[i];
            if (instr.absorbed()) continue;  // run, and its outputs allocated, by the instruction that carries it
            if (side_mode) {
                const size_t idx = S.index.at(&instr);
                if (issued[idx]) continue;  // went out early, behind the side instruction it reads
                if (S.side[idx] == 1) {
                    issue_side(idx);
                    continue;
                }
                issued[idx] = 1;  // (an early instruction left for here - under instruction timing - runs on the main stream)
                if (early_done) {
                    bool reads_early = false;
                    for (uint32_t d : S.deps[idx]) reads_early = reads_early || S.side[d] == 2;
                    if (reads_early) {
                        HE_HIP(hipStreamWaitEvent(st.s[0], early_done->e, 0));
                        local.event_waits++;
                        early_done.reset();
                    }
                }
                main_dirty = true;
                main_end_known = false;
                if (&instr == closing) {
                    if (used_streams.count(1)) {
                        prev_streams = {1};
                        join({0});
                        prev_streams = {0};
                    }
                    side_joined = true;
                } else if (!instr_timing && !getenv("HELIUM_HIP_NO_LAUNCH_EVENTS")) {
                    // when a side instruction comes next, this instruction's last launch carries the event it will wait
                    // for, which saves the main stream a record of its own
                    size_t next = idx + 1;
                    while (next < issued.size() && issued[next]) next++;
                    if (next < issued.size() && S.side[next] == 1) {
                        launch_events.push_back(pool.take_event());
                        set_pending_stop_event(launch_events.back()->e);
                        run_instr(instr, i % width, false, waited);
                        main_end_known = take_pending_stop_event() == nullptr;
                        continue;
                    }
                }
            }
            run_instr(instr, i % width, false, waited);
        }
        // every stream of the next steps is ordered after this step's streams, so one wait per tensor is enough
        synced.insert(waited.begin(), waited.end());
        prev_streams = cur;
    }
    } catch (...) {
        try {
            prev_streams.assign(used_streams.begin(), used_streams.end());
            join({0});
            HE_HIP(hipEventRecord(done->e, st.s[0]));
            st.exec_end = done;
            st.has_run = true;
            pool.end_scope_after(scope, done);
        } catch (...) {
            (void)hipDeviceSynchronize();
            pool.end_scope(scope);
        }
        retire_join_events(events);
        throw;
    }
    ht.lap(3);
    if (side_mode && used_streams.count(1) && !side_joined) prev_streams = {0, 1};
    // Drop of the executor (cuda.rs:232-260): when everything queued above has run, the scope's freed blocks
    // become available to everyone. Stream 0 joins the last step and carries the event the pool polls.
    join({0});
    if (!done_recorded) HE_HIP(hipEventRecord(done->e, st.s[0]));
    // The same event orders this thread's next execution after this one, and it is the ready event of every tensor
    // that outlives the plan (enumerate_output_tensors, cuda.rs:142-153, records one per tensor).
    for (NodeId out : alive) tensors.at(out)->ready = done;
    st.exec_end = done;
    st.has_run = true;
    pool.end_scope_after(scope, std::move(done));
    retire_join_events(events);
    local.streams_used = (int)used_streams.size();
    if (stats) *stats = local;

    if (!instr_times.empty()) {
        static std::atomic<int> reports{0};
        if (reports.fetch_add(1) == 1) {  // the second execution: kernels are compiled and loaded by then
            std::sort(instr_times.begin(), instr_times.end(), [](const InstrTime& a, const InstrTime& b) { return a.us > b.us; });
            double total = 0;
            for (auto& t : instr_times) total += t.us;
            fprintf(stderr, "[instr timing] %zu instructions, %.1f us in all; slowest:\n", instr_times.size(), total);
            const int top = atoi(getenv("HELIUM_HIP_INSTR_TIMING"));
            for (int i = 0; i < top && i < (int)instr_times.size(); i++) {
                const std::string d = instr_times[i].instr->describe();
                const auto k = instr_times[i].instr->kernel();
                fprintf(stderr, "  #%-4zu %8.1f us %8.1f MB %6.2f TB/s  %s  %s\n", instr_times[i].order, instr_times[i].us, instr_times[i].bytes / 1e6,
                        instr_times[i].bytes / instr_times[i].us / 1e6, d.substr(0, 60).c_str(), k ? k->describe().substr(0, 260).c_str() : "");
            }
        }
    }
    std::map<NodeId, TensorRef> result;
    for (NodeId out : graph->outputs()) {
        NodeId from = graph->inbound(out)[0];
        auto it = tensors.find(from);
        HE_REQUIRE(it != tensors.end(), HE_ERR_INTERNAL, "output node %u has no storage", out);
        result[prepared.caller_output.empty() ? out : prepared.caller_output.at(out)] = it->second;
    }
    ht.lap(5);
    if (HostTimer::on()) {
        for (int i = 0; i < 8; i++) g_host_acc[i] += ht.acc[i];
        if (++g_host_calls % 100 == 0) {
            fprintf(stderr, "[exec timing] per graph, us: copy+optimize %.1f, plan lookup %.1f, setup %.1f, alloc+waits %.1f, joins %.1f, launches %.1f, finish %.1f\n",
                    g_host_acc[0] / 100, g_host_acc[1] / 100, g_host_acc[2] / 100, g_host_acc[3] / 100, g_host_acc[6] / 100, g_host_acc[4] / 100, g_host_acc[5] / 100);
            for (double& v : g_host_acc) v = 0;
        }
    }
    return result;
}

}  // namespace he::exec
