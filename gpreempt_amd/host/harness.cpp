// Multi-tenant benchmark harness: tenants with priorities share one GPU; the policy decides how
// a higher-priority request takes the GPU from lower-priority work.
//
// It plays the role of the reference's DISB suite (third_party/disb/src/benchmark.cpp:182-338,
// load.cpp:71-260, analyzer.cpp:90-170) together with the client programs that carry the
// scheduling policies (src/cuda-clients/blpclient.cpp:163-198 "wb", src/common-clients/
// baseclient.cpp "np", seqclient.cpp:82-102 "seq", rtonlyclient.cpp:120-141 "lco"), and reads
// the same task-file schema (config/A.json).  Unlike DISB it keeps every request's latency, so
// percentiles can be reported, and it seeds the Poisson generator from the task file instead of
// the clock (load.cpp:190).
#include "harness.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstring>
#include <ctime>
#include <condition_variable>
#include <memory>
#include <map>
#include <mutex>
#include <queue>
#include <thread>

#include "executor.h"
#include "gpreempt.h"
#include "mini_json.h"
#include "numeric.h"

namespace foo {

// Policy names: "wb" (reference), "wb-async", "wb-chunk", "wb-chunk-async".
static bool is_wb(const std::string &p) { return p == "wb" || p == "wb-async" || p == "wb-chunk" || p == "wb-chunk-async"; }
static bool is_chunked(const std::string &p) { return p == "wb-chunk" || p == "wb-chunk-async"; }
static bool is_async(const std::string &p) { return p == "wb-async" || p == "wb-chunk-async"; }


using clock_type = std::chrono::steady_clock;
static inline int64_t now_ns() { return std::chrono::duration_cast<std::chrono::nanoseconds>(clock_type::now().time_since_epoch()).count(); }
static inline void spin_pause() { __builtin_ia32_pause(); }

namespace {

constexpr int kMaxLevels = 8;
constexpr int kWarmups = 10;          // third_party/disb/include/benchmark.h:39
constexpr int kStandAloneRuns = 100;  // third_party/disb/include/benchmark.h:40

// ---- arrival processes (third_party/disb/src/load.cpp) -----------------------------------------
struct Load {
    std::string type = "continuous";
    double frequency = 0;
    uint64_t seed = 1;
    int64_t next = 0, end = 0;
    numeric::Rng rng{1};
    std::vector<int64_t> trace_ms;  // "trace": arrival times in milliseconds from the start (load.cpp:239-248)
    size_t next_trace = 0;
    int64_t begin = 0;
    int load_priority = 0;      // the load's own "priority" key: only loads with 0 are staggered (load.cpp:58-61)
    int64_t launch_delay = 0;   // "periodic": set by the coordinator (load.cpp:47-69)

    int64_t gap_ns() {
        if (type == "poisson") {  // exponential gaps: -ln(u) / frequency (load.cpp:230-237)
            double u = rng.uniform01();
            if (u < 1e-12) u = 1e-12;
            return (int64_t)(-std::log(u) / frequency * 1e9);
        }
        return (int64_t)(1e9 / frequency);
    }
    void start(int64_t begin_, int64_t end_) {
        begin = begin_; end = end_;
        next = begin + (type == "periodic" ? launch_delay : 0);
        rng = numeric::Rng(seed);
        next_trace = 0;
        std::sort(trace_ms.begin(), trace_ms.end());
    }
    // When the request after the one being served arrives (0: not known, or never).
    int64_t following() const {
        if (type == "continuous") return 0;
        if (type == "trace") return next_trace < trace_ms.size() ? begin + trace_ms[next_trace] * 1000000 : 0;
        return frequency > 0 && next < end ? next : 0;
    }
    // Returns false when the run is over.  A launch whose successor is already due is given up,
    // as in DISB ("always choose the newest frame", load.cpp:196-222).  *scheduled receives the
    // arrival time of the request that is served.
    bool wait_next(int64_t *scheduled) {
        int64_t now = now_ns();
        if (type == "continuous") {
            *scheduled = now;
            return now < end;
        }
        if (type == "trace") {
            // the arrival whose successor is already due is given up (load.cpp:258-296)
            if (next_trace >= trace_ms.size()) return false;
            int64_t launch = begin + trace_ms[next_trace] * 1000000;
            size_t nn = next_trace + 1;
            while (nn < trace_ms.size() && begin + trace_ms[nn] * 1000000 < now) { launch = begin + trace_ms[nn] * 1000000; ++nn; }
            next_trace = nn;
            if (launch >= end) return false;
            while (now_ns() < launch) {
                int64_t left = launch - now_ns();
                if (left > 200000) std::this_thread::sleep_for(std::chrono::nanoseconds(left - 100000));
                else spin_pause();
            }
            *scheduled = launch;
            return true;
        }
        if (frequency <= 0) return false;
        int64_t nn = next + gap_ns();
        while (nn < now) { next = nn; nn = next + gap_ns(); }
        if (next >= end) return false;
        while (now_ns() < next) {
            int64_t left = next - now_ns();
            if (left > 200000) std::this_thread::sleep_for(std::chrono::nanoseconds(left - 100000));
            else spin_pause();
        }
        *scheduled = next;
        next = nn;
        return true;
    }
};

struct Stats {
    std::vector<double> v;  // microseconds
    void add(double us) { v.push_back(us); }
    double pct(double p) const {
        if (v.empty()) return 0;
        std::vector<double> s(v);
        std::sort(s.begin(), s.end());
        double idx = p * (s.size() - 1);
        size_t lo = (size_t)idx;
        size_t hi = std::min(lo + 1, s.size() - 1);
        return s[lo] + (s[hi] - s[lo]) * (idx - lo);
    }
    double mean() const {
        if (v.empty()) return 0;
        double t = 0;
        for (double x : v) t += x;
        return t / v.size();
    }
    double max() const { return v.empty() ? 0 : *std::max_element(v.begin(), v.end()); }
    json::Value to_json() const {
        json::Value o = json::Value::object();
        o.set("count") = v.size();
        o.set("mean") = mean(); o.set("p50") = pct(0.5); o.set("p90") = pct(0.9); o.set("p99") = pct(0.99); o.set("max") = max();
        return o;
    }
};

// ---- shared scheduling state -------------------------------------------------------------------
// Level p tenants obey flag word p-1, which is up while any tenant of a level < p is active
// (the reference has two levels and one word, blpclient.cpp:185-195; the three-tenant
// configuration needs one word per level).
// Pre-preemption hints (reference src/cuda-clients/gpreemptclient.cpp:51-60, 203-219, 267-291):
// a latency-critical client that knows its request will reach the GPU after `preprocess_time`
// posts a hint on arrival; a daemon orders the hints by deadline and raises the flag words
// `switch_us` before the kernels are due, so that the lower levels drain while the client is
// still preprocessing on the CPU.  Whoever comes first, daemon or client, begins the request in
// the PreemptDomain (exactly once); the client ends it.
class HintDaemon {
public:
    struct Hint {
        int64_t deadline_ns;
        int priority;
        std::shared_ptr<std::atomic<int>> state;  // 0 pending, 1 begun by the daemon, 2 begun by the client
        bool operator>(const Hint &o) const { return deadline_ns > o.deadline_ns; }
    };
    explicit HintDaemon(PreemptDomain *d) : domain_(d), thread_([this] { run(); }) {}
    ~HintDaemon() {
        {
            std::lock_guard<std::mutex> g(mu_);
            quit_ = true;
        }
        cv_.notify_all();
        thread_.join();
    }
    std::shared_ptr<std::atomic<int>> post(int64_t deadline_ns, int priority) {
        auto st = std::make_shared<std::atomic<int>>(0);
        {
            std::lock_guard<std::mutex> g(mu_);
            heap_.push(Hint{deadline_ns, priority, st});
        }
        cv_.notify_all();
        return st;
    }
    long fired() const { return fired_.load(); }

private:
    void run() {
        std::unique_lock<std::mutex> lk(mu_);
        while (!quit_) {
            if (heap_.empty()) { cv_.wait(lk); continue; }
            Hint h = heap_.top();
            int64_t now = now_ns();
            if (now < h.deadline_ns) {
                // sleep most of the way, spin the last stretch: a condition variable alone wakes tens of us late
                int64_t left = h.deadline_ns - now;
                if (left > 60000) cv_.wait_for(lk, std::chrono::nanoseconds(left - 50000));
                else { lk.unlock(); spin_pause(); lk.lock(); }
                continue;
            }
            heap_.pop();
            int expect = 0;
            if (h.state->compare_exchange_strong(expect, 1)) {
                lk.unlock();
                domain_->begin(h.priority);
                fired_.fetch_add(1);
                lk.lock();
            }
        }
    }
    PreemptDomain *domain_;
    std::mutex mu_;
    std::condition_variable cv_;
    std::priority_queue<Hint, std::vector<Hint>, std::greater<Hint>> heap_;
    bool quit_ = false;
    std::atomic<long> fired_{0};
    std::thread thread_;
};

struct Shared {
    std::string policy;
    int levels = 2;
    std::unique_ptr<PreemptDomain> domain;  // flag words and per-level request counts (gpreempt.h)
    std::unique_ptr<HintDaemon> hints;      // null: no pre-preemption hints
    int64_t hint_switch_us = 0;             // how long before the kernels are due the flag goes up
    std::atomic<int> on_gpu[kMaxLevels];    // preemptible tenants of this level with work in flight
    std::atomic<int> seq_waiting{0};        // "seq": latency-critical requests waiting for the lock
    std::mutex seq_mu;
    std::mutex stats_mu;
    Stats preempt_latency;                  // flag store -> lower-priority stream drained
    // the same preemptions split by device time stamps ("device_stamps": true): flag store -> stop recorded
    // on the GPU -> last workgroup of the tenant gone -> the host notices; and, after the higher level has
    // finished, resubmission -> first tile claimed
    bool device_stamps = false;
    long corun_discard = 0;                 // the first requests of every priority-0 tenant are served but not counted
    bool hold_backlog = true;               // see end_request
    int64_t hold_us = 30;
    // busy_above[L]: time during which at least one request of a level above L (a smaller number)
    // was being served: what a continuous tenant of level L could not have used
    std::mutex busy_mu;
    int serving_above[kMaxLevels] = {};
    int64_t busy_since[kMaxLevels] = {};
    int64_t busy_above[kMaxLevels] = {};
    void serving(int p, int delta) {
        const int64_t now = now_ns();
        std::lock_guard<std::mutex> g(busy_mu);
        for (int l = p + 1; l < levels; ++l) {
            if (delta > 0 && serving_above[l]++ == 0) busy_since[l] = now;
            if (delta < 0 && --serving_above[l] == 0) busy_above[l] += now - busy_since[l];
        }
    }
    std::atomic<int> cores{0};
    bool verify_outputs = false;            // hash every request's output and compare it with the tenant's stand-alone output
    bool hp_gate = false;                   // non-preemptible tenants of level 0 submit behind a gate kernel (gpreemptclient.cpp:74-81)
    long hp_requests = 0;                   // > 0: the run ends once every priority-0 tenant served this many
    std::atomic<int> hp_unfinished{0};
    std::atomic<bool> stop{false};

    Shared() {
        for (int i = 0; i < kMaxLevels; ++i) on_gpu[i] = 0;
    }
    int active_above(int p) const { return domain->active_above(p); }
    int on_gpu_below(int p) const {
        int n = 0;
        for (int i = p + 1; i < levels; ++i) n += on_gpu[i].load(std::memory_order_acquire);
        return n;
    }
};

struct Tenant {
    std::string id, name, model_name;
    int priority = 0;
    bool use_graph = true;
    bool resident_io = false, input_resident = false;
    std::string launch_mode;  // "program" | "graph" | "launch"; empty = "program" when use_cuda_graph, else "launch"
    int64_t preprocess_us = 0;
    Load load;
    std::unique_ptr<Executor> ex;
    BLPExecutor *blp = nullptr;
    GPUstream stream = nullptr;
    void *input = nullptr, *output = nullptr;
    size_t input_size = 0, output_size = 0;
    Stats standalone, total, infer, queueing;
    // DISB's six phases (analyzer.cpp:90-150); prepareInput and postprocess are empty in the reference's clients
    double phase_sum_us[4] = {0, 0, 0, 0};  // preprocess, copyInput, infer, copyOutput
    NvContext nvctx;
    volatile int *gate_host = nullptr;      // hp_gate: the word the gate kernels wait for
    void *gate_dev = nullptr;
    int *gate_timed_out = nullptr;          // device word set by a gate that gave up
    // the slowest drains of this tenant: how long, and which kernel the stop index named afterwards
    struct Drain { double us; int stop_kernel; int queued; unsigned long long stop_ticks = 0, exit_ticks = 0; int64_t raised = 0; double since_launch_us = 0; bool resumed = false; };
    std::vector<Drain> drains;
    bool have_ref_hash = false;
    uint64_t ref_hash = 0;
    long output_mismatches = 0;
    int64_t preemptions = 0, requests = 0;
    std::vector<double> first_latencies;    // total latency of the first co-run requests, in arrival order
    long discarded = 0;
    int64_t resubmitted_ns = 0;             // device stamps: when the kernels of a stopped model were submitted again
    bool holding = false;                   // the level stayed up after the last request (end_request)
    long held = 0;                          // how often
    // one preemption (or resubmission) as the host and the GPU saw it: host clock nanoseconds and raw device ticks
    struct StampSample { int64_t raised = 0, drained = 0, resubmitted = 0; unsigned long long stop = 0, exit = 0, claim = 0; };
    std::vector<StampSample> stamp_samples;
    int64_t first_ns = 0, last_ns = 0;
    Status error = Status::Succ;
    gp_event chunk_events[3] = {nullptr, nullptr, nullptr};
};

void fill_input(Tenant &t) {
    // synthetic input: N(0,1) values for images, uniform token ids for BERT (int64 storage)
    numeric::Rng rng(0xDA7A + std::hash<std::string>()(t.id) % 1000);
    auto m = t.ex->get_model();
    size_t idx = 0;
    if (!m || m->find_storage_idx("data", idx) != Status::Succ) return;  // a workload without input (miniweather)
    const std::string &st = m->get_storage_info(idx).stype;
    if (st == "int64") { int64_t *p = (int64_t *)t.input; for (size_t i = 0; i < t.input_size / 8; ++i) p[i] = (int64_t)(rng.next() % 30522); }
    else if (st == "float32") { float *p = (float *)t.input; for (size_t i = 0; i < t.input_size / 4; ++i) p[i] = rng.normal(); }
    else if (st == "float16") { uint16_t *p = (uint16_t *)t.input; for (size_t i = 0; i < t.input_size / 2; ++i) p[i] = numeric::f32_to_f16(rng.normal()); }
    else { uint16_t *p = (uint16_t *)t.input; for (size_t i = 0; i < t.input_size / 2; ++i) p[i] = numeric::f32_to_bf16(rng.normal()); }
}

Status init_tenant(Tenant &t, Shared &sh) {
    const bool preemptible = t.priority > 0 && is_wb(sh.policy);
    if (preemptible) { t.blp = new BLPExecutor(); t.ex.reset(t.blp); }
    else t.ex.reset(new BaseExecutor());
    RETURN_STATUS(t.ex->init(t.model_name));
    t.input_size = t.ex->get_data_size("data");
    t.output_size = t.ex->get_data_size("heads");
    if (t.input_size) CUDA_RETURN_STATUS(gp_host_alloc(&t.input, t.input_size));
    if (t.output_size) CUDA_RETURN_STATUS(gp_host_alloc(&t.output, t.output_size));
    fill_input(t);
    CUDA_RETURN_STATUS(gp_stream_create(t.priority, &t.stream));
    // gpreemptclient.cpp:170-177: look the tenant's context up and give it its priority
    t.nvctx.stream = t.stream;
    if (NvRmQuery(&t.nvctx) != 0 || set_priority(t.nvctx, t.priority) != 0) {
        std::fprintf(stderr, "Failed to set priority %d for %s\n", t.priority, t.id.c_str());
        return Status::Fail;
    }
    if (sh.hp_gate && t.priority == 0 && !preemptible) {
        CUDA_RETURN_STATUS(gp_flag_create(&t.gate_host, &t.gate_dev));
        CUDA_RETURN_STATUS(gp_malloc((void **)&t.gate_timed_out, sizeof(int)));
        CUDA_RETURN_STATUS(gp_fill32_async(t.gate_timed_out, 0, 1, nullptr));
        CUDA_RETURN_STATUS(gp_stream_sync(nullptr));
    }
    if (t.blp) {
        t.blp->dpStop = sh.domain->flag_for(t.priority);
        if (sh.domain->relayed()) t.blp->poll_every = 1;  // the flag is a device-memory mirror
    }
    // "wb-chunk" feeds a preemptible tenant's kernels a few at a time, so it never uses a
    // captured graph or program for that tenant.
    const bool chunked = t.blp && is_chunked(sh.policy);
    if (!chunked && t.launch_mode != "launch") {
        setenv("GPREEMPT_USE_HIPGRAPH", t.launch_mode == "graph" ? "1" : "0", 1);
        t.ex->capture_graph(t.stream);
    }
    if (chunked) for (int i = 0; i < 3; ++i) CUDA_RETURN_STATUS(gp_event_create(&t.chunk_events[i]));
    static const bool use_events = [] { const char *e = getenv("GPREEMPT_CHUNK_EVENTS"); return e && *e == '1'; }();
    if (chunked && !use_events && !t.ex->graph_workload()) RETURN_STATUS(t.blp->enable_launch_tracking());
    if (chunked && sh.device_stamps && !t.ex->graph_workload()) RETURN_STATUS(t.blp->enable_device_stamps(t.stream));
    return Status::Succ;
}

// Waits until a preemptible tenant's work has left the GPU.  In program mode the kernel itself
// tells the host (BLPExecutor::program_vacated); *vacated_ns receives that moment.  What follows
// on the stream (reading the stop index back, relaunching) is ordered behind the kernel anyway.
Status drain(GPUstream s);
Status drain_blp(BLPExecutor *ex, GPUstream s, int64_t *vacated_ns) {
    for (int i = 0;; ++i) {
        if (ex->program_vacated()) break;  // a plain load of host memory
        if ((i & 15) == 15) {              // the queue is asked now and then as well (per-kernel mode, errors)
            int idle = 0;
            CUDA_RETURN_STATUS(gp_stream_query(s, &idle));
            if (idle) break;
        }
        spin_pause();
    }
    *vacated_ns = now_ns();
    return Status::Succ;
}

// Waits until the stream is idle by polling, which reacts faster than a blocking wait.
Status drain(GPUstream s) {
    for (;;) {
        int idle = 0;
        CUDA_RETURN_STATUS(gp_stream_query(s, &idle));
        if (idle) return Status::Succ;
        spin_pause();
    }
}

// The same for a tenant with launch tracking: a marker behind what is queued, then loads of host memory.  (The queue
// is still asked now and then, so that an error on the stream ends the wait.)
Status drain_marked(BLPExecutor *ex, GPUstream s) {
    RETURN_STATUS(ex->mark_stream(s));
    for (long i = 1;; ++i) {
        if (ex->stream_left()) return Status::Succ;
        if ((i & 0xffff) == 0) {
            int idle = 0;
            CUDA_RETURN_STATUS(gp_stream_query(s, &idle));
            if (idle) return Status::Succ;
        }
        spin_pause();
    }
}

// "wb-chunk" / "wb-chunk-async": the best-effort model is submitted launch by launch
// (Executor::launch_kernel, the reference's own launch loop, src/executor.cpp:222-225) but never far ahead of the
// GPU: with launch tracking (the default) at most queue_depth() launches that have not started, as the launches
// themselves report; without it (GPREEMPT_CHUNK_EVENTS=1) never
// more than two chunks of kernels ahead of the GPU, by an event behind every chunk, which costs the stream 3.7 us.  A preempted model then has at most two chunks
// of queued kernels to flush (each leaves at its first look at the stop index, about 4 us apiece
// on MI355X) instead of the rest of the network, while every kernel keeps its own occupancy.
// Measured with BERT over ResNet-152: chunks of 6 / 3 / 2 / 1 kernels drain in 44 / 32 / 28 / 23 us
// (mean) and cost 0 / 3 / 7 / 16 % of the best-effort throughput; the default is 2
// (environment variable GPREEMPT_CHUNK overrides it).
static int chunk_size() {
    static const int v = [] { const char *e = getenv("GPREEMPT_CHUNK"); int c = e ? atoi(e) : 2; return c < 1 ? 1 : c; }();
    return v;
}
static int queue_depth() {
    static const int v = [] { const char *e = getenv("GPREEMPT_QUEUE"); int c = e ? atoi(e) : 2; return c < 1 ? 1 : c; }();
    return v;
}
Status infer_chunked(Tenant &t, Shared &sh, int p) {
    BLPExecutor *ex = t.blp;
    const size_t n = ex->get_kernel_num();
    Status st = ex->reset_counters(t.stream);
    size_t next = 0;
    int inflight = 0, head = 0, tail = 0;  // ring of 3 events, at most 2 in flight
    // With launch tracking (BLPExecutor::enable_launch_tracking) no events are needed: every launch reports its start,
    // and at most queue_depth() launches are kept submitted and not started (one, behind a kernel of 3 GFLOP or more).
    const bool tracked = ex->launch_tracking_enabled();
    if (tracked) ex->restart_launch_tracking();
    double last_flops = 0;
    bool tail_marked = false;              // the marker behind the model's last kernel has been submitted
    unsigned long idle_spins = 0;
    int64_t first_launch_ns = 0;           // when the first kernel of this request, or of its latest resumption, was submitted
    bool resumed = false;
    ex->running = true;
    sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
    while (st == Status::Succ && (tracked || next < n || inflight > 0)) {
        if (sh.active_above(p) > 0) {
            // a higher level wants the GPU: stop feeding, let what is queued leave
            int queued = inflight;
            // (tracked: the launches that have not started, and the one that has, if the tail marker has not run yet)
            if (tracked) queued = ex->launches_submitted() - ex->launches_started() + (ex->launches_submitted() > 0 && !(tail_marked && ex->stream_left()) ? 1 : 0);
            st = tracked ? drain_marked(ex, t.stream) : drain(t.stream);
            tail_marked = false;
            if (st != Status::Succ) break;
            int64_t drained = now_ns();
            inflight = 0; head = tail;
            if (tracked) ex->restart_launch_tracking();  // nothing of this tenant is in flight
            sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
            // read the stop index back (and re-arm it) while the higher level has the GPU: nothing of
            // this tenant is in flight, and the blocking read-back (10-20 us) then costs nobody anything
            st = ex->getStopPoint(t.stream);
            if (st != Status::Succ) { sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel); break; }
            const int stop = ex->last_stop_index();
            const int64_t raised = sh.domain->raised_ns(p);
            unsigned long long stop_ticks = 0, exit_ticks = 0;
            if (ex->device_stamps_enabled()) {
                // the GPU's own account of this preemption (and of the resume before it, if there was one)
                BLPExecutor::DeviceStamps ds;
                st = ex->read_device_stamps(t.stream, ds);
                if (st == Status::Succ) st = ex->clear_device_stamps(t.stream);
                if (st != Status::Succ) { sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel); break; }
                Tenant::StampSample smp;
                if ((queued > 0 || stop >= 0) && raised > 0 && drained >= raised && ds.last_exit) {
                    smp.raised = raised; smp.drained = drained; smp.exit = ds.last_exit;
                    smp.stop = stop >= 0 ? ds.stop_recorded : 0;
                    stop_ticks = smp.stop; exit_ticks = smp.exit;
                }
                if (t.resubmitted_ns && ds.first_claim) { smp.resubmitted = t.resubmitted_ns; smp.claim = ds.first_claim; }
                if (smp.raised || smp.resubmitted) t.stamp_samples.push_back(smp);
                t.resubmitted_ns = 0;
            }
            // a preemption-latency sample needs something to have been preempted: kernels in flight
            // when the request was noticed, or a kernel recorded as stopped.  (A request that finds
            // this tenant between two submissions waits for nothing.)
            if ((queued > 0 || stop >= 0) && raised > 0 && drained >= raised) {
                const double drain_us = (drained - raised) / 1e3;
                {
                    std::lock_guard<std::mutex> g(sh.stats_mu);
                    sh.preempt_latency.add(drain_us);
                }
                t.drains.push_back({drain_us, stop, queued});
                t.drains.back().raised = raised; t.drains.back().stop_ticks = stop_ticks; t.drains.back().exit_ticks = exit_ticks;
                t.drains.back().since_launch_us = (raised - first_launch_ns) / 1e3; t.drains.back().resumed = resumed;
            }
            while (sh.active_above(p) > 0) spin_pause();
            sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
            if (stop >= 0) { next = (size_t)stop; ++t.preemptions; resumed = true; first_launch_ns = 0; }  // kernels from the stopped one on are submitted again
            if (stop >= 0 && ex->device_stamps_enabled()) t.resubmitted_ns = now_ns();
            continue;
        }
        if (tracked) {
            const int waiting = ex->launches_submitted() - ex->launches_started();
            if (next < n && waiting < (last_flops >= 3e9 ? 1 : queue_depth())) {
                if (!first_launch_ns) first_launch_ns = now_ns();
                auto model = ex->get_model();
                last_flops = model ? model->get_kernel_info(next).flops : 0;
                st = ex->launch_kernel(next, t.stream);
                ++next;
                continue;
            }
            if (next >= n) {
                if (!tail_marked) {
                    st = ex->mark_stream(t.stream);
                    tail_marked = true;
                    continue;
                }
                if (ex->stream_left()) {
                    tail_marked = false;
                    // everything was submitted and has left the GPU; a late stop may still have cut it short
                    st = ex->getStopPoint(t.stream);
                    if (st == Status::Succ && ex->last_stop_index() >= 0) {
                        next = (size_t)ex->last_stop_index(); ++t.preemptions;
                        ex->restart_launch_tracking();
                        continue;
                    }
                    break;
                }
            }
            // (a launch that never reported its start would leave this loop waiting for it: the queue is asked now
            // and then, and an idle queue means that everything submitted has run)
            if ((++idle_spins & 0x3ffff) == 0) {
                int idle = 0;
                if (gp_stream_query(t.stream, &idle) != 0) { st = Status::Fail; break; }
                if (idle && !tail_marked) ex->restart_launch_tracking();
            }
            spin_pause();
            continue;
        }
        if (next < n && inflight < 2) {
            // (a kernel of 3 GFLOP and more, 10 us and up, ends its chunk: behind such kernels the host keeps up with one
            // chunk queued, and every queued kernel is one more to flush when a stop comes, 4-7 us apiece next to
            // VGG-16 b16)
            size_t end = next;
            double flops = 0;
            auto model = ex->get_model();
            while (end < n && end - next < (size_t)chunk_size()) {
                if (model) flops += model->get_kernel_info(end).flops;
                ++end;
                if (flops >= 3e9) break;
            }
            if (!first_launch_ns) first_launch_ns = now_ns();
            for (size_t i = next; i < end && st == Status::Succ; ++i) st = ex->launch_kernel(i, t.stream);
            if (st != Status::Succ) break;
            if (gp_event_record(t.chunk_events[tail], t.stream) != 0) { st = Status::Fail; break; }
            tail = (tail + 1) % 3;
            ++inflight;
            next = end;
            continue;
        }
        int done = 0;
        if (gp_event_query(t.chunk_events[head], &done) != 0) { st = Status::Fail; break; }
        if (done) { head = (head + 1) % 3; --inflight; }
        else spin_pause();
        if (next >= n && inflight == 0) {
            // everything was submitted and has left the GPU; a late stop may still have cut it short
            st = ex->getStopPoint(t.stream);
            if (st == Status::Succ && ex->last_stop_index() >= 0) { next = (size_t)ex->last_stop_index(); ++t.preemptions; }
        }
    }
    if (st == Status::Succ && t.resubmitted_ns && ex->device_stamps_enabled()) {
        BLPExecutor::DeviceStamps ds;
        if (ex->read_device_stamps(t.stream, ds) == Status::Succ && ds.first_claim) {
            Tenant::StampSample smp;
            smp.resubmitted = t.resubmitted_ns; smp.claim = ds.first_claim;
            t.stamp_samples.push_back(smp);
        }
        ex->clear_device_stamps(t.stream);
        t.resubmitted_ns = 0;
    }
    ex->running = false;
    sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
    return st;
}

// One inference under the policy.  Mirrors FooClient::infer of the reference's clients.
Status infer(Tenant &t, Shared &sh) {
    const int p = std::min(t.priority, sh.levels - 1);
    const std::string &pol = sh.policy;
    if (pol == "seq") {
        // seqclient.cpp:82-102: one model at a time; a best-effort tenant yields while a
        // latency-critical request is waiting.
        if (p > 0) while (sh.seq_waiting.load() > 0) spin_pause();
        else sh.seq_waiting.fetch_add(1);
        std::lock_guard<std::mutex> g(sh.seq_mu);
        RETURN_STATUS(t.ex->execute(t.stream));
        RETURN_STATUS(drain(t.stream));
        if (p == 0) sh.seq_waiting.fetch_sub(1);
        return Status::Succ;
    }
    if (!is_wb(pol)) {  // "np", "lco" and anything unknown
        // baseclient.cpp: every tenant submits on its own stream, nothing is preempted
        sh.serving(p, +1);
        Status st = t.ex->execute(t.stream);
        if (st == Status::Succ) st = drain(t.stream);
        sh.serving(p, -1);
        return st;
    }
    // ---- "wb": cooperative block-level preemption ------------------------------------------
    // (the request was announced by begin_request(): the flag words of every lower level are up)
    sh.serving(p, +1);
    // "wb" / "wb-chunk": wait until lower-priority work has left the GPU (blpclient.cpp:189);
    // "wb-async" submits at once and lets the hardware start workgroups as the others retire.
    if (!is_async(pol)) while (sh.on_gpu_below(p) > 0) spin_pause();
    Status st = Status::Succ;
    if (!t.blp) {
        if (t.gate_host) {
            // start_blocking_stream / end_blocking_stream of the reference (gpreemptclient.cpp:74-81,
            // 232-235): two gate kernels hold the stream while the request's kernels are queued
            // behind them, then one host store lets everything run back to back.  The wait is
            // bounded (about a second of polls), so a lost release cannot hang the device.
            *t.gate_host = 0;
            for (int i = 0; i < 2 && st == Status::Succ; ++i)
                if (gp_launch_gate((const int *)t.gate_dev, 1ull << 22, t.gate_timed_out, t.stream) != 0) st = Status::Fail;
        }
        if (st == Status::Succ) st = t.ex->execute(t.stream);
        if (t.gate_host) *t.gate_host = 1;
        if (st == Status::Succ) st = drain(t.stream);
    } else if (t.ex->graph_workload()) {
        // graph workloads drive their own loop inside execute() (graphcompute.tr.cu:142-174);
        // when stopped they come back here through wait_for_turn
        while (sh.active_above(p) > 0) spin_pause();
        t.blp->wait_for_turn = [&t, &sh, p]() {
            int64_t drained = now_ns();
            sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
            int64_t raised = sh.domain->raised_ns(p);
            if (sh.active_above(p) > 0 && raised > 0 && drained >= raised) {
                std::lock_guard<std::mutex> g(sh.stats_mu);
                sh.preempt_latency.add((drained - raised) / 1e3);
            }
            while (sh.active_above(p) > 0) spin_pause();
            sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
            ++t.preemptions;
        };
        sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
        st = t.blp->execute(t.stream);
        sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
    } else if (is_chunked(pol)) {
        while (sh.active_above(p) > 0) spin_pause();
        st = infer_chunked(t, sh, p);
    } else {
        // preemptible tenant (blpclient.cpp:163-183): run, and after every drain ask whether a
        // kernel was stopped; if so wait for the higher levels to finish and resume.
        while (sh.active_above(p) > 0) spin_pause();
        sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
        t.blp->running = true;
        st = t.blp->execute(t.stream);
        while (st == Status::Succ) {
            int64_t drained = 0;
            st = drain_blp(t.blp, t.stream, &drained);
            if (st != Status::Succ) break;
            const bool contended = sh.active_above(p) > 0;
            sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
            if (contended) {
                int64_t raised = sh.domain->raised_ns(p);
                if (raised > 0 && drained >= raised) {
                    std::lock_guard<std::mutex> g(sh.stats_mu);
                    sh.preempt_latency.add((drained - raised) / 1e3);
                }
                while (sh.active_above(p) > 0) spin_pause();
            }
            sh.on_gpu[p].fetch_add(1, std::memory_order_acq_rel);
            st = t.blp->resume(t.stream);  // reads the stop index; -1 means the model had finished
            if (st != Status::Succ) break;
            if (t.blp->last_stop_index() == -1) break;
            ++t.preemptions;
        }
        t.blp->running = false;
        sh.on_gpu[p].fetch_sub(1, std::memory_order_acq_rel);
    }
    sh.serving(p, -1);
    return st;
}

static bool preempting_policy(const Shared &sh) { return is_wb(sh.policy); }

// A request of level p announces itself before it touches the GPU at all (its input copy
// included): a persistent best-effort kernel leaves no gap for even a small copy kernel, so the
// flag has to go up first.  This is where the reference posts its pre-preemption hint
// (src/cuda-clients/gpreemptclient.cpp:203-219).  Raises the flag words of every lower level
// (blpclient.cpp:185-188); end_request() lowers them when the level has no request left.
// A tenant whose next request has arrived by the time this one ends (or will within hold_us) keeps its level up across
// the two ("hold_backlog", on by default; loads with arrival times only).  Lowering the flag words for the instant
// between two requests makes every lower level submit its stopped kernels again, and the raise that follows at once
// finds them on their way onto the GPU: they have to start, pick their work up and leave again, the longest
// preemptions there are (BERT-384 over the 8192^3 GEMM: 40-60 us of flag store to drained, one request in eight).
void begin_request(Tenant &t, Shared &sh) {
    if (!preempting_policy(sh)) return;
    if (t.holding) { t.holding = false; return; }  // the level is still up from the request before
    sh.domain->begin(t.priority);
}
void end_request(Tenant &t, Shared &sh) {
    if (!preempting_policy(sh)) return;
    if (sh.hold_backlog && t.preprocess_us == 0 && !sh.stop.load(std::memory_order_acquire)) {
        const int64_t f = t.load.following();
        if (f != 0 && f <= now_ns() + sh.hold_us * 1000) { t.holding = true; ++t.held; return; }
    }
    sh.domain->end(t.priority);
}

// One request: the six DISB phases (benchmark.cpp:66-135); prepareInput and postprocess are empty
// in the reference's clients, preprocess sleeps preprocess_time (blpclient.cpp:153-155).
static uint64_t fnv1a(const void *p, size_t n) {
    const unsigned char *b = (const unsigned char *)p;
    uint64_t h = 1469598103934665603ull;
    for (size_t i = 0; i < n; ++i) { h ^= b[i]; h *= 1099511628211ull; }
    return h;
}

Status infer_once(Tenant &t, Shared &sh, double *total_us, double *infer_us) {
    int64_t t0 = now_ns();
    std::shared_ptr<std::atomic<int>> hint;
    if (sh.hints && preempting_policy(sh) && t.preprocess_us > sh.hint_switch_us)
        hint = sh.hints->post(t0 + (t.preprocess_us - sh.hint_switch_us) * 1000, t.priority);
    if (t.preprocess_us > 0) {
        // the reference sleeps (blpclient.cpp:153-155); a sleep overshoots by 50+ us, so the tail is spun
        int64_t until = t0 + t.preprocess_us * 1000;
        if (t.preprocess_us > 200) std::this_thread::sleep_for(std::chrono::microseconds(t.preprocess_us - 150));
        while (now_ns() < until) spin_pause();
    }
    int64_t tp = now_ns();
    int expect = 0;
    if (!hint || hint->compare_exchange_strong(expect, 2)) begin_request(t, sh);  // else the daemon has begun it
    struct Retire { Tenant &t; Shared &sh; ~Retire() { end_request(t, sh); } } retire{t, sh};
    // "resident_io": operands stay in device memory (a 8192^2 matrix is 134 MB: copied per
    // request it would be the whole request); the input is uploaded once, the output never read back
    if (t.input_size && (!t.resident_io || !t.input_resident)) {
        RETURN_STATUS(t.ex->set_input("data", t.input, t.input_size, t.stream));
        CUDA_RETURN_STATUS(gp_stream_sync(t.stream));
        t.input_resident = true;
    }
    int64_t t1 = now_ns();
    RETURN_STATUS(infer(t, sh));
    int64_t t2 = now_ns();
    if (t.output_size && !t.resident_io) {
        RETURN_STATUS(t.ex->get_output("heads", t.output, t.output_size, t.stream));
        CUDA_RETURN_STATUS(gp_stream_sync(t.stream));
    }
    int64_t t3 = now_ns();
    *total_us = (t3 - t0) / 1e3;
    *infer_us = (t2 - t1) / 1e3;
    t.phase_sum_us[0] += (tp - t0) / 1e3; t.phase_sum_us[1] += (t1 - tp) / 1e3;
    t.phase_sum_us[2] += (t2 - t1) / 1e3; t.phase_sum_us[3] += (t3 - t2) / 1e3;
    if (sh.verify_outputs && t.output_size && !t.resident_io) {
        // same input every time, deterministic kernels: every request's output has the same bits,
        // however often the tenant was stopped and resumed on the way
        const uint64_t h = fnv1a(t.output, t.output_size);
        if (!t.have_ref_hash) { t.ref_hash = h; t.have_ref_hash = true; }
        else if (h != t.ref_hash) ++t.output_mismatches;
    }
    return Status::Succ;
}

void tenant_thread(Tenant *t, Shared *sh, std::atomic<int> *ready, int n_tasks, int64_t begin, int64_t end) {
    bind_core(sh->cores.fetch_add(1));  // blpclient.cpp:147
    util::init_cuda();
    ready->fetch_add(1);
    while (ready->load() < n_tasks) spin_pause();
    t->load.start(begin, end);
    int64_t scheduled = 0;
    bool counted = false;
    while (!sh->stop.load(std::memory_order_acquire) && t->load.wait_next(&scheduled)) {
        if (sh->stop.load(std::memory_order_acquire)) break;
        double total = 0, inf = 0;
        int64_t start = now_ns();
        Status s = infer_once(*t, *sh, &total, &inf);
        if (s != Status::Succ) { t->error = s; break; }
        if (t->first_latencies.size() < 32) t->first_latencies.push_back(total);
        if (t->priority == 0 && t->discarded < sh->corun_discard) { ++t->discarded; continue; }
        if (t->requests == 0) t->first_ns = start;
        t->last_ns = now_ns();
        ++t->requests;
        t->total.add(total);
        t->infer.add(inf);
        t->queueing.add((start - scheduled) / 1e3);
        if (sh->hp_requests > 0 && t->priority == 0 && !counted && t->requests >= sh->hp_requests) {
            counted = true;
            if (sh->hp_unfinished.fetch_sub(1) == 1) sh->stop.store(true, std::memory_order_release);
            break;
        }
    }
    if (sh->hp_requests > 0 && t->priority == 0 && !counted && sh->hp_unfinished.fetch_sub(1) == 1) sh->stop.store(true, std::memory_order_release);
    if (t->holding) { t->holding = false; sh->domain->end(t->priority); }  // no request followed after all
}

}  // namespace

Status run_scenario(const std::string &config_text, std::string &report_text) {
    json::Value cfg;
    if (!json::parse(config_text, cfg) || cfg.type != json::Value::Object) {
        std::fprintf(stderr, "scenario: malformed JSON\n");
        return Status::Fail;
    }
    util::init_cuda();
    Shared sh;
    sh.policy = cfg["policy"].string("wb");
    double seconds = cfg["time"].number(5);
    int standalone_runs = (int)cfg["standalone_runs"].number(kStandAloneRuns);
    int warmups = (int)cfg["warmups"].number(kWarmups);
    sh.hp_requests = (long)cfg["hp_requests"].number(0);
    sh.verify_outputs = cfg["verify_outputs"].boolean(false);
    sh.hp_gate = cfg["hp_gate"].boolean(false);
    sh.device_stamps = cfg["device_stamps"].boolean(false);
    sh.corun_discard = (long)cfg["corun_discard"].number(0);
    sh.hold_backlog = cfg["hold_backlog"].boolean(true);
    sh.hold_us = (int64_t)cfg["hold_us"].number(30);
    const json::Value &tasks = cfg["tasks"];
    std::vector<std::unique_ptr<Tenant>> tenants;
    // Declared after `tenants`, so it runs first on every exit path: executors free device memory
    // when they are destroyed, and a free waits for the whole device, relay kernel included.
    struct RelayGuard { Shared &sh; ~RelayGuard() { if (sh.domain) sh.domain->stop_relay(); } } relay_guard{sh};
    int max_prio = 0;
    for (const json::Value &tv : tasks.arr) {
        std::unique_ptr<Tenant> t(new Tenant());
        const json::Value &c = tv["client"], &l = tv["load"];
        t->id = tv["id"].string(c["name"].string("task"));
        t->name = c["name"].string(t->id);
        t->model_name = c["model_name"].string();
        t->priority = (int)c["priority"].number(0);
        t->use_graph = c["use_cuda_graph"].boolean(true);
        t->resident_io = c["resident_io"].boolean(false);
        t->launch_mode = c["launch_mode"].string(t->use_graph ? "program" : "launch");
        t->preprocess_us = (int64_t)c["preprocess_time"].number(0);
        t->load.type = l["type"].string("continuous");
        t->load.frequency = l["frequency"].number(0);
        t->load.seed = (uint64_t)l["seed"].number(1 + (double)tenants.size());
        for (const json::Value &v : l["trace"].arr) t->load.trace_ms.push_back((int64_t)v.number(0));
        t->load.load_priority = (int)l["priority"].number(0);
        if (sh.policy == "lco" && t->priority != 0) continue;  // rtonlyclient.cpp:120-141: keep the real-time tasks only
        max_prio = std::max(max_prio, t->priority);
        tenants.push_back(std::move(t));
    }
    if (tenants.empty()) return Status::NotFound;
    sh.levels = std::min(max_prio + 1, kMaxLevels);
    if (sh.levels < 2) sh.levels = 2;
    const bool relay = cfg["flag_relay"].boolean(false);  // measured slower: a second resident kernel slows every launch
    sh.domain.reset(new PreemptDomain(sh.levels, relay));
    if (!sh.domain->ok()) return Status::Fail;
    // "pre_preempt_hint_us" > 0: tenants with a preprocess_time longer than that post hints
    sh.hint_switch_us = (int64_t)cfg["pre_preempt_hint_us"].number(0);
    if (sh.hint_switch_us > 0) sh.hints.reset(new HintDaemon(sh.domain.get()));
    for (auto &t : tenants) RETURN_STATUS(init_tenant(*t, sh));

    // warm-up and stand-alone latency, one tenant at a time (benchmark.cpp:221-299)
    for (auto &t : tenants) {
        for (int i = 0; i < warmups + standalone_runs; ++i) {
            double total = 0, inf = 0;
            RETURN_STATUS(infer_once(*t, sh, &total, &inf));
            if (i >= warmups) t->standalone.add(total);
        }
        t->preemptions = 0;
        for (double &v : t->phase_sum_us) v = 0;
    }
    {
        std::lock_guard<std::mutex> g(sh.stats_mu);
        sh.preempt_latency = Stats();
    }
    for (int l = 0; l < kMaxLevels; ++l) sh.serving_above[l] = 0, sh.busy_above[l] = 0;
    // DISB's load coordinator (load.cpp:47-69): periodic loads of one frequency do not all fire at
    // the same instant; each starts later than the one before by the sum of that one's stand-alone
    // latencies ("stagger": false keeps them aligned)
    if (cfg["stagger"].boolean(true)) {
        std::map<long, int64_t> delay_by_freq;
        for (auto &t : tenants) {
            if (t->load.type != "periodic" || t->load.load_priority > 0) continue;
            const long f = (long)t->load.frequency;
            t->load.launch_delay = delay_by_freq[f];
            double sum_us = 0;
            for (double v : t->standalone.v) sum_us += v;
            delay_by_freq[f] += (int64_t)(sum_us * 1e3);
        }
    }

    // co-run
    for (auto &t : tenants) if (t->priority == 0) sh.hp_unfinished.fetch_add(1);
    std::atomic<int> ready{0};
    int64_t begin = now_ns() + 50 * 1000 * 1000;
    int64_t end = begin + (int64_t)(seconds * 1e9);
    std::vector<std::thread> threads;
    for (auto &t : tenants) threads.emplace_back(tenant_thread, t.get(), &sh, &ready, (int)tenants.size(), begin, end);
    for (auto &th : threads) th.join();
    double wall_s = (now_ns() - begin) / 1e9;

    json::Value rep = json::Value::object();
    rep.set("policy") = sh.policy;
    rep.set("time(s)") = wall_s;
    json::Value &jt = rep.set("tasks");
    jt = json::Value::object();
    double hp_ratio = 0, be_kept = 0;
    int n_hp = 0, n_be = 0;
    auto busy_fraction = [&](int level) { return std::min(1.0, sh.busy_above[std::min(std::max(level, 1), sh.levels - 1)] / 1e9 / std::max(wall_s, 1e-9)); };
    double busy_frac = busy_fraction(1);
    Status result = Status::Succ;
    for (auto &t : tenants) {
        json::Value &o = jt.set(t->id);
        o = json::Value::object();
        o.set("model") = t->model_name;
        o.set("priority") = t->priority;
        o.set("kernels") = t->ex->get_kernel_num();
        o.set("requests") = (long)t->requests;
        double span = t->requests > 0 ? (t->last_ns - t->first_ns) / 1e9 : 0;
        double thr = span > 0 ? t->requests / span : 0;
        o.set("avgThroughput(req/s)") = thr;
        o.set("avgTotalLatency(us)") = t->total.mean();
        o.set("standAloneTotalLatency(us)") = t->standalone.mean();
        o.set("avgTotalLatencyIncrease(us)") = t->total.mean() - t->standalone.mean();
        o.set("totalLatency(us)") = t->total.to_json();
        o.set("inferLatency(us)") = t->infer.to_json();
        o.set("queueing(us)") = t->queueing.to_json();
        o.set("standAlone(us)") = t->standalone.to_json();
        o.set("preemptions") = (long)t->preemptions;
        o.set("levelHeldAcrossRequests") = t->held;
        double alone_thr = t->standalone.mean() > 0 ? 1e6 / t->standalone.mean() : 0;
        o.set("standAloneThroughput(req/s)") = alone_thr;
        if (t->priority == 0) {
            double r = t->standalone.pct(0.99) > 0 ? t->total.pct(0.99) / t->standalone.pct(0.99) : 0;
            o.set("p99_vs_isolated") = r;
            hp_ratio = std::max(hp_ratio, r);
            ++n_hp;
        } else if (t->load.type == "continuous") {
            // throughput the idle gaps allow = isolated throughput x fraction of time without a
            // request of a higher level being served
            double allowed = alone_thr * (1.0 - busy_fraction(t->priority));
            o.set("higher_levels_busy_fraction") = busy_fraction(t->priority);
            double kept = allowed > 0 ? thr / allowed : 0;
            o.set("throughput_kept") = kept;
            be_kept += kept;
            ++n_be;
        }
        if (!t->drains.empty()) {
            std::sort(t->drains.begin(), t->drains.end(), [](const Tenant::Drain &a, const Tenant::Drain &b) { return a.us > b.us; });
            json::Value &sd = o.set("slowestDrains");
            sd = json::Value::array();
            auto model = t->ex->get_model();
            for (size_t i = 0; i < t->drains.size() && i < 12; ++i) {
                json::Value e = json::Value::object();
                e.set("us") = t->drains[i].us;
                e.set("stopKernel") = t->drains[i].stop_kernel;
                e.set("chunksInFlight") = t->drains[i].queued;
                e.set("sinceSubmission(us)") = t->drains[i].since_launch_us;
                e.set("resumedBefore") = t->drains[i].resumed;
                if (t->blp && t->blp->device_stamps_enabled() && t->drains[i].exit_ticks && t->blp->calibrate_device_clock(t->stream) == Status::Succ) {
                    if (t->drains[i].stop_ticks) e.set("flagStore_to_stopRecorded(us)") = (t->blp->device_ticks_to_ns(t->drains[i].stop_ticks) - t->drains[i].raised) / 1e3;
                    e.set("flagStore_to_lastWorkgroupExit(us)") = (t->blp->device_ticks_to_ns(t->drains[i].exit_ticks) - t->drains[i].raised) / 1e3;
                }
                if (model && t->drains[i].stop_kernel >= 0 && (size_t)t->drains[i].stop_kernel < model->get_kernel_num()) {
                    KernelInfo &k = model->get_kernel_info(t->drains[i].stop_kernel);
                    e.set("name") = k.name;
                    e.set("tiles") = k.total_blocks;
                    e.set("gflop") = k.flops / 1e9;
                }
                sd.push(e);
            }
        }
        {
            json::Value &fl = o.set("firstLatencies(us)");
            fl = json::Value::array();
            for (double v : t->first_latencies) fl.push(json::Value(v));
            if (t->discarded) o.set("discardedRequests") = (long)t->discarded;
        }
        if (sh.verify_outputs) o.set("outputMismatches") = t->output_mismatches;
        if (t->error != Status::Succ) { o.set("error") = status_name(t->error); result = t->error; }
    }
    // The same run in the shape DISB writes and the reference's scripts/plot/plot.py reads
    // (third_party/disb/src/benchmark.cpp:340-354, client.cpp:74-87, analyzer.cpp:90-170): one entry
    // per client with its analyzers' reports; latencies are whole microseconds, the throughput is
    // requests over the whole benchmark time.
    {
        auto stamp = [](std::chrono::system_clock::time_point tp) {
            char buf[25] = {0};
            time_t tt = std::chrono::system_clock::to_time_t(tp);
            struct tm lt;
            localtime_r(&tt, &lt);
            strftime(buf, sizeof(buf), "%Y-%m-%d %H:%M:%S", &lt);
            return std::string(buf);
        };
        const auto wall_end = std::chrono::system_clock::now();
        const auto wall_begin = wall_end - std::chrono::nanoseconds((int64_t)(wall_s * 1e9));
        rep.set("beginTime") = stamp(wall_begin);
        rep.set("endTime") = stamp(wall_end);
        rep.set("benchmarkTime(s)") = (long)wall_s;
        json::Value &results = rep.set("results");
        results = json::Value::array();
        for (auto &t : tenants) {
            json::Value a = json::Value::object();
            const double n = (double)std::max<int64_t>(t->requests, 1);
            const long pre = (long)(t->phase_sum_us[0] / n), cin = (long)(t->phase_sum_us[1] / n), inf = (long)(t->phase_sum_us[2] / n),
                       cout = (long)(t->phase_sum_us[3] / n);
            const long total = t->requests > 0 ? pre + cin + inf + cout : 0, alone = (long)t->standalone.mean();
            a.set("type") = "basic";
            a.set("avgThroughput(req/s)") = t->requests > 0 && wall_s > 0 ? t->requests / wall_s : 0.0;
            a.set("standAloneTotalLatency(us)") = alone;
            a.set("avgPrepareInputLatency(us)") = 0L;
            a.set("avgPreprocessLatency(us)") = t->requests > 0 ? pre : 0L;
            a.set("avgCopyInputLatency(us)") = t->requests > 0 ? cin : 0L;
            a.set("avgInferLatency(us)") = t->requests > 0 ? inf : 0L;
            a.set("avgCopyOutputLatency(us)") = t->requests > 0 ? cout : 0L;
            a.set("avgPostprocessLatency(us)") = 0L;
            a.set("avgTotalLatency(us)") = total;
            a.set("avgTotalLatencyIncrease(us)") = total - alone;
            json::Value c = json::Value::object();
            c.set("clientName") = t->name;
            json::Value &an = c.set("analyzers");
            an = json::Value::array();
            an.push(a);
            results.push(c);
        }
    }
    rep.set("hp_busy_fraction") = busy_frac;
    rep.set("hp_p99_vs_isolated") = hp_ratio;
    rep.set("be_throughput_kept") = n_be ? be_kept / n_be : 0.0;
    rep.set("preemptLatency(us)") = sh.preempt_latency.to_json();
    rep.set("hints_fired") = (double)(sh.hints ? sh.hints->fired() : 0);
    if (sh.device_stamps) {
        // device ticks -> host clock through a second calibration now, a run's length after the first
        Stats raise_to_stop, stop_to_exit, raise_to_exit, exit_to_host, resub_to_claim;
        for (auto &t : tenants) {
            if (!t->blp || !t->blp->device_stamps_enabled()) continue;
            if (t->blp->calibrate_device_clock(t->stream) != Status::Succ) continue;
            for (const Tenant::StampSample &m : t->stamp_samples) {
                if (m.raised && m.exit) {
                    const int64_t ex_ns = t->blp->device_ticks_to_ns(m.exit);
                    raise_to_exit.add((ex_ns - m.raised) / 1e3);
                    exit_to_host.add((m.drained - ex_ns) / 1e3);
                    if (m.stop && m.exit >= m.stop) {
                        const int64_t st_ns = t->blp->device_ticks_to_ns(m.stop);
                        raise_to_stop.add((st_ns - m.raised) / 1e3);
                        stop_to_exit.add((ex_ns - st_ns) / 1e3);
                    }
                }
                if (m.resubmitted && m.claim) resub_to_claim.add((t->blp->device_ticks_to_ns(m.claim) - m.resubmitted) / 1e3);
            }
        }
        json::Value &ds = rep.set("deviceStamps(us)");
        ds = json::Value::object();
        ds.set("flagStore_to_lastWorkgroupExit") = raise_to_exit.to_json();
        ds.set("lastWorkgroupExit_to_hostNotices") = exit_to_host.to_json();
        ds.set("flagStore_to_stopRecorded") = raise_to_stop.to_json();
        ds.set("stopRecorded_to_lastWorkgroupExit") = stop_to_exit.to_json();
        ds.set("resubmission_to_firstTileClaimed") = resub_to_claim.to_json();
    }
    report_text = rep.dump();

    sh.hints.reset();         // joins the daemon before the domain goes
    sh.domain->stop_relay();  // frees below synchronise the device
    for (auto &t : tenants) {
        t->ex->clear();
        gp_host_free(t->input);
        gp_host_free(t->output);
        for (gp_event e : t->chunk_events) if (e) gp_event_destroy(e);
        if (t->gate_host) gp_flag_destroy(t->gate_host);
        if (t->gate_timed_out) gp_free(t->gate_timed_out);
        gp_stream_destroy(t->stream);
    }
    tenants.clear();
    sh.domain.reset();
    return result;
}

// Per-kernel preemption and resume latency of one best-effort model: the model runs back to
// back; an injector raises the flag at random instants, waits for the stream to drain, notes
// which kernel was stopped (the stop index) and how long the drain took, then clears the flag
// and the model resumes.
// Kernels [from, n) of the executor's model submitted one by one, never more than queue_depth() launches ahead of the
// GPU (one, behind a kernel of 3 GFLOP or more), as infer_chunked does for a tenant.  With raise_at != 0 the flag goes
// up at that time (CLOCK_MONOTONIC nanoseconds) wherever the submission stands, and nothing more is submitted;
// *raised then holds the time of the store.  Returns with the stream drained.
static Status submit_tracked(BLPExecutor &ex, GPUstream stream, size_t from, volatile int *flag_host, int64_t raise_at, int64_t *raised) {
    const size_t n = ex.get_kernel_num();
    auto model = ex.get_model();
    ex.restart_launch_tracking();
    size_t next = from;
    double last_flops = 0;
    bool marked = false;
    for (;;) {
        if (raise_at && !*raised && now_ns() >= raise_at) {
            *raised = now_ns();
            *flag_host = 1;
            break;
        }
        const int waiting = ex.launches_submitted() - ex.launches_started();
        if (next < n && waiting < (last_flops >= 3e9 ? 1 : queue_depth())) {
            last_flops = model ? model->get_kernel_info(next).flops : 0;
            RETURN_STATUS(ex.launch_kernel(next, stream));
            ++next;
            continue;
        }
        if (next >= n) {
            if (!marked) { RETURN_STATUS(ex.mark_stream(stream)); marked = true; }
            else if (ex.stream_left() && !(raise_at && !*raised)) return Status::Succ;  // (a probe waits for its instant)
        }
        spin_pause();
    }
    return drain_marked(&ex, stream);
}

Status preempt_probe(const std::string &workload, int trials, int use_graph, uint64_t seed, std::string &report_text) {
    util::init_cuda();
    BLPExecutor ex;
    RETURN_STATUS(ex.init(workload));
    volatile int *flag_host = nullptr;
    void *flag_dev = nullptr;
    CUDA_RETURN_STATUS(gp_flag_create(&flag_host, &flag_dev));
    ex.dpStop = flag_dev;
    GPUstream stream;
    CUDA_RETURN_STATUS(gp_stream_create(1, &stream));
    // use_graph: 0 = every kernel launched at once (execute), 1 = the captured form (the whole-model program), 2 = kernel
    // by kernel with a bounded queue, which is how the scenario runner feeds a best-effort tenant
    const bool tracked = use_graph == 2;
    if (use_graph == 1) ex.capture_graph(stream);
    if (tracked) RETURN_STATUS(ex.enable_launch_tracking());
    // the GPU's own time stamps ride along (GPREEMPT_PROBE_STAMPS=0 switches them off)
    const char *ps = getenv("GPREEMPT_PROBE_STAMPS");
    const bool stamps = !(ps && *ps == '0') && ex.enable_device_stamps(stream) == Status::Succ;
    struct ProbeSample { int64_t raised, drained, r0; unsigned long long stop, exit, claim; };
    std::vector<ProbeSample> probe_samples;
    size_t n = ex.get_kernel_num();
    // isolated duration of one inference
    Stats iso;
    for (int i = 0; i < 12; ++i) {
        int64_t t0 = now_ns();
        if (tracked) {
            RETURN_STATUS(ex.reset_counters(stream));
            RETURN_STATUS(submit_tracked(ex, stream, 0, flag_host, 0, nullptr));
        } else {
            RETURN_STATUS(ex.execute(stream));
            RETURN_STATUS(drain(stream));
        }
        if (i >= 2) iso.add((now_ns() - t0) / 1e3);
    }
    double span_us = iso.mean();
    std::vector<Stats> per_kernel(n), per_kernel_resume(n);
    Stats all, all_resume;
    numeric::Rng rng(seed);
    int hits = 0;
    for (int tr = 0; tr < trials; ++tr) {
        ex.running = true;
        int64_t wait = (int64_t)(rng.uniform01() * span_us * 0.95 * 1e3);
        int64_t raised = 0;
        if (tracked) {
            RETURN_STATUS(ex.reset_counters(stream));
            RETURN_STATUS(submit_tracked(ex, stream, 0, flag_host, now_ns() + wait, &raised));
        } else {
            RETURN_STATUS(ex.execute(stream));
            int64_t t0 = now_ns();
            while (now_ns() - t0 < wait) spin_pause();
            raised = now_ns();
            *flag_host = 1;
            RETURN_STATUS(drain(stream));
        }
        int64_t drained = now_ns();
        *flag_host = 0;
        BLPExecutor::DeviceStamps ds;
        if (stamps) {
            RETURN_STATUS(ex.read_device_stamps(stream, ds));
            RETURN_STATUS(ex.clear_device_stamps(stream));
            RETURN_STATUS(drain(stream));
        }
        int64_t r0 = now_ns();
        int64_t r1 = r0;
        int stop = -1;
        if (tracked) {
            // the tenant's resume: read the stop index back, submit from the stopped kernel on
            RETURN_STATUS(ex.getStopPoint(stream));
            stop = ex.last_stop_index();
            r1 = now_ns();
            if (stop >= 0) RETURN_STATUS(submit_tracked(ex, stream, (size_t)stop, flag_host, 0, nullptr));
        } else {
            RETURN_STATUS(ex.resume(stream));
            r1 = now_ns();
            stop = ex.last_stop_index();
            RETURN_STATUS(drain(stream));
        }
        if (stamps && stop >= 0) {
            BLPExecutor::DeviceStamps rs;
            RETURN_STATUS(ex.read_device_stamps(stream, rs));
            probe_samples.push_back({raised, drained, r0, ds.stop_recorded, ds.last_exit, rs.first_claim});
            RETURN_STATUS(ex.clear_device_stamps(stream));
        }
        if (stop >= 0 && (size_t)stop < n) {
            ++hits;
            per_kernel[stop].add((drained - raised) / 1e3);
            per_kernel_resume[stop].add((r1 - r0) / 1e3);
            all.add((drained - raised) / 1e3);
            all_resume.add((r1 - r0) / 1e3);
        }
        ex.running = false;
    }
    json::Value rep = json::Value::object();
    rep.set("workload") = workload;
    rep.set("kernels") = n;
    rep.set("trials") = trials;
    rep.set("interrupted") = hits;
    rep.set("isolated(us)") = iso.to_json();
    rep.set("preemptLatency(us)") = all.to_json();
    rep.set("resumeCall(us)") = all_resume.to_json();
    if (stamps && ex.calibrate_device_clock(stream) == Status::Succ) {
        Stats st_raise_to_stop, st_stop_to_exit, st_exit_to_host, st_resume_to_claim;
        for (const ProbeSample &m : probe_samples) {
            if (m.stop && m.exit >= m.stop) {
                const int64_t st_ns = ex.device_ticks_to_ns(m.stop), ex_ns = ex.device_ticks_to_ns(m.exit);
                st_raise_to_stop.add((st_ns - m.raised) / 1e3);
                st_stop_to_exit.add((ex_ns - st_ns) / 1e3);
                st_exit_to_host.add((m.drained - ex_ns) / 1e3);
            }
            if (m.claim) st_resume_to_claim.add((ex.device_ticks_to_ns(m.claim) - m.r0) / 1e3);  // resume() entered -> first tile claimed
        }
        json::Value &dsj = rep.set("deviceStamps(us)");
        dsj = json::Value::object();
        dsj.set("flagStore_to_stopRecorded") = st_raise_to_stop.to_json();
        dsj.set("stopRecorded_to_lastWorkgroupExit") = st_stop_to_exit.to_json();
        dsj.set("lastWorkgroupExit_to_hostNotices") = st_exit_to_host.to_json();
        dsj.set("resumeEntered_to_firstTileClaimed") = st_resume_to_claim.to_json();
    }
    json::Value &pk = rep.set("perKernel");
    pk = json::Value::array();
    auto model = ex.get_model();
    for (size_t i = 0; i < n; ++i) {
        if (per_kernel[i].v.empty()) continue;
        json::Value o = json::Value::object();
        o.set("kernel") = i;
        o.set("name") = model->get_kernel_info(i).name;
        // known once the kernel has been launched on its own (not when the whole model runs as one program)
        if (model->get_kernel_info(i).total_blocks > 0) o.set("tiles") = model->get_kernel_info(i).total_blocks;
        o.set("samples") = per_kernel[i].v.size();
        o.set("preempt_mean(us)") = per_kernel[i].mean();
        o.set("preempt_max(us)") = per_kernel[i].max();
        o.set("resume_mean(us)") = per_kernel_resume[i].mean();
        pk.push(o);
    }
    report_text = rep.dump();
    ex.clear();
    gp_stream_destroy(stream);
    gp_flag_destroy(flag_host);
    return Status::Succ;
}

}  // namespace foo
