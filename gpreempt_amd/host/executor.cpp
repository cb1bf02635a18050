// Executor launch loop and the block-level-preemption protocol on the host side.
// Behaviour follows the reference's src/executor.cpp (cited per function).
#include "executor.h"
#include "util/slice_map.h"

#include <algorithm>
#include <cstdlib>
#include <set>
#include <thread>

namespace foo {

static const std::set<std::string> kGraphCompute = {"cc", "bfs", "pagerank", "sssp"};  // reference executor.cpp:13

static void split_workload(const std::string &workload, std::string &name, std::string &options) {
    size_t at = workload.find('@');
    name = workload.substr(0, at);
    options = at == std::string::npos ? "" : workload.substr(at + 1);
}
static long option_int(const std::string &options, const std::string &key, long fallback) {
    size_t pos = 0;
    while (pos < options.size()) {
        size_t end = options.find(',', pos);
        if (end == std::string::npos) end = options.size();
        const std::string kv = options.substr(pos, end - pos);
        size_t eq = kv.find('=');
        if (eq != std::string::npos && kv.substr(0, eq) == key) return std::atol(kv.c_str() + eq + 1);
        pos = end + 1;
    }
    return fallback;
}

static std::string model_root() {
    const char *e = std::getenv("GPREEMPT_MODEL_PATH");
    return e && *e ? std::string(e) : std::string("./model");
}

Status Executor::set_graph_path(const std::string &path) {
    graph_path = path;
    return Status::Succ;
}

Executor::~Executor() {
    if (graph_exec) gp_graph_destroy(graph_exec);
}

// reference executor.cpp:23-45 (dnn branch)
// reference executor.cpp:26-34 (graph branch).  The reference reads its dataset from a fixed
// directory (:12) that does not ship with it; here the graph comes from set_graph_path(),
// $GPREEMPT_GRAPH_PATH or, by default, a seeded random graph.
Status Executor::init_graph(const std::string &kind, const std::string &options) {
    type = "graph";
    GraphCompute::CsrGraph g;
    const char *env = std::getenv("GPREEMPT_GRAPH_PATH");
    std::string base = !graph_path.empty() ? graph_path : (env && *env ? std::string(env) : std::string());
    if (!base.empty()) {
        RETURN_STATUS(GraphCompute::read_graph(base, g, kind == "sssp"));
    } else {
        long n = option_int(options, "n", 1 << 20), deg = option_int(options, "deg", 8), seed = option_int(options, "seed", 1);
        if (n < 2 || n >= (1L << 28) || deg < 1 || deg > 256 || n * deg > (1L << 27)) return Status::OutOfRange;  // at most 2^28 directed edges
        g = GraphCompute::synthetic_graph((uint64_t)n, (unsigned)deg, (uint64_t)seed);
    }
    graph_compute = GraphCompute::Workload::create(kind, g);
    return graph_compute ? Status::Succ : Status::Fail;
}

Status Executor::init(std::string workload) {
    std::string name, options;
    split_workload(workload, name, options);
    if (kGraphCompute.count(name)) return init_graph(name, options);
    type = "dnn";
    RETURN_STATUS(this->load_model(model_root() + "/" + workload));
    RETURN_STATUS(this->load_param(model_root() + "/" + workload));
    return Status::Succ;
}

// reference executor.cpp:47-95
Status Executor::set_input(const std::string &key, void *value, size_t len, GPUstream stream) {
    size_t idx;
    if (!model || model->find_storage_idx(key, idx) != Status::Succ) return Status::NotFound;
    return model->set(idx, value, len, stream);
}
Status Executor::set_input(const std::string &key, std::vector<float> &value, GPUstream stream) {
    return set_input(key, value.data(), value.size() * sizeof(float), stream);
}
Status Executor::get_output(const std::string &key, void *value, size_t len, GPUstream stream) {
    size_t idx;
    if (!model || model->find_storage_idx(key, idx) != Status::Succ) return Status::NotFound;
    return model->get(idx, value, len, stream);
}
Status Executor::get_output(const std::string &key, std::vector<float> &value, GPUstream stream) {
    return get_output(key, value.data(), value.size() * sizeof(float), stream);
}
size_t Executor::get_data_size(const std::string &key) {
    size_t idx;
    if (!model || model->find_storage_idx(key, idx) != Status::Succ) return 0;
    return model->get_storage_size(idx);
}

void Executor::clear() {
    if (model) model->clear();
}

// reference executor.cpp:110-117
Status Executor::load_model(std::string model_path) {
    model = std::make_shared<Model>();
    return model->load_model(model_path + "/mod.json", model_path + "/host.json", model_path + "/mod.co");
}
Status Executor::load_param(std::string model_path) { return model->load_param((model_path + "/mod.params").c_str()); }

// reference executor.cpp:119-134
Status Executor::execute(GPUstream stream) {
    if (graph_compute) return graph_compute->compute(stream, nullptr);
    if (use_program) return model->launch_program(stream, true);
    if (use_cuda_graph) {
        CUDA_RETURN_STATUS(gp_graph_launch(graph_exec, stream));
        return Status::Succ;
    }
    for (size_t i = 0; i < get_kernel_num(); i++) RETURN_STATUS(launch_kernel(i, stream));
    return Status::Succ;
}

// reference executor.cpp:136-164
Status Executor::launch_kernel(size_t kernel_offset, GPUstream stream) { return model->launch(kernel_offset, stream); }

size_t Executor::get_kernel_num() const { return model ? model->get_kernel_num() : 0; }

// reference executor.cpp:176-196.  On failure the executor stays in launch-by-launch mode.
static bool want_hipgraph() {
    const char *e = std::getenv("GPREEMPT_USE_HIPGRAPH");
    return e && *e && *e != '0';
}

void Executor::capture_graph(GPUstream stream) {
    if (graph_compute) return;  // a host loop cannot be captured (the reference records one iteration's launches, executor.cpp:183-186)
    if (graph_exec) { gp_graph_destroy(graph_exec); graph_exec = nullptr; }
    use_cuda_graph = false;
    use_program = false;
    if (!want_hipgraph()) {
        if (model && model->build_program() == Status::Succ) { use_cuda_graph = true; use_program = true; }
        else std::fprintf(stderr, "capture_graph: no program, staying with per-kernel launches\n");
        return;
    }
    if (gp_graph_begin(stream) != 0) return;
    model->counters_cleared(false);
    bool ok = true;
    for (size_t i = 0; i < get_kernel_num() && ok; i++) ok = launch_kernel(i, stream) == Status::Succ;
    gp_graph g = nullptr;
    if (gp_graph_end(stream, &g) != 0 || !ok) {
        if (g) gp_graph_destroy(g);
        std::fprintf(stderr, "capture_graph failed: %s\n", gp_last_error());
        return;
    }
    graph_exec = g;
    use_cuda_graph = true;
}

BaseExecutor::BaseExecutor() {}
BaseExecutor::~BaseExecutor() {}

BLPExecutor::BLPExecutor() {}

BLPExecutor::~BLPExecutor() {
    if (dpStopIndex) gp_free(dpStopIndex);
    if (executed) gp_free(executed);
    if (ckpt) gp_free(ckpt);
    if (stamps) gp_free(stamps);
    if (stamps_host) gp_host_free(stamps_host);
    if (stop_host) gp_host_free(stop_host);
    if (left_host) gp_flag_destroy(left_host);
    if (started_host) gp_flag_destroy(started_host);
    if (mark_host) gp_flag_destroy(mark_host);
}

bool BLPExecutor::program_vacated() const {
    return use_program && left_host && *left_host == model->last_launch_tag();
}

// reference executor.cpp:300-342 (dnn branch): build the model, allocate the stop index (-1) and
// one counter per kernel, append (flag, stop index) by reference to every kernel and the
// per-kernel preemption arguments, then load parameters.
Status BLPExecutor::init(std::string workload) {
    std::string name, options;
    split_workload(workload, name, options);
    if (kGraphCompute.count(name)) {
        // reference executor.cpp:304-316: stop index and three counters, then the workload
        RETURN_STATUS(init_graph(name, options));
        CUDA_RETURN_STATUS(gp_malloc(&dpStopIndex, sizeof(int)));
        CUDA_RETURN_STATUS(gp_fill32_async(dpStopIndex, 0xFFFFFFFFu, 1, nullptr));
        const size_t counter_ints = 3 * (size_t)kCounterGroups * kCounterStride;
        CUDA_RETURN_STATUS(gp_malloc(&executed, sizeof(int) * counter_ints));
        CUDA_RETURN_STATUS(gp_fill32_async(executed, 0, counter_ints, nullptr));
        CUDA_RETURN_STATUS(gp_stream_sync(nullptr));
        return Status::Succ;
    }
    type = "dnn";
    model = std::make_shared<Model>();
    std::string model_path = model_root() + "/" + workload;
    RETURN_STATUS(model->load_model(model_path + "/mod.json", model_path + "/host.json", model_path + "/mod.tr.co"));
    CUDA_RETURN_STATUS(gp_malloc(&dpStopIndex, sizeof(int)));
    CUDA_RETURN_STATUS(gp_host_alloc((void **)&stop_host, sizeof(int)));
    CUDA_RETURN_STATUS(gp_flag_create(&left_host, &left_dev));
    model->set_left_word(left_dev);
    stopIndex = -1;
    CUDA_RETURN_STATUS(gp_memcpy_h2d(dpStopIndex, &stopIndex, sizeof(int)));
    model->batchAddParam(&this->dpStop);
    model->batchAddParam(&this->dpStopIndex);
    // (twice the claim counters: behind them, laid out alike, the counters of workers that have left a launch of
    // long tiles; GPREEMPT_LONG_TILES=0 leaves them unused: such tiles are then finished, as the reference finishes them)
    const size_t counter_ints = model->get_kernel_num() * (size_t)kCounterGroups * kCounterStride;
    CUDA_RETURN_STATUS(gp_malloc(&executed, sizeof(int) * counter_ints * 2));
    CUDA_RETURN_STATUS(gp_fill32_async(executed, 0, counter_ints * 2, nullptr));
    CUDA_RETURN_STATUS(gp_stream_sync(nullptr));
    const char *lt = std::getenv("GPREEMPT_LONG_TILES");
    if (!(lt && *lt == '0')) model->set_done_counters(sizeof(int) * counter_ints);
    // GPREEMPT_SINGLE_COUNTER=1 selects the reference's one-counter-per-kernel layout (for A/B timing)
    const char *single = std::getenv("GPREEMPT_SINGLE_COUNTER");
    RETURN_STATUS(model->add_block_preemption_param(executed, (single && *single == '1') ? 1 : kCounterGroups));
    // long GEMM tiles may be left half-way: one slot per workgroup for their accumulators
    // (GPREEMPT_NO_CHECKPOINT=1 keeps the reference's "finish the tile you owe" for A/B timing)
    const char *nock = std::getenv("GPREEMPT_NO_CHECKPOINT");
    ckpt_bytes = (nock && *nock == '1') ? 0 : model->checkpoint_bytes_wanted();
    if (ckpt_bytes > 0) {
        CUDA_RETURN_STATUS(gp_malloc(&ckpt, ckpt_bytes));
        CUDA_RETURN_STATUS(gp_ckpt_reset_async(ckpt, nullptr));
        CUDA_RETURN_STATUS(gp_stream_sync(nullptr));
        model->set_checkpoint_workspace(ckpt, ckpt_bytes);
    }
    RETURN_STATUS(this->load_param(model_path));
    return Status::Succ;
}

Status BLPExecutor::launch_kernel(size_t kernel_offset, GPUstream stream) {
    model->set_poll_every(poll_every);
    int inject = ((int)kernel_offset == inject_kernel) ? inject_claim : -1;
    return model->launch(kernel_offset, stream, inject);
}

// reference executor.cpp:211-232: zero every tile counter, then launch (or replay the graph).
// The counters are cleared by a fill kernel outside the captured graph.
Status BLPExecutor::execute(GPUstream stream) {
    if (graph_compute) {
        // reference executor.cpp:226-228: the workload's own loop, handed the flag, the counters
        // and the two task counts; it returns when the algorithm has converged
        GraphCompute::PreemptEnv env;
        env.flag = dpStop; env.stop_index = dpStopIndex; env.executed = executed;
        env.counter_groups = kCounterGroups; env.counter_stride = kCounterStride; env.poll_every = poll_every;
        std::atomic<int> *lc = lc_tasks, *be = be_tasks;
        if (wait_for_turn) env.higher_priority_active = [this]() { wait_for_turn(); return false; };
        else if (lc) env.higher_priority_active = [lc, be]() {
            // waits here while a latency-critical task is active; meanwhile this workload is not
            // counted as running (the be_tasks.fetch_sub / fetch_add pair around the reference's
            // wait loops, graphcompute.tr.cu:163-165)
            if (lc->load() == 0) return false;
            if (be) be->fetch_sub(1);
            while (lc->load() != 0) std::this_thread::yield();
            if (be) be->fetch_add(1);
            return false;
        };
        env.inject_iteration = inject_iteration; env.inject_kernel = inject_kernel; env.inject_claim = inject_claim;
        return graph_compute->compute(stream, dpStop ? &env : nullptr);
    }
    model->set_poll_every(poll_every);
    if (use_program) return model->launch_program(stream, true, inject_kernel, inject_claim);
    RETURN_STATUS(reset_counters(stream));
    if (use_cuda_graph) {
        CUDA_RETURN_STATUS(gp_graph_launch(graph_exec, stream));
        model->launched_once_more();  // (a resume relaunches kernel by kernel and has to know)
        return Status::Succ;
    }
    for (size_t i = 0; i < get_kernel_num(); i++) RETURN_STATUS(launch_kernel(i, stream));
    return Status::Succ;
}

void BLPExecutor::capture_graph(GPUstream stream) { Executor::capture_graph(stream); }

void BLPExecutor::clear() {
    if (model) model->clear();
}

// reference executor.cpp:269-278
Status BLPExecutor::getStopPoint(GPUstream stream) {
    if (graph_compute) { stopIndex = -1; return Status::Succ; }  // the workload's loop resumes itself
    CUDA_RETURN_STATUS(gp_memcpy_d2h_async(stop_host, dpStopIndex, sizeof(int), stream));
    CUDA_RETURN_STATUS(gp_stream_sync(stream));
    stopIndex = *stop_host;
    if (stopIndex == -1) return Status::Succ;
    CUDA_RETURN_STATUS(gp_fill32_async(dpStopIndex, 0xFFFFFFFFu, 1, stream));
    return Status::Succ;
}

// reference executor.cpp:280-298: no-op unless running; kernels before the stop index completed,
// the one at the stop index continues from its counter, later ones start from zero claims.
// Always launch-by-launch, never through the captured graph.
Status BLPExecutor::resume(GPUstream stream) {
    if (!running || graph_compute) return Status::Succ;
    RETURN_STATUS(getStopPoint(stream));
    if (stopIndex == -1) return Status::Succ;
    // the program continues from its own per-layer counters; per-kernel mode relaunches one by one
    model->set_poll_every(poll_every);
    if (use_program) return model->launch_program(stream, false, inject_kernel, inject_claim);
    for (size_t i = (size_t)stopIndex; i < get_kernel_num(); i++) RETURN_STATUS(launch_kernel(i, stream));
    return Status::Succ;
}

Status BLPExecutor::enable_launch_tracking() {
    if (graph_compute || !model) return Status::Fail;
    if (started_host) return Status::Succ;
    CUDA_RETURN_STATUS(gp_flag_create(&started_host, &started_dev));
    *started_host = 0;
    model->set_started_word(started_dev);
    return Status::Succ;
}
Status BLPExecutor::mark_stream(GPUstream stream) {
    if (!mark_host) {
        CUDA_RETURN_STATUS(gp_flag_create(&mark_host, &mark_dev));
        *mark_host = 0;
    }
    mark_seq = mark_seq == 0x7fffffff ? 1 : mark_seq + 1;
    CUDA_RETURN_STATUS(gp_store_word_async(stream, (int *)mark_dev, mark_seq));
    return Status::Succ;
}
int BLPExecutor::launches_submitted() const { return model ? model->launch_number() : 0; }
void BLPExecutor::restart_launch_tracking() {
    if (!started_host || !model) return;
    *started_host = 0;
    model->restart_launch_numbers();
}

Status BLPExecutor::enable_device_stamps(GPUstream stream) {
    if (graph_compute || !model) return Status::Fail;
    if (stamps) return Status::Succ;
    RETURN_STATUS(calibrate_device_clock(stream));
    CUDA_RETURN_STATUS(gp_malloc(&stamps, sizeof(unsigned long long) * GP_STAMP_WORDS));
    CUDA_RETURN_STATUS(gp_host_alloc((void **)&stamps_host, sizeof(unsigned long long) * GP_STAMP_WORDS));
    RETURN_STATUS(clear_device_stamps(stream));
    CUDA_RETURN_STATUS(gp_stream_sync(stream));
    model->set_stamps(stamps);
    return Status::Succ;
}

Status BLPExecutor::clear_device_stamps(GPUstream stream) {
    if (!stamps) return Status::Fail;
    CUDA_RETURN_STATUS(gp_fill32_async(stamps, 0, 2 * (size_t)GP_STAMP_WORDS, stream));
    return Status::Succ;
}

Status BLPExecutor::read_device_stamps(GPUstream stream, DeviceStamps &out) {
    if (!stamps) return Status::Fail;
    CUDA_RETURN_STATUS(gp_memcpy_d2h_async(stamps_host, stamps, sizeof(unsigned long long) * GP_STAMP_WORDS, stream));
    CUDA_RETURN_STATUS(gp_stream_sync(stream));
    unsigned long long last = 0;
    out = DeviceStamps();
    for (int i = 0; i < GP_STAMP_EXIT_SLOTS; ++i) {
        const unsigned long long v = stamps_host[GP_STAMP_EXIT0 + i];
        if (v) ++out.exits;
        if (v > last) last = v;
    }
    out.stop_recorded = stamps_host[GP_STAMP_STOP];
    out.first_claim = stamps_host[GP_STAMP_FIRST_CLAIM];
    out.last_exit = last;
    return Status::Succ;
}

Status BLPExecutor::calibrate_device_clock(GPUstream stream) {
    double offset = 0;
    unsigned long long ticks = 0;
    CUDA_RETURN_STATUS(gp_device_clock(stream, 32, &stamp_tick_ns, &offset, &ticks));
    const int slot = cal_ticks[0] ? 1 : 0;
    cal_ticks[slot] = ticks;
    cal_host_ns[slot] = (double)ticks * stamp_tick_ns + offset;
    return Status::Succ;
}

int64_t BLPExecutor::device_ticks_to_ns(unsigned long long ticks) const {
    if (!ticks || !cal_ticks[0]) return 0;
    // between two calibrations the measured rate, with one the nominal rate
    double rate = stamp_tick_ns;
    if (cal_ticks[1] > cal_ticks[0] + 1000000ull) rate = (cal_host_ns[1] - cal_host_ns[0]) / (double)(cal_ticks[1] - cal_ticks[0]);
    return (int64_t)(cal_host_ns[0] + ((double)ticks - (double)cal_ticks[0]) * rate);
}

Status BLPExecutor::reset_counters(GPUstream stream) {
    if (graph_compute) return Status::Succ;
    CUDA_RETURN_STATUS(gp_fill32_async(executed, 0, 2 * model->get_kernel_num() * (size_t)kCounterGroups * kCounterStride, stream));
    if (ckpt) CUDA_RETURN_STATUS(gp_ckpt_reset_async(ckpt, stream));  // a fresh run has no tile to continue
    // launches recorded into a graph are replayed with the arguments of the recording: never fresh
    model->counters_cleared(!use_cuda_graph);
    return Status::Succ;
}

Status BLPExecutor::read_counters(std::vector<int> &out) {
    if (graph_compute) { out.clear(); return Status::Succ; }
    if (use_program) {
        std::vector<int> done;
        int error = 0;
        RETURN_STATUS(model->read_program_counters(out, done, error));
        return error ? Status::Timeout : Status::Succ;
    }
    // per-kernel claim count = sum over the counter groups, each clamped to its slice (a counter
    // overshoots by one per workgroup that found its slice handed out)
    const size_t n = model->get_kernel_num();
    std::vector<int> raw(n * (size_t)kCounterGroups * kCounterStride);
    CUDA_RETURN_STATUS(gp_memcpy_d2h(raw.data(), executed, sizeof(int) * raw.size()));
    out.assign(n, 0);
    for (size_t i = 0; i < n; ++i) {
        const long total = model->get_kernel_info(i).total_blocks;
        long sum = 0;
        if (model->counter_groups() == 1) { out[i] = raw[i]; continue; }
        // slices follow the workgroup distribution of the last launch (device layer, tile_loop.hpp)
        const long grid = std::max<long>(1, (long)model->get_kernel_info(i).launch_params[0] - model->get_kernel_info(i).front_workgroups);  // the workers
        if (model->get_kernel_info(i).fixed_claims) {  // int 0 of every line is an exact count
            for (int g = 0; g < kCounterGroups; ++g) sum += raw[(i * kCounterGroups + g) * kCounterStride];
            out[i] = (int)sum;
            continue;
        }
        auto begin = [&](int g) { return (long)gp::group_slice_begin((int)total, g, kCounterGroups, (int)grid); };
        for (int g = 0; g < kCounterGroups; ++g) {
            long size = begin(g + 1) - begin(g);
            long c = raw[(i * kCounterGroups + g) * kCounterStride];
            sum += total > 0 ? std::min(c, size) : c;
        }
        out[i] = (int)sum;
    }
    return Status::Succ;
}

}  // namespace foo
