// foo::Executor / BaseExecutor / BLPExecutor — the model-level API of the preemptible executor:
// load, set input, submit, preempt (by the shared flag), resume, read output.
//
// Interface of the reference's include/executor.h:14-84: same class names, method names,
// argument meaning, public data members (BLPExecutor::dpStop, BLPExecutor::running) and Status
// results.  Workload names select natively built models ("resnet152", "bert", "miniweather", ...)
// or one of the graph workloads ("cc", "bfs", "pagerank", "sssp"), which run a host loop of their
// own inside execute() as in the reference (src/executor.cpp:125-130, :226-228).
#pragma once
#include <atomic>
#include <functional>
#include <memory>
#include <string>
#include <vector>
#include "model.h"
#include "workloads/graphcompute.h"

namespace foo {

class Executor {
public:
    Status set_graph_path(const std::string &path);

    // model_path = <MODEL_PATH>/<workload>; the workload's graph is built natively.
    virtual Status load_model(std::string model_path);
    // Loads <model_path>/mod.params when it exists; otherwise the seeded random init stays.
    virtual Status load_param(std::string model_path);

    // Submits the whole model asynchronously on `stream`.
    virtual Status execute(GPUstream stream);
    virtual Status launch_kernel(size_t kernel_offset, GPUstream stream = 0);

    // Root directory of model files: $GPREEMPT_MODEL_PATH, else "./model".
    virtual Status init(std::string workload);
    virtual Status set_input(const std::string &key, void *value, size_t len, GPUstream stream);
    virtual Status set_input(const std::string &key, std::vector<float> &value, GPUstream stream);
    virtual Status get_output(const std::string &key, void *value, size_t len, GPUstream stream);
    virtual Status get_output(const std::string &key, std::vector<float> &value, GPUstream stream);
    virtual size_t get_data_size(const std::string &key);

    virtual void clear();
    size_t get_kernel_num() const;
    // Prepares the launch-free submission path: by default the whole model becomes one
    // persistent device kernel (a "program"); with GPREEMPT_USE_HIPGRAPH=1 in the environment a
    // HIP graph of the per-kernel launches is captured instead, as the reference does.
    virtual void capture_graph(GPUstream stream);
    virtual ~Executor();

    // additions over the reference
    std::shared_ptr<Model> get_model() const { return model; }
    bool uses_graph() const { return use_cuda_graph; }
    bool uses_program() const { return use_program; }
    // the graph workload behind a "cc" / "bfs" / "pagerank" / "sssp" executor (else null)
    GraphCompute::Workload *graph_workload() const { return graph_compute.get(); }

protected:
    std::shared_ptr<Model> model;
    std::string type;
    bool use_cuda_graph = false;  // a launch-free path is active (program or HIP graph)
    bool use_program = false;     // ... and it is the persistent program
    GPUgraphExec graph_exec = nullptr;
    std::string graph_path;
    std::unique_ptr<GraphCompute::Workload> graph_compute;
    // "cc@n=..,deg=..,seed=.." builds a seeded random graph; set_graph_path() (or
    // $GPREEMPT_GRAPH_PATH) names <base> of <base>.col/.dst/.val files instead
    Status init_graph(const std::string &kind, const std::string &options);
};

class BaseExecutor : public Executor {
public:
    BaseExecutor();
    virtual ~BaseExecutor();
};

class BLPExecutor : public Executor {
public:
    BLPExecutor();
    virtual ~BLPExecutor();
    // Reads the stop index back (blocks on `stream`); re-arms it to -1 when a kernel was stopped.
    Status getStopPoint(GPUstream stream);
    // Relaunches kernels [stop index, N) without resetting their tile counters.
    Status resume(GPUstream stream);
    virtual Status init(std::string workload) override;
    virtual Status execute(GPUstream stream) override;
    virtual Status launch_kernel(size_t kernel_offset, GPUstream stream = 0) override;
    virtual void capture_graph(GPUstream stream) override;
    virtual void clear() override;
    void set_lc_be_tasks(std::atomic<int> &lc_tasks, std::atomic<int> &be_tasks) {
        this->lc_tasks = &lc_tasks;
        this->be_tasks = &be_tasks;
    }

    // additions over the reference (test and measurement hooks)
    int last_stop_index() const { return stopIndex; }
    // Arms deterministic preemption: the workgroup whose claim on kernel `kernel` returns
    // `claim` raises the flag itself.  Applies to the next execute()/resume(); -1 disarms.
    void inject_preempt(int kernel, int claim) { inject_kernel = kernel; inject_claim = claim; }
    // graph workloads: the same hook for iteration `iteration` of the host loop (-1 = set-up kernels)
    void inject_preempt_graph(int iteration, int kernel, int claim) { inject_iteration = iteration; inject_kernel = kernel; inject_claim = claim; }
    Status read_counters(std::vector<int> &out);
    // Zeroes every tile counter on `stream` (what execute() does first), for callers that
    // launch kernel by kernel.
    Status reset_counters(GPUstream stream);
    // True once every workgroup of the last program launch has left the GPU (read from a host
    // word the kernel sets; cheaper and earlier than a stream query).  Always false when the
    // executor is not in program mode.
    bool program_vacated() const;
    // Device-side time stamps of preemptions, a measurement mode (per-kernel launches only; off by default).
    // What src/cuda-clients/blpclient.cpp:185-195 measures with the host's clock around a spin, taken on the
    // GPU: when the stop was recorded, when the tenant's last workgroup left, when the first tile was claimed
    // after a resume.  Raw device clock ticks; 0 = not written since the last clear.  The device clock drifts
    // against the host's by tens of microseconds per second, so the ticks are converted afterwards:
    // calibrate_device_clock() notes a (ticks, host time) pair (enable_device_stamps takes the first one), and
    // device_ticks_to_ns() interpolates between the first and the latest pair (CLOCK_MONOTONIC nanoseconds, good to
    // 1-2 us once two pairs a run apart exist).
    struct DeviceStamps { unsigned long long stop_recorded = 0, last_exit = 0, first_claim = 0; int exits = 0; };
    Status enable_device_stamps(GPUstream stream);
    Status read_device_stamps(GPUstream stream, DeviceStamps &out);   // blocks on `stream`
    Status clear_device_stamps(GPUstream stream);                      // a fill kernel on `stream`
    Status calibrate_device_clock(GPUstream stream);                   // blocks on `stream`
    int64_t device_ticks_to_ns(unsigned long long ticks) const;
    bool device_stamps_enabled() const { return stamps != nullptr; }

    // Flow control for a host that submits the model kernel by kernel (launch_kernel, src/executor.cpp:222-225) and
    // wants a bounded number of launches queued: after enable_launch_tracking() every preemptible launch stores its
    // number (1, 2, ... since the last restart) in a word of host memory when its first workgroup starts, i.e. when
    // all launches before it have left the GPU.  launches_submitted() - launches_started() are queued and have not
    // begun.  An event per few kernels does the same and costs the stream 3.7 us each on MI355X.
    Status enable_launch_tracking();
    bool launch_tracking_enabled() const { return started_host != nullptr; }
    int launches_submitted() const;
    int launches_started() const { return started_host ? *started_host : 0; }
    void restart_launch_tracking();  // only while nothing of this executor is in flight
    // mark_stream() puts a one-workgroup marker on the stream; stream_left() is true once it has run, i.e. once
    // everything submitted before it has left the GPU (a plain load of host memory, where a stream query costs
    // 3-5 us and is only as fresh as its last answer).
    Status mark_stream(GPUstream stream);
    bool stream_left() const { return mark_host && *mark_host == mark_seq; }

    // Claim counters per kernel.  The reference keeps one int per kernel (src/executor.cpp:333);
    // claims from several hundred workgroups serialise on a single address, so each kernel gets
    // 32 counters here, each owning a slice of the kernel's tiles.
    static constexpr int kCounterGroups = 32;
    static constexpr int kCounterStride = 16;  // ints between counters

public:
    GPUdeviceptr dpStop = nullptr;  // the preempt flag: allocated by the caller, shared by all best-effort tenants
    std::atomic<bool> running{false};
    // How often kernels read *dpStop: the claim numbered c reads it when c % poll_every == 0
    // (a power of two; 0 = the device layer's default, 8).  Use 1 when dpStop is device memory.
    int poll_every = 0;
    // Graph workloads: called by the workload's loop when it has been stopped; returns when the
    // workload may go back to the GPU.  Unset: the loop waits for *lc_tasks == 0 as in the
    // reference (set_lc_be_tasks).
    std::function<void()> wait_for_turn;

private:
    GPUdeviceptr dpStopIndex = nullptr;  // owned
    GPUdeviceptr executed = nullptr;     // owned: kCounterGroups tile counters per kernel, one per 64-byte line
    int stopIndex = -1;
    int *stop_host = nullptr;            // pinned landing slot for the stop index
    volatile int *left_host = nullptr;   // fine-grained host word written by a program's last leaving workgroup
    void *left_dev = nullptr;
    volatile int *started_host = nullptr;  // fine-grained host word: the number of the latest launch that has started
    void *started_dev = nullptr;
    volatile int *mark_host = nullptr;     // fine-grained host word of mark_stream()
    void *mark_dev = nullptr;
    int mark_seq = 0;
    GPUdeviceptr ckpt = nullptr;         // owned: checkpoint workspace of long GEMM tiles, or null
    size_t ckpt_bytes = 0;
    GPUdeviceptr stamps = nullptr;       // owned: GP_STAMP_WORDS 64-bit words, or null
    unsigned long long *stamps_host = nullptr;  // pinned landing area
    double stamp_tick_ns = 10.0;
    unsigned long long cal_ticks[2] = {0, 0};   // first and latest calibration: device ticks ...
    double cal_host_ns[2] = {0, 0};             // ... and the host clock at that moment
    int inject_kernel = -1, inject_claim = -1, inject_iteration = -2;
    std::atomic<int> *lc_tasks = nullptr;
    std::atomic<int> *be_tasks = nullptr;
};

}  // namespace foo
