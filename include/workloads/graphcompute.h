// Graph workloads (connected components, BFS, PageRank, SSSP) on the host side.
//
// Counterpart of the reference's include/workloads/graphcompute.h (namespaces GraphComputeRaw /
// GraphComputeBlp: read_graph, copy_gpu_graph, classes CC / BFS / PageRank / SSSP with
// compute(stream[, preempted, executed, lc_tasks, be_tasks])) and of the host loops in
// src/workloads/graphcompute.tr.cu:142-174 (CC), :257-285 (BFS), :450-495 (PageRank), :635-675
// (SSSP).  One class drives all four: an algorithm is a list of kernels per iteration plus a few
// host actions, and the loop that launches, notices a stop, waits for its turn and relaunches from
// the stopped kernel is shared (the reference repeats it with `goto resume` per algorithm).
#pragma once
#include <cstdint>
#include <functional>
#include <memory>
#include <string>
#include <vector>
#include "util/common.h"
#include "util/gpu_util.h"

namespace GraphCompute {


struct CsrGraph {
    uint64_t vertex_count = 0, edge_count = 0;
    std::vector<uint64_t> vertexList;   // vertex_count + 1 offsets into edgeList
    std::vector<uint64_t> edgeList;     // neighbour ids
    std::vector<uint32_t> weightList;   // per edge; empty when the graph has none
};

// Files <base>.col (offsets), <base>.dst (neighbours), <base>.val (weights, optional): each is
// a u64 element count, a u64 type tag and the payload (reference src/workloads/graphcompute.cu:16-45,
// graphcompute.tr.cu:618-627; the count in .col is vertex_count + 1).
Status read_graph(const std::string &base, CsrGraph &g, bool with_weights);
Status write_graph(const std::string &base, const CsrGraph &g);
// Seeded random graph for runs without the reference's dataset: every vertex gets `degree`
// distinct-source edges in each direction (symmetric), weights uniform in 1..64.
CsrGraph synthetic_graph(uint64_t vertices, unsigned degree, uint64_t seed);

// What a preemptible run needs from its executor (BLPExecutor's flag, stop index and counters).
struct PreemptEnv {
    GPUdeviceptr flag = nullptr, stop_index = nullptr, executed = nullptr;
    int counter_groups = 1, counter_stride = 1;   // counters of kernel k start at executed + k * groups * stride ints
    int poll_every = 0;
    std::function<bool()> higher_priority_active;  // true while this workload has to stay off the GPU
    // test hook: in iteration inject_iteration (0 = first loop iteration, -1 = the set-up kernels)
    // the claim `inject_claim` of kernel `inject_kernel` raises the flag itself; the loop clears the
    // flag again once the stop has been seen
    int inject_iteration = -2, inject_kernel = -1, inject_claim = -1;
};

class Workload {
public:
    // kind: "cc" | "bfs" | "pagerank" | "sssp"; nullptr for anything else (or sssp without weights)
    static std::unique_ptr<Workload> create(const std::string &kind, const CsrGraph &g);
    ~Workload();
    // Runs the algorithm to convergence on `stream` (blocking: the host reads the convergence
    // word every iteration, as the reference does).  env == nullptr: not preemptible.
    Status compute(GPUstream stream, const PreemptEnv *env);

    // results: "comp" (u64 per vertex), "label" (u32 BFS level), "value" (f32 PageRank), "cost" (u32 distance)
    size_t result_bytes(const std::string &key) const;
    Status read_result(const std::string &key, void *out, size_t len) const;
    const std::string &kind() const { return kind_; }
    uint64_t vertex_count() const { return n_; }
    uint64_t edge_count() const { return m_; }
    int iterations() const { return iterations_; }
    int preemptions() const { return preemptions_; }
    int kernels_launched() const { return launches_; }

private:
    Workload() = default;
    Status run_kernels(const std::vector<int> &kernels, GPUstream stream, const PreemptEnv *env, int iteration, bool *changed);
    Status begin(GPUstream stream);
    std::string kind_;
    uint64_t n_ = 0, m_ = 0;
    int iterations_ = 0, preemptions_ = 0, launches_ = 0;
    uint32_t level_ = 0;
    int lanes_ = 64;
    bool injected_ = false, flag_to_lower_ = false;  // test hook state (PreemptEnv::inject_*)
    // device arrays (owned)
    GPUdeviceptr vertex_list_ = nullptr, edge_list_ = nullptr, weight_list_ = nullptr;
    GPUdeviceptr label_ = nullptr, active_ = nullptr, next_active_ = nullptr, comp_ = nullptr;
    GPUdeviceptr delta_ = nullptr, residual_ = nullptr, value_ = nullptr, cost_ = nullptr, new_cost_ = nullptr;
    GPUdeviceptr changed_ = nullptr;
    int *host_words_ = nullptr;  // pinned: [0] stop index, [1] changed
};

}  // namespace GraphCompute
