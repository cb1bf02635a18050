// Host loops of the graph workloads (reference src/workloads/graphcompute.tr.cu:142-174, :257-285,
// :450-495, :635-675) and the graph file format (src/workloads/graphcompute.cu:16-45).
#include "workloads/graphcompute.h"

#include <algorithm>
#include <chrono>
#include <cstdio>
#include <cstring>
#include <thread>

#include "numeric.h"

namespace GraphCompute {

using namespace foo::util;

namespace {

template <class T>
bool read_array(const std::string &path, std::vector<T> &out) {
    FILE *fp = std::fopen(path.c_str(), "rb");
    if (!fp) return false;
    uint64_t count = 0, tag = 0;
    bool ok = std::fread(&count, sizeof(count), 1, fp) == 1 && std::fread(&tag, sizeof(tag), 1, fp) == 1 && count < (1ULL << 36);
    if (ok) {  // the header's count must fit what is left of the file, before anything is allocated for it
        const long here = std::ftell(fp);
        ok = here >= 0 && std::fseek(fp, 0, SEEK_END) == 0;
        const long end = ok ? std::ftell(fp) : -1;
        ok = ok && end >= here && (uint64_t)(end - here) / sizeof(T) >= count && std::fseek(fp, here, SEEK_SET) == 0;
    }
    if (ok) {
        out.resize(count);
        ok = std::fread(out.data(), sizeof(T), count, fp) == count;
    }
    std::fclose(fp);
    return ok;
}
template <class T>
bool write_array(const std::string &path, const std::vector<T> &v) {
    FILE *fp = std::fopen(path.c_str(), "wb");
    if (!fp) return false;
    uint64_t count = v.size(), tag = sizeof(T);
    bool ok = std::fwrite(&count, sizeof(count), 1, fp) == 1 && std::fwrite(&tag, sizeof(tag), 1, fp) == 1 &&
              std::fwrite(v.data(), sizeof(T), v.size(), fp) == v.size();
    return std::fclose(fp) == 0 && ok;
}

size_t round4(size_t n) { return (n + 3) / 4 * 4; }

}  // namespace

Status read_graph(const std::string &base, CsrGraph &g, bool with_weights) {
    if (!read_array(base + ".col", g.vertexList) || !read_array(base + ".dst", g.edgeList)) return Status::NotFound;
    if (g.vertexList.size() < 2) return Status::Fail;
    g.vertex_count = g.vertexList.size() - 1;
    g.edge_count = g.edgeList.size();
    // a malformed file must not turn into out-of-bounds reads on the GPU
    if (g.vertexList.front() != 0 || g.vertexList.back() != g.edge_count) return Status::Fail;
    for (size_t i = 0; i + 1 < g.vertexList.size(); ++i)
        if (g.vertexList[i] > g.vertexList[i + 1]) return Status::Fail;
    for (uint64_t e : g.edgeList)
        if (e >= g.vertex_count) return Status::OutOfRange;
    g.weightList.clear();
    if (with_weights) {
        if (!read_array(base + ".val", g.weightList)) return Status::NotFound;
        if (g.weightList.size() != g.edge_count) return Status::Fail;
    }
    return Status::Succ;
}

Status write_graph(const std::string &base, const CsrGraph &g) {
    if (!write_array(base + ".col", g.vertexList) || !write_array(base + ".dst", g.edgeList)) return Status::Fail;
    if (!g.weightList.empty() && !write_array(base + ".val", g.weightList)) return Status::Fail;
    return Status::Succ;
}

CsrGraph synthetic_graph(uint64_t n, unsigned degree, uint64_t seed) {
    foo::numeric::Rng rng(seed);
    std::vector<std::vector<std::pair<uint64_t, uint32_t>>> adj(n);
    for (uint64_t v = 0; v < n; ++v) {
        for (unsigned d = 0; d < degree; ++d) {
            // mostly short-range edges with a few long ones: several components are unlikely,
            // the diameter stays at tens of hops
            uint64_t u = (d % 4 == 0) ? rng.next() % n : (v + 1 + rng.next() % 64) % n;
            if (u == v) continue;
            uint32_t w = 1 + (uint32_t)(rng.next() % 64);
            adj[v].push_back({u, w});
            adj[u].push_back({v, w});
        }
    }
    CsrGraph g;
    g.vertex_count = n;
    g.vertexList.assign(n + 1, 0);
    for (uint64_t v = 0; v < n; ++v) g.vertexList[v + 1] = g.vertexList[v] + adj[v].size();
    g.edge_count = g.vertexList[n];
    g.edgeList.resize(g.edge_count);
    g.weightList.resize(g.edge_count);
    for (uint64_t v = 0; v < n; ++v) {
        std::sort(adj[v].begin(), adj[v].end());
        uint64_t o = g.vertexList[v];
        for (auto &e : adj[v]) { g.edgeList[o] = e.first; g.weightList[o] = e.second; ++o; }
    }
    return g;
}

// ---- the workload ---------------------------------------------------------------------------
#define GC_CHECK(call)                                                                          \
    do {                                                                                        \
        if ((call) != 0) {                                                                      \
            std::fprintf(stderr, "%s failed: %s (%s:%d)\n", #call, gp_last_error(), __FILE__, __LINE__); \
            return Status::Fail;                                                                \
        }                                                                                       \
    } while (0)

std::unique_ptr<Workload> Workload::create(const std::string &kind, const CsrGraph &g) {
    if (kind != "cc" && kind != "bfs" && kind != "pagerank" && kind != "sssp") return nullptr;
    if (g.vertex_count == 0 || g.vertex_count >= (1ULL << 32) || g.vertexList.size() != g.vertex_count + 1) return nullptr;
    if (kind == "sssp" && g.weightList.size() != g.edge_count) return nullptr;
    std::unique_ptr<Workload> w(new Workload());
    w->kind_ = kind;
    w->n_ = g.vertex_count;
    w->m_ = g.edge_count;
    // lanes per neighbour list: the width nearest the average degree keeps most lanes busy
    const double avg_degree = (double)g.edge_count / (double)g.vertex_count;
    w->lanes_ = avg_degree <= 24 ? 16 : avg_degree <= 48 ? 32 : 64;
    const size_t n = g.vertex_count;
    auto dev = [](GPUdeviceptr *p, size_t bytes) { return gp_malloc(p, bytes ? bytes : 4) == 0; };
    auto up = [&](GPUdeviceptr *p, const void *src, size_t bytes) { return dev(p, bytes) && (bytes == 0 || gp_memcpy_h2d(*p, src, bytes) == 0); };
    bool ok = up(&w->vertex_list_, g.vertexList.data(), (n + 1) * 8) && up(&w->edge_list_, g.edgeList.data(), g.edge_count * 8);
    ok = ok && dev(&w->changed_, 4) && gp_host_alloc((void **)&w->host_words_, 2 * sizeof(int)) == 0;
    if (kind == "bfs") ok = ok && dev(&w->label_, n * 4);
    if (kind == "cc") {
        ok = ok && dev(&w->comp_, n * 8) && dev(&w->active_, round4(n)) && dev(&w->next_active_, round4(n));
    }
    if (kind == "pagerank") ok = ok && dev(&w->active_, round4(n)) && dev(&w->delta_, n * 4) && dev(&w->residual_, n * 4) && dev(&w->value_, n * 4);
    if (kind == "sssp")
        ok = ok && up(&w->weight_list_, g.weightList.data(), g.edge_count * 4) && dev(&w->active_, round4(n)) && dev(&w->cost_, n * 4) && dev(&w->new_cost_, n * 4);
    if (!ok) {
        std::fprintf(stderr, "graph workload: allocation failed: %s\n", gp_last_error());
        return nullptr;
    }
    return w;
}

Workload::~Workload() {
    for (GPUdeviceptr p : {vertex_list_, edge_list_, weight_list_, label_, active_, next_active_, comp_, delta_, residual_, value_, cost_, new_cost_, changed_})
        if (p) gp_free(p);
    if (host_words_) gp_host_free(host_words_);
}

// initial state of a run (the memsets and single-element copies at the top of each reference loop)
Status Workload::begin(GPUstream stream) {
    const size_t n = n_;
    const uint32_t zero = 0;
    const unsigned char one = 1;
    if (kind_ == "bfs") {
        GC_CHECK(gp_fill32_async(label_, 0xFFFFFFFFu, n, stream));
        GC_CHECK(gp_stream_sync(stream));
        GC_CHECK(gp_memcpy_h2d(label_, &zero, 4));  // source = vertex 0 (graphcompute.tr.cu:255)
        level_ = 0;
    } else if (kind_ == "sssp") {
        GC_CHECK(gp_fill32_async(cost_, 0xFFFFFFFFu, n, stream));
        GC_CHECK(gp_fill32_async(new_cost_, 0xFFFFFFFFu, n, stream));
        GC_CHECK(gp_fill32_async(active_, 0, round4(n) / 4, stream));
        GC_CHECK(gp_stream_sync(stream));
        GC_CHECK(gp_memcpy_h2d(active_, &one, 1));
        GC_CHECK(gp_memcpy_h2d(cost_, &zero, 4));
        GC_CHECK(gp_memcpy_h2d(new_cost_, &zero, 4));
    }
    return Status::Succ;
}

// Launches `kernels` in order; when a stop was recorded, waits for the workload's turn and
// relaunches from the stopped kernel on, counters untouched, until the list has run to its end.
Status Workload::run_kernels(const std::vector<int> &kernels, GPUstream stream, const PreemptEnv *env, int iteration, bool *changed) {
    const int K = (int)kernels.size();
    const size_t per_kernel = env ? (size_t)env->counter_groups * env->counter_stride : 0;
    if (env) GC_CHECK(gp_fill32_async(env->executed, 0, per_kernel * K, stream));
    GC_CHECK(gp_fill32_async(changed_, 0, 1, stream));
    const bool inject = env && env->inject_iteration == iteration && env->inject_kernel >= 0 && env->inject_kernel < K;
    int from = 0;
    for (;;) {
        for (int k = from; k < K; ++k) {
            gp_graph_params p;
            std::memset(&p, 0, sizeof(p));
            p.kernel = kernels[k];
            p.level = level_;
            p.vertex_count = n_;
            p.vertex_list = (const unsigned long long *)vertex_list_;
            p.edge_list = (const unsigned long long *)edge_list_;
            p.weight_list = (const unsigned int *)weight_list_;
            p.label = (unsigned int *)label_;
            p.active = (unsigned char *)active_;
            p.next_active = (unsigned char *)next_active_;
            p.comp = (unsigned long long *)comp_;
            p.delta = (float *)delta_; p.residual = (float *)residual_; p.value = (float *)value_;
            p.alpha = 0.85f; p.tolerance = 0.001f;  // graphcompute.h:83-84
            p.cost = (unsigned int *)cost_; p.new_cost = (unsigned int *)new_cost_;
            p.changed = (unsigned int *)changed_;
            p.lanes_per_vertex = lanes_;
            if (env) {
                gp_preempt_ctx ctx;
                std::memset(&ctx, 0, sizeof(ctx));
                ctx.flag = (int *)env->flag; ctx.stop_index = (int *)env->stop_index;
                ctx.executed = (int *)env->executed + per_kernel * k;
                ctx.kernel_id = k;
                ctx.inject_at = (inject && !injected_ && k == env->inject_kernel) ? env->inject_claim : -1;
                if (ctx.inject_at >= 0) { injected_ = true; flag_to_lower_ = true; }
                ctx.poll_every = env->poll_every;
                ctx.counter_groups = env->counter_groups;
                GC_CHECK(gp_launch_graph(&p, &ctx, stream, nullptr));
            } else {
                GC_CHECK(gp_launch_graph(&p, nullptr, stream, nullptr));
            }
            ++launches_;
        }
        host_words_[0] = -1;
        if (env) GC_CHECK(gp_memcpy_d2h_async(&host_words_[0], env->stop_index, sizeof(int), stream));
        GC_CHECK(gp_memcpy_d2h_async(&host_words_[1], changed_, sizeof(int), stream));
        // polled, not a blocking wait: a blocked thread wakes up tens of microseconds late, which
        // is paid once per iteration and on every preemption
        for (;;) {
            int idle = 0;
            GC_CHECK(gp_stream_query(stream, &idle));
            if (idle) break;
        }
        const int stop = host_words_[0];
        if (!env || stop < 0) break;
        // stopped in kernel `stop`: stay off the GPU while a higher priority needs it
        ++preemptions_;
        if (flag_to_lower_) {  // nobody else will lower a flag the kernel raised itself
            GC_CHECK(gp_fill32_async(env->flag, 0, 1, stream));  // a device store, as the raise was
            GC_CHECK(gp_stream_sync(stream));
            flag_to_lower_ = false;
        }
        if (env->higher_priority_active) {
            while (env->higher_priority_active()) std::this_thread::yield();
        } else {
            // nobody to ask: give whoever raised the flag time to lower it instead of relaunching
            // kernels that would leave at once
            std::this_thread::sleep_for(std::chrono::microseconds(50));
        }
        GC_CHECK(gp_fill32_async(env->stop_index, 0xFFFFFFFFu, 1, stream));
        from = stop < K ? stop : K - 1;
    }
    *changed = host_words_[1] != 0;
    return Status::Succ;
}

Status Workload::compute(GPUstream stream, const PreemptEnv *env) {
    iterations_ = 0;
    injected_ = false;
    RETURN_STATUS(begin(stream));
    bool changed = false;
    std::vector<int> loop;
    int max_iter = 1 << 30;
    if (kind_ == "bfs") loop = {GP_GRAPH_BFS_STEP};
    else if (kind_ == "cc") {
        loop = {GP_GRAPH_CC_STEP};
        // labels and frontier are set up by a kernel (the reference uploads 8 bytes per vertex
        // from the host on every run, graphcompute.tr.cu:143-146)
        RETURN_STATUS(run_kernels({GP_GRAPH_CC_INIT}, stream, env, -1, &changed));
    }
    else if (kind_ == "sssp") loop = {GP_GRAPH_SSSP_RELAX, GP_GRAPH_SSSP_UPDATE};
    else {
        loop = {GP_GRAPH_PR_PUSH, GP_GRAPH_PR_UPDATE};
        max_iter = 100;  // graphcompute.h:82
        RETURN_STATUS(run_kernels({GP_GRAPH_PR_INIT}, stream, env, -1, &changed));
    }
    do {
        RETURN_STATUS(run_kernels(loop, stream, env, iterations_, &changed));
        if (kind_ == "bfs") ++level_;
        if (kind_ == "cc") {  // the frontier just used is cleared and becomes the next one's buffer
            GC_CHECK(gp_fill32_async(active_, 0, round4(n_) / 4, stream));
            std::swap(active_, next_active_);
        }
        ++iterations_;
    } while (changed && iterations_ < max_iter);
    if (flag_to_lower_ && env) {  // raised by the very last claims: no later claim saw it
        GC_CHECK(gp_fill32_async(env->flag, 0, 1, stream));
        GC_CHECK(gp_stream_sync(stream));
        flag_to_lower_ = false;
    }
    return Status::Succ;
}

size_t Workload::result_bytes(const std::string &key) const {
    if (key == "comp" && comp_) return n_ * 8;
    if (key == "label" && label_) return n_ * 4;
    if (key == "value" && value_) return n_ * 4;
    if (key == "cost" && cost_) return n_ * 4;
    return 0;
}

Status Workload::read_result(const std::string &key, void *out, size_t len) const {
    const size_t bytes = result_bytes(key);
    if (bytes == 0) return Status::NotFound;
    if (len < bytes) return Status::OutOfRange;
    GPUdeviceptr src = key == "comp" ? comp_ : key == "label" ? label_ : key == "value" ? value_ : cost_;
    GC_CHECK(gp_stream_sync(nullptr));
    GC_CHECK(gp_memcpy_d2h(out, src, bytes));
    return Status::Succ;
}

}  // namespace GraphCompute
