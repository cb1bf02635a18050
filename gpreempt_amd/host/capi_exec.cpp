// extern "C" forwarding layer over foo::Executor / foo::BLPExecutor (include/gpreempt_exec_c.h).
#include <atomic>
#include <cstring>
#include "executor.h"
#include "gpreempt_exec_c.h"
#include "workloads/scicomput.h"
#include "harness.h"
#include "gpreempt.h"
#include "mini_json.h"
#include "tvm_export.h"
#include <exception>
#include <fstream>
#include <iterator>
#include <map>
#include <mutex>

using namespace foo;

namespace {
struct Handle {
    std::unique_ptr<Executor> ex;
    BLPExecutor *blp = nullptr;
    std::atomic<int> lc_tasks{0}, be_tasks{1};  // handed to BLPExecutor::set_lc_be_tasks
};
Handle *H(gpx_executor e) { return static_cast<Handle *>(e); }
void copy_str(char *dst, size_t n, const std::string &s) {
    if (!dst || !n) return;
    std::strncpy(dst, s.c_str(), n - 1);
    dst[n - 1] = 0;
}
// No exception may cross the C boundary (a corrupt file can make a std::vector throw
// bad_alloc or length_error): it becomes Status::Fail with a line on stderr.
template <class F>
int guarded(const char *what, F &&f) {
    try {
        return (int)f();
    } catch (const std::exception &e) {
        std::fprintf(stderr, "%s: %s\n", what, e.what());
    } catch (...) {
        std::fprintf(stderr, "%s: unknown exception\n", what);
    }
    return Status::Fail;
}
std::mutex g_dom_mu;
std::map<int, std::unique_ptr<PreemptDomain>> g_domains;  // gpx_domain_create's domains by handle
}  // namespace

extern "C" {

gpx_executor gpx_create(int blp) {
    Handle *h = new Handle();
    if (blp) { h->blp = new BLPExecutor(); h->ex.reset(h->blp); h->blp->set_lc_be_tasks(h->lc_tasks, h->be_tasks); }
    else h->ex.reset(new BaseExecutor());
    return h;
}
void gpx_destroy(gpx_executor e) { delete H(e); }
int gpx_init(gpx_executor e, const char *workload) { return guarded("gpx_init", [&] { return H(e)->ex->init(workload ? workload : ""); }); }
int gpx_set_input(gpx_executor e, const char *key, void *value, size_t len, gp_stream s) { return H(e)->ex->set_input(key, value, len, s); }
int gpx_get_output(gpx_executor e, const char *key, void *value, size_t len, gp_stream s) { return H(e)->ex->get_output(key, value, len, s); }
size_t gpx_get_data_size(gpx_executor e, const char *key) { return H(e)->ex->get_data_size(key); }
int gpx_execute(gpx_executor e, gp_stream s) { return guarded("gpx_execute", [&] { return H(e)->ex->execute(s); }); }
int gpx_launch_kernel(gpx_executor e, size_t idx, gp_stream s) { return H(e)->ex->launch_kernel(idx, s); }
size_t gpx_get_kernel_num(gpx_executor e) { return H(e)->ex->get_kernel_num(); }
int gpx_capture_graph(gpx_executor e, gp_stream s) {
    H(e)->ex->capture_graph(s);
    return H(e)->ex->uses_graph() ? Status::Succ : Status::Fail;  // capture_graph itself returns void
}
int gpx_uses_program(gpx_executor e) { return H(e)->ex->uses_program() ? 1 : 0; }
void gpx_clear(gpx_executor e) { H(e)->ex->clear(); }

int gpx_set_flag(gpx_executor e, void *dp) { if (!H(e)->blp) return Status::Fail; H(e)->blp->dpStop = dp; return Status::Succ; }
int gpx_set_running(gpx_executor e, int r) { if (!H(e)->blp) return Status::Fail; H(e)->blp->running = r != 0; return Status::Succ; }
int gpx_resume(gpx_executor e, gp_stream s) { return H(e)->blp ? H(e)->blp->resume(s) : Status::Fail; }
int gpx_get_stop_point(gpx_executor e, gp_stream s, int *stop) {
    if (!H(e)->blp) return Status::Fail;
    Status st = H(e)->blp->getStopPoint(s);
    if (stop) *stop = H(e)->blp->last_stop_index();
    return st;
}
int gpx_last_stop_index(gpx_executor e) { return H(e)->blp ? H(e)->blp->last_stop_index() : -1; }
int gpx_inject_preempt(gpx_executor e, int kernel, int claim) { if (!H(e)->blp) return Status::Fail; H(e)->blp->inject_preempt(kernel, claim); return Status::Succ; }
int gpx_reset_counters(gpx_executor e, gp_stream s) { return H(e)->blp ? H(e)->blp->reset_counters(s) : Status::Fail; }
int gpx_read_counters(gpx_executor e, int *out, size_t n) {
    if (!H(e)->blp) return Status::Fail;
    std::vector<int> v;
    Status st = H(e)->blp->read_counters(v);
    if (st != Status::Succ) return st;
    std::memcpy(out, v.data(), sizeof(int) * std::min(n, v.size()));
    return Status::Succ;
}

size_t gpx_storage_num(gpx_executor e) { auto m = H(e)->ex->get_model(); return m ? m->get_storage_num() : 0; }

int gpx_kernel_info(gpx_executor e, size_t idx, char *name, size_t name_len, double *flops, double *bytes, int *total_blocks, int *grid) {
    auto m = H(e)->ex->get_model();
    if (!m || idx >= m->get_kernel_num()) return Status::OutOfRange;
    KernelInfo &k = m->get_kernel_info(idx);
    copy_str(name, name_len, k.name);
    if (flops) *flops = k.flops;
    if (bytes) *bytes = k.bytes;
    if (total_blocks) *total_blocks = k.total_blocks;
    if (grid) *grid = (int)k.launch_params[0];
    return Status::Succ;
}

int gpx_read_storage(gpx_executor e, const char *key, void *out, size_t len) {
    auto m = H(e)->ex->get_model();
    if (!m) return Status::Fail;
    Status st = m->get(key, out, len, nullptr);
    if (st != Status::Succ) return st;
    return gp_stream_sync(nullptr) == 0 ? Status::Succ : Status::Fail;
}

}  // extern "C"

extern "C" int gpx_graph_info(gpx_executor e, unsigned long long info[5]) {
    GraphCompute::Workload *w = H(e)->ex->graph_workload();
    if (!w) return Status::NotFound;
    info[0] = w->vertex_count(); info[1] = w->edge_count(); info[2] = (unsigned long long)w->iterations();
    info[3] = (unsigned long long)w->preemptions(); info[4] = (unsigned long long)w->kernels_launched();
    return Status::Succ;
}
extern "C" size_t gpx_graph_result_bytes(gpx_executor e, const char *key) {
    GraphCompute::Workload *w = H(e)->ex->graph_workload();
    return w ? w->result_bytes(key) : 0;
}
extern "C" int gpx_graph_result(gpx_executor e, const char *key, void *out, size_t len) {
    GraphCompute::Workload *w = H(e)->ex->graph_workload();
    return w ? w->read_result(key, out, len) : Status::NotFound;
}
extern "C" int gpx_graph_inject_preempt(gpx_executor e, int iteration, int kernel, int claim) {
    if (!H(e)->blp) return Status::Fail;
    H(e)->blp->inject_preempt_graph(iteration, kernel, claim);
    return Status::Succ;
}
extern "C" int gpx_set_lc_tasks(gpx_executor e, int n) { H(e)->lc_tasks.store(n); return Status::Succ; }
extern "C" int gpx_set_graph_path(gpx_executor e, const char *base) { return H(e)->ex->set_graph_path(base ? base : ""); }
extern "C" int gpx_write_synthetic_graph(const char *base, unsigned long long vertices, unsigned degree, unsigned long long seed) {
    if (!base || vertices < 2 || vertices >= (1ULL << 28) || degree < 1 || degree > 256 || vertices * degree > (1ULL << 27)) return Status::OutOfRange;
    return guarded("gpx_write_synthetic_graph", [&] { return GraphCompute::write_graph(base, GraphCompute::synthetic_graph(vertices, degree, seed)); });
}

extern "C" int gpx_miniweather_reductions(gpx_executor e, double *mass, double *te) {
    auto m = H(e)->ex->get_model();
    if (!m || m->get_kernel_num() == 0 || m->get_kernel_info(0).op != OpKind::Stencil) return Status::NotFound;
    const gp_miniweather_params &p = m->get_kernel_info(0).p.miniweather;
    const SciCompute::Grid g = SciCompute::make_grid(p.nx, p.nz);
    std::vector<float> state(SciCompute::state_elems(g)), hydro(SciCompute::hydro_elems(g));
    Status st = m->get("state", state.data(), state.size() * sizeof(float), nullptr);
    if (st == Status::Succ) st = m->get("hydro", hydro.data(), hydro.size() * sizeof(float), nullptr);
    if (st != Status::Succ) return st;
    if (gp_stream_sync(nullptr) != 0) return Status::Fail;
    SciCompute::reductions(g, state.data(), hydro.data(), *mass, *te);
    return Status::Succ;
}

extern "C" int gpx_storage_info(gpx_executor e, size_t idx, char *name, size_t name_len, char *stype, size_t stype_len,
                                size_t *bytes, int *is_param, size_t *disk_elems, int dims[8]) {
    auto m = H(e)->ex->get_model();
    if (!m || idx >= m->get_storage_num()) return Status::OutOfRange;
    StorageInfo &s = m->get_storage_info(idx);
    const ParamLayout &L = m->get_param_layout(idx);
    copy_str(name, name_len, s.name);
    copy_str(stype, stype_len, s.stype);
    if (bytes) *bytes = s.size;
    if (is_param) *is_param = L.is_param;
    if (disk_elems) *disk_elems = L.disk_elems;
    if (dims) { int d[8] = {(int)L.kind, L.o, L.i, L.r, L.s, L.c, L.h, L.w}; std::memcpy(dims, d, sizeof(d)); }
    return Status::Succ;
}

static int copy_report(Status st, const std::string &rep, char *report, size_t report_len) {
    if (report && report_len) {
        std::strncpy(report, rep.c_str(), report_len - 1);
        report[report_len - 1] = 0;
    }
    if (st == Status::Succ && rep.size() + 1 > report_len) return Status::Full;
    return st;
}

extern "C" int gpx_run_scenario(const char *config_json, char *report, size_t report_len) {
    return guarded("gpx_run_scenario", [&] {
        std::string rep;
        Status st = foo::run_scenario(config_json ? config_json : "", rep);
        return copy_report(st, rep, report, report_len);
    });
}

extern "C" int gpx_preempt_probe(const char *workload, int trials, int use_graph, unsigned long long seed, char *report, size_t report_len) {
    return guarded("gpx_preempt_probe", [&] {
        std::string rep;
        Status st = foo::preempt_probe(workload ? workload : "", trials, use_graph, seed, rep);
        return copy_report(st, rep, report, report_len);
    });
}

extern "C" long gpx_parse_params(const char *path, const char *key, float *out, size_t n, size_t *len) {
    std::unique_ptr<ModelParam> params;
    try {
        params.reset(ModelParamParser::parse_from_file(path));
    } catch (const std::exception &e) {
        std::fprintf(stderr, "gpx_parse_params: %s\n", e.what());
    }
    if (!params) return -1;
    if (key) {
        auto it = params->find(key);
        if (len) *len = it == params->end() ? 0 : it->second.size();
        if (it != params->end() && out) std::memcpy(out, it->second.data(), sizeof(float) * std::min(n, it->second.size()));
    }
    return (long)params->size();
}

// ---- gpreempt.h through the C view ------------------------------------------------------------------
extern "C" int gpx_set_priority(gp_stream s, int priority) {
    NvContext ctx;
    ctx.stream = s;
    if (NvRmQuery(&ctx) != 0) return -1;
    return set_priority(ctx, priority);
}
extern "C" int gpx_domain_create(int levels) {
    return guarded("gpx_domain_create", [&] {
        std::unique_ptr<PreemptDomain> d(new PreemptDomain(levels));
        if (!d->ok()) return -1;
        const int fd = d->fd();
        std::lock_guard<std::mutex> g(g_dom_mu);
        g_domains[fd] = std::move(d);
        return fd;
    });
}
extern "C" int gpx_domain_destroy(int fd) {
    std::lock_guard<std::mutex> g(g_dom_mu);
    return g_domains.erase(fd) ? 0 : -1;
}
extern "C" int gpx_get_fd(void) { return hipGetFd(); }
extern "C" void *gpx_domain_flag(int fd, int priority) {
    std::lock_guard<std::mutex> g(g_dom_mu);
    auto it = g_domains.find(fd);
    return it == g_domains.end() ? nullptr : it->second->flag_for(priority);
}
extern "C" int gpx_domain_flag_value(int fd, int priority) {
    std::lock_guard<std::mutex> g(g_dom_mu);
    auto it = g_domains.find(fd);
    return it == g_domains.end() ? -1 : it->second->flag_value(priority);
}
extern "C" int gpx_domain_begin(int fd, int priority) {
    std::lock_guard<std::mutex> g(g_dom_mu);
    auto it = g_domains.find(fd);
    if (it == g_domains.end()) return -1;
    it->second->begin(priority);
    return 0;
}
extern "C" int gpx_domain_end(int fd, int priority) {
    std::lock_guard<std::mutex> g(g_dom_mu);
    auto it = g_domains.find(fd);
    if (it == g_domains.end()) return -1;
    it->second->end(priority);
    return 0;
}
extern "C" int gpx_suspend_streams(int fd, const int *levels, int n) {
    std::vector<int> v(levels, levels + (n > 0 ? n : 0));
    return hipSuspendStreams(fd, v);
}
extern "C" int gpx_resume_streams(int fd, const int *levels, int n) {
    std::vector<int> v(levels, levels + (n > 0 ? n : 0));
    return hipResumeStreams(fd, v);
}

// ---- exported-model reader ---------------------------------------------------------------------------
extern "C" int gpx_parse_tvm_export(const char *device_json, const char *host_json, const char *ops_json, char *report, size_t report_len) {
    return guarded("gpx_parse_tvm_export", [&] {
        TvmExport ex;
        Status st = load_tvm_export(device_json ? device_json : "", host_json ? host_json : "", ex);
        json::Value rep = json::Value::object();
        if (st == Status::Succ && ops_json && *ops_json) {
            std::ifstream f(ops_json, std::ios::binary);
            if (!f.is_open()) { st = Status::NotFound; ex.error = std::string("Cannot open the json file: ") + ops_json; }
            else {
                std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
                ExportOps ops;
                st = parse_export_ops(text, ops);
                if (st != Status::Succ) ex.error = ops.error;
                else st = check_export_ops(ex, ops, ex.error);
                json::Value &jo = rep.set("ops");
                jo = json::Value::array();
                for (const ExportOp &o : ops.funcs) {
                    json::Value e = json::Value::object();
                    e.set("name") = o.func; e.set("op") = o.op;
                    json::Value &a = e.set("attrs");
                    a = json::Value::object();
                    for (const auto &kv : o.attrs) { json::Value &l = a.set(kv.first); l = json::Value::array(); for (long v : kv.second) l.push(json::Value(v)); }
                    json::Value &ep = e.set("epilogue");
                    ep = json::Value::array();
                    for (const std::string &t : o.epilogue) ep.push(json::Value(t));
                    json::Value &in = e.set("inputs");
                    in = json::Value::object();
                    for (const auto &kv : o.inputs) in.set(kv.first) = kv.second;
                    jo.push(e);
                }
                rep.set("layout") = ops.layout;
            }
        }
        rep.set("error") = ex.error;
        rep.set("global_len") = ex.global_len;
        rep.set("heads_index") = ex.heads_index;
        json::Value &js = rep.set("storages");
        js = json::Value::array();
        for (const StorageInfo &s : ex.storage_infos) {
            json::Value e = json::Value::object();
            e.set("name") = s.name; e.set("stype") = s.stype; e.set("size") = s.size;
            js.push(e);
        }
        json::Value &jk = rep.set("kernels");
        jk = json::Value::array();
        for (size_t i = 0; i < ex.kernel_infos.size(); ++i) {
            const KernelInfo &k = ex.kernel_infos[i];
            json::Value e = json::Value::object();
            e.set("name") = k.name; e.set("func") = ex.kernel_func[i];
            json::Value &lp = e.set("launch_params");
            lp = json::Value::array();
            for (int j = 0; j < 6; ++j) lp.push(json::Value((long)k.launch_params[j]));
            json::Value &ai = e.set("args_index");
            ai = json::Value::array();
            for (size_t a : k.args_index) ai.push(json::Value(a));
            jk.push(e);
        }
        return copy_report(st, rep.dump(), report, report_len);
    });
}

// The native kernel list an exported model maps to, without touching a GPU.
extern "C" int gpx_plan_tvm_export(const char *device_json, const char *host_json, const char *ops_json, const char *dtype, char *report, size_t report_len) {
    return guarded("gpx_plan_tvm_export", [&] {
        Model m;
        json::Value rep = json::Value::object();
        Status st = m.load_from_json(device_json ? device_json : "", host_json ? host_json : "");
        std::string err = m.tvm_export() ? m.tvm_export()->error : "";
        if (st == Status::Succ) {
            std::ifstream f(ops_json ? ops_json : "", std::ios::binary);
            if (!f.is_open()) { st = Status::NotFound; err = std::string("Cannot open the json file: ") + (ops_json ? ops_json : ""); }
            else {
                std::string text((std::istreambuf_iterator<char>(f)), std::istreambuf_iterator<char>());
                st = m.build_from_export(dtype && *dtype ? std::string("export@dtype=") + dtype : std::string("export"), text);
                if (st != Status::Succ) err = m.tvm_export()->error;
            }
        }
        rep.set("error") = err;
        rep.set("dtype") = m.dtype();
        json::Value &js = rep.set("storages");
        js = json::Value::array();
        for (size_t i = 0; st == Status::Succ && i < m.get_storage_num(); ++i) {
            const StorageInfo &s = m.get_storage_info(i);
            const ParamLayout &L = m.get_param_layout(i);
            json::Value e = json::Value::object();
            e.set("name") = s.name; e.set("stype") = s.stype; e.set("size") = s.size;
            e.set("is_param") = L.is_param ? 1 : 0; e.set("kind") = (int)L.kind; e.set("disk_elems") = L.disk_elems;
            js.push(e);
        }
        json::Value &jk = rep.set("kernels");
        jk = json::Value::array();
        for (size_t i = 0; st == Status::Succ && i < m.get_kernel_num(); ++i) {
            const KernelInfo &k = m.get_kernel_info(i);
            json::Value e = json::Value::object();
            e.set("name") = k.name;
            json::Value &ar = e.set("args");
            ar = json::Value::array();
            for (const ArgRef &r : k.refs) ar.push(r.storage == SIZE_MAX ? json::Value("") : json::Value(m.get_storage_info(r.storage).name));
            json::Value &p = e.set("params");
            p = json::Value::object();
            switch (k.op) {
                case OpKind::Conv: {
                    const gp_conv_params &c = k.p.conv;
                    p.set("N") = c.N; p.set("H") = c.H; p.set("W") = c.W; p.set("Cin") = c.Cin; p.set("Cout") = c.Cout; p.set("R") = c.R; p.set("S") = c.S;
                    p.set("stride_h") = c.stride_h; p.set("stride_w") = c.stride_w; p.set("pad_h") = c.pad_h; p.set("pad_w") = c.pad_w; p.set("act") = c.act;
                    p.set("in_pix_stride") = c.in_pix_stride; p.set("out_pix_stride") = c.out_pix_stride;
                    break;
                }
                case OpKind::Gemm: {
                    const gp_gemm_params &g = k.p.gemm;
                    p.set("M") = g.M; p.set("N") = g.N; p.set("K") = g.K; p.set("lda") = g.lda; p.set("ldc") = g.ldc; p.set("act") = g.act;
                    if (g.batch > 1) {  // a batched product: how the heads are laid out
                        p.set("batch") = g.batch; p.set("batch_inner") = g.batch_inner; p.set("ldb") = g.ldb; p.set("b_is_nk") = g.b_is_nk; p.set("alpha") = (double)g.alpha;
                        p.set("stride_a") = g.stride_a; p.set("stride_b") = g.stride_b; p.set("stride_c") = g.stride_c;
                        p.set("stride_a_outer") = g.stride_a_outer; p.set("stride_b_outer") = g.stride_b_outer; p.set("stride_c_outer") = g.stride_c_outer;
                    }
                    break;
                }
                case OpKind::Pool: {
                    const gp_pool_params &q = k.p.pool;
                    p.set("N") = q.N; p.set("H") = q.H; p.set("W") = q.W; p.set("C") = q.C; p.set("R") = q.R; p.set("stride") = q.stride; p.set("pad") = q.pad; p.set("mode") = q.mode;
                    break;
                }
                case OpKind::Eltwise: {
                    const gp_eltwise_params &q = k.p.eltwise;
                    p.set("rows") = q.rows; p.set("cols") = q.cols; p.set("a_stride") = q.a_stride; p.set("out_stride") = q.out_stride; p.set("act") = q.act;
                    break;
                }
                case OpKind::Softmax: p.set("rows") = k.p.softmax.rows; p.set("cols") = k.p.softmax.cols; break;
                case OpKind::Layernorm: p.set("rows") = k.p.layernorm.rows; p.set("cols") = k.p.layernorm.cols; p.set("eps") = (double)k.p.layernorm.eps; break;
                case OpKind::Embed: p.set("tokens") = k.p.embed.tokens; p.set("seq") = k.p.embed.seq; p.set("hidden") = k.p.embed.hidden; p.set("vocab") = k.p.embed.vocab; break;
                case OpKind::Layout: p.set("N") = k.p.layout.N; p.set("C") = k.p.layout.C; p.set("H") = k.p.layout.H; p.set("W") = k.p.layout.W; p.set("c_pad") = k.p.layout.c_pad; break;
                default: break;
            }
            jk.push(e);
        }
        return copy_report(st, rep.dump(), report, report_len);
    });
}

