// Reader of mod.json / host.json (and the ops.json sidecar); see include/tvm_export.h.
#include "tvm_export.h"

#include <fstream>
#include <iterator>
#include <set>

#include "mini_json.h"

namespace foo {

namespace {

bool read_file(const char *path, std::string &out) {
    std::ifstream f(path, std::ios::binary);
    if (!f.is_open()) return false;
    out.assign(std::istreambuf_iterator<char>(f), std::istreambuf_iterator<char>());
    return true;
}

Status fail(std::string &err, const std::string &what) {
    err = what;
    return Status::Fail;
}

// a non-negative integer a double holds exactly (below 2^53: beyond that the cast back is not defined for every value)
bool is_uint(const json::Value &v) { return v.type == json::Value::Number && v.num >= 0 && v.num < 9007199254740992.0 && v.num == (double)(uint64_t)v.num; }

}  // namespace

Status parse_tvm_export(const std::string &device_json_text, const std::string &host_json_text, TvmExport &out) {
    out = TvmExport();
    json::Value d, h;
    if (!json::parse(device_json_text, d) || d.type != json::Value::Object) return fail(out.error, "device json: malformed");
    if (!json::parse(host_json_text, h) || h.type != json::Value::Object) return fail(out.error, "host json: malformed");

    // attrs.dltype = ["list_str", [...]], attrs.shape = ["list_shape", [[...], ...]]: one entry per
    // node (src/model.cpp:157-160 indexes both by node id)
    const json::Value &dltypes = d["attrs"]["dltype"].arr.size() > 1 ? d["attrs"]["dltype"].arr[1] : json::Value();
    const json::Value &shapes = d["attrs"]["shape"].arr.size() > 1 ? d["attrs"]["shape"].arr[1] : json::Value();
    const json::Value &nodes = d["nodes"];
    const size_t global_len = dltypes.arr.size();
    if (dltypes.type != json::Value::Array || shapes.type != json::Value::Array || nodes.type != json::Value::Array)
        return fail(out.error, "device json: attrs.dltype, attrs.shape and nodes must be arrays");
    if (shapes.arr.size() != global_len || nodes.arr.size() < global_len)
        return fail(out.error, "device json: dltype, shape and nodes disagree in length");
    out.global_len = global_len;

    // global storages: one per graph node (src/model.cpp:162-173)
    for (size_t i = 0; i < global_len; ++i) {
        StorageInfo s;
        s.name = nodes.arr[i]["name"].string();
        s.stype = dltypes.arr[i].string();
        size_t elems = 1;
        for (const json::Value &dim : shapes.arr[i].arr) {
            // every dimension below 2^31 and every tensor below 2^40 elements: the product cannot wrap
            if (!is_uint(dim) || dim.num >= 2147483648.0) return fail(out.error, "device json: bad shape of node " + std::to_string(i));
            elems *= (size_t)dim.num;
            if (elems >= ((size_t)1 << 40)) return fail(out.error, "device json: node " + std::to_string(i) + " holds more than 2^40 elements");
        }
        const size_t es = Model::get_stype_size(s.stype);
        if (es == 0) return fail(out.error, "device json: unknown dltype '" + s.stype + "' of node " + std::to_string(i));
        s.size = elems * es;
        out.storage_infos.push_back(s);
        ExportNode n;
        n.name = s.name; n.stype = s.stype;
        for (const json::Value &dim : shapes.arr[i].arr) n.shape.push_back((long)dim.num);
        out.nodes.push_back(n);
    }
    // temporary storages, typed float32 whatever they hold (src/model.cpp:176-183)
    for (const json::Value &t : h["temp_args"].arr) {
        if (!is_uint(t) || t.num >= 1099511627776.0) return fail(out.error, "host json: bad temp_args entry");
        StorageInfo s;
        s.name = "temp"; s.stype = "float32"; s.size = (size_t)t.num;
        out.storage_infos.push_back(s);
    }
    const size_t temp_len = out.storage_infos.size() - global_len;

    // host functions in graph order: the nodes that have inputs; arguments = inputs..., the node itself
    // (src/model.cpp:186-197; only element [0] of an input entry is read)
    std::vector<std::pair<std::string, std::vector<size_t>>> func_args;
    for (size_t i = 0; i < global_len; ++i) {
        const json::Value &node = nodes.arr[i];
        if (node["inputs"].arr.empty()) continue;
        std::vector<size_t> args;
        for (const json::Value &in : node["inputs"].arr) {
            if (in.arr.empty() || !is_uint(in.arr[0]) || (size_t)in.arr[0].num >= global_len)
                return fail(out.error, "device json: bad input of node " + std::to_string(i));
            args.push_back((size_t)in.arr[0].num);
        }
        out.nodes[i].inputs = args;
        out.nodes[i].func = node["attrs"]["func_name"].string();
        args.push_back(i);
        func_args.emplace_back(out.nodes[i].func, args);
    }

    auto push_nop = [&](const std::vector<size_t> &args) {
        KernelInfo k;
        k.name = "nop";
        k.args_index = args;  // copy args_index[0] -> args_index[1] (src/executor.cpp:139-146)
        std::fill(k.launch_params, k.launch_params + 6, 0u);
        out.kernel_infos.push_back(k);
        out.kernel_func.push_back("__nop");
    };
    // kernels: host.json's functions matched against the graph's in order, "__nop" nodes (reshape,
    // flatten) becoming copies (src/model.cpp:199-229)
    size_t fi = 0;
    for (const json::Value &func : h["funcs"].arr) {
        while (fi < func_args.size() && func_args[fi].first == "__nop") push_nop(func_args[fi++].second);
        if (fi >= func_args.size()) return fail(out.error, "host json has more functions than the graph has operator nodes");
        const std::string fname = func["name"].string();
        if (fname != func_args[fi].first) return fail(out.error, "Function name mismatch: " + fname + " vs " + func_args[fi].first);
        const std::vector<size_t> &args = func_args[fi++].second;
        for (const json::Value &kernel : func["kernels"].arr) {
            KernelInfo k;
            k.name = kernel["name"].string();
            for (const json::Value &a : kernel["args"].arr) {
                if (a.type != json::Value::Number || a.num != (double)(long)a.num) return fail(out.error, "host json: bad argument index in " + k.name);
                const long idx = (long)a.num;
                if (idx >= 0) {  // the idx-th argument of the host function
                    if ((size_t)idx >= args.size()) return fail(out.error, "host json: argument " + std::to_string(idx) + " of " + k.name + " is past the function's arguments");
                    k.args_index.push_back(args[idx]);
                } else {         // -1 is the first temporary buffer, -2 the second, ... (src/model.cpp:217-221)
                    const size_t t = (size_t)(-idx - 1);
                    if (t >= temp_len) return fail(out.error, "host json: temporary " + std::to_string(idx) + " of " + k.name + " does not exist");
                    k.args_index.push_back(global_len + t);
                }
            }
            const json::Value &lp = kernel["launch_params"];
            if (lp.arr.size() != 6) return fail(out.error, "host json: launch_params of " + k.name + " must have 6 entries");
            for (int j = 0; j < 6; ++j) {
                if (!is_uint(lp.arr[j])) return fail(out.error, "host json: bad launch_params of " + k.name);
                k.launch_params[j] = (uint32_t)lp.arr[j].num;
            }
            out.kernel_infos.push_back(k);
            out.kernel_func.push_back(fname);
        }
    }
    // copies behind the last function (the reference's loop never reaches them; a graph that ends in a
    // reshape would leave "heads" unwritten there)
    while (fi < func_args.size() && func_args[fi].first == "__nop") push_nop(func_args[fi++].second);
    if (fi != func_args.size()) return fail(out.error, "the graph has operator nodes that host json does not list (first: " + func_args[fi].first + ")");

    // the output node is renamed (src/model.cpp:231)
    const json::Value &heads = d["heads"];
    if (heads.arr.empty() || heads.arr[0].arr.empty() || !is_uint(heads.arr[0].arr[0]) || (size_t)heads.arr[0].arr[0].num >= global_len)
        return fail(out.error, "device json: bad heads");
    out.heads_index = (size_t)heads.arr[0].arr[0].num;
    out.storage_infos[out.heads_index].name = "heads";
    return Status::Succ;
}

Status load_tvm_export(const char *device_json_path, const char *host_json_path, TvmExport &out) {
    std::string d, h;
    out = TvmExport();
    if (!read_file(device_json_path, d)) { out.error = std::string("Cannot open the json file: ") + device_json_path; return Status::NotFound; }
    if (!read_file(host_json_path, h)) { out.error = std::string("Cannot open the json file: ") + host_json_path; return Status::NotFound; }
    return parse_tvm_export(d, h, out);
}

Status parse_export_ops(const std::string &text, ExportOps &out) {
    out = ExportOps();
    json::Value v;
    if (!json::parse(text, v) || v.type != json::Value::Object) return fail(out.error, "ops json: malformed");
    out.layout = v["layout"].string("NCHW");
    if (out.layout != "NCHW" && out.layout != "NHWC") return fail(out.error, "ops json: layout must be NCHW or NHWC");
    static const std::set<std::string> known = {"conv2d", "dense", "max_pool2d", "avg_pool2d", "global_avg_pool2d", "add", "softmax", "layer_norm",
                                                "batch_matmul", "take", "scale_shift", "concatenate", "reshape", "transpose", "gelu"};
    static const std::set<std::string> tails = {"bias", "residual", "relu", "gelu"};
    for (const json::Value &f : v["funcs"].arr) {
        ExportOp op;
        op.func = f["name"].string();
        op.op = f["op"].string();
        if (op.func.empty()) return fail(out.error, "ops json: a function without a name");
        if (!known.count(op.op)) return fail(out.error, "ops json: unknown op '" + op.op + "' for " + op.func);
        for (const auto &kv : f["attrs"].obj) {
            std::vector<long> vals;
            if (kv.second.type == json::Value::Number) vals.push_back((long)kv.second.num);
            else if (kv.second.type == json::Value::Array) for (const json::Value &e : kv.second.arr) {
                if (e.type != json::Value::Number) return fail(out.error, "ops json: attribute " + kv.first + " of " + op.func + " must hold integers");
                vals.push_back((long)e.num);
            } else return fail(out.error, "ops json: attribute " + kv.first + " of " + op.func + " must be an integer or a list");
            op.attrs[kv.first] = vals;
        }
        for (const json::Value &e : f["epilogue"].arr) {
            if (!tails.count(e.string())) return fail(out.error, "ops json: unknown epilogue step '" + e.string() + "' for " + op.func);
            op.epilogue.push_back(e.string());
        }
        for (const auto &kv : f["inputs"].obj) {
            if (!is_uint(kv.second)) return fail(out.error, "ops json: input role " + kv.first + " of " + op.func + " needs an argument index");
            op.inputs[kv.first] = (int)kv.second.num;
        }
        out.funcs.push_back(op);
    }
    return Status::Succ;
}

Status check_export_ops(const TvmExport &ex, const ExportOps &ops, std::string &error) {
    std::map<std::string, int> described;
    for (const ExportOp &o : ops.funcs) ++described[o.func];
    std::set<std::string> wanted;
    for (const std::string &f : ex.kernel_func) if (f != "__nop") wanted.insert(f);
    for (const std::string &f : wanted) {
        auto it = described.find(f);
        if (it == described.end()) return fail(error, "ops json does not describe " + f);
        if (it->second != 1) return fail(error, "ops json describes " + f + " more than once");
    }
    for (const auto &kv : described)
        if (!wanted.count(kv.first)) return fail(error, "ops json describes " + kv.first + ", which the export does not contain");
    return Status::Succ;
}

}  // namespace foo
