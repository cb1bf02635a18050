// Reader of the reference's exported model directory: TVM's graph-executor JSON (mod.json), the
// patched TVM's host-side launch record (host.json) and, as an extension, an operator-attribute
// sidecar (ops.json).
//
// parse_tvm_export follows Model::load_from_json of the reference (src/model.cpp:128-235) rule by
// rule; what it yields is the reference's own view of a model: storages (graph nodes first, then
// the temporary buffers) and device kernels with launch dimensions and storage indices.  The
// exported files do not say what a kernel computes (a convolution's stride and padding, a pool's
// window, which input of a fused add is the residual live only inside the generated device code),
// so running an export on the native operators needs the sidecar, which the export script can
// write from the Relay module it holds (scripts/compile/compile.py:46-57).
#pragma once
#include <map>
#include <string>
#include <vector>
#include "model.h"

namespace foo {

// One node of mod.json's graph: a tensor (an input or parameter when `func` is empty, else the result of
// the host function `func`, "__nop" for a reshape).  The reference reads only the flattened view below;
// the node view is what the native loader builds its kernels from.
struct ExportNode {
    std::string name, func, stype;
    std::vector<long> shape;
    std::vector<size_t> inputs;  // node ids
};

struct TvmExport {
    std::vector<ExportNode> nodes;           // [0, global_len)
    std::vector<StorageInfo> storage_infos;  // [0, global_len): graph nodes; then one "temp" per host.json temp_args entry
    std::vector<KernelInfo> kernel_infos;    // name, launch_params, args_index as the reference fills them; "nop" for __nop nodes
    std::vector<std::string> kernel_func;    // host function (fused operator) each kernel belongs to; "__nop" for copies
    size_t global_len = 0;
    size_t heads_index = 0;                  // the storage renamed to "heads"
    std::string error;                       // what went wrong when the result is not Succ
};

// NotFound: a file cannot be opened.  Fail: malformed JSON, a missing key, a function-name mismatch
// between the two files (src/model.cpp:208-211), or an argument index out of range.
Status parse_tvm_export(const std::string &device_json_text, const std::string &host_json_text, TvmExport &out);
Status load_tvm_export(const char *device_json_path, const char *host_json_path, TvmExport &out);

// ---- operator-attribute sidecar (ops.json) ----------------------------------------------------------
// { "layout": "NCHW",
//   "funcs": [ { "name": "<host function, as in host.json>",
//                "op": "conv2d" | "dense" | "max_pool2d" | "avg_pool2d" | "global_avg_pool2d" | "add" | "softmax" |
//                      "layer_norm" | "batch_matmul" | "take" | "scale_shift" | "concatenate" | "reshape",
//                "attrs": { "strides": [1,1], "padding": [1,1,1,1], "dilation": [1,1], "groups": 1, "pool_size": [3,3],
//                           "count_include_pad": 0, "axis": 1, "epsilon_e12": 1, ... },       integers or integer lists
//                "epilogue": ["bias", "residual", "relu"],     fused tail, in order, of "bias" "residual" "relu" "gelu"
//                "inputs": {"data": 0, "weight": 1, "bias": 2, "residual": 3} } ] }   role -> index among the function's arguments
struct ExportOp {
    std::string func, op;
    std::map<std::string, std::vector<long>> attrs;
    std::vector<std::string> epilogue;
    std::map<std::string, int> inputs;
};
struct ExportOps {
    std::string layout = "NCHW";
    std::vector<ExportOp> funcs;
    std::string error;
};
Status parse_export_ops(const std::string &ops_json_text, ExportOps &out);
// Every non-"__nop" host function of the export must be described exactly once, by name.
Status check_export_ops(const TvmExport &ex, const ExportOps &ops, std::string &error);

// ---- an export on the native operators ----------------------------------------------------------------
// Appends to `m` the storages and kernels that compute the exported graph with the operators of
// libgpreempt_hip.so, in the element type `dtype` ("f32" "f16" "bf16"; empty = the export's own).
// Activations are kept NHWC; parameters keep the export's node names ("p0", "p1", ...) and are declared
// in the export's on-disk convention (fp32; OIHW convolution weights; dense weights [units][features]
// over an NCHW flatten), so that the export's own mod.params loads into them (src/model.cpp:263-282).
// "data" and "heads" have the export's shapes (NCHW data).  Mapped: conv2d (groups 1, dilation 1,
// symmetric padding), dense, max / average / global-average pooling, add, scale_shift, softmax over the
// last axis, concatenate over channels (its arguments are computed in place in its buffer where they can
// be, copied otherwise), reshape / __nop between a 4-D tensor and its NCHW flatten.  Anything
// else (the attention and layer-norm functions of a BERT export among them) is Status::Fail with `error`
// naming the function: nothing is guessed.
class GraphBuilder;
Status build_export_graph(GraphBuilder &b, const TvmExport &ex, const ExportOps &ops, std::string &error);

}  // namespace foo
