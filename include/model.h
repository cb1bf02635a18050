// foo::Model — storages + kernel list of one DNN, and its on-disk parameter format.
//
// Public interface of the reference's include/model.h:12-100 (same class and method names,
// argument meaning and Status results).  What differs underneath: the reference loads a
// TVM-compiled GPU module and two JSON files; here the kernel list is built natively from the
// workload name and every kernel is an operator of libgpreempt_hip.so.
#pragma once
#include <cstdint>
#include <memory>
#include <string>
#include <unordered_map>
#include <vector>
#include "util/common.h"
#include "util/gpu_util.h"

namespace foo {

using namespace foo::util;
struct TvmExport;

class StorageInfo {
public:
    std::string name;
    size_t size;        // bytes
    std::string stype;  // "float32" "float16" "bfloat16" "int64" "int32" "byte" "uint1"
};

// How a parameter that is stored on disk in the reference's convention (fp32; OIHW convolution
// weights; dense weights [out][in] over an NCHW flatten) maps onto the device layout
// (model dtype; [O][H][W][I padded]; dense over an NHWC flatten).
struct ParamLayout {
    enum Kind { Plain, ConvOIHW, DenseOverCHW, MatKN } kind = Plain;
    int o = 0, i = 0, r = 0, s = 0, i_pad = 0;  // ConvOIHW; MatKN: a K x N matrix on disk (i = K, o = N), kept N x K on the device
    int c = 0, h = 0, w = 0;                    // DenseOverCHW: input features were flattened from C x H x W (device rows: H x W x max(C, i_pad))
    size_t disk_elems = 0;                      // fp32 values expected on disk
    bool is_param = false;
    // seeded initial value when no parameter file is given
    enum Init { InitZero, InitNormal /* N(0, a) */, InitUniform /* U[a, b] */, InitConst /* a */, InitData /* *init_data */ } init = InitZero;
    float init_a = 0.f, init_b = 0.f;
    std::shared_ptr<std::vector<float>> init_data;  // InitData: disk_elems values computed by the builder
};

enum class OpKind { Nop, Gemm, Conv, Layout, Pool, Eltwise, Softmax, Layernorm, Embed, Attention, Stencil };

struct ArgRef {
    size_t storage = SIZE_MAX;  // SIZE_MAX = absent
    size_t byte_offset = 0;
};

class KernelInfo {
public:
    std::string name;            // operator name; "nop" is a device-to-device copy (reference model.cpp:201-207)
    uint32_t launch_params[6];   // grid x,y,z and block x,y,z as last planned by the device layer
    OpKind op = OpKind::Nop;
    union {
        gp_gemm_params gemm;
        gp_conv_params conv;
        gp_attention_params attention;
        gp_layout_params layout;
        gp_pool_params pool;
        gp_eltwise_params eltwise;
        gp_softmax_params softmax;
        gp_layernorm_params layernorm;
        gp_embed_params embed;
        gp_miniweather_params miniweather;
    } p;
    std::vector<size_t> args_index;       // storage index per pointer slot (SIZE_MAX = absent)
    std::vector<ArgRef> refs;             // same slots with byte offsets into the storage
    std::vector<GPUdeviceptr> args;       // resolved device pointers
    std::vector<GPUdeviceptr *> args_ptr; // extra by-reference arguments appended by batchAddParam
    // block-level preemption arguments (reference model.cpp:366-396)
    bool preemptible = false;
    int total_blocks = 0;
    bool fixed_claims = false;            // how the last launch recorded its claims (gp_launch_info)
    int front_workgroups = 0;             // of launch_params[0], the workgroups that own no claim (gp_launch_info::front)
    GPUdeviceptr executed = nullptr;
    int kernel_id = 0;
    double flops = 0, bytes = 0;          // algorithmic work of one launch
    // Launch fusion (Model::plan_fusions): a layer-norm whose only job before the next kernel is to feed
    // that kernel's A operand is not launched (`fused_away`); the dense layer behind it runs `ln_gemm`,
    // the same GEMM with the layer-norm as its prologue (preemptible or not).  The kernel list, its
    // indices and the whole-model program keep the two-kernel form.
    bool fused_away = false;
    bool has_ln_gemm = false;
    gp_gemm_params ln_gemm;
};

class Model {
public:
    Model();
    Model(const std::string &device_json, const std::string &host_json, const std::string &cuda_module);
    ~Model();

    // The three paths name files inside MODEL_PATH/<workload>/ as in the reference
    // (src/executor.cpp:110-113); the workload is the name of that directory and the graph is
    // built natively from it.  `workload` may carry options: "resnet152@b=8,dtype=f16".
    // When mod.json and host.json exist they are read as the reference reads them (load_from_json).
    // With an ops.json next to them (the operator sidecar of include/tvm_export.h) the exported graph
    // is what runs, operator by operator on the native kernels, under whatever name the directory
    // has.  Without one the native graph of that workload name runs, and the export must describe a
    // model with the same input ("data") and output ("heads") sizes; a mismatch, or files that do
    // not parse, is Status::Fail (a caller that brings a different graph under a known name must
    // not silently get the built-in one).
    Status load_model(const std::string &device_json, const std::string &host_json, const std::string &cuda_module);
    // Model::load_from_json of the reference (src/model.cpp:128-235): storages and device kernels
    // of an exported model.  The result is kept for inspection (tvm_export()); it does not replace
    // the native graph.
    Status load_from_json(const char *device_json, const char *host_json);
    const struct TvmExport *tvm_export() const { return export_.get(); }
    Status build(const std::string &workload);
    // Fills the kernel list from the export read by load_from_json plus the text of its operator
    // sidecar; allocates nothing (load_model does that next).
    Status build_from_export(const std::string &workload, const std::string &ops_json_text);

    // Reads a "TVM_MODEL_PARAMS" file (format of reference src/model.cpp:15-55) and uploads every
    // tensor whose key names a storage.  Parameters missing from the file keep their seeded
    // random initialisation.  A missing file is not an error: the model stays random-init.
    Status load_param(const char *param_file_path);

    bool is_loaded();
    size_t get_kernel_num() const;
    size_t get_storage_num() const;
    size_t get_storage_size(size_t idx);
    StorageInfo &get_storage_info(size_t idx);
    KernelInfo &get_kernel_info(size_t idx);
    GPUdeviceptr get_storage_ptr(size_t idx);
    const ParamLayout &get_param_layout(size_t idx) const { return layouts[idx]; }

    Status get(size_t idx, void *out, size_t len, GPUstream stream);
    Status get(const std::string &key, void *out, size_t len, GPUstream stream);
    Status set(size_t idx, void *value, size_t len, GPUstream stream);
    Status set(const std::string &key, void *value, size_t len, GPUstream stream);

    static size_t get_stype_size(std::string &stype);
    Status find_storage_idx(const std::string &name, size_t &idx);
    Status get_global_ptr(const std::string &name, GPUdeviceptr *ptr);
    Status clear();

    Status batchAddParam(GPUdeviceptr *ptr);
    // `ptr` holds the claim counters: counter_groups counters per kernel, 64 bytes apart
    // (counter_groups = 1 is the reference's one int per kernel, src/model.cpp:366-396).
    Status add_block_preemption_param(GPUdeviceptr ptr, int counter_groups = 1);

    // Launches kernel `idx` on `stream` (what src/executor.cpp:136-164 does with
    // GPULaunchKernel); preemptible kernels take their flag and stop index from the by-reference
    // arguments added with batchAddParam.  inject_at is a test hook (-1 = off).
    Status launch(size_t idx, GPUstream stream, int inject_at = -1);
    void set_poll_every(int n) { poll_every_ = n; }
    // The claim counters have just been cleared (or are about to be, earlier on the same stream):
    // until its next launch every kernel is known to have made no claim (gp_preempt_ctx::fresh).
    // `on` = false withdraws that for all kernels (launches that are recorded and replayed).
    void counters_cleared(bool on) { fresh_.assign(kernel_infos.size(), on ? 1 : 0); launches_.assign(kernel_infos.size(), 0); }
    // every kernel has been launched once more by something else than launch() (a replayed graph)
    void launched_once_more() { for (int &n : launches_) ++n; }
    // counters of the workers that have left, behind the claim counters (gp_preempt_ctx::done): byte distance from `executed`
    void set_done_counters(size_t byte_offset) { done_offset_ = byte_offset; }
    // device-visible address of a host word that a program's last leaving workgroup sets to the
    // launch number returned by launch_program()
    void set_left_word(GPUdeviceptr p) { left_word_ = p; }
    // workspace that lets long GEMM tiles be left between two K-steps (gp_preempt_ctx::ckpt)
    void set_checkpoint_workspace(GPUdeviceptr p, size_t bytes) { ckpt_ = p; ckpt_bytes_ = bytes; }
    // device time stamps of preemptions (gp_preempt_ctx::stamps); null = off
    void set_stamps(GPUdeviceptr p) { stamps_ = p; }
    // A word of host memory (its device-visible address) in which every preemptible launch stores its number when its
    // first workgroup starts (gp_preempt_ctx::started_host); launch numbers count from 1 after restart_launch_numbers().
    void set_started_word(GPUdeviceptr p) { started_ = p; launch_seq_ = 0; }
    void restart_launch_numbers() { launch_seq_ = 0; }
    int launch_number() const { return launch_seq_; }
    // largest such workspace any kernel of the model can use (0: none can)
    size_t checkpoint_bytes_wanted() const;
    int last_launch_tag() const { return last_launch_tag_; }

    // Whole-model program: all kernels as one persistent device kernel (the counterpart of the
    // captured graph of src/executor.cpp:176-196).  build_program() is idempotent.
    Status build_program();
    bool has_program() const { return program_ != nullptr; }
    // reset = true starts from the first tile, false continues from the counters of a stopped run.
    Status launch_program(GPUstream stream, bool reset, int inject_layer = -1, int inject_claim = -1);
    // per-layer claim counters of the program (blocking)
    Status read_program_counters(std::vector<int> &executed, std::vector<int> &done, int &error);

    int counter_groups() const { return counter_groups_; }
    const std::string &workload() const { return workload_; }
    const std::string &dtype() const { return dtype_; }
    double total_flops() const;
    double total_bytes() const;

    friend class GraphBuilder;

private:
    bool loaded_ = false;
    gp_program program_ = nullptr;
    int counter_groups_ = 1;
    int poll_every_ = 0;
    std::vector<char> fresh_;
    std::vector<int> launches_;           // per kernel: launches since the counters were cleared (gp_preempt_ctx::done_launches)
    size_t done_offset_ = 0;              // 0: no done counters
    GPUdeviceptr left_word_ = nullptr;
    GPUdeviceptr ckpt_ = nullptr;
    size_t ckpt_bytes_ = 0;
    GPUdeviceptr stamps_ = nullptr;
    GPUdeviceptr started_ = nullptr;      // see set_started_word
    int launch_seq_ = 0;
    int last_launch_tag_ = 0;
    std::string workload_, dtype_;
    std::shared_ptr<struct TvmExport> export_;
    std::vector<StorageInfo> storage_infos;
    std::vector<ParamLayout> layouts;
    std::vector<KernelInfo> kernel_infos;
    std::vector<GPUdeviceptr> storages;
    std::unordered_map<std::string, size_t> storages_idx;

    Status allocate_and_bind();
    void plan_fusions();
    bool fuse_launches_ = true;  // GPREEMPT_FUSE_LN=0 in the environment keeps every launch of the kernel list
    bool eager_tiles_ = true;    // first launches start their tiles before the stop index has come back (gp_preempt_ctx::fresh = 2); GPREEMPT_EAGER_TILES=0 makes them wait for it
    Status upload_param(size_t idx, const float *disk, size_t n);
    void bind_pointers(KernelInfo &k);
};

typedef std::unordered_map<std::string, std::vector<float>> ModelParam;

class ModelParamParser {
public:
    // nullptr when the file is missing or malformed (the reference aborts instead).
    static ModelParam *parse_from_file(const char *param_file);
};

}  // namespace foo
