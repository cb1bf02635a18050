// foo::Model: storage planning, parameter loading and kernel launch over the C ABI.
// Follows the behaviour of the reference's src/model.cpp (cited per function); the graph itself
// comes from the native builders in zoo.cpp instead of TVM's mod.json / host.json.
#include "model.h"
#include <cstdlib>

#include <cmath>
#include <cstring>
#include <fstream>

#include "numeric.h"
#include "tvm_export.h"
#include "graph_builder.h"
#include "zoo.h"
#include <sys/stat.h>

namespace foo {

static const char kParamMagic[] = "TVM_MODEL_PARAMS";  // 16 chars + NUL = 17 bytes on disk

// File layout (reference src/model.cpp:15-55): magic[17] | u64 count | count x { key\0 | u64 n | f32[n] }.
ModelParam *ModelParamParser::parse_from_file(const char *param_file) {
    FILE *fp = std::fopen(param_file, "rb");
    if (!fp) return nullptr;
    // every count read from the file is checked against what the file can still hold before
    // anything is allocated for it: a corrupt header must not ask for 64 GiB
    struct stat sb;
    const uint64_t file_size = fstat(fileno(fp), &sb) == 0 && sb.st_size > 0 ? (uint64_t)sb.st_size : 0;
    std::unique_ptr<ModelParam> params(new ModelParam());
    char magic[sizeof(kParamMagic)];
    uint64_t count = 0;
    bool ok = std::fread(magic, 1, sizeof(magic), fp) == sizeof(magic) && std::memcmp(magic, kParamMagic, sizeof(magic)) == 0 &&
              std::fread(&count, sizeof(count), 1, fp) == 1 && count != 0 && count <= file_size / 10;  // a tensor takes >= 10 bytes
    for (uint64_t i = 0; ok && i < count; ++i) {
        std::string key;
        int c;
        while ((c = std::fgetc(fp)) != EOF && c != 0 && key.size() < 255) key.push_back((char)c);
        uint64_t n = 0;
        ok = c == 0 && std::fread(&n, sizeof(n), 1, fp) == 1 && n != 0 && n < (1ull << 34);
        const long at = ok ? std::ftell(fp) : -1;
        ok = ok && at >= 0 && (uint64_t)at <= file_size && n <= (file_size - (uint64_t)at) / sizeof(float);
        if (!ok) break;
        std::vector<float> values(n);
        ok = std::fread(values.data(), sizeof(float), n, fp) == n;
        if (ok) (*params)[key] = std::move(values);
    }
    std::fclose(fp);
    if (!ok) {
        std::fprintf(stderr, "malformed parameter file %s\n", param_file);
        return nullptr;
    }
    return params.release();
}

Model::Model() {}

Model::Model(const std::string &device_json, const std::string &host_json, const std::string &cuda_module) {
    load_model(device_json, host_json, cuda_module);
}

Model::~Model() { clear(); }

// reference src/model.cpp:69-77, extended with the 16-bit float types the configurations need
size_t Model::get_stype_size(std::string &stype) {
    if (stype == "float32") return 4;
    if (stype == "float16" || stype == "bfloat16") return 2;
    if (stype == "int64") return 8;
    if (stype == "int32") return 4;
    if (stype == "byte" || stype == "uint1") return 1;
    std::fprintf(stderr, "Unknown stype: %s\n", stype.c_str());
    return 0;
}

static std::string parent_dir_name(const std::string &path) {
    size_t end = path.find_last_of('/');
    if (end == std::string::npos) return "";
    std::string dir = path.substr(0, end);
    while (!dir.empty() && dir.back() == '/') dir.pop_back();
    size_t b = dir.find_last_of('/');
    return b == std::string::npos ? dir : dir.substr(b + 1);
}

Status Model::load_model(const std::string &device_json, const std::string &host_json, const std::string & /*module*/) {
    if (is_loaded()) {
        std::fprintf(stderr, "The model is already loaded\n");  // reference model.cpp:81-84
        return Status::Fail;
    }
    std::string name = parent_dir_name(device_json);
    if (name.empty()) return Status::NotFound;
    // an exported graph next to the parameters is read the reference's way and checked below
    std::ifstream dj(device_json), hj(host_json);
    const bool have_export = dj.is_open() && hj.is_open();
    dj.close(); hj.close();
    if (have_export) {
        Status s = load_from_json(device_json.c_str(), host_json.c_str());
        if (s != Status::Succ) {
            std::fprintf(stderr, "load_model: %s\n", export_ ? export_->error.c_str() : "cannot read the exported graph");
            return s;
        }
    }
    if (have_export) {
        // with an operator sidecar next to it, the export itself is the graph that runs
        const std::string ops_json = device_json.substr(0, device_json.find_last_of('/') + 1) + "ops.json";
        std::ifstream oj(ops_json);
        if (oj.is_open()) {
            const std::string text((std::istreambuf_iterator<char>(oj)), std::istreambuf_iterator<char>());
            RETURN_STATUS(build_from_export(name, text));
            return allocate_and_bind();
        }
    }
    RETURN_STATUS(build(name));
    if (have_export) {
        // the native graph runs; the export must at least agree with it on what goes in and comes out
        // (in ELEMENTS: the reference's exports are float32 while the native graphs default to 16-bit
        // types, and the same model in another element type is still the same model)
        auto find = [](std::vector<StorageInfo> &v, const std::string &key) -> StorageInfo * {
            for (StorageInfo &s : v) if (s.name == key) return &s;
            return nullptr;
        };
        for (const char *key : {"data", "heads"}) {
            StorageInfo *a = find(export_->storage_infos, key), *b = find(storage_infos, key);
            const size_t ea = a ? get_stype_size(a->stype) : 0, eb = b ? get_stype_size(b->stype) : 0;
            const long na = ea ? (long)(a->size / ea) : -1, nb = eb ? (long)(b->size / eb) : -1;
            if (na != nb) {
                std::fprintf(stderr, "load_model: %s describes a model whose \"%s\" holds %ld elements (%s); the native graph of workload '%s' has %ld (%s): "
                                     "refusing to run a different model under this name (name the directory with the options that match the export, e.g. '%s@b=1')\n",
                             device_json.c_str(), key, na, a ? a->stype.c_str() : "absent", name.c_str(), nb, b ? b->stype.c_str() : "absent", name.substr(0, name.find('@')).c_str());
                clear();
                return Status::Fail;
            }
        }
        std::fprintf(stderr, "load_model: %s and %s read (%zu storages, %zu kernels); the kernels that run are the native ones of workload '%s'\n",
                     device_json.c_str(), host_json.c_str(), export_->storage_infos.size(), export_->kernel_infos.size(), name.c_str());
    }
    return Status::Succ;
}

Status Model::load_from_json(const char *device_json, const char *host_json) {
    export_ = std::make_shared<TvmExport>();
    return load_tvm_export(device_json, host_json, *export_);
}

// The export's host functions replaced one for one by native operators (include/tvm_export.h).  The element type
// is the export's own unless the workload name asks for another ("<directory>@dtype=f16").
Status Model::build_from_export(const std::string &workload, const std::string &ops_json_text) {
    if (is_loaded() || !export_) return Status::Fail;
    ExportOps ops;
    std::string err;
    Status s = parse_export_ops(ops_json_text, ops);
    if (s != Status::Succ) err = ops.error;
    if (s == Status::Succ) s = check_export_ops(*export_, ops, err);
    std::string dt;
    size_t at = workload.find("dtype=");
    if (at != std::string::npos && workload.find('@') < at) dt = workload.substr(at + 6, workload.find(',', at) == std::string::npos ? std::string::npos : workload.find(',', at) - at - 6);
    if (s == Status::Succ && dt.empty()) {
        auto type_of = [](const std::string &stype) { return stype == "float32" ? "f32" : stype == "float16" ? "f16" : ""; };
        for (const ExportNode &n : export_->nodes)
            if (n.func.empty() && n.name == "data") dt = type_of(n.stype);
        // a model fed token ids (int64 "data"): the element type is that of its output
        if (dt.empty() && export_->heads_index < export_->nodes.size()) dt = type_of(export_->nodes[export_->heads_index].stype);
        if (dt.empty()) { err = "neither the export's data nor its output is float32 or float16"; s = Status::Fail; }
    }
    if (s == Status::Succ && dt != "f32" && dt != "f16" && dt != "bf16") { err = "unknown dtype '" + dt + "'"; s = Status::Fail; }
    if (s == Status::Succ) {
        GraphBuilder b(*this, dt);
        s = build_export_graph(b, *export_, ops, err);
    }
    if (s != Status::Succ) {
        std::fprintf(stderr, "load_model: %s\n", err.c_str());
        export_->error = err;
        storage_infos.clear(); layouts.clear(); kernel_infos.clear();
        return s;
    }
    workload_ = workload;
    return Status::Succ;
}

Status Model::build(const std::string &workload) {
    if (is_loaded()) return Status::Fail;
    workload_ = workload;
    Status s = zoo_build(*this, workload);
    if (s != Status::Succ) {
        storage_infos.clear(); layouts.clear(); kernel_infos.clear();
        return s;
    }
    return allocate_and_bind();
}

// One zero-filled device buffer per storage, then resolve every kernel's pointer slots
// (reference src/model.cpp:100-124).
Status Model::allocate_and_bind() {
    storages.assign(storage_infos.size(), nullptr);
    for (size_t i = 0; i < storage_infos.size(); ++i) {
        size_t bytes = storage_infos[i].size;
        CUDA_RETURN_STATUS(gp_malloc(&storages[i], bytes));
        CUDA_RETURN_STATUS(gp_fill32_async(storages[i], 0, bytes / 4, nullptr));
        if (bytes % 4) {
            std::vector<char> z(bytes % 4, 0);
            CUDA_RETURN_STATUS(gp_memcpy_h2d((char *)storages[i] + bytes - bytes % 4, z.data(), z.size()));
        }
        storages_idx.emplace(storage_infos[i].name, i);
    }
    CUDA_RETURN_STATUS(gp_stream_sync(nullptr));
    for (KernelInfo &k : kernel_infos) {
        k.args.clear();
        k.args_index.clear();
        k.args.reserve(k.refs.size() + 10);
        for (const ArgRef &r : k.refs) {
            k.args_index.push_back(r.storage);
            k.args.push_back(r.storage == SIZE_MAX ? nullptr : (GPUdeviceptr)((char *)storages[r.storage] + r.byte_offset));
        }
        bind_pointers(k);
    }
    loaded_ = true;
    plan_fusions();
    // seeded random initialisation of every parameter (overwritten by load_param when a file exists)
    uint64_t seed = 0x5EEDull;
    for (size_t i = 0; i < storage_infos.size(); ++i) {
        const ParamLayout &L = layouts[i];
        if (!L.is_param) continue;
        std::vector<float> host(L.disk_elems, 0.f);
        numeric::Rng rng(seed + 7919 * (uint64_t)i);
        switch (L.init) {
            case ParamLayout::InitZero: break;
            case ParamLayout::InitConst: for (float &v : host) v = L.init_a; break;
            case ParamLayout::InitUniform: for (float &v : host) v = rng.uniform(L.init_a, L.init_b); break;
            case ParamLayout::InitNormal: for (float &v : host) v = rng.normal() * L.init_a; break;
            case ParamLayout::InitData: if (L.init_data && L.init_data->size() == host.size()) host = *L.init_data; break;
        }
        RETURN_STATUS(upload_param(i, host.data(), host.size()));
    }
    return Status::Succ;
}

// layer_norm -> dense pairs that run as one launch (gp_gemm_params::ln_gamma), where the device layer says the
// fused launch has the bits of the two (gp_gemm_ln_supported).  For a preemptible tenant the fused launch
// carries the dense layer's kernel index, claim counters and tiles: the layer-norm's index is never launched,
// so it never appears as a stop index, its counters stay zero, and a preemption injected at it (a test hook)
// does not fire; a run stopped inside the fused launch resumes there, and the tiles that are left redo
// their rows (the workgroups of tile column 0 are the ones that store them).
void Model::plan_fusions() {
    const char *env = std::getenv("GPREEMPT_FUSE_LN");
    fuse_launches_ = !(env && std::atoi(env) == 0);
    env = std::getenv("GPREEMPT_EAGER_TILES");
    eager_tiles_ = !(env && std::atoi(env) == 0);
    for (size_t i = 0; i + 1 < kernel_infos.size(); ++i) {
        KernelInfo &ln = kernel_infos[i], &mm = kernel_infos[i + 1];
        ln.fused_away = false; mm.has_ln_gemm = false;
        if (ln.op != OpKind::Layernorm || mm.op != OpKind::Gemm) continue;
        const gp_layernorm_params &l = ln.p.layernorm;
        const gp_gemm_params &g = mm.p.gemm;
        if (l.residual || g.A != l.out || g.K != l.cols || g.lda != l.cols || (long)g.M != l.rows || g.batch > 1 || g.dtype != l.dtype) continue;
        if (g.C == l.out || g.residual == l.out || g.C == l.x || l.out == l.x) continue;
        if (gp_gemm_ln_supported(&g) != 1) continue;
        mm.ln_gemm = g;
        mm.ln_gemm.A = l.x;
        mm.ln_gemm.ln_gamma = l.gamma; mm.ln_gemm.ln_beta = l.beta; mm.ln_gemm.ln_out = l.out; mm.ln_gemm.ln_eps = l.eps;
        mm.has_ln_gemm = true;
        ln.fused_away = true;
    }
}

// Slot order per operator is fixed by the builders in zoo.cpp.
void Model::bind_pointers(KernelInfo &k) {
    auto P = [&](size_t j) -> void * { return j < k.args.size() ? k.args[j] : nullptr; };
    switch (k.op) {
        case OpKind::Nop: break;
        case OpKind::Gemm: k.p.gemm.A = P(0); k.p.gemm.B = P(1); k.p.gemm.bias = P(2); k.p.gemm.residual = P(3); k.p.gemm.C = P(4); break;
        case OpKind::Conv: k.p.conv.in = P(0); k.p.conv.weight = P(1); k.p.conv.bias = P(2); k.p.conv.residual = P(3); k.p.conv.out = P(4); break;
        case OpKind::Layout: k.p.layout.in = P(0); k.p.layout.out = P(1); break;
        case OpKind::Pool: k.p.pool.in = P(0); k.p.pool.out = P(1); break;
        case OpKind::Eltwise: k.p.eltwise.a = P(0); k.p.eltwise.b = P(1); k.p.eltwise.scale = P(2); k.p.eltwise.shift = P(3); k.p.eltwise.out = P(4); break;
        case OpKind::Softmax: k.p.softmax.x = P(0); k.p.softmax.out = P(1); break;
        case OpKind::Layernorm: k.p.layernorm.x = P(0); k.p.layernorm.residual = P(1); k.p.layernorm.gamma = P(2); k.p.layernorm.beta = P(3); k.p.layernorm.out = P(4); break;
        case OpKind::Attention: k.p.attention.q = P(0); k.p.attention.k = P(1); k.p.attention.v = P(2); k.p.attention.out = P(3); break;
        case OpKind::Stencil:
            k.p.miniweather.state = (float *)P(0); k.p.miniweather.flux = (float *)P(1); k.p.miniweather.state_init = (const float *)P(2);
            k.p.miniweather.state_out = (float *)P(3); k.p.miniweather.hydro = (const float *)P(4);
            break;
        case OpKind::Embed: k.p.embed.ids = (const int64_t *)P(0); k.p.embed.tok = P(1); k.p.embed.pos = P(2); k.p.embed.seg = P(3); k.p.embed.out = P(4); break;
    }
}

// disk convention (fp32, OIHW / dense over CHW) -> device layout and dtype
Status Model::upload_param(size_t idx, const float *disk, size_t n) {
    const ParamLayout &L = layouts[idx];
    StorageInfo &info = storage_infos[idx];
    size_t es = get_stype_size(info.stype);
    size_t dev_elems = info.size / es;
    if (n < L.disk_elems) return Status::OutOfRange;
    std::vector<float> dev(dev_elems, 0.f);
    switch (L.kind) {
        case ParamLayout::Plain:
            std::memcpy(dev.data(), disk, sizeof(float) * std::min(dev_elems, n));
            break;
        case ParamLayout::ConvOIHW:
            for (int o = 0; o < L.o; ++o)
                for (int i = 0; i < L.i; ++i)
                    for (int r = 0; r < L.r; ++r)
                        for (int s = 0; s < L.s; ++s)
                            dev[(((size_t)o * L.r + r) * L.s + s) * L.i_pad + i] = disk[(((size_t)o * L.i + i) * L.r + r) * L.s + s];
            break;
        case ParamLayout::MatKN:  // K x N -> N x K: the matrix kernels want both operands K-contiguous
            for (int k = 0; k < L.i; ++k)
                for (int nn = 0; nn < L.o; ++nn) dev[(size_t)nn * L.i + k] = disk[(size_t)k * L.o + nn];
            break;
        case ParamLayout::DenseOverCHW: {
            // rows of C x H x W features on disk, H x W x (C padded to i_pad) on the device
            const size_t feat = (size_t)L.c * L.h * L.w, cp = L.i_pad > L.c ? (size_t)L.i_pad : (size_t)L.c, feat_dev = cp * L.h * L.w;
            if ((size_t)L.o * feat_dev > dev_elems) return Status::OutOfRange;
            for (int o = 0; o < L.o; ++o)
                for (int c = 0; c < L.c; ++c)
                    for (int h = 0; h < L.h; ++h)
                        for (int w = 0; w < L.w; ++w)
                            dev[o * feat_dev + ((size_t)h * L.w + w) * cp + c] = disk[o * feat + ((size_t)c * L.h + h) * L.w + w];
            break;
        }
    }
    if (info.stype == "float32") {
        CUDA_RETURN_STATUS(gp_memcpy_h2d(storages[idx], dev.data(), info.size));
    } else {
        std::vector<uint16_t> half(dev_elems);
        const bool bf = info.stype == "bfloat16";
        for (size_t i = 0; i < dev_elems; ++i) half[i] = bf ? numeric::f32_to_bf16(dev[i]) : numeric::f32_to_f16(dev[i]);
        CUDA_RETURN_STATUS(gp_memcpy_h2d(storages[idx], half.data(), info.size));
    }
    return Status::Succ;
}

// reference src/model.cpp:263-282: copy a tensor only if a storage of the same name exists
Status Model::load_param(const char *param_file_path) {
    if (!is_loaded()) return Status::Fail;
    std::ifstream probe(param_file_path, std::ios::binary);
    if (!probe.is_open()) return Status::Succ;  // random-init model
    probe.close();
    std::unique_ptr<ModelParam> params(ModelParamParser::parse_from_file(param_file_path));
    if (!params) return Status::Fail;
    for (size_t i = 0; i < storages.size(); ++i) {
        auto it = params->find(storage_infos[i].name);
        if (it == params->end()) continue;
        if (!layouts[i].is_param) continue;
        RETURN_STATUS(upload_param(i, it->second.data(), it->second.size()));
    }
    return Status::Succ;
}

bool Model::is_loaded() { return loaded_; }

Status Model::find_storage_idx(const std::string &name, size_t &idx) {
    auto it = storages_idx.find(name);
    if (it == storages_idx.end()) return Status::NotFound;
    idx = it->second;
    return Status::Succ;
}

// reference src/model.cpp:296-313: `len` is the caller's buffer size; exactly storage.size bytes move
Status Model::get(size_t idx, void *out, size_t len, GPUstream stream) {
    if (idx >= storages.size()) return Status::OutOfRange;
    size_t size = storage_infos[idx].size;
    if (len < size) return Status::Fail;
    CUDA_RETURN_STATUS(gp_memcpy_d2h_async(out, storages[idx], size, stream));
    return Status::Succ;
}
Status Model::get(const std::string &key, void *out, size_t len, GPUstream stream) {
    size_t idx;
    if (find_storage_idx(key, idx) != Status::Succ) return Status::NotFound;
    return get(idx, out, len, stream);
}
// reference src/model.cpp:315-330
Status Model::set(size_t idx, void *value, size_t len, GPUstream stream) {
    if (idx >= storages.size()) return Status::OutOfRange;
    size_t size = storage_infos[idx].size;
    if (len < size) return Status::OutOfRange;
    CUDA_RETURN_STATUS(gp_memcpy_h2d_async(storages[idx], value, size, stream));
    return Status::Succ;
}
Status Model::set(const std::string &key, void *value, size_t len, GPUstream stream) {
    size_t idx;
    if (find_storage_idx(key, idx) != Status::Succ) return Status::NotFound;
    return set(idx, value, len, stream);
}

size_t Model::get_kernel_num() const { return kernel_infos.size(); }
size_t Model::get_storage_num() const { return storage_infos.size(); }
StorageInfo &Model::get_storage_info(size_t idx) { return storage_infos[idx]; }
GPUdeviceptr Model::get_storage_ptr(size_t idx) { return storages[idx]; }
size_t Model::get_storage_size(size_t idx) { return storage_infos[idx].size; }
KernelInfo &Model::get_kernel_info(size_t idx) { return kernel_infos[idx]; }

// The reference resolves a symbol of the loaded GPU module (model.cpp:353-356); the native
// kernels have no module-level globals, so a name can only denote a storage.
Status Model::get_global_ptr(const std::string &name, GPUdeviceptr *ptr) {
    size_t idx;
    if (find_storage_idx(name, idx) != Status::Succ) return Status::NotFound;
    *ptr = storages[idx];
    return Status::Succ;
}

Status Model::clear() {
    if (program_) { gp_program_destroy(program_); program_ = nullptr; }
    if (!loaded_) return Status::Succ;
    for (GPUdeviceptr p : storages) CUDA_RETURN_STATUS(gp_free(p));
    storage_infos.clear(); layouts.clear(); kernel_infos.clear(); storages.clear(); storages_idx.clear();
    loaded_ = false;
    return Status::Succ;
}

// Appends one by-reference argument to every kernel, "nop" included (reference model.cpp:358-364).
// BLPExecutor::init calls it twice: first &dpStop (the flag), then &dpStopIndex.
Status Model::batchAddParam(GPUdeviceptr *ptr) {
    for (KernelInfo &k : kernel_infos) k.args_ptr.push_back(ptr);
    return Status::Succ;
}

// Per kernel: total_blocks, &executed[i], kernel id i; "nop" kernels are skipped but keep their
// index (reference model.cpp:366-396).  The persistent grid (min(total_blocks, resident
// workgroups)) is resolved by the device layer at launch.
Status Model::add_block_preemption_param(GPUdeviceptr ptr, int counter_groups) {
    counter_groups_ = counter_groups > 1 ? counter_groups : 1;
    for (size_t i = 0; i < kernel_infos.size(); ++i) {
        KernelInfo &k = kernel_infos[i];
        if (k.name == "nop") continue;
        if (k.args_ptr.size() < 2) return Status::Fail;
        k.preemptible = true;
        const size_t per_kernel = counter_groups_ > 1 ? sizeof(int) * counter_groups_ * 16 : sizeof(int);
        k.executed = (GPUdeviceptr)((char *)ptr + i * per_kernel);
        k.kernel_id = (int)i;
    }
    return Status::Succ;
}

size_t Model::checkpoint_bytes_wanted() const {
    size_t want = 0;
    for (const KernelInfo &k : kernel_infos) {
        if (!k.preemptible) continue;
        size_t b = 0;
        if (k.op == OpKind::Gemm && gp_gemm_ckpt_bytes(&k.p.gemm, &b) == 0 && b > want) want = b;
        // convolutions only on request: their checkpointing body is 25 % slower than the plain one
        // (VGG-16 b16: 187 vs 149 us per 128 x 128-tiled layer) for a drain that is 20 us shorter
        static const bool conv_ckpt = [] { const char *e = std::getenv("GPREEMPT_CONV_CHECKPOINT"); return e && *e == '1'; }();
        if (conv_ckpt && k.op == OpKind::Conv && gp_conv_ckpt_bytes(&k.p.conv, &b) == 0 && b > want) want = b;
    }
    return want;
}

Status Model::launch(size_t idx, GPUstream stream, int inject_at) {
    if (idx >= kernel_infos.size()) return Status::OutOfRange;
    KernelInfo &k = kernel_infos[idx];
    if (k.op == OpKind::Nop) {
        // reference src/executor.cpp:139-146: copy size(args_index[0]) bytes, args[1] <- args[0]
        size_t size = get_storage_size(k.args_index[0]);
        CUDA_RETURN_STATUS(gp_memcpy_d2d_async(k.args[1], k.args[0], size, stream));
        return Status::Succ;
    }
    const bool fuse = fuse_launches_;
    if (fuse && k.fused_away) return Status::Succ;  // the next kernel's prologue does this one's work
    gp_preempt_ctx ctx{};
    const gp_preempt_ctx *pc = nullptr;
    if (k.preemptible) {
        size_t n = k.args_ptr.size();
        ctx.flag = (int *)*k.args_ptr[n - 2];
        ctx.stop_index = (int *)*k.args_ptr[n - 1];
        ctx.executed = (int *)k.executed;
        ctx.kernel_id = k.kernel_id;
        ctx.inject_at = inject_at;
        ctx.max_workgroups = 0;
        ctx.poll_every = poll_every_;
        ctx.counter_groups = counter_groups_;
        ctx.fresh = idx < fresh_.size() && fresh_[idx] ? (eager_tiles_ ? 2 : 1) : 0;
        ctx.ckpt = ckpt_;
        ctx.ckpt_bytes = ckpt_bytes_;
        ctx.stamps = (unsigned long long *)stamps_;
        if (done_offset_) {
            ctx.done = (int *)((char *)k.executed + done_offset_);
            ctx.done_launches = idx < launches_.size() ? launches_[idx] : 0;
        }
        if (started_) {
            ctx.started_host = (int *)started_;
            ctx.started_seq = launch_seq_ + 1;
        }
        pc = &ctx;
    }
    gp_launch_info info{};
    int rc = GP_FAIL;
    switch (k.op) {
        case OpKind::Gemm: rc = gp_launch_gemm(fuse && k.has_ln_gemm ? &k.ln_gemm : &k.p.gemm, pc, stream, &info); break;
        case OpKind::Conv: rc = gp_launch_conv2d(&k.p.conv, pc, stream, &info); break;
        case OpKind::Layout: rc = gp_launch_nchw_to_nhwc(&k.p.layout, pc, stream, &info); break;
        case OpKind::Pool: rc = gp_launch_pool2d(&k.p.pool, pc, stream, &info); break;
        case OpKind::Eltwise: rc = gp_launch_eltwise(&k.p.eltwise, pc, stream, &info); break;
        case OpKind::Softmax: rc = gp_launch_softmax(&k.p.softmax, pc, stream, &info); break;
        case OpKind::Layernorm: rc = gp_launch_layernorm(&k.p.layernorm, pc, stream, &info); break;
        case OpKind::Embed: rc = gp_launch_embed(&k.p.embed, pc, stream, &info); break;
        case OpKind::Attention: rc = gp_launch_attention(&k.p.attention, pc, stream, &info); break;
        case OpKind::Stencil: rc = gp_launch_miniweather(&k.p.miniweather, pc, stream, &info); break;
        case OpKind::Nop: break;
    }
    if (idx < fresh_.size()) fresh_[idx] = 0;  // launched (or refused): from here on only its counters know
    if (idx < launches_.size() && rc == 0) ++launches_[idx];
    if (pc && started_ && rc == 0) ++launch_seq_;
    CUDA_RETURN_STATUS(rc);
    k.total_blocks = info.total_tiles;
    k.fixed_claims = info.fixed_claims != 0;
    k.launch_params[0] = (uint32_t)info.grid; k.launch_params[1] = 1; k.launch_params[2] = 1;
    k.front_workgroups = info.front;
    k.launch_params[3] = (uint32_t)info.block; k.launch_params[4] = 1; k.launch_params[5] = 1;
    return Status::Succ;
}

Status Model::build_program() {
    if (program_) return Status::Succ;
    if (!loaded_) return Status::Fail;
    int dt = dtype_ == "f32" ? GP_F32 : dtype_ == "f16" ? GP_F16 : GP_BF16;
    gp_program pr = nullptr;
    CUDA_RETURN_STATUS(gp_program_create(dt, &pr));
    for (size_t i = 0; i < kernel_infos.size(); ++i) {
        KernelInfo &k = kernel_infos[i];
        int rc = GP_FAIL;
        switch (k.op) {
            case OpKind::Nop: rc = gp_program_add_copy(pr, k.args[0], k.args[1], get_storage_size(k.args_index[0])); break;
            case OpKind::Gemm: rc = gp_program_add_gemm(pr, &k.p.gemm); break;
            case OpKind::Conv: rc = gp_program_add_conv2d(pr, &k.p.conv); break;
            case OpKind::Layout: rc = gp_program_add_nchw_to_nhwc(pr, &k.p.layout); break;
            case OpKind::Pool: rc = gp_program_add_pool2d(pr, &k.p.pool); break;
            case OpKind::Eltwise: rc = gp_program_add_eltwise(pr, &k.p.eltwise); break;
            case OpKind::Softmax: rc = gp_program_add_softmax(pr, &k.p.softmax); break;
            case OpKind::Layernorm: rc = gp_program_add_layernorm(pr, &k.p.layernorm); break;
            case OpKind::Embed: rc = gp_program_add_embed(pr, &k.p.embed); break;
            case OpKind::Attention: rc = gp_program_add_attention(pr, &k.p.attention); break;
            case OpKind::Stencil:  // launched kernel by kernel only
                std::fprintf(stderr, "build_program: the miniweather workload has no whole-model program\n");
                gp_program_destroy(pr);
                return Status::Fail;
        }
        if (rc != 0) {
            std::fprintf(stderr, "build_program: kernel %zu (%s): %s\n", i, k.name.c_str(), gp_last_error());
            gp_program_destroy(pr);
            return Status::Fail;
        }
    }
    if (gp_program_finalize(pr) != 0) {
        std::fprintf(stderr, "build_program: %s\n", gp_last_error());
        gp_program_destroy(pr);
        return Status::Fail;
    }
    program_ = pr;
    return Status::Succ;
}

Status Model::launch_program(GPUstream stream, bool reset, int inject_layer, int inject_claim) {
    if (!program_) return Status::Fail;
    gp_preempt_ctx ctx{};
    const gp_preempt_ctx *pc = nullptr;
    // preemptible when the executor attached its flag and stop index (batchAddParam)
    if (!kernel_infos.empty() && kernel_infos[0].args_ptr.size() >= 2) {
        size_t n = kernel_infos[0].args_ptr.size();
        ctx.flag = (int *)*kernel_infos[0].args_ptr[n - 2];
        ctx.stop_index = (int *)*kernel_infos[0].args_ptr[n - 1];
        ctx.kernel_id = inject_layer;
        ctx.inject_at = inject_layer >= 0 ? inject_claim : -1;
        ctx.poll_every = poll_every_;
        ctx.left_host = (int *)left_word_;
        ctx.stamps = (unsigned long long *)stamps_;
        pc = &ctx;
    }
    gp_launch_info info{};
    CUDA_RETURN_STATUS(gp_program_launch(program_, pc, reset ? 1 : 0, stream, &info));
    last_launch_tag_ = info.shape[1];
    return Status::Succ;
}

Status Model::read_program_counters(std::vector<int> &executed, std::vector<int> &done, int &error) {
    if (!program_) return Status::Fail;
    executed.assign(kernel_infos.size(), 0);
    done.assign(kernel_infos.size(), 0);
    int cursor = 0;
    CUDA_RETURN_STATUS(gp_program_read_state(program_, executed.data(), done.data(), &cursor, &error));
    return Status::Succ;
}

double Model::total_flops() const {
    double f = 0;
    for (const KernelInfo &k : kernel_infos) f += k.flops;
    return f;
}
double Model::total_bytes() const {
    double b = 0;
    for (const KernelInfo &k : kernel_infos) b += k.bytes;
    return b;
}

}  // namespace foo
