// Native graph builders: the model set the reference exports through TVM
// (scripts/compile/compile.py:28-44: resnet, vgg, densenet, inception; compile-bert.py) rebuilt
// as kernel lists over the operators of libgpreempt_hip.so, at the shapes the benchmark
// configurations name.  Activations are NHWC with 16-byte aligned channel counts; parameters are
// declared in the reference's on-disk convention (fp32, OIHW) and re-laid-out at load time.
#include "zoo.h"
#include "graph_builder.h"
#include "workloads/scicomput.h"

#include <cmath>
#include <cstring>
#include <map>
#include <memory>
#include <sstream>

namespace foo {

namespace {

// ---- option parsing: "name@key=value,key=value" ------------------------------------------------
struct Options {
    std::string name;
    std::map<std::string, std::string> kv;
    int geti(const std::string &k, int d) const { auto it = kv.find(k); return it == kv.end() ? d : std::atoi(it->second.c_str()); }
    std::string gets(const std::string &k, const std::string &d) const { auto it = kv.find(k); return it == kv.end() ? d : it->second; }
};

Options parse(const std::string &workload) {
    Options o;
    size_t at = workload.find('@');
    o.name = workload.substr(0, at);
    if (at != std::string::npos) {
        std::stringstream ss(workload.substr(at + 1));
        std::string item;
        while (std::getline(ss, item, ',')) {
            size_t eq = item.find('=');
            if (eq != std::string::npos) o.kv[item.substr(0, eq)] = item.substr(eq + 1);
        }
    }
    return o;
}

bool valid_dtype(const std::string &d) { return d == "f32" || d == "f16" || d == "bf16"; }

// ---- config 1 / config 5: C = act(A * B + bias) as a one-kernel model --------------------------
// storages: "data" = A (M x K), "B" (K x N, or N x K with layout=nk), "bias" (N), "heads" = C.
// B is a parameter: whatever its layout on disk, the device copy is N x K (K-contiguous rows feed
// the direct-to-LDS loads), as convolution weights are re-laid out at load time.
Status build_gemm(Model &m, const Options &o, int M, int N, int K, const std::string &dt_default, int act_default) {
    std::string dt = o.gets("dtype", dt_default);
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    M = o.geti("m", M); N = o.geti("n", N); K = o.geti("k", K);
    bool nk = o.gets("layout", "kn") == "nk";
    int act = o.geti("act", act_default);
    int tile = o.geti("tile", 0);
    size_t a = g.add_storage("data", (size_t)M * K, g.stype_);
    ParamLayout LB; LB.disk_elems = (size_t)K * N; LB.init = ParamLayout::InitUniform; LB.init_a = -1.f; LB.init_b = 1.f;
    if (!nk) { LB.kind = ParamLayout::MatKN; LB.i = K; LB.o = N; }
    size_t b = g.add_param("B", (size_t)K * N, LB);
    ParamLayout Lb; Lb.disk_elems = N; Lb.init = ParamLayout::InitUniform; Lb.init_a = -0.1f; Lb.init_b = 0.1f;
    size_t bias = g.add_param("bias", N, Lb);
    size_t c = g.add_storage("heads", (size_t)M * N, g.stype_);
    bool use_bias = o.geti("bias", 1) != 0;
    double flops = 2.0 * M * N * (double)K + (use_bias ? 2.0 * M * N : 0);
    double bytes = g.es() * ((double)M * K + (double)K * N + (use_bias ? N : 0) + (double)M * N);
    KernelInfo &k = g.add_kernel("gemm", OpKind::Gemm, {GraphBuilder::ref(a), GraphBuilder::ref(b), use_bias ? GraphBuilder::ref(bias) : GraphBuilder::none(), GraphBuilder::none(), GraphBuilder::ref(c)}, flops, bytes);
    gp_gemm_params &p = k.p.gemm;
    p.dtype = g.gp_dtype(); p.M = M; p.N = N; p.K = K; p.lda = K; p.ldb = K; p.b_is_nk = 1; p.ldc = N; p.alpha = 1.f; p.act = act; p.batch = 1;
    p.tile_m = p.tile_n = tile;
    return Status::Succ;
}

// ---- Inception-v3 ------------------------------------------------------------------------------
// The architecture of relay.testing.inception_v3 (the reference's "inception" model,
// scripts/compile/compile.py:36-38): 299x299 input, a five-convolution stem, three A blocks
// (35x35), a reducing B block, four C blocks (17x17, factorised 7x7), a reducing D block, two E
// blocks (8x8), global average pool, FC 1000, softmax.  Every convolution carries a folded
// batch-norm and a ReLU.  Branch outputs are written straight into their channel slice of the
// block's output (no concatenation kernel); average pools count the padding, as relay's do.
Status build_inception_v3(Model &m, const Options &o) {
    std::string dt = o.gets("dtype", "f16");
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    const int N = o.geti("b", 1), HW = o.geti("hw", 299), classes = o.geti("classes", 1000);
    if (HW < 75) return Status::OutOfRange;  // below that the 8x8 stage has no pixel left
    auto cv = [&](const std::string &n, const Tensor &in, int cout, int kh, int kw, int stride, int ph, int pw, const Tensor *into = nullptr) {
        return g.conv_hw(n, in, cout, kh, kw, stride, ph, pw, GP_ACT_RELU, nullptr, into);
    };
    auto out_size = [](int h, int k, int s, int p) { return (h + 2 * p - k) / s + 1; };
    Tensor x = g.input_nchw(N, 3, HW, HW);
    x = g.conv_hw("conv", x, 32, 3, 3, 2, 0, 0, GP_ACT_RELU, nullptr, nullptr, 3);
    x = cv("conv_1", x, 32, 3, 3, 1, 0, 0);
    x = cv("conv_2", x, 64, 3, 3, 1, 1, 1);
    x = g.pool("pool", x, 3, 2, 0, 0);
    x = cv("conv_3", x, 80, 1, 1, 1, 0, 0);
    x = cv("conv_4", x, 192, 3, 3, 1, 0, 0);
    x = g.pool("pool1", x, 3, 2, 0, 0);
    int idx = 0;
    auto block_name = [&]() { return "mixed" + std::to_string(idx++); };
    // A: 1x1 | 1x1 -> 5x5 | 1x1 -> 3x3 -> 3x3 | avgpool -> 1x1
    for (int proj : {32, 64, 64}) {
        const std::string n = block_name();
        Tensor out = g.activation(n + ".out", N, x.H, x.W, 64 + 64 + 96 + proj);
        Tensor s0 = GraphBuilder::slice(out, 0, 64), s1 = GraphBuilder::slice(out, 64, 64), s2 = GraphBuilder::slice(out, 128, 96), s3 = GraphBuilder::slice(out, 224, proj);
        cv(n + ".1x1", x, 64, 1, 1, 1, 0, 0, &s0);
        Tensor t = cv(n + ".5x5_r", x, 48, 1, 1, 1, 0, 0);
        cv(n + ".5x5", t, 64, 5, 5, 1, 2, 2, &s1);
        t = cv(n + ".3x3_r", x, 64, 1, 1, 1, 0, 0);
        t = cv(n + ".3x3_1", t, 96, 3, 3, 1, 1, 1);
        cv(n + ".3x3_2", t, 96, 3, 3, 1, 1, 1, &s2);
        t = g.pool(n + ".pool", x, 3, 1, 1, 3);
        cv(n + ".proj", t, proj, 1, 1, 1, 0, 0, &s3);
        x = out;
    }
    {   // B: 3x3/2 | 1x1 -> 3x3 -> 3x3/2 | maxpool/2
        const std::string n = block_name();
        const int H = out_size(x.H, 3, 2, 0);
        Tensor out = g.activation(n + ".out", N, H, H, 384 + 96 + x.C);
        Tensor s0 = GraphBuilder::slice(out, 0, 384), s1 = GraphBuilder::slice(out, 384, 96), s2 = GraphBuilder::slice(out, 480, x.C);
        cv(n + ".3x3", x, 384, 3, 3, 2, 0, 0, &s0);
        Tensor t = cv(n + ".d3x3_r", x, 64, 1, 1, 1, 0, 0);
        t = cv(n + ".d3x3_1", t, 96, 3, 3, 1, 1, 1);
        cv(n + ".d3x3_2", t, 96, 3, 3, 2, 0, 0, &s1);
        g.pool(n + ".pool", x, 3, 2, 0, 0, &s2);
        x = out;
    }
    // C: 1x1 | 1x1 -> 1x7 -> 7x1 | 1x1 -> 7x1 -> 1x7 -> 7x1 -> 1x7 | avgpool -> 1x1
    for (int c7 : {128, 160, 160, 192}) {
        const std::string n = block_name();
        Tensor out = g.activation(n + ".out", N, x.H, x.W, 192 * 4);
        Tensor s0 = GraphBuilder::slice(out, 0, 192), s1 = GraphBuilder::slice(out, 192, 192), s2 = GraphBuilder::slice(out, 384, 192), s3 = GraphBuilder::slice(out, 576, 192);
        cv(n + ".1x1", x, 192, 1, 1, 1, 0, 0, &s0);
        Tensor t = cv(n + ".7_r", x, c7, 1, 1, 1, 0, 0);
        t = cv(n + ".7_1", t, c7, 1, 7, 1, 0, 3);
        cv(n + ".7_2", t, 192, 7, 1, 1, 3, 0, &s1);
        t = cv(n + ".d7_r", x, c7, 1, 1, 1, 0, 0);
        t = cv(n + ".d7_1", t, c7, 7, 1, 1, 3, 0);
        t = cv(n + ".d7_2", t, c7, 1, 7, 1, 0, 3);
        t = cv(n + ".d7_3", t, c7, 7, 1, 1, 3, 0);
        cv(n + ".d7_4", t, 192, 1, 7, 1, 0, 3, &s2);
        t = g.pool(n + ".pool", x, 3, 1, 1, 3);
        cv(n + ".proj", t, 192, 1, 1, 1, 0, 0, &s3);
        x = out;
    }
    {   // D: 1x1 -> 3x3/2 | 1x1 -> 1x7 -> 7x1 -> 3x3/2 | maxpool/2
        const std::string n = block_name();
        const int H = out_size(x.H, 3, 2, 0);
        Tensor out = g.activation(n + ".out", N, H, H, 320 + 192 + x.C);
        Tensor s0 = GraphBuilder::slice(out, 0, 320), s1 = GraphBuilder::slice(out, 320, 192), s2 = GraphBuilder::slice(out, 512, x.C);
        Tensor t = cv(n + ".3x3_r", x, 192, 1, 1, 1, 0, 0);
        cv(n + ".3x3", t, 320, 3, 3, 2, 0, 0, &s0);
        t = cv(n + ".7x3_r", x, 192, 1, 1, 1, 0, 0);
        t = cv(n + ".7x3_1", t, 192, 1, 7, 1, 0, 3);
        t = cv(n + ".7x3_2", t, 192, 7, 1, 1, 3, 0);
        cv(n + ".7x3_3", t, 192, 3, 3, 2, 0, 0, &s1);
        g.pool(n + ".pool", x, 3, 2, 0, 0, &s2);
        x = out;
    }
    // E: 1x1 | 1x1 -> {1x3, 3x1} | 1x1 -> 3x3 -> {1x3, 3x1} | pool -> 1x1 (average, then max)
    for (int pool_mode : {3, 0}) {
        const std::string n = block_name();
        Tensor out = g.activation(n + ".out", N, x.H, x.W, 320 + 768 + 768 + 192);
        Tensor s0 = GraphBuilder::slice(out, 0, 320), s1a = GraphBuilder::slice(out, 320, 384), s1b = GraphBuilder::slice(out, 704, 384);
        Tensor s2a = GraphBuilder::slice(out, 1088, 384), s2b = GraphBuilder::slice(out, 1472, 384), s3 = GraphBuilder::slice(out, 1856, 192);
        cv(n + ".1x1", x, 320, 1, 1, 1, 0, 0, &s0);
        Tensor t = cv(n + ".3_r", x, 384, 1, 1, 1, 0, 0);
        cv(n + ".3_a", t, 384, 1, 3, 1, 0, 1, &s1a);
        cv(n + ".3_b", t, 384, 3, 1, 1, 1, 0, &s1b);
        t = cv(n + ".d3_r", x, 448, 1, 1, 1, 0, 0);
        t = cv(n + ".d3_1", t, 384, 3, 3, 1, 1, 1);
        cv(n + ".d3_a", t, 384, 1, 3, 1, 0, 1, &s2a);
        cv(n + ".d3_b", t, 384, 3, 1, 1, 1, 0, &s2b);
        t = g.pool(n + ".pool", x, 3, 1, 1, pool_mode);
        cv(n + ".proj", t, 192, 1, 1, 1, 0, 0, &s3);
        x = out;
    }
    Tensor gap = g.pool("global_pool", x, 0, 1, 0, 2);
    size_t logits = g.add_storage("fc1.out", (size_t)N * classes, g.stype_);
    g.dense("fc1", gap.st, 0, N, gap.C, gap.C, classes, GP_ACT_NONE, SIZE_MAX, logits, 0, classes, 0.01f);
    size_t heads = g.add_storage("heads", (size_t)N * classes, g.stype_);
    g.softmax(logits, heads, N, classes, 1.f);
    return Status::Succ;
}

// ---- miniWeather ---------------------------------------------------------------------------------
// One perform_timestep of the reference (src/workloads/miniweather.tr.cu:184-206) as a kernel list:
// four direction sweeps (x, z, z, x), three Runge-Kutta stages each, three kernels per stage (halo
// exchange, interface fluxes, state update) = 36 kernels, so the stop index of a preempted step is
// the reference's `start_from` (= stage * 3 + kernel).  The state lives in the model's storages
// and advances by two time steps of `dt` per execute().
Status build_miniweather(Model &m, const Options &o) {
    GraphBuilder g(m, "f32");
    const int nx = o.geti("nx", 3200), nz = o.geti("nz", 1600), spec = o.geti("spec", SciCompute::Collision);
    if (nx < 4 || nz < 4 || (long)nx * nz > (1L << 27)) return Status::OutOfRange;
    if (spec != 1 && spec != 2 && spec != 3 && spec != 5 && spec != 6) return Status::OutOfRange;
    const SciCompute::Grid grid = SciCompute::make_grid(nx, nz);
    auto state0 = std::make_shared<std::vector<float>>();
    auto hydro0 = std::make_shared<std::vector<float>>();
    SciCompute::initial_state(grid, spec, *state0, *hydro0);
    ParamLayout LS; LS.disk_elems = state0->size(); LS.init = ParamLayout::InitData; LS.init_data = state0;
    ParamLayout LH; LH.disk_elems = hydro0->size(); LH.init = ParamLayout::InitData; LH.init_data = hydro0;
    const size_t state = g.add_param("state", state0->size(), LS);
    const size_t state_tmp = g.add_param("state_tmp", state0->size(), LS);
    const size_t hydro = g.add_param("hydro", hydro0->size(), LH);
    const size_t flux = g.add_storage("flux", SciCompute::flux_elems(grid), "float32");
    static const char *names[6] = {"set_halo_values_x", "compute_tendencies_x", "compute_tendencies_x_r",
                                   "set_halo_values_z", "compute_tendencies_z", "compute_tendencies_z_r"};
    const double cells = (double)nx * nz;
    for (int kid = 0; kid < 36; ++kid) {
        const int step = kid / 3, sub = kid % 3, sweep = step / 3, stage = step % 3;
        const bool dir_z = sweep == 1 || sweep == 2;
        const size_t forcing = stage == 0 ? state : state_tmp, out = stage == 2 ? state : state_tmp;
        const int kernel = (dir_z ? 3 : 0) + sub;
        // algorithmic traffic: fluxes read the 4 state fields and write 4 flux fields; updates read
        // 4 flux fields and 4 state fields (+ density for gravity) and write 4 state fields
        double bytes = 0, flops = 0;
        if (sub == 0) bytes = 4.0 * 4 * 4 * 2 * (dir_z ? nx + 4 : nz);
        else if (sub == 1) { bytes = 4.0 * 8 * cells; flops = 60 * cells; }
        else { bytes = 4.0 * (12 + (dir_z ? 1 : 0)) * cells; flops = 4 * 4 * cells; }
        KernelInfo &k = g.add_kernel(names[kernel], OpKind::Stencil,
                                     {GraphBuilder::ref(forcing), GraphBuilder::ref(flux), GraphBuilder::ref(state), GraphBuilder::ref(out), GraphBuilder::ref(hydro)},
                                     flops, bytes);
        gp_miniweather_params &p = k.p.miniweather;
        p.kernel = kernel; p.nx = nx; p.nz = nz;
        p.dt = stage == 0 ? grid.dt / 3 : stage == 1 ? grid.dt / 2 : grid.dt / 1;
        p.dx = grid.dx; p.dz = grid.dz;
    }
    return Status::Succ;
}

// ---- ResNet v1 with bottleneck blocks ----------------------------------------------------------
// conv7x7/2-64 -> maxpool3x3/2 -> stages of [1x1, 3x3, 1x1(+shortcut)] -> global average pool ->
// FC 1000 -> softmax.  Batch-norm is folded into each convolution's weight and bias.  The stride
// of a down-sampling block sits on its first 1x1 convolution (the original "v1" placement) and
// on the 1x1 projection shortcut.
Status build_resnet(Model &m, const Options &o, const int (&blocks)[4], int batch_default, const std::string &dt_default) {
    std::string dt = o.gets("dtype", dt_default);
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    int N = o.geti("b", batch_default), HW = o.geti("hw", 224), classes = o.geti("classes", 1000);
    int base = o.geti("width", 64);
    Tensor x = g.input_nchw(N, 3, HW, HW);
    x = g.conv("conv1", x, base, 7, 2, 3, GP_ACT_RELU, nullptr, nullptr, 3);
    x = g.pool("pool1", x, 3, 2, 1, 0);
    for (int s = 0; s < 4; ++s) {
        int width = base << s;
        for (int b = 0; b < blocks[s]; ++b) {
            std::string n = "layer" + std::to_string(s + 1) + "." + std::to_string(b);
            int stride = (b == 0 && s > 0) ? 2 : 1;
            Tensor shortcut = x;
            if (b == 0) shortcut = g.conv(n + ".downsample", x, width * 4, 1, stride, 0, GP_ACT_NONE);
            Tensor y = g.conv(n + ".conv1", x, width, 1, stride, 0, GP_ACT_RELU);
            y = g.conv(n + ".conv2", y, width, 3, 1, 1, GP_ACT_RELU);
            // The block's last convolution starts small (a folded batch-norm with a small gamma):
            // without it 50 un-normalised residual additions overflow fp16.
            x = g.conv(n + ".conv3", y, width * 4, 1, 1, 0, GP_ACT_RELU, &shortcut, nullptr, -1, 0.2f);
        }
    }
    Tensor gap = g.pool("avgpool", x, 0, 1, 0, 2);
    size_t logits = g.add_storage("fc.out", (size_t)N * classes, g.stype_);
    g.dense("fc", gap.st, 0, N, gap.C, gap.C, classes, GP_ACT_NONE, SIZE_MAX, logits, 0, classes, 0.01f);
    size_t heads = g.add_storage("heads", (size_t)N * classes, g.stype_);
    g.softmax(logits, heads, N, classes, 1.f);
    return Status::Succ;
}

// ---- VGG-16 -----------------------------------------------------------------------------------
Status build_vgg16(Model &m, const Options &o) {
    std::string dt = o.gets("dtype", "f16");
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    int N = o.geti("b", 16), HW = o.geti("hw", 224), classes = o.geti("classes", 1000), fc = o.geti("fc", 4096);
    int div = o.geti("wdiv", 1);
    const int cfg[] = {64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512, -1};
    Tensor x = g.input_nchw(N, 3, HW, HW);
    int ci = 0, pi = 0;
    bool first = true;
    for (int c : cfg) {
        if (c < 0) x = g.pool("pool" + std::to_string(++pi), x, 2, 2, 0, 0);
        else {
            x = g.conv("conv" + std::to_string(++ci), x, c / div, 3, 1, 1, GP_ACT_RELU, nullptr, nullptr, first ? 3 : -1);
            first = false;
        }
    }
    // flatten is a view (the reference copies through a "__nop" kernel, src/model.cpp:201-207);
    // fc1's weight is declared over the NCHW flatten and permuted to NHWC order at load time.
    int feat = x.H * x.W * x.C;
    ParamLayout L; L.kind = ParamLayout::DenseOverCHW; L.c = x.C; L.h = x.H; L.w = x.W;
    size_t h1 = g.add_storage("fc1.out", (size_t)N * fc, g.stype_);
    g.dense("fc1", x.st, 0, N, feat, feat, fc, GP_ACT_RELU, SIZE_MAX, h1, 0, fc, std::sqrt(2.f / feat), &L);
    size_t h2 = g.add_storage("fc2.out", (size_t)N * fc, g.stype_);
    g.dense("fc2", h1, 0, N, fc, fc, fc, GP_ACT_RELU, SIZE_MAX, h2, 0, fc, std::sqrt(2.f / fc));
    size_t logits = g.add_storage("fc3.out", (size_t)N * classes, g.stype_);
    g.dense("fc3", h2, 0, N, fc, fc, classes, GP_ACT_NONE, SIZE_MAX, logits, 0, classes, 0.01f);
    size_t heads = g.add_storage("heads", (size_t)N * classes, g.stype_);
    g.softmax(logits, heads, N, classes, 1.f);
    return Status::Succ;
}

// ---- DenseNet-201 -----------------------------------------------------------------------------
// conv7x7/2 -> maxpool -> dense blocks [6,12,48,32] with growth 32 and 1x1 bottlenecks of 128,
// transitions halve channels and average-pool 2x2.  Batch-norm precedes each convolution here,
// so only the norm that FOLLOWS a convolution (stem, bottleneck 1x1) folds into it; the others
// run as per-channel scale-shift-ReLU kernels.  A dense block is one NHWC buffer as wide as its
// final channel count: every layer writes its 32 new channels into its slice of that buffer,
// which is concatenation without a copy.
Status build_densenet201(Model &m, const Options &o) {
    std::string dt = o.gets("dtype", "f16");
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    int N = o.geti("b", 4), HW = o.geti("hw", 224), classes = o.geti("classes", 1000);
    int growth = o.geti("growth", 32), init_c = o.geti("init", 64), bn_size = 4;
    int blocks[4] = {o.geti("l1", 6), o.geti("l2", 12), o.geti("l3", 48), o.geti("l4", 32)};
    Tensor x = g.input_nchw(N, 3, HW, HW);
    x = g.conv("conv0", x, init_c, 7, 2, 3, GP_ACT_RELU, nullptr, nullptr, 3);  // + norm0 folded + relu
    int C = init_c;
    int H = (x.H + 2 - 3) / 2 + 1;
    Tensor buf = g.activation("block1.buf", N, H, H, C + blocks[0] * growth);
    Tensor first = GraphBuilder::slice(buf, 0, C);
    g.pool("pool0", x, 3, 2, 1, 0, &first);
    for (int b = 0; b < 4; ++b) {
        std::string bn = "block" + std::to_string(b + 1);
        for (int l = 0; l < blocks[b]; ++l) {
            std::string n = bn + ".layer" + std::to_string(l + 1);
            Tensor in = GraphBuilder::slice(buf, 0, C);
            Tensor t = g.eltwise(n + ".norm1", in, nullptr, n + ".norm1", GP_ACT_RELU);
            t = g.conv(n + ".conv1", t, bn_size * growth, 1, 1, 0, GP_ACT_RELU);          // + norm2 folded + relu
            Tensor dst = GraphBuilder::slice(buf, C, growth);
            g.conv(n + ".conv2", t, growth, 3, 1, 1, GP_ACT_NONE, nullptr, &dst);
            C += growth;
        }
        if (b < 3) {
            std::string n = "transition" + std::to_string(b + 1);
            if ((C / 2) % g.vec() != 0) return Status::OutOfRange;  // halved channel count must stay 16-byte aligned
            Tensor t = g.eltwise(n + ".norm", buf, nullptr, n + ".norm", GP_ACT_RELU);
            t = g.conv(n + ".conv", t, C / 2, 1, 1, 0, GP_ACT_NONE);
            C /= 2;
            Tensor next = g.activation("block" + std::to_string(b + 2) + ".buf", N, t.H / 2, t.W / 2, C + blocks[b + 1] * growth);
            Tensor dst = GraphBuilder::slice(next, 0, C);
            g.pool(n + ".pool", t, 2, 2, 0, 1, &dst);
            buf = next;
        }
    }
    Tensor t = g.eltwise("norm5", buf, nullptr, "norm5", GP_ACT_RELU);
    Tensor gap = g.pool("avgpool", t, 0, 1, 0, 2);
    size_t logits = g.add_storage("classifier.out", (size_t)N * classes, g.stype_);
    g.dense("classifier", gap.st, 0, N, gap.C, gap.C, classes, GP_ACT_NONE, SIZE_MAX, logits, 0, classes, 0.01f);
    size_t heads = g.add_storage("heads", (size_t)N * classes, g.stype_);
    g.softmax(logits, heads, N, classes, 1.f);
    return Status::Succ;
}

// ---- BERT encoder -----------------------------------------------------------------------------
// token + position + segment-0 embedding -> LayerNorm -> L x { fused QKV dense, per-head
// softmax(Q K^T / sqrt(d)) V (one fused kernel for 16-bit models, else two batched GEMMs over head
// slices of the QKV buffer around a softmax), output
// dense + residual, LayerNorm, FFN dense + erf-GELU, dense + residual, LayerNorm }; eps 1e-12.
// "data" holds int64 token ids (reference src/tests/test-dnn.cpp:21-23); "heads" is the last
// hidden state [batch*seq, hidden].
Status build_bert(Model &m, const Options &o) {
    std::string dt = o.gets("dtype", "f16");
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    int B = o.geti("b", 1), S = o.geti("s", 128), L = o.geti("layers", 12), Hd = o.geti("hidden", 768);
    int heads = o.geti("heads", 12), F = o.geti("ffn", 3072), vocab = o.geti("vocab", 30522), maxpos = o.geti("maxpos", 512);
    if (Hd % heads || S > maxpos) return Status::OutOfRange;
    int d = Hd / heads;
    // 16-bit models with 64-wide heads use the fused attention kernel ("fused_attention=0" keeps
    // the exported graph's batch_matmul / softmax / batch_matmul sequence)
    const bool fused = o.geti("fused_attention", 1) != 0 && dt != "f32" && d == 64 && S <= 512;
    long T = (long)B * S;
    const float std_ = 0.02f;
    size_t es = g.es();
    auto table = [&](const std::string &name, size_t rows) {
        ParamLayout P; P.o = (int)rows; P.disk_elems = rows * Hd; P.init = ParamLayout::InitNormal; P.init_a = std_;
        return g.add_param(name, rows * Hd, P);
    };
    auto ln_params = [&](const std::string &name, size_t &gamma, size_t &beta) {
        ParamLayout G; G.disk_elems = Hd; G.init = ParamLayout::InitConst; G.init_a = 1.f;
        gamma = g.add_param(name + ".gamma", Hd, G);
        ParamLayout Bt; Bt.disk_elems = Hd; Bt.init = ParamLayout::InitZero;
        beta = g.add_param(name + ".beta", Hd, Bt);
    };
    auto layernorm = [&](const std::string &name, size_t x, size_t res, size_t out) {
        size_t ga, be;
        ln_params(name, ga, be);
        double e = (double)T * Hd;
        KernelInfo &k = g.add_kernel("layernorm", OpKind::Layernorm, {GraphBuilder::ref(x), res == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(res), GraphBuilder::ref(ga), GraphBuilder::ref(be), GraphBuilder::ref(out)},
                                     8 * e, es * e * (res == SIZE_MAX ? 2 : 3));
        gp_layernorm_params &p = k.p.layernorm;
        p.dtype = g.gp_dtype(); p.rows = T; p.cols = Hd; p.eps = 1e-12f;
    };

    size_t ids = g.add_storage("data", (size_t)T, "int64");
    size_t tok = table("embeddings.word", vocab), pos = table("embeddings.position", maxpos), seg = table("embeddings.token_type", 1);
    size_t emb = g.add_storage("embeddings.sum", (size_t)T * Hd, g.stype_);
    {
        KernelInfo &k = g.add_kernel("embed", OpKind::Embed, {GraphBuilder::ref(ids), GraphBuilder::ref(tok), GraphBuilder::ref(pos), GraphBuilder::ref(seg), GraphBuilder::ref(emb)},
                                     2.0 * T * Hd, 8.0 * T + es * 4.0 * T * Hd);
        gp_embed_params &p = k.p.embed;
        p.dtype = g.gp_dtype(); p.tokens = T; p.seq = S; p.hidden = Hd; p.vocab = vocab;
    }
    size_t x = g.add_storage("embeddings.out", (size_t)T * Hd, g.stype_);
    layernorm("embeddings.ln", emb, SIZE_MAX, x);

    for (int l = 0; l < L; ++l) {
        std::string n = "layer" + std::to_string(l);
        size_t qkv = g.add_storage(n + ".qkv", (size_t)T * 3 * Hd, g.stype_);
        g.dense(n + ".attn.qkv", x, 0, T, Hd, Hd, 3 * Hd, GP_ACT_NONE, SIZE_MAX, qkv, 0, 3 * Hd, std_);
        size_t ctx = g.add_storage(n + ".context", (size_t)T * Hd, g.stype_);
        if (fused) {
            // one kernel: softmax(Q K^T / sqrt(d)) V per head, scores never leave the chip
            double flops = 4.0 * B * heads * (double)S * S * d;
            KernelInfo &k = g.add_kernel("attention", OpKind::Attention, {GraphBuilder::ref(qkv, 0), GraphBuilder::ref(qkv, (size_t)Hd * es), GraphBuilder::ref(qkv, (size_t)2 * Hd * es), GraphBuilder::ref(ctx)},
                                         flops, es * 4.0 * T * Hd);
            gp_attention_params &p = k.p.attention;
            p.dtype = g.gp_dtype(); p.batch = B; p.heads = heads; p.seq = S; p.head_dim = d;
            p.ld_qkv = 3 * Hd; p.ld_out = Hd; p.scale = 1.f / std::sqrt((float)d);
        } else {
            size_t sc = g.add_storage(n + ".scores", (size_t)B * heads * S * S, g.stype_);
            {   // scores[b,h] = Q[b,h] K[b,h]^T / sqrt(d)
                double flops = 2.0 * B * heads * (double)S * S * d;
                KernelInfo &k = g.add_kernel("batch_matmul_qk", OpKind::Gemm, {GraphBuilder::ref(qkv, 0), GraphBuilder::ref(qkv, (size_t)Hd * es), GraphBuilder::none(), GraphBuilder::none(), GraphBuilder::ref(sc)},
                                             flops, es * (2.0 * T * Hd + (double)B * heads * S * S));
                gp_gemm_params &p = k.p.gemm;
                p.dtype = g.gp_dtype(); p.M = S; p.N = S; p.K = d; p.lda = 3 * Hd; p.ldb = 3 * Hd; p.b_is_nk = 1; p.ldc = S;
                p.alpha = 1.f / std::sqrt((float)d); p.act = GP_ACT_NONE; p.batch = B * heads; p.batch_inner = heads;
                p.stride_a = d; p.stride_b = d; p.stride_c = (long)S * S;
                p.stride_a_outer = (long)S * 3 * Hd; p.stride_b_outer = (long)S * 3 * Hd; p.stride_c_outer = (long)heads * S * S;
            }
            size_t pr = g.add_storage(n + ".probs", (size_t)B * heads * S * S, g.stype_);
            g.softmax(sc, pr, (long)B * heads * S, S, 1.f);
            {   // context[b,:,h] = probs[b,h] V[b,h]
                double flops = 2.0 * B * heads * (double)S * S * d;
                KernelInfo &k = g.add_kernel("batch_matmul_pv", OpKind::Gemm, {GraphBuilder::ref(pr), GraphBuilder::ref(qkv, (size_t)2 * Hd * es), GraphBuilder::none(), GraphBuilder::none(), GraphBuilder::ref(ctx)},
                                             flops, es * ((double)B * heads * S * S + 2.0 * T * Hd));
                gp_gemm_params &p = k.p.gemm;
                p.dtype = g.gp_dtype(); p.M = S; p.N = d; p.K = S; p.lda = S; p.ldb = 3 * Hd; p.b_is_nk = 0; p.ldc = Hd;
                p.alpha = 1.f; p.act = GP_ACT_NONE; p.batch = B * heads; p.batch_inner = heads;
                p.stride_a = (long)S * S; p.stride_b = d; p.stride_c = d;
                p.stride_a_outer = (long)heads * S * S; p.stride_b_outer = (long)S * 3 * Hd; p.stride_c_outer = (long)S * Hd;
            }
        }
        size_t ao = g.add_storage(n + ".attn.out", (size_t)T * Hd, g.stype_);
        g.dense(n + ".attn.proj", ctx, 0, T, Hd, Hd, Hd, GP_ACT_NONE, x, ao, 0, Hd, std_);   // + residual x
        size_t x1 = g.add_storage(n + ".ln1.out", (size_t)T * Hd, g.stype_);
        layernorm(n + ".ln1", ao, SIZE_MAX, x1);
        size_t f1 = g.add_storage(n + ".ffn1.out", (size_t)T * F, g.stype_);
        g.dense(n + ".ffn1", x1, 0, T, Hd, Hd, F, GP_ACT_GELU, SIZE_MAX, f1, 0, F, std_);
        size_t f2 = g.add_storage(n + ".ffn2.out", (size_t)T * Hd, g.stype_);
        g.dense(n + ".ffn2", f1, 0, T, F, F, Hd, GP_ACT_NONE, x1, f2, 0, Hd, std_);          // + residual x1
        size_t x2 = g.add_storage(l == L - 1 ? std::string("heads") : n + ".ln2.out", (size_t)T * Hd, g.stype_);
        layernorm(n + ".ln2", f2, SIZE_MAX, x2);
        x = x2;
    }
    return Status::Succ;
}

// ---- a tiny chain with a "nop" copy, used to test the executor plumbing ------------------------
Status build_toy(Model &m, const Options &o) {
    std::string dt = o.gets("dtype", "f32");
    if (!valid_dtype(dt)) return Status::OutOfRange;
    GraphBuilder g(m, dt);
    int rows = o.geti("rows", 64), cols = o.geti("cols", 64), n = o.geti("n", 3);
    size_t cur = g.add_storage("data", (size_t)rows * cols, g.stype_);
    for (int i = 0; i < n; ++i) {
        Tensor a; a.st = cur; a.N = 1; a.H = 1; a.W = rows; a.C = cols; a.ps = cols;
        Tensor t = g.eltwise("scale" + std::to_string(i), a, &a, "", GP_ACT_NONE);  // x -> 2x
        size_t copy = g.add_storage(i == n - 1 ? std::string("heads") : "copy" + std::to_string(i), (size_t)rows * cols, g.stype_);
        KernelInfo &k = g.add_kernel("nop", OpKind::Nop, {GraphBuilder::ref(t.st), GraphBuilder::ref(copy)}, 0, 2.0 * g.es() * rows * cols);
        (void)k;
        cur = copy;
    }
    return Status::Succ;
}

}  // namespace

Status zoo_build(Model &m, const std::string &workload) {
    Options o = parse(workload);
    const std::string &n = o.name;
    static const int r50[4] = {3, 4, 6, 3}, r101[4] = {3, 4, 23, 3}, r152[4] = {3, 8, 36, 3};
    if (n == "gemm" || n == "gemm1024") return build_gemm(m, o, 1024, 1024, 1024, "f32", GP_ACT_RELU);
    if (n == "gemm8192") { Options q = o; if (!q.kv.count("layout")) q.kv["layout"] = "nk"; if (!q.kv.count("bias")) q.kv["bias"] = "0"; return build_gemm(m, q, 8192, 8192, 8192, "bf16", GP_ACT_NONE); }
    if (n == "resnet50") return build_resnet(m, o, r50, 1, "f32");
    if (n == "resnet101") return build_resnet(m, o, r101, 1, "f16");
    if (n == "resnet152" || n == "resnet") return build_resnet(m, o, r152, 8, "f16");
    if (n == "vgg" || n == "vgg16") return build_vgg16(m, o);
    if (n == "densenet" || n == "densenet201") return build_densenet201(m, o);
    if (n == "inception" || n == "inception_v3") return build_inception_v3(m, o);
    if (n == "bert") return build_bert(m, o);
    if (n == "toy") return build_toy(m, o);
    if (n == "miniweather") return build_miniweather(m, o);
    std::fprintf(stderr, "unknown workload '%s' (known: gemm1024 gemm8192 resnet50 resnet101 resnet152 vgg16 densenet201 inception bert miniweather toy; graph workloads: cc bfs pagerank sssp)\n", n.c_str());
    return Status::NotFound;
}

}  // namespace foo
