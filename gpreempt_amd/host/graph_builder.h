// GraphBuilder: appends storages and kernels of the native operators to a foo::Model.  Used by the
// built-in model builders and by the loader of exported models.
#pragma once
#include <cmath>
#include <cstring>
#include <string>
#include <vector>
#include "model.h"

namespace foo {

struct Tensor {            // NHWC view into a storage
    size_t st = SIZE_MAX;
    size_t off = 0;        // element offset of channel 0 of pixel 0
    int N = 0, H = 0, W = 0, C = 0;
    long ps = 0;           // pixel stride in elements
};

class GraphBuilder {
public:
    GraphBuilder(Model &m, const std::string &dt) : m_(m), dt_(dt) {
        if (dt == "f32") { stype_ = "float32"; gp_dt_ = GP_F32; es_ = 4; vec_ = 4; }
        else if (dt == "f16") { stype_ = "float16"; gp_dt_ = GP_F16; es_ = 2; vec_ = 8; }
        else { stype_ = "bfloat16"; gp_dt_ = GP_BF16; es_ = 2; vec_ = 8; }
        m_.dtype_ = dt;
    }
    int vec() const { return vec_; }
    int gp_dtype() const { return gp_dt_; }
    size_t es() const { return es_; }
    int pad_c(int c) const { return (c + vec_ - 1) / vec_ * vec_; }

    size_t add_storage(const std::string &name, size_t elems, const std::string &stype, const ParamLayout &L = ParamLayout()) {
        StorageInfo info;
        info.name = name; info.stype = stype;
        std::string st = stype;
        info.size = elems * Model::get_stype_size(st);
        m_.storage_infos.push_back(info);
        m_.layouts.push_back(L);
        return m_.storage_infos.size() - 1;
    }
    size_t add_param(const std::string &name, size_t dev_elems, ParamLayout L) {
        L.is_param = true;
        return add_storage(name, dev_elems, stype_, L);
    }
    const std::string &storage_name(size_t st) const { return m_.storage_infos[st].name; }
    void rename_storage(size_t st, const std::string &name) { m_.storage_infos[st].name = name; }
    const ParamLayout &param_layout(size_t st) const { return m_.layouts[st]; }
    Tensor activation(const std::string &name, int N, int H, int W, int C) {
        Tensor t;
        t.st = add_storage(name, (size_t)N * H * W * C, stype_);
        t.N = N; t.H = H; t.W = W; t.C = C; t.ps = C;
        return t;
    }
    static Tensor slice(const Tensor &t, int c0, int c) {
        Tensor s = t;
        s.off += c0; s.C = c;
        return s;
    }
    ArgRef ref(const Tensor &t) const { ArgRef r; r.storage = t.st; r.byte_offset = t.off * es_; return r; }
    static ArgRef ref(size_t st, size_t byte_off = 0) { ArgRef r; r.storage = st; r.byte_offset = byte_off; return r; }
    static ArgRef none() { return ArgRef(); }

    KernelInfo &add_kernel(const std::string &name, OpKind op, std::vector<ArgRef> refs, double flops, double bytes) {
        KernelInfo k;
        k.name = name; k.op = op; k.refs = std::move(refs); k.flops = flops; k.bytes = bytes;
        std::memset(&k.p, 0, sizeof(k.p));
        std::memset(k.launch_params, 0, sizeof(k.launch_params));
        m_.kernel_infos.push_back(std::move(k));
        return m_.kernel_infos.back();
    }

    // conv + folded-BN bias + optional residual + activation; writes into `into` when given
    Tensor conv(const std::string &name, const Tensor &in, int cout, int k, int stride, int pad, int act,
                const Tensor *residual = nullptr, const Tensor *into = nullptr, int cin_logical = -1, float init_gain = 1.f) {
        return conv_hw(name, in, cout, k, k, stride, pad, pad, act, residual, into, cin_logical, init_gain);
    }
    // the same with a kh x kw filter and separate vertical / horizontal padding (Inception's 1x7 and 7x1)
    Tensor conv_hw(const std::string &name, const Tensor &in, int cout, int kh, int kw, int stride, int ph, int pw, int act,
                   const Tensor *residual = nullptr, const Tensor *into = nullptr, int cin_logical = -1, float init_gain = 1.f) {
        int Ho = (in.H + 2 * ph - kh) / stride + 1, Wo = (in.W + 2 * pw - kw) / stride + 1;
        int cin = cin_logical > 0 ? cin_logical : in.C;
        ParamLayout L;
        L.kind = ParamLayout::ConvOIHW; L.o = cout; L.i = cin; L.r = kh; L.s = kw; L.i_pad = in.C;
        L.disk_elems = (size_t)cout * cin * kh * kw;
        L.init = ParamLayout::InitNormal; L.init_a = init_gain * std::sqrt(2.f / (float)(cin * kh * kw));  // He-normal
        size_t w = add_param(name + ".weight", (size_t)cout * kh * kw * in.C, L);
        ParamLayout LB; LB.disk_elems = cout; LB.init = ParamLayout::InitZero;
        size_t b = add_param(name + ".bias", cout, LB);
        Tensor out = into ? *into : activation(name + ".out", in.N, Ho, Wo, cout);
        double flops = 2.0 * in.N * Ho * Wo * cout * (double)cin * kh * kw;
        double bytes = es_ * ((double)in.N * in.H * in.W * cin + (double)cout * cin * kh * kw + cout + (double)in.N * Ho * Wo * cout * (residual ? 2 : 1));
        KernelInfo &ki = add_kernel("conv2d", OpKind::Conv, {ref(in), ref(w), ref(b), residual ? ref(*residual) : none(), ref(out)}, flops, bytes);
        gp_conv_params &p = ki.p.conv;
        p.dtype = gp_dt_; p.N = in.N; p.H = in.H; p.W = in.W; p.Cin = in.C; p.Cout = cout; p.R = kh; p.S = kw;
        p.stride_h = p.stride_w = stride; p.pad_h = ph; p.pad_w = pw;
        p.in_pix_stride = in.ps; p.res_pix_stride = residual ? residual->ps : 0; p.out_pix_stride = out.ps; p.act = act;
        Tensor o = out; o.N = in.N; o.H = Ho; o.W = Wo; o.C = cout;
        return o;
    }

    Tensor pool(const std::string &name, const Tensor &in, int k, int stride, int pad, int mode, const Tensor *into = nullptr) {
        int Ho = mode == 2 ? 1 : (in.H + 2 * pad - k) / stride + 1, Wo = mode == 2 ? 1 : (in.W + 2 * pad - k) / stride + 1;
        Tensor out = into ? *into : activation(name + ".out", in.N, Ho, Wo, in.C);
        double bytes = es_ * ((double)in.N * in.H * in.W * in.C + (double)in.N * Ho * Wo * in.C);
        KernelInfo &ki = add_kernel("pool2d", OpKind::Pool, {ref(in), ref(out)}, 0, bytes);
        gp_pool_params &p = ki.p.pool;
        p.dtype = gp_dt_; p.N = in.N; p.H = in.H; p.W = in.W; p.C = in.C; p.R = k; p.S = k; p.stride = stride; p.pad = pad; p.mode = mode;
        p.in_pix_stride = in.ps; p.out_pix_stride = out.ps;
        Tensor o = out; o.N = in.N; o.H = Ho; o.W = Wo; o.C = in.C;
        return o;
    }

    // out = act((a [+ b]) * scale + shift); scale/shift are parameters when affine_name is set
    Tensor eltwise(const std::string &name, const Tensor &a, const Tensor *b, const std::string &affine_name, int act, const Tensor *into = nullptr) {
        Tensor out = into ? *into : activation(name + ".out", a.N, a.H, a.W, a.C);
        size_t sc = SIZE_MAX, sh = SIZE_MAX;
        if (!affine_name.empty()) {
            ParamLayout L1; L1.disk_elems = a.C; L1.init = ParamLayout::InitConst; L1.init_a = 1.f;
            sc = add_param(affine_name + ".scale", a.C, L1);
            ParamLayout L0; L0.disk_elems = a.C; L0.init = ParamLayout::InitZero;
            sh = add_param(affine_name + ".shift", a.C, L0);
        }
        double elems = (double)a.N * a.H * a.W * a.C;
        KernelInfo &ki = add_kernel("eltwise", OpKind::Eltwise, {ref(a), b ? ref(*b) : none(), sc == SIZE_MAX ? none() : ref(sc), sh == SIZE_MAX ? none() : ref(sh), ref(out)},
                                    elems, es_ * elems * (b ? 3 : 2));
        gp_eltwise_params &p = ki.p.eltwise;
        p.dtype = gp_dt_; p.rows = (long)a.N * a.H * a.W; p.cols = a.C; p.a_stride = a.ps; p.b_stride = b ? b->ps : 0; p.out_stride = out.ps; p.act = act;
        Tensor o = out; o.N = a.N; o.H = a.H; o.W = a.W; o.C = a.C;
        return o;
    }

    // dense layer: rows x in_features -> rows x units; weight on disk [units][in_features]
    size_t dense(const std::string &name, size_t in_st, size_t in_off_bytes, long rows, int in_f, long lda, int units, int act,
                 size_t residual_st, size_t out_st, size_t out_off_bytes, long ldc, float init_std, const ParamLayout *wl = nullptr) {
        ParamLayout L;
        if (wl) L = *wl;
        L.o = units; L.disk_elems = (size_t)units * in_f; L.init = ParamLayout::InitNormal; L.init_a = init_std;
        size_t w = add_param(name + ".weight", (size_t)units * in_f, L);
        ParamLayout LB; LB.disk_elems = units; LB.init = ParamLayout::InitZero;
        size_t b = add_param(name + ".bias", units, LB);
        double flops = 2.0 * rows * units * (double)in_f;
        double bytes = es_ * ((double)rows * in_f + (double)units * in_f + units + (double)rows * units * (residual_st == SIZE_MAX ? 1 : 2));
        KernelInfo &ki = add_kernel("dense", OpKind::Gemm, {ref(in_st, in_off_bytes), ref(w), ref(b), residual_st == SIZE_MAX ? none() : ref(residual_st), ref(out_st, out_off_bytes)}, flops, bytes);
        gp_gemm_params &p = ki.p.gemm;
        p.dtype = gp_dt_; p.M = (int)rows; p.N = units; p.K = in_f; p.lda = lda; p.ldb = in_f; p.b_is_nk = 1; p.ldc = ldc; p.alpha = 1.f; p.act = act; p.batch = 1;
        return w;
    }

    void softmax(size_t x_st, size_t out_st, long rows, int cols, float scale) {
        double e = (double)rows * cols;
        KernelInfo &ki = add_kernel("softmax", OpKind::Softmax, {ref(x_st), ref(out_st)}, 5 * e, 2 * es_ * e);
        gp_softmax_params &p = ki.p.softmax;
        p.dtype = gp_dt_; p.rows = rows; p.cols = cols; p.scale = scale;
    }

    Tensor input_nchw(int N, int C, int H, int W) {
        // "data" is NCHW in the model dtype, as the reference feeds it (src/tests/test-dnn.cpp:25-30)
        size_t data = add_storage("data", (size_t)N * C * H * W, stype_);
        Tensor t = activation("data.nhwc", N, H, W, pad_c(C));
        double e = (double)N * H * W;
        KernelInfo &ki = add_kernel("nchw_to_nhwc", OpKind::Layout, {ref(data), ref(t)}, 0, es_ * e * (C + t.C));
        gp_layout_params &p = ki.p.layout;
        p.dtype_in = p.dtype_out = gp_dt_; p.N = N; p.C = C; p.H = H; p.W = W; p.c_pad = t.C;
        return t;
    }

    Model &m_;
    std::string dt_, stype_;
    int gp_dt_ = 0, vec_ = 4;
    size_t es_ = 4;
};

}  // namespace foo
