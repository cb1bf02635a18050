// An exported model (mod.json + host.json + ops.json) on the native operators; see include/tvm_export.h.
//
// The export's graph is walked in node order.  Every node becomes a view of a storage: an NHWC
// tensor whose channel count may be padded to a 16-byte multiple (padding channels hold zeros and
// stay zero through every mapped operator), or the same with H = W = 1 for the export's 1-D and 2-D
// tensors.  A flatten of an H x W x C tensor keeps the memory as it is and remembers C, H, W, so that the
// dense layer behind it can re-order its weight's columns from the export's C-major order at load time.
#include "tvm_export.h"

#include <cmath>
#include <map>

#include "graph_builder.h"

namespace foo {

namespace {

struct Val {
    bool set = false, is_param = false;
    Tensor t;           // t.C = channels held in memory (>= c_log), t.ps = pixel stride
    int c_log = 0;      // channels the export knows about
    int fc = 0, fh = 0, fw = 0;  // a flattened fh x fw x fc tensor (t.H = t.W = 1, c_log = fh * fw * fc, t.C counts the padding channels too); 0 = not one
    size_t param_st = SIZE_MAX;
    int param_role = 0;
};

long prod(const std::vector<long> &s) { long p = 1; for (long d : s) p *= d; return p; }

struct Mapper {
    GraphBuilder &b;
    const TvmExport &ex;
    const ExportOps &ops;
    std::string &error;
    std::vector<Val> vals;
    std::map<std::string, const ExportOp *> by_func;
    // concatenation without a copy: a tensor that a channel concatenation takes as an argument is written
    // straight into its slice of the concatenation's buffer by the operator that computes it
    struct Place { size_t into = SIZE_MAX; int off = 0; };
    std::vector<Place> place;          // per node: the concatenation it lives in, and at which channel
    std::map<size_t, Tensor> buffers;  // per root node: the buffer made for it, perhaps before its turn

    Mapper(GraphBuilder &b_, const TvmExport &e, const ExportOps &o, std::string &err) : b(b_), ex(e), ops(o), error(err) {}

    Status fail(size_t node, const std::string &what) {
        error = "export node " + std::to_string(node) + " (" + ex.nodes[node].name + (ex.nodes[node].func.empty() ? "" : ", " + ex.nodes[node].func) + "): " + what;
        return Status::Fail;
    }

    static long attr(const ExportOp &op, const std::string &key, size_t i, long dflt) {
        auto it = op.attrs.find(key);
        if (it == op.attrs.end() || it->second.empty()) return dflt;
        return it->second.size() == 1 ? it->second[0] : (i < it->second.size() ? it->second[i] : dflt);
    }
    static bool has_tail(const ExportOp &op, const char *what) {
        for (const std::string &e : op.epilogue) if (e == what) return true;
        return false;
    }
    // the tail must read bias, residual, activation in that order: it is the only order the operators fuse
    Status tail_act(size_t node, const ExportOp &op, int &act) {
        int stage = 0;
        act = GP_ACT_NONE;
        for (const std::string &e : op.epilogue) {
            int s = e == "bias" ? 1 : e == "residual" ? 2 : 3;
            if (s < stage || (s == 3 && stage == 3)) return fail(node, "epilogue steps must be bias, residual, one activation, in that order");
            stage = s;
            if (e == "relu") act = GP_ACT_RELU;
            if (e == "gelu") act = GP_ACT_GELU;
        }
        return Status::Succ;
    }
    // argument `role` of the function that made `node` (by the sidecar's "inputs", else position `dflt`)
    bool input_of(size_t node, const ExportOp &op, const std::string &role, int dflt, size_t &in_node) const {
        auto it = op.inputs.find(role);
        int idx = it == op.inputs.end() ? dflt : it->second;
        if (idx < 0 || (size_t)idx >= ex.nodes[node].inputs.size()) return false;
        in_node = ex.nodes[node].inputs[idx];
        return true;
    }

    // ---- parameters: declared by their consumer, under the export's node name -------------------------
    Status param(size_t user, size_t node, size_t dev_elems, ParamLayout L, int role, size_t &st) {
        Val &v = vals[node];
        if (!v.is_param) return fail(user, "argument '" + ex.nodes[node].name + "' must be a parameter of the export");
        if ((size_t)prod(ex.nodes[node].shape) != L.disk_elems)
            return fail(user, "parameter '" + ex.nodes[node].name + "' holds " + std::to_string(prod(ex.nodes[node].shape)) + " values, the operator needs " + std::to_string(L.disk_elems));
        if (v.param_st != SIZE_MAX) {
            const ParamLayout &P = b.param_layout(v.param_st);
            const bool same = v.param_role == role && P.kind == L.kind && P.o == L.o && P.i == L.i && P.r == L.r && P.s == L.s && P.i_pad == L.i_pad && P.c == L.c && P.h == L.h && P.w == L.w;
            if (!same) return fail(user, "parameter '" + ex.nodes[node].name + "' is used by two operators that need different device layouts");
            st = v.param_st;
            return Status::Succ;
        }
        st = v.param_st = b.add_param(ex.nodes[node].name, dev_elems, L);
        v.param_role = role;
        return Status::Succ;
    }
    Status vector_param(size_t user, size_t node, int c_log, int c_mem, ParamLayout::Init init, float a, int role, size_t &st) {
        ParamLayout L;
        L.disk_elems = (size_t)c_log; L.init = init; L.init_a = a;
        return param(user, node, (size_t)c_mem, L, role, st);
    }

    // ---- shapes ---------------------------------------------------------------------------------------
    // what the export says node `i` looks like, as (N, C, H, W) with H = W = 1 below four dimensions
    bool nchw_of(size_t i, int &N, int &C, int &H, int &W) const {
        const std::vector<long> &s = ex.nodes[i].shape;
        for (long d : s) if (d <= 0 || d >= (1L << 31)) return false;
        if (s.size() == 4) { N = (int)s[0]; C = (int)s[1]; H = (int)s[2]; W = (int)s[3]; return true; }
        if (s.size() == 2) { N = (int)s[0]; C = (int)s[1]; H = W = 1; return true; }
        if (s.size() == 1) { N = 1; C = (int)s[0]; H = W = 1; return true; }
        return false;
    }
    Status check_shape(size_t node, const Val &v) {
        int N, C, H, W;
        if (!nchw_of(node, N, C, H, W)) return fail(node, "tensors of 1, 2 or 4 dimensions only");
        const int c = v.c_log;
        if (N != v.t.N || C != c || H != v.t.H || W != v.t.W)
            return fail(node, "the export says " + std::to_string(N) + "x" + std::to_string(C) + "x" + std::to_string(H) + "x" + std::to_string(W) + ", the operator attributes give " +
                                  std::to_string(v.t.N) + "x" + std::to_string(c) + "x" + std::to_string(v.t.H) + "x" + std::to_string(v.t.W));
        return Status::Succ;
    }
    const ExportOp *op_of(size_t node) const {
        auto it = by_func.find(ex.nodes[node].func);
        return it == by_func.end() ? nullptr : it->second;
    }
    // Which arguments of which concatenations can be computed in place.  An argument qualifies when one of
    // the operators that can write a channel slice makes it, it is not already placed (a tensor lives in
    // one place; a second concatenation of it copies), and its first channel falls on a 16-byte boundary.
    void plan_concatenations() {
        place.assign(ex.global_len, Place());
        // a tensor that is also flattened, soft-maxed or the model's output must lie in plain memory
        std::vector<char> plain(ex.global_len, 0);
        plain[ex.heads_index] = 1;
        for (size_t i = 0; i < ex.global_len; ++i) {
            const ExportOp *op = op_of(i);
            if (ex.nodes[i].func == "__nop" || (op && (op->op == "reshape" || op->op == "softmax")))
                for (size_t j : ex.nodes[i].inputs) if (j < ex.global_len) plain[j] = 1;
        }
        for (size_t i = 0; i < ex.global_len; ++i) {
            const ExportOp *op = op_of(i);
            if (!op || op->op != "concatenate" || attr(*op, "axis", 0, 1) != 1 || ex.nodes[i].shape.size() != 4) continue;
            int off = 0;
            for (size_t j : ex.nodes[i].inputs) {
                const ExportOp *src = j < i ? op_of(j) : nullptr;
                if (j >= ex.global_len || ex.nodes[j].shape.size() != 4) break;
                const bool writes_slices = src && (src->op == "conv2d" || src->op == "max_pool2d" || src->op == "avg_pool2d" || src->op == "global_avg_pool2d" || src->op == "add" ||
                                                   src->op == "scale_shift" || src->op == "concatenate");
                if (writes_slices && !plain[j] && place[j].into == SIZE_MAX && off % b.vec() == 0) { place[j].into = i; place[j].off = off; }
                off += (int)ex.nodes[j].shape[1];
            }
        }
    }
    // where node `i` of the given shape is to be written: its slice of a concatenation's buffer, or a
    // buffer of its own
    Status out_for(size_t i, int N, int H, int W, int c_log, Val &v) {
        size_t root = i;
        int off = 0;
        while (place[root].into != SIZE_MAX) { off += place[root].off; root = place[root].into; }
        auto it = buffers.find(root);
        if (it == buffers.end()) {
            int rn, rc, rh, rw;
            if (root == i) { rn = N; rc = c_log; rh = H; rw = W; }
            else if (!nchw_of(root, rn, rc, rh, rw)) return fail(root, "tensors of 1, 2 or 4 dimensions only");
            it = buffers.emplace(root, b.activation(ex.nodes[root].name, rn, rh, rw, b.pad_c(rc))).first;
        }
        const Tensor &buf = it->second;
        if (buf.N != N || buf.H != H || buf.W != W || off + b.pad_c(c_log) > buf.C)
            return fail(i, "the concatenation this result belongs to has another batch or image size");
        v = Val();
        v.set = true; v.c_log = c_log;
        v.t = GraphBuilder::slice(buf, off, b.pad_c(c_log));
        return Status::Succ;
    }
    Status need_act(size_t user, size_t node, const Val *&v) {
        if (node >= vals.size() || !vals[node].set || vals[node].is_param) return fail(user, "argument '" + ex.nodes[node].name + "' must be a tensor computed earlier in the graph");
        v = &vals[node];
        return Status::Succ;
    }

    // ---- operators ------------------------------------------------------------------------------------
    Status conv2d(size_t i, const ExportOp &op) {
        size_t dn, wn, bn = 0, rn = 0;
        if (!input_of(i, op, "data", 0, dn) || !input_of(i, op, "weight", 1, wn)) return fail(i, "conv2d needs data and weight");
        const Val *in;
        RETURN_STATUS(need_act(i, dn, in));
        if (in->fc) return fail(i, "conv2d over a flattened tensor");
        const std::vector<long> &ws = ex.nodes[wn].shape;
        if (ws.size() != 4) return fail(i, "conv2d weight must be O x I x R x S");
        const int O = (int)ws[0], I = (int)ws[1], R = (int)ws[2], S = (int)ws[3];
        if (attr(op, "groups", 0, 1) != 1) return fail(i, "grouped convolution is not mapped");
        if (attr(op, "dilation", 0, 1) != 1 || attr(op, "dilation", 1, 1) != 1) return fail(i, "dilated convolution is not mapped");
        if (I != in->c_log) return fail(i, "weight has " + std::to_string(I) + " input channels, the data " + std::to_string(in->c_log));
        const int sh = (int)attr(op, "strides", 0, 1), sw = (int)attr(op, "strides", 1, 1);
        // relay's padding: one value, (vertical, horizontal), or (top, left, bottom, right)
        auto pit = op.attrs.find("padding");
        const std::vector<long> pv = pit == op.attrs.end() || pit->second.empty() ? std::vector<long>{0} : pit->second;
        if (pv.size() != 1 && pv.size() != 2 && pv.size() != 4) return fail(i, "padding takes 1, 2 or 4 values");
        const int pt = (int)pv[0], pl2 = (int)(pv.size() == 1 ? pv[0] : pv[1]);
        const int pb = (int)(pv.size() == 4 ? pv[2] : pv[0]), pr = (int)(pv.size() == 4 ? pv[3] : pl2);
        if (pt != pb || pl2 != pr) return fail(i, "asymmetric padding is not mapped");
        if (sh <= 0 || sw <= 0 || pt < 0 || pl2 < 0) return fail(i, "bad strides or padding");
        const int Ho = (in->t.H + 2 * pt - R) / sh + 1, Wo = (in->t.W + 2 * pl2 - S) / sw + 1;
        if (Ho <= 0 || Wo <= 0) return fail(i, "empty convolution output");
        int act;
        RETURN_STATUS(tail_act(i, op, act));

        ParamLayout L;
        L.kind = ParamLayout::ConvOIHW; L.o = O; L.i = I; L.r = R; L.s = S; L.i_pad = in->t.C;
        L.disk_elems = (size_t)O * I * R * S;
        L.init = ParamLayout::InitNormal; L.init_a = std::sqrt(2.f / (float)(I * R * S));
        size_t w, bias = SIZE_MAX;
        RETURN_STATUS(param(i, wn, (size_t)O * R * S * in->t.C, L, 1, w));
        if (has_tail(op, "bias")) {
            if (!input_of(i, op, "bias", 2, bn)) return fail(i, "the epilogue names a bias the function has no argument for");
            RETURN_STATUS(vector_param(i, bn, O, O, ParamLayout::InitZero, 0.f, 2, bias));
        }
        const Val *res = nullptr;
        Val out;
        RETURN_STATUS(out_for(i, in->t.N, Ho, Wo, O, out));
        if (has_tail(op, "residual")) {
            if (!input_of(i, op, "residual", 3, rn)) return fail(i, "the epilogue names a residual the function has no argument for");
            RETURN_STATUS(need_act(i, rn, res));
            if (res->t.N != out.t.N || res->t.H != Ho || res->t.W != Wo || res->c_log != O) return fail(i, "the residual's shape differs from the output's");
        }
        const double flops = 2.0 * in->t.N * Ho * Wo * O * (double)I * R * S;
        const double bytes = b.es() * ((double)in->t.N * in->t.H * in->t.W * I + (double)O * I * R * S + O + (double)in->t.N * Ho * Wo * O * (res ? 2 : 1));
        KernelInfo &ki = b.add_kernel("conv2d", OpKind::Conv, {b.ref(in->t), GraphBuilder::ref(w), bias == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(bias),
                                                                res ? b.ref(res->t) : GraphBuilder::none(), b.ref(out.t)}, flops, bytes);
        gp_conv_params &p = ki.p.conv;
        p.dtype = b.gp_dtype(); p.N = in->t.N; p.H = in->t.H; p.W = in->t.W; p.Cin = in->t.C; p.Cout = O; p.R = R; p.S = S;
        p.stride_h = sh; p.stride_w = sw; p.pad_h = pt; p.pad_w = pl2;
        p.in_pix_stride = in->t.ps; p.res_pix_stride = res ? res->t.ps : 0; p.out_pix_stride = out.t.ps; p.act = act;
        vals[i] = out;
        return Status::Succ;
    }

    Status dense(size_t i, const ExportOp &op) {
        size_t dn, wn, bn = 0;
        if (!input_of(i, op, "data", 0, dn) || !input_of(i, op, "weight", 1, wn)) return fail(i, "dense needs data and weight");
        const Val *in;
        RETURN_STATUS(need_act(i, dn, in));
        if (in->t.H != 1 || in->t.W != 1) return fail(i, "dense over a tensor that was not flattened");
        const std::vector<long> &ws = ex.nodes[wn].shape;
        if (ws.size() != 2) return fail(i, "dense weight must be units x features");
        const int units = (int)ws[0], feat = (int)ws[1];
        if (feat != in->c_log) return fail(i, "weight has " + std::to_string(feat) + " input features, the data " + std::to_string(in->c_log));
        const int K = in->t.C;  // features as they lie in memory: padding channels take zero weights
        if (K % b.vec() || in->t.ps % b.vec()) return fail(i, "dense over " + std::to_string(feat) + " features, which is not a multiple of " + std::to_string(b.vec()));
        if (has_tail(op, "residual")) return fail(i, "a residual in a dense epilogue is not mapped");
        int act;
        RETURN_STATUS(tail_act(i, op, act));
        ParamLayout L;
        const int fc = in->fc ? in->fc : feat, fh = in->fc ? in->fh : 1, fw = in->fc ? in->fw : 1;
        if (fh * fw > 1 || K != feat) { L.kind = ParamLayout::DenseOverCHW; L.c = fc; L.h = fh; L.w = fw; L.i_pad = K / (fh * fw); }
        L.o = units; L.disk_elems = (size_t)units * feat;
        L.init = ParamLayout::InitNormal; L.init_a = std::sqrt(1.f / (float)feat);
        size_t w, bias = SIZE_MAX;
        RETURN_STATUS(param(i, wn, (size_t)units * K, L, 3, w));
        if (has_tail(op, "bias")) {
            if (!input_of(i, op, "bias", 2, bn)) return fail(i, "the epilogue names a bias the function has no argument for");
            RETURN_STATUS(vector_param(i, bn, units, units, ParamLayout::InitZero, 0.f, 2, bias));
        }
        // the result is a plain rows x units matrix: what "heads" must be, and what softmax reads
        Val out;
        out.set = true; out.c_log = units;
        out.t.st = b.add_storage(ex.nodes[i].name, (size_t)in->t.N * units, b.stype_);
        out.t.N = in->t.N; out.t.H = out.t.W = 1; out.t.C = units; out.t.ps = units;
        const long rows = in->t.N;
        const double flops = 2.0 * rows * units * (double)feat;
        const double bytes = b.es() * ((double)rows * feat + (double)units * feat + units + (double)rows * units);
        KernelInfo &ki = b.add_kernel("dense", OpKind::Gemm, {b.ref(in->t), GraphBuilder::ref(w), bias == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(bias), GraphBuilder::none(), b.ref(out.t)}, flops, bytes);
        gp_gemm_params &p = ki.p.gemm;
        p.dtype = b.gp_dtype(); p.M = (int)rows; p.N = units; p.K = K; p.lda = in->t.ps; p.ldb = K; p.b_is_nk = 1; p.ldc = units; p.alpha = 1.f; p.act = act; p.batch = 1;
        vals[i] = out;
        return Status::Succ;
    }

    Status pool(size_t i, const ExportOp &op) {
        size_t dn;
        if (!input_of(i, op, "data", 0, dn)) return fail(i, "pooling needs data");
        const Val *in;
        RETURN_STATUS(need_act(i, dn, in));
        if (in->fc) return fail(i, "pooling over a flattened tensor");
        int mode, k = 1, stride = 1, pad = 0;
        if (op.op == "global_avg_pool2d") mode = 2;
        else {
            k = (int)attr(op, "pool_size", 0, 0);
            stride = (int)attr(op, "strides", 0, 1);
            pad = (int)attr(op, "padding", 0, 0);
            auto same = [&](const char *key, long v) {
                auto it = op.attrs.find(key);
                if (it == op.attrs.end()) return true;
                for (long e : it->second) if (e != v) return false;
                return true;
            };
            if (k <= 0 || !same("pool_size", k) || !same("strides", stride) || !same("padding", pad)) return fail(i, "square windows with one stride and one padding only");
            if (attr(op, "ceil_mode", 0, 0) != 0) return fail(i, "ceil_mode is not mapped");
            if (attr(op, "dilation", 0, 1) != 1) return fail(i, "dilated pooling is not mapped");
            mode = op.op == "max_pool2d" ? 0 : (attr(op, "count_include_pad", 0, 0) ? 3 : 1);
        }
        const int Ho = mode == 2 ? 1 : (in->t.H + 2 * pad - k) / stride + 1, Wo = mode == 2 ? 1 : (in->t.W + 2 * pad - k) / stride + 1;
        if (Ho <= 0 || Wo <= 0) return fail(i, "empty pooling output");
        Val out;
        RETURN_STATUS(out_for(i, in->t.N, Ho, Wo, in->c_log, out));
        const double bytes = b.es() * ((double)in->t.N * in->t.H * in->t.W * in->t.C + (double)in->t.N * Ho * Wo * in->t.C);
        KernelInfo &ki = b.add_kernel("pool2d", OpKind::Pool, {b.ref(in->t), b.ref(out.t)}, 0, bytes);
        gp_pool_params &p = ki.p.pool;
        p.dtype = b.gp_dtype(); p.N = in->t.N; p.H = in->t.H; p.W = in->t.W; p.C = in->t.C; p.R = k; p.S = k; p.stride = stride; p.pad = pad; p.mode = mode;
        p.in_pix_stride = in->t.ps; p.out_pix_stride = out.t.ps;
        vals[i] = out;
        return Status::Succ;
    }

    // out = act((a [+ other]) * scale + shift) over every pixel of `a`
    void emit_eltwise(const Tensor &a, const Tensor *other, size_t scale, size_t shift, const Tensor &out, int act) {
        const double elems = (double)a.N * a.H * a.W * a.C;
        KernelInfo &ki = b.add_kernel("eltwise", OpKind::Eltwise, {b.ref(a), other ? b.ref(*other) : GraphBuilder::none(), scale == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(scale),
                                                                    shift == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(shift), b.ref(out)}, elems, b.es() * elems * (other ? 3 : 2));
        gp_eltwise_params &p = ki.p.eltwise;
        p.dtype = b.gp_dtype(); p.rows = (long)a.N * a.H * a.W; p.cols = a.C; p.a_stride = a.ps; p.b_stride = other ? other->ps : 0; p.out_stride = out.ps; p.act = act;
    }
    Status elementwise_ready(size_t i, const Val &v) {
        if (v.t.C % b.vec() || v.t.ps % b.vec() || v.t.off % b.vec()) return fail(i, "an element-wise operator over rows of " + std::to_string(v.t.C) + " values, which is not a multiple of " + std::to_string(b.vec()));
        return Status::Succ;
    }

    Status add(size_t i, const ExportOp &op) {
        size_t an, bn;
        if (!input_of(i, op, "lhs", 0, an) || !input_of(i, op, "rhs", 1, bn)) return fail(i, "add needs two arguments");
        if (vals[an].is_param && !vals[bn].is_param) std::swap(an, bn);
        const Val *a;
        RETURN_STATUS(need_act(i, an, a));
        RETURN_STATUS(elementwise_ready(i, *a));
        int act;
        RETURN_STATUS(tail_act(i, op, act));
        if (has_tail(op, "bias") || has_tail(op, "residual")) return fail(i, "add takes an activation as its only epilogue step");
        Val out;
        RETURN_STATUS(out_for(i, a->t.N, a->t.H, a->t.W, a->c_log, out));
        out.fc = vals[an].fc; out.fh = vals[an].fh; out.fw = vals[an].fw;
        if (vals[bn].is_param) {  // a per-channel constant
            if (a->fc) return fail(i, "a per-channel constant added to a flattened tensor");
            size_t shift;
            RETURN_STATUS(vector_param(i, bn, a->c_log, a->t.C, ParamLayout::InitZero, 0.f, 2, shift));
            emit_eltwise(a->t, nullptr, SIZE_MAX, shift, out.t, act);
        } else {
            const Val *o;
            RETURN_STATUS(need_act(i, bn, o));
            if (o->t.N != a->t.N || o->t.H != a->t.H || o->t.W != a->t.W || o->c_log != a->c_log || o->t.C != a->t.C || o->fc != a->fc || o->fh != a->fh || o->fw != a->fw)
                return fail(i, "the two arguments differ in shape (broadcasting is not mapped)");
            RETURN_STATUS(elementwise_ready(i, *o));
            emit_eltwise(a->t, &o->t, SIZE_MAX, SIZE_MAX, out.t, act);
        }
        vals[i] = out;
        return Status::Succ;
    }

    Status scale_shift(size_t i, const ExportOp &op) {
        size_t dn, sn, hn;
        if (!input_of(i, op, "data", 0, dn) || !input_of(i, op, "scale", 1, sn) || !input_of(i, op, "shift", 2, hn)) return fail(i, "scale_shift needs data, scale and shift");
        const Val *a;
        RETURN_STATUS(need_act(i, dn, a));
        if (a->fc) return fail(i, "scale_shift over a flattened tensor");
        RETURN_STATUS(elementwise_ready(i, *a));
        int act;
        RETURN_STATUS(tail_act(i, op, act));
        if (has_tail(op, "bias") || has_tail(op, "residual")) return fail(i, "scale_shift takes an activation as its only epilogue step");
        size_t scale, shift;
        RETURN_STATUS(vector_param(i, sn, a->c_log, a->t.C, ParamLayout::InitConst, 1.f, 4, scale));
        RETURN_STATUS(vector_param(i, hn, a->c_log, a->t.C, ParamLayout::InitZero, 0.f, 2, shift));
        Val out;
        RETURN_STATUS(out_for(i, a->t.N, a->t.H, a->t.W, a->c_log, out));
        emit_eltwise(a->t, nullptr, scale, shift, out.t, act);
        vals[i] = out;
        return Status::Succ;
    }

    Status softmax(size_t i, const ExportOp &op) {
        size_t dn;
        if (!input_of(i, op, "data", 0, dn)) return fail(i, "softmax needs data");
        const Val *a;
        RETURN_STATUS(need_act(i, dn, a));
        const long axis = attr(op, "axis", 0, -1);
        const long rank = (long)ex.nodes[dn].shape.size();
        if (a->t.H != 1 || a->t.W != 1 || (axis != -1 && axis != rank - 1)) return fail(i, "softmax over the last axis of a matrix only");
        if (a->t.off != 0 || a->t.ps != a->t.C || a->t.C != a->c_log) return fail(i, "softmax over a padded or sliced matrix");
        if (!op.epilogue.empty()) return fail(i, "softmax takes no epilogue");
        Val out;
        out.set = true; out.c_log = a->c_log; out.fc = a->fc; out.fh = a->fh; out.fw = a->fw;
        out.t.st = b.add_storage(ex.nodes[i].name, (size_t)a->t.N * a->t.C, b.stype_);
        out.t.N = a->t.N; out.t.H = out.t.W = 1; out.t.C = out.t.ps = a->t.C;
        b.softmax(a->t.st, out.t.st, a->t.N, a->t.C, 1.f);
        vals[i] = out;
        return Status::Succ;
    }

    Status concatenate(size_t i, const ExportOp &op) {
        if (attr(op, "axis", 0, 1) != 1) return fail(i, "concatenation over the channel axis only");
        if (!op.epilogue.empty()) return fail(i, "concatenate takes no epilogue");
        const std::vector<size_t> &ins = ex.nodes[i].inputs;
        if (ins.empty()) return fail(i, "concatenate needs arguments");
        int total = 0;
        for (size_t j = 0; j < ins.size(); ++j) {
            const Val *v;
            RETURN_STATUS(need_act(i, ins[j], v));
            if (v->fc) return fail(i, "concatenation of flattened tensors");
            if (v->t.N != vals[ins[0]].t.N || v->t.H != vals[ins[0]].t.H || v->t.W != vals[ins[0]].t.W) return fail(i, "the arguments differ in batch or image size");
            if (j + 1 < ins.size() && v->t.C != v->c_log) return fail(i, "an argument of " + std::to_string(v->c_log) + " channels, which is not a multiple of " + std::to_string(b.vec()) + ", in front of another");
            total += v->c_log;
        }
        const Val &first = vals[ins[0]];
        Val out;
        RETURN_STATUS(out_for(i, first.t.N, first.t.H, first.t.W, total, out));
        int at = 0;
        for (size_t j : ins) {
            const Val &v = vals[j];
            Tensor slice = GraphBuilder::slice(out.t, at, v.t.C);
            // an argument that was computed in place is already there
            const bool in_place = v.t.st == slice.st && v.t.off == slice.off && v.t.ps == slice.ps;
            if (!in_place) emit_eltwise(v.t, nullptr, SIZE_MAX, SIZE_MAX, slice, GP_ACT_NONE);
            at += v.c_log;
        }
        vals[i] = out;
        return Status::Succ;
    }

    // reshape, flatten, squeeze: the memory stays, the view changes
    Status reshape(size_t i) {
        if (ex.nodes[i].inputs.size() != 1) return fail(i, "a reshape has one argument");
        const size_t dn = ex.nodes[i].inputs[0];
        const Val *a;
        RETURN_STATUS(need_act(i, dn, a));
        int N, C, H, W;
        if (!nchw_of(i, N, C, H, W)) return fail(i, "tensors of 1, 2 or 4 dimensions only");
        const long have = (long)a->t.N * a->t.H * a->t.W * a->c_log;
        if ((long)N * C * H * W != have) return fail(i, "a reshape that changes the number of elements");
        Val out = *a;
        if (a->t.H * a->t.W > 1) {
            // N x C x H x W -> N x (C H W): NHWC memory read as one row per image
            if (H != 1 || W != 1 || N != a->t.N) return fail(i, "of a 4-D tensor only the flatten to N x (C H W) is mapped");
            // padding channels stay in the row: the dense layer behind it gives them zero weights
            if (a->t.ps != a->t.C) return fail(i, "flatten of a channel slice");
            out.fc = a->c_log; out.fh = a->t.H; out.fw = a->t.W;
            out.t.H = out.t.W = 1; out.c_log = C; out.t.C = out.t.ps = a->t.H * a->t.W * a->t.C;
        } else if (H * W > 1) {
            return fail(i, "a reshape from a matrix to an image is not mapped");
        } else if (N != a->t.N) {
            // rows regrouped: only for plain, unpadded memory, and the flatten's channel order is gone
            if (a->t.C != a->c_log || a->t.ps != a->t.C || (a->fc && a->fh * a->fw > 1)) return fail(i, "a reshape across rows of padded or re-ordered memory");
            out.fc = out.fh = out.fw = 0;
            out.t.N = N; out.t.C = out.c_log = C; out.t.ps = C;
        }
        vals[i] = out;
        return Status::Succ;
    }

    Status run() {
        for (const ExportOp &o : ops.funcs) by_func[o.func] = &o;
        if (ops.layout != "NCHW") { error = "ops json: only exports in NCHW layout are mapped"; return Status::Fail; }
        for (size_t i = 0; i < ex.global_len; ++i) {
            if (ex.nodes[i].shape.empty() || ex.nodes[i].shape.size() > 4) return fail(i, "tensors of 1 to 4 dimensions only");
            for (long d : ex.nodes[i].shape) if (d <= 0 || d >= (1L << 31)) return fail(i, "a dimension of " + std::to_string(d));
            if (prod(ex.nodes[i].shape) >= (1L << 40)) return fail(i, "more than 2^40 elements");
        }
        vals.assign(ex.global_len, Val());
        plan_concatenations();
        bool have_data = false;
        for (size_t i = 0; i < ex.global_len; ++i) {
            const ExportNode &n = ex.nodes[i];
            if (n.func.empty()) {
                if (n.name != "data") { vals[i].set = true; vals[i].is_param = true; continue; }
                if (have_data) return fail(i, "two inputs named data");
                have_data = true;
                int N, C, H, W;
                if (!nchw_of(i, N, C, H, W)) return fail(i, "tensors of 1, 2 or 4 dimensions only");
                Val v;
                v.set = true; v.c_log = C;
                if (n.shape.size() == 4) v.t = b.input_nchw(N, C, H, W);
                else {
                    v.t.st = b.add_storage("data", (size_t)N * C, b.stype_);
                    v.t.N = N; v.t.H = v.t.W = 1; v.t.C = v.t.ps = C;
                }
                vals[i] = v;
                continue;
            }
            if (n.func == "__nop") { RETURN_STATUS(reshape(i)); continue; }
            auto it = by_func.find(n.func);
            if (it == by_func.end()) return fail(i, "ops json does not describe this function");
            const ExportOp &op = *it->second;
            Status s;
            if (op.op == "conv2d") s = conv2d(i, op);
            else if (op.op == "dense") s = dense(i, op);
            else if (op.op == "max_pool2d" || op.op == "avg_pool2d" || op.op == "global_avg_pool2d") s = pool(i, op);
            else if (op.op == "add") s = add(i, op);
            else if (op.op == "scale_shift") s = scale_shift(i, op);
            else if (op.op == "softmax") s = softmax(i, op);
            else if (op.op == "concatenate") s = concatenate(i, op);
            else if (op.op == "reshape") s = reshape(i);
            else s = fail(i, "operator '" + op.op + "' is not mapped onto the native kernels");
            RETURN_STATUS(s);
            RETURN_STATUS(check_shape(i, vals[i]));
        }
        if (!have_data) { error = "the export has no input named data"; return Status::Fail; }
        // "heads": the storage behind the output node takes that name (src/model.cpp:231)
        const Val &h = vals[ex.heads_index];
        if (!h.set || h.is_param) return fail(ex.heads_index, "the output node is not computed");
        if (h.t.H * h.t.W > 1) return fail(ex.heads_index, "an image as the model's output is not mapped (the export holds it NCHW)");
        if (h.t.off != 0 || h.t.ps != h.t.C || h.t.C != h.c_log) return fail(ex.heads_index, "the output of " + std::to_string(h.c_log) + " values per row sits in padded or sliced memory");
        if (b.storage_name(h.t.st) == "data") return fail(ex.heads_index, "the output is the input");
        b.rename_storage(h.t.st, "heads");
        return Status::Succ;
    }
};

}  // namespace

Status build_export_graph(GraphBuilder &b, const TvmExport &ex, const ExportOps &ops, std::string &error) {
    if (ex.nodes.size() != ex.global_len || ex.heads_index >= ex.global_len) { error = "the export was not parsed"; return Status::Fail; }
    Mapper m(b, ex, ops, error);
    return m.run();
}

}  // namespace foo
