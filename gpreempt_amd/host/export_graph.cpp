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

// A strided view of a storage, for the tensors of a transformer between its matrix products: [batch, sequence,
// heads, head size] and its transposes.  Always held as four dimensions (leading ones of size 1 where the
// export has fewer); `merged` says the export sees the first two as one ([batch * heads, rows, columns]).
struct SeqView {
    bool on = false, merged = false;
    long dim[4] = {1, 1, 1, 1}, str[4] = {0, 0, 0, 0};  // elements
    bool contiguous() const {
        long want = 1;
        for (int i = 3; i >= 0; --i) { if (dim[i] != 1 && str[i] != want) return false; want *= dim[i]; }
        return true;
    }
    long elems() const { return dim[0] * dim[1] * dim[2] * dim[3]; }
};

struct Val {
    bool set = false, is_param = false;
    bool is_ids = false;  // int64 token ids (a transformer's "data")
    SeqView sv;           // on: `t` only names the storage and the offset
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
        if (s.size() == 3) { if (s[0] * s[1] >= (1L << 31)) return false; N = (int)(s[0] * s[1]); C = (int)s[2]; H = W = 1; return true; }  // [batch, sequence, width]: rows of a matrix
        if (s.size() == 2) { N = (int)s[0]; C = (int)s[1]; H = W = 1; return true; }
        if (s.size() == 1) { N = 1; C = (int)s[0]; H = W = 1; return true; }
        return false;
    }
    Status check_shape(size_t node, const Val &v) {
        if (v.sv.on) return check_view_shape(node, v.sv);
        int N, C, H, W;
        if (!nchw_of(node, N, C, H, W)) return fail(node, "tensors of 1 to 4 dimensions only");
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
            else if (!nchw_of(root, rn, rc, rh, rw)) return fail(root, "tensors of 1 to 4 dimensions only");
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
        if (vals[node].is_ids) return fail(user, "argument '" + ex.nodes[node].name + "' holds token ids: only take reads those");
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
        if (in->sv.on) return fail(i, "dense over a view of a matrix (reshape it back to rows x features first)");
        if (in->t.H != 1 || in->t.W != 1) return fail(i, "dense over a tensor that was not flattened");
        const std::vector<long> &ws = ex.nodes[wn].shape;
        if (ws.size() != 2) return fail(i, "dense weight must be units x features");
        const int units = (int)ws[0], feat = (int)ws[1];
        if (feat != in->c_log) return fail(i, "weight has " + std::to_string(feat) + " input features, the data " + std::to_string(in->c_log));
        const int K = in->t.C;  // features as they lie in memory: padding channels take zero weights
        if (K % b.vec() || in->t.ps % b.vec()) return fail(i, "dense over " + std::to_string(feat) + " features, which is not a multiple of " + std::to_string(b.vec()));
        int act;
        RETURN_STATUS(tail_act(i, op, act));
        const Val *res = nullptr;
        if (has_tail(op, "residual")) {
            size_t rn;
            if (!input_of(i, op, "residual", 3, rn)) return fail(i, "the epilogue names a residual the function has no argument for");
            RETURN_STATUS(need_act(i, rn, res));
            // the GEMM reads the residual with the output's row stride
            if (!plain_matrix(*res) || res->t.N != in->t.N || res->t.C != units) return fail(i, "the residual of a dense layer must be a plain rows x units matrix");
        }
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
        KernelInfo &ki = b.add_kernel("dense", OpKind::Gemm, {b.ref(in->t), GraphBuilder::ref(w), bias == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(bias), res ? b.ref(res->t) : GraphBuilder::none(), b.ref(out.t)}, flops, bytes);
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
        if (v.sv.on) return fail(i, "an element-wise operator over a view of a matrix (reshape it back first)");
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
        if (a->sv.on) return softmax_view(i, op, *a);
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
        // a view of a transformer's tensors, or a plain matrix about to become one
        if (a->sv.on || (plain_matrix(*a) && ex.nodes[i].shape.size() == 4)) return reshape_seq(i, *a);
        int N, C, H, W;
        if (!nchw_of(i, N, C, H, W)) return fail(i, "tensors of 1 to 4 dimensions only");
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

    // ---- transformer operators (the functions of a BERT export, scripts/compile/compile-bert.py:76-77) -----------
    // A plain matrix: rows x columns in unpadded, unsliced memory (what the dense layers and layer-norms of a
    // transformer read and write).
    static bool plain_matrix(const Val &v) { return !v.sv.on && !v.is_ids && v.t.H == 1 && v.t.W == 1 && v.t.off == 0 && v.t.ps == v.t.C && v.t.C == v.c_log && !v.fc; }
    Val matrix_val(const std::string &name, long rows, int cols) {
        Val out;
        out.set = true; out.c_log = cols;
        out.t.st = b.add_storage(name, (size_t)rows * cols, b.stype_);
        out.t.N = (int)rows; out.t.H = out.t.W = 1; out.t.C = cols; out.t.ps = cols;
        return out;
    }
    // the shape the export states for node i, as four dimensions (leading ones)
    bool dims4_of(size_t i, long d[4], int &rank) const {
        const std::vector<long> &s = ex.nodes[i].shape;
        rank = (int)s.size();
        if (rank < 1 || rank > 4) return false;
        for (int k = 0; k < 4; ++k) d[k] = 1;
        for (int k = 0; k < rank; ++k) d[4 - rank + k] = s[k];
        return true;
    }
    Status check_view_shape(size_t i, const SeqView &v) {
        long d[4]; int rank;
        if (!dims4_of(i, d, rank)) return fail(i, "tensors of 1 to 4 dimensions only");
        bool ok;
        if (v.merged) ok = rank == 3 && d[1] == v.dim[0] * v.dim[1] && d[2] == v.dim[2] && d[3] == v.dim[3];
        else ok = d[0] == v.dim[0] && d[1] == v.dim[1] && d[2] == v.dim[2] && d[3] == v.dim[3];
        if (!ok) return fail(i, "the export's shape differs from what the operator attributes give (" + std::to_string(v.dim[0]) + "x" + std::to_string(v.dim[1]) + "x" +
                                    std::to_string(v.dim[2]) + "x" + std::to_string(v.dim[3]) + (v.merged ? ", first two merged)" : ")"));
        return Status::Succ;
    }
    static float attr_eps(const ExportOp &op) {  // "epsilon": [mantissa, decimal exponent], e.g. [1, -12]
        auto it = op.attrs.find("epsilon");
        if (it == op.attrs.end() || it->second.size() != 2) return 1e-5f;
        return (float)((double)it->second[0] * std::pow(10.0, (double)it->second[1]));
    }

    // take(table, indices) [+ position rows] [+ one segment row]: the embedding sum of a BERT encoder
    Status take(size_t i, const ExportOp &op) {
        size_t tn, in, pn = SIZE_MAX, sn = SIZE_MAX;
        if (!input_of(i, op, "table", 0, tn) || !input_of(i, op, "indices", 1, in)) return fail(i, "take needs a table and indices");
        if (!vals[in].is_ids) return fail(i, "take: the indices must be the model's int64 input");
        if (attr(op, "axis", 0, 0) != 0) return fail(i, "take along axis 0 only");
        const std::vector<long> &ts = ex.nodes[tn].shape, &is = ex.nodes[in].shape;
        if (ts.size() != 2) return fail(i, "take: the table must be rows x width");
        const long vocab = ts[0]; const int Hd = (int)ts[1];
        if (Hd % b.vec()) return fail(i, "take: rows of " + std::to_string(Hd) + " values, which is not a multiple of " + std::to_string(b.vec()));
        const long T = prod(is), S = is.empty() ? 1 : is.back();
        ParamLayout L; L.o = (int)vocab; L.disk_elems = (size_t)vocab * Hd; L.init = ParamLayout::InitNormal; L.init_a = 0.02f;
        size_t tab, pos, seg = SIZE_MAX;
        RETURN_STATUS(param(i, tn, (size_t)vocab * Hd, L, 5, tab));
        if (op.inputs.count("position")) {
            if (!input_of(i, op, "position", 2, pn)) return fail(i, "take: no argument for the position rows");
            const long rows = prod(ex.nodes[pn].shape) / Hd;
            if (prod(ex.nodes[pn].shape) != rows * Hd || rows < S) return fail(i, "take: the position rows must be (at least) sequence x width");
            ParamLayout P; P.o = (int)rows; P.disk_elems = (size_t)rows * Hd; P.init = ParamLayout::InitNormal; P.init_a = 0.02f;
            RETURN_STATUS(param(i, pn, (size_t)rows * Hd, P, 6, pos));
        } else {
            // a bare gather: position rows of zeros (never on disk, so they stay zero)
            ParamLayout Z; Z.disk_elems = (size_t)S * Hd; Z.init = ParamLayout::InitZero;
            pos = b.add_param(ex.nodes[i].name + ".zero_rows", (size_t)S * Hd, Z);
        }
        if (op.inputs.count("segment")) {
            if (!input_of(i, op, "segment", 3, sn)) return fail(i, "take: no argument for the segment row");
            if (prod(ex.nodes[sn].shape) != Hd) return fail(i, "take: the segment row must hold one row of the table's width");
            ParamLayout G; G.o = 1; G.disk_elems = (size_t)Hd; G.init = ParamLayout::InitNormal; G.init_a = 0.02f;
            RETURN_STATUS(param(i, sn, (size_t)Hd, G, 7, seg));
        }
        Val out = matrix_val(ex.nodes[i].name, T, Hd);
        KernelInfo &k = b.add_kernel("embed", OpKind::Embed, {b.ref(vals[in].t), GraphBuilder::ref(tab), GraphBuilder::ref(pos), seg == SIZE_MAX ? GraphBuilder::none() : GraphBuilder::ref(seg), b.ref(out.t)},
                                     2.0 * T * Hd, 8.0 * T + b.es() * 4.0 * T * Hd);
        gp_embed_params &p = k.p.embed;
        p.dtype = b.gp_dtype(); p.tokens = T; p.seq = (int)S; p.hidden = Hd; p.vocab = vocab;
        vals[i] = out;
        return Status::Succ;
    }

    Status layer_norm(size_t i, const ExportOp &op) {
        size_t dn, gn, bn, rn;
        if (!input_of(i, op, "data", 0, dn) || !input_of(i, op, "gamma", 1, gn) || !input_of(i, op, "beta", 2, bn)) return fail(i, "layer_norm needs data, gamma and beta");
        const Val *a, *res = nullptr;
        RETURN_STATUS(need_act(i, dn, a));
        if (!plain_matrix(*a)) return fail(i, "layer_norm over the rows of a plain matrix only");
        const long axis = attr(op, "axis", 0, -1);
        if (axis != -1 && axis != (long)ex.nodes[dn].shape.size() - 1) return fail(i, "layer_norm over the last axis only");
        if (!op.epilogue.empty()) return fail(i, "layer_norm takes no epilogue");
        if (a->t.C % b.vec()) return fail(i, "layer_norm over rows of " + std::to_string(a->t.C) + " values, which is not a multiple of " + std::to_string(b.vec()));
        if (op.inputs.count("residual")) {  // layer_norm(data + residual): the add in front of it fused in
            if (!input_of(i, op, "residual", 3, rn)) return fail(i, "layer_norm: no argument for the residual");
            RETURN_STATUS(need_act(i, rn, res));
            if (!plain_matrix(*res) || res->t.N != a->t.N || res->t.C != a->t.C) return fail(i, "layer_norm: the residual's shape differs from the data's");
        }
        size_t ga, be;
        RETURN_STATUS(vector_param(i, gn, a->t.C, a->t.C, ParamLayout::InitConst, 1.f, 4, ga));
        RETURN_STATUS(vector_param(i, bn, a->t.C, a->t.C, ParamLayout::InitZero, 0.f, 2, be));
        Val out = matrix_val(ex.nodes[i].name, a->t.N, a->t.C);
        const double e = (double)a->t.N * a->t.C;
        KernelInfo &k = b.add_kernel("layernorm", OpKind::Layernorm, {b.ref(a->t), res ? b.ref(res->t) : GraphBuilder::none(), GraphBuilder::ref(ga), GraphBuilder::ref(be), b.ref(out.t)},
                                     8 * e, b.es() * e * (res ? 3 : 2));
        gp_layernorm_params &p = k.p.layernorm;
        p.dtype = b.gp_dtype(); p.rows = a->t.N; p.cols = a->t.C; p.eps = attr_eps(op);
        vals[i] = out;
        return Status::Succ;
    }

    // erf-GELU as a function of its own
    Status gelu(size_t i, const ExportOp &op) {
        size_t dn;
        if (!input_of(i, op, "data", 0, dn)) return fail(i, "gelu needs data");
        const Val *a;
        RETURN_STATUS(need_act(i, dn, a));
        if (!plain_matrix(*a)) return fail(i, "gelu over a plain matrix only");
        RETURN_STATUS(elementwise_ready(i, *a));
        if (!op.epilogue.empty()) return fail(i, "gelu takes no epilogue");
        Val out = matrix_val(ex.nodes[i].name, a->t.N, a->t.C);
        emit_eltwise(a->t, nullptr, SIZE_MAX, SIZE_MAX, out.t, GP_ACT_GELU);
        vals[i] = out;
        return Status::Succ;
    }

    // transpose: a new view of the same memory (the matrix products read and write through strides)
    Status transpose(size_t i, const ExportOp &op) {
        if (ex.nodes[i].inputs.size() != 1) return fail(i, "a transpose has one argument");
        const Val *a;
        RETURN_STATUS(need_act(i, ex.nodes[i].inputs[0], a));
        if (!a->sv.on) return fail(i, "transpose of a tensor that is not a view of a matrix (reshape it to its dimensions first)");
        auto it = op.attrs.find("axes");
        if (it == op.attrs.end()) return fail(i, "transpose needs axes");
        const std::vector<long> &ax = it->second;
        const int rank = a->sv.merged ? 3 : 4;
        // fewer axes than four: the leading dimensions of size 1 stay in front
        int lead = 0;
        if (!a->sv.merged) while (lead < 4 && (int)ax.size() < 4 - lead && a->sv.dim[lead] == 1) ++lead;
        if ((int)ax.size() != rank - lead) return fail(i, "transpose: " + std::to_string(ax.size()) + " axes for a tensor of " + std::to_string(rank - lead) + " dimensions");
        Val out = *a;
        if (a->sv.merged) {
            if (ax[0] != 0 || !((ax[1] == 1 && ax[2] == 2) || (ax[1] == 2 && ax[2] == 1))) return fail(i, "of a [batch x heads, rows, columns] tensor only the last two axes can be swapped");
            if (ax[1] == 2) { std::swap(out.sv.dim[2], out.sv.dim[3]); std::swap(out.sv.str[2], out.sv.str[3]); }
        } else {
            bool seen[4] = {false, false, false, false};
            for (size_t k = 0; k < ax.size(); ++k) {
                if (ax[k] < 0 || ax[k] >= (long)ax.size() || seen[ax[k]]) return fail(i, "transpose: axes must be a permutation");
                seen[ax[k]] = true;
                out.sv.dim[lead + k] = a->sv.dim[lead + ax[k]];
                out.sv.str[lead + k] = a->sv.str[lead + ax[k]];
            }
        }
        vals[i] = out;
        return check_view_shape(i, out.sv);
    }

    // which batch_matmul results are read back as [batch, rows, heads x columns] (reshape, transpose (0,2,1,3),
    // reshape): those are written in that order, so that the way back costs nothing
    std::vector<char> interleave;
    void plan_batch_matmuls() {
        interleave.assign(ex.global_len, 0);
        std::vector<std::vector<size_t>> users(ex.global_len);
        for (size_t i = 0; i < ex.global_len; ++i) for (size_t j : ex.nodes[i].inputs) if (j < ex.global_len) users[j].push_back(i);
        auto is_reshape = [&](size_t n) { const ExportOp *o = op_of(n); return ex.nodes[n].func == "__nop" || (o && o->op == "reshape"); };
        for (size_t i = 0; i < ex.global_len; ++i) {
            const ExportOp *o = op_of(i);
            if (!o || o->op != "batch_matmul" || users[i].size() != 1 || (size_t)ex.heads_index == i) continue;
            const size_t r = users[i][0];
            if (!is_reshape(r) || ex.nodes[r].shape.size() != 4 || users[r].size() != 1) continue;
            const ExportOp *t = op_of(users[r][0]);
            if (!t || t->op != "transpose") continue;
            auto it = t->attrs.find("axes");
            if (it != t->attrs.end() && it->second == std::vector<long>{0, 2, 1, 3}) interleave[i] = 1;
        }
    }

    // batch_matmul(lhs [b, M, K], rhs [b, N, K]) -> [b, M, N] (relay's nn.batch_matmul; "transpose_b": 0 for rhs [b, K, N]);
    // "scale_rsqrt": d multiplies the products by 1 / sqrt(d)
    Status batch_matmul(size_t i, const ExportOp &op) {
        size_t an, bn;
        if (!input_of(i, op, "lhs", 0, an) || !input_of(i, op, "rhs", 1, bn)) return fail(i, "batch_matmul needs two arguments");
        const Val *A, *B;
        RETURN_STATUS(need_act(i, an, A));
        RETURN_STATUS(need_act(i, bn, B));
        if (!A->sv.on || !B->sv.on) return fail(i, "batch_matmul over tensors that are not views of matrices (reshape them to their dimensions first)");
        if (!op.epilogue.empty()) return fail(i, "batch_matmul takes no epilogue");
        const bool tb = attr(op, "transpose_b", 0, 1) != 0;
        const SeqView &a = A->sv, &r = B->sv;
        const long bo = a.dim[0], bi = a.dim[1], M = a.dim[2], K = a.dim[3];
        const long N = tb ? r.dim[2] : r.dim[3], Kb = tb ? r.dim[3] : r.dim[2];
        if (r.dim[0] != bo || r.dim[1] != bi || Kb != K) return fail(i, "batch_matmul: the arguments' batch or inner dimensions differ");
        if (a.str[3] != 1) return fail(i, "batch_matmul: the rows of the first argument must be contiguous");
        // the second argument as the GEMM wants it: N x K with K contiguous, or K x N with N contiguous
        const long k_str = tb ? r.str[3] : r.str[2], n_str = tb ? r.str[2] : r.str[3];
        int b_is_nk; long ldb;
        if (k_str == 1) { b_is_nk = 1; ldb = n_str; }
        else if (n_str == 1) { b_is_nk = 0; ldb = k_str; }
        else return fail(i, "batch_matmul: neither dimension of the second argument is contiguous");
        const int vec = b.vec();
        if (K % vec || a.str[2] % vec || ldb % vec || a.str[0] % vec || a.str[1] % vec || r.str[0] % vec || r.str[1] % vec || (!b_is_nk && N % vec) ||
            A->t.off % vec || B->t.off % vec)
            return fail(i, "batch_matmul: dimensions and strides must be multiples of " + std::to_string(vec) + " elements");
        if (M >= (1L << 31) || N >= (1L << 31) || bo * bi >= (1L << 24)) return fail(i, "batch_matmul: too large");
        Val out;
        out.set = true; out.c_log = (int)N;
        out.t.st = b.add_storage(ex.nodes[i].name, (size_t)(bo * bi * M * N), b.stype_);
        out.sv.on = true; out.sv.merged = true;
        out.sv.dim[0] = bo; out.sv.dim[1] = bi; out.sv.dim[2] = M; out.sv.dim[3] = N;
        if (interleave[i]) { out.sv.str[0] = M * bi * N; out.sv.str[1] = N; out.sv.str[2] = bi * N; out.sv.str[3] = 1; }
        else { out.sv.str[0] = bi * M * N; out.sv.str[1] = M * N; out.sv.str[2] = N; out.sv.str[3] = 1; }
        const long scale = attr(op, "scale_rsqrt", 0, 0);
        const double flops = 2.0 * bo * bi * M * N * (double)K;
        const double bytes = b.es() * ((double)bo * bi * (M * K + N * K + M * N));
        KernelInfo &k = b.add_kernel("batch_matmul", OpKind::Gemm, {b.ref(A->t), b.ref(B->t), GraphBuilder::none(), GraphBuilder::none(), b.ref(out.t)}, flops, bytes);
        gp_gemm_params &p = k.p.gemm;
        p.dtype = b.gp_dtype(); p.M = (int)M; p.N = (int)N; p.K = (int)K; p.lda = a.str[2]; p.ldb = ldb; p.b_is_nk = b_is_nk; p.ldc = out.sv.str[2];
        p.alpha = scale > 0 ? 1.f / std::sqrt((float)scale) : 1.f; p.act = GP_ACT_NONE;
        p.batch = (int)(bo * bi);
        if (bi > 1) {
            p.batch_inner = (int)bi;
            p.stride_a = a.str[1]; p.stride_b = r.str[1]; p.stride_c = out.sv.str[1];
            p.stride_a_outer = a.str[0]; p.stride_b_outer = r.str[0]; p.stride_c_outer = out.sv.str[0];
        } else {
            p.batch_inner = 0;
            p.stride_a = a.str[0]; p.stride_b = r.str[0]; p.stride_c = out.sv.str[0];
        }
        vals[i] = out;
        return check_view_shape(i, out.sv);
    }

    // softmax over the last axis of a contiguous view (the attention scores)
    Status softmax_view(size_t i, const ExportOp &op, const Val &a) {
        const long axis = attr(op, "axis", 0, -1);
        const long rank = (long)ex.nodes[i].shape.size();
        if (axis != -1 && axis != rank - 1) return fail(i, "softmax over the last axis only");
        if (!a.sv.contiguous() || a.t.off != 0) return fail(i, "softmax over a transposed or sliced tensor");
        if (!op.epilogue.empty()) return fail(i, "softmax takes no epilogue");
        Val out = a;
        out.t.st = b.add_storage(ex.nodes[i].name, (size_t)a.sv.elems(), b.stype_);
        b.softmax(a.t.st, out.t.st, a.sv.elems() / a.sv.dim[3], (int)a.sv.dim[3], 1.f);
        vals[i] = out;
        return check_view_shape(i, out.sv);
    }

    // reshapes of a transformer: a matrix seen as [batch, sequence, heads, head size] and back
    Status reshape_seq(size_t i, const Val &a) {
        long d[4]; int rank;
        if (!dims4_of(i, d, rank)) return fail(i, "tensors of 1 to 4 dimensions only");
        Val out = a;
        if (!a.sv.on) {
            // a plain matrix seen as four dimensions: a contiguous view
            if (prod(ex.nodes[i].shape) != (long)a.t.N * a.c_log) return fail(i, "a reshape that changes the number of elements");
            out.sv.on = true; out.sv.merged = false;
            long st = 1;
            for (int k = 3; k >= 0; --k) { out.sv.dim[k] = d[k]; out.sv.str[k] = st; st *= d[k]; }
            vals[i] = out;
            return Status::Succ;
        }
        if (prod(ex.nodes[i].shape) != a.sv.elems()) return fail(i, "a reshape that changes the number of elements");
        const SeqView &v = a.sv;
        // the same four dimensions, the first two seen as one or as two again
        if (rank == 3 && d[1] == v.dim[0] * v.dim[1] && d[2] == v.dim[2] && d[3] == v.dim[3]) { out.sv.merged = true; vals[i] = out; return Status::Succ; }
        if (rank == 4 && d[0] == v.dim[0] && d[1] == v.dim[1] && d[2] == v.dim[2] && d[3] == v.dim[3]) { out.sv.merged = false; vals[i] = out; return Status::Succ; }
        if (!v.contiguous()) return fail(i, "a reshape of a transposed tensor that is more than joining its first two dimensions");
        if (rank <= 3) {  // contiguous memory read as a matrix again: rows x last dimension
            out.sv = SeqView();
            out.c_log = (int)d[3];
            out.t.N = (int)(a.sv.elems() / d[3]); out.t.H = out.t.W = 1; out.t.C = (int)d[3]; out.t.ps = d[3];
        } else {
            out.sv.merged = false;
            long st = 1;
            for (int k = 3; k >= 0; --k) { out.sv.dim[k] = d[k]; out.sv.str[k] = st; st *= d[k]; }
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
        plan_batch_matmuls();
        bool have_data = false;
        for (size_t i = 0; i < ex.global_len; ++i) {
            const ExportNode &n = ex.nodes[i];
            if (n.func.empty()) {
                if (n.name != "data") { vals[i].set = true; vals[i].is_param = true; continue; }
                if (have_data) return fail(i, "two inputs named data");
                have_data = true;
                int N, C, H, W;
                if (!nchw_of(i, N, C, H, W)) return fail(i, "tensors of 1 to 4 dimensions only");
                Val v;
                v.set = true; v.c_log = C;
                if (n.stype == "int64") {  // token ids (src/tests/test-dnn.cpp:21-23): read by take only
                    v.is_ids = true;
                    v.t.st = b.add_storage("data", (size_t)prod(n.shape), "int64");
                    v.t.N = (int)prod(n.shape); v.t.H = v.t.W = 1; v.t.C = v.t.ps = 1; v.c_log = 1;
                } else if (n.shape.size() == 4) v.t = b.input_nchw(N, C, H, W);
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
            else if (op.op == "take") s = take(i, op);
            else if (op.op == "layer_norm") s = layer_norm(i, op);
            else if (op.op == "gelu") s = gelu(i, op);
            else if (op.op == "transpose") s = transpose(i, op);
            else if (op.op == "batch_matmul") s = batch_matmul(i, op);
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
