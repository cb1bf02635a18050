"""Writes small models in the reference's export schema (mod.json as TVM's graph executor stores it,
host.json as patch/tvm.patch:296-311 adds it, mod.params as scripts/compile/compile.py:73-83 writes
it) plus the operator sidecar ops.json, and computes what the model must output with the oracle's
operators on the way.  TEST INFRASTRUCTURE: the reference ships no exported model, so the tests
build their own; names follow TVM's (parameters p0, p1, ...; one fused function per operator group,
identical groups sharing a function, host.json listing one entry per operator node in graph order as
src/model.cpp:199-229 walks it)."""
import json
import os

import numpy as np

from oracle import oracle as O
from gpreempt_amd.executor import write_params


class ExportWriter:
    def __init__(self, dt="f32", seed=0):
        self.dt = dt
        self.rng = np.random.default_rng(seed)
        self.nodes, self.shapes, self.values = [], [], []
        self.dtypes = {}     # node -> dltype, where it is not the model's element type (int64 token ids)
        self.params = {}
        self.funcs = {}      # (base, key) -> function name
        self.taken = {}      # base -> how many functions carry it
        self.ops = []        # sidecar entries, one per function
        self.host = []       # host.json entries, one per operator node
        self.n_temp = 0
        self.alias = {}      # name of the same parameter in the built-in graphs -> export name

    # ---- graph bookkeeping -------------------------------------------------------------------------
    def _r(self, a):
        return O.round_to(np.asarray(a, np.float32), self.dt)

    def _node(self, name, inputs, value, func=None):
        node = {"op": "tvm_op" if func else "null", "name": name, "inputs": [[i, 0, 0] for i in inputs]}
        if func:
            node["attrs"] = {"num_outputs": "1", "num_inputs": str(len(inputs)), "flatten_data": "0", "func_name": func}
        self.nodes.append(node)
        self.shapes.append(list(value.shape))
        self.values.append(value)
        return len(self.nodes) - 1

    def _func(self, base, key, op, attrs, epilogue, inputs):
        k = (base, key)
        if k not in self.funcs:
            n = self.taken.get(base, 0)
            self.taken[base] = n + 1
            name = "tvmgen_default_fused_" + base + (f"_{n}" if n else "")
            self.funcs[k] = name
            self.ops.append({"name": name, "op": op, "attrs": attrs, "epilogue": epilogue, "inputs": inputs})
        return self.funcs[k]

    def _op(self, base, key, op, attrs, epilogue, roles, inputs, value, temps=0):
        func = self._func(base, key, op, attrs, epilogue, roles)
        node = self._node(func.replace("tvmgen_default_", ""), inputs, value, func)
        args = list(range(len(inputs) + 1))
        kernels = [{"name": func + "_kernel0", "launch_params": [max(1, value.size // 256), 1, 1, 256, 1, 1], "args": args}]
        if temps:  # a function whose first kernel leaves an intermediate in a temporary buffer
            self.n_temp = max(self.n_temp, temps)
            kernels = [{"name": func + "_kernel0", "launch_params": [1, 1, 1, 64, 1, 1], "args": args[:-1] + [-1]},
                       {"name": func + "_kernel1", "launch_params": [1, 1, 1, 64, 1, 1], "args": [-1, args[-1]]}]
        self.host.append({"name": func, "kernels": kernels})
        return node

    # ---- tensors -----------------------------------------------------------------------------------
    def data(self, x):
        return self._node("data", [], self._r(x))

    def param(self, value):
        name = f"p{len(self.params)}"
        self.params[name] = np.asarray(value, np.float32)
        return self._node(name, [], self._r(value))

    def value(self, node):
        return self.values[node]

    # ---- operators ---------------------------------------------------------------------------------
    def conv2d(self, x, cout, k, stride=1, pad=0, bias=True, residual=None, relu=True, gain=1.0, temps=0, name=None):
        kh, kw = (k, k) if isinstance(k, int) else k
        sh, sw = (stride, stride) if isinstance(stride, int) else stride
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        cin = self.shapes[x][1]
        w = self.param(self.rng.normal(0, gain * np.sqrt(2.0 / (cin * kh * kw)), (cout, cin, kh, kw)))
        inputs, roles, epi, base = [x, w], {"data": 0, "weight": 1}, [], "nn_conv2d"
        if name:
            self.alias[name + ".weight"] = self.nodes[w]["name"]
        bv = None
        if bias:
            b = self.param(self.rng.normal(0, 0.1, (cout, 1, 1)))
            if name:
                self.alias[name + ".bias"] = self.nodes[b]["name"]
            bv = self.values[b].reshape(-1)
            roles["bias"] = len(inputs); inputs.append(b); epi.append("bias"); base += "_add"
        rv = None
        if residual is not None:
            rv = self.values[residual]
            roles["residual"] = len(inputs); inputs.append(residual); epi.append("residual"); base += "_add"
        if relu:
            epi.append("relu"); base += "_nn_relu"
        out = self._r(O.conv2d(self.values[x], self.values[w], bv, (sh, sw), (ph, pw), rv, O.ACT_RELU if relu else O.ACT_NONE))
        attrs = {"strides": [sh, sw], "padding": [ph, pw, ph, pw], "dilation": [1, 1], "groups": 1}
        key = (tuple(self.shapes[x]), cout, kh, kw, sh, sw, ph, pw, tuple(epi))
        return self._op(base, key, "conv2d", attrs, epi, roles, inputs, out, temps)

    def dense(self, x, units, bias=True, relu=False, name=None, gelu=False, residual=None, std=None):
        feat = self.shapes[x][1]
        w = self.param(self.rng.normal(0, std if std else np.sqrt(1.0 / feat), (units, feat)))
        inputs, roles, epi, base = [x, w], {"data": 0, "weight": 1}, [], "nn_dense"
        if name:
            self.alias[name + ".weight"] = self.nodes[w]["name"]
        bv = None
        if bias:
            b = self.param(self.rng.normal(0, 0.1, (units,)))
            if name:
                self.alias[name + ".bias"] = self.nodes[b]["name"]
            bv = self.values[b]
            roles["bias"] = 2; inputs.append(b); epi.append("bias"); base += "_add"
        rv = None
        if residual is not None:
            rv = self.values[residual]
            roles["residual"] = len(inputs); inputs.append(residual); epi.append("residual"); base += "_add"
        if relu:
            epi.append("relu"); base += "_nn_relu"
        if gelu:
            epi.append("gelu"); base += "_multiply_erf_add_multiply_multiply"
        act = O.ACT_RELU if relu else O.ACT_GELU if gelu else O.ACT_NONE
        out = self._r(O.gemm_bias_act(self.values[x], self.values[w], bv, rv, act, b_is_nk=True))
        return self._op(base, (tuple(self.shapes[x]), units, tuple(epi)), "dense", {}, epi, roles, inputs, out)

    # ---- transformer operators (the functions of a BERT export) -------------------------------------
    def data_ids(self, ids):
        n = self._node("data", [], np.asarray(ids, np.int64))
        self.dtypes[n] = "int64"
        return n

    def take_embed(self, ids, vocab, hidden, position=True, segment=True, names=None):
        """take(word table, ids) + position rows + segment row: one fused function, as TVM fuses a gather with the
        broadcast additions behind it"""
        B, S = self.shapes[ids]
        word = self.param(self.rng.normal(0, 0.02, (vocab, hidden)))
        inputs, roles, base = [word, ids], {"table": 0, "indices": 1}, "take"
        pos_v = np.zeros((S, hidden), np.float32)
        seg_v = None
        if position:
            pos = self.param(self.rng.normal(0, 0.02, (1, S, hidden)))  # the first S position rows, folded to a constant
            pos_v = self.values[pos].reshape(S, hidden)
            roles["position"] = len(inputs); inputs.append(pos); base += "_add"
        if segment:
            seg = self.param(self.rng.normal(0, 0.02, (1, 1, hidden)))
            seg_v = self.values[seg].reshape(hidden)
            roles["segment"] = len(inputs); inputs.append(seg); base += "_add"
        if names:
            self.alias[names[0]] = self.nodes[word]["name"]
            if position: self.alias[names[1]] = self.nodes[pos]["name"]
            if segment: self.alias[names[2]] = self.nodes[seg]["name"]
        out = self._r(O.embed(self.values[ids], self.values[word], pos_v, seg_v, S)).reshape(B, S, hidden)
        return self._op(base, (B, S, vocab, hidden, position, segment), "take", {"axis": 0}, [], roles, inputs, out)

    def layer_norm(self, x, eps=(1, -12), residual=None, name=None):
        c = self.shapes[x][-1]
        g = self.param(self.rng.uniform(0.8, 1.2, (c,)))
        bt = self.param(self.rng.uniform(-0.1, 0.1, (c,)))
        if name:
            self.alias[name + ".gamma"], self.alias[name + ".beta"] = self.nodes[g]["name"], self.nodes[bt]["name"]
        inputs, roles = [x, g, bt], {"data": 0, "gamma": 1, "beta": 2}
        rv = None
        if residual is not None:
            rv = self.values[residual]
            roles["residual"] = 3; inputs.append(residual)
        out = self._r(O.layernorm(self.values[x], self.values[g], self.values[bt], eps[0] * 10.0 ** eps[1], rv))
        return self._op("add_layer_norm" if residual is not None else "layer_norm", (tuple(self.shapes[x]), eps, residual is not None), "layer_norm",
                        {"axis": -1, "epsilon": list(eps)}, [], roles, inputs, out)

    def gelu(self, x):
        out = self._r(O.add_act(self.values[x], None, O.ACT_GELU))
        return self._op("multiply_erf_add_multiply_multiply", tuple(self.shapes[x]), "gelu", {}, [], {"data": 0}, [x], out)

    def reshape(self, x, shape):
        """a reshape that TVM turns into a __nop node (it shares its argument's memory)"""
        return self._node("reshape_nop", [x], self.values[x].reshape(shape), "__nop")

    def transpose(self, x, axes):
        out = np.ascontiguousarray(np.transpose(self.values[x], axes))
        return self._op("transpose", (tuple(self.shapes[x]), tuple(axes)), "transpose", {"axes": list(axes)}, [], {"data": 0}, [x], out)

    def batch_matmul(self, a, b, scale_rsqrt=0, transpose_b=True):
        alpha = 1.0 / np.sqrt(scale_rsqrt) if scale_rsqrt else 1.0
        out = self._r(O.bmm(self.values[a], self.values[b], alpha=alpha, b_is_nk=transpose_b))
        attrs = {"transpose_b": int(transpose_b)}
        if scale_rsqrt:
            attrs["scale_rsqrt"] = int(scale_rsqrt)
        return self._op("nn_batch_matmul" + ("_multiply" if scale_rsqrt else ""), (tuple(self.shapes[a]), tuple(self.shapes[b]), scale_rsqrt, transpose_b), "batch_matmul", attrs, [],
                        {"lhs": 0, "rhs": 1}, [a, b], out)

    def pool(self, x, kind, k=2, stride=2, pad=0, count_include_pad=False):
        if kind == "global_avg":
            n, c = self.shapes[x][:2]
            out = self._r(O.global_avgpool(self.values[x])).reshape(n, c, 1, 1)
            return self._op("nn_global_avg_pool2d", tuple(self.shapes[x]), "global_avg_pool2d", {}, [], {"data": 0}, [x], out)
        mode = "max" if kind == "max" else ("avg_pad" if count_include_pad else "avg")
        out = self._r(O.pool2d(self.values[x], k, stride, pad, mode))
        attrs = {"pool_size": [k, k], "strides": [stride, stride], "padding": [pad, pad, pad, pad], "ceil_mode": 0}
        if kind == "avg":
            attrs["count_include_pad"] = int(count_include_pad)
        op = "max_pool2d" if kind == "max" else "avg_pool2d"
        return self._op("nn_" + op, (tuple(self.shapes[x]), k, stride, pad, count_include_pad), op, attrs, [], {"data": 0}, [x], out)

    def add(self, a, b, relu=False):
        out = self._r(O.add_act(self.values[a], self.values[b], O.ACT_RELU if relu else O.ACT_NONE))
        return self._op("add" + ("_nn_relu" if relu else ""), (tuple(self.shapes[a]), relu), "add", {}, ["relu"] if relu else [], {"lhs": 0, "rhs": 1}, [a, b], out)

    def add_channel_constant(self, x, relu=False):
        c = self.shapes[x][1]
        p = self.param(self.rng.normal(0, 0.2, (c, 1, 1)))
        out = self._r(O.scale_shift_act(self.values[x], np.ones(c, np.float32), self.values[p].reshape(-1), O.ACT_RELU if relu else O.ACT_NONE))
        return self._op("add" + ("_nn_relu" if relu else ""), (tuple(self.shapes[x]), relu, "const"), "add", {}, ["relu"] if relu else [], {"lhs": 0, "rhs": 1}, [x, p], out)

    def scale_shift(self, x, relu=True, name=None):
        c = self.shapes[x][1]
        s = self.param(self.rng.uniform(0.5, 1.5, (c, 1, 1)))
        h = self.param(self.rng.normal(0, 0.2, (c, 1, 1)))
        if name:
            self.alias[name + ".scale"], self.alias[name + ".shift"] = self.nodes[s]["name"], self.nodes[h]["name"]
        out = self._r(O.scale_shift_act(self.values[x], self.values[s].reshape(-1), self.values[h].reshape(-1), O.ACT_RELU if relu else O.ACT_NONE))
        return self._op("multiply_add" + ("_nn_relu" if relu else ""), (tuple(self.shapes[x]), relu), "scale_shift", {}, ["relu"] if relu else [],
                        {"data": 0, "scale": 1, "shift": 2}, [x, s, h], out)

    def softmax(self, x):
        return self._op("nn_softmax", tuple(self.shapes[x]), "softmax", {"axis": -1}, [], {"data": 0}, [x], self._r(O.softmax(self.values[x])))

    def concatenate(self, xs):
        out = np.concatenate([self.values[x] for x in xs], axis=1)
        return self._op("concatenate", tuple(tuple(self.shapes[x]) for x in xs), "concatenate", {"axis": 1}, [], {}, list(xs), out)

    def flatten(self, x):
        """batch_flatten, which TVM turns into a __nop node (a reshape that shares its argument's memory)"""
        v = self.values[x]
        return self._node("reshape_nop", [x], v.reshape(v.shape[0], -1), "__nop")

    # ---- files -------------------------------------------------------------------------------------
    def write(self, directory, head, sidecar=True, params=True):
        os.makedirs(directory, exist_ok=True)
        stype = {"f32": "float32", "f16": "float16", "bf16": "float32"}[self.dt]
        n = len(self.nodes)
        mod = {"nodes": self.nodes, "arg_nodes": [i for i, nd in enumerate(self.nodes) if nd["op"] == "null"], "heads": [[head, 0, 0]],
               "attrs": {"dltype": ["list_str", [self.dtypes.get(i, stype) for i in range(n)]], "device_index": ["list_int", [2] * n], "storage_id": ["list_int", list(range(n))],
                         "shape": ["list_shape", self.shapes]},
               "node_row_ptr": list(range(n + 1))}
        host = {"temp_args": [4096] * self.n_temp, "funcs": self.host}
        with open(os.path.join(directory, "mod.json"), "w") as f:
            json.dump(mod, f)
        with open(os.path.join(directory, "host.json"), "w") as f:
            json.dump(host, f)
        if sidecar:
            with open(os.path.join(directory, "ops.json"), "w") as f:
                json.dump({"layout": "NCHW", "funcs": self.ops}, f)
        if params:
            write_params(os.path.join(directory, "mod.params"), self.params)
        return self.values[head]


def mini_resnet(dt, batch=2, hw=32, seed=1):
    """stem, max-pool, two bottleneck blocks (one with a projected shortcut, one with the identity), a
    concatenation, a per-channel scale and shift, average pool, global pool, classifier, softmax"""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (batch, 3, hw, hw)))
    y = w.conv2d(x, 16, 7, 2, 3, temps=1)
    y = w.pool(y, "max", 3, 2, 1)
    sc = w.conv2d(y, 32, 1, relu=False)
    z = w.conv2d(y, 8, 1)
    z = w.conv2d(z, 8, 3, 1, 1)
    y = w.conv2d(z, 32, 1, residual=sc, gain=0.5)
    z = w.conv2d(y, 8, 1)
    z = w.conv2d(z, 8, 3, 1, 1)          # same shapes and attributes as the block before: the same function
    y2 = w.conv2d(z, 32, 1, residual=y, gain=0.5)
    br = w.conv2d(y2, 16, (1, 3), 1, (0, 1), bias=False)
    cat = w.concatenate([y2, br])
    y = w.pool(w.scale_shift(cat), "avg", 2, 2, 0)
    y = w.add(y, w.pool(cat, "avg", 3, 2, 1, count_include_pad=True))
    y = w.pool(y, "global_avg")
    y = w.flatten(y)
    y = w.dense(y, 10)
    return w, w.softmax(y)


def mini_vgg(dt, batch=1, hw=16, seed=2):
    """convolutions without fused bias, a separate per-channel add, 2x2 max-pools, a flatten of a 4 x 4
    image (dense weights stored over C x H x W) and two dense layers"""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (batch, 3, hw, hw)))
    y = w.conv2d(x, 8, 3, 1, 1, bias=False, relu=False)
    y = w.add_channel_constant(y, relu=True)
    y = w.pool(y, "max", 2, 2)
    y = w.conv2d(y, 16, 3, 1, 1)
    y = w.pool(y, "max", 2, 2)
    y = w.flatten(y)
    y = w.dense(y, 32, relu=True)
    return w, w.dense(y, 10, bias=False)


def padded_channels(dt, seed=3):
    """channel counts that are no multiple of the 16-byte vector: 12 and 20 channels, the narrow one last
    in a concatenation"""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (1, 3, 12, 12)))
    a = w.conv2d(x, 16, 3, 1, 1)
    b = w.conv2d(a, 12, 3, 2, 1)
    c = w.conv2d(b, 20, 1)
    d = w.pool(w.conv2d(a, 16, 3, 2, 1), "max", 3, 1, 1)
    y = w.concatenate([d, c])            # 16 + 20
    y = w.conv2d(y, 24, 3, 1, 1)
    y = w.pool(y, "global_avg")
    y = w.flatten(y)
    return w, w.dense(y, 5)


def resnet(dt, blocks, batch=1, hw=224, seed=4):
    """ResNet v1 with bottleneck blocks as the built-in "resnet50" / "resnet101" / "resnet152" graphs hold it
    (batch norm folded into the convolutions, stride on the first 1x1 of a down-sampling block);
    `alias` maps the built-in graph's parameter names to the export's."""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (batch, 3, hw, hw)))
    x = w.conv2d(x, 64, 7, 2, 3, name="conv1")
    x = w.pool(x, "max", 3, 2, 1)
    for s in range(4):
        width = 64 << s
        for b in range(blocks[s]):
            n = f"layer{s + 1}.{b}"
            stride = 2 if (b == 0 and s > 0) else 1
            shortcut = w.conv2d(x, 4 * width, 1, stride, 0, relu=False, name=n + ".downsample") if b == 0 else x
            y = w.conv2d(x, width, 1, stride, 0, name=n + ".conv1")
            y = w.conv2d(y, width, 3, 1, 1, name=n + ".conv2")
            x = w.conv2d(y, 4 * width, 1, residual=shortcut, gain=0.5, name=n + ".conv3")
    x = w.flatten(w.pool(x, "global_avg"))
    return w, w.softmax(w.dense(x, 1000, name="fc"))


def densenet(dt, layers=(2, 2, 2, 2), growth=8, init=16, batch=2, hw=32, classes=10, seed=5):
    """DenseNet as the built-in "densenet" graph holds it: norm-ReLU in front of every convolution inside
    the blocks, each layer's new channels concatenated behind everything before them."""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (batch, 3, hw, hw)))
    x = w.pool(w.conv2d(x, init, 7, 2, 3, name="conv0"), "max", 3, 2, 1)
    for b, n_layers in enumerate(layers):
        for l in range(n_layers):
            n = f"block{b + 1}.layer{l + 1}"
            t = w.scale_shift(x, name=n + ".norm1")
            t = w.conv2d(t, 4 * growth, 1, name=n + ".conv1")
            x = w.concatenate([x, w.conv2d(t, growth, 3, 1, 1, relu=False, name=n + ".conv2")])
        if b + 1 < len(layers):
            n = f"transition{b + 1}"
            t = w.conv2d(w.scale_shift(x, name=n + ".norm"), w.shapes[x][1] // 2, 1, relu=False, name=n + ".conv")
            x = w.pool(t, "avg", 2, 2, 0)
    x = w.flatten(w.pool(w.scale_shift(x, name="norm5"), "global_avg"))
    return w, w.softmax(w.dense(x, classes, name="classifier"))


def shared_concat(dt, seed=6):
    """one tensor in two concatenations: it is computed in place for the first and copied for the second;
    an inception-style block whose four branches all land in place"""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (1, 3, 8, 8)))
    a = w.conv2d(x, 8, 3, 1, 1)
    b = w.conv2d(x, 16, 1)
    y = w.add(w.concatenate([a, b]), w.concatenate([b, a]))
    y = w.concatenate([w.conv2d(y, 8, 1), w.conv2d(y, 8, 3, 1, 1), w.pool(y, "max", 3, 1, 1), w.pool(y, "avg", 3, 1, 1)])
    # a tensor that is both concatenated and flattened stays in plain memory (the concatenation copies it)
    p = w.pool(y, "global_avg")
    q = w.pool(w.conv2d(y, 8, 1), "global_avg")
    y = w.add(w.dense(w.flatten(w.concatenate([p, q])), 8, bias=False), w.dense(w.flatten(q), 8))
    return w, w.dense(y, 6)


def mlp(dt, seed=7):
    """a model whose input is a matrix: two dense layers and a softmax"""
    w = ExportWriter(dt, seed)
    x = w.data(w.rng.normal(0, 1, (6, 64)))
    y = w.dense(x, 48, relu=True)
    return w, w.softmax(w.dense(y, 16))


def bert(dt, layers=2, batch=2, seq=32, hidden=128, heads=2, ffn=256, vocab=96, seed=8, separate_tail=False):
    """A BERT encoder as a PyTorch model reaches TVM (scripts/compile/compile-bert.py:33-52): embedding gather with
    the position and segment rows added, layer-norm, then per layer separate query / key / value projections,
    [batch, sequence, heads, size] reshapes and transposes around two batch_matmul functions and a softmax, the
    output projection with the residual, layer-norm, and the feed-forward pair with erf-GELU.  separate_tail:
    GELU and the residual additions as functions of their own (the add in front of a layer-norm fused into it)
    instead of dense epilogues.  Returns (writer, head node, parameters under the built-in "bert" graph's names)."""
    w = ExportWriter(dt, seed)
    d = hidden // heads
    T = batch * seq
    ids = w.data_ids(w.rng.integers(0, vocab, (batch, seq)))
    x = w.take_embed(ids, vocab, hidden, names=("embeddings.word", "embeddings.position", "embeddings.token_type"))
    x = w.layer_norm(x, name="embeddings.ln")
    x = w.reshape(x, (T, hidden))
    builtin = {}
    for l in range(layers):
        n = f"layer{l}"
        def heads_of(t):  # [T, hidden] -> [batch * heads, seq, d]
            t = w.reshape(t, (batch, seq, heads, d))
            t = w.transpose(t, (0, 2, 1, 3))
            return w.reshape(t, (batch * heads, seq, d))
        qkv = [w.dense(x, hidden, std=0.02, name=f"{n}.attn.{r}") for r in ("q", "k", "v")]
        q, k, v = (heads_of(t) for t in qkv)
        scores = w.batch_matmul(q, k, scale_rsqrt=d)
        probs = w.softmax(scores)
        vt = w.transpose(v, (0, 2, 1))                 # relay's batch_matmul wants [b, N, K]
        ctx = w.batch_matmul(probs, vt)
        ctx = w.reshape(ctx, (batch, heads, seq, d))
        ctx = w.transpose(ctx, (0, 2, 1, 3))
        ctx = w.reshape(ctx, (T, hidden))
        if separate_tail:
            ao = w.dense(ctx, hidden, std=0.02, name=n + ".attn.proj")
            x1 = w.layer_norm(ao, residual=x, name=n + ".ln1")
            f1 = w.gelu(w.dense(x1, ffn, std=0.02, name=n + ".ffn1"))
            f2 = w.add(w.dense(f1, hidden, std=0.02, name=n + ".ffn2"), x1)
            x = w.layer_norm(f2, name=n + ".ln2")
        else:
            ao = w.dense(ctx, hidden, std=0.02, residual=x, name=n + ".attn.proj")
            x1 = w.layer_norm(ao, name=n + ".ln1")
            f1 = w.dense(x1, ffn, std=0.02, gelu=True, name=n + ".ffn1")
            f2 = w.dense(f1, hidden, std=0.02, residual=x1, name=n + ".ffn2")
            x = w.layer_norm(f2, name=n + ".ln2")
        # the built-in graph holds the three projections as one matrix
        for part in ("weight", "bias"):
            builtin[f"{n}.attn.qkv.{part}"] = np.concatenate([w.params[w.alias[f"{n}.attn.{r}.{part}"]] for r in ("q", "k", "v")], axis=0)
    for name, pname in w.alias.items():
        if ".attn.q." in name or ".attn.k." in name or ".attn.v." in name:
            continue
        builtin[name] = w.params[pname]
    builtin["embeddings.position"] = builtin["embeddings.position"].reshape(seq, hidden)
    builtin["embeddings.token_type"] = builtin["embeddings.token_type"].reshape(1, hidden)
    head = w.reshape(x, (batch, seq, hidden))
    return w, head, builtin
