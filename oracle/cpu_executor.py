"""Front end of the CPU executor (oracle_exec.c): builds the kernel list of a model from the same
parameter dictionaries as oracle/models.py and runs it on the host cores through the
block-level-preemption tile loop.

TEST / MEASUREMENT INFRASTRUCTURE ONLY: used by tests/ and by the cpu_baseline leg of bench.py.
The graphs follow oracle/models.py function by function (gemm, bert, resnet); storage is fp32,
activations NHWC, convolution weights [Cout][R][S][Cin], as in the GPU build.
"""
import ctypes as C
import os

import numpy as np

from . import oracle as O

GEMM, CONV, POOL, ELTWISE, SOFTMAX, LAYERNORM, EMBED, ATTENTION = range(8)
vp = C.c_void_p


class Layer(C.Structure):
    _fields_ = [("op", C.c_int), ("act", C.c_int), ("M", C.c_int), ("N", C.c_int), ("K", C.c_int),
                ("lda", C.c_long), ("ldc", C.c_long), ("ldr", C.c_long),
                ("a", vp), ("b", vp), ("bias", vp), ("res", vp), ("c", vp), ("alpha", C.c_float),
                ("n", C.c_int), ("h", C.c_int), ("w", C.c_int), ("cin", C.c_int), ("cout", C.c_int), ("r", C.c_int), ("s", C.c_int),
                ("stride", C.c_int), ("ph", C.c_int), ("pw", C.c_int), ("ho", C.c_int), ("wo", C.c_int),
                ("in_ps", C.c_long), ("out_ps", C.c_long), ("res_ps", C.c_long),
                ("mode", C.c_int), ("rows", C.c_long), ("cols", C.c_int), ("eps", C.c_float), ("scale", C.c_float),
                ("gamma", vp), ("beta", vp), ("ids", vp), ("tok", vp), ("pos", vp), ("seg", vp), ("seq", C.c_int), ("vocab", C.c_int),
                ("batch", C.c_int), ("heads", C.c_int), ("head_dim", C.c_int), ("ld_qkv", C.c_long),
                ("q", vp), ("k", vp), ("v", vp), ("tiles", C.c_int), ("sx", C.c_int), ("sy", C.c_int)]


def _lib():
    lib = O.lib()
    assert lib.orx_layer_bytes() == C.sizeof(Layer), "oracle_exec.c and cpu_executor.py disagree on the layer struct"
    return lib


def default_threads():
    return int(os.environ.get("OMP_NUM_THREADS", 0)) or len(os.sched_getaffinity(0))


class Graph:
    """A kernel list plus the numpy buffers it points into (kept alive here)."""

    def __init__(self):
        self.layers, self.keep, self.flops = [], [], 0.0

    def buf(self, *shape):
        a = np.zeros(shape, np.float32)
        self.keep.append(a)
        return a

    def hold(self, a, dtype=np.float32):
        a = np.ascontiguousarray(a, dtype)
        self.keep.append(a)
        return a

    @staticmethod
    def p(a):
        return None if a is None else a.ctypes.data

    def gemm(self, a, w_nk, bias, out, act=0, res=None, alpha=1.0, M=None, lda=None, ldc=None, ldr=None):
        M = a.shape[0] if M is None else M
        N, K = w_nk.shape
        self.layers.append(Layer(op=GEMM, act=act, M=M, N=N, K=K, lda=lda or a.shape[-1], ldc=ldc or out.shape[-1], ldr=ldr or (res.shape[-1] if res is not None else 0),
                                 a=self.p(a), b=self.p(w_nk), bias=self.p(bias), res=self.p(res), c=self.p(out), alpha=alpha))
        self.flops += 2.0 * M * N * K

    def conv(self, x, w_ohwi, bias, out, stride, pad, act, res=None):
        n, h, w, cin = x.shape
        cout, r, s, _ = w_ohwi.shape
        ph, pw = (pad, pad) if isinstance(pad, int) else pad
        self.layers.append(Layer(op=CONV, act=act, n=n, h=h, w=w, cin=cin, cout=cout, r=r, s=s, stride=stride, ph=ph, pw=pw, in_ps=cin, out_ps=cout,
                                 res_ps=cout if res is not None else 0, a=self.p(x), b=self.p(w_ohwi), bias=self.p(bias), res=self.p(res), c=self.p(out), alpha=1.0))
        self.flops += 2.0 * out.shape[0] * out.shape[1] * out.shape[2] * cout * cin * r * s

    def pool(self, x, out, k, stride, pad, mode):
        n, h, w, c = x.shape
        self.layers.append(Layer(op=POOL, mode=mode, n=n, h=h, w=w, cin=c, r=k, stride=max(stride, 1), ph=pad, pw=pad, in_ps=c, out_ps=c, a=self.p(x), c=self.p(out)))

    def rows(self, op, x, out, rows, cols, **kw):
        self.layers.append(Layer(op=op, rows=rows, cols=cols, lda=cols, ldc=cols, ldr=cols, a=self.p(x), c=self.p(out), **kw))

    def run(self, threads=None, passes=1):
        arr = (Layer * len(self.layers))(*self.layers)
        ms = np.zeros(passes, np.float64)
        rc = _lib().orx_run(arr, len(self.layers), threads or default_threads(), passes, ms.ctypes.data_as(vp))
        assert rc == 0
        return ms

    def run_preempted(self, kernel, claim, threads=None):
        arr = (Layer * len(self.layers))(*self.layers)
        claims = np.zeros(len(self.layers), np.int32)
        stop = _lib().orx_run_preempted(arr, len(self.layers), threads or default_threads(), kernel, claim, claims.ctypes.data_as(vp))
        return stop, claims

    def tiles(self):
        arr = (Layer * len(self.layers))(*self.layers)
        _lib().orx_plan(arr, len(self.layers))
        return [l.tiles for l in arr]


def gemm_graph(A, B_kn, bias, act=O.ACT_RELU):
    """config 1: C = act(A B + bias); B on disk is K x N, kept N x K like the device copy."""
    g = Graph()
    a, w = g.hold(A), g.hold(np.ascontiguousarray(np.asarray(B_kn, np.float32).T))
    out = g.buf(A.shape[0], w.shape[0])
    g.gemm(a, w, g.hold(bias), out, act)
    return g, out


def bert_graph(params, ids, batch=1, seq=128, layers=12, hidden=768, heads=12):
    """oracle/models.py: bert, in fp32 storage."""
    g = Graph()
    T, d = batch * seq, hidden // heads
    P = lambda n: g.hold(params[n])
    idbuf = g.hold(ids, np.int64)
    emb, x = g.buf(T, hidden), g.buf(T, hidden)
    tok = P("embeddings.word")
    g.layers.append(Layer(op=EMBED, rows=T, cols=hidden, ldc=hidden, ids=g.p(idbuf), tok=g.p(tok), pos=g.p(P("embeddings.position")),
                          seg=g.p(g.hold(params["embeddings.token_type"][0])), seq=seq, vocab=tok.shape[0], c=g.p(emb)))
    g.rows(LAYERNORM, emb, x, T, hidden, gamma=g.p(P("embeddings.ln.gamma")), beta=g.p(P("embeddings.ln.beta")), eps=1e-12)
    for l in range(layers):
        n = f"layer{l}"
        qkv, ctx, ao, x1, f1, f2, x2 = g.buf(T, 3 * hidden), g.buf(T, hidden), g.buf(T, hidden), g.buf(T, hidden), g.buf(T, params[n + ".ffn1.weight"].shape[0]), g.buf(T, hidden), g.buf(T, hidden)
        g.gemm(x, P(n + ".attn.qkv.weight"), P(n + ".attn.qkv.bias"), qkv)
        g.layers.append(Layer(op=ATTENTION, batch=batch, heads=heads, head_dim=d, seq=seq, ld_qkv=3 * hidden, ldc=hidden, scale=1.0 / np.sqrt(d),
                              q=g.p(qkv), k=g.p(qkv) + 4 * hidden, v=g.p(qkv) + 8 * hidden, c=g.p(ctx)))
        g.flops += 4.0 * batch * heads * seq * seq * d
        g.gemm(ctx, P(n + ".attn.proj.weight"), P(n + ".attn.proj.bias"), ao, res=x)
        g.rows(LAYERNORM, ao, x1, T, hidden, gamma=g.p(P(n + ".ln1.gamma")), beta=g.p(P(n + ".ln1.beta")), eps=1e-12)
        g.gemm(x1, P(n + ".ffn1.weight"), P(n + ".ffn1.bias"), f1, act=O.ACT_GELU)
        g.gemm(f1, P(n + ".ffn2.weight"), P(n + ".ffn2.bias"), f2, res=x1)
        g.rows(LAYERNORM, f2, x2, T, hidden, gamma=g.p(P(n + ".ln2.gamma")), beta=g.p(P(n + ".ln2.beta")), eps=1e-12)
        x = x2
    return g, x


def resnet_graph(params, x_nchw, blocks):
    """oracle/models.py: resnet (v1 bottlenecks, stride on the first 1x1 of a down-sampling block, BN folded), fp32 storage."""
    g = Graph()
    x = g.hold(np.transpose(np.asarray(x_nchw, np.float32), (0, 2, 3, 1)))
    N = x.shape[0]

    def conv(name, t, stride, pad, act, res=None):
        w = g.hold(np.transpose(params[name + ".weight"], (0, 2, 3, 1)))
        k = w.shape[1]
        ho, wo = (t.shape[1] + 2 * pad - k) // stride + 1, (t.shape[2] + 2 * pad - k) // stride + 1
        out = g.buf(N, ho, wo, w.shape[0])
        g.conv(t, w, g.hold(params[name + ".bias"]), out, stride, pad, act, res)
        return out

    x = conv("conv1", x, 2, 3, O.ACT_RELU)
    pooled = g.buf(N, (x.shape[1] + 2 - 3) // 2 + 1, (x.shape[2] + 2 - 3) // 2 + 1, x.shape[3])
    g.pool(x, pooled, 3, 2, 1, 0)
    x = pooled
    for s in range(4):
        for b in range(blocks[s]):
            n = f"layer{s + 1}.{b}"
            stride = 2 if (b == 0 and s > 0) else 1
            shortcut = conv(n + ".downsample", x, stride, 0, O.ACT_NONE) if b == 0 else x
            y = conv(n + ".conv1", x, stride, 0, O.ACT_RELU)
            y = conv(n + ".conv2", y, 1, 1, O.ACT_RELU)
            x = conv(n + ".conv3", y, 1, 0, O.ACT_RELU, res=shortcut)
    gap = g.buf(N, 1, 1, x.shape[3])
    g.pool(x, gap, 0, 1, 0, 2)
    w = g.hold(params["fc.weight"])
    logits, probs = g.buf(N, w.shape[0]), g.buf(N, w.shape[0])
    g.gemm(gap.reshape(N, -1), w, g.hold(params["fc.bias"]), logits, M=N, lda=x.shape[3])
    g.rows(SOFTMAX, logits, probs, N, w.shape[0], scale=1.0)
    return g, probs


def timed(graph, warmups, runs, threads=None):
    """(mean, p50, p99) in ms over `runs` passes after `warmups` untimed ones; one set of pinned workers for all of them."""
    ms = graph.run(threads, warmups + runs)[warmups:]
    s = np.sort(ms)
    return float(ms.mean()), float(s[len(s) // 2]), float(s[min(len(s) - 1, int(np.ceil(0.99 * len(s))) - 1)])
