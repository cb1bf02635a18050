"""Layer-by-layer CPU restatement of the model graphs, composed from the oracle operators.

TEST INFRASTRUCTURE ONLY.  The reference takes its vision models from tvm.relay.testing and
"bert" from a traced HuggingFace model (scripts/compile/compile.py:28-44, compile-bert.py:33-52)
and ships neither weights nor outputs, so these functions restate the published architectures
at the shapes BASELINE.json names; parity with TVM's compiled numbers is UNPINNED.  What is
pinned: every operator against mathematics (tests/test_oracle_ops.py) and, for the conv/pool/
dense stacks, the composition against torch.nn.functional on CPU (tests/test_oracle_models.py).

`params` maps parameter names to fp32 arrays in the reference's on-disk convention (OIHW
convolution weights, [units][in_features] dense weights).  `dt` in {"f32","f16","bf16"} models
the storage type: parameters and every activation that a kernel writes to memory are rounded
to it; arithmetic inside an operator is double.
"""
import numpy as np

from . import oracle as O

RESNET_BLOCKS = {"resnet50": (3, 4, 6, 3), "resnet101": (3, 4, 23, 3), "resnet152": (3, 8, 36, 3)}
VGG16_CFG = (64, 64, -1, 128, 128, -1, 256, 256, 256, -1, 512, 512, 512, -1, 512, 512, 512, -1)


class _Ctx:
    def __init__(self, params, dt):
        self.params, self.dt = params, dt

    def R(self, a):
        return O.round_to(a, self.dt)

    def P(self, name):
        return O.round_to(self.params[name], self.dt)

    def conv(self, name, x, stride, pad, act, residual=None):
        return self.R(O.conv2d(x, self.P(name + ".weight"), self.P(name + ".bias"), stride, pad, residual, act))

    def dense(self, name, x, act=O.ACT_NONE, residual=None):
        return self.R(O.gemm_bias_act(x, self.P(name + ".weight"), self.P(name + ".bias"), residual, act, b_is_nk=True))


def resnet(params, x, blocks, dt="f32", logits=False):
    """ResNet v1, bottleneck blocks, stride on the first 1x1 of a down-sampling block, BN folded."""
    c = _Ctx(params, dt)
    x = c.R(x)
    x = c.conv("conv1", x, 2, 3, O.ACT_RELU)
    x = O.pool2d(x, 3, 2, 1, "max")
    for s in range(4):
        for b in range(blocks[s]):
            n = f"layer{s + 1}.{b}"
            stride = 2 if (b == 0 and s > 0) else 1
            shortcut = c.conv(n + ".downsample", x, stride, 0, O.ACT_NONE) if b == 0 else x
            y = c.conv(n + ".conv1", x, stride, 0, O.ACT_RELU)
            y = c.conv(n + ".conv2", y, 1, 1, O.ACT_RELU)
            x = c.conv(n + ".conv3", y, 1, 0, O.ACT_RELU, residual=shortcut)
    gap = c.R(O.global_avgpool(x))
    lg = c.dense("fc", gap)
    return (c.R(O.softmax(lg)), lg) if logits else c.R(O.softmax(lg))


def vgg16(params, x, dt="f16", wdiv=1, logits=False):
    c = _Ctx(params, dt)
    x = c.R(x)
    ci = 0
    for ch in VGG16_CFG:
        if ch < 0:
            x = O.pool2d(x, 2, 2, 0, "max")
        else:
            ci += 1
            x = c.conv(f"conv{ci}", x, 1, 1, O.ACT_RELU)
    x = x.reshape(x.shape[0], -1)  # NCHW flatten, as relay's batch_flatten
    x = c.dense("fc1", x, O.ACT_RELU)
    x = c.dense("fc2", x, O.ACT_RELU)
    lg = c.dense("fc3", x)
    return (c.R(O.softmax(lg)), lg) if logits else c.R(O.softmax(lg))


def densenet(params, x, dt="f16", blocks=(6, 12, 48, 32), growth=32, logits=False):
    c = _Ctx(params, dt)
    x = c.R(x)
    x = c.conv("conv0", x, 2, 3, O.ACT_RELU)
    x = O.pool2d(x, 3, 2, 1, "max")
    for b in range(4):
        for l in range(blocks[b]):
            n = f"block{b + 1}.layer{l + 1}"
            t = c.R(O.scale_shift_act(x, c.P(n + ".norm1.scale"), c.P(n + ".norm1.shift"), O.ACT_RELU))
            t = c.conv(n + ".conv1", t, 1, 0, O.ACT_RELU)
            t = c.conv(n + ".conv2", t, 1, 1, O.ACT_NONE)
            x = np.concatenate([x, t], axis=1)
        if b < 3:
            n = f"transition{b + 1}"
            t = c.R(O.scale_shift_act(x, c.P(n + ".norm.scale"), c.P(n + ".norm.shift"), O.ACT_RELU))
            t = c.conv(n + ".conv", t, 1, 0, O.ACT_NONE)
            x = c.R(O.pool2d(t, 2, 2, 0, "avg"))
    t = c.R(O.scale_shift_act(x, c.P("norm5.scale"), c.P("norm5.shift"), O.ACT_RELU))
    gap = c.R(O.global_avgpool(t))
    lg = c.dense("classifier", gap)
    return (c.R(O.softmax(lg)), lg) if logits else c.R(O.softmax(lg))


def inception_v3(params, x, dt="f16", logits=False):
    """Inception-v3 as relay.testing.inception_v3 lays it out: stem, 3 x A, B, 4 x C, D, 2 x E,
    global average pool, FC, softmax; every convolution with folded batch-norm and ReLU; average
    pools count their padding."""
    c = _Ctx(params, dt)

    def cv(name, t, stride=1, pad=0):
        return c.conv(name, t, stride, pad, O.ACT_RELU)

    x = c.R(x)
    x = cv("conv", x, 2)
    x = cv("conv_1", x)
    x = cv("conv_2", x, 1, 1)
    x = O.pool2d(x, 3, 2, 0, "max")
    x = cv("conv_3", x)
    x = cv("conv_4", x)
    x = O.pool2d(x, 3, 2, 0, "max")
    i = 0
    for _ in range(3):
        n = f"mixed{i}"
        i += 1
        b0 = cv(n + ".1x1", x)
        b1 = cv(n + ".5x5", cv(n + ".5x5_r", x), 1, 2)
        b2 = cv(n + ".3x3_2", cv(n + ".3x3_1", cv(n + ".3x3_r", x), 1, 1), 1, 1)
        b3 = cv(n + ".proj", c.R(O.pool2d(x, 3, 1, 1, "avg_pad")))
        x = np.concatenate([b0, b1, b2, b3], axis=1)
    n = f"mixed{i}"
    i += 1
    b0 = cv(n + ".3x3", x, 2)
    b1 = cv(n + ".d3x3_2", cv(n + ".d3x3_1", cv(n + ".d3x3_r", x), 1, 1), 2)
    x = np.concatenate([b0, b1, O.pool2d(x, 3, 2, 0, "max")], axis=1)
    for _ in range(4):
        n = f"mixed{i}"
        i += 1
        b0 = cv(n + ".1x1", x)
        b1 = cv(n + ".7_2", cv(n + ".7_1", cv(n + ".7_r", x), 1, (0, 3)), 1, (3, 0))
        t = cv(n + ".d7_r", x)
        t = cv(n + ".d7_1", t, 1, (3, 0))
        t = cv(n + ".d7_2", t, 1, (0, 3))
        t = cv(n + ".d7_3", t, 1, (3, 0))
        b2 = cv(n + ".d7_4", t, 1, (0, 3))
        b3 = cv(n + ".proj", c.R(O.pool2d(x, 3, 1, 1, "avg_pad")))
        x = np.concatenate([b0, b1, b2, b3], axis=1)
    n = f"mixed{i}"
    i += 1
    b0 = cv(n + ".3x3", cv(n + ".3x3_r", x), 2)
    t = cv(n + ".7x3_2", cv(n + ".7x3_1", cv(n + ".7x3_r", x), 1, (0, 3)), 1, (3, 0))
    b1 = cv(n + ".7x3_3", t, 2)
    x = np.concatenate([b0, b1, O.pool2d(x, 3, 2, 0, "max")], axis=1)
    for mode in ("avg_pad", "max"):
        n = f"mixed{i}"
        i += 1
        b0 = cv(n + ".1x1", x)
        t = cv(n + ".3_r", x)
        b1 = np.concatenate([cv(n + ".3_a", t, 1, (0, 1)), cv(n + ".3_b", t, 1, (1, 0))], axis=1)
        t = cv(n + ".d3_1", cv(n + ".d3_r", x), 1, 1)
        b2 = np.concatenate([cv(n + ".d3_a", t, 1, (0, 1)), cv(n + ".d3_b", t, 1, (1, 0))], axis=1)
        b3 = cv(n + ".proj", c.R(O.pool2d(x, 3, 1, 1, mode)))
        x = np.concatenate([b0, b1, b2, b3], axis=1)
    gap = c.R(O.global_avgpool(x))
    lg = c.dense("fc1", gap)
    return (c.R(O.softmax(lg)), lg) if logits else c.R(O.softmax(lg))


def bert(params, ids, dt="f16", batch=1, seq=128, layers=12, hidden=768, heads=12, fused_attention=None):
    """BERT encoder: embeddings + LayerNorm, then `layers` post-LN transformer blocks with
    erf GELU and eps 1e-12; returns the last hidden state [batch*seq, hidden].
    fused_attention (default: 16-bit dtypes): scores and probabilities are not rounded to the
    storage dtype between the two products, as in a kernel that never writes them out."""
    if fused_attention is None:
        fused_attention = dt != "f32"
    RA = (lambda a: a) if fused_attention else None
    c = _Ctx(params, dt)
    d = hidden // heads
    T = batch * seq
    x = c.R(O.embed(ids, c.P("embeddings.word"), c.P("embeddings.position"), c.P("embeddings.token_type")[0], seq))
    x = c.R(O.layernorm(x, c.P("embeddings.ln.gamma"), c.P("embeddings.ln.beta"), 1e-12))
    for l in range(layers):
        n = f"layer{l}"
        qkv = c.dense(n + ".attn.qkv", x)
        q, k, v = (qkv[:, i * hidden:(i + 1) * hidden].reshape(batch, seq, heads, d).transpose(0, 2, 1, 3).reshape(batch * heads, seq, d) for i in range(3))
        RS = RA or c.R
        scores = RS(O.bmm(q, k, alpha=1.0 / np.sqrt(d), b_is_nk=True))
        probs = RS(O.softmax(scores))
        ctxv = c.R(O.bmm(probs, v))
        ctxv = ctxv.reshape(batch, heads, seq, d).transpose(0, 2, 1, 3).reshape(T, hidden)
        ao = c.dense(n + ".attn.proj", ctxv, residual=x)
        x1 = c.R(O.layernorm(ao, c.P(n + ".ln1.gamma"), c.P(n + ".ln1.beta"), 1e-12))
        f1 = c.dense(n + ".ffn1", x1, O.ACT_GELU)
        f2 = c.dense(n + ".ffn2", f1, residual=x1)
        x = c.R(O.layernorm(f2, c.P(n + ".ln2.gamma"), c.P(n + ".ln2.beta"), 1e-12))
    return x


def random_params(shapes, seed, family):
    """Seeded parameters for `shapes` = {name: disk shape}.  Convolutions and dense layers of the
    vision models are He-normal (std = sqrt(2 / fan_in)); BERT matrices are N(0, 0.02); biases
    are small but non-zero and norm scales are near 1 so that a dropped term would show."""
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in shapes.items():
        if name.endswith(".weight") or name.startswith("embeddings.") and not name.startswith("embeddings.ln"):
            if family == "bert":
                out[name] = rng.normal(0, 0.02, shape).astype(np.float32)
            else:
                fan_in = int(np.prod(shape[1:]))
                # the convolution that closes a residual block is scaled down (a folded
                # batch-norm with a small gamma), otherwise 50 un-normalised residual adds
                # overflow fp16
                gain = 0.2 if name.endswith("conv3.weight") else 1.0
                out[name] = rng.normal(0, gain * np.sqrt(2.0 / fan_in), shape).astype(np.float32)
        elif name.endswith(".scale") or name.endswith(".gamma"):
            out[name] = rng.uniform(0.8, 1.2, shape).astype(np.float32)
        elif name == "B":
            out[name] = rng.uniform(-1, 1, shape).astype(np.float32)
        else:  # bias, shift, beta
            out[name] = rng.uniform(-0.1, 0.1, shape).astype(np.float32)
    return out
