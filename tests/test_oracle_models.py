"""Pins the composition of the oracle's model graphs against torch.nn.functional on CPU (fp32
storage, small variants of the same builders), so that a mis-wired residual, a wrong stride
placement or a swapped attention operand fails."""
import numpy as np
import torch
import torch.nn.functional as F

from oracle import models as OM


def T(a):
    return torch.from_numpy(np.asarray(a, np.float32)).double()


def resnet_shapes(blocks, width=8, classes=10):
    s = {"conv1.weight": (width, 3, 7, 7), "conv1.bias": (width,)}
    cin = width
    for st in range(4):
        w = width << st
        for b in range(blocks[st]):
            n = f"layer{st + 1}.{b}"
            if b == 0:
                s[n + ".downsample.weight"] = (4 * w, cin, 1, 1); s[n + ".downsample.bias"] = (4 * w,)
            s[n + ".conv1.weight"] = (w, cin, 1, 1); s[n + ".conv1.bias"] = (w,)
            s[n + ".conv2.weight"] = (w, w, 3, 3); s[n + ".conv2.bias"] = (w,)
            s[n + ".conv3.weight"] = (4 * w, w, 1, 1); s[n + ".conv3.bias"] = (4 * w,)
            cin = 4 * w
    s["fc.weight"] = (classes, cin); s["fc.bias"] = (classes,)
    return s


def test_resnet_composition_vs_torch():
    blocks = (2, 1, 2, 1)
    p = OM.random_params(resnet_shapes(blocks), 1, "cnn")
    x = np.random.default_rng(2).normal(size=(2, 3, 40, 40)).astype(np.float32)
    got = OM.resnet(p, x, blocks, "f32")
    c = lambda n, t, s, pad: F.conv2d(t, T(p[n + ".weight"]), T(p[n + ".bias"]), s, pad)
    t = F.relu(c("conv1", T(x), 2, 3))
    t = F.max_pool2d(t, 3, 2, 1)
    for st in range(4):
        for b in range(blocks[st]):
            n = f"layer{st + 1}.{b}"
            stride = 2 if (b == 0 and st > 0) else 1
            sc = c(n + ".downsample", t, stride, 0) if b == 0 else t
            y = F.relu(c(n + ".conv1", t, stride, 0))
            y = F.relu(c(n + ".conv2", y, 1, 1))
            t = F.relu(c(n + ".conv3", y, 1, 0) + sc)
    t = t.mean(dim=(2, 3))
    t = torch.softmax(t @ T(p["fc.weight"]).T + T(p["fc.bias"]), 1).numpy()
    assert np.abs(got - t).max() / np.abs(t).max() < 1e-4


def test_bert_composition_vs_torch():
    Hd, heads, F_, L, S, B, V = 32, 4, 64, 2, 6, 2, 50
    shapes = {"embeddings.word": (V, Hd), "embeddings.position": (16, Hd), "embeddings.token_type": (1, Hd),
              "embeddings.ln.gamma": (Hd,), "embeddings.ln.beta": (Hd,)}
    for l in range(L):
        n = f"layer{l}"
        shapes.update({n + ".attn.qkv.weight": (3 * Hd, Hd), n + ".attn.qkv.bias": (3 * Hd,), n + ".attn.proj.weight": (Hd, Hd),
                       n + ".attn.proj.bias": (Hd,), n + ".ln1.gamma": (Hd,), n + ".ln1.beta": (Hd,), n + ".ffn1.weight": (F_, Hd),
                       n + ".ffn1.bias": (F_,), n + ".ffn2.weight": (Hd, F_), n + ".ffn2.bias": (Hd,), n + ".ln2.gamma": (Hd,), n + ".ln2.beta": (Hd,)})
    p = OM.random_params(shapes, 3, "bert")
    for k in p:
        if k.endswith(".weight"):
            p[k] = (p[k] * 10).astype(np.float32)  # make attention non-uniform so operand order matters
    ids = np.random.default_rng(4).integers(0, V, B * S)
    got = OM.bert(p, ids, "f32", B, S, L, Hd, heads)
    d = Hd // heads
    x = T(p["embeddings.word"])[ids] + T(p["embeddings.position"])[torch.arange(B * S) % S] + T(p["embeddings.token_type"])[0]
    ln = lambda t, n: F.layer_norm(t, (Hd,), T(p[n + ".gamma"]), T(p[n + ".beta"]), 1e-12)
    x = ln(x, "embeddings.ln")
    for l in range(L):
        n = f"layer{l}"
        qkv = x @ T(p[n + ".attn.qkv.weight"]).T + T(p[n + ".attn.qkv.bias"])
        q, k, v = (qkv[:, i * Hd:(i + 1) * Hd].reshape(B, S, heads, d).permute(0, 2, 1, 3) for i in range(3))
        a = torch.softmax(q @ k.transpose(-1, -2) / np.sqrt(d), -1) @ v
        a = a.permute(0, 2, 1, 3).reshape(B * S, Hd)
        x = ln(a @ T(p[n + ".attn.proj.weight"]).T + T(p[n + ".attn.proj.bias"]) + x, n + ".ln1")
        f = F.gelu(x @ T(p[n + ".ffn1.weight"]).T + T(p[n + ".ffn1.bias"]))
        x = ln(f @ T(p[n + ".ffn2.weight"]).T + T(p[n + ".ffn2.bias"]) + x, n + ".ln2")
    assert np.abs(got - x.numpy()).max() / np.abs(x.numpy()).max() < 1e-4


def test_vgg_and_densenet_composition_vs_torch():
    rng = np.random.default_rng(5)
    # VGG-16 at width/8 on a 32x32 image
    shapes, cin, ci = {}, 3, 0
    for ch in OM.VGG16_CFG:
        if ch > 0:
            ci += 1
            shapes[f"conv{ci}.weight"] = (ch // 8, cin, 3, 3); shapes[f"conv{ci}.bias"] = (ch // 8,)
            cin = ch // 8
    shapes.update({"fc1.weight": (32, cin), "fc1.bias": (32,), "fc2.weight": (32, 32), "fc2.bias": (32,), "fc3.weight": (10, 32), "fc3.bias": (10,)})
    p = OM.random_params(shapes, 6, "cnn")
    x = rng.normal(size=(2, 3, 32, 32)).astype(np.float32)
    got = OM.vgg16(p, x, "f32")
    t, ci = T(x), 0
    for ch in OM.VGG16_CFG:
        if ch < 0:
            t = F.max_pool2d(t, 2, 2)
        else:
            ci += 1
            t = F.relu(F.conv2d(t, T(p[f"conv{ci}.weight"]), T(p[f"conv{ci}.bias"]), 1, 1))
    t = t.flatten(1)
    for i, act in ((1, True), (2, True), (3, False)):
        t = t @ T(p[f"fc{i}.weight"]).T + T(p[f"fc{i}.bias"])
        if act:
            t = F.relu(t)
    assert np.abs(got - torch.softmax(t, 1).numpy()).max() < 1e-5

    # DenseNet with blocks (2,2,1,1), growth 4
    blocks, growth, C = (2, 2, 1, 1), 4, 8
    shapes = {"conv0.weight": (C, 3, 7, 7), "conv0.bias": (C,)}
    for b in range(4):
        for l in range(blocks[b]):
            n = f"block{b + 1}.layer{l + 1}"
            shapes.update({n + ".norm1.scale": (C,), n + ".norm1.shift": (C,), n + ".conv1.weight": (4 * growth, C, 1, 1), n + ".conv1.bias": (4 * growth,),
                           n + ".conv2.weight": (growth, 4 * growth, 3, 3), n + ".conv2.bias": (growth,)})
            C += growth
        if b < 3:
            n = f"transition{b + 1}"
            shapes.update({n + ".norm.scale": (C,), n + ".norm.shift": (C,), n + ".conv.weight": (C // 2, C, 1, 1), n + ".conv.bias": (C // 2,)})
            C //= 2
    shapes.update({"norm5.scale": (C,), "norm5.shift": (C,), "classifier.weight": (10, C), "classifier.bias": (10,)})
    p = OM.random_params(shapes, 7, "cnn")
    x = rng.normal(size=(1, 3, 64, 64)).astype(np.float32)
    got = OM.densenet(p, x, "f32", blocks, growth)
    aff = lambda t, n: F.relu(t * T(p[n + ".scale"])[None, :, None, None] + T(p[n + ".shift"])[None, :, None, None])
    t = F.max_pool2d(F.relu(F.conv2d(T(x), T(p["conv0.weight"]), T(p["conv0.bias"]), 2, 3)), 3, 2, 1)
    for b in range(4):
        for l in range(blocks[b]):
            n = f"block{b + 1}.layer{l + 1}"
            y = F.relu(F.conv2d(aff(t, n + ".norm1"), T(p[n + ".conv1.weight"]), T(p[n + ".conv1.bias"])))
            y = F.conv2d(y, T(p[n + ".conv2.weight"]), T(p[n + ".conv2.bias"]), 1, 1)
            t = torch.cat([t, y], 1)
        if b < 3:
            n = f"transition{b + 1}"
            t = F.avg_pool2d(F.conv2d(aff(t, n + ".norm"), T(p[n + ".conv.weight"]), T(p[n + ".conv.bias"])), 2, 2)
    t = aff(t, "norm5").mean(dim=(2, 3))
    t = torch.softmax(t @ T(p["classifier.weight"]).T + T(p["classifier.bias"]), 1).numpy()
    assert np.abs(got - t).max() < 1e-5


def test_inception_v3_composition_vs_torch():
    """Inception-v3 (stem, 3 x A, B, 4 x C, D, 2 x E; TVM's relay.testing.inception_v3 layout) at an
    eighth of the widths on a 107 x 107 image, against torch.nn.functional: branch order inside each
    concatenation, the (kh, kw) / padding pairs of the factorised 7 x 7 and 3 x 3 filters, strides
    of the reducing blocks and which pools count their padding."""
    W8 = lambda c: max(c // 8, 1)
    shapes = {}

    def conv(name, cin, cout, kh=1, kw=1):
        shapes[name + ".weight"] = (cout, cin, kh, kw)
        shapes[name + ".bias"] = (cout,)
        return cout

    c = conv("conv", 3, W8(32), 3, 3)
    c = conv("conv_1", c, W8(32), 3, 3)
    c = conv("conv_2", c, W8(64), 3, 3)
    c = conv("conv_3", c, W8(80))
    c = conv("conv_4", c, W8(192), 3, 3)
    i = 0
    for proj in (32, 64, 64):
        n = f"mixed{i}"; i += 1
        o = conv(n + ".1x1", c, W8(64))
        t = conv(n + ".5x5_r", c, W8(48)); o += conv(n + ".5x5", t, W8(64), 5, 5)
        t = conv(n + ".3x3_r", c, W8(64)); t = conv(n + ".3x3_1", t, W8(96), 3, 3); o += conv(n + ".3x3_2", t, W8(96), 3, 3)
        o += conv(n + ".proj", c, W8(proj))
        c = o
    n = f"mixed{i}"; i += 1
    o = conv(n + ".3x3", c, W8(384), 3, 3)
    t = conv(n + ".d3x3_r", c, W8(64)); t = conv(n + ".d3x3_1", t, W8(96), 3, 3); o += conv(n + ".d3x3_2", t, W8(96), 3, 3)
    c = o + c
    for c7 in (128, 160, 160, 192):
        n = f"mixed{i}"; i += 1
        o = conv(n + ".1x1", c, W8(192))
        t = conv(n + ".7_r", c, W8(c7)); t = conv(n + ".7_1", t, W8(c7), 1, 7); o += conv(n + ".7_2", t, W8(192), 7, 1)
        t = conv(n + ".d7_r", c, W8(c7)); t = conv(n + ".d7_1", t, W8(c7), 7, 1); t = conv(n + ".d7_2", t, W8(c7), 1, 7)
        t = conv(n + ".d7_3", t, W8(c7), 7, 1); o += conv(n + ".d7_4", t, W8(192), 1, 7)
        o += conv(n + ".proj", c, W8(192))
        c = o
    n = f"mixed{i}"; i += 1
    t = conv(n + ".3x3_r", c, W8(192)); o = conv(n + ".3x3", t, W8(320), 3, 3)
    t = conv(n + ".7x3_r", c, W8(192)); t = conv(n + ".7x3_1", t, W8(192), 1, 7); t = conv(n + ".7x3_2", t, W8(192), 7, 1)
    o += conv(n + ".7x3_3", t, W8(192), 3, 3)
    c = o + c
    for _ in range(2):
        n = f"mixed{i}"; i += 1
        o = conv(n + ".1x1", c, W8(320))
        t = conv(n + ".3_r", c, W8(384)); o += conv(n + ".3_a", t, W8(384), 1, 3) + conv(n + ".3_b", t, W8(384), 3, 1)
        t = conv(n + ".d3_r", c, W8(448)); t = conv(n + ".d3_1", t, W8(384), 3, 3)
        o += conv(n + ".d3_a", t, W8(384), 1, 3) + conv(n + ".d3_b", t, W8(384), 3, 1)
        o += conv(n + ".proj", c, W8(192))
        c = o
    shapes["fc1.weight"] = (10, c); shapes["fc1.bias"] = (10,)
    p = OM.random_params(shapes, 11, "cnn")
    x = np.random.default_rng(12).normal(size=(2, 3, 107, 107)).astype(np.float32)
    got = OM.inception_v3(p, x, "f32")

    def cv(name, t, stride=1, pad=0):
        return F.relu(F.conv2d(t, T(p[name + ".weight"]), T(p[name + ".bias"]), stride, pad))

    avg = lambda t: F.avg_pool2d(t, 3, 1, 1, count_include_pad=True)
    t = cv("conv", T(x), 2)
    t = cv("conv_1", t)
    t = cv("conv_2", t, 1, 1)
    t = F.max_pool2d(t, 3, 2)
    t = cv("conv_3", t)
    t = cv("conv_4", t)
    t = F.max_pool2d(t, 3, 2)
    assert t.shape[2] == 11
    for k in range(3):  # A blocks: 1x1 | 1x1-5x5 | 1x1-3x3-3x3 | avgpool-1x1
        n = f"mixed{k}"
        t = torch.cat([cv(n + ".1x1", t), cv(n + ".5x5", cv(n + ".5x5_r", t), 1, 2),
                       cv(n + ".3x3_2", cv(n + ".3x3_1", cv(n + ".3x3_r", t), 1, 1), 1, 1), cv(n + ".proj", avg(t))], 1)
    n = "mixed3"  # B: 3x3/2 | 1x1-3x3-3x3/2 | maxpool/2
    t = torch.cat([cv(n + ".3x3", t, 2), cv(n + ".d3x3_2", cv(n + ".d3x3_1", cv(n + ".d3x3_r", t), 1, 1), 2), F.max_pool2d(t, 3, 2)], 1)
    assert t.shape[2] == 5
    for k in range(4, 8):  # C blocks: 1x1 | 1x1-1x7-7x1 | 1x1-7x1-1x7-7x1-1x7 | avgpool-1x1
        n = f"mixed{k}"
        b1 = cv(n + ".7_2", cv(n + ".7_1", cv(n + ".7_r", t), 1, (0, 3)), 1, (3, 0))
        b2 = cv(n + ".d7_r", t)
        b2 = cv(n + ".d7_1", b2, 1, (3, 0)); b2 = cv(n + ".d7_2", b2, 1, (0, 3)); b2 = cv(n + ".d7_3", b2, 1, (3, 0)); b2 = cv(n + ".d7_4", b2, 1, (0, 3))
        t = torch.cat([cv(n + ".1x1", t), b1, b2, cv(n + ".proj", avg(t))], 1)
    n = "mixed8"  # D: 1x1-3x3/2 | 1x1-1x7-7x1-3x3/2 | maxpool/2
    b1 = cv(n + ".7x3_3", cv(n + ".7x3_2", cv(n + ".7x3_1", cv(n + ".7x3_r", t), 1, (0, 3)), 1, (3, 0)), 2)
    t = torch.cat([cv(n + ".3x3", cv(n + ".3x3_r", t), 2), b1, F.max_pool2d(t, 3, 2)], 1)
    assert t.shape[2] == 2
    for k, pool in ((9, avg), (10, lambda u: F.max_pool2d(u, 3, 1, 1))):  # E blocks
        n = f"mixed{k}"
        u = cv(n + ".3_r", t)
        v = cv(n + ".d3_1", cv(n + ".d3_r", t), 1, 1)
        t = torch.cat([cv(n + ".1x1", t), cv(n + ".3_a", u, 1, (0, 1)), cv(n + ".3_b", u, 1, (1, 0)),
                       cv(n + ".d3_a", v, 1, (0, 1)), cv(n + ".d3_b", v, 1, (1, 0)), cv(n + ".proj", pool(t))], 1)
    t = t.mean(dim=(2, 3))
    want = torch.softmax(t @ T(p["fc1.weight"]).T + T(p["fc1.bias"]), 1).numpy()
    assert np.abs(got - want).max() / np.abs(want).max() < 1e-4
