"""Pins the CPU oracle's operators against what the mathematics fixes: closed forms, brute
force on tiny shapes, invariants, and library routines (numpy, torch on CPU).  Each check is
chosen so that a plausible slip (dropped bias, transposed operand, wrong stride/pad index,
biased-vs-unbiased variance, tanh-vs-erf GELU) fails it."""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import oracle as O


def rng(seed=0):
    return np.random.default_rng(seed)


def test_gemm_closed_forms():
    r = rng(1)
    A = r.uniform(-1, 1, (7, 5)).astype(np.float32)
    B = r.uniform(-1, 1, (5, 3)).astype(np.float32)
    bias = r.uniform(-1, 1, 3).astype(np.float32)
    res = r.uniform(-1, 1, (7, 3)).astype(np.float32)
    want = A.astype(np.float64) @ B + bias + res
    assert np.allclose(O.gemm_bias_act(A, B, bias, res), want, atol=1e-6)
    assert np.allclose(O.gemm_bias_act(A, B.T.copy(), bias, res, b_is_nk=True), want, atol=1e-6)  # transposed layout
    assert np.array_equal(O.gemm_bias_act(A, B, bias, res, O.ACT_RELU), np.maximum(want, 0).astype(np.float32))
    # identity / permutation / all-ones
    X = r.uniform(-1, 1, (6, 6)).astype(np.float32)
    assert np.array_equal(O.gemm_bias_act(np.eye(6, dtype=np.float32), X), X)
    p = r.permutation(6)
    assert np.array_equal(O.gemm_bias_act(np.eye(6, dtype=np.float32)[p], X), X[p])
    assert np.array_equal(O.gemm_bias_act(np.ones((4, 9), np.float32), np.ones((9, 2), np.float32)), np.full((4, 2), 9, np.float32))
    # non-square so that a swapped M/N or lda/ldb cannot pass
    assert O.gemm_bias_act(A, B).shape == (7, 3)


def test_bmm_matches_einsum():
    r = rng(2)
    A = r.normal(size=(3, 4, 5)).astype(np.float32)
    B = r.normal(size=(3, 5, 6)).astype(np.float32)
    assert np.allclose(O.bmm(A, B, 0.5), 0.5 * np.einsum("bmk,bkn->bmn", A.astype(np.float64), B), atol=1e-6)
    Bt = np.ascontiguousarray(B.transpose(0, 2, 1))
    assert np.allclose(O.bmm(A, Bt, 0.5, b_is_nk=True), 0.5 * np.einsum("bmk,bkn->bmn", A.astype(np.float64), B), atol=1e-6)


def brute_conv(x, w, b, stride, pad):
    N, C, H, W = x.shape
    Co, _, R, S = w.shape
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    out = np.zeros((N, Co, Ho, Wo))
    for n in range(N):
        for co in range(Co):
            for ho in range(Ho):
                for wo in range(Wo):
                    s = b[co]
                    for ci in range(C):
                        for r_ in range(R):
                            for s_ in range(S):
                                hi, wi = ho * stride - pad + r_, wo * stride - pad + s_
                                if 0 <= hi < H and 0 <= wi < W:
                                    s += float(x[n, ci, hi, wi]) * float(w[co, ci, r_, s_])
                    out[n, co, ho, wo] = s
    return out


@pytest.mark.parametrize("cfg", [(1, 2, 5, 6, 3, 3, 1, 1), (2, 3, 7, 5, 2, 3, 2, 1), (1, 1, 4, 4, 1, 1, 2, 0), (1, 2, 6, 6, 2, 5, 1, 2)])
def test_conv_brute_force_and_torch(cfg):
    N, C, H, W, Co, k, stride, pad = cfg
    r = rng(sum(cfg))
    x = r.normal(size=(N, C, H, W)).astype(np.float32)
    w = r.normal(size=(Co, C, k, k)).astype(np.float32)
    b = r.normal(size=Co).astype(np.float32)
    got = O.conv2d(x, w, b, stride, pad)
    assert np.allclose(got, brute_conv(x, w, b, stride, pad), atol=1e-5)
    t = F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(), stride, pad).numpy()
    assert np.allclose(got, t, atol=1e-5)


def test_conv_1x1_is_gemm_and_epilogue_order():
    r = rng(5)
    x = r.normal(size=(2, 8, 3, 3)).astype(np.float32)
    w = r.normal(size=(4, 8, 1, 1)).astype(np.float32)
    b = r.normal(size=4).astype(np.float32)
    res = r.normal(size=(2, 4, 3, 3)).astype(np.float32)
    g = O.gemm_bias_act(x.transpose(0, 2, 3, 1).reshape(-1, 8), w.reshape(4, 8), b, b_is_nk=True).reshape(2, 3, 3, 4).transpose(0, 3, 1, 2)
    assert np.allclose(O.conv2d(x, w, b), g, atol=1e-6)
    # residual is added BEFORE the activation
    want = np.maximum(O.conv2d(x, w, b).astype(np.float64) + res, 0)
    assert np.allclose(O.conv2d(x, w, b, residual=res, act=O.ACT_RELU), want, atol=1e-6)


def test_pooling_vs_torch():
    r = rng(6)
    x = r.normal(size=(2, 3, 9, 8)).astype(np.float32)
    tx = torch.from_numpy(x)
    assert np.array_equal(O.pool2d(x, 3, 2, 1, "max"), F.max_pool2d(tx, 3, 2, 1).numpy())
    assert np.array_equal(O.pool2d(x, 2, 2, 0, "max"), F.max_pool2d(tx, 2, 2, 0).numpy())
    assert np.allclose(O.pool2d(x, 2, 2, 0, "avg"), F.avg_pool2d(tx, 2, 2, 0).numpy(), atol=1e-6)
    assert np.allclose(O.pool2d(x, 3, 1, 1, "avg"), F.avg_pool2d(tx, 3, 1, 1, count_include_pad=False).numpy(), atol=1e-6)
    assert np.allclose(O.pool2d(x, 3, 1, 1, "avg_pad"), F.avg_pool2d(tx, 3, 1, 1, count_include_pad=True).numpy(), atol=1e-6)
    assert np.allclose(O.global_avgpool(x), x.mean(axis=(2, 3)), atol=1e-6)
    # all-negative input: padding must never win a max
    assert (O.pool2d(-np.abs(x) - 1, 3, 2, 1, "max") < 0).all()


def test_softmax_layernorm_gelu_identities():
    r = rng(7)
    x = r.normal(size=(5, 33)).astype(np.float32) * 4
    s = O.softmax(x)
    assert np.allclose(s.sum(axis=1), 1, atol=1e-6)
    assert np.allclose(s, torch.softmax(torch.from_numpy(x).double(), 1).numpy(), atol=1e-7)
    assert np.allclose(O.softmax(x + 100), s, atol=1e-6)  # shift invariance (max subtraction)
    g, b = r.uniform(0.5, 1.5, 33).astype(np.float32), r.normal(size=33).astype(np.float32)
    ln = O.layernorm(x, np.ones(33, np.float32), np.zeros(33, np.float32), 0.0)
    assert np.allclose(ln.mean(axis=1), 0, atol=1e-6) and np.allclose(ln.var(axis=1), 1, atol=1e-5)  # biased variance
    t = F.layer_norm(torch.from_numpy(x).double(), (33,), torch.from_numpy(g).double(), torch.from_numpy(b).double(), 1e-12).numpy()
    assert np.allclose(O.layernorm(x, g, b, 1e-12), t, atol=1e-5)
    assert np.allclose(O.layernorm(x, g, b, 1e-12, residual=x), O.layernorm(2 * x, g, b, 1e-12), atol=1e-5)
    # erf GELU (not the tanh approximation): GELU(0)=0, GELU(x)-GELU(-x)=x, matches torch's exact form
    v = np.linspace(-4, 4, 41).astype(np.float32)
    ge = O.add_act(v, None, O.ACT_GELU)
    assert ge[20] == 0 and np.allclose(ge - ge[::-1], v, atol=1e-6)
    assert np.allclose(ge, F.gelu(torch.from_numpy(v).double()).numpy(), atol=1e-7)
    assert np.abs(ge - F.gelu(torch.from_numpy(v), approximate="tanh").numpy()).max() > 1e-4


def test_embed_and_scale_shift():
    r = rng(8)
    tok, pos, seg = r.normal(size=(10, 4)).astype(np.float32), r.normal(size=(3, 4)).astype(np.float32), r.normal(size=4).astype(np.float32)
    ids = np.array([9, 0, 3, 3, 1, 7])
    want = tok[ids] + pos[np.arange(6) % 3] + seg
    assert np.allclose(O.embed(ids, tok, pos, seg, 3), want, atol=1e-6)
    x = r.normal(size=(2, 3, 2, 2)).astype(np.float32)
    sc, sh = np.array([1, 2, 3], np.float32), np.array([0.5, -0.5, 0], np.float32)
    assert np.allclose(O.scale_shift_act(x, sc, sh, O.ACT_RELU), np.maximum(x * sc[None, :, None, None] + sh[None, :, None, None], 0), atol=1e-6)


def test_bn_fold_equals_conv_then_bn():
    r = rng(9)
    x = r.normal(size=(1, 3, 6, 6)).astype(np.float32)
    w = r.normal(size=(4, 3, 3, 3)).astype(np.float32)
    b = r.normal(size=4).astype(np.float32)
    gamma, beta = r.uniform(0.5, 2, 4).astype(np.float32), r.normal(size=4).astype(np.float32)
    mean, var = r.normal(size=4).astype(np.float32), r.uniform(0.5, 2, 4).astype(np.float32)
    y = O.conv2d(x, w, b, 1, 1)
    bn = (y - mean[None, :, None, None]) / np.sqrt(var[None, :, None, None] + 1e-5) * gamma[None, :, None, None] + beta[None, :, None, None]
    w2, b2 = O.fold_bn(w, b, gamma, beta, mean, var, 1e-5)
    assert np.allclose(O.conv2d(x, w2, b2, 1, 1), bn, atol=1e-5)
    tb = F.batch_norm(torch.from_numpy(y), torch.from_numpy(mean), torch.from_numpy(var), torch.from_numpy(gamma), torch.from_numpy(beta), False, 0.0, 1e-5).numpy()
    assert np.allclose(bn, tb, atol=1e-5)


def test_rounding_matches_library_types():
    r = rng(10)
    x = np.concatenate([r.normal(size=1000) * 10.0 ** r.integers(-6, 6, 1000), [0.0, -0.0, 1.0, 65504.0]]).astype(np.float32)
    assert np.array_equal(O.round_bf16(x), torch.from_numpy(x).to(torch.bfloat16).float().numpy())
    assert np.array_equal(O.round_f16(x), torch.from_numpy(x).to(torch.float16).float().numpy())


def test_conv_with_a_1x7_and_a_7x1_filter_vs_torch():
    r = rng(11)
    x = r.normal(size=(1, 5, 9, 10)).astype(np.float32)
    for (kh, kw, ph, pw) in ((1, 7, 0, 3), (7, 1, 3, 0), (1, 3, 0, 1), (3, 1, 1, 0)):
        w = r.normal(size=(4, 5, kh, kw)).astype(np.float32)
        b = r.normal(size=4).astype(np.float32)
        got = O.conv2d(x, w, b, 1, (ph, pw), None, O.ACT_RELU)
        t = F.relu(F.conv2d(torch.from_numpy(x).double(), torch.from_numpy(w).double(), torch.from_numpy(b).double(), 1, (ph, pw))).numpy()
        assert got.shape == (1, 4, 9, 10) and np.allclose(got, t, atol=1e-5)
