"""Pins the CPU executor (oracle/oracle_exec.c + oracle/cpu_executor.py: the cpu_baseline of
bench.py) against the layer-by-layer compositions of oracle/models.py, and its preempt/resume
against the uninterrupted run bit for bit (the memcmp criterion of the reference's
src/cuda-clients/blp_resume_test.cpp:60-118).  CPU only."""
import numpy as np
import pytest

from oracle import cpu_executor as X
from oracle import models as OM
from oracle import oracle as O
from test_oracle_models import resnet_shapes

TOL = 2e-4  # fp32 accumulation in the executor against double accumulation in the oracle


def bert_shapes(Hd, F_, L, V, P):
    s = {"embeddings.word": (V, Hd), "embeddings.position": (P, Hd), "embeddings.token_type": (1, Hd), "embeddings.ln.gamma": (Hd,), "embeddings.ln.beta": (Hd,)}
    for l in range(L):
        n = f"layer{l}"
        s.update({n + ".attn.qkv.weight": (3 * Hd, Hd), n + ".attn.qkv.bias": (3 * Hd,), n + ".attn.proj.weight": (Hd, Hd), n + ".attn.proj.bias": (Hd,),
                  n + ".ln1.gamma": (Hd,), n + ".ln1.beta": (Hd,), n + ".ffn1.weight": (F_, Hd), n + ".ffn1.bias": (F_,), n + ".ffn2.weight": (Hd, F_),
                  n + ".ffn2.bias": (Hd,), n + ".ln2.gamma": (Hd,), n + ".ln2.beta": (Hd,)})
    return s


def rel(got, ref):
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


@pytest.mark.parametrize("M,N,K,act", [(100, 72, 40, O.ACT_RELU), (16, 64, 8, O.ACT_NONE), (33, 130, 257, O.ACT_GELU), (1, 5, 3, O.ACT_NONE)])
def test_gemm_matches_oracle(M, N, K, act):
    rng = np.random.default_rng(M * 7 + N)
    A, B, bias = rng.uniform(-1, 1, (M, K)).astype(np.float32), rng.uniform(-1, 1, (K, N)).astype(np.float32), rng.uniform(-1, 1, N).astype(np.float32)
    g, out = X.gemm_graph(A, B, bias, act)
    g.run(threads=3)
    assert rel(out, O.gemm_bias_act(A, B, bias, None, act)) < TOL


def test_bert_matches_oracle_composition():
    Hd, heads, F_, L, S, B, V = 32, 4, 64, 2, 20, 2, 50
    p = OM.random_params(bert_shapes(Hd, F_, L, V, 32), 3, "bert")
    for k in p:
        if k.endswith(".weight"):
            p[k] = (p[k] * 10).astype(np.float32)  # non-uniform attention, so that the operand order matters
    ids = np.random.default_rng(4).integers(0, V, B * S)
    g, out = X.bert_graph(p, ids, B, S, L, Hd, heads)
    g.run(threads=4)
    assert rel(out, OM.bert(p, ids, "f32", B, S, L, Hd, heads)) < TOL
    assert len(g.layers) == 2 + 7 * L


def test_resnet_matches_oracle_composition():
    blocks = (2, 1, 2, 1)
    p = OM.random_params(resnet_shapes(blocks), 1, "cnn")
    x = np.random.default_rng(2).normal(size=(2, 3, 40, 40)).astype(np.float32)
    g, out = X.resnet_graph(p, x, blocks)
    g.run(threads=4)
    assert rel(out, OM.resnet(p, x, blocks, "f32")) < TOL


def test_thread_count_does_not_change_the_bits():
    rng = np.random.default_rng(0)
    A, B, bias = rng.uniform(-1, 1, (70, 90)).astype(np.float32), rng.uniform(-1, 1, (90, 200)).astype(np.float32), np.zeros(200, np.float32)
    outs = []
    for t in (1, 2, 5):
        g, out = X.gemm_graph(A, B, bias)
        g.run(threads=t)
        outs.append(out.copy())
    assert outs[0].tobytes() == outs[1].tobytes() == outs[2].tobytes()


@pytest.mark.parametrize("frac", [0.0, 0.25, 0.5, 0.75, 1.0])
def test_gemm_preempt_resume_is_bit_exact(frac):
    rng = np.random.default_rng(5)
    A, B, bias = rng.uniform(-1, 1, (200, 64)).astype(np.float32), rng.uniform(-1, 1, (64, 300)).astype(np.float32), rng.uniform(-1, 1, 300).astype(np.float32)
    g0, ref = X.gemm_graph(A, B, bias)
    g0.run(threads=4)
    g, out = X.gemm_graph(A, B, bias)
    tiles = g.tiles()[0]
    stop, claims = g.run_preempted(0, int(frac * tiles), threads=4)
    assert stop == (0 if frac < 1.0 else -1)  # a claim index past the last tile never comes up
    assert int(frac * tiles) <= claims[0] <= tiles + 4  # every worker may over-claim once at the end
    assert out.tobytes() == ref.tobytes()


def test_bert_preempted_mid_graph_resumes_bit_exact():
    Hd, heads, F_, L, S, B, V = 32, 4, 64, 2, 24, 1, 50
    p = OM.random_params(bert_shapes(Hd, F_, L, V, 32), 9, "bert")
    ids = np.random.default_rng(1).integers(0, V, B * S)
    g0, ref = X.bert_graph(p, ids, B, S, L, Hd, heads)
    g0.run(threads=4)
    for kernel in (0, 3, 9, len(g0.layers) - 1):
        g, out = X.bert_graph(p, ids, B, S, L, Hd, heads)
        stop, claims = g.run_preempted(kernel, 1, threads=4)
        assert stop == kernel
        assert (claims[kernel + 1:] == 0).all()  # nothing after the stopped kernel had started
        assert out.tobytes() == ref.tobytes()
