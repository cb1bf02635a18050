"""Pins the graph oracle (oracle/graphs.py) against library routines: scipy's breadth-first
distances, weakly connected components and Dijkstra, and the linear system PageRank converges to.
Also checks the graph file format written by the host library (reference
src/workloads/graphcompute.cu:16-45) without touching a GPU."""
import ctypes as C
import os

import numpy as np
import pytest
import scipy.sparse as sp
import scipy.sparse.csgraph as csg

from oracle import graphs as G


def random_graph(n, deg, seed, components=1):
    """symmetric random graph in CSR; `components` disjoint blocks of vertices"""
    rng = np.random.default_rng(seed)
    block = n // components
    src = np.repeat(np.arange(n), deg)
    dst = (src // block) * block + rng.integers(0, block, src.size)
    dst = np.minimum(dst, n - 1)
    keep = src != dst
    src, dst = src[keep], dst[keep]
    w = rng.integers(1, 65, src.size).astype(np.uint32)
    a = np.concatenate([src, dst])
    b = np.concatenate([dst, src])
    ww = np.concatenate([w, w])
    order = np.lexsort((b, a))
    a, b, ww = a[order], b[order], ww[order]
    indptr = np.zeros(n + 1, np.int64)
    np.add.at(indptr, a + 1, 1)
    return np.cumsum(indptr), b.astype(np.int64), ww


def to_scipy(indptr, indices, w=None):
    n = len(indptr) - 1
    data = np.ones(len(indices)) if w is None else w.astype(np.float64)
    return sp.csr_matrix((data, indices, indptr), shape=(n, n))


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_bfs_matches_scipy(seed):
    indptr, indices, _ = random_graph(3000, 3, seed, components=2)
    label, iters = G.bfs(indptr, indices)
    d = csg.shortest_path(to_scipy(indptr, indices), method="D", unweighted=True, indices=0)
    want = np.where(np.isinf(d), float(G.INF), d).astype(np.uint32)
    assert np.array_equal(label, want)
    assert iters == int(d[np.isfinite(d)].max()) + 1
    assert (label == G.INF).sum() >= 1000  # the second block is unreachable


@pytest.mark.parametrize("seed,components", [(0, 1), (1, 5), (2, 40)])
def test_cc_matches_scipy(seed, components):
    indptr, indices, _ = random_graph(4000, 2, seed, components)
    comp, _ = G.cc(indptr, indices)
    ncomp, lab = csg.connected_components(to_scipy(indptr, indices), directed=True, connection="weak")
    # every component is labelled with its smallest vertex id
    smallest = np.full(ncomp, 1 << 62, np.int64)
    np.minimum.at(smallest, lab, np.arange(4000))
    assert np.array_equal(comp.astype(np.int64), smallest[lab])
    assert ncomp >= components


def test_cc_on_a_directed_path_is_weak_connectivity():
    # edges only point forward: 0 -> 1 -> 2 ... ; the label still reaches every vertex
    n = 50
    indptr = np.arange(n + 1, dtype=np.int64)
    indptr[-1] = n - 1
    indices = np.arange(1, n, dtype=np.int64)
    comp, iters = G.cc(indptr, indices)
    assert (comp == 0).all() and iters >= 2


@pytest.mark.parametrize("seed", [0, 3])
def test_sssp_matches_dijkstra(seed):
    indptr, indices, w = random_graph(3000, 3, seed, components=2)
    cost, _ = G.sssp(indptr, indices, w)
    d = csg.dijkstra(to_scipy(indptr, indices, w), indices=0)
    want = np.where(np.isinf(d), float(G.INF), d).astype(np.uint32)
    assert np.array_equal(cost, want)


def test_pagerank_converges_to_the_linear_system():
    indptr, indices, _ = random_graph(2000, 4, 5)
    value, iters = G.pagerank(indptr, indices)
    exact = G.pagerank_exact(indptr, indices)
    # what is left in the residuals is below the tolerance per vertex, amplified by at most 1/(1-alpha)
    assert np.abs(value - exact).max() < 0.001 / (1 - 0.85) + 1e-4
    assert iters < 100
    assert abs(value.sum() / exact.sum() - 1) < 5e-3
    # a tighter tolerance lands closer
    tight, _ = G.pagerank(indptr, indices, tolerance=1e-6, max_iter=1000)
    assert np.abs(tight - exact).max() < 1e-4


def test_pagerank_exact_matches_a_direct_solve():
    import scipy.sparse.linalg as spl
    indptr, indices, _ = random_graph(300, 3, 8)
    n = 300
    s = np.repeat(np.arange(n), np.diff(indptr))
    P = sp.csr_matrix((1.0 / np.diff(indptr)[s], (s, indices)), shape=(n, n))
    x = spl.spsolve((sp.identity(n) - 0.85 * P.T).tocsc(), np.full(n, 0.15))
    assert np.allclose(G.pagerank_exact(indptr, indices), x, atol=1e-11)


def test_pagerank_on_a_ring_is_uniform():
    n = 64
    indptr = np.arange(n + 1, dtype=np.int64)
    indices = (np.arange(n, dtype=np.int64) + 1) % n
    value, _ = G.pagerank(indptr, indices, tolerance=1e-7, max_iter=1000)
    assert np.allclose(value, 1.0, atol=1e-4)


def test_graph_files_round_trip(tmp_path):
    from gpreempt_amd import executor
    lib = executor.lib()
    base = str(tmp_path / "g")
    assert lib.gpx_write_synthetic_graph(base.encode(), C.c_ulonglong(500), 4, C.c_ulonglong(9)) == 0
    assert os.path.getsize(base + ".col") == 16 + 8 * 501
    indptr, indices, w = G.read_graph(base, weights=True)
    assert indptr[0] == 0 and indptr[-1] == len(indices) == len(w) and (np.diff(indptr) >= 0).all()
    assert indices.min() >= 0 and indices.max() < 500 and w.min() >= 1 and w.max() <= 64
    # symmetric: the transposed edge list is the same multiset
    s = np.repeat(np.arange(500), np.diff(indptr))
    fwd = np.sort(s * 500 + indices)
    bwd = np.sort(indices * 500 + s)
    assert np.array_equal(fwd, bwd)
    # the same seed gives the same graph
    assert lib.gpx_write_synthetic_graph((base + "2").encode(), C.c_ulonglong(500), 4, C.c_ulonglong(9)) == 0
    assert open(base + ".dst", "rb").read() == open(base + "2.dst", "rb").read()
    assert lib.gpx_write_synthetic_graph(base.encode(), C.c_ulonglong(1), 4, C.c_ulonglong(9)) != 0


GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def test_golden_graph_by_hand():
    """the hand-worked answers of tests/golden/tiny_graph against the oracle"""
    import json
    indptr, indices, w = G.read_graph(os.path.join(GOLDEN, "tiny_graph"), weights=True)
    want = json.load(open(os.path.join(GOLDEN, "tiny_graph.expected.json")))
    assert len(indptr) == 11 and len(indices) == 20
    assert G.bfs(indptr, indices)[0].tolist() == want["bfs_levels"]
    assert G.cc(indptr, indices)[0].tolist() == want["components"]
    assert G.sssp(indptr, indices, w)[0].tolist() == want["distances"]
    value, _ = G.pagerank(indptr, indices, tolerance=1e-7, max_iter=1000)
    assert np.allclose(value, G.pagerank_exact(indptr, indices), atol=1e-4)


def test_golden_param_file():
    from gpreempt_amd import executor
    lib = executor.lib()
    lib.gpx_parse_params.restype = C.c_long
    path = os.path.join(GOLDEN, "tiny.mod.params").encode()
    out = np.zeros(8, np.float32)
    n = C.c_size_t(0)
    assert lib.gpx_parse_params(path, b"p0", out.ctypes.data_as(C.c_void_p), C.c_size_t(8), C.byref(n)) == 2
    assert n.value == 6 and out[:6].tolist() == [1.0, -2.5, 3.25, 0.0, np.float32(1e-3), 65504.0]
    assert lib.gpx_parse_params(path, b"fc.bias", out.ctypes.data_as(C.c_void_p), C.c_size_t(8), C.byref(n)) == 2
    assert n.value == 2 and out[:2].tolist() == [0.5, -0.5]
