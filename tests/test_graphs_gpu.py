"""Graph workloads on the GPU ("cc", "bfs", "pagerank", "sssp" executors and gp_launch_graph) against
the numpy oracle and scipy, and preempt-then-resume of their host loops (reference
src/workloads/graphcompute.tr.cu; BLPExecutor::execute graph branch, src/executor.cpp:226-228).

Component labels, BFS levels and SSSP distances are integers with a unique answer: compared
bit-exactly.  PageRank adds fp32 residuals with atomics in arrival order, so two runs differ in the
last bits and may stop one iteration apart: compared to the linear system's solution within 0.02
(values are of order 1; the residual-push iteration leaves up to 0.001 per vertex unpushed, which
the oracle's own run turns into an error of 0.008 on this graph)."""
import ctypes as C
import threading
import time

import numpy as np
import pytest

from oracle import graphs as G

pytestmark = pytest.mark.gpu

N, DEG = 30000, 5
PR_TOL = 0.02


@pytest.fixture(scope="module")
def ex_mod(gp):
    from gpreempt_amd import executor
    return executor


@pytest.fixture(scope="module")
def graph(ex_mod, tmp_path_factory):
    base = str(tmp_path_factory.mktemp("graph") / "g")
    assert ex_mod.lib().gpx_write_synthetic_graph(base.encode(), C.c_ulonglong(N), DEG, C.c_ulonglong(7)) == 0
    indptr, indices, w = G.read_graph(base, weights=True)
    return base, indptr, indices, w


def expected(kind, graph):
    _, indptr, indices, w = graph
    if kind == "bfs":
        return "label", np.uint32, G.bfs(indptr, indices)[0]
    if kind == "cc":
        return "comp", np.uint64, G.cc(indptr, indices)[0]
    if kind == "sssp":
        return "cost", np.uint32, G.sssp(indptr, indices, w)[0]
    return "value", np.float32, G.pagerank_exact(indptr, indices)


def check(kind, got, want):
    if kind == "pagerank":
        assert np.abs(got - want).max() < PR_TOL
    else:
        assert np.array_equal(got, want)


@pytest.mark.parametrize("kind", ["bfs", "cc", "sssp", "pagerank"])
@pytest.mark.parametrize("blp", [False, True])
def test_workload_matches_oracle(gp, ex_mod, graph, kind, blp):
    ex = ex_mod.Executor(kind, blp=blp, graph_path=graph[0])
    if blp:
        ex.set_flag(gp.Flag())
    stream = gp.Stream(1)
    key, dt, want = expected(kind, graph)
    for _ in range(2):  # a second execute starts from scratch
        ex.execute(stream)
        check(kind, ex.graph_result(key, dt), want)
    info = ex.graph_info()
    assert info["vertices"] == N and info["edges"] == len(graph[2]) and info["preemptions"] == 0
    assert info["iterations"] >= 3


def test_synthetic_default_and_bad_names(gp, ex_mod):
    ex = ex_mod.Executor("bfs@n=5000,deg=4,seed=3")
    ex.execute()
    label = ex.graph_result("label", np.uint32)
    assert label[0] == 0 and (label != G.INF).sum() > 4000
    assert ex.kernel_num() == 0
    with pytest.raises(ex_mod.StatusError):
        ex.graph_result("cost", np.uint32)
    with pytest.raises(ex_mod.StatusError):
        ex_mod.Executor("bfs@n=1")
    with pytest.raises(ex_mod.StatusError):
        ex_mod.Executor("bfs", graph_path="/nonexistent/graph")


# (iteration, kernel, claim): -1 = PageRank's set-up kernel
INJECT = {"bfs": [(0, 0, 0), (2, 0, 900), (4, 0, 1500)],
          "cc": [(-1, 0, 5), (0, 0, 1500), (1, 0, 10), (2, 0, 1800)],
          "sssp": [(1, 0, 100), (3, 1, 60), (6, 0, 1700)],
          "pagerank": [(-1, 0, 50), (0, 0, 1000), (1, 1, 20), (5, 0, 1600)]}


@pytest.mark.parametrize("kind", ["bfs", "cc", "sssp", "pagerank"])
def test_injected_preemption_then_resume(gp, ex_mod, graph, kind):
    key, dt, want = expected(kind, graph)
    ex = ex_mod.Executor(kind, blp=True, graph_path=graph[0])
    flag = gp.Flag()
    ex.set_flag(flag)
    stream = gp.Stream(1)
    total = 0
    for it, kernel, claim in INJECT[kind]:
        flag.set(0)
        ex.graph_inject_preempt(it, kernel, claim)
        ex.execute(stream)
        info = ex.graph_info()
        assert flag.get() == 0  # raised by the kernel, lowered by the loop after the stop was seen
        # (a flag raised by the last claims of a short kernel is first seen by the next kernel)
        assert info["preemptions"] == total + 1, (it, kernel, claim, info)
        total = info["preemptions"]
        check(kind, ex.graph_result(key, dt), want)


def test_pagerank_push_runs_every_tile_exactly_once(gp):
    """The push kernel is not idempotent: with residual increments of 0.5 (exact in fp32 in any
    order) the residual of a vertex must equal half its in-degree, also when the launch is stopped
    half-way and continued."""
    rng = np.random.default_rng(0)
    n, deg = 20000, 8
    indices = rng.integers(0, n, n * deg).astype(np.uint64)
    indptr = (np.arange(n + 1) * deg).astype(np.uint64)
    want = np.bincount(indices.astype(np.int64), minlength=n).astype(np.float32) * 0.5
    bufs = dict(vl=gp.DevBuf.from_array(indptr), el=gp.DevBuf.from_array(indices),
                active=gp.DevBuf.from_array(np.ones(n, np.uint8)), delta=gp.DevBuf.from_array(np.full(n, 0.5, np.float32)),
                residual=gp.DevBuf.from_array(np.zeros(n, np.float32)), value=gp.DevBuf.from_array(np.zeros(n, np.float32)),
                changed=gp.DevBuf.from_array(np.zeros(1, np.uint32)))
    p = gp.GraphParams(3, 0, n, bufs["vl"].ptr, bufs["el"].ptr, None, None, bufs["active"].ptr, None, None,
                       bufs["delta"].ptr, bufs["residual"].ptr, bufs["value"].ptr, 0.85, 0.001, None, None, bufs["changed"].ptr, 0)
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    info = gp.launch("gp_launch_graph", p, st.ctx(0, inject_at=40))
    gp.check(gp.lib().gp_stream_sync(None))
    assert info.total_tiles >= n // 4 // 16
    assert st.stop_index() == 0 and flag.get() == 1
    part = bufs["residual"].download(np_dtype=np.float32)
    assert not np.array_equal(part, want)
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_graph", p, st.ctx(0))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == -1
    assert np.array_equal(bufs["residual"].download(np_dtype=np.float32), want)
    assert not bufs["active"].download(np_dtype=np.uint8).any()


@pytest.mark.parametrize("lanes", [16, 32, 64])
def test_bfs_step_lane_widths(gp, graph, lanes):
    """one BFS level through the C ABI at each lane-group width, against the oracle's frontier"""
    _, indptr, indices, _ = graph
    label = np.full(N, G.INF, np.uint32)
    label[0] = 0
    want, _ = G.bfs(indptr, indices)
    bufs = dict(vl=gp.DevBuf.from_array(indptr.astype(np.uint64)), el=gp.DevBuf.from_array(indices.astype(np.uint64)),
                label=gp.DevBuf.from_array(label), changed=gp.DevBuf.from_array(np.zeros(1, np.uint32)))
    for level in range(3):
        p = gp.GraphParams(0, level, N, bufs["vl"].ptr, bufs["el"].ptr, None, bufs["label"].ptr, None, None, None,
                           None, None, None, 0, 0, None, None, bufs["changed"].ptr, lanes)
        info = gp.launch("gp_launch_graph", p)
        assert info.total_tiles == (N + 256 // lanes - 1) // (256 // lanes)
    gp.check(gp.lib().gp_stream_sync(None))
    got = bufs["label"].download(np_dtype=np.uint32)
    assert np.array_equal(got[want <= 3], want[want <= 3]) and (got[want > 3] == G.INF).all()
    p = gp.GraphParams(0, 0, N, bufs["vl"].ptr, bufs["el"].ptr, None, bufs["label"].ptr, None, None, None,
                       None, None, None, 0, 0, None, None, bufs["changed"].ptr, 8)
    with pytest.raises(gp.GpError):
        gp.launch("gp_launch_graph", p)


@pytest.mark.parametrize("kind", ["cc", "pagerank"])
def test_host_timed_preemption(gp, ex_mod, kind):
    """The flag goes up whenever the host gets to it, several times per run, while the count of
    active latency-critical tasks is non-zero (the reference's lc_tasks); the result is the same."""
    wl = f"{kind}@n=400000,deg=6,seed=11"
    base = ex_mod.Executor(wl)
    base.execute()
    key, dt = ("comp", np.uint64) if kind == "cc" else ("value", np.float32)
    want = base.graph_result(key, dt).copy()
    ex = ex_mod.Executor(wl, blp=True)
    flag = gp.Flag()
    ex.set_flag(flag)
    stream = gp.Stream(1)
    preempted = 0
    for _ in range(4):
        done = threading.Event()

        def run():
            ex.execute(stream)
            done.set()
        t = threading.Thread(target=run)
        t.start()
        while not done.is_set():
            ex.set_lc_tasks(1)
            flag.set(1)
            time.sleep(0.0003)
            flag.set(0)
            ex.set_lc_tasks(0)
            time.sleep(0.0005)
        t.join()
        got = ex.graph_result(key, dt)
        if kind == "cc":
            assert np.array_equal(got, want)
        else:
            assert np.abs(got - want).max() < 2 * PR_TOL
        preempted = ex.graph_info()["preemptions"]
    assert preempted > 0


def test_golden_graph_on_the_gpu(gp, ex_mod):
    """tests/golden/tiny_graph (10 vertices, answers worked out by hand) through the executors"""
    import json
    import os
    base = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "tiny_graph")
    want = json.load(open(base + ".expected.json"))
    for kind, key, dt, field in (("bfs", "label", np.uint32, "bfs_levels"), ("cc", "comp", np.uint64, "components"), ("sssp", "cost", np.uint32, "distances")):
        ex = ex_mod.Executor(kind, blp=True, graph_path=base)
        ex.set_flag(gp.Flag())
        ex.execute()
        assert ex.graph_result(key, dt).tolist() == want[field], kind


def test_ragged_graph_with_sinks_and_isolated_vertices(gp, ex_mod, tmp_path):
    """directed edges, a sink (no out-edges), an isolated vertex, a self-contained pair, and a
    vertex whose neighbour list is longer than a wavefront"""
    import os
    import struct
    n = 200
    adj = {v: [] for v in range(n)}
    for v in range(1, 150):
        adj[0].append(v)          # a hub with 149 out-edges
    for v in range(1, 100):
        adj[v].append(v + 1)      # a directed chain 1 -> 2 -> ... -> 100
    adj[150].append(151)
    adj[151].append(150)          # a pair on its own
    # 100..149 are sinks; 152..199 are isolated
    indptr, indices = [0], []
    for v in range(n):
        indices += sorted(adj[v])
        indptr.append(len(indices))
    w = [1 + (i * 7) % 13 for i in range(len(indices))]
    base = str(tmp_path / "ragged")
    for ext, arr, fmt, size in ((".col", indptr, "Q", 8), (".dst", indices, "Q", 8), (".val", w, "I", 4)):
        with open(base + ext, "wb") as f:
            f.write(struct.pack("<QQ", len(arr), size))
            f.write(struct.pack("<%d%s" % (len(arr), fmt), *arr))
    ip, ix, ww = G.read_graph(base, weights=True)
    for kind, key, dt, want in (("bfs", "label", np.uint32, G.bfs(ip, ix)[0]), ("cc", "comp", np.uint64, G.cc(ip, ix)[0]),
                                ("sssp", "cost", np.uint32, G.sssp(ip, ix, ww)[0])):
        ex = ex_mod.Executor(kind, blp=True, graph_path=base)
        ex.set_flag(gp.Flag())
        ex.execute()
        assert np.array_equal(ex.graph_result(key, dt), want), kind
    ex = ex_mod.Executor("pagerank", blp=True, graph_path=base)
    ex.set_flag(gp.Flag())
    ex.execute()
    value = ex.graph_result("value", np.float32)
    ref, _ = G.pagerank(ip, ix)
    assert np.isfinite(value).all() and np.abs(value - ref).max() < 5e-3
    assert np.allclose(value[152:], 0.15)  # nobody points at the isolated vertices
    # a malformed file is refused, not launched
    with open(base + ".dst", "r+b") as f:
        f.seek(16)
        f.write(struct.pack("<Q", 10 ** 6))
    with pytest.raises(ex_mod.StatusError):
        ex_mod.Executor("bfs", graph_path=base)
