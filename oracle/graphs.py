"""CPU restatement of the reference's graph workloads (src/workloads/graphcompute.tr.cu), in numpy.

TEST INFRASTRUCTURE ONLY: imported by tests/ and checkers, never by the product path.

Each function follows the reference's host loop and kernel semantics (cited per function) with the
frontier processed as whole arrays; tests/test_oracle_graphs.py pins them against scipy's
csgraph routines (breadth-first distances, weakly connected components, Dijkstra) and, for
PageRank, against the linear system the iteration converges to.
"""
import numpy as np

INF = np.uint32(0xFFFFFFFF)


def read_array(path, dtype):
    """u64 count, u64 type tag, payload (reference src/workloads/graphcompute.cu:28-40)"""
    with open(path, "rb") as f:
        count = int(np.frombuffer(f.read(8), np.uint64)[0])
        f.read(8)
        return np.frombuffer(f.read(count * np.dtype(dtype).itemsize), dtype).copy()


def read_graph(base, weights=False):
    indptr = read_array(base + ".col", np.uint64)
    indices = read_array(base + ".dst", np.uint64)
    w = read_array(base + ".val", np.uint32) if weights else None
    return indptr.astype(np.int64), indices.astype(np.int64), w


def _sources(indptr):
    return np.repeat(np.arange(len(indptr) - 1), np.diff(indptr))


def bfs(indptr, indices, src=0):
    """bfs_kernel_coalesce + BFS::compute (:218-241, :257-285): vertices labelled `level` give
    level+1 to unlabelled neighbours until nothing changes; returns (labels, iterations)."""
    n = len(indptr) - 1
    label = np.full(n, INF, np.uint32)
    label[src] = 0
    s = _sources(indptr)
    level, iters = 0, 0
    while True:
        on = label[s] == level
        nxt = indices[on]
        nxt = nxt[label[nxt] == INF]
        changed = nxt.size > 0
        label[nxt] = level + 1
        level += 1
        iters += 1
        if not changed:
            return label, iters


def cc(indptr, indices):
    """cc_kernel_coalesce + CC::compute (:88-127, :142-174): labels start as vertex ids; along every
    edge of an active vertex the smaller label is written (atomic min) to the end holding the
    larger one, which becomes active for the next round."""
    n = len(indptr) - 1
    comp = np.arange(n, dtype=np.uint64)
    s = _sources(indptr)
    active = np.ones(n, bool)
    iters = 0
    while True:
        on = active[s]
        a, b = s[on], indices[on]
        ca, cb = comp[a], comp[b]
        nxt = np.zeros(n, bool)
        fwd = ca < cb
        bwd = cb < ca
        new = comp.copy()
        np.minimum.at(new, b[fwd], ca[fwd])
        np.minimum.at(new, a[bwd], cb[bwd])
        nxt[b[fwd]] = True
        nxt[a[bwd]] = True
        changed = bool(fwd.any() or bwd.any())
        comp = new
        active = nxt
        iters += 1
        if not changed:
            return comp, iters


def sssp(indptr, indices, weights, src=0):
    """sssp_kernel_coalesce + sssp_update + SSSP::compute (:540-561, :592-603, :635-675): active
    vertices offer cost + weight to their neighbours (atomic min into new_cost); vertices whose
    new_cost dropped below cost take it and become active."""
    n = len(indptr) - 1
    cost = np.full(n, INF, np.uint32)
    new_cost = cost.copy()
    active = np.zeros(n, bool)
    cost[src] = new_cost[src] = 0
    active[src] = True
    s = _sources(indptr)
    w = weights.astype(np.uint64)
    iters = 0
    while True:
        on = active[s]
        via = new_cost[s[on]].astype(np.uint64) + w[on]
        nc = new_cost.astype(np.uint64)
        np.minimum.at(nc, indices[on], via)
        new_cost = nc.astype(np.uint32)
        active[:] = False
        better = new_cost < cost
        cost[better] = new_cost[better]
        active[better] = True
        iters += 1
        if not better.any():
            return cost, iters


def pagerank(indptr, indices, alpha=0.85, tolerance=0.001, max_iter=100):
    """pr_initialize / pr_kernel_coalesce / pr_update + PageRank::compute (:327-335, :367-384,
    :416-425, :450-495): residual-push PageRank in fp32."""
    n = len(indptr) - 1
    deg = np.diff(indptr).astype(np.float32)
    safe = np.where(deg > 0, deg, 1).astype(np.float32)
    value = np.full(n, 1.0 - alpha, np.float32)
    delta = np.where(deg > 0, np.float32((1.0 - alpha) * alpha) / safe, 0).astype(np.float32)
    residual = np.zeros(n, np.float32)
    active = np.ones(n, bool)
    s = _sources(indptr)
    iters = 0
    while True:
        on = active[s]
        np.add.at(residual, indices[on], delta[s[on]])
        active[:] = False
        up = residual > np.float32(tolerance)
        value[up] += residual[up]
        delta[up] = np.where(deg[up] > 0, residual[up] * np.float32(alpha) / safe[up], 0)
        residual[up] = 0
        active[up] = True
        iters += 1
        if not up.any() or iters >= max_iter:
            return value, iters


def pagerank_exact(indptr, indices, alpha=0.85):
    """Fixed point of the push iteration with tolerance 0: x = (1-alpha) 1 + alpha P^T x, where
    P[v, u] = 1/outdeg(v) for every edge v -> u; solved by fp64 fixed-point iteration (the map
    contracts by alpha per step) down to 1e-13, checked against a direct solve on small graphs."""
    import scipy.sparse as sp
    n = len(indptr) - 1
    deg = np.diff(indptr).astype(np.float64)
    s = _sources(indptr)
    PT = sp.csr_matrix((1.0 / deg[s], (indices, s)), shape=(n, n))
    x = np.full(n, 1.0 - alpha)
    for _ in range(1000):
        nx = (1.0 - alpha) + alpha * (PT @ x)
        if np.abs(nx - x).max() < 1e-13:
            return nx
        x = nx
    return x
