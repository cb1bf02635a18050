"""Writes the small fixtures of this directory.  The reference ships no golden vectors for this
path (its tests only print), so these are authored here, by hand, in the reference's file formats:

  tiny.mod.params            "TVM_MODEL_PARAMS" parameter file (reference src/model.cpp:15-55,
                             writer scripts/compile/compile.py:73-83): two tensors
  tiny_graph.col/.dst/.val   CSR graph in the graph workloads' format (reference
                             src/workloads/graphcompute.cu:16-45): 10 vertices, two components
  tiny_graph.expected.json   BFS levels, component labels and shortest distances from vertex 0,
                             worked out by hand from the drawing below

        0 --1-- 1 --1-- 2        7 --2-- 8
        |       |                 \\     /
        4       1                  5   1
        |       |                   \\ /
        3 --1-- 4 --7-- 5 --1-- 6    9

Run from the repository root: python tests/golden/make_fixtures.py
"""
import json
import os
import struct

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def write_params(path, tensors):
    with open(path, "wb") as f:
        f.write(b"TVM_MODEL_PARAMS\0")
        f.write(struct.pack("<Q", len(tensors)))
        for key, values in tensors:
            f.write(key.encode() + b"\0")
            f.write(struct.pack("<Q", len(values)))
            f.write(np.asarray(values, "<f4").tobytes())


def write_array(path, values, dtype):
    a = np.asarray(values, dtype)
    with open(path, "wb") as f:
        f.write(struct.pack("<QQ", a.size, a.itemsize))
        f.write(a.tobytes())


def main():
    write_params(os.path.join(HERE, "tiny.mod.params"),
                 [("p0", [1.0, -2.5, 3.25, 0.0, 1e-3, 65504.0]), ("fc.bias", [0.5, -0.5])])
    edges = [(0, 1, 1), (1, 2, 1), (0, 3, 4), (1, 4, 1), (3, 4, 1), (4, 5, 7), (5, 6, 1), (7, 8, 2), (7, 9, 5), (8, 9, 1)]
    adj = {v: [] for v in range(10)}
    for a, b, w in edges:
        adj[a].append((b, w))
        adj[b].append((a, w))
    col, dst, val = [0], [], []
    for v in range(10):
        for b, w in sorted(adj[v]):
            dst.append(b)
            val.append(w)
        col.append(len(dst))
    base = os.path.join(HERE, "tiny_graph")
    write_array(base + ".col", col, "<u8")
    write_array(base + ".dst", dst, "<u8")
    write_array(base + ".val", val, "<u4")
    inf = 0xFFFFFFFF
    expected = {
        "bfs_levels": [0, 1, 2, 1, 2, 3, 4, inf, inf, inf],
        "components": [0, 0, 0, 0, 0, 0, 0, 7, 7, 7],
        # 0-1-4 costs 2 (the direct 0-3 edge costs 4, 0-1-4-3 costs 3), 4-5 costs 7, 5-6 costs 1
        "distances": [0, 1, 2, 3, 2, 9, 10, inf, inf, inf],
    }
    with open(base + ".expected.json", "w") as f:
        json.dump(expected, f, indent=1)


if __name__ == "__main__":
    main()
