"""Pins the CPU restatement of the block-level-preemption protocol by invariants that must hold
for every interleaving (reference: scripts/compile/convert_to_blp.py:40-69, src/executor.cpp:211-298)."""
import numpy as np
import pytest

from oracle import oracle as O


def test_decode_exhaustive_small_shapes():
    for sx in range(1, 5):
        for sy in range(1, 5):
            for sz in range(1, 4):
                seen = set()
                for idx in range(sx * sy * sz):
                    x, y, z = O.blp_decode(idx, sx, sy)
                    assert (x, y, z) == (idx % sx, (idx // sx) % sy, idx // (sx * sy))
                    assert 0 <= x < sx and 0 <= y < sy and 0 <= z < sz
                    seen.add((x, y, z))
                assert len(seen) == sx * sy * sz  # a bijection onto the grid


@pytest.mark.parametrize("workers", [1, 3, 8])
def test_every_tile_exactly_once_without_preemption(workers):
    shapes = [(4, 3, 2), (7, 1, 1), (1, 1, 1), (5, 5, 1)]
    r = O.blp_run_chain(shapes, workers)
    assert r["bad"] == 0
    for v in r["visits"]:
        assert (v == 1).all()
    # every workgroup overshoots the counter once (convert_to_blp.py:48-51)
    for (sx, sy, sz), e in zip(shapes, r["executed"]):
        total = sx * sy * sz
        assert e == total + min(total, workers)


@pytest.mark.parametrize("workers", [1, 4, 8])
@pytest.mark.parametrize("inj", [[(0, 0)], [(1, 3)], [(0, 5), (0, 11)], [(0, 2), (2, 0), (3, 24)], [(3, 24)]])
def test_every_tile_exactly_once_with_preemptions(workers, inj):
    shapes = [(4, 3, 2), (7, 1, 1), (2, 2, 2), (5, 5, 1)]
    r = O.blp_run_chain(shapes, workers, inj)
    assert r["bad"] == 0
    for v in r["visits"]:
        assert (v == 1).all()
    # the stop index is the kernel that claimed the injecting tile, or its successor when that
    # claim was the kernel's last (the flag is first seen by the next kernel in the stream)
    for (k, claim), stop in zip(inj, r["stops"]):
        total = int(np.prod(shapes[k]))
        assert stop in ((k, k + 1) if claim == total - 1 and k + 1 < len(shapes) else (k,)), (k, claim, stop)


def test_flag_after_last_claim_of_last_kernel_makes_resume_a_no_op():
    r = O.blp_run_chain([(3, 1, 1)], 1, [(0, 2)])
    # single worker: it claims tile 2 (raising the flag), runs it, then sees the flag and records kernel 0
    assert (r["visits"][0] == 1).all() and r["stops"] == [0]


def test_counters_reset_only_by_execute():
    # after a preempted run and a resume the counter keeps counting up: total claims + overshoots of both launches
    r = O.blp_run_chain([(10, 1, 1)], 2, [(0, 4)])
    assert (r["visits"][0] == 1).all()
    assert r["executed"][0] >= 10 + 2  # never reset to zero by resume


@pytest.mark.parametrize("fracs", [(0.25,), (0.5,), (0.75,), (0.25, 0.5, 0.75)])
def test_config1_cpu_gemm_preempted_equals_uninterrupted(fracs):
    """BASELINE config 1 on the CPU path: 1024^3 is kept for the GPU; here 256^3 with the same
    protocol.  The resumed result must be bit-identical."""
    rng = np.random.default_rng(0xC0FFEE)
    n, tile = 256, 32
    A = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    B = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, n).astype(np.float32)
    base, hits0 = O.blp_gemm(A, B, bias, tile, tile, 8)
    assert hits0 == 0 and not np.isnan(base).any()
    tiles = (n // tile) ** 2
    got, hits = O.blp_gemm(A, B, bias, tile, tile, 8, [int(np.ceil(f * tiles)) - 1 for f in fracs])
    assert hits == len(fracs)
    assert got.tobytes() == base.tobytes()
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU)
    assert np.abs(got - ref).max() / np.abs(ref).max() < 1e-4
