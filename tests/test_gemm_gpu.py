"""Parity of the preemptible GEMM (C ABI gp_launch_gemm) with the CPU oracle, and bit-exact
preempt/resume (BASELINE config 1; protocol of reference src/tests/test-dnn-blp.cpp:36-42)."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

# Tolerances stated by the north star: 1e-4 relative for fp32, 1e-2 for fp16 / bf16.  "Relative"
# is taken against the magnitude of the output tensor (max |ref|), because single elements of a
# GEMM can cancel to ~0 where an element-wise ratio is meaningless.
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def rel_err(got, ref):
    return float(np.abs(got - ref).max() / max(np.abs(ref).max(), 1e-30))


def run_gemm(gp, dt, M, N, K, b_is_nk, act, use_bias, use_res, seed, ctx_fn=None, tile=0, batch=1, alpha=1.0, variant=0, tile_n=None):
    rng = np.random.default_rng(seed)
    dtype = gp.DTYPE_BY_NAME[dt]
    A = O.round_to(rng.uniform(-1, 1, (batch, M, K)).astype(np.float32), dt)
    Bshape = (batch, N, K) if b_is_nk else (batch, K, N)
    B = O.round_to(rng.uniform(-1, 1, Bshape).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt) if use_bias else None
    res = O.round_to(rng.uniform(-1, 1, (batch, M, N)).astype(np.float32), dt) if use_res else None
    dA, dB = gp.DevBuf.from_array(A, dtype), gp.DevBuf.from_array(B, dtype)
    dbias = gp.DevBuf.from_array(bias, dtype) if use_bias else None
    dres = gp.DevBuf.from_array(res, dtype) if use_res else None
    dC = gp.DevBuf(batch * M * N * gp.DTYPE_SIZE[dtype])
    dC.fill32(0xFFFFFFFF if dt == "f32" else 0x7E007E00)  # NaN pattern: unwritten elements show up
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, stride_a=M * K, B=dB.ptr,
                      ldb=K if b_is_nk else N, stride_b=N * K, b_is_nk=int(b_is_nk), C=dC.ptr, ldc=N,
                      stride_c=M * N, bias=gp._ptr(dbias), residual=gp._ptr(dres), alpha=alpha, act=act,
                      batch=batch, tile_m=tile, tile_n=tile if tile_n is None else tile_n, variant=variant)
    info = ctx_fn(p, dC) if ctx_fn else gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    got = dC.download(dtype, (batch, M, N)).copy()
    ref = np.stack([O.gemm_bias_act(A[b] * np.float32(alpha), B[b], bias, None if res is None else res[b], act, b_is_nk)
                    for b in range(batch)])
    return got, ref, info


@pytest.mark.parametrize("dt", ["f32", "f16", "bf16"])
@pytest.mark.parametrize("b_is_nk", [False, True])
@pytest.mark.parametrize("shape", [(256, 256, 128), (200, 136, 72), (64, 1000, 512), (1, 8, 8), (130, 264, 40), (128, 768, 3072), (1568, 256, 2304)])
def test_gemm_matches_oracle(gp, dt, b_is_nk, shape):
    M, N, K = shape
    # every kernel variant and tile size that supports the layout (B stored K x N needs the
    # register-staged kernel), plus the launcher's own choice
    variants = [(64, gp.MAT_STAGED), (128, gp.MAT_STAGED), (0, gp.MAT_AUTO)]
    if b_is_nk:
        variants += [(64, gp.MAT_PIPE), (128, gp.MAT_PIPE), (64, gp.MAT_PIPE_SPLITK), (32, gp.MAT_PIPE_SPLITK)]
    for tile, variant in variants:
        got, ref, info = run_gemm(gp, dt, M, N, K, b_is_nk, gp.ACT_RELU, True, True, seed=M + N + K, tile=tile, variant=variant)
        if tile:
            assert info.total_tiles == -(-M // tile) * -(-N // tile)
        assert np.isfinite(got).all(), (dt, shape, tile, variant)
        assert rel_err(got, ref) < TOL[dt], (dt, shape, tile, variant)
    if b_is_nk:  # wide split-K bodies: 16 or 8 wavefronts per tile
        for tm, tn, variant in ((32, 32, gp.MAT_WIDE), (32, 32, gp.MAT_WIDE8), (64, 32, gp.MAT_WIDE), (64, 64, gp.MAT_WIDE8)):
            got, ref, info = run_gemm(gp, dt, M, N, K, True, gp.ACT_RELU, True, True, seed=M + N + K, tile=tm, tile_n=tn, variant=variant)
            assert info.total_tiles == -(-M // tm) * -(-N // tn) and info.block == (1024 if variant == gp.MAT_WIDE else 512)
            assert np.isfinite(got).all(), (dt, shape, tm, tn, variant)
            assert rel_err(got, ref) < TOL[dt], (dt, shape, tm, tn, variant)
    else:
        with pytest.raises(gp.GpError):
            run_gemm(gp, dt, M, N, K, False, gp.ACT_RELU, True, True, seed=1, tile=32, variant=gp.MAT_WIDE)


@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("variant", [1, 2, 3])
def test_gemm_batched_alpha_gelu(gp, dt, variant):
    got, ref, info = run_gemm(gp, dt, 128, 64, 64, True, gp.ACT_GELU, True, False, seed=3, batch=6, alpha=0.125, variant=variant)
    assert info.shape[2] == 6
    assert rel_err(got, ref) < TOL[dt]


def test_gemm_known_answers(gp):
    """Identity, permutation and all-ones operands: results fixed by the mathematics."""
    n = 128
    eye = np.eye(n, dtype=np.float32)
    rng = np.random.default_rng(1)
    X = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    perm = rng.permutation(n)
    for A, B, want in ((eye, X, X), (X, eye, X), (eye[perm], X, X[perm]), (np.ones((n, n), np.float32), np.ones((n, n), np.float32), np.full((n, n), n, np.float32))):
        dA, dB, dC = gp.DevBuf.from_array(A, gp.F32), gp.DevBuf.from_array(B, gp.F32), gp.DevBuf(4 * n * n)
        p = gp.GemmParams(dtype=gp.F32, M=n, N=n, K=n, A=dA.ptr, lda=n, B=dB.ptr, ldb=n, b_is_nk=0, C=dC.ptr, ldc=n, alpha=1.0, batch=1)
        gp.launch("gp_launch_gemm", p)
        gp.check(gp.lib().gp_stream_sync(None))
        assert np.array_equal(dC.download(gp.F32, (n, n)), want)


def test_gemm_rejects_bad_arguments(gp):
    d = gp.DevBuf(4096)
    bad = gp.GemmParams(dtype=gp.F32, M=8, N=8, K=6, A=d.ptr, lda=6, B=d.ptr, ldb=8, C=d.ptr, ldc=8, batch=1)
    with pytest.raises(gp.GpError) as e:
        gp.launch("gp_launch_gemm", bad)
    assert e.value.status == gp.OUTOFRANGE and "multiples" in str(e.value)
    bad = gp.GemmParams(dtype=7, M=8, N=8, K=8, A=d.ptr, lda=8, B=d.ptr, ldb=8, C=d.ptr, ldc=8, batch=1)
    with pytest.raises(gp.GpError):
        gp.launch("gp_launch_gemm", bad)


# ---- config 1: 1024^3 fp32 GEMM + bias + ReLU, preempt at 25/50/75 %, resume, bit-exact ----

def _config1(gp, tile):
    rng = np.random.default_rng(0xC0FFEE)
    A = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    B = rng.uniform(-1, 1, (1024, 1024)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, 1024).astype(np.float32)
    dA, dB, db = (gp.DevBuf.from_array(x, gp.F32) for x in (A, B, bias))
    dC = gp.DevBuf(4 * 1024 * 1024)
    p = gp.GemmParams(dtype=gp.F32, M=1024, N=1024, K=1024, A=dA.ptr, lda=1024, B=dB.ptr, ldb=1024, b_is_nk=0,
                      C=dC.ptr, ldc=1024, bias=db.ptr, alpha=1.0, act=gp.ACT_RELU, batch=1, tile_m=tile, tile_n=tile)
    return A, B, bias, p, dC, (dA, dB, db)


@pytest.mark.parametrize("tile", [64, 128])
def test_config1_preempt_resume_bit_exact(gp, tile):
    A, B, bias, p, dC, keep = _config1(gp, tile)
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    # uninterrupted, non-preemptible launch (BaseExecutor path)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download(gp.F32, (1024, 1024)).copy()
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU)
    assert rel_err(base, ref) < 1e-4
    # uninterrupted, preemptible launch: same bits.  The grid is capped below the tile count so
    # that claims are spread over the kernel's run: with one workgroup per tile every claim is made
    # in the first microsecond and whether one of them sees the injected flag is a race.
    WGS = 16
    dC.fill32(0xFFFFFFFF)
    info = gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=WGS))
    gp.check(gp.lib().gp_stream_sync(None))
    total = info.total_tiles
    assert total == (1024 // tile) ** 2 and info.grid <= total
    assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base)
    assert st.stop_index() == -1
    assert st.counters()[0] == total + info.grid  # every workgroup overshoots once (convert_to_blp.py:48-51)
    for frac in (0.25, 0.5, 0.75):
        k = int(np.ceil(frac * total))
        st.reset()
        flag.set(0)
        dC.fill32(0xFFFFFFFF)
        gp.launch("gp_launch_gemm", p, st.ctx(inject_at=k - 1, max_workgroups=WGS))  # claim number k raises the flag
        gp.check(gp.lib().gp_stream_sync(None))
        assert flag.get() == 1
        assert st.stop_index() == 0
        done = st.counters()[0]
        # the flag is read from host memory by every 8th claim; the claims in between and one
        # claim per resident workgroup may still be made before the stop is seen
        assert k <= done <= min(total, k + info.grid + 8), (k, done, info.grid)
        part = dC.download(gp.F32, (1024, 1024))
        assert np.isnan(part).any() or done == total  # really interrupted
        # host: *flag = 0; resume (executor.cpp:280-298): counters are NOT reset
        flag.set(0)
        st.clear_stop()
        gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=WGS))
        gp.check(gp.lib().gp_stream_sync(None))
        assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base), f"resume after {frac:.0%} differs"
        assert st.stop_index() == -1


def test_flag_set_before_launch(gp):
    """A submission that starts while the flag is up: the first kernel stops after at most one
    tile per resident workgroup (the first claim reads the flag), every later kernel of the
    submission does no tile at all, and a resume completes the work bit-exactly."""
    A, B, bias, p, dC, keep = _config1(gp, 64)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(2, flag)
    flag.set(1)
    dC.fill32(0xFFFFFFFF)
    info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, max_workgroups=32))
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=1, max_workgroups=32))
    gp.check(gp.lib().gp_stream_sync(None))
    c = st.counters()
    assert 1 <= c[0] <= 32 and c[1] == 0 and st.stop_index() == 0
    assert np.isnan(dC.download(gp.F32, (1024, 1024))).any()
    # per-tile polling (poll_every = 1) gives the same bound
    st.reset(); st.clear_stop(); dC.fill32(0xFFFFFFFF)
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, max_workgroups=32, poll_every=1))
    gp.check(gp.lib().gp_stream_sync(None))
    assert 1 <= st.counters()[0] <= 32 and st.stop_index() == 0
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0))
    gp.check(gp.lib().gp_stream_sync(None))
    assert np.array_equal(dC.download(), base)
    with pytest.raises(gp.GpError):
        gp.launch("gp_launch_gemm", p, st.ctx(poll_every=3))


@pytest.mark.parametrize("tile", [128, 64])
def test_flag_is_seen_after_the_first_four_counter_groups_ran_out(gp, tile):
    """With 32 claim counters the first four groups read the flag for everybody.  A relaunch that finds their
    slices handed out (here: their counters set past the end by the test) while the flag is up must still
    stop: the other groups take the reading over (128 x 128 tiles: one workgroup per compute unit), or the
    workgroup in front of the workers, which reads the flag for such a launch, has recorded the stop before
    anybody claims (64 x 64 tiles).  Lowering the flag and relaunching completes the work with the bits of an
    uninterrupted run."""
    rng = np.random.default_rng(21)
    M = N = 4096
    K = 256
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), "f16")
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), "f16")
    dA, dB = (gp.DevBuf.from_array(x, gp.F16) for x in (A, B))
    dC = gp.DevBuf(2 * M * N)
    p = gp.GemmParams(dtype=gp.F16, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, alpha=1.0, batch=1,
                      tile_m=tile, tile_n=tile)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)   # fewer workgroups than tiles below, so that claims go through the counters
    S = st.COUNTER_STRIDE
    gone = np.zeros(32 * S, np.int32)
    gone[[0, S, 2 * S, 3 * S]] = 1 << 20
    st.executed.upload(gone)
    flag.set(1)
    dC.fill32(0)
    info = gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=512))
    gp.check(gp.lib().gp_stream_sync(None))
    assert info.total_tiles == (4096 // tile) ** 2 and info.grid < info.total_tiles and info.fixed_claims == 0
    assert st.stop_index() == 0
    c = st.counters()[::S]
    if tile == 128:
        # the first claim of every group has a number that reads the flag: about one tile per workgroup (a second
        # one where a tile ends before the read of host memory has come back), of the tiles these groups own
        assert info.front == 0 and 0 < int(c[4:].sum()) <= 2 * info.grid, c
    else:
        # the workgroup in front starts first and reads the flag first: hardly a claim is made before the stop is recorded
        assert info.front == 8 and int(c[4:].sum()) <= 2 * info.grid, c
    assert not np.array_equal(dC.download(), base)
    # the four groups get their slices back; the flag comes down; the relaunch finishes everything
    now = st.counters()
    now[[0, S, 2 * S, 3 * S]] = 0
    st.executed.upload(now)
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=512))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == -1
    assert np.array_equal(dC.download(), base)


@pytest.mark.parametrize("K", [64, 128, 256])
@pytest.mark.parametrize("N,res", [(256, True), (64, False)])
def test_shallow_gemm_plain_and_preemptible_launches_agree(gp, N, K, res):
    """One to four K-steps over many rows (the first pointwise layers of a CNN at batch 8): the 64 x 64 body
    with its two-stage ring, launched plainly, with fixed claims on fresh counters (waiting for the stop
    index, and starting the tile without waiting) and on counters that may hold claims; each against the
    oracle and all four with the same bits."""
    M = 8192
    rng = np.random.default_rng(K + N)
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), "f16")
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), "f16")
    bias = O.round_to(rng.uniform(-1, 1, N).astype(np.float32), "f16")
    R = O.round_to(rng.uniform(-1, 1, (M, N)).astype(np.float32), "f16")
    dA, dB, db, dR = (gp.DevBuf.from_array(x, gp.F16) for x in (A, B, bias, R))
    dC = gp.DevBuf(2 * M * N)
    p = gp.GemmParams(dtype=gp.F16, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, bias=db.ptr,
                      residual=dR.ptr if res else None, ldr=N, alpha=1.0, act=gp.ACT_RELU, batch=1)
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU, b_is_nk=True, residual=R if res else None)
    flag = gp.Flag()
    flag.set(0)
    outs = []
    for fresh in (None, 1, 2, 0):
        dC.fill32(0)
        if fresh is None:
            gp.launch("gp_launch_gemm", p)
        else:
            st = gp.BlpState(1, flag, 32)
            info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=fresh))
            assert info.fixed_claims == 1
        gp.check(gp.lib().gp_stream_sync(None))
        outs.append(dC.download().copy())
        assert rel_err(gp.from_storage(outs[-1], gp.F16).reshape(M, N), ref) < 1e-2, fresh
    assert all(np.array_equal(outs[0], o) for o in outs[1:])


def test_fixed_claims_of_a_one_claim_per_workgroup_launch(gp):
    """With several counters per kernel and at least as many workgroups as claims, a workgroup's
    claim is fixed by its index and a bit per workgroup (ints 1..15 of the counter's line) says
    whether it was made; int 0 counts.  A first launch (fresh) sets them without looking; a relaunch
    runs exactly the claims whose bits are clear."""
    A, B, bias, p, dC, keep = _config1(gp, 64)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download(gp.F32, (1024, 1024)).copy()
    flag = gp.Flag()
    G = 32
    st = gp.BlpState(1, flag, G)

    def lines():
        return st.counters().reshape(G, 16).copy()

    def popcount(a):
        return int(np.unpackbits(a.view(np.uint8)).sum())

    def tiles_written():
        c = dC.download(gp.F32, (1024, 1024)).reshape(16, 64, 16, 64)
        return int((~np.isnan(c).any(axis=(1, 3))).sum())

    dC.fill32(0xFFFFFFFF)
    info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))
    gp.check(gp.lib().gp_stream_sync(None))
    total = info.total_tiles
    assert total == 256 and info.grid >= total, "the launch must have a workgroup per claim for this test"
    assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base)
    full = lines()
    assert full[:, 0].sum() == total and popcount(full[:, 1:]) == total and st.stop_index() == -1
    # a second launch finds every claim made
    dC.fill32(0xFFFFFFFF)
    gp.launch("gp_launch_gemm", p, st.ctx())
    gp.check(gp.lib().gp_stream_sync(None))
    assert tiles_written() == 0 and np.array_equal(lines(), full)
    # a random half of the claims marked as made: the relaunch runs the others, once each
    rng = np.random.default_rng(5)
    bits = np.unpackbits(full[:, 1:].copy().view(np.uint8).reshape(G, -1), axis=1)
    keep_mask = (rng.random(bits.shape) < 0.5).astype(np.uint8)
    made = bits & keep_mask
    state = np.zeros_like(full)
    state[:, 1:] = np.packbits(made, axis=1).view(np.int32).reshape(G, 15)
    state[:, 0] = made.sum(axis=1)
    n_made = int(made.sum())
    assert 0 < n_made < total
    st.executed.upload(state.reshape(-1))
    gp.launch("gp_launch_gemm", p, st.ctx())
    gp.check(gp.lib().gp_stream_sync(None))
    assert tiles_written() == total - n_made
    assert np.array_equal(lines(), full)
    # ... and the complement fills in the rest: every claim stands for a tile of its own
    rest = bits & (1 - keep_mask)
    state[:, 1:] = np.packbits(rest, axis=1).view(np.int32).reshape(G, 15)
    state[:, 0] = rest.sum(axis=1)
    st.executed.upload(state.reshape(-1))
    gp.launch("gp_launch_gemm", p, st.ctx())
    gp.check(gp.lib().gp_stream_sync(None))
    assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base)
    # a stop recorded by an earlier kernel: nothing is claimed, fresh or not
    st.reset()
    st.stop.upload(np.array([7], np.int32))
    dC.fill32(0xFFFFFFFF)
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, fresh=1))
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0))
    gp.check(gp.lib().gp_stream_sync(None))
    assert tiles_written() == 0 and not lines().any() and st.stop_index() == 7
    # the flag up at launch: the polling workgroups record the stop, a relaunch completes the work
    st.clear_stop()
    flag.set(1)
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, fresh=1))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == 0
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0))
    gp.check(gp.lib().gp_stream_sync(None))
    assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base) and np.array_equal(lines(), full)


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("tile,variant", [(128, 2), (64, 2), (64, 3), (32, 3)])
def test_pipelined_gemm_preempt_resume_bit_exact(gp, dt, tile, variant):
    """The direct-to-LDS kernels (N x K weights) under the same protocol as config 1."""
    M, N, K = 1024, 512, 1024
    rng = np.random.default_rng(7)
    dtype = gp.DTYPE_BY_NAME[dt]
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt)
    dA, dB, db = (gp.DevBuf.from_array(x, dtype) for x in (A, B, bias))
    dC = gp.DevBuf(M * N * gp.DTYPE_SIZE[dtype])
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, bias=db.ptr,
                      alpha=1.0, act=gp.ACT_RELU, batch=1, tile_m=tile, tile_n=tile, variant=variant)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download().copy()
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU, b_is_nk=True)
    assert rel_err(dC.download(dtype, (M, N)), ref) < TOL[dt]
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    total = (M // tile) * (N // tile)
    for frac in (0.25, 0.75):
        st.reset()
        flag.set(0)
        dC.fill32(0)
        info = gp.launch("gp_launch_gemm", p, st.ctx(inject_at=int(frac * total), max_workgroups=4))
        gp.check(gp.lib().gp_stream_sync(None))
        assert flag.get() == 1 and st.stop_index() == 0 and st.counters()[0] < total
        flag.set(0)
        st.clear_stop()
        gp.launch("gp_launch_gemm", p, st.ctx())
        gp.check(gp.lib().gp_stream_sync(None))
        assert np.array_equal(dC.download(), base)


@pytest.mark.parametrize("dt", ["f16", "bf16", "f32"])
@pytest.mark.parametrize("tm,tn,variant", [(32, 32, 4), (32, 32, 5), (64, 32, 4), (64, 64, 5)])
def test_wide_gemm_preempt_resume_bit_exact(gp, dt, tm, tn, variant):
    """The wide split-K bodies under config 1's protocol: stopped at a tile boundary and resumed, the
    output has the bits of the uninterrupted run; batched with GELU and alpha as well."""
    M, N, K = 512, 384, 1600 if dt != "f32" else 800  # K is not a multiple of a 16-wavefront stage
    rng = np.random.default_rng(17)
    dtype = gp.DTYPE_BY_NAME[dt]
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt)
    dA, dB, db = (gp.DevBuf.from_array(x, dtype) for x in (A, B, bias))
    dC = gp.DevBuf(M * N * gp.DTYPE_SIZE[dtype])
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, bias=db.ptr,
                      alpha=1.0, act=gp.ACT_RELU, batch=1, tile_m=tm, tile_n=tn, variant=variant)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download().copy()
    assert rel_err(dC.download(dtype, (M, N)), O.gemm_bias_act(A, B, bias, act=O.ACT_RELU, b_is_nk=True)) < TOL[dt]
    # the same summation as the four-wavefront split-K bodies (which the whole-model program uses): same bits
    p.tile_m = p.tile_n = 32
    p.variant = gp.MAT_PIPE_SPLITK
    dC.fill32(0)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    assert np.array_equal(dC.download(), base)
    p.tile_m, p.tile_n, p.variant = tm, tn, variant
    flag = gp.Flag()
    total = (M // tm) * (N // tn)
    for groups, wgs in ((1, 4), (32, 0)):  # one counter and few workgroups; the executor's 32 counters and fixed claims
        st = gp.BlpState(1, flag, groups)
        for frac in (0.25, 0.75):
            st.reset(); st.clear_stop(); flag.set(0)
            dC.fill32(0)
            info = gp.launch("gp_launch_gemm", p, st.ctx(inject_at=int(frac * total), max_workgroups=wgs, fresh=1))
            gp.check(gp.lib().gp_stream_sync(None))
            assert flag.get() == 1
            if wgs:
                assert st.stop_index() == 0 and st.counters()[0] < total
            flag.set(0)
            st.clear_stop()
            gp.launch("gp_launch_gemm", p, st.ctx())
            gp.check(gp.lib().gp_stream_sync(None))
            assert np.array_equal(dC.download(), base), (groups, frac)
    got, ref, info = run_gemm(gp, dt, 128, 64, 192, True, gp.ACT_GELU, True, False, seed=3, batch=6, alpha=0.125, tile=tm, tile_n=tn, variant=variant)
    assert info.shape[2] == 6 and rel_err(got, ref) < TOL[dt]


# ---- long tiles left between two K-steps ---------------------------------------------------------
def _ckpt_gemm(gp, dt, M, N, K, seed=5):
    rng = np.random.default_rng(seed)
    A = rng.uniform(-1, 1, (M, K)).astype(np.float32)
    B = rng.uniform(-1, 1, (N, K)).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, N).astype(np.float32)
    dtype = gp.DTYPE_BY_NAME[dt]
    dA, dB, db = gp.DevBuf.from_array(A, dtype), gp.DevBuf.from_array(B, dtype), gp.DevBuf.from_array(bias, dtype)
    dC = gp.DevBuf(M * N * gp.DTYPE_SIZE[dtype])
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N,
                      bias=db.ptr, alpha=1.0, act=gp.ACT_RELU, batch=1, tile_m=256, tile_n=256)
    return p, (dA, dB, db, dC)


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_long_tiles_are_left_mid_k_and_resumed_bit_exact(gp, dt):
    """256 x 256 tiles over a long K: with a checkpoint workspace a stop request is honoured between
    two K-steps (workgroups store accumulators + K position), not only between tiles; the relaunch
    continues from the stored state and the result is bit-identical to the uninterrupted run."""
    M, N, K = 1024, 1024, 8192 if dt != "f32" else 4096
    p, bufs = _ckpt_gemm(gp, dt, M, N, K)
    dC = bufs[3]
    stream = gp.Stream(1)
    gp.launch("gp_launch_gemm", p, None, stream)
    stream.sync()
    want = dC.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    assert st.enable_checkpoints(p) > 0
    tiles = (M // 256) * (N // 256)
    stops = 0
    for inject in (0, 5, tiles - 1):
        dC.fill32(0)
        st.reset()
        st.clear_stop()
        flag.set(0)
        gp.check(gp.lib().gp_ckpt_reset_async(gp.vp(st.ckpt.ptr), None))
        info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, inject_at=inject), stream)
        stream.sync()
        assert flag.get() == 1
        assert info.grid == tiles  # every tile is claimed at once: only a mid-tile stop can interrupt
        hdr = st.checkpoint_headers(info.grid)
        n_ck = int(hdr[:, 0].sum())
        if st.stop_index() == 0:
            stops += 1
            assert n_ck > 0
            live = hdr[hdr[:, 0] == 1]
            assert (live[:, 1] == 0).all() and (live[:, 3] > 0).all() and (live[:, 3] * (64 if dt != "f32" else 32) < K).all()
            assert len(set(live[:, 2].tolist())) == len(live)  # distinct tiles
            assert not np.array_equal(dC.download(), want)
        # resume until complete (the flag is down, so one relaunch finishes)
        flag.set(0)
        st.clear_stop()
        gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
        stream.sync()
        assert st.stop_index() == -1
        assert int(st.checkpoint_headers(info.grid)[:, 0].sum()) == 0
        assert np.array_equal(dC.download(), want), (dt, inject)
    assert stops >= 2, "the stop request was never seen inside a tile"


def test_long_tiles_stopped_twice_then_finished(gp):
    """A tile can be left more than once; every relaunch continues where the last one stopped."""
    M, N, K = 512, 512, 16384
    p, bufs = _ckpt_gemm(gp, "bf16", M, N, K, seed=9)
    dC = bufs[3]
    stream = gp.Stream(1)
    gp.launch("gp_launch_gemm", p, None, stream)
    stream.sync()
    want = dC.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    st.enable_checkpoints(p)
    dC.fill32(0)
    flag.set(0)
    info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, inject_at=0), stream)
    stream.sync()
    first = st.checkpoint_headers(info.grid)
    assert st.stop_index() == 0 and first[:, 0].sum() > 0
    # second launch with the flag still up: workgroups with a stored tile leave it where it is
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
    stream.sync()
    second = st.checkpoint_headers(info.grid)
    assert st.stop_index() == 0
    # (a tile that no workgroup had started before the first stop may be started, and left, by the second launch:
    # only the workgroups that already held a tile are compared)
    held = first[:, 0] == 1
    assert (second[held, 0] == 1).all() and (second[held, 2] == first[held, 2]).all() and (second[held, 3] >= first[held, 3]).all()
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
    stream.sync()
    assert st.stop_index() == -1
    assert np.array_equal(dC.download(), want)


def test_without_workspace_long_tiles_are_finished(gp):
    """No checkpoint workspace: the reference's behaviour, a workgroup finishes the tile it owes."""
    p, bufs = _ckpt_gemm(gp, "bf16", 512, 512, 4096)
    dC = bufs[3]
    stream = gp.Stream(1)
    gp.launch("gp_launch_gemm", p, None, stream)
    stream.sync()
    want = dC.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    dC.fill32(0)
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, inject_at=0), stream)
    stream.sync()
    assert flag.get() == 1
    assert np.array_equal(dC.download(), want)  # all four tiles were owed and finished


# ---- the 256 x 256 body (config 5's kernel) against the oracle ------------------------------------
@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
@pytest.mark.parametrize("shape", [(512, 768, 1024), (300, 520, 192), (256, 256, 64)])
def test_gemm_256_body_matches_oracle(gp, dt, shape):
    """Plain and preemptible launches of the 256 x 256 body, full and ragged tiles, with bias,
    residual and ReLU, against the oracle."""
    M, N, K = shape
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)

    def preemptible(p, dC):
        return gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))

    for ctx_fn in (None, preemptible):
        st.reset()
        got, ref, info = run_gemm(gp, dt, M, N, K, True, gp.ACT_RELU, True, True, seed=M + N + K, ctx_fn=ctx_fn, tile=256)
        assert info.total_tiles == -(-M // 256) * -(-N // 256)
        assert np.isfinite(got).all(), (dt, shape)
        assert rel_err(got, ref) < TOL[dt], (dt, shape, ctx_fn is not None)
        assert st.stop_index() == -1


@pytest.mark.parametrize("dt", ["bf16", "f16", "f32"])
def test_gemm_256_body_left_mid_k_matches_oracle(gp, dt):
    """The checkpointing form of the 256 x 256 body: uninterrupted, and stopped between two K-steps
    and resumed, both against the oracle (not only against another launch of the same body)."""
    M, N, K = 768, 512, 4096 if dt != "f32" else 2048
    rng = np.random.default_rng(11)
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt)
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU, b_is_nk=True)
    dtype = gp.DTYPE_BY_NAME[dt]
    dA, dB, db = gp.DevBuf.from_array(A, dtype), gp.DevBuf.from_array(B, dtype), gp.DevBuf.from_array(bias, dtype)
    dC = gp.DevBuf(M * N * gp.DTYPE_SIZE[dtype])
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N,
                      bias=db.ptr, alpha=1.0, act=gp.ACT_RELU, batch=1, tile_m=256, tile_n=256)
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    assert st.enable_checkpoints(p) > 0
    stream = gp.Stream(1)
    # uninterrupted run of the checkpointing instantiation
    dC.fill32(0)
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
    stream.sync()
    assert st.stop_index() == -1
    assert rel_err(dC.download(dtype, (M, N)), ref) < TOL[dt]
    whole = dC.download().copy()
    # stopped by the first claim, resumed
    dC.fill32(0)
    st.reset(); st.clear_stop(); flag.set(0)
    gp.check(gp.lib().gp_ckpt_reset_async(gp.vp(st.ckpt.ptr), None))
    info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, inject_at=0), stream)
    stream.sync()
    assert flag.get() == 1 and st.stop_index() == 0
    assert int(st.checkpoint_headers(info.grid)[:, 0].sum()) > 0, "no tile was left half-way"
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
    stream.sync()
    assert st.stop_index() == -1
    assert rel_err(dC.download(dtype, (M, N)), ref) < TOL[dt]
    assert np.array_equal(dC.download(), whole)


# ---- config 5 at full size: bf16 8192^3 on 256 x 256 tiles ----------------------------------------
def gp_to_bf16(a):
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    return ((u + (((u >> 16) & 1) + 0x7FFF)) >> 16).astype(np.uint16)


def test_config5_gemm8192_bf16_full_size(gp):
    """Config 5's best-effort kernel at its real size: U[-1,1) bf16 operands, 1024 tiles of
    256 x 256.  Checked on 96 seeded full output rows against the oracle, exactly on all-ones and
    identity operands, and bit-exactly under preemption at 25 / 50 / 75 % of the tiles with the
    executor's context (32 claim counters, checkpoint workspace: tiles are left between K-steps)."""
    n = 8192
    rng = np.random.default_rng(0x5EED5)
    dA, dB, dC = gp.DevBuf(2 * n * n), gp.DevBuf(2 * n * n), gp.DevBuf(2 * n * n)
    p = gp.GemmParams(dtype=gp.BF16, M=n, N=n, K=n, A=dA.ptr, lda=n, B=dB.ptr, ldb=n, b_is_nk=1, C=dC.ptr, ldc=n,
                      alpha=1.0, act=gp.ACT_NONE, batch=1)
    stream = gp.Stream(1)

    def run_plain():
        dC.fill32(0x7FC07FC0)  # bf16 NaN pattern: unwritten elements show up
        info = gp.launch("gp_launch_gemm", p, None, stream)
        stream.sync()
        assert info.total_tiles == 1024 and info.shape[0] == 32 and info.shape[1] == 32, "config 5 must run on 256 x 256 tiles"
        return dC.download(np_dtype=np.uint16).reshape(n, n)

    # known answers: ones x ones = K (8192 is a bf16 number); identity x B^T = B^T
    ones = np.full(n * n, 0x3F80, np.uint16)
    dA.upload(ones); dB.upload(ones)
    got = run_plain()
    assert (got == gp_to_bf16(np.float32(n))).all()
    Bf = rng.uniform(-1, 1, (n, n)).astype(np.float32)
    Bb = gp_to_bf16(Bf)
    eye = np.zeros((n, n), np.uint16)
    eye[np.arange(n), np.arange(n)] = 0x3F80
    dA.upload(eye); dB.upload(Bb)
    del eye, ones
    got = run_plain()
    assert np.array_equal(got, Bb.T)
    # seeded operands; rows spread over every tile row, checked against the oracle
    Ab = gp_to_bf16(rng.uniform(-1, 1, (n, n)).astype(np.float32))
    dA.upload(Ab)
    base = run_plain().copy()
    rows = np.sort(rng.choice(n, 96, replace=False))
    A32 = (Ab[rows].astype(np.uint32) << 16).view(np.float32)
    B32 = (Bb.astype(np.uint32) << 16).view(np.float32)
    ref = O.gemm_bias_act(A32, B32, b_is_nk=True)
    got32 = (base[rows].astype(np.uint32) << 16).view(np.float32)
    assert np.isfinite(got32).all()
    assert rel_err(got32, ref) < TOL["bf16"]
    # element-wise too: |C| ~ sqrt(K)/3 = 30, bf16 rounding of the result 2^-9 relative
    assert np.abs(got32 - ref).max() < 0.5
    del A32, B32, Ab, Bf
    # preemptible launch with the executor's context: same bits
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)
    assert st.enable_checkpoints(p) > 0
    dC.fill32(0x7FC07FC0)
    info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
    stream.sync()
    assert info.total_tiles == 1024 and st.stop_index() == -1
    assert np.array_equal(dC.download(np_dtype=np.uint16).reshape(n, n), base)
    for frac in (0.25, 0.5, 0.75):
        st.reset(); st.clear_stop(); flag.set(0)
        gp.check(gp.lib().gp_ckpt_reset_async(gp.vp(st.ckpt.ptr), None))
        dC.fill32(0x7FC07FC0)
        # 256 resident workgroups, 32 counters owning 32 consecutive tiles each: the first claims of
        # every counter are made at once, so "after frac of the tiles" is claim number frac * 32
        # of one counter's slice (here the sixth counter's)
        info = gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0, inject_at=5 * 32 + int(frac * 32)), stream)
        assert info.grid == 256
        stream.sync()
        assert flag.get() == 1 and st.stop_index() == 0, frac
        part = dC.download(np_dtype=np.uint16)
        assert (part == 0x7FC0).any(), "the kernel was not interrupted"
        relaunches = 0
        flag.set(0)
        while st.stop_index() != -1 or relaunches == 0:
            st.clear_stop()
            gp.launch("gp_launch_gemm", p, st.ctx(kernel_id=0), stream)
            stream.sync()
            relaunches += 1
            assert relaunches < 4
        assert np.array_equal(dC.download(np_dtype=np.uint16).reshape(n, n), base), f"resume after {frac:.0%} differs"


# ---- layer-norm prologue -----------------------------------------------------------------------------
@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("M,N,K,act", [(128, 2304, 768, 0), (128, 3072, 768, 2), (100, 72, 256, 1), (384, 200, 832, 0)])
def test_gemm_with_layernorm_prologue_has_the_bits_of_two_launches(gp, dt, M, N, K, act):
    """gp_launch_gemm with ln_gamma set = gp_launch_layernorm, then gp_launch_gemm: same C, same normalised
    rows, bit for bit (BERT-base's QKV and first FFN projection at sequence 128 among the shapes); within
    tolerance of the oracle's layer-norm and GEMM; stopped at a tile boundary and resumed, still the same."""
    rng = np.random.default_rng(M + N + K)
    dtype = gp.DTYPE_BY_NAME[dt]
    es = gp.DTYPE_SIZE[dtype]
    X = O.round_to(rng.normal(0.1, 1.5, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32) * 0.05, dt)
    gamma = O.round_to(rng.uniform(0.5, 1.5, K).astype(np.float32), dt)
    beta = O.round_to(rng.normal(0, 0.2, K).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt)
    res = O.round_to(rng.uniform(-1, 1, (M, N)).astype(np.float32), dt)
    dX, dB, dg, dbeta, dbias, dres = (gp.DevBuf.from_array(a, dtype) for a in (X, B, gamma, beta, bias, res))
    dLN, dC = gp.DevBuf(M * K * es), gp.DevBuf(M * N * es)
    # two launches
    gp.launch("gp_launch_layernorm", gp.LayernormParams(dtype, M, K, dX.ptr, None, dg.ptr, dbeta.ptr, dLN.ptr, 1e-12))
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dLN.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, bias=dbias.ptr,
                      residual=dres.ptr, alpha=1.0, act=act, batch=1)
    # the model loader fuses only where the launcher's own choice for the plain GEMM sums K as the prologue body does
    assert gp.lib().gp_gemm_ln_supported(C.byref(p)) == (1 if K >= 768 else 0)  # K = 256 runs on a body that keeps K in one wavefront
    p.tile_m = p.tile_n = 32
    p.variant = gp.MAT_PIPE_SPLITK  # K split over four wavefronts: the order of the wide bodies and of the prologue body
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    ln_two, c_two = dLN.download().copy(), dC.download().copy()
    ln_ref = O.round_to(O.layernorm(X, gamma, beta, 1e-12), dt)
    assert rel_err(dLN.download(dtype, (M, K)), ln_ref) < TOL[dt]
    assert rel_err(dC.download(dtype, (M, N)), O.gemm_bias_act(ln_ref, B, bias, res, act, b_is_nk=True)) < TOL[dt]
    # one launch
    dLN.fill32(0x7E007E00); dC.fill32(0x7E007E00)
    p.A = dX.ptr
    p.tile_m = p.tile_n = p.variant = 0
    p.ln_gamma, p.ln_beta, p.ln_out, p.ln_eps = dg.ptr, dbeta.ptr, dLN.ptr, 1e-12
    info = gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    assert info.total_tiles == ((M + 31) // 32) * ((N + 63) // 64)
    assert np.array_equal(dLN.download(), ln_two) and np.array_equal(dC.download(), c_two)
    # preempted and resumed
    flag = gp.Flag()
    total = info.total_tiles
    for groups, wgs in ((1, 4), (32, 0)):
        st = gp.BlpState(1, flag, groups)
        for frac in (0.3, 0.8):
            st.reset(); st.clear_stop(); flag.set(0)
            dLN.fill32(0); dC.fill32(0)
            gp.launch("gp_launch_gemm", p, st.ctx(inject_at=int(frac * total), max_workgroups=wgs, fresh=1))
            gp.check(gp.lib().gp_stream_sync(None))
            assert flag.get() == 1
            flag.set(0)
            st.clear_stop()
            gp.launch("gp_launch_gemm", p, st.ctx())
            gp.check(gp.lib().gp_stream_sync(None))
            assert np.array_equal(dLN.download(), ln_two) and np.array_equal(dC.download(), c_two), (groups, frac)


def test_layernorm_prologue_is_refused_where_it_does_not_fit(gp):
    dA = gp.DevBuf(1 << 20)
    def params(**kw):
        base = dict(dtype=gp.F16, M=128, N=256, K=768, A=dA.ptr, lda=768, B=dA.ptr, ldb=768, b_is_nk=1, C=dA.ptr, ldc=256, alpha=1.0, batch=1)
        base.update(kw)
        return gp.GemmParams(**base)
    assert gp.lib().gp_gemm_ln_supported(C.byref(params())) == 1
    for kw in (dict(dtype=gp.F32), dict(K=1024, lda=1024, ldb=1024), dict(K=72, lda=72, ldb=72), dict(lda=776), dict(b_is_nk=0, ldb=256), dict(batch=2), dict(M=1 << 16)):
        p = params(**kw)
        assert gp.lib().gp_gemm_ln_supported(C.byref(p)) == 0, kw
        p.ln_gamma = p.ln_beta = p.ln_out = dA.ptr
        with pytest.raises(gp.GpError):
            gp.launch("gp_launch_gemm", p)


# ---- a kernel started eagerly behind a stopped one -------------------------------------------------

def _chain_second(gp, family, dX_ptr, M, K, dtype, es, rng, dt):
    """The second kernel of a two-kernel chain, reading the first one's output (M x K): (params, output buffer, kept buffers)."""
    N = 256
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32) * 0.05, dt)
    dB, dC = gp.DevBuf.from_array(B, dtype), gp.DevBuf(M * N * es)
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dX_ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, alpha=1.0, act=gp.ACT_RELU, batch=1)
    keep = [dB]
    if family == "pipe":
        p.tile_m = p.tile_n = 64; p.variant = gp.MAT_PIPE
    elif family == "wide":
        p.tile_m = p.tile_n = 32; p.variant = gp.MAT_WIDE
    elif family == "ln":
        gamma = O.round_to(rng.uniform(0.5, 1.5, K).astype(np.float32), dt)
        beta = O.round_to(rng.normal(0, 0.2, K).astype(np.float32), dt)
        dg, dbeta, dLN = gp.DevBuf.from_array(gamma, dtype), gp.DevBuf.from_array(beta, dtype), gp.DevBuf(M * K * es)
        p.ln_gamma, p.ln_beta, p.ln_out, p.ln_eps = dg.ptr, dbeta.ptr, dLN.ptr, 1e-12
        keep += [dg, dbeta, dLN]
    return p, dC, keep


@pytest.mark.parametrize("family,K", [("pipe", 512), ("pipe", 64), ("wide", 768), ("wide", 64), ("ln", 768), ("ln", 64)])
def test_kernel_started_eagerly_behind_a_stopped_one_withdraws_every_claim(gp, family, K):
    """Kernel N is stopped late by an injected flag; kernel N+1, which reads N's output, is queued behind it as a first
    launch with an eager start (fresh = 2): its workgroups begin their tiles before they know of the stop, find it with
    their first operands, withdraw their claims (every count back to zero, every bit clear) and write nothing.
    After the resume of both the chain's output has the bits of an uninterrupted run.  In every body family with an
    early look (pipelined, wide, layer-norm prologue), also with a K of one step."""
    dt = "f16"
    dtype, es = gp.DTYPE_BY_NAME[dt], 2
    rng = np.random.default_rng(K + len(family))
    M, K0 = 1024, 256  # kernel N: 32 x K/32 tiles of 32 x 32 on 32 workgroups, so that its claims go through the counters
    A = O.round_to(rng.uniform(-1, 1, (M, K0)).astype(np.float32), dt)
    W0 = O.round_to(rng.uniform(-1, 1, (K, K0)).astype(np.float32) * 0.1, dt)
    dA, dW0, dX = gp.DevBuf.from_array(A, dtype), gp.DevBuf.from_array(W0, dtype), gp.DevBuf(M * K * es)
    p0 = gp.GemmParams(dtype=dtype, M=M, N=K, K=K0, A=dA.ptr, lda=K0, B=dW0.ptr, ldb=K0, b_is_nk=1, C=dX.ptr, ldc=K, alpha=1.0, batch=1,
                       tile_m=32, tile_n=32, variant=gp.MAT_PIPE_SPLITK)
    p1, dC, keep = _chain_second(gp, family, dX.ptr, M, K, dtype, es, rng, dt)
    # uninterrupted chain, plain launches
    gp.launch("gp_launch_gemm", p0); gp.launch("gp_launch_gemm", p1)
    gp.check(gp.lib().gp_stream_sync(None))
    want_x, want_c = dX.download().copy(), dC.download().copy()
    want_ln = keep[-1].download().copy() if family == "ln" else None
    flag = gp.Flag()
    st = gp.BlpState(2, flag, 32)
    G = 32
    # kernel N: few workgroups, claims through the counters, so that its polls see the flag it raises itself
    dX.fill32(0); dC.fill32(0x7E007E00)
    if family == "ln":
        keep[-1].fill32(0x7E007E00)
    info0 = gp.launch("gp_launch_gemm", p0, st.ctx(kernel_id=0, inject_at=info_total(M, K) // 2, max_workgroups=8, fresh=1, poll_every=1))
    assert info0.fixed_claims == 0 and info0.total_tiles == info_total(M, K)
    info1 = gp.launch("gp_launch_gemm", p1, st.ctx(kernel_id=1, fresh=2))
    gp.check(gp.lib().gp_stream_sync(None))
    assert info1.fixed_claims == 1, "the second kernel must have a workgroup per claim for this test"
    assert flag.get() == 1 and st.stop_index() == 0
    lines1 = st.counters().reshape(2, G, 16)[1]
    assert not lines1.any(), "every eager claim of the queued kernel must have been withdrawn"
    assert np.all(dC.download(np_dtype=np.uint16) == 0x7E00), "the queued kernel wrote output on incomplete input"
    if family == "ln":
        assert np.all(keep[-1].download(np_dtype=np.uint16) == 0x7E00), "the queued kernel stored normalised rows of incomplete input"
    x_part = dX.download(np_dtype=np.uint16).reshape(M // 32, 32, K // 32, 32)
    assert (x_part == 0).all(axis=(1, 3)).any(), "kernel N was not really interrupted"
    # resume (executor.cpp:280-298): stop index re-armed, counters kept, kernels from the stopped one on
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_gemm", p0, st.ctx(kernel_id=0, max_workgroups=8, poll_every=1))
    gp.launch("gp_launch_gemm", p1, st.ctx(kernel_id=1))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == -1
    assert np.array_equal(dX.download(), want_x) and np.array_equal(dC.download(), want_c)
    if family == "ln":
        assert np.array_equal(keep[-1].download(), want_ln)
    assert st.counters().reshape(2, G, 16)[1][:, 0].sum() == info1.total_tiles


def info_total(M, N, tile=32):
    return -(-M // tile) * -(-N // tile)


def test_device_time_stamps_of_a_preemption(gp):
    """gp_preempt_ctx::stamps: the stop is stamped by the workgroup that records it, every workgroup that leaves
    with a stop recorded stamps its exit, the first claim after the stamps were cleared is stamped; all on the
    device's constant-rate clock, which gp_device_clock ties to the host's monotonic clock."""
    import time
    A, B, bias, p, dC, keep = _config1(gp, 64)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    base = dC.download(gp.F32, (1024, 1024)).copy()
    tick, off = C.c_double(0), C.c_double(0)
    gp.check(gp.lib().gp_device_clock(None, 16, C.byref(tick), C.byref(off), None))
    assert 1.0 <= tick.value <= 100.0  # 100 MHz on this GPU: 10 ns
    to_host_ns = lambda ticks: ticks * tick.value + off.value
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)
    st.enable_stamps()
    WGS = 32
    t0 = time.monotonic_ns()
    info = gp.launch("gp_launch_gemm", p, st.ctx(inject_at=100, max_workgroups=WGS, fresh=1, poll_every=1))
    gp.check(gp.lib().gp_stream_sync(None))
    t1 = time.monotonic_ns()
    assert st.stop_index() == 0 and info.fixed_claims == 0
    stop, first, last_exit, exits = st.read_stamps()
    assert stop and first and last_exit
    assert first <= stop <= last_exit           # claims began before the stop; the tiles owed were finished after it
    assert 1 <= exits <= WGS
    assert (last_exit - stop) * tick.value < 5e6  # the drain of 64 x 64 tiles: far below 5 ms
    slack = 200e3  # the offset is good to a few microseconds; host-side launch and sync cost tens
    assert t0 - slack <= to_host_ns(first) <= to_host_ns(last_exit) <= t1 + slack
    # resume with cleared stamps: a first claim, no stop, every workgroup stamps its exit
    st.stamps.upload(np.zeros(st.STAMP_WORDS, np.uint64))
    flag.set(0)
    st.clear_stop()
    info = gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=WGS, poll_every=1))
    gp.check(gp.lib().gp_stream_sync(None))
    stop2, first2, last2, exits2 = st.read_stamps()
    assert stop2 == 0 and exits2 == info.grid and last_exit < first2 < last2
    assert np.array_equal(dC.download(gp.F32, (1024, 1024)), base)
    # fixed claims (a workgroup per tile) with the flag already up: the spare workgroups record and stamp the stop
    st.reset(); st.stamps.upload(np.zeros(st.STAMP_WORDS, np.uint64))
    flag.set(1)
    info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))
    gp.check(gp.lib().gp_stream_sync(None))
    assert info.fixed_claims == 1 and st.stop_index() == 0
    stop3, first3, last3, exits3 = st.read_stamps()
    assert stop3 and first3 and last3 >= stop3 and exits3 >= 1


@pytest.mark.parametrize("family", ["wide", "pipe", "pipe_two_rounds"])
def test_long_tiles_are_given_up_on_a_stop_and_redone_bit_exact(gp, family):
    """Tiles of 3 x 10^7 multiply-adds (about 100 us each; VGG-16's 25088-deep dense layer and ResNet-50's fp32
    7 x 7 stage have such tiles) in a launch that has a workgroup per tile: with gp_preempt_ctx::done the launch keeps
    a workgroup in front of its workers that reads the flag until they have all left, and the tiles look at the stop
    index every few K-stages.  A flag raised by the host while the tiles run is recorded within microseconds, the
    tiles are given up (their claims withdrawn), the launch is over long before a tile would have ended, and the
    relaunch computes them from the start: the bits of an uninterrupted run."""
    import time
    dt, dtype = "f16", gp.F16
    if family == "wide":
        M, N, K, tm, tn, variant = 64, 2048, 32768, 32, 32, gp.MAT_WIDE
    elif family == "pipe":
        M, N, K, tm, tn, variant = 1024, 1024, 8192, 64, 64, gp.MAT_PIPE
    else:
        # 320 tiles of 128 x 128, one to a compute unit: two rounds of workgroups, a workgroup per claim all the same
        # (a persistent grid would have to finish the tiles it is in), the front workgroup in one of the 256 places
        M, N, K, tm, tn, variant = 2560, 2048, 4096, 128, 128, gp.MAT_PIPE
    rng = np.random.default_rng(K)
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32) * 0.02, dt)
    dA, dB, dC = gp.DevBuf.from_array(A, dtype), gp.DevBuf.from_array(B, dtype), gp.DevBuf(M * N * 2)
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, alpha=1.0, act=gp.ACT_RELU, batch=1,
                      tile_m=tm, tile_n=tn, variant=variant)
    stream = gp.Stream(1)
    e0, e1 = gp.Event(), gp.Event()
    e0.record(stream)
    gp.launch("gp_launch_gemm", p, None, stream)
    e1.record(stream); e1.sync()
    whole_us = e0.elapsed_ms(e1) * 1e3
    base = dC.download().copy()
    assert rel_err(dC.download(dtype, (M, N))[:8], O.gemm_bias_act(A[:8], B, None, None, gp.ACT_RELU, b_is_nk=True)) < TOL[dt]
    tick, off = C.c_double(0), C.c_double(0)
    gp.check(gp.lib().gp_device_clock(None, 8, C.byref(tick), C.byref(off), None))
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)
    st.enable_done_counters()
    st.enable_stamps()
    given_up = 0
    for attempt in range(6):
        st.reset(); st.clear_stop(); flag.set(0)
        st.stamps.upload(np.zeros(st.STAMP_WORDS, np.uint64))
        dC.fill32(0x7E007E00)
        info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1), stream)
        t0 = time.perf_counter()
        while time.perf_counter() - t0 < 15e-6 * (attempt + 1):  # the flag lands at another depth of the tiles every time
            pass
        flag.set(1)
        stream.sync()
        assert info.fixed_claims == 1 and info.front == 8 and info.total_tiles == (M // tm) * (N // tn)
        made = int(st.counters().reshape(32, 16)[:, 0].sum())
        left = int(st.done.download(np_dtype=np.int32).reshape(32, 16)[:, 0].sum())
        assert left == info.grid - info.front  # every worker of the launch counted itself on its way out
        stop, first, last_exit, exits = st.read_stamps()
        if st.stop_index() == 0 and made < info.total_tiles:
            given_up += 1
            # the launch was over within microseconds of the recorded stop, not a tile's length later
            assert (last_exit - stop) * tick.value < 25e3, ((last_exit - stop) * tick.value, whole_us)
            part = dC.download(np_dtype=np.uint16).reshape(M // tm, tm, N // tn, tn)
            untouched = int((part == 0x7E00).all(axis=(1, 3)).sum())
            assert untouched == info.total_tiles - made  # a tile that was given up wrote nothing
        # the host's resume: flag down, stop index re-armed, the same kernel again (its second launch since the reset)
        flag.set(0)
        st.clear_stop()
        gp.launch("gp_launch_gemm", p, st.ctx(done_launches=1), stream)
        stream.sync()
        assert st.stop_index() == -1 and np.array_equal(dC.download(), base), attempt
        assert int(st.counters().reshape(32, 16)[:, 0].sum()) == info.total_tiles
    assert given_up >= 1, f"no attempt stopped the launch while its tiles ran (a plain launch takes {whole_us:.0f} us)"


_LOOKS_SWEEP = r'''
import sys, numpy as np
sys.path.insert(0, sys.argv[1])
from gpreempt_amd import capi as gp
gp.init(0)
rng = np.random.default_rng(11)
flag = gp.Flag()
cases = 0
for variant, tm, tn, M, N, ks in ((gp.MAT_PIPE, 64, 64, 256, 256, (64, 128, 192, 256, 320, 704, 768, 832, 1280)),
                                  (gp.MAT_PIPE, 128, 128, 256, 256, (64, 192, 256, 704, 1216)),
                                  (gp.MAT_WIDE, 32, 32, 64, 128, (1024, 2048, 3072, 5120, 9216))):
    for K in ks:
        A = rng.uniform(-1, 1, (M, K)).astype(np.float16)
        B = (rng.uniform(-1, 1, (N, K)) * 0.05).astype(np.float16)
        dA, dB, dC = gp.DevBuf.from_array(A, gp.F16), gp.DevBuf.from_array(B, gp.F16), gp.DevBuf(M * N * 2)
        p = gp.GemmParams(dtype=gp.F16, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, alpha=1.0, act=gp.ACT_NONE,
                          batch=1, tile_m=tm, tile_n=tn, variant=variant)
        gp.launch("gp_launch_gemm", p, None)
        gp.check(gp.lib().gp_stream_sync(None))
        base = dC.download().copy()
        tiles = (M // tm) * (N // tn)
        st = gp.BlpState(1, flag, 32)
        st.enable_done_counters()
        # (1) no stop: the bits of the plain launch, and every worker counted itself exactly once
        flag.set(0); st.reset(); st.clear_stop(); dC.fill32(0x7E007E00)
        info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))
        gp.check(gp.lib().gp_stream_sync(None))
        assert info.fixed_claims == 1 and info.front == 8 and info.total_tiles == tiles, (variant, tm, K, info.fixed_claims, info.front)
        assert np.array_equal(dC.download(), base), ("bits", variant, tm, K)
        done = int(st.done.download(np_dtype=np.int32).reshape(32, 16)[:, 0].sum())
        assert done == info.grid - info.front, ("done", variant, tm, K, done, info.grid)
        # (2) the flag up before the launch: tiles are given up wherever they are; the relaunch finishes the rest
        flag.set(1); st.reset(); st.clear_stop(); dC.fill32(0x7E007E00)
        info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))
        gp.check(gp.lib().gp_stream_sync(None))
        made = int(st.counters().reshape(32, 16)[:, 0].sum())
        done = int(st.done.download(np_dtype=np.int32).reshape(32, 16)[:, 0].sum())
        assert done == info.grid - info.front, ("done after stop", variant, tm, K, done)
        part = dC.download(np_dtype=np.uint16).reshape(M // tm, tm, N // tn, tn)
        assert int((part == 0x7E00).all(axis=(1, 3)).sum()) == tiles - made, ("untouched", variant, tm, K, made)
        flag.set(0); st.clear_stop()
        gp.launch("gp_launch_gemm", p, st.ctx(done_launches=1))
        gp.check(gp.lib().gp_stream_sync(None))
        assert np.array_equal(dC.download(), base), ("bits after resume", variant, tm, K)
        assert int(st.counters().reshape(32, 16)[:, 0].sum()) == tiles
        cases += 1
print("OK", cases)
'''


def test_looks_at_every_count_of_k_steps(gp):
    """The instantiation that looks again during a tile, on tiles of 1 to 20 K-steps (no run of 8, exactly one, one and
    a rest, two; fewer K-steps than stages) and on split-K tiles of 4 to 36 stages: the bits of the plain launch, every
    worker counted once in gp_preempt_ctx::done whether it finished its tile or gave it up, and a launch that finds
    the flag up leaves its tiles unwritten for the relaunch.  The threshold that selects the instantiation is read
    once per process, hence the child process with GPREEMPT_LONG_TILE_MACS=1."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", _LOOKS_SWEEP, root], capture_output=True, text=True, timeout=110,
                         env={**os.environ, "GPREEMPT_LONG_TILE_MACS": "1"})
    assert out.returncode == 0 and out.stdout.strip().startswith("OK 19"), (out.stdout[-300:], out.stderr[-1500:])
