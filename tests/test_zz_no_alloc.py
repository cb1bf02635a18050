"""gp_launch_gemm_noalloc (the preemptible GEMM launch that allocates nothing: its claim counters
and stop index live in a device array inside the library) against gp_launch_gemm with a
caller-allocated context, bit for bit, on two calls in a row, the second with a smaller input."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle as O

pytestmark = pytest.mark.gpu

CLEAR, REARM = 1, 2


def _problem(gp, dt, M, N, K, seed):
    rng = np.random.default_rng(seed)
    dtype = gp.DTYPE_BY_NAME[dt]
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), dt)
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), dt)
    bias = O.round_to(rng.uniform(-0.1, 0.1, N).astype(np.float32), dt)
    bufs = [gp.DevBuf.from_array(x, dtype) for x in (A, B, bias)]
    dC = gp.DevBuf(M * N * gp.DTYPE_SIZE[dtype])
    p = gp.GemmParams(dtype=dtype, M=M, N=N, K=K, A=bufs[0].ptr, lda=K, B=bufs[1].ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N,
                      bias=bufs[2].ptr, alpha=1.0, act=gp.ACT_RELU, batch=1)
    ref = O.gemm_bias_act(A, B, bias, act=O.ACT_RELU, b_is_nk=True)
    return p, dC, bufs, ref, dtype


def _noalloc(gp, p, flag, slot, mode, inject_at, stop_out, stream=None):
    info = gp.LaunchInfo()
    gp.check(gp.lib().gp_launch_gemm_noalloc(C.byref(p), gp.vp(flag.dev) if flag else None, slot, mode, inject_at,
                                             gp.vp(stop_out.ptr) if stop_out else None, stream.h if stream else None, C.byref(info)))
    return info


def test_noalloc_gemm_matches_the_allocating_entry_point(gp):
    flag = gp.Flag()
    stop_out = gp.DevBuf(4)
    tol = {"f16": 1e-2, "f32": 1e-4}
    # two calls in a row on the same slot, the second smaller (and ragged): the array keeps the
    # first call's counters, so the second must clear what has to start at zero
    for dt, (M, N, K), seed in (("f16", (1024, 1024, 512), 1), ("f16", (300, 264, 72), 2), ("f32", (130, 264, 40), 3)):
        p, dC, bufs, ref, dtype = _problem(gp, dt, M, N, K, seed)
        st = gp.BlpState(1, flag, 32)
        flag.set(0)
        dC.fill32(0)
        want_info = gp.launch("gp_launch_gemm", p, st.ctx(fresh=1))
        gp.check(gp.lib().gp_stream_sync(None))
        want = dC.download().copy()
        assert float(np.abs(gp.from_storage(want, dtype).reshape(M, N) - ref).max() / np.abs(ref).max()) < tol[dt]
        dC.fill32(0)
        stop_out.fill32(0x55)
        info = _noalloc(gp, p, flag, 0, CLEAR | REARM, -1, stop_out)
        gp.check(gp.lib().gp_stream_sync(None))
        assert (info.total_tiles, info.grid, info.fixed_claims) == (want_info.total_tiles, want_info.grid, want_info.fixed_claims)
        assert np.array_equal(dC.download(), want), (dt, M, N, K)
        assert stop_out.download(np_dtype=np.int32)[0] == -1


def test_noalloc_gemm_preempt_and_resume(gp):
    """Stopped by an injected flag, continued with mode 0 counters (REARM only): the same bits as
    the uninterrupted run; another slot is untouched by it."""
    flag = gp.Flag()
    stop_out = gp.DevBuf(4)
    # 4096 tiles, more than the GPU holds at once, so claims go through the counters; deep enough that the
    # tiles left after the injection outlast the flag's trip through host memory.  Claim 2064 is the 16th
    # of 128 in its counter's slice: the flag goes up with most of every slice still to be handed out.
    p, dC, bufs, ref, dtype = _problem(gp, "f16", 4096, 4096, 1024, 5)
    p.tile_m = p.tile_n = 64
    flag.set(0)
    gp.launch("gp_launch_gemm", p)
    gp.check(gp.lib().gp_stream_sync(None))
    want = dC.download().copy()
    for slot in (3, 63):
        dC.fill32(0)
        flag.set(0)
        info = _noalloc(gp, p, flag, slot, CLEAR | REARM, 2064, stop_out)
        gp.check(gp.lib().gp_stream_sync(None))
        assert flag.get() == 1 and stop_out.download(np_dtype=np.int32)[0] == slot
        assert not np.array_equal(dC.download(), want), "the kernel was not interrupted"
        # flag still up: a relaunch that re-arms stops again at once and claims (almost) nothing
        _noalloc(gp, p, flag, slot, REARM, -1, stop_out)
        gp.check(gp.lib().gp_stream_sync(None))
        assert stop_out.download(np_dtype=np.int32)[0] == slot
        flag.set(0)
        _noalloc(gp, p, flag, slot, REARM, -1, stop_out)
        gp.check(gp.lib().gp_stream_sync(None))
        assert stop_out.download(np_dtype=np.int32)[0] == -1
        assert np.array_equal(dC.download(), want), slot
        # everything is claimed now: a continuation (mode 0) writes nothing
        dC.fill32(0)
        _noalloc(gp, p, flag, slot, 0, -1, None)
        gp.check(gp.lib().gp_stream_sync(None))
        assert not dC.download().any()


def test_noalloc_gemm_rejects_what_the_scratch_cannot_hold(gp):
    p, dC, bufs, ref, dtype = _problem(gp, "f16", 64, 64, 64, 7)
    for slot in (-1, 64, 1000):
        with pytest.raises(gp.GpError) as e:
            _noalloc(gp, p, None, slot, 3, -1, None)
        assert e.value.status == gp.OUTOFRANGE and "slot" in str(e.value)
    with pytest.raises(gp.GpError):
        _noalloc(gp, p, None, 0, 7, -1, None)
    # 2^25 tiles of 32 x 32 would need more claims than a slot counts
    big = gp.GemmParams(dtype=dtype, M=32 * 8192, N=32 * 4096, K=64, A=bufs[0].ptr, lda=64, B=bufs[1].ptr, ldb=64, b_is_nk=1, C=dC.ptr, ldc=32 * 4096,
                        alpha=1.0, batch=1, tile_m=32, tile_n=32, variant=gp.MAT_PIPE_SPLITK)
    with pytest.raises(gp.GpError) as e:
        _noalloc(gp, big, None, 0, 3, -1, None)
    assert "tiles" in str(e.value)
