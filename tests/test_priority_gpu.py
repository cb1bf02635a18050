"""gpreempt.h's call shapes (set_priority, hipGetFd / hipSuspendStreams / hipResumeStreams) through
the C view, the gate kernels that replace gpu_block / gpu_noop (reference src/block.cu:1-7, used by
src/cuda-clients/gpreemptclient.cpp:74-81), and a three-level scenario (BASELINE config 4's
distinguishing feature: one flag word per priority boundary)."""
import ctypes as C
import json
import time

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_set_priority_relabels_the_tenant_stream(gp):
    from gpreempt_amd import executor as gx
    s = gp.Stream(1)
    pr = C.c_int(-1)
    gp.check(gp.lib().gp_stream_priority(s.h, C.byref(pr)))
    assert pr.value == 1
    assert gx.lib().gpx_set_priority(s.h, 0) == 0          # reference: 0 = high, 1 = low; returns 0
    gp.check(gp.lib().gp_stream_priority(s.h, C.byref(pr)))
    assert pr.value == 0
    assert gx.lib().gpx_set_priority(s.h, 2) == 0          # a third level (config 4)
    gp.check(gp.lib().gp_stream_priority(s.h, C.byref(pr)))
    assert pr.value == 2
    assert gx.lib().gpx_set_priority(s.h, -1) == -1        # bad priority
    assert gx.lib().gpx_set_priority(None, 0) == -1        # NvRmQuery finds no context
    gp.check(gp.lib().gp_stream_priority(s.h, C.byref(pr)))
    assert pr.value == 2
    s.destroy()


def _word(gx, fd, level):
    """current value of the flag word that `level` obeys"""
    assert gx.lib().gpx_domain_flag(fd, level)
    return gx.lib().gpx_domain_flag_value(fd, level)


def test_suspend_and_resume_streams_raise_and_lower_flag_words(gp):
    from gpreempt_amd import executor as gx
    L = gx.lib()
    fd = L.gpx_domain_create(3)
    assert fd >= 0 and L.gpx_get_fd() == fd
    assert L.gpx_domain_flag(fd, 0) is None                 # the highest level obeys no word
    assert _word(gx, fd, 1) == 0 and _word(gx, fd, 2) == 0
    two = (C.c_int * 1)(2)
    assert L.gpx_suspend_streams(fd, two, 1) == 0           # stop the lowest level only
    assert _word(gx, fd, 1) == 0 and _word(gx, fd, 2) == 1
    both = (C.c_int * 2)(1, 2)
    assert L.gpx_suspend_streams(fd, both, 2) == 0
    assert _word(gx, fd, 1) == 1 and _word(gx, fd, 2) == 1
    assert L.gpx_resume_streams(fd, both, 2) == 0
    assert _word(gx, fd, 1) == 0 and _word(gx, fd, 2) == 1  # level 2 was suspended twice
    assert L.gpx_resume_streams(fd, two, 1) == 0
    assert _word(gx, fd, 2) == 0
    bad = (C.c_int * 1)(0)
    assert L.gpx_suspend_streams(fd, bad, 1) == -1          # level 0 cannot be stopped
    assert L.gpx_suspend_streams(fd + 77, two, 1) == -1     # unknown handle
    # requests: a level-1 request stops level 2 only; a level-0 request stops both
    assert L.gpx_domain_begin(fd, 1) == 0
    assert _word(gx, fd, 1) == 0 and _word(gx, fd, 2) == 1
    assert L.gpx_domain_begin(fd, 0) == 0
    assert _word(gx, fd, 1) == 1 and _word(gx, fd, 2) == 1
    assert L.gpx_domain_end(fd, 0) == 0
    assert _word(gx, fd, 1) == 0 and _word(gx, fd, 2) == 1
    assert L.gpx_domain_end(fd, 1) == 0
    assert _word(gx, fd, 2) == 0
    # a suspended level's kernel really leaves: a preemptible GEMM polls the word of level 2
    assert L.gpx_suspend_streams(fd, two, 1) == 0
    n = 1024
    a = gp.DevBuf.from_array(np.ones((n, n), np.float32), gp.F32)
    c = gp.DevBuf(4 * n * n)
    c.fill32(0)
    p = gp.GemmParams(dtype=gp.F32, M=n, N=n, K=n, A=a.ptr, lda=n, B=a.ptr, ldb=n, b_is_nk=1, C=c.ptr, ldc=n, alpha=1.0, batch=1, tile_m=64, tile_n=64)

    class W:  # a Flag-like view of the domain's word
        dev = L.gpx_domain_flag(fd, 2)
    st = gp.BlpState(1, W)
    info = gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=8))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == 0 and st.counters()[0] <= 8
    assert L.gpx_resume_streams(fd, two, 1) == 0
    st.clear_stop()
    gp.launch("gp_launch_gemm", p, st.ctx(max_workgroups=8))
    gp.check(gp.lib().gp_stream_sync(None))
    assert st.stop_index() == -1
    assert (c.download(gp.F32) == n).all()
    assert L.gpx_domain_destroy(fd) == 0
    assert L.gpx_get_fd() == -1


def test_gate_holds_the_stream_until_the_host_releases_it(gp):
    """gpu_block: the kernel queued behind the gate does not run before the host stores 1."""
    flag = gp.Flag()
    flag.set(0)
    s = gp.Stream(0)
    out = gp.DevBuf(256)
    out.fill32(0)
    timed_out = gp.DevBuf(4)
    timed_out.fill32(0)
    L = gp.lib()
    # two gates, as start_blocking_stream launches them; bounded at ~4 M polls (seconds)
    for _ in range(2):
        gp.check(L.gp_launch_gate(gp.vp(flag.dev), C.c_ulonglong(1 << 22), gp.vp(timed_out.ptr), s.h))
    gp.check(L.gp_fill32_async(gp.vp(out.ptr), C.c_uint32(0x1234), C.c_size_t(64), s.h))
    time.sleep(0.05)
    assert not s.idle(), "the gate let the stream through before its release"
    flag.set(1)  # end_blocking_stream
    t0 = time.perf_counter()
    s.sync()
    assert time.perf_counter() - t0 < 1.0
    host = np.empty(64, np.uint32)
    gp.check(L.gp_memcpy_d2h(host.ctypes.data_as(gp.vp), gp.vp(out.ptr), C.c_size_t(256)))
    assert (host == 0x1234).all()
    assert timed_out.download(np_dtype=np.int32)[0] == 0
    # an open gate is passed at once; the noop kernel runs and ends
    gp.check(L.gp_launch_gate(gp.vp(flag.dev), C.c_ulonglong(1 << 22), gp.vp(timed_out.ptr), s.h))
    gp.check(L.gp_launch_noop(s.h))
    s.sync()
    assert timed_out.download(np_dtype=np.int32)[0] == 0
    s.destroy()


def test_gate_gives_up_after_its_spin_limit(gp):
    """A release that never comes: the wait is bounded from the host side, the gate stores 1 to
    *timed_out, exits normally, and the stream carries on."""
    flag = gp.Flag()
    flag.set(0)
    s = gp.Stream(0)
    out = gp.DevBuf(256)
    out.fill32(0)
    timed_out = gp.DevBuf(4)
    timed_out.fill32(0)
    L = gp.lib()
    gp.check(L.gp_launch_gate(gp.vp(flag.dev), C.c_ulonglong(2000), gp.vp(timed_out.ptr), s.h))
    gp.check(L.gp_fill32_async(gp.vp(out.ptr), C.c_uint32(7), C.c_size_t(64), s.h))
    s.sync()
    assert flag.get() == 0
    assert timed_out.download(np_dtype=np.int32)[0] == 1
    assert (out.download(np_dtype=np.uint32) == 7).all()
    with pytest.raises(gp.GpError):
        gp.check(L.gp_launch_gate(gp.vp(flag.dev), C.c_ulonglong(0), None, s.h))  # an unbounded wait is refused
    s.destroy()


def _scenario(cfg):
    from gpreempt_amd import executor as gx
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_run_scenario(json.dumps(cfg).encode(), buf, C.c_size_t(len(buf)))
    assert rc == 0, buf.value[:400]
    return json.loads(buf.value.decode())


@pytest.mark.parametrize("policy", ["wb-chunk-async", "wb"])
def test_three_priority_levels(gp, policy):
    """Config 4 in small: BERT (level 0) over DenseNet (level 1) over VGG (level 2).  The middle
    tenant is stopped by level 0 and stops level 2; every request of every tenant returns the bits
    of that tenant's uninterrupted run."""
    cfg = {"time": 4.0, "policy": policy, "warmups": 3, "standalone_runs": 10, "verify_outputs": True, "tasks": [
        {"id": "hp", "load": {"type": "poisson", "frequency": 400, "seed": 3},
         "client": {"name": "hp_rt", "model_name": "bert@layers=4,s=128", "priority": 0, "launch_mode": "launch"}},
        {"id": "mid", "load": {"type": "poisson", "frequency": 150, "seed": 4},
         "client": {"name": "mid_be", "model_name": "densenet201@b=4,hw=128,l1=4,l2=8,l3=12,l4=8", "priority": 1, "launch_mode": "launch" if "chunk" in policy else "program"}},
        {"id": "be", "load": {"type": "continuous"},
         "client": {"name": "be_be", "model_name": "vgg16@b=8,hw=128,fc=1024", "priority": 2, "launch_mode": "launch" if "chunk" in policy else "program"}}]}
    rep = _scenario(cfg)
    t = rep["tasks"]
    assert t["hp"]["requests"] > 800 and t["mid"]["requests"] > 300 and t["be"]["requests"] > 20
    assert t["hp"]["preemptions"] == 0
    assert t["mid"]["preemptions"] > 5, "level 1 was never stopped by level 0"
    assert t["be"]["preemptions"] > t["mid"]["preemptions"], "level 2 is stopped by both higher levels"
    for k in ("hp", "mid", "be"):
        assert t[k]["outputMismatches"] == 0, (k, t[k]["outputMismatches"])
    # the reference's report shape (DISB): what scripts/plot/plot.py reads
    names = [r["clientName"] for r in rep["results"]]
    assert names == ["hp_rt", "mid_be", "be_be"]
    for r in rep["results"]:
        a = r["analyzers"][0]
        assert a["type"] == "basic" and a["avgThroughput(req/s)"] > 0
        for key in ("standAloneTotalLatency(us)", "avgPrepareInputLatency(us)", "avgPreprocessLatency(us)", "avgCopyInputLatency(us)",
                    "avgInferLatency(us)", "avgCopyOutputLatency(us)", "avgPostprocessLatency(us)", "avgTotalLatency(us)", "avgTotalLatencyIncrease(us)"):
            assert isinstance(a[key], int), key
        assert a["avgTotalLatencyIncrease(us)"] == a["avgTotalLatency(us)"] - a["standAloneTotalLatency(us)"]
    assert "beginTime" in rep and "endTime" in rep and isinstance(rep["benchmarkTime(s)"], int)


def test_config4_at_full_size_with_verified_outputs(gp):
    """BASELINE config 4 as the scenario file states it (BERT-base at 100 req/s over DenseNet-201 b4 at 50 req/s over
    VGG-16 b16 back to back, all at 224 x 224 and full width) for two seconds: every request of every tenant returns
    the bits of that tenant's uninterrupted run, and both lower levels were really stopped."""
    import os
    with open(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "gpreempt_amd", "config", "config4_bert_densenet201_vgg16.json")) as f:
        cfg = json.load(f)
    cfg.update({"time": 2.0, "warmups": 2, "standalone_runs": 5, "verify_outputs": True, "device_stamps": True})
    rep = _scenario(cfg)
    t = rep["tasks"]
    hp, mid, be = t["bert_rt"], t["densenet201_mid"], t["vgg16_be"]
    assert hp["requests"] > 100 and mid["requests"] > 40 and be["requests"] > 100
    assert mid["preemptions"] > 3 and be["preemptions"] > 50
    for k, v in t.items():
        assert v["outputMismatches"] == 0, (k, v["outputMismatches"])
    # the GPU's own account of the preemptions: the stop is recorded after the flag store, the last workgroup
    # leaves after that, and the host notices later still
    # (the two clocks are tied together to a few microseconds: hence the slack)
    ds = rep["deviceStamps(us)"]
    assert ds["flagStore_to_lastWorkgroupExit"]["count"] > 50
    assert -5 < ds["flagStore_to_lastWorkgroupExit"]["p50"] < rep["preemptLatency(us)"]["p50"] + 5
    assert -5 < ds["lastWorkgroupExit_to_hostNotices"]["p50"] < 100
    assert ds["stopRecorded_to_lastWorkgroupExit"]["count"] > 10 and ds["flagStore_to_stopRecorded"]["p50"] > -5
    assert ds["resubmission_to_firstTileClaimed"]["count"] > 50 and 0 < ds["resubmission_to_firstTileClaimed"]["p50"] < 500


def test_hp_gate_policy_option(gp):
    """The reference's blocking stream (gpreemptclient.cpp:74-81,232-235) as a scenario option: the
    high-priority tenant queues its kernels behind two gate kernels and releases them at once."""
    cfg = {"time": 2.0, "policy": "wb-chunk-async", "hp_gate": True, "hp_requests": 100, "warmups": 3, "standalone_runs": 10, "verify_outputs": True, "tasks": [
        {"id": "hp", "load": {"type": "poisson", "frequency": 300, "seed": 5},
         "client": {"name": "hp_rt", "model_name": "bert@layers=2,s=64", "priority": 0, "launch_mode": "launch"}},
        {"id": "be", "load": {"type": "continuous"},
         "client": {"name": "be_be", "model_name": "resnet50", "priority": 1, "launch_mode": "launch"}}]}
    rep = _scenario(cfg)
    assert rep["tasks"]["hp"]["requests"] >= 100 and rep["tasks"]["be"]["preemptions"] > 0
    assert rep["tasks"]["hp"]["outputMismatches"] == 0 and rep["tasks"]["be"]["outputMismatches"] == 0
    # a gate that had given up would have cost its whole spin limit (seconds)
    assert rep["tasks"]["hp"]["totalLatency(us)"]["max"] < 50000


def test_a_level_stays_up_across_back_to_back_requests(gp):
    """Requests of the high-priority tenant that arrive while one is being served follow it at once.  With
    "hold_backlog" (the default) the level's flag words stay up between the two, so the lower level is not sent
    back onto the GPU for an instant only to be stopped again; without it the words go down and up per request, as
    in the reference's client.  Either way every best-effort request returns the bits of an uninterrupted run."""
    def run(hold):
        cfg = {"time": 1.5, "policy": "wb-chunk-async", "warmups": 3, "standalone_runs": 10, "verify_outputs": True, "hold_backlog": hold, "tasks": [
            {"id": "hp", "load": {"type": "poisson", "frequency": 4000, "seed": 11},
             "client": {"name": "hp_rt", "model_name": "bert@layers=2,s=128", "priority": 0, "launch_mode": "launch"}},
            {"id": "be", "load": {"type": "continuous"},
             "client": {"name": "be_be", "model_name": "resnet50@b=2", "priority": 1, "launch_mode": "launch"}}]}
        return _scenario(cfg)["tasks"]
    held, plain = run(True), run(False)
    assert held["hp"]["levelHeldAcrossRequests"] > 50, held["hp"]
    assert plain["hp"]["levelHeldAcrossRequests"] == 0
    for t in (held, plain):
        assert t["hp"]["requests"] > 500 and t["be"]["requests"] > 20 and t["be"]["preemptions"] > 20
        assert t["be"]["outputMismatches"] == 0 and t["hp"]["outputMismatches"] == 0
    # a level that stays up stops the lower one less often for the same arrivals
    assert held["be"]["preemptions"] < plain["be"]["preemptions"]
