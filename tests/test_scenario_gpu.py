"""Two-tenant scenarios through the C view of the harness (gpx_run_scenario): every policy runs
to completion, serves the high-priority requests and, where it preempts, records preemptions.
Mirrors what the reference's client executables report (DISB result JSON, benchmark.h:40-60)."""
import ctypes as C
import json

import pytest

pytestmark = pytest.mark.gpu


def _run(policy, hp_requests=60, be_mode="program", hp_model="bert", be_model="resnet50"):
    from gpreempt_amd import executor as gx
    cfg = {
        "time": 3.0, "policy": policy, "hp_requests": hp_requests, "warmups": 3, "standalone_runs": 20,
        "tasks": [
            {"id": "hp", "load": {"type": "poisson", "frequency": 300, "seed": 7},
             "client": {"name": "hp", "model_name": hp_model, "priority": 0, "use_cuda_graph": False, "launch_mode": "launch", "preprocess_time": 0}},
            {"id": "be", "load": {"type": "continuous"},
             "client": {"name": "be", "model_name": be_model, "priority": 1, "use_cuda_graph": True, "launch_mode": be_mode, "preprocess_time": 0}},
        ],
    }
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_run_scenario(json.dumps(cfg).encode(), buf, C.c_size_t(len(buf)))
    assert rc == 0, buf.value[:400]
    return json.loads(buf.value.decode())


@pytest.mark.parametrize("policy", ["wb", "wb-async", "wb-chunk", "wb-chunk-async"])
def test_preempting_policies_serve_hp_and_preempt_be(gp, policy):
    rep = _run(policy, hp_requests=200)
    hp, be = rep["tasks"]["hp"], rep["tasks"]["be"]
    assert rep["policy"] == policy
    assert hp["requests"] >= 200
    assert be["requests"] > 0
    assert be["preemptions"] > 0, "the best-effort tenant was never interrupted"
    assert rep["preemptLatency(us)"]["count"] > 0
    # a drain is bounded by queued kernels x launch turnaround: far below a millisecond here
    assert 0 < rep["preemptLatency(us)"]["p50"] < 1000
    # co-run latency stays within a small factor of the isolated latency (np is ~50x on this pair): the
    # typical request tightly, the tail (arrivals queue behind one another at 300 Hz, and 1 request in 100
    # is two requests here) loosely
    assert hp["inferLatency(us)"]["p50"] < 2.5 * hp["standAloneTotalLatency(us)"], (hp["inferLatency(us)"], hp["standAloneTotalLatency(us)"])
    assert 0.5 < rep["hp_p99_vs_isolated"] < 8.0, rep["hp_p99_vs_isolated"]
    assert hp["preemptions"] == 0


@pytest.mark.parametrize("policy", ["np", "seq"])
def test_non_preempting_policies_complete(gp, policy):
    rep = _run(policy, hp_requests=30)
    hp, be = rep["tasks"]["hp"], rep["tasks"]["be"]
    assert hp["requests"] >= 30 and be["requests"] > 0
    assert be["preemptions"] == 0
    assert rep["preemptLatency(us)"]["count"] == 0


def test_unknown_model_is_reported(gp):
    from gpreempt_amd import executor as gx
    cfg = {"time": 1.0, "policy": "wb", "tasks": [{"id": "x", "load": {"type": "continuous"},
           "client": {"name": "x", "model_name": "no_such_model", "priority": 0}}]}
    buf = C.create_string_buffer(1 << 16)
    rc = gx.lib().gpx_run_scenario(json.dumps(cfg).encode(), buf, C.c_size_t(len(buf)))
    assert rc != 0


def _run_cfg(cfg):
    from gpreempt_amd import executor as gx
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_run_scenario(json.dumps(cfg).encode(), buf, C.c_size_t(len(buf)))
    assert rc == 0, buf.value[:400]
    return json.loads(buf.value.decode())


def test_pre_preemption_hints_hide_the_drain(gp):
    """gpreemptclient.cpp:203-219: a client that preprocesses for a while posts a hint, and the
    daemon raises the flag shortly before the kernels are due; under the waiting policy ("wb") the
    request then finds the GPU already vacated instead of waiting for the drain itself."""
    def cfg(hint_us):
        return {"time": 3.0, "policy": "wb", "hp_requests": 80, "warmups": 3, "standalone_runs": 20, "pre_preempt_hint_us": hint_us,
                "tasks": [
                    {"id": "hp", "load": {"type": "poisson", "frequency": 200, "seed": 11},
                     "client": {"name": "hp", "model_name": "bert", "priority": 0, "use_cuda_graph": False, "launch_mode": "launch", "preprocess_time": 400}},
                    {"id": "be", "load": {"type": "continuous"},
                     "client": {"name": "be", "model_name": "resnet50", "priority": 1, "use_cuda_graph": True, "launch_mode": "program", "preprocess_time": 0}}]}
    plain = _run_cfg(cfg(0))
    hinted = _run_cfg(cfg(150))
    assert plain["hints_fired"] == 0
    assert hinted["hints_fired"] >= 0.9 * hinted["tasks"]["hp"]["requests"]
    assert hinted["tasks"]["be"]["preemptions"] > 0
    # the drain no longer sits inside the request's GPU phase
    assert hinted["tasks"]["hp"]["inferLatency(us)"]["p50"] < plain["tasks"]["hp"]["inferLatency(us)"]["p50"] + 5.0


def test_graph_and_stencil_tenants_under_a_latency_critical_model(gp):
    """the reference's configs Y and Z in small: a periodic high-priority DNN over a miniWeather
    tenant and a graph tenant, all of which must make progress and be preempted"""
    cfg = {"time": 1.5, "policy": "wb-chunk-async", "tasks": [
        {"id": "hp", "load": {"type": "periodic", "frequency": 200},
         "client": {"name": "hp", "model_name": "toy", "priority": 0, "launch_mode": "launch"}},
        {"id": "mw", "load": {"type": "continuous"},
         "client": {"name": "mw", "model_name": "miniweather@nx=800,nz=400", "priority": 1, "launch_mode": "launch"}},
        {"id": "cc", "load": {"type": "continuous"},
         "client": {"name": "cc", "model_name": "cc@n=200000,deg=6,seed=2", "priority": 1, "launch_mode": "launch"}}]}
    rep = _run_cfg(cfg)
    t = rep["tasks"]
    assert t["hp"]["requests"] >= 250
    assert t["mw"]["requests"] > 50 and t["cc"]["requests"] > 50
    assert t["mw"]["preemptions"] + t["cc"]["preemptions"] > 20


def test_trace_load_serves_the_newest_arrival(gp):
    """DISB's "trace" load (third_party/disb/src/load.cpp:239-296): arrival times in milliseconds;
    an arrival whose successor is already due is skipped."""
    trace = [0, 5, 10, 200, 200, 200, 201, 400, 405, 410, 415, 1600]  # the last one falls past the end
    cfg = {"time": 1.0, "policy": "wb-chunk-async", "tasks": [
        {"id": "hp", "load": {"type": "trace", "trace": trace},
         "client": {"name": "hp", "model_name": "toy", "priority": 0, "launch_mode": "launch"}},
        {"id": "be", "load": {"type": "continuous"},
         "client": {"name": "be", "model_name": "resnet50", "priority": 1, "launch_mode": "launch"}}]}
    rep = _run_cfg(cfg)
    n = rep["tasks"]["hp"]["requests"]
    assert 7 <= n <= 11, n  # the burst at 200 ms collapses; nothing is served after the end
    assert rep["tasks"]["be"]["requests"] > 10


def test_exported_model_as_best_effort_tenant(gp, tmp_path):
    """A model directory in the reference's export format (plus the operator sidecar) takes the place of a
    built-in workload name in a task file: it is preempted by the high-priority tenant and every one of its
    outputs afterwards has the bits of its output when run alone."""
    import os
    import export_writer as EW
    from gpreempt_amd import executor as gx
    w, head = EW.resnet("f16", (1, 1, 1, 1), batch=4, hw=96)
    w.write(str(tmp_path / "exported_net"), head)
    os.environ["GPREEMPT_MODEL_PATH"] = str(tmp_path)
    cfg = {
        "time": 2.0, "policy": "wb-chunk-async", "hp_requests": 40, "warmups": 3, "standalone_runs": 10, "verify_outputs": True,
        "tasks": [
            {"id": "hp", "load": {"type": "poisson", "frequency": 400, "seed": 3},
             "client": {"name": "hp", "model_name": "bert@layers=2", "priority": 0, "use_cuda_graph": False, "launch_mode": "launch", "preprocess_time": 0}},
            {"id": "be", "load": {"type": "continuous"},
             "client": {"name": "be", "model_name": "exported_net", "priority": 1, "use_cuda_graph": False, "launch_mode": "launch", "preprocess_time": 0}},
        ],
    }
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_run_scenario(json.dumps(cfg).encode(), buf, C.c_size_t(len(buf)))
    assert rc == 0, buf.value[:400]
    rep = json.loads(buf.value.decode())
    hp, be = rep["tasks"]["hp"], rep["tasks"]["be"]
    assert hp["requests"] >= 40 and be["requests"] > 0 and be["preemptions"] > 0
    assert be["kernels"] == 1 + 1 + 1 + 4 * 4 + 1 + 1 + 1   # layout, stem, pool, four blocks of four convolutions, pool, classifier, softmax
    assert hp["outputMismatches"] == 0 and be["outputMismatches"] == 0


@pytest.mark.parametrize("mode", [2, 1, 0])
def test_preempt_probe_of_config2(gp, mode):
    """BASELINE config 2 through gpx_preempt_probe: ResNet-50 fp32 b1 stopped at random instants by the host and
    resumed (the protocol of src/tests/test-dnn-blp.cpp:36-42), fed kernel by kernel with a bounded queue (2), as
    one persistent program (1) or with every kernel launched at once as BLPExecutor::execute does (0).  Every mode
    reports its interruptions; the bounded queue, which is how a tenant is fed, drains in well under 50 us."""
    from gpreempt_amd import executor as gx
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_preempt_probe(b"resnet50", 80, mode, C.c_ulonglong(3), buf, C.c_size_t(len(buf)))
    assert rc == 0, buf.value[:400]
    r = json.loads(buf.value.decode())
    assert r["kernels"] > 50 and r["trials"] == 80 and r["interrupted"] > 40
    lat = r["preemptLatency(us)"]
    assert lat["count"] == r["interrupted"] and 0 < lat["mean"] < 400
    assert {"flagStore_to_stopRecorded", "stopRecorded_to_lastWorkgroupExit", "lastWorkgroupExit_to_hostNotices"} <= set(r["deviceStamps(us)"])
    assert all(k["samples"] > 0 and k["preempt_max(us)"] >= k["preempt_mean(us)"] > 0 for k in r["perKernel"])
    if mode == 2:
        assert lat["p99"] < 50, lat


def test_chunked_policy_with_an_event_per_chunk_still_works(gp, tmp_path):
    """The chunked policies keep their queue short through the launches' own start reports by default; with
    GPREEMPT_CHUNK_EVENTS=1 (read once per process, hence the child process) they fall back to an event behind
    every chunk of GPREEMPT_CHUNK kernels.  Both ways the tenant is preempted and every request returns the bits of
    an uninterrupted run."""
    import os
    import subprocess
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = {"time": 1.5, "policy": "wb-chunk-async", "warmups": 3, "standalone_runs": 10, "verify_outputs": True, "tasks": [
        {"id": "hp", "load": {"type": "poisson", "frequency": 300, "seed": 5},
         "client": {"name": "hp", "model_name": "bert@layers=2,s=128", "priority": 0, "launch_mode": "launch"}},
        {"id": "be", "load": {"type": "continuous"},
         "client": {"name": "be", "model_name": "resnet50@b=2", "priority": 1, "launch_mode": "launch"}}]}
    path = tmp_path / "cfg.json"
    path.write_text(json.dumps(cfg))
    for env_extra in ({"GPREEMPT_CHUNK_EVENTS": "1", "GPREEMPT_CHUNK": "3"}, {"GPREEMPT_QUEUE": "1"}):
        out = subprocess.run([os.path.join(root, "gpreempt_amd", "gpreempt_bench"), str(path)], capture_output=True, text=True,
                             env={**os.environ, **env_extra}, timeout=100)
        assert out.returncode == 0, out.stderr[-400:]
        rep = json.loads(out.stdout.strip().splitlines()[-1])
        t = rep["tasks"]
        assert t["hp"]["requests"] > 200 and t["be"]["requests"] > 50 and t["be"]["preemptions"] > 50, (env_extra, t["be"])
        assert t["be"]["outputMismatches"] == 0 and t["hp"]["outputMismatches"] == 0
        assert rep["preemptLatency(us)"]["count"] > 50 and rep["preemptLatency(us)"]["p99"] < 200
