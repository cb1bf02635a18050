"""Whole-model parity: the C++ Executor (through its C view) against the layer-by-layer oracle
on the same seeded weights, which travel through a TVM_MODEL_PARAMS file as in the reference
(src/model.cpp:263-282), plus the preempt-then-resume protocol of src/tests/test-dnn-blp.cpp."""
import os

import numpy as np
import pytest

from oracle import models as OM
from oracle import oracle as O
from helpers import TOL, rel_err

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ex_mod(gp):
    from gpreempt_amd import executor
    return executor


def make_model(ex_mod, tmp_path, workload, family, seed, blp=False):
    """Builds the executor once to learn the parameter shapes, writes seeded parameters to
    <root>/<workload>/mod.params, and builds it again so that they load from the file."""
    root = str(tmp_path)
    probe = ex_mod.Executor(workload, model_root=root)
    shapes = probe.param_shapes()
    probe.destroy()
    params = OM.random_params(shapes, seed, family)
    os.makedirs(os.path.join(root, workload), exist_ok=True)
    ex_mod.write_params(os.path.join(root, workload, "mod.params"), params)
    return ex_mod.Executor(workload, blp=blp, model_root=root), params


def run(gp, ex, x_raw, dtype, out_shape):
    ex.set_input("data", x_raw)
    ex.execute()
    return gp.from_storage(ex.get_output("heads"), dtype).reshape(out_shape).copy()


def logits_of(gp, ex, storage, dtype, shape):
    """The classifier's output in front of the softmax, read from its storage by name (Model::get): probabilities
    alone can hide a wrong logit that does not move the top class."""
    return gp.from_storage(ex.get_output(storage), dtype).reshape(shape).copy()


def test_gemm1024_workload_matches_oracle(gp, ex_mod, tmp_path):
    ex, params = make_model(ex_mod, tmp_path, "gemm1024", "gemm", 1)
    A = np.random.default_rng(0xC0FFEE).uniform(-1, 1, (1024, 1024)).astype(np.float32)
    got = run(gp, ex, A, gp.F32, (1024, 1024))
    ref = O.gemm_bias_act(A, params["B"].reshape(1024, 1024), params["bias"], act=O.ACT_RELU)
    assert rel_err(got, ref) < TOL["f32"]


@pytest.mark.parametrize("workload,dt,blocks", [
    ("resnet50", "f32", OM.RESNET_BLOCKS["resnet50"]),                 # BASELINE config 2 at full size
    ("resnet152@b=2,hw=64", "f16", OM.RESNET_BLOCKS["resnet152"]),     # config 3's tenant, reduced image
])
def test_resnet_matches_oracle(gp, ex_mod, tmp_path, workload, dt, blocks):
    ex, params = make_model(ex_mod, tmp_path, workload, "cnn", 2)
    dtype = gp.DTYPE_BY_NAME[dt]
    n = 2 if "b=2" in workload else 1
    hw = 64 if "hw=64" in workload else 224
    x = O.round_to(np.random.default_rng(3).normal(0, 1, (n, 3, hw, hw)).astype(np.float32), dt)
    got = run(gp, ex, gp.to_storage(x, dtype), dtype, (n, 1000))
    ref, ref_logits = OM.resnet(params, x, blocks, dt, logits=True)
    assert np.isfinite(got).all()
    assert rel_err(got, ref) < TOL[dt]
    assert abs(got.sum(axis=1) - 1).max() < 2e-2
    assert rel_err(logits_of(gp, ex, "fc.out", dtype, (n, 1000)), ref_logits) < TOL[dt]


def test_vgg16_matches_oracle(gp, ex_mod, tmp_path):
    wl = "vgg16@b=2,hw=64,fc=512"
    ex, params = make_model(ex_mod, tmp_path, wl, "cnn", 4)
    x = O.round_to(np.random.default_rng(5).normal(0, 1, (2, 3, 64, 64)).astype(np.float32), "f16")
    got = run(gp, ex, gp.to_storage(x, gp.F16), gp.F16, (2, 1000))
    ref, ref_logits = OM.vgg16(params, x, "f16", logits=True)
    assert rel_err(got, ref) < TOL["f16"]
    assert rel_err(logits_of(gp, ex, "fc3.out", gp.F16, (2, 1000)), ref_logits) < TOL["f16"]


def test_vgg16_full_size_logits_match_oracle(gp, ex_mod, tmp_path):
    """BASELINE config 4's best-effort model at its real shape (224 x 224, 4096-wide classifier), one image:
    the 25088 -> 4096 dense layer (K = 25088, M = 1) and the 224 x 224 x 64 convolutions, on the logits."""
    wl = "vgg16@b=1"
    ex, params = make_model(ex_mod, tmp_path, wl, "cnn", 14)
    x = O.round_to(np.random.default_rng(15).normal(0, 1, (1, 3, 224, 224)).astype(np.float32), "f16")
    got = run(gp, ex, gp.to_storage(x, gp.F16), gp.F16, (1, 1000))
    ref, ref_logits = OM.vgg16(params, x, "f16", logits=True)
    assert np.isfinite(got).all() and abs(got.sum() - 1) < 2e-2
    assert rel_err(logits_of(gp, ex, "fc3.out", gp.F16, (1, 1000)), ref_logits) < TOL["f16"]
    assert rel_err(got, ref) < TOL["f16"]


def test_densenet_matches_oracle(gp, ex_mod, tmp_path):
    wl = "densenet201@b=1,hw=64,l1=2,l2=4,l3=5,l4=3"
    ex, params = make_model(ex_mod, tmp_path, wl, "cnn", 6)
    x = O.round_to(np.random.default_rng(7).normal(0, 1, (1, 3, 64, 64)).astype(np.float32), "f16")
    got = run(gp, ex, gp.to_storage(x, gp.F16), gp.F16, (1, 1000))
    ref, ref_logits = OM.densenet(params, x, "f16", (2, 4, 5, 3), logits=True)
    assert rel_err(got, ref) < TOL["f16"]
    assert rel_err(logits_of(gp, ex, "classifier.out", gp.F16, (1, 1000)), ref_logits) < TOL["f16"]


def test_densenet201_full_size_logits_match_oracle(gp, ex_mod, tmp_path):
    """BASELINE config 4's mid-priority model at its real shape (blocks 6 / 12 / 48 / 32, 224 x 224), one image."""
    wl = "densenet201@b=1"
    ex, params = make_model(ex_mod, tmp_path, wl, "cnn", 16)
    x = O.round_to(np.random.default_rng(17).normal(0, 1, (1, 3, 224, 224)).astype(np.float32), "f16")
    got = run(gp, ex, gp.to_storage(x, gp.F16), gp.F16, (1, 1000))
    ref, ref_logits = OM.densenet(params, x, "f16", logits=True)
    assert np.isfinite(got).all() and abs(got.sum() - 1) < 2e-2
    assert rel_err(logits_of(gp, ex, "classifier.out", gp.F16, (1, 1000)), ref_logits) < TOL["f16"]
    assert rel_err(got, ref) < TOL["f16"]


def test_inception_v3_matches_oracle(gp, ex_mod, tmp_path):
    # full widths, 107 x 107 input (the 8 x 8 stage of the 299 x 299 network becomes 1 x 1)
    wl = "inception@b=1,hw=107"
    ex, params = make_model(ex_mod, tmp_path, wl, "cnn", 8)
    assert ex.kernel_num() > 100
    x = O.round_to(np.random.default_rng(9).normal(0, 1, (1, 3, 107, 107)).astype(np.float32), "f16")
    got = run(gp, ex, gp.to_storage(x, gp.F16), gp.F16, (1, 1000))
    assert np.isfinite(got).all() and abs(got.sum() - 1) < 2e-2
    ref, ref_logits = OM.inception_v3(params, x, "f16", logits=True)
    assert rel_err(got, ref) < TOL["f16"]
    assert rel_err(logits_of(gp, ex, "fc1.out", gp.F16, (1, 1000)), ref_logits) < TOL["f16"]


@pytest.mark.parametrize("workload,kw", [
    ("bert", dict(batch=1, seq=128, layers=12)),                       # config 3's high-priority tenant, full size
    ("bert@b=2,s=48,layers=2,dtype=f32", dict(batch=2, seq=48, layers=2)),
    ("bert@s=384", dict(batch=1, seq=384, layers=12)),                 # config 5's high-priority tenant, full size
])
def test_bert_matches_oracle(gp, ex_mod, tmp_path, workload, kw):
    dt = "f32" if "f32" in workload else "f16"
    ex, params = make_model(ex_mod, tmp_path, workload, "bert", 8)
    ids = np.random.default_rng(9).integers(0, 30522, kw["batch"] * kw["seq"]).astype(np.int64)
    dtype = gp.DTYPE_BY_NAME[dt]
    got = run(gp, ex, ids, dtype, (kw["batch"] * kw["seq"], 768))
    ref = OM.bert(params, ids, dt, **kw)
    assert rel_err(got, ref) < TOL[dt]


def test_toy_chain_with_nop_copies(gp, ex_mod, tmp_path):
    ex = ex_mod.Executor("toy@n=3", model_root=str(tmp_path))
    assert [k["name"] for k in ex.kernels()] == ["eltwise", "nop"] * 3
    x = np.arange(64 * 64, dtype=np.float32)
    got = run(gp, ex, x, gp.F32, (64 * 64,))
    assert np.array_equal(got, 8 * x)


def test_executor_error_paths(gp, ex_mod, tmp_path):
    with pytest.raises(ex_mod.StatusError) as e:
        ex_mod.Executor("no_such_model", model_root=str(tmp_path))
    assert e.value.status == 3  # NotFound
    ex = ex_mod.Executor("toy", model_root=str(tmp_path))
    with pytest.raises(ex_mod.StatusError) as e:
        ex.set_input("data", np.zeros(8, np.float32))  # shorter than the storage: OutOfRange (model.cpp:319)
    assert e.value.status == 4
    with pytest.raises(ex_mod.StatusError) as e:
        ex.set_input("nope", np.zeros(8, np.float32))
    assert e.value.status == 3
    assert ex.data_size("nope") == 0
    with pytest.raises(ex_mod.StatusError):
        ex.resume()  # BaseExecutor has no resume


# ---- preempt-then-resume on whole models ----------------------------------------------------

def _blp_roundtrip(gp, ex_mod, tmp_path, workload, x_raw, injections, graph=False, hipgraph=False):
    root = str(tmp_path)
    os.environ["GPREEMPT_USE_HIPGRAPH"] = "1" if hipgraph else "0"
    base = ex_mod.Executor(workload, blp=False, model_root=root)
    base.set_input("data", x_raw)
    base.execute()
    want = base.get_output("heads").copy()
    ex = ex_mod.Executor(workload, blp=True, model_root=root)
    flag = gp.Flag()
    ex.set_flag(flag)
    stream = gp.Stream(1)
    if graph:
        ex.capture_graph(stream)
        assert ex.uses_program() == (not hipgraph)
    program = graph and not hipgraph
    ex.set_input("data", x_raw, stream)
    # uninterrupted preemptible run: same bits as the non-preemptible executor
    ex.execute(stream)
    ex.set_running(True)
    assert np.array_equal(ex.get_output("heads", stream), want)
    assert ex.stop_point(stream) == -1
    n = ex.kernel_num()
    for kernel, claim in injections:
        kernel = kernel if kernel >= 0 else n + kernel
        flag.set(0)
        ex.inject_preempt(kernel, claim)
        if graph and hipgraph:
            ex.capture_graph(stream)  # the injection point is a kernel argument: re-capture
        ex.execute(stream)
        ex.set_running(True)
        stream.sync()
        assert flag.get() == 1, (kernel, claim)
        cnt = ex.counters()
        # Per-kernel launches: every later kernel left at its first flag check.  Inside the
        # program, workgroups that found a layer's counter exhausted may already hold claims on
        # the next layers when the flag is seen, but nothing far ahead can have started.
        # Per-kernel launches: the flag is read by some claims only, so a small kernel may be
        # over before anyone has looked and the next kernel notices (after its first claims).
        # Program: the resident workgroups hold one claim each; over small layers these span many layers.
        slack = 48 if program else 3
        assert (cnt[kernel + slack:] == 0).all(), (kernel, cnt)
        ex.inject_preempt(-1, -1)
        flag.set(0)  # host clears the flag, then resumes (test-dnn-blp.cpp:41-42)
        ex.resume(stream)
        if ex.last_stop_index() == -1:
            # the flag went up so late that no later claim looked at it: the model had finished
            # (only some claims read the flag, and the last kernels are short)
            assert kernel >= n - 3, (kernel, n)
        else:
            assert kernel <= ex.last_stop_index() <= kernel + slack, (ex.last_stop_index(), kernel)
        stream.sync()
        assert np.array_equal(ex.get_output("heads", stream), want), (kernel, claim)
        assert ex.stop_point(stream) == -1
        ex.resume(stream)  # nothing stopped: must be a no-op
        assert np.array_equal(ex.get_output("heads", stream), want)
    ex.set_running(False)
    return ex


def test_resnet50_preempt_resume_bit_exact(gp, ex_mod, tmp_path):
    x = np.random.default_rng(1).normal(0, 1, (1, 3, 224, 224)).astype(np.float32)
    _blp_roundtrip(gp, ex_mod, tmp_path, "resnet50", x, [(1, 10), (20, 3), (-3, 0), (5, 0)])


def test_resnet50_preempt_resume_bit_exact_with_hip_graph(gp, ex_mod, tmp_path):
    x = np.random.default_rng(2).normal(0, 1, (1, 3, 224, 224)).astype(np.float32)
    _blp_roundtrip(gp, ex_mod, tmp_path, "resnet50", x, [(7, 5), (40, 1)], graph=True, hipgraph=True)


@pytest.mark.parametrize("workload,shape,injections", [
    ("toy@n=3,rows=512,cols=512", (512 * 512,), [(0, 3), (3, 10), (5, 0)]),
    ("resnet50", (1, 3, 224, 224), [(1, 10), (7, 5), (20, 3), (40, 1), (-3, 0), (-1, 0)]),
    ("gemm@m=2048,n=2048,k=512,tile=64", (2048, 512), [(0, 64), (0, 300), (0, 700)]),  # 1024 tiles > resident workgroups
])
def test_program_preempt_resume_bit_exact(gp, ex_mod, tmp_path, workload, shape, injections):
    """The whole model as one persistent kernel: stop inside a layer, leave, relaunch."""
    x = np.random.default_rng(2).normal(0, 1, shape).astype(np.float32)
    ex = _blp_roundtrip(gp, ex_mod, tmp_path, workload, x, injections, graph=True)
    assert ex.uses_program()


def test_program_bert_and_resnet152_match_per_kernel_path(gp, ex_mod, tmp_path):
    """Program output == per-kernel output, bit for bit, with and without preemption."""
    ids = np.random.default_rng(3).integers(0, 30522, 128).astype(np.int64)
    _blp_roundtrip(gp, ex_mod, tmp_path, "bert", ids, [(0, 3), (2, 17), (57, 0), (-1, 10)], graph=True)
    x = gp.to_storage(np.random.default_rng(4).normal(0, 1, (8, 3, 224, 224)).astype(np.float32), gp.F16)
    _blp_roundtrip(gp, ex_mod, tmp_path, "resnet152", x, [(3, 100), (80, 7), (-2, 0)], graph=True)


def test_program_non_preemptible_executor(gp, ex_mod, tmp_path):
    """BaseExecutor (the high-priority tenant) through the program: same bits as launch by launch."""
    os.environ["GPREEMPT_USE_HIPGRAPH"] = "0"
    ids = np.random.default_rng(5).integers(0, 30522, 128).astype(np.int64)
    a = ex_mod.Executor("bert", model_root=str(tmp_path))
    a.set_input("data", ids)
    a.execute()
    want = a.get_output("heads").copy()
    b = ex_mod.Executor("bert", model_root=str(tmp_path))
    stream = gp.Stream(0)
    b.capture_graph(stream)
    assert b.uses_program()
    b.set_input("data", ids, stream)
    for _ in range(3):
        b.execute(stream)
        assert np.array_equal(b.get_output("heads", stream), want)


def test_bert_preempt_resume_bit_exact(gp, ex_mod, tmp_path):
    ids = np.random.default_rng(3).integers(0, 30522, 128).astype(np.int64)
    # (kernel 57 is a layer-norm that runs as the prologue of kernel 58, the dense layer behind it)
    _blp_roundtrip(gp, ex_mod, tmp_path, "bert", ids, [(0, 3), (2, 17), (58, 0), (-1, 10)])


@pytest.mark.parametrize("program,eager", [(False, True), (True, True), (False, False)])
def test_host_timed_preempt_like_reference_test(gp, ex_mod, tmp_path, program, eager, monkeypatch):
    """src/tests/test-dnn-blp.cpp:36-42 verbatim: execute; set the flag from the host right
    away; sync; clear; resume; sync.  Where the flag lands is up to timing; the result is not.
    (eager, the default: first launches start their tiles before the stop index has come back;
    GPREEMPT_EAGER_TILES=0 makes them wait for it)"""
    root = str(tmp_path)
    if not eager:
        monkeypatch.setenv("GPREEMPT_EAGER_TILES", "0")
    x = gp.to_storage(np.full((8, 3, 224, 224), 10.0, np.float32), gp.F16)  # the reference's all-10.0 image
    base = ex_mod.Executor("resnet152", model_root=root)
    base.set_input("data", x)
    base.execute()
    want = base.get_output("heads").copy()
    ex = ex_mod.Executor("resnet152", blp=True, model_root=root)
    flag = gp.Flag()
    ex.set_flag(flag)
    stream = gp.Stream(1)
    os.environ["GPREEMPT_USE_HIPGRAPH"] = "0"
    if program:
        ex.capture_graph(stream)
    ex.set_input("data", x, stream)
    stream.sync()
    stops = []
    for _ in range(5):
        ex.execute(stream)
        ex.set_running(True)
        flag.set(1)
        stream.sync()
        flag.set(0)
        ex.resume(stream)
        stops.append(ex.last_stop_index())
        stream.sync()
        assert np.array_equal(ex.get_output("heads", stream), want)
    assert any(s != -1 for s in stops), stops  # at least one run was really interrupted
    ex.set_running(False)
    ex.resume(stream)  # running == false: no-op (executor.cpp:281)


def test_vgg16_b16_full_size_host_timed_preempt_bit_exact(gp, ex_mod, tmp_path):
    """The same protocol on BASELINE config 4's best-effort tenant at its real shape (VGG-16, batch 16, 224 x 224):
    its deep 3 x 3 layers take 64 x 64 tiles when preemptible (K >= 2304) and run in several rounds of workgroups,
    its 25088 -> 4096 layer is the longest K of any model here."""
    root = str(tmp_path)
    os.environ["GPREEMPT_USE_HIPGRAPH"] = "0"
    x = gp.to_storage(np.random.default_rng(21).normal(0, 1, (16, 3, 224, 224)).astype(np.float32), gp.F16)
    base = ex_mod.Executor("vgg16", model_root=root)
    base.set_input("data", x)
    base.execute()
    want = base.get_output("heads").copy()
    want_logits = base.get_output("fc3.out").copy()
    base.destroy()
    ex = ex_mod.Executor("vgg16", blp=True, model_root=root)
    flag = gp.Flag()
    ex.set_flag(flag)
    stream = gp.Stream(1)
    ex.set_input("data", x, stream)
    stream.sync()
    import time
    stops = []
    for i in range(4):
        ex.execute(stream)
        ex.set_running(True)
        time.sleep(0.0002 * i)  # the flag lands in another part of the network every time
        flag.set(1)
        stream.sync()
        flag.set(0)
        ex.resume(stream)
        stops.append(ex.last_stop_index())
        stream.sync()
        assert np.array_equal(ex.get_output("heads", stream), want)
        assert np.array_equal(ex.get_output("fc3.out", stream), want_logits)
    assert any(s != -1 for s in stops), stops
    ex.set_running(False)


def test_exported_graph_next_to_the_model_is_read_and_checked(gp, ex_mod, tmp_path):
    """mod.json + host.json in the model directory are read as the reference reads them; an export
    that describes another model than the native graph of that name is refused, not ignored."""
    import json

    def export(n_elems):
        mod = {"nodes": [{"op": "null", "name": "data", "inputs": []},
                         {"op": "tvm_op", "name": "fused_add", "attrs": {"func_name": "fused_add"}, "inputs": [[0, 0, 0]]}],
               "heads": [[1, 0, 0]],
               "attrs": {"dltype": ["list_str", ["float32", "float32"]], "shape": ["list_shape", [[n_elems], [n_elems]]]}}
        host = {"temp_args": [], "funcs": [{"name": "fused_add", "kernels": [{"name": "fused_add_kernel0", "launch_params": [16, 1, 1, 256, 1, 1], "args": [0, 1]}]}]}
        return mod, host

    root = tmp_path / "models"
    d = root / "toy"
    d.mkdir(parents=True)
    mod, host = export(64 * 64)
    (d / "mod.json").write_text(json.dumps(mod)); (d / "host.json").write_text(json.dumps(host))
    ex = ex_mod.Executor("toy", model_root=str(root))  # agrees with the native toy graph (64 x 64 fp32 in and out)
    x = np.arange(64 * 64, dtype=np.float32)
    assert np.array_equal(run(gp, ex, x, gp.F32, (64 * 64,)), 8 * x)
    # the reference's exports are float32; the same model run in a 16-bit type is still the same model:
    # what must agree is the number of elements, not of bytes
    d16 = root / "toy@dtype=f16"
    d16.mkdir()
    (d16 / "mod.json").write_text(json.dumps(mod)); (d16 / "host.json").write_text(json.dumps(host))
    ex16 = ex_mod.Executor("toy@dtype=f16", model_root=str(root))
    x16 = (np.arange(64 * 64) % 128).astype(np.float32)
    assert np.array_equal(run(gp, ex16, gp.to_storage(x16, gp.F16), gp.F16, (64 * 64,)), 8 * x16)
    mod, host = export(100)
    (d / "mod.json").write_text(json.dumps(mod))
    with pytest.raises(ex_mod.StatusError) as e:
        ex_mod.Executor("toy", model_root=str(root))
    assert e.value.status == 1  # Fail
    (d / "mod.json").write_text("{ not json")
    with pytest.raises(ex_mod.StatusError) as e:
        ex_mod.Executor("toy", model_root=str(root))
    assert e.value.status == 1
    # the model root is process-wide (an environment variable): leave one without exported files behind
    (d / "mod.json").unlink(); (d / "host.json").unlink()
    os.environ["GPREEMPT_MODEL_PATH"] = str(tmp_path)


# ---- exported models on the native operators ------------------------------------------------------
# The reference loads an export's own device code (src/model.cpp:84-98); here mod.json + host.json +
# the operator sidecar ops.json become native kernels and the export's mod.params loads into them by the
# export's parameter names.  The exports are written by tests/export_writer.py, which computes the expected
# output with the oracle's operators while it writes.

@pytest.mark.parametrize("dt", ["f32", "f16"])
@pytest.mark.parametrize("maker", ["mini_resnet", "mini_vgg", "padded_channels", "shared_concat", "densenet", "mlp"])
def test_exported_model_matches_oracle(gp, ex_mod, tmp_path, maker, dt):
    import export_writer as EW
    w, head = getattr(EW, maker)(dt)
    want = w.write(str(tmp_path / maker), head)
    ex = ex_mod.Executor(maker, model_root=str(tmp_path))
    dtype = gp.DTYPE_BY_NAME[dt]
    got = run(gp, ex, gp.to_storage(w.value(0), dtype), dtype, want.shape)
    assert rel_err(got, want) < TOL[dt], maker
    names = {s["name"] for s in ex.storages() if s["is_param"]}
    assert names == set(w.params)  # every parameter of the export, under the export's name
    ex.destroy()


def test_exported_model_in_another_element_type_and_without_parameters(gp, ex_mod, tmp_path):
    import export_writer as EW
    # an fp32 export run in bf16: the workload name carries the element type, as for the built-in models
    w, head = EW.mini_vgg("bf16")
    want = w.write(str(tmp_path / "mini_vgg@dtype=bf16"), head)
    ex = ex_mod.Executor("mini_vgg@dtype=bf16", model_root=str(tmp_path))
    got = run(gp, ex, gp.to_storage(w.value(0), gp.BF16), gp.BF16, want.shape)
    assert rel_err(got, want) < TOL["bf16"]
    ex.destroy()
    # no mod.params: the seeded initialisation stays, the model still runs (src/model.cpp:263-282 copies only what the file holds)
    w, head = EW.mini_resnet("f16")
    w.write(str(tmp_path / "noparams"), head, params=False)
    ex = ex_mod.Executor("noparams", model_root=str(tmp_path))
    got = run(gp, ex, gp.to_storage(w.value(0), gp.F16), gp.F16, (2, 10))
    assert np.isfinite(got).all() and np.allclose(got.sum(axis=1), 1, atol=1e-2)
    ex.destroy()
    # an export that cannot be mapped is refused at load time, by name
    w, head = EW.mini_vgg("f32")
    w.ops[0]["attrs"]["groups"] = 2
    w.write(str(tmp_path / "grouped"), head)
    with pytest.raises(ex_mod.StatusError) as e:
        ex_mod.Executor("grouped", model_root=str(tmp_path))
    assert e.value.status == 1


@pytest.mark.parametrize("program", [False, True])
def test_exported_model_preempt_resume_bit_exact(gp, ex_mod, tmp_path, program):
    import export_writer as EW
    w, head = EW.mini_resnet("f16", batch=4, hw=64)
    w.write(str(tmp_path / "mini_resnet"), head)
    x = gp.to_storage(w.value(0), gp.F16)
    _blp_roundtrip(gp, ex_mod, tmp_path, "mini_resnet", x, [(1, 0), (6, 0), (9, 0)], graph=program)


def test_exported_resnet50_equals_the_builtin_graph(gp, ex_mod, tmp_path):
    """A ResNet-50 written as an export maps onto the same kernels as the built-in graph of that name: the
    same number of launches, and with the same parameters the same bits."""
    import export_writer as EW
    w, head = EW.resnet("f16", OM.RESNET_BLOCKS["resnet50"], batch=2, hw=64)
    want = w.write(str(tmp_path / "exported_resnet"), head)
    x = gp.to_storage(w.value(0), gp.F16)
    ex = ex_mod.Executor("exported_resnet", model_root=str(tmp_path))
    got = run(gp, ex, x, gp.F16, want.shape)
    assert rel_err(got, want) < TOL["f16"]
    builtin = "resnet50@b=2,hw=64,dtype=f16"
    os.makedirs(str(tmp_path / builtin))
    ex_mod.write_params(str(tmp_path / builtin / "mod.params"), {name: w.params[p] for name, p in w.alias.items()})
    ref = ex_mod.Executor(builtin, model_root=str(tmp_path))
    assert set(w.alias) == {s["name"] for s in ref.storages() if s["is_param"]}
    assert ex.kernel_num() == ref.kernel_num()
    assert np.array_equal(got, run(gp, ref, x, gp.F16, want.shape))
    ex.destroy(); ref.destroy()


def test_exported_densenet_equals_the_builtin_graph(gp, ex_mod, tmp_path):
    """The growing concatenations of a DenseNet export cost no copies: every layer writes its new channels
    into the block's buffer, which is the built-in graph's layout; same launches, same bits."""
    import export_writer as EW
    w, head = EW.densenet("f16", layers=(2, 4, 2, 2), growth=16, init=32, batch=2, hw=64, classes=24)
    want = w.write(str(tmp_path / "exported_densenet"), head)
    x = gp.to_storage(w.value(0), gp.F16)
    ex = ex_mod.Executor("exported_densenet", model_root=str(tmp_path))
    got = run(gp, ex, x, gp.F16, want.shape)
    assert rel_err(got, want) < TOL["f16"]
    builtin = "densenet@b=2,hw=64,l1=2,l2=4,l3=2,l4=2,growth=16,init=32,classes=24,dtype=f16"
    os.makedirs(str(tmp_path / builtin))
    ex_mod.write_params(str(tmp_path / builtin / "mod.params"), {name: w.params[p] for name, p in w.alias.items()})
    ref = ex_mod.Executor(builtin, model_root=str(tmp_path))
    assert set(w.alias) == {s["name"] for s in ref.storages() if s["is_param"]}
    assert [k["name"] for k in ex.kernels()] == [k["name"] for k in ref.kernels()]
    assert np.array_equal(got, run(gp, ref, x, gp.F16, want.shape))
    ex.destroy(); ref.destroy()


@pytest.mark.parametrize("dt", ["f16", "f32"])
@pytest.mark.parametrize("separate_tail", [False, True])
def test_exported_bert_matches_oracle(gp, ex_mod, tmp_path, dt, separate_tail):
    """A BERT encoder written as an export (take, layer_norm, three projections, reshapes and transposes around two
    batch_matmul functions and a softmax, erf-GELU): against the oracle's operators applied node by node as the
    writer goes, and against the oracle's own BERT composition on the same parameters."""
    import export_writer as EW
    w, head, builtin = EW.bert(dt, layers=2, separate_tail=separate_tail)
    want = w.write(str(tmp_path / "bert_export"), head)
    ex = ex_mod.Executor("bert_export", model_root=str(tmp_path))
    dtype = gp.DTYPE_BY_NAME[dt]
    ids = w.value(0).astype(np.int64)
    got = run(gp, ex, ids, dtype, (64, 128))
    assert rel_err(got, want.reshape(64, 128)) < TOL[dt]
    ref = OM.bert(builtin, ids.reshape(-1), dt, batch=2, seq=32, layers=2, hidden=128, heads=2, fused_attention=False)
    assert rel_err(got, ref) < TOL[dt]
    assert {s["name"] for s in ex.storages() if s["is_param"]} == set(w.params)
    ex.destroy()


def test_exported_bert_equals_the_builtin_graph(gp, ex_mod, tmp_path):
    """The same encoder from the export and from the built-in "bert" graph (its attention as batch_matmul, softmax,
    batch_matmul; the three projections there are one matrix) on the same parameters: the same bits."""
    import export_writer as EW
    w, head, builtin_params = EW.bert("f16", layers=2)
    w.write(str(tmp_path / "bert_export"), head)
    ids = w.value(0).astype(np.int64)
    ex = ex_mod.Executor("bert_export", model_root=str(tmp_path))
    got = run(gp, ex, ids, gp.F16, (64, 128))
    builtin = "bert@b=2,s=32,layers=2,hidden=128,heads=2,ffn=256,vocab=96,maxpos=32,fused_attention=0,dtype=f16"
    os.makedirs(str(tmp_path / builtin))
    ex_mod.write_params(str(tmp_path / builtin / "mod.params"), builtin_params)
    ref = ex_mod.Executor(builtin, model_root=str(tmp_path))
    assert set(builtin_params) == {s["name"] for s in ref.storages() if s["is_param"]}
    assert ex.kernel_num() == ref.kernel_num() + 2 * 2  # three projections per layer where the built-in graph has one
    assert np.array_equal(got, run(gp, ref, ids, gp.F16, (64, 128)))
    ex.destroy(); ref.destroy()


@pytest.mark.parametrize("program", [False, True])
def test_exported_bert_preempt_resume_bit_exact(gp, ex_mod, tmp_path, program):
    import export_writer as EW
    w, head, _ = EW.bert("f16", layers=2, batch=4, seq=64)
    w.write(str(tmp_path / "bert_export"), head)
    ids = w.value(0).astype(np.int64)
    # the embedding, a projection, both batched products, a dense layer with a residual, the last layer-norm
    _blp_roundtrip(gp, ex_mod, tmp_path, "bert_export", ids, [(0, 0), (3, 1), (5, 2), (7, 1), (8, 0), (-1, 1)], graph=program)
