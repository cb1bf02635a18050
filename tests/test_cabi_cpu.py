"""CPU-only checks of the drop-in boundary: the shared libraries load, export every symbol the
headers declare, and the host logic that needs no GPU (parameter-file parser) behaves like the
reference's (src/model.cpp:15-55)."""
import ctypes as C
import os
import re
import struct

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared(header, prefix):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(" + prefix + r"[a-z0-9_]+)\s*\(", text)))


def test_device_library_exports_every_declared_symbol():
    from gpreempt_amd import capi
    lib = C.CDLL(capi.LIB_PATH)  # loads without a GPU
    names = declared("gpreempt_hip.h", "gp_")
    assert len(names) >= 40
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(capi.SYMBOLS) == names  # the binding covers exactly the header


def test_executor_library_exports_every_declared_symbol():
    from gpreempt_amd import executor
    lib = executor.lib()
    names = declared("gpreempt_exec_c.h", "gpx_")
    for n in names:
        assert hasattr(lib, n), n
    assert sorted(executor.SYMBOLS) == names


def test_struct_sizes_match_header():
    """The ctypes mirrors must have the C layout: compile a tiny program against the header."""
    import subprocess
    import tempfile
    from gpreempt_amd import capi
    src = '#include <stdio.h>\n#include "gpreempt_hip.h"\nint main(){printf("%zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu %zu\\n",' \
          'sizeof(gp_preempt_ctx),sizeof(gp_launch_info),sizeof(gp_gemm_params),sizeof(gp_conv_params),sizeof(gp_layout_params),' \
          'sizeof(gp_pool_params),sizeof(gp_eltwise_params),sizeof(gp_softmax_params),sizeof(gp_layernorm_params),sizeof(gp_embed_params),sizeof(gp_attention_params),sizeof(gp_miniweather_params),sizeof(gp_graph_params));}'
    with tempfile.TemporaryDirectory() as d:
        open(os.path.join(d, "s.c"), "w").write(src)
        subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), os.path.join(d, "s.c"), "-o", os.path.join(d, "s")])
        sizes = [int(v) for v in subprocess.check_output([os.path.join(d, "s")]).split()]
    mirrors = [capi.PreemptCtx, capi.LaunchInfo, capi.GemmParams, capi.ConvParams, capi.LayoutParams, capi.PoolParams,
               capi.EltwiseParams, capi.SoftmaxParams, capi.LayernormParams, capi.EmbedParams, capi.AttentionParams, capi.MiniweatherParams, capi.GraphParams]
    assert sizes == [C.sizeof(m) for m in mirrors]


def test_param_file_round_trip_and_malformed(tmp_path):
    from gpreempt_amd import executor
    lib = executor.lib()
    lib.gpx_parse_params.restype = C.c_long
    rng = np.random.default_rng(0)
    params = {"p0": rng.normal(size=(4, 3)).astype(np.float32), "conv1.weight": rng.normal(size=7).astype(np.float32)}
    path = str(tmp_path / "mod.params")
    executor.write_params(path, params)
    raw = open(path, "rb").read()
    assert raw[:17] == b"TVM_MODEL_PARAMS\0" and struct.unpack("<Q", raw[17:25])[0] == 2  # layout of model.cpp:15-27
    out = np.zeros(12, np.float32)
    n = C.c_size_t()
    assert lib.gpx_parse_params(path.encode(), b"p0", out.ctypes.data_as(C.c_void_p), C.c_size_t(12), C.byref(n)) == 2
    assert n.value == 12 and np.array_equal(out, params["p0"].reshape(-1))
    assert lib.gpx_parse_params(path.encode(), b"missing", None, C.c_size_t(0), C.byref(n)) == 2 and n.value == 0
    # missing file, bad magic, truncated payload -> -1 (the reference aborts; here the caller gets an error)
    assert lib.gpx_parse_params(str(tmp_path / "nope").encode(), None, None, C.c_size_t(0), None) == -1
    open(path, "wb").write(b"NOT_A_PARAM_FILE\0" + raw[17:])
    assert lib.gpx_parse_params(path.encode(), None, None, C.c_size_t(0), None) == -1
    open(path, "wb").write(raw[:-5])
    assert lib.gpx_parse_params(path.encode(), None, None, C.c_size_t(0), None) == -1


def test_bench_refuses_more_than_one_gpu():
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr
