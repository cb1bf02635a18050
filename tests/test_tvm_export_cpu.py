"""The reader of the reference's exported model files (mod.json + host.json) against hand-written
fixtures under tests/golden/tiny_export/, rule by rule of Model::load_from_json (reference
src/model.cpp:128-235; host.json schema patch/tvm.patch:296-311): node storages then temporaries,
negative argument indices, "__nop" nodes, the "heads" rename, the function-name check.  The
fixtures were written by hand from those two descriptions; the expected values below were worked
out from the fixture text, not produced by the reader.  No GPU needed."""
import ctypes as C
import json
import os
import shutil

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIX = os.path.join(ROOT, "tests", "golden", "tiny_export")


def parse(device, host, ops=None):
    from gpreempt_amd import executor as gx
    buf = C.create_string_buffer(1 << 16)
    rc = gx.lib().gpx_parse_tvm_export(device.encode(), host.encode(), ops.encode() if ops else None, buf, C.c_size_t(len(buf)))
    return rc, json.loads(buf.value.decode()) if buf.value else {}


def test_tiny_export_storages_and_kernels():
    rc, rep = parse(os.path.join(FIX, "mod.json"), os.path.join(FIX, "host.json"))
    assert rc == 0, rep
    assert rep["global_len"] == 7 and rep["heads_index"] == 6
    st = rep["storages"]
    # seven graph nodes (4 bytes x the product of the shape), then the two temporaries, typed float32
    assert [s["name"] for s in st] == ["data", "p0", "p1", "tvmgen_default_fused_nn_conv2d_add_nn_relu", "reshape_nop", "p2", "heads", "temp", "temp"]
    assert [s["size"] for s in st] == [768, 432, 16, 1024, 1024, 10240, 40, 512, 64]
    assert all(s["stype"] == "float32" for s in st)
    k = rep["kernels"]
    assert [x["name"] for x in k] == ["tvmgen_default_fused_nn_conv2d_add_nn_relu_kernel0", "tvmgen_default_fused_nn_conv2d_add_nn_relu_kernel1",
                                      "nop", "tvmgen_default_fused_nn_dense_kernel0"]
    # the conv function's arguments are nodes [0, 1, 2, 3]; -1 / -2 are temporaries 7 / 8
    assert k[0]["args_index"] == [0, 1, 7] and k[0]["launch_params"] == [4, 1, 1, 64, 1, 1]
    assert k[1]["args_index"] == [7, 2, 3, 8] and k[1]["launch_params"] == [1, 2, 1, 256, 1, 1]
    # the __nop node copies node 3 into node 4, in front of the function that follows it
    assert k[2]["args_index"] == [3, 4] and k[2]["func"] == "__nop"
    # the dense function's arguments are nodes [4, 5, 6]
    assert k[3]["args_index"] == [4, 5, 6] and k[3]["launch_params"] == [10, 1, 1, 64, 1, 1]
    assert k[3]["func"] == "tvmgen_default_fused_nn_dense"


def test_ops_sidecar_is_parsed_and_checked_against_the_export():
    rc, rep = parse(os.path.join(FIX, "mod.json"), os.path.join(FIX, "host.json"), os.path.join(FIX, "ops.json"))
    assert rc == 0, rep
    assert rep["layout"] == "NCHW"
    conv, dense = rep["ops"]
    assert conv["op"] == "conv2d" and conv["attrs"]["padding"] == [1, 1, 1, 1] and conv["attrs"]["groups"] == [1]
    assert conv["epilogue"] == ["bias", "relu"] and conv["inputs"] == {"bias": 2, "data": 0, "weight": 1}
    assert dense["op"] == "dense"


def _edited(tmp_path, name, fn):
    d = str(tmp_path / name)
    shutil.copytree(FIX, d)
    for f in ("mod.json", "host.json", "ops.json"):
        doc = json.load(open(os.path.join(d, f)))
        fn(f, doc)
        json.dump(doc, open(os.path.join(d, f), "w"))
    return d


def test_malformed_exports_are_errors_not_aborts(tmp_path):
    # a missing file: NotFound, with the reference's message
    rc, rep = parse(os.path.join(FIX, "mod.json"), str(tmp_path / "nope.json"))
    assert rc == 3 and "Cannot open the json file" in rep["error"]
    # function names must agree between the two files (src/model.cpp:208-211)
    d = _edited(tmp_path, "rename", lambda f, doc: doc["funcs"][1].__setitem__("name", "something_else") if f == "host.json" else None)
    rc, rep = parse(d + "/mod.json", d + "/host.json")
    assert rc == 1 and "Function name mismatch: something_else vs tvmgen_default_fused_nn_dense" in rep["error"]
    # a temporary that does not exist, an argument past the function's arguments
    d = _edited(tmp_path, "temp", lambda f, doc: doc["funcs"][0]["kernels"][0].__setitem__("args", [0, 1, -3]) if f == "host.json" else None)
    assert parse(d + "/mod.json", d + "/host.json")[0] == 1
    d = _edited(tmp_path, "arg", lambda f, doc: doc["funcs"][1]["kernels"][0].__setitem__("args", [0, 1, 3]) if f == "host.json" else None)
    assert parse(d + "/mod.json", d + "/host.json")[0] == 1
    # a host.json that lists fewer functions than the graph has
    d = _edited(tmp_path, "short", lambda f, doc: doc["funcs"].pop() if f == "host.json" else None)
    rc, rep = parse(d + "/mod.json", d + "/host.json")
    assert rc == 1 and "does not list" in rep["error"]
    # truncated text, and nesting deeper than any real file (must not recurse without bound)
    open(str(tmp_path / "cut.json"), "w").write(open(os.path.join(FIX, "mod.json")).read()[:200])
    assert parse(str(tmp_path / "cut.json"), os.path.join(FIX, "host.json"))[0] == 1
    open(str(tmp_path / "deep.json"), "w").write("[" * 100000 + "]" * 100000)
    assert parse(str(tmp_path / "deep.json"), os.path.join(FIX, "host.json"))[0] == 1
    # sidecar: an undescribed function, an unknown operator
    d = _edited(tmp_path, "ops1", lambda f, doc: doc["funcs"].pop() if f == "ops.json" else None)
    rc, rep = parse(d + "/mod.json", d + "/host.json", d + "/ops.json")
    assert rc == 1 and "does not describe tvmgen_default_fused_nn_dense" in rep["error"]
    d = _edited(tmp_path, "ops2", lambda f, doc: doc["funcs"][0].__setitem__("op", "fft") if f == "ops.json" else None)
    assert parse(d + "/mod.json", d + "/host.json", d + "/ops.json")[0] == 1


def test_trailing_nop_is_kept(tmp_path):
    """A graph that ends in a reshape: the copy into "heads" is emitted behind the last function."""
    def edit(f, doc):
        if f == "mod.json":
            doc["nodes"].append({"op": "tvm_op", "name": "final_reshape", "attrs": {"func_name": "__nop"}, "inputs": [[6, 0, 0]]})
            doc["attrs"]["dltype"][1].append("float32")
            doc["attrs"]["shape"][1].append([10])
            doc["heads"] = [[7, 0, 0]]
    d = _edited(tmp_path, "tail", edit)
    rc, rep = parse(d + "/mod.json", d + "/host.json")
    assert rc == 0, rep
    assert rep["kernels"][-1]["name"] == "nop" and rep["kernels"][-1]["args_index"] == [6, 7]
    assert rep["storages"][7]["name"] == "heads" and rep["storages"][6]["name"] == "tvmgen_default_fused_nn_dense"
    assert rep["storages"][8]["name"] == "temp"


def test_huge_counts_in_a_parameter_file_are_refused(tmp_path):
    """A header that claims more values than the file holds is an error before anything is allocated."""
    import struct
    from gpreempt_amd import executor as gx
    lib = gx.lib()
    lib.gpx_parse_params.restype = C.c_long
    path = str(tmp_path / "bad.params")
    open(path, "wb").write(b"TVM_MODEL_PARAMS\0" + struct.pack("<Q", 1) + b"p0\0" + struct.pack("<Q", (1 << 34) - 1) + b"\0" * 64)
    assert lib.gpx_parse_params(path.encode(), None, None, C.c_size_t(0), None) == -1
    open(path, "wb").write(b"TVM_MODEL_PARAMS\0" + struct.pack("<Q", 1 << 60) + b"p0\0" + struct.pack("<Q", 4) + b"\0" * 16)
    assert lib.gpx_parse_params(path.encode(), None, None, C.c_size_t(0), None) == -1
