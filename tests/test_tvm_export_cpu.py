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


# ---- the export mapped onto the native operators (no GPU: the kernel list only) -----------------------------

def plan(d, dtype=None):
    from gpreempt_amd import executor as gx
    buf = C.create_string_buffer(1 << 20)
    rc = gx.lib().gpx_plan_tvm_export((d + "/mod.json").encode(), (d + "/host.json").encode(), (d + "/ops.json").encode(),
                                      dtype.encode() if dtype else None, buf, C.c_size_t(len(buf)))
    return rc, json.loads(buf.value.decode()) if buf.value else {}


def test_tiny_export_maps_to_three_native_kernels():
    rc, rep = plan(FIX)
    assert rc == 0, rep
    assert rep["dtype"] == "f32"
    k = rep["kernels"]
    assert [x["name"] for x in k] == ["nchw_to_nhwc", "conv2d", "dense"]  # the reshape is a view, not a copy
    # 3 channels padded to one 16-byte vector; 3x3, stride 1, padding 1 from the sidecar; bias and ReLU fused
    assert k[0]["params"] == {"N": 1, "C": 3, "H": 8, "W": 8, "c_pad": 4}
    conv = k[1]["params"]
    assert (conv["Cin"], conv["Cout"], conv["R"], conv["S"], conv["stride_h"], conv["pad_h"], conv["pad_w"], conv["act"]) == (4, 4, 3, 3, 1, 1, 1, 1)
    assert k[1]["args"] == ["data.nhwc", "p0", "p1", "", "tvmgen_default_fused_nn_conv2d_add_nn_relu"]
    # the dense layer reads the convolution's memory as one row of 256 and writes the renamed output
    assert k[2]["params"] == {"M": 1, "N": 10, "K": 256, "lda": 256, "ldc": 10, "act": 0}
    assert k[2]["args"] == ["tvmgen_default_fused_nn_conv2d_add_nn_relu", "p2", "", "", "heads"]
    st = {s["name"]: s for s in rep["storages"]}
    # parameters keep the export's names and its on-disk sizes: OIHW convolution weight, dense over C x H x W
    assert (st["p0"]["is_param"], st["p0"]["kind"], st["p0"]["disk_elems"], st["p0"]["size"]) == (1, 1, 108, 4 * 4 * 3 * 3 * 4)
    assert (st["p1"]["kind"], st["p1"]["disk_elems"]) == (0, 4)
    assert (st["p2"]["kind"], st["p2"]["disk_elems"]) == (2, 2560)
    assert st["data"]["size"] == 768 and st["heads"]["size"] == 40
    rc, rep = plan(FIX, "f16")
    assert rc == 0 and rep["dtype"] == "f16" and rep["kernels"][1]["params"]["Cin"] == 8
    assert {s["name"]: s["size"] for s in rep["storages"]}["data"] == 384


def test_generated_exports_map_operator_by_operator(tmp_path):
    import export_writer as EW
    w, head = EW.mini_resnet("f32")
    d = str(tmp_path / "r")
    w.write(d, head)
    rc, rep = plan(d)
    assert rc == 0, rep
    names = [k["name"] for k in rep["kernels"]]
    # layout, 9 convolutions, 4 pools, scale-shift, add, classifier, softmax; the concatenation costs nothing:
    # both of its arguments are written into their slices of its buffer by the convolutions that make them
    assert names.count("conv2d") == 9 and names.count("pool2d") == 4 and names.count("eltwise") == 2
    cat = [k["params"] for k in rep["kernels"] if k["name"] == "conv2d" and k["params"]["out_pix_stride"] == 48]
    assert [c["Cout"] for c in cat] == [32, 16]
    assert names[0] == "nchw_to_nhwc" and names[-2:] == ["dense", "softmax"]
    stem = rep["kernels"][1]["params"]
    assert (stem["R"], stem["stride_h"], stem["pad_h"], stem["Cout"], stem["act"]) == (7, 2, 3, 16, 1)
    wide = [k["params"] for k in rep["kernels"] if k["name"] == "conv2d" and k["params"]["R"] == 1 and k["params"]["S"] == 3][0]
    assert (wide["pad_h"], wide["pad_w"]) == (0, 1)
    pools = [k["params"] for k in rep["kernels"] if k["name"] == "pool2d"]
    assert [p["mode"] for p in pools] == [0, 1, 3, 2]   # max; average; average counting the padding; global
    res = [k for k in rep["kernels"] if k["name"] == "conv2d" and k["args"][3]]
    assert len(res) == 2                                  # the two residual inputs are fused into their convolutions
    assert rep["storages"][-1]["name"] == "heads"
    # channel counts that are no multiple of eight halves are padded; the padding is invisible to the export
    w, head = EW.padded_channels("f16")
    d = str(tmp_path / "p")
    w.write(d, head)
    rc, rep = plan(d)
    assert rc == 0, rep
    convs = [k["params"] for k in rep["kernels"] if k["name"] == "conv2d"]
    assert [(c["Cin"], c["Cout"], c["out_pix_stride"]) for c in convs] == [(8, 16, 16), (16, 12, 16), (16, 20, 40), (16, 16, 16), (40, 24, 24)]
    assert not [k for k in rep["kernels"] if k["name"] == "eltwise"]
    # a tensor lives in one place: the second concatenation of the same two tensors copies them
    w, head = EW.shared_concat("f16")
    d = str(tmp_path / "s")
    w.write(d, head)
    rc, rep = plan(d)
    assert rc == 0, rep
    copies = [k for k in rep["kernels"] if k["name"] == "eltwise" and k["args"][1] == ""]
    # ... and a tensor that is also flattened stays in plain memory, so its concatenation copies it (8 of 72 channels)
    assert [(c["params"]["cols"], c["params"]["out_stride"]) for c in copies] == [(16, 24), (8, 24), (8, 72)]
    assert len([k for k in rep["kernels"] if k["name"] == "eltwise"]) == 5   # the three copies and the two adds
    # a DenseNet's growing concatenations: no copies at all, as in the built-in graph
    w, head = EW.densenet("f16")
    d = str(tmp_path / "d")
    w.write(d, head)
    rc, rep = plan(d)
    assert rc == 0, rep
    names = [k["name"] for k in rep["kernels"]]
    assert names.count("eltwise") == 8 + 3 + 1 and names.count("conv2d") == 1 + 16 + 3   # the norms; stem, two per layer, transitions


def test_what_cannot_be_mapped_is_refused_by_name(tmp_path):
    def conv_attr(key, value):
        return lambda f, doc: doc["funcs"][0]["attrs"].__setitem__(key, value) if f == "ops.json" else None
    for name, edit, text in [
        ("groups", conv_attr("groups", 2), "grouped convolution is not mapped"),
        ("dilation", conv_attr("dilation", [2, 2]), "dilated convolution is not mapped"),
        ("asym", conv_attr("padding", [0, 0, 2, 2]), "asymmetric padding is not mapped"),
        # the sidecar's attributes must reproduce the shapes the export states
        ("stride", conv_attr("strides", [2, 2]), "the export says 1x4x8x8, the operator attributes give 1x4x4x4"),
        ("tail", lambda f, doc: doc["funcs"][0].__setitem__("epilogue", ["relu", "bias"]) if f == "ops.json" else None, "in that order"),
        ("role", lambda f, doc: doc["funcs"][0]["inputs"].__setitem__("weight", 0) if f == "ops.json" else None, "must be a parameter"),
        ("bert", lambda f, doc: doc["funcs"][1].__setitem__("op", "layer_norm") if f == "ops.json" else None, "layer_norm needs data, gamma and beta"),
        ("view", lambda f, doc: doc["funcs"][1].update(op="transpose", attrs={"axes": [1, 0]}) if f == "ops.json" else None, "a transpose has one argument"),
        ("layout", lambda f, doc: doc.__setitem__("layout", "NHWC") if f == "ops.json" else None, "NCHW"),
    ]:
        d = _edited(tmp_path, name, edit)
        rc, rep = plan(d)
        assert rc == 1 and text in rep["error"], (name, rep["error"])
        assert rep["kernels"] == [] and rep["storages"] == []

    # an image as the model's output would have to be converted back to NCHW
    def image_head(f, doc):
        if f == "mod.json":
            doc["heads"] = [[3, 0, 0]]
    rc, rep = plan(_edited(tmp_path, "head", image_head))
    assert rc == 1 and "an image as the model's output" in rep["error"]
    rc, rep = plan(FIX, "f64")
    assert rc == 1 and "unknown dtype" in rep["error"]
    # shapes that no tensor can have
    def zero_dim(f, doc):
        if f == "mod.json":
            doc["attrs"]["shape"][1][1] = [4, 0, 3, 3]
    rc, rep = plan(_edited(tmp_path, "zero", zero_dim))
    assert rc == 1 and "a dimension of 0" in rep["error"]
    def huge_dim(f, doc):
        if f == "mod.json":
            doc["attrs"]["shape"][1][5] = [10, 1 << 33]
    rc, rep = plan(_edited(tmp_path, "huge", huge_dim))
    assert rc == 1 and "bad shape of node 5" in rep["error"]  # the reader itself bounds every dimension (< 2^31)
    def huge_tensor(f, doc):
        if f == "mod.json":
            doc["attrs"]["shape"][1][5] = [1 << 20, 1 << 20]
    rc, rep = plan(_edited(tmp_path, "huge2", huge_tensor))
    assert rc == 1 and "more than 2^40 elements" in rep["error"]  # ... and every tensor: a storage size cannot wrap
    def not_an_integer(f, doc):
        if f == "mod.json":
            doc["attrs"]["shape"][1][5] = [10, 1e300]
    rc, rep = plan(_edited(tmp_path, "huge3", not_an_integer))
    assert rc == 1 and "bad shape of node 5" in rep["error"]


def test_bert_export_maps_onto_the_transformer_kernels(tmp_path):
    """The functions of a BERT export (scripts/compile/compile-bert.py:76-77: take, layer_norm, dense, reshape /
    transpose around batch_matmul, softmax, erf-GELU) become embed, layernorm, dense and batched GEMM launches; the
    reshapes and transposes between them cost no kernel: the batched products read the heads through strides and
    the second one writes its result where the transpose back would have put it."""
    import export_writer as EW
    B, S, H, heads, d, F = 2, 32, 128, 2, 64, 256
    w, head, builtin = EW.bert("f16", layers=2, batch=B, seq=S, hidden=H, heads=heads, ffn=F)
    dd = str(tmp_path / "bert")
    w.write(dd, head)
    rc, rep = plan(dd)
    assert rc == 0, rep
    assert rep["dtype"] == "f16"  # "data" holds int64 token ids: the element type is the output's
    k = rep["kernels"]
    per_layer = ["dense", "dense", "dense", "batch_matmul", "softmax", "batch_matmul", "dense", "layernorm", "dense", "dense", "layernorm"]
    assert [x["name"] for x in k] == ["embed", "layernorm"] + per_layer * 2
    assert k[0]["params"] == {"tokens": B * S, "seq": S, "hidden": H, "vocab": 96} and k[0]["args"][0] == "data"
    assert abs(k[1]["params"]["eps"] - 1e-12) < 1e-18
    qk, sm, pv, proj, ln1, f1, f2 = k[5], k[6], k[7], k[8], k[9], k[10], k[11]
    # Q K^T per head: rows of the [tokens, hidden] projections, a head every 64 columns, a batch every S rows
    assert qk["params"] == {"M": S, "N": S, "K": d, "lda": H, "ldc": S, "act": 0, "batch": B * heads, "batch_inner": heads, "ldb": H, "b_is_nk": 1, "alpha": 0.125,
                            "stride_a": d, "stride_b": d, "stride_c": S * S, "stride_a_outer": S * H, "stride_b_outer": S * H, "stride_c_outer": heads * S * S}
    assert sm["params"] == {"rows": B * heads * S, "cols": S}
    # P V: V is read untransposed (K x N with the model's row stride); the result lands as [tokens, hidden]
    assert pv["params"]["b_is_nk"] == 0 and pv["params"]["ldb"] == H and pv["params"]["ldc"] == H
    assert (pv["params"]["stride_c"], pv["params"]["stride_c_outer"]) == (d, S * H)
    assert proj["args"][3] != "" and f2["args"][3] != ""      # the residuals ride in the dense epilogues
    assert f1["params"]["act"] == 2                              # erf-GELU in the epilogue
    assert proj["params"]["lda"] == H and k[-1]["args"][-1] == "heads"
    st = {x["name"]: x for x in rep["storages"]}
    assert st["data"]["stype"] == "int64" and st["data"]["size"] == 8 * B * S
    assert st["heads"]["size"] == 2 * B * S * H
    assert {x["name"] for x in rep["storages"] if x["is_param"]} == set(w.params)
    # GELU and the residual additions as functions of their own: an element-wise launch each, the add in front of a
    # layer-norm inside it
    w, head, _ = EW.bert("f32", layers=1, separate_tail=True)
    dd = str(tmp_path / "bert_sep")
    w.write(dd, head)
    rc, rep = plan(dd)
    assert rc == 0, rep
    names = [x["name"] for x in rep["kernels"]]
    assert names == ["embed", "layernorm", "dense", "dense", "dense", "batch_matmul", "softmax", "batch_matmul", "dense", "layernorm", "dense", "eltwise", "dense", "eltwise", "layernorm"]
    assert rep["kernels"][9]["args"][1] != ""  # layer_norm(data + residual)
    assert rep["kernels"][11]["params"]["act"] == 2
    # what the views cannot express is refused by name
    w, head, _ = EW.bert("f16", layers=1)
    for fn in w.ops:
        if fn["op"] == "transpose" and fn["attrs"]["axes"] == [0, 2, 1, 3]:
            fn["attrs"]["axes"] = [0, 1, 3, 2]
            break
    dd = str(tmp_path / "bert_bad")
    w.write(dd, head)
    rc, rep = plan(dd)
    assert rc == 1 and "the export's shape differs" in rep["error"]
