"""ctypes binding of include/gpreempt_exec_c.h (libgpreempt_exec.so): the C++ Executor /
BLPExecutor classes as seen from Python.  Used by tests and bench.py; no fallback path."""
import ctypes as C
import os
import struct

import numpy as np

from . import capi

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgpreempt_exec.so")
vp = C.c_void_p

SYMBOLS = """gpx_create gpx_destroy gpx_init gpx_set_input gpx_get_output gpx_get_data_size gpx_execute
gpx_launch_kernel gpx_get_kernel_num gpx_capture_graph gpx_uses_program gpx_clear gpx_set_flag gpx_set_running gpx_resume
gpx_get_stop_point gpx_last_stop_index gpx_inject_preempt gpx_read_counters gpx_reset_counters gpx_storage_num gpx_storage_info
gpx_kernel_info gpx_read_storage gpx_miniweather_reductions gpx_graph_info gpx_graph_result_bytes gpx_graph_result
gpx_graph_inject_preempt gpx_set_lc_tasks gpx_set_graph_path gpx_write_synthetic_graph gpx_run_scenario gpx_preempt_probe gpx_parse_params gpx_parse_tvm_export gpx_plan_tvm_export gpx_set_priority gpx_domain_create gpx_domain_destroy gpx_get_fd gpx_domain_flag gpx_domain_flag_value
gpx_domain_begin gpx_domain_end gpx_suspend_streams gpx_resume_streams""".split()

STATUS = ["Succ", "Fail", "Timeout", "NotFound", "OutOfRange", "Full"]
_lib = None


def lib():
    global _lib
    if _lib is None:
        capi.lib()  # the device layer must be there first
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(LIB_PATH)
        _lib.gpx_create.restype = vp
        _lib.gpx_get_data_size.restype = C.c_size_t
        _lib.gpx_get_kernel_num.restype = C.c_size_t
        _lib.gpx_storage_num.restype = C.c_size_t
        _lib.gpx_graph_result_bytes.restype = C.c_size_t
        _lib.gpx_domain_flag.restype = vp
        _lib.gpx_destroy.restype = None
        _lib.gpx_clear.restype = None
    return _lib


class StatusError(RuntimeError):
    def __init__(self, status, what):
        super().__init__(f"{what}: Status::{STATUS[status] if 0 <= status < 6 else status}")
        self.status = status


def _chk(rc, what):
    if rc != 0:
        raise StatusError(rc, what)


def write_params(path, params):
    """Writes {name: float array} in the reference's TVM_MODEL_PARAMS format
    (reader: reference src/model.cpp:15-55, writer: scripts/compile/compile.py:73-83)."""
    with open(path, "wb") as f:
        f.write(b"TVM_MODEL_PARAMS\0")
        f.write(struct.pack("<Q", len(params)))
        for k, v in params.items():
            a = np.ascontiguousarray(v, np.float32).reshape(-1)
            f.write(k.encode() + b"\0")
            f.write(struct.pack("<Q", a.size))
            f.write(a.tobytes())


class Executor:
    def __init__(self, workload, blp=False, model_root=None, graph_path=None):
        if model_root is not None:
            os.environ["GPREEMPT_MODEL_PATH"] = model_root
        self.blp = blp
        self.h = vp(lib().gpx_create(int(blp)))
        if graph_path:
            _chk(lib().gpx_set_graph_path(self.h, graph_path.encode()), "set_graph_path")
        _chk(lib().gpx_init(self.h, workload.encode()), f"init({workload})")

    # -- introspection
    def storages(self):
        out = []
        for i in range(lib().gpx_storage_num(self.h)):
            name, st = C.create_string_buffer(256), C.create_string_buffer(32)
            nbytes, isp, de = C.c_size_t(), C.c_int(), C.c_size_t()
            dims = (C.c_int * 8)()
            _chk(lib().gpx_storage_info(self.h, C.c_size_t(i), name, C.c_size_t(256), st, C.c_size_t(32), C.byref(nbytes),
                                        C.byref(isp), C.byref(de), dims), "storage_info")
            out.append(dict(name=name.value.decode(), stype=st.value.decode(), bytes=nbytes.value, is_param=bool(isp.value),
                            disk_elems=de.value, dims=list(dims)))
        return out

    def param_shapes(self):
        """{name: shape on disk} for every parameter (fp32; OIHW conv weights; [units][in] dense)."""
        shapes = {}
        for s in self.storages():
            if not s["is_param"]:
                continue
            kind, o, i, r, ss, c, h, w = s["dims"]
            if kind == 1:
                shapes[s["name"]] = (o, i, r, ss)
            elif kind == 2:
                shapes[s["name"]] = (o, c * h * w)
            elif o > 0 and s["disk_elems"] % o == 0 and s["disk_elems"] != o:
                shapes[s["name"]] = (o, s["disk_elems"] // o)
            else:
                shapes[s["name"]] = (s["disk_elems"],)
        return shapes

    def kernels(self):
        out = []
        for i in range(self.kernel_num()):
            name = C.create_string_buffer(64)
            fl, by, tb, gr = C.c_double(), C.c_double(), C.c_int(), C.c_int()
            _chk(lib().gpx_kernel_info(self.h, C.c_size_t(i), name, C.c_size_t(64), C.byref(fl), C.byref(by), C.byref(tb), C.byref(gr)), "kernel_info")
            out.append(dict(name=name.value.decode(), flops=fl.value, bytes=by.value, total_blocks=tb.value, grid=gr.value))
        return out

    def kernel_num(self):
        return lib().gpx_get_kernel_num(self.h)

    def data_size(self, key):
        return lib().gpx_get_data_size(self.h, key.encode())

    # -- data
    def set_input(self, key, raw, stream=None):
        raw = np.ascontiguousarray(raw)
        _chk(lib().gpx_set_input(self.h, key.encode(), raw.ctypes.data_as(vp), C.c_size_t(raw.nbytes), stream.h if stream else None), f"set_input({key})")
        self._keep = raw

    def get_output(self, key="heads", stream=None):
        raw = np.empty(self.data_size(key), np.uint8)
        _chk(lib().gpx_get_output(self.h, key.encode(), raw.ctypes.data_as(vp), C.c_size_t(raw.nbytes), stream.h if stream else None), f"get_output({key})")
        capi.check(capi.lib().gp_stream_sync(stream.h if stream else None))
        return raw

    def read_storage(self, key):
        raw = np.empty(self.data_size(key), np.uint8)
        _chk(lib().gpx_read_storage(self.h, key.encode(), raw.ctypes.data_as(vp), C.c_size_t(raw.nbytes)), f"read_storage({key})")
        return raw

    # -- execution
    # -- graph workloads
    def graph_info(self):
        v = (C.c_ulonglong * 5)()
        _chk(lib().gpx_graph_info(self.h, v), "graph_info")
        return dict(vertices=v[0], edges=v[1], iterations=v[2], preemptions=v[3], kernels_launched=v[4])

    def graph_result(self, key, np_dtype):
        raw = np.empty(lib().gpx_graph_result_bytes(self.h, key.encode()), np.uint8)
        _chk(lib().gpx_graph_result(self.h, key.encode(), raw.ctypes.data_as(vp), C.c_size_t(raw.nbytes)), f"graph_result({key})")
        return raw.view(np_dtype)

    def graph_inject_preempt(self, iteration, kernel, claim):
        _chk(lib().gpx_graph_inject_preempt(self.h, iteration, kernel, claim), "graph_inject_preempt")

    def set_lc_tasks(self, n):
        _chk(lib().gpx_set_lc_tasks(self.h, int(n)), "set_lc_tasks")

    def miniweather_reductions(self):
        """(mass, total energy) of the "miniweather" workload's current state"""
        m, t = C.c_double(), C.c_double()
        _chk(lib().gpx_miniweather_reductions(self.h, C.byref(m), C.byref(t)), "miniweather_reductions")
        return m.value, t.value

    def execute(self, stream=None):
        _chk(lib().gpx_execute(self.h, stream.h if stream else None), "execute")

    def launch_kernel(self, i, stream=None):
        _chk(lib().gpx_launch_kernel(self.h, C.c_size_t(i), stream.h if stream else None), f"launch_kernel({i})")

    def capture_graph(self, stream):
        _chk(lib().gpx_capture_graph(self.h, stream.h), "capture_graph")

    def uses_program(self):
        return bool(lib().gpx_uses_program(self.h))

    # -- block-level preemption
    def set_flag(self, flag):
        _chk(lib().gpx_set_flag(self.h, vp(flag.dev)), "set_flag")
        self._flag = flag

    def set_running(self, v):
        _chk(lib().gpx_set_running(self.h, int(v)), "set_running")

    def resume(self, stream=None):
        _chk(lib().gpx_resume(self.h, stream.h if stream else None), "resume")

    def stop_point(self, stream=None):
        v = C.c_int()
        _chk(lib().gpx_get_stop_point(self.h, stream.h if stream else None, C.byref(v)), "getStopPoint")
        return v.value

    def last_stop_index(self):
        return lib().gpx_last_stop_index(self.h)

    def inject_preempt(self, kernel, claim):
        _chk(lib().gpx_inject_preempt(self.h, kernel, claim), "inject_preempt")

    def counters(self):
        out = np.zeros(self.kernel_num(), np.int32)
        _chk(lib().gpx_read_counters(self.h, out.ctypes.data_as(vp), C.c_size_t(out.size)), "read_counters")
        return out

    def reset_counters(self, stream=None):
        _chk(lib().gpx_reset_counters(self.h, stream.h if stream else None), "reset_counters")

    def destroy(self):
        if self.h:
            lib().gpx_clear(self.h)
            lib().gpx_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
