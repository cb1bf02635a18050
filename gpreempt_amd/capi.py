"""ctypes binding of include/gpreempt_hip.h (libgpreempt_hip.so).

Fails loudly when the library is missing: there is no fallback path.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgpreempt_hip.so")

F32, F16, BF16, I32, I64 = 0, 1, 2, 3, 4
ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2
MAT_AUTO, MAT_STAGED, MAT_PIPE, MAT_PIPE_SPLITK, MAT_WIDE, MAT_WIDE8 = 0, 1, 2, 3, 4, 5
SUCC, FAIL, TIMEOUT, NOTFOUND, OUTOFRANGE, FULL = range(6)
DTYPE_SIZE = {F32: 4, F16: 2, BF16: 2, I32: 4, I64: 8}
DTYPE_BY_NAME = {"f32": F32, "f16": F16, "bf16": BF16}

vp = C.c_void_p


class PreemptCtx(C.Structure):
    _fields_ = [("flag", vp), ("stop_index", vp), ("executed", vp), ("kernel_id", C.c_int),
                ("inject_at", C.c_int), ("max_workgroups", C.c_int), ("poll_every", C.c_int), ("counter_groups", C.c_int), ("fresh", C.c_int), ("left_host", vp),
                ("ckpt", vp), ("ckpt_bytes", C.c_ulonglong), ("done", vp), ("done_launches", C.c_int), ("stamps", vp),
                ("started_host", vp), ("started_seq", C.c_int)]


class LaunchInfo(C.Structure):
    _fields_ = [("total_tiles", C.c_int), ("shape", C.c_int * 3), ("grid", C.c_int), ("block", C.c_int), ("fixed_claims", C.c_int), ("front", C.c_int)]


class GemmParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("M", C.c_int), ("N", C.c_int), ("K", C.c_int),
                ("A", vp), ("lda", C.c_long), ("stride_a", C.c_long),
                ("B", vp), ("ldb", C.c_long), ("stride_b", C.c_long), ("b_is_nk", C.c_int),
                ("C", vp), ("ldc", C.c_long), ("stride_c", C.c_long),
                ("bias", vp), ("residual", vp), ("alpha", C.c_float), ("act", C.c_int), ("batch", C.c_int),
                ("batch_inner", C.c_int), ("stride_a_outer", C.c_long), ("stride_b_outer", C.c_long),
                ("stride_c_outer", C.c_long), ("tile_m", C.c_int), ("tile_n", C.c_int), ("variant", C.c_int),
                ("ln_gamma", vp), ("ln_beta", vp), ("ln_out", vp), ("ln_eps", C.c_float)]


class ConvParams(C.Structure):
    _fields_ = [("dtype", C.c_int)] + [(n, C.c_int) for n in
                ("N", "H", "W", "Cin", "Cout", "R", "S", "stride_h", "stride_w", "pad_h", "pad_w")] + [
                ("in_", vp), ("in_pix_stride", C.c_long), ("weight", vp), ("bias", vp),
                ("residual", vp), ("res_pix_stride", C.c_long), ("out", vp), ("out_pix_stride", C.c_long),
                ("act", C.c_int), ("tile_m", C.c_int), ("tile_n", C.c_int), ("variant", C.c_int)]


class LayoutParams(C.Structure):
    _fields_ = [("dtype_in", C.c_int), ("dtype_out", C.c_int), ("N", C.c_int), ("C", C.c_int), ("H", C.c_int),
                ("W", C.c_int), ("c_pad", C.c_int), ("in_", vp), ("out", vp)]


class PoolParams(C.Structure):
    _fields_ = [("dtype", C.c_int)] + [(n, C.c_int) for n in ("N", "H", "W", "C", "R", "S", "stride", "pad", "mode")] + [
                ("in_", vp), ("in_pix_stride", C.c_long), ("out", vp), ("out_pix_stride", C.c_long)]


class EltwiseParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("rows", C.c_long), ("cols", C.c_int), ("a", vp), ("a_stride", C.c_long),
                ("b", vp), ("b_stride", C.c_long), ("scale", vp), ("shift", vp), ("out", vp),
                ("out_stride", C.c_long), ("act", C.c_int)]


class SoftmaxParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("rows", C.c_long), ("cols", C.c_int), ("x", vp), ("out", vp), ("scale", C.c_float)]


class LayernormParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("rows", C.c_long), ("cols", C.c_int), ("x", vp), ("residual", vp),
                ("gamma", vp), ("beta", vp), ("out", vp), ("eps", C.c_float)]


class AttentionParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("batch", C.c_int), ("heads", C.c_int), ("seq", C.c_int), ("head_dim", C.c_int),
                ("q", vp), ("k", vp), ("v", vp), ("ld_qkv", C.c_long), ("out", vp), ("ld_out", C.c_long), ("scale", C.c_float)]


class MiniweatherParams(C.Structure):
    _fields_ = [("kernel", C.c_int), ("nx", C.c_int), ("nz", C.c_int), ("dt", C.c_float), ("dx", C.c_float), ("dz", C.c_float),
                ("state", vp), ("flux", vp), ("state_init", vp), ("state_out", vp), ("hydro", vp)]


class GraphParams(C.Structure):
    _fields_ = [("kernel", C.c_int), ("level", C.c_uint), ("vertex_count", C.c_ulonglong), ("vertex_list", vp), ("edge_list", vp),
                ("weight_list", vp), ("label", vp), ("active", vp), ("next_active", vp), ("comp", vp), ("delta", vp), ("residual", vp),
                ("value", vp), ("alpha", C.c_float), ("tolerance", C.c_float), ("cost", vp), ("new_cost", vp), ("changed", vp), ("lanes_per_vertex", C.c_int)]


class EmbedParams(C.Structure):
    _fields_ = [("dtype", C.c_int), ("tokens", C.c_long), ("seq", C.c_int), ("hidden", C.c_int), ("vocab", C.c_long),
                ("ids", vp), ("tok", vp), ("pos", vp), ("seg", vp), ("out", vp)]


# every symbol include/gpreempt_hip.h declares
SYMBOLS = """gp_init gp_last_error gp_device_info gp_device_clock gp_stream_create gp_stream_destroy gp_stream_sync
gp_stream_query gp_stream_priority gp_stream_set_priority gp_stream_native gp_event_create gp_event_destroy gp_event_record
gp_event_sync gp_event_query gp_event_elapsed_ms gp_malloc gp_free gp_host_alloc gp_host_free gp_memcpy_h2d gp_memcpy_d2h
gp_memcpy_h2d_async gp_memcpy_d2h_async gp_memcpy_d2d_async gp_fill32_async gp_flag_create gp_flag_destroy gp_store_word_async gp_flag_relay_start
gp_launch_gemm gp_gemm_ln_supported gp_launch_gemm_noalloc gp_gemm_ckpt_bytes gp_conv_ckpt_bytes gp_ckpt_reset_async gp_launch_conv2d gp_launch_nchw_to_nhwc gp_launch_pool2d gp_launch_eltwise gp_launch_softmax
gp_launch_layernorm gp_launch_attention gp_launch_miniweather gp_launch_graph gp_launch_embed gp_launch_gate gp_launch_noop gp_graph_begin gp_graph_end gp_graph_launch
gp_graph_destroy gp_program_create gp_program_destroy gp_program_add_gemm gp_program_add_conv2d
gp_program_add_nchw_to_nhwc gp_program_add_pool2d gp_program_add_eltwise gp_program_add_softmax gp_program_add_layernorm
gp_program_add_attention gp_program_add_embed gp_program_add_copy gp_program_finalize gp_program_launch gp_program_layers gp_program_read_state""".split()

_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(LIB_PATH)
        _lib.gp_last_error.restype = C.c_char_p
        _lib.gp_stream_native.restype = vp
    return _lib


class GpError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__(f"gp status {status}: {msg}")
        self.status = status


def check(rc):
    if rc != 0:
        raise GpError(rc, lib().gp_last_error().decode())


def init(device=0):
    check(lib().gp_init(device))


def device_info():
    cus, khz = C.c_int(), C.c_int()
    name = C.create_string_buffer(256)
    check(lib().gp_device_info(C.byref(cus), C.byref(khz), name, C.c_size_t(256)))
    return cus.value, khz.value, name.value.decode()


# ---- numpy <-> 16-bit storage -------------------------------------------------------------

def to_storage(a, dtype):
    """float array -> bytes-compatible numpy array of the device dtype."""
    a = np.asarray(a)
    if dtype == F32:
        return np.ascontiguousarray(a, np.float32)
    if dtype == F16:
        return np.ascontiguousarray(a.astype(np.float16))
    if dtype == BF16:
        u = np.ascontiguousarray(a, np.float32).view(np.uint32)
        r = ((u >> 16) & 1) + 0x7FFF
        return ((u + r) >> 16).astype(np.uint16)
    if dtype == I64:
        return np.ascontiguousarray(a, np.int64)
    if dtype == I32:
        return np.ascontiguousarray(a, np.int32)
    raise ValueError(dtype)


def from_storage(raw, dtype):
    if dtype == F32:
        return raw.view(np.float32)
    if dtype == F16:
        return raw.view(np.float16).astype(np.float32)
    if dtype == BF16:
        return (raw.view(np.uint16).astype(np.uint32) << 16).view(np.float32)
    if dtype == I64:
        return raw.view(np.int64)
    if dtype == I32:
        return raw.view(np.int32)
    raise ValueError(dtype)


class DevBuf:
    """A device allocation owned through gp_malloc / gp_free."""

    def __init__(self, nbytes):
        self.nbytes = int(nbytes)
        p = vp()
        check(lib().gp_malloc(C.byref(p), C.c_size_t(self.nbytes)))
        self.ptr = p.value

    @classmethod
    def from_array(cls, a, dtype=None):
        raw = np.ascontiguousarray(a) if dtype is None else to_storage(a, dtype)
        b = cls(raw.nbytes)
        b.upload(raw)
        b.shape, b.dtype = np.asarray(a).shape, dtype
        return b

    def upload(self, raw):
        raw = np.ascontiguousarray(raw)
        assert raw.nbytes <= self.nbytes
        check(lib().gp_memcpy_h2d(vp(self.ptr), raw.ctypes.data_as(vp), C.c_size_t(raw.nbytes)))

    def download(self, dtype=None, shape=None, np_dtype=np.uint8):
        raw = np.empty(self.nbytes, np.uint8)
        check(lib().gp_memcpy_d2h(raw.ctypes.data_as(vp), vp(self.ptr), C.c_size_t(self.nbytes)))
        out = from_storage(raw, dtype) if dtype is not None else raw.view(np_dtype)
        return out.reshape(shape) if shape is not None else out

    def fill32(self, value=0):
        check(lib().gp_fill32_async(vp(self.ptr), C.c_uint32(value & 0xFFFFFFFF), C.c_size_t(self.nbytes // 4), None))
        check(lib().gp_stream_sync(None))

    def free(self):
        if self.ptr:
            check(lib().gp_free(vp(self.ptr)))
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class Stream:
    def __init__(self, priority=0):
        h = vp()
        check(lib().gp_stream_create(priority, C.byref(h)))
        self.h = h

    def sync(self):
        check(lib().gp_stream_sync(self.h))

    def idle(self):
        v = C.c_int()
        check(lib().gp_stream_query(self.h, C.byref(v)))
        return bool(v.value)

    def destroy(self):
        if self.h:
            check(lib().gp_stream_destroy(self.h))
            self.h = None


class Event:
    def __init__(self):
        h = vp()
        check(lib().gp_event_create(C.byref(h)))
        self.h = h

    def record(self, stream=None):
        check(lib().gp_event_record(self.h, stream.h if stream else None))

    def sync(self):
        check(lib().gp_event_sync(self.h))

    def elapsed_ms(self, later):
        ms = C.c_float()
        check(lib().gp_event_elapsed_ms(self.h, later.h, C.byref(ms)))
        return ms.value


class Flag:
    """The shared preempt flag: host-visible int, device-visible address."""

    def __init__(self):
        hp, dp = C.POINTER(C.c_int)(), vp()
        check(lib().gp_flag_create(C.byref(hp), C.byref(dp)))
        self.host, self.dev = hp, dp.value

    def set(self, v):
        self.host[0] = int(v)

    def get(self):
        return int(self.host[0])

    def destroy(self):
        if self.host:
            check(lib().gp_flag_destroy(self.host))
            self.host = None


class BlpState:
    """stop_index (one int, -1) and executed[n] counters in device memory
    (BLPExecutor::init, reference src/executor.cpp:328-334)."""

    COUNTER_STRIDE = 16  # ints between the counters of one kernel when it has several (64-byte lines)

    def __init__(self, n_kernels, flag, counter_groups=1):
        """counter_groups = 1 is the reference's layout (one int per kernel); BLPExecutor uses 32
        counters per kernel, each on its own line (gp_preempt_ctx::counter_groups)."""
        self.n = n_kernels
        self.flag = flag
        self.groups = counter_groups
        self.ints_per_kernel = 1 if counter_groups <= 1 else counter_groups * self.COUNTER_STRIDE
        self.stop = DevBuf(4)
        self.executed = DevBuf(4 * n_kernels * self.ints_per_kernel)
        self.stop.upload(np.array([-1], np.int32))
        self.reset()

    def reset(self):
        self.executed.upload(np.zeros(self.n * self.ints_per_kernel, np.int32))
        if getattr(self, "done", None):
            self.done.upload(np.zeros(self.n * self.ints_per_kernel, np.int32))

    def ctx(self, kernel_id=0, inject_at=-1, max_workgroups=0, poll_every=0, fresh=0, done_launches=0, started=None, started_seq=0):
        ck = getattr(self, "ckpt", None)
        return PreemptCtx(self.flag.dev, self.stop.ptr, self.executed.ptr + 4 * kernel_id * self.ints_per_kernel, kernel_id, inject_at, max_workgroups,
                          poll_every, self.groups if self.groups > 1 else 0, fresh, None, ck.ptr if ck else None, ck.nbytes if ck else 0,
                          (self.done.ptr + 4 * kernel_id * self.ints_per_kernel) if getattr(self, "done", None) else None, done_launches,
                          self.stamps.ptr if getattr(self, "stamps", None) else None,
                          started.dev if started is not None else None, started_seq)

    def enable_done_counters(self):
        """Counters of the workers that have left (gp_preempt_ctx::done), cleared by reset()."""
        self.done = DevBuf(4 * self.n * self.ints_per_kernel)
        self.done.upload(np.zeros(self.n * self.ints_per_kernel, np.int32))

    STAMP_WORDS = 8 + 1024

    def enable_stamps(self):
        """Device time stamps of the preemption (gp_preempt_ctx::stamps), cleared."""
        self.stamps = DevBuf(8 * self.STAMP_WORDS)
        self.stamps.upload(np.zeros(self.STAMP_WORDS, np.uint64))

    def read_stamps(self):
        """(stop recorded, first claim, latest exit, number of exit stamps) in device clock ticks; 0 = not written."""
        raw = np.empty(self.STAMP_WORDS, np.uint64)
        check(lib().gp_memcpy_d2h(raw.ctypes.data_as(vp), vp(self.stamps.ptr), C.c_size_t(raw.nbytes)))
        ex = raw[8:]
        return int(raw[0]), int(raw[1]), int(ex.max()), int((ex != 0).sum())

    def enable_checkpoints(self, params):
        """Allocates the workspace that lets the GEMM `params` leave its tiles half-way (if it can)."""
        n = C.c_size_t(0)
        fn = lib().gp_conv_ckpt_bytes if isinstance(params, ConvParams) else lib().gp_gemm_ckpt_bytes
        check(fn(C.byref(params), C.byref(n)))
        self.ckpt = DevBuf(n.value) if n.value else None
        if self.ckpt:
            check(lib().gp_ckpt_reset_async(vp(self.ckpt.ptr), None))
            check(lib().gp_stream_sync(None))
        return n.value

    def checkpoint_headers(self, n):
        """valid / kernel id / tile / next K-step of the first n workgroup slots."""
        raw = np.empty(n * 16, np.int32)
        check(lib().gp_memcpy_d2h(raw.ctypes.data_as(vp), vp(self.ckpt.ptr), C.c_size_t(raw.nbytes)))
        return raw.reshape(n, 16)[:, :4].copy()

    def stop_index(self):
        return int(self.stop.download(np_dtype=np.int32)[0])

    def clear_stop(self):
        self.stop.upload(np.array([-1], np.int32))

    def counters(self):
        return self.executed.download(np_dtype=np.int32).copy()


def _ptr(b):
    return None if b is None else (b.ptr if isinstance(b, DevBuf) else b)


def launch(fn_name, params, ctx=None, stream=None):
    info = LaunchInfo()
    fn = getattr(lib(), fn_name)
    check(fn(C.byref(params), C.byref(ctx) if ctx is not None else None, stream.h if stream else None, C.byref(info)))
    return info
