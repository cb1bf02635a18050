"""numpy front end of the C oracle (oracle_ops.c, oracle_blp.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by
the cpu_baseline leg of bench.py, never by the product path.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None

ACT_NONE, ACT_RELU, ACT_GELU = 0, 1, 2


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        _LIB = C.CDLL(path)
    return _LIB


def _f(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def gemm_bias_act(A, B, bias=None, residual=None, act=ACT_NONE, b_is_nk=False):
    A, B = _f(A), _f(B)
    M, K = A.shape
    N = B.shape[0] if b_is_nk else B.shape[1]
    assert (B.shape[1] if b_is_nk else B.shape[0]) == K
    bias = None if bias is None else _f(bias)
    residual = None if residual is None else _f(residual)
    out = np.empty((M, N), np.float32)
    lib().orc_gemm_bias_act(C.c_int(M), C.c_int(N), C.c_int(K), _p(A), C.c_long(K), _p(B),
                            C.c_long(B.shape[1]), C.c_int(int(b_is_nk)), _p(bias), _p(residual),
                            C.c_long(N), C.c_int(act), _p(out), C.c_long(N))
    return out


def bmm(A, B, alpha=1.0, b_is_nk=False):
    A, B = _f(A), _f(B)
    batch, M, K = A.shape
    N = B.shape[1] if b_is_nk else B.shape[2]
    out = np.empty((batch, M, N), np.float32)
    lib().orc_bmm(C.c_int(batch), C.c_int(M), C.c_int(N), C.c_int(K), _p(A), C.c_long(K),
                  C.c_long(M * K), _p(B), C.c_long(B.shape[2]), C.c_long(B.shape[1] * B.shape[2]),
                  C.c_int(int(b_is_nk)), C.c_float(alpha), _p(out), C.c_long(N), C.c_long(M * N))
    return out


def conv2d(x, w, bias=None, stride=1, pad=0, residual=None, act=ACT_NONE):
    """x NCHW, w OIHW."""
    x, w = _f(x), _f(w)
    N, Cin, H, W = x.shape
    Cout, Cin2, R, S = w.shape
    assert Cin == Cin2
    sh, sw = (stride, stride) if isinstance(stride, int) else stride
    ph, pw = (pad, pad) if isinstance(pad, int) else pad
    Ho, Wo = (H + 2 * ph - R) // sh + 1, (W + 2 * pw - S) // sw + 1
    bias = None if bias is None else _f(bias)
    residual = None if residual is None else _f(residual)
    out = np.empty((N, Cout, Ho, Wo), np.float32)
    lib().orc_conv2d_nchw(*(C.c_int(v) for v in (N, Cin, H, W, Cout, R, S, sh, sw, ph, pw)),
                          _p(x), _p(w), _p(bias), _p(residual), C.c_int(act), _p(out))
    return out


def pool2d(x, k, stride, pad, mode):
    """mode: 'max' | 'avg' (count_include_pad False) | 'avg_pad' (padding counted as zeros)."""
    x = _f(x)
    N, Cc, H, W = x.shape
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    out = np.empty((N, Cc, Ho, Wo), np.float32)
    lib().orc_pool2d_nchw(*(C.c_int(v) for v in (N, Cc, H, W, k, k, stride, stride, pad, pad,
                                                 {"max": 0, "avg": 1, "avg_pad": 3}[mode])), _p(x), _p(out))
    return out


def global_avgpool(x):
    x = _f(x)
    N, Cc, H, W = x.shape
    out = np.empty((N, Cc), np.float32)
    lib().orc_global_avgpool_nchw(C.c_int(N), C.c_int(Cc), C.c_int(H * W), _p(x), _p(out))
    return out


def add_act(a, b=None, act=ACT_NONE):
    a = _f(a)
    b = None if b is None else _f(b)
    out = np.empty_like(a)
    lib().orc_add_act(C.c_long(a.size), _p(a), _p(b), C.c_int(act), _p(out))
    return out


def scale_shift_act(x, scale, shift, act=ACT_NONE):
    x, scale, shift = _f(x), _f(scale), _f(shift)
    N, Cc, H, W = x.shape
    out = np.empty_like(x)
    lib().orc_scale_shift_act_nchw(C.c_int(N), C.c_int(Cc), C.c_int(H * W), _p(x), _p(scale),
                                   _p(shift), C.c_int(act), _p(out))
    return out


def softmax(x):
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_softmax(C.c_long(x.size // x.shape[-1]), C.c_int(x.shape[-1]), _p(x), _p(out))
    return out


def layernorm(x, gamma, beta, eps, residual=None):
    x, gamma, beta = _f(x), _f(gamma), _f(beta)
    residual = None if residual is None else _f(residual)
    out = np.empty_like(x)
    lib().orc_layernorm(C.c_long(x.size // x.shape[-1]), C.c_int(x.shape[-1]), _p(x), _p(residual),
                        _p(gamma), _p(beta), C.c_float(eps), _p(out))
    return out


def embed(ids, tok, pos, seg=None, seq=None):
    ids = np.ascontiguousarray(ids, dtype=np.int64).reshape(-1)
    tok, pos = _f(tok), _f(pos)
    seg = None if seg is None else _f(seg)
    hidden = tok.shape[1]
    seq = seq or ids.size
    out = np.empty((ids.size, hidden), np.float32)
    lib().orc_embed(C.c_long(ids.size), C.c_int(seq), C.c_int(hidden), _p(ids), _p(tok), _p(pos),
                    _p(seg), _p(out))
    return out


def fold_bn(w, b, gamma, beta, mean, var, eps=1e-5):
    w = _f(w)
    Cout = w.shape[0]
    b = None if b is None else _f(b)
    gamma, beta, mean, var = _f(gamma), _f(beta), _f(mean), _f(var)
    w2, b2 = np.empty_like(w), np.empty(Cout, np.float32)
    lib().orc_fold_bn(C.c_int(Cout), C.c_long(w.size // Cout), _p(w), _p(b), _p(gamma), _p(beta),
                      _p(mean), _p(var), C.c_float(eps), _p(w2), _p(b2))
    return w2, b2


def round_bf16(x):
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_round_bf16(C.c_long(x.size), _p(x), _p(out))
    return out


def round_f16(x):
    return np.asarray(x, np.float32).astype(np.float16).astype(np.float32)


def round_to(x, dtype):
    """Model storage of an activation in `dtype` ('f32' | 'f16' | 'bf16')."""
    if dtype == "f16":
        return round_f16(x)
    if dtype == "bf16":
        return round_bf16(x)
    return np.asarray(x, np.float32)


# ---- block-level-preemption protocol -------------------------------------

def blp_decode(idx, sx, sy):
    x, y, z = C.c_int(), C.c_int(), C.c_int()
    lib().orc_blp_decode(C.c_int(idx), C.c_int(sx), C.c_int(sy), C.byref(x), C.byref(y), C.byref(z))
    return x.value, y.value, z.value


def blp_run_chain(shapes, n_workers, injections=()):
    """shapes: list of (sx, sy, sz); injections: list of (kernel, claim).
    Returns dict(visits=[per-kernel arrays], stops=[...], executed=[...], bad=int)."""
    shape = np.ascontiguousarray(np.array(shapes, np.int32).reshape(-1, 3))
    nk = shape.shape[0]
    totals = shape.prod(axis=1)
    ik = np.ascontiguousarray([i[0] for i in injections], dtype=np.int32)
    ic = np.ascontiguousarray([i[1] for i in injections], dtype=np.int32)
    visits = np.zeros(max(int(totals.sum()), 1), np.int32)
    stops = np.full(max(len(injections), 1), -2, np.int32)
    executed = np.zeros(nk, np.int32)
    bad = lib().orc_blp_run_chain(C.c_int(nk), _p(shape), C.c_int(n_workers), C.c_int(len(injections)),
                                  _p(ik), _p(ic), _p(visits), _p(stops), _p(executed))
    offs = np.concatenate([[0], np.cumsum(totals)])
    return dict(visits=[visits[offs[k]:offs[k + 1]] for k in range(nk)],
                stops=list(stops[:len(injections)]), executed=executed, bad=bad)


def blp_gemm(A, B, bias, tm, tn, n_workers, inject_claims=()):
    A, B, bias = _f(A), _f(B), _f(bias)
    M, K = A.shape
    N = B.shape[1]
    out = np.full((M, N), np.nan, np.float32)
    ic = np.ascontiguousarray(list(inject_claims), dtype=np.int32)
    hits = lib().orc_blp_gemm(C.c_int(M), C.c_int(N), C.c_int(K), _p(A), _p(B), _p(bias), _p(out),
                              C.c_int(tm), C.c_int(tn), C.c_int(n_workers), C.c_int(len(ic)), _p(ic))
    return out, hits
