"""Shared helpers of the GPU parity tests: tolerances, layout conversion, operator drivers that
call the C ABI and return numpy arrays in the oracle's NCHW / row-major conventions."""
import numpy as np

from oracle import oracle as O

# Tolerances stated by the north star: 1e-4 relative for fp32, 1e-2 for fp16 / bf16.  "Relative"
# is measured against the magnitude of the reference tensor (max |ref|): single elements of a
# dot product can cancel to ~0, where an element-wise ratio says nothing.
TOL = {"f32": 1e-4, "f16": 1e-2, "bf16": 1e-2}


def rel_err(got, ref):
    return float(np.abs(np.asarray(got, np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))


def nchw_to_nhwc(x, c_pad=None):
    x = np.transpose(x, (0, 2, 3, 1))
    if c_pad and c_pad > x.shape[3]:
        x = np.concatenate([x, np.zeros(x.shape[:3] + (c_pad - x.shape[3],), x.dtype)], axis=3)
    return np.ascontiguousarray(x)


def nhwc_to_nchw(x):
    return np.ascontiguousarray(np.transpose(x, (0, 3, 1, 2)))


def oihw_to_ohwi(w, c_pad=None):
    w = np.transpose(w, (0, 2, 3, 1))
    if c_pad and c_pad > w.shape[3]:
        w = np.concatenate([w, np.zeros(w.shape[:3] + (c_pad - w.shape[3],), w.dtype)], axis=3)
    return np.ascontiguousarray(w)


def sync(gp):
    gp.check(gp.lib().gp_stream_sync(None))


def gpu_conv2d(gp, dt, x, w, bias=None, stride=1, pad=0, residual=None, act=0, ctx=None, tile=0, variant=0, tile_n=None):
    """x NCHW, w OIHW, residual NCHW (already rounded to dt).  Returns (NCHW result, info)."""
    dtype = gp.DTYPE_BY_NAME[dt]
    vec = 4 if dt == "f32" else 8
    N, Cin, H, W = x.shape
    Cout, _, R, S = w.shape
    cp = -(-Cin // vec) * vec
    Ho, Wo = (H + 2 * pad - R) // stride + 1, (W + 2 * pad - S) // stride + 1
    dx = gp.DevBuf.from_array(nchw_to_nhwc(x, cp), dtype)
    dw = gp.DevBuf.from_array(oihw_to_ohwi(w, cp), dtype)
    db = gp.DevBuf.from_array(bias, dtype) if bias is not None else None
    dr = gp.DevBuf.from_array(nchw_to_nhwc(residual), dtype) if residual is not None else None
    do = gp.DevBuf(N * Ho * Wo * Cout * gp.DTYPE_SIZE[dtype])
    do.fill32(0xFFFFFFFF if dt == "f32" else 0x7E007E00)
    p = gp.ConvParams(dtype=dtype, N=N, H=H, W=W, Cin=cp, Cout=Cout, R=R, S=S, stride_h=stride, stride_w=stride,
                      pad_h=pad, pad_w=pad, in_=dx.ptr, in_pix_stride=cp, weight=dw.ptr, bias=gp._ptr(db),
                      residual=gp._ptr(dr), res_pix_stride=Cout, out=do.ptr, out_pix_stride=Cout, act=act,
                      tile_m=tile, tile_n=tile if tile_n is None else tile_n, variant=variant)
    info = gp.launch("gp_launch_conv2d", p, ctx)
    sync(gp)
    out = do.download(dtype, (N, Ho, Wo, Cout)).copy()
    return nhwc_to_nchw(out), info, (p, do, (dx, dw, db, dr))
