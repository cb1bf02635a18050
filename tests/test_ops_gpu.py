"""Parity of every operator kernel behind the C ABI with the CPU oracle, on seeded inputs."""
import numpy as np
import pytest

from oracle import oracle as O
from helpers import TOL, gpu_conv2d, nchw_to_nhwc, nhwc_to_nchw, rel_err, sync

pytestmark = pytest.mark.gpu
DTS = ["f32", "f16", "bf16"]


def rnd(rng, shape, dt, lo=-1.0, hi=1.0):
    return O.round_to(rng.uniform(lo, hi, shape).astype(np.float32), dt)


CONV_CASES = [
    # N, Cin, H, W, Cout, k, stride, pad
    (1, 3, 32, 32, 64, 7, 2, 3),     # stem: Cin padded to the vector width
    (2, 64, 14, 14, 64, 1, 1, 0),    # 1x1 == GEMM
    (1, 64, 15, 13, 96, 3, 1, 1),    # odd sizes, ragged tiles
    (1, 128, 16, 16, 256, 3, 2, 1),  # strided 3x3
    (2, 256, 8, 8, 512, 1, 2, 0),    # strided 1x1 (projection shortcut)
    (1, 8, 5, 5, 8, 5, 1, 2),        # window as large as the image
    (2, 96, 9, 9, 64, 3, 1, 1),      # Cin not a multiple of the K-step: taps straddle stages
    (8, 256, 14, 14, 256, 3, 1, 1),  # the dominant layer of ResNet-152 at batch 8
]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("case", CONV_CASES)
def test_conv2d_matches_oracle(gp, dt, case):
    N, Cin, H, W, Cout, k, stride, pad = case
    rng = np.random.default_rng(hash(case) % 2**31)
    x = rnd(rng, (N, Cin, H, W), dt)
    w = rnd(rng, (Cout, Cin, k, k), dt, -0.2, 0.2)
    b = rnd(rng, (Cout,), dt, -0.1, 0.1)
    Ho, Wo = (H + 2 * pad - k) // stride + 1, (W + 2 * pad - k) // stride + 1
    res = rnd(rng, (N, Cout, Ho, Wo), dt)
    ref = O.conv2d(x, w, b, stride, pad, res, O.ACT_RELU)
    for tile, variant in ((64, 1), (128, 1), (0, 0), (64, 2), (128, 2), (64, 3), (32, 3)):
        got, info, _ = gpu_conv2d(gp, dt, x, w, b, stride, pad, res, gp.ACT_RELU, tile=tile, variant=variant)
        assert np.isfinite(got).all(), (dt, case, tile, variant)
        assert rel_err(got, ref) < TOL[dt], (dt, case, tile, variant)
    # the wide split-K bodies (16 or 8 wavefronts per tile): pointwise convolutions run on their GEMM form, the others
    # on the gathered-operand form, which needs whole K-blocks per filter tap and at most 32 taps
    bk = 32 if dt == "f32" else 64
    if (k == 1 and stride == 1 and pad == 0) or (Cin % bk == 0 and k * k <= 32):
        split_k = gpu_conv2d(gp, dt, x, w, b, stride, pad, res, gp.ACT_RELU, tile=32, variant=3)[0]
        for tm, tn, variant in ((32, 32, gp.MAT_WIDE), (32, 32, gp.MAT_WIDE8), (64, 32, gp.MAT_WIDE), (64, 64, gp.MAT_WIDE8)):
            got, info, _ = gpu_conv2d(gp, dt, x, w, b, stride, pad, res, gp.ACT_RELU, tile=tm, tile_n=tn, variant=variant)
            assert info.total_tiles == -(-N * Ho * Wo // tm) * -(-Cout // tn) and info.block == (1024 if variant == gp.MAT_WIDE else 512)
            assert rel_err(got, ref) < TOL[dt], (dt, case, tm, tn, variant)
            # the same summation as the four-wavefront split-K body: the same bits
            assert got.tobytes() == split_k.tobytes(), (dt, case, tm, tn, variant)
    else:
        with pytest.raises(gp.GpError):
            gpu_conv2d(gp, dt, x, w, b, stride, pad, res, gp.ACT_RELU, tile=32, variant=gp.MAT_WIDE)


def test_conv2d_channel_slices(gp):
    """Reading and writing channel slices of wider NHWC buffers (concatenation without a copy)."""
    rng = np.random.default_rng(5)
    N, H, W, Cin, Cout, Cbuf = 1, 6, 6, 32, 32, 96
    x = rnd(rng, (N, Cin, H, W), "f32")
    w = rnd(rng, (Cout, Cin, 3, 3), "f32", -0.2, 0.2)
    buf = np.zeros((N, H, W, Cbuf), np.float32)
    buf[..., :Cin] = nchw_to_nhwc(x)
    dbuf = gp.DevBuf.from_array(buf, gp.F32)
    dw = gp.DevBuf.from_array(np.ascontiguousarray(np.transpose(w, (0, 2, 3, 1))), gp.F32)
    p = gp.ConvParams(dtype=gp.F32, N=N, H=H, W=W, Cin=Cin, Cout=Cout, R=3, S=3, stride_h=1, stride_w=1, pad_h=1, pad_w=1,
                      in_=dbuf.ptr, in_pix_stride=Cbuf, weight=dw.ptr, out=dbuf.ptr + 4 * 64, out_pix_stride=Cbuf)
    gp.launch("gp_launch_conv2d", p)
    sync(gp)
    out = dbuf.download(gp.F32, (N, H, W, Cbuf))
    assert np.array_equal(out[..., :Cin], buf[..., :Cin]) and np.all(out[..., Cin:64] == 0)
    assert rel_err(nhwc_to_nchw(out[..., 64:]), O.conv2d(x, w, None, 1, 1)) < 1e-4
    # the same through the wide bodies' gathered-operand form (Cin = 32 is one fp32 K-block per filter tap)
    results = []
    for tm, tn, variant in ((32, 32, gp.MAT_PIPE_SPLITK), (32, 32, gp.MAT_WIDE), (64, 64, gp.MAT_WIDE8)):
        dbuf.upload(buf)
        p.tile_m, p.tile_n, p.variant = tm, tn, variant
        gp.launch("gp_launch_conv2d", p)
        sync(gp)
        results.append(dbuf.download(gp.F32, (N, H, W, Cbuf)).copy())
        assert rel_err(nhwc_to_nchw(results[-1][..., 64:]), O.conv2d(x, w, None, 1, 1)) < 1e-4
        assert np.array_equal(results[-1][..., :64], out[..., :64])
    # the split-K summation of the four-wavefront body, bit for bit
    assert np.array_equal(results[1], results[0]) and np.array_equal(results[2], results[0])


@pytest.mark.parametrize("dt_in,dt_out", [("f32", "f32"), ("f32", "f16"), ("f16", "f16"), ("f32", "bf16")])
def test_nchw_to_nhwc(gp, dt_in, dt_out):
    rng = np.random.default_rng(2)
    N, Cc, H, W = 2, 3, 19, 23
    cp = 4 if dt_out == "f32" else 8
    x = rnd(rng, (N, Cc, H, W), dt_in)
    di = gp.DevBuf.from_array(x, gp.DTYPE_BY_NAME[dt_in])
    do = gp.DevBuf(N * H * W * cp * gp.DTYPE_SIZE[gp.DTYPE_BY_NAME[dt_out]])
    p = gp.LayoutParams(gp.DTYPE_BY_NAME[dt_in], gp.DTYPE_BY_NAME[dt_out], N, Cc, H, W, cp, di.ptr, do.ptr)
    info = gp.launch("gp_launch_nchw_to_nhwc", p)
    sync(gp)
    got = do.download(gp.DTYPE_BY_NAME[dt_out], (N, H, W, cp))
    assert np.array_equal(got, O.round_to(nchw_to_nhwc(x, cp), dt_out))  # a pure copy/convert: exact
    assert info.total_tiles == N * -(-H * W // 256)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("cfg", [(3, 2, 1, "max"), (2, 2, 0, "max"), (2, 2, 0, "avg"), (3, 1, 1, "avg"), (3, 1, 1, "avg_pad"), (7, 1, 0, "gap"),
                                 # 3 x 3 windows moving by 2 take the path with four outputs per item: odd and even output sizes, every mode
                                 (3, 2, 0, "max", 15, 13), (3, 2, 1, "avg", 15, 13), (3, 2, 1, "avg_pad", 16, 9), (3, 2, 1, "max", 9, 16), (3, 2, 0, "avg", 5, 5)])
def test_pool2d(gp, dt, cfg):
    k, stride, pad, mode = cfg[:4]
    rng = np.random.default_rng(k * 10 + stride)
    N, Cc, H, W = 2, 24, 14, 14 if mode != "gap" else 7
    if mode == "gap":
        H = 7
    if len(cfg) > 4:
        H, W = cfg[4:]
    x = rnd(rng, (N, Cc, H, W), dt)
    dtype = gp.DTYPE_BY_NAME[dt]
    di = gp.DevBuf.from_array(nchw_to_nhwc(x), dtype)
    if mode == "gap":
        ref = O.global_avgpool(x).reshape(N, Cc, 1, 1)
        Ho = Wo = 1
    else:
        ref = O.pool2d(x, k, stride, pad, mode)
        Ho, Wo = ref.shape[2:]
    do = gp.DevBuf(N * Ho * Wo * Cc * gp.DTYPE_SIZE[dtype])
    p = gp.PoolParams(dtype, N, H, W, Cc, k, k, stride, pad, {"max": 0, "avg": 1, "gap": 2, "avg_pad": 3}[mode], di.ptr, Cc, do.ptr, Cc)
    gp.launch("gp_launch_pool2d", p)
    sync(gp)
    got = nhwc_to_nchw(do.download(dtype, (N, Ho, Wo, Cc)))
    if mode == "max":
        assert np.array_equal(got, ref)  # selection only: exact in every dtype
    else:
        assert rel_err(got, ref) < TOL[dt]


@pytest.mark.parametrize("dt", DTS)
def test_eltwise_add_scale_shift_relu(gp, dt):
    rng = np.random.default_rng(4)
    rows, cols = 777, 40
    a, b = rnd(rng, (rows, cols), dt), rnd(rng, (rows, cols), dt)
    sc, sh = rnd(rng, (cols,), dt, 0.5, 1.5), rnd(rng, (cols,), dt)
    dtype = gp.DTYPE_BY_NAME[dt]
    da, db, dsc, dsh = (gp.DevBuf.from_array(v, dtype) for v in (a, b, sc, sh))
    do = gp.DevBuf(rows * cols * gp.DTYPE_SIZE[dtype])
    # add + relu (residual join)
    p = gp.EltwiseParams(dtype, rows, cols, da.ptr, cols, db.ptr, cols, None, None, do.ptr, cols, gp.ACT_RELU)
    gp.launch("gp_launch_eltwise", p)
    sync(gp)
    assert rel_err(do.download(dtype, (rows, cols)), O.add_act(a, b, O.ACT_RELU)) < TOL[dt]
    # per-channel affine + relu (unfolded batch-norm), checked through the NCHW oracle
    p = gp.EltwiseParams(dtype, rows, cols, da.ptr, cols, None, 0, dsc.ptr, dsh.ptr, do.ptr, cols, gp.ACT_RELU)
    gp.launch("gp_launch_eltwise", p)
    sync(gp)
    ref = O.scale_shift_act(a.T.reshape(1, cols, rows, 1), sc, sh, O.ACT_RELU).reshape(cols, rows).T
    assert rel_err(do.download(dtype, (rows, cols)), ref) < TOL[dt]
    # gelu
    p = gp.EltwiseParams(dtype, rows, cols, da.ptr, cols, None, 0, None, None, do.ptr, cols, gp.ACT_GELU)
    gp.launch("gp_launch_eltwise", p)
    sync(gp)
    assert rel_err(do.download(dtype, (rows, cols)), O.add_act(a, None, O.ACT_GELU)) < TOL[dt]


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape", [(12 * 128, 128), (5, 1000), (3, 7), (33, 384)])
def test_softmax(gp, dt, shape):
    rng = np.random.default_rng(shape[1])
    x = rnd(rng, shape, dt, -8, 8)
    dtype = gp.DTYPE_BY_NAME[dt]
    dx = gp.DevBuf.from_array(x, dtype)
    do = gp.DevBuf(x.size * gp.DTYPE_SIZE[dtype])
    gp.launch("gp_launch_softmax", gp.SoftmaxParams(dtype, shape[0], shape[1], dx.ptr, do.ptr, 0.125))
    sync(gp)
    got = do.download(dtype, shape)
    assert rel_err(got, O.softmax(x * np.float32(0.125))) < TOL[dt]
    assert np.abs(got.sum(axis=1) - 1).max() < (1e-5 if dt == "f32" else 2e-2)


@pytest.mark.parametrize("dt", DTS)
@pytest.mark.parametrize("shape", [(128, 768), (7, 3072), (5, 8)])
def test_layernorm(gp, dt, shape):
    rng = np.random.default_rng(shape[1])
    x, r = rnd(rng, shape, dt, -2, 2), rnd(rng, shape, dt, -2, 2)
    g, b = rnd(rng, (shape[1],), dt, 0.5, 1.5), rnd(rng, (shape[1],), dt)
    dtype = gp.DTYPE_BY_NAME[dt]
    dx, dr, dg, db = (gp.DevBuf.from_array(v, dtype) for v in (x, r, g, b))
    do = gp.DevBuf(x.size * gp.DTYPE_SIZE[dtype])
    for res in (None, dr):
        p = gp.LayernormParams(dtype, shape[0], shape[1], dx.ptr, gp._ptr(res), dg.ptr, db.ptr, do.ptr, 1e-12)
        gp.launch("gp_launch_layernorm", p)
        sync(gp)
        ref = O.layernorm(x, g, b, 1e-12, None if res is None else r)
        assert rel_err(do.download(dtype, shape), ref) < TOL[dt]


def _sample_rows(rng, rows):
    return np.unique(np.concatenate([np.arange(512), np.arange(rows - 512, rows), rng.integers(0, rows, 1024)]))


@pytest.mark.parametrize("op,dt,rows,cols", [("add", "f16", 65539, 1024), ("layernorm", "f16", 65537, 768), ("layernorm", "f32", 16385, 256),
                                             ("layernorm", "bf16", 16386, 1024), ("softmax", "f16", (1 << 19) + 5, 128)])
def test_large_tensors_streamed_and_paired_rows(gp, op, dt, rows, cols):
    """Tensors past the last-level cache take nontemporal loads and stores, full eltwise tiles skip
    their bounds checks, and layer-norm gives a wavefront two rows: sampled rows against the oracle,
    and bit for bit against the same rows sent through a small launch (the default forms)."""
    rng = np.random.default_rng(rows)
    dtype = gp.DTYPE_BY_NAME[dt]
    x, r = rnd(rng, (rows, cols), dt, -2, 2), rnd(rng, (rows, cols), dt, -2, 2)
    g, b = rnd(rng, (cols,), dt, 0.5, 1.5), rnd(rng, (cols,), dt)
    idx = _sample_rows(rng, rows)

    def run(xa, ra):
        n = xa.shape[0]
        dx, dr, dg, db = (gp.DevBuf.from_array(v, dtype) for v in (xa, ra, g, b))
        do = gp.DevBuf(xa.size * gp.DTYPE_SIZE[dtype])
        if op == "add":
            gp.launch("gp_launch_eltwise", gp.EltwiseParams(dtype, n, cols, dx.ptr, cols, dr.ptr, cols, None, None, do.ptr, cols, gp.ACT_RELU))
        elif op == "layernorm":
            gp.launch("gp_launch_layernorm", gp.LayernormParams(dtype, n, cols, dx.ptr, dr.ptr, dg.ptr, db.ptr, do.ptr, 1e-12))
        else:
            gp.launch("gp_launch_softmax", gp.SoftmaxParams(dtype, n, cols, dx.ptr, do.ptr, 0.125))
        sync(gp)
        return do.download(dtype, (n, cols))

    big = run(x, r)
    xs, rs = np.ascontiguousarray(x[idx]), np.ascontiguousarray(r[idx])
    small = run(xs, rs)
    bad = np.nonzero((big[idx] != small).any(axis=1))[0]
    assert bad.size == 0, f"{bad.size} of {idx.size} sampled rows differ from the small launch, first rows {idx[bad[:8]]}, max diff {np.abs(big[idx] - small).max()}"
    ref = O.add_act(xs, rs, O.ACT_RELU) if op == "add" else O.layernorm(xs, g, b, 1e-12, rs) if op == "layernorm" else O.softmax(xs * np.float32(0.125))
    assert rel_err(big[idx], ref) < TOL[dt]
    if op == "add":  # cheap enough to check everywhere
        assert big.tobytes() == O.round_to(np.maximum(x + r, 0), dt).astype(big.dtype).tobytes()


@pytest.mark.parametrize("dt", DTS)
def test_embed(gp, dt):
    rng = np.random.default_rng(9)
    vocab, seq, hidden, batch = 500, 16, 64, 3
    ids = rng.integers(0, vocab, batch * seq)
    tok, pos, seg = rnd(rng, (vocab, hidden), dt), rnd(rng, (seq, hidden), dt), rnd(rng, (1, hidden), dt)
    dtype = gp.DTYPE_BY_NAME[dt]
    dids = gp.DevBuf.from_array(ids.astype(np.int64))
    dt_, dp, ds = (gp.DevBuf.from_array(v, dtype) for v in (tok, pos, seg))
    do = gp.DevBuf(batch * seq * hidden * gp.DTYPE_SIZE[dtype])
    p = gp.EmbedParams(dtype, batch * seq, seq, hidden, vocab, dids.ptr, dt_.ptr, dp.ptr, ds.ptr, do.ptr)
    gp.launch("gp_launch_embed", p)
    sync(gp)
    assert rel_err(do.download(dtype, (batch * seq, hidden)), O.embed(ids, tok, pos, seg[0], seq)) < TOL[dt]


def test_every_op_resumes_bit_exact(gp):
    """Each memory-bound kernel, preempted at a tile boundary and resumed, equals its
    uninterrupted run bit for bit."""
    rng = np.random.default_rng(11)
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    rows, cols = 4096, 256
    a = rnd(rng, (rows, cols), "f16")
    g = rnd(rng, (cols,), "f16")
    da, dg = gp.DevBuf.from_array(a, gp.F16), gp.DevBuf.from_array(g, gp.F16)
    do = gp.DevBuf(rows * cols * 2)
    cases = {
        "gp_launch_eltwise": gp.EltwiseParams(gp.F16, rows, cols, da.ptr, cols, da.ptr, cols, dg.ptr, dg.ptr, do.ptr, cols, gp.ACT_GELU),
        "gp_launch_softmax": gp.SoftmaxParams(gp.F16, rows, cols, da.ptr, do.ptr, 1.0),
        "gp_launch_layernorm": gp.LayernormParams(gp.F16, rows, cols, da.ptr, da.ptr, dg.ptr, dg.ptr, do.ptr, 1e-5),
        "gp_launch_pool2d": gp.PoolParams(gp.F16, 1, 64, 64, cols, 3, 3, 2, 1, 0, da.ptr, cols, do.ptr, cols),
    }
    for fn, p in cases.items():
        do.fill32(0)
        info = gp.launch(fn, p)
        sync(gp)
        base = do.download().copy()
        st.reset()
        do.fill32(0)
        gp.launch(fn, p, st.ctx(inject_at=info.total_tiles // 3, max_workgroups=8))
        sync(gp)
        assert flag.get() == 1 and st.stop_index() == 0, fn
        assert st.counters()[0] < info.total_tiles, fn
        assert not np.array_equal(do.download(), base), fn
        flag.set(0)
        st.clear_stop()
        gp.launch(fn, p, st.ctx())
        sync(gp)
        assert np.array_equal(do.download(), base), fn
        assert st.stop_index() == -1


def test_conv2d_fixed_claims_beyond_the_resident_grid(gp):
    """ResNet's 56 x 56 1x1 layer at batch 8 on the 64 x 64 body: 1568 tiles, more than the
    workgroups the GPU holds at once, still a workgroup per claim (gp_launch_info::fixed_claims).
    Claims marked as made are skipped by a relaunch, the others run exactly once, and a first
    launch that is told so (fresh) marks every claim without looking."""
    rng = np.random.default_rng(33)
    N, H, Cin, Cout = 8, 56, 64, 256
    x = rnd(rng, (N, Cin, H, H), "f16")
    w = rnd(rng, (Cout, Cin, 1, 1), "f16", -0.2, 0.2)
    b = rnd(rng, (Cout,), "f16", -0.1, 0.1)
    want, info0, (p, do, keep) = gpu_conv2d(gp, "f16", x, w, b, 1, 0, None, gp.ACT_RELU, tile=64, variant=2)
    raw_want = do.download().copy()
    G = 32
    flag = gp.Flag()
    st = gp.BlpState(1, flag, G)
    do.fill32(0xFFFFFFFF)
    info = gp.launch("gp_launch_conv2d", p, st.ctx(fresh=1))
    sync(gp)
    total = info.total_tiles
    # (eight workgroups in front of the workers own no claim: the first of them reads the flag while claims are being made)
    assert total == 1568 and info.fixed_claims == 1 and info.front == 8 and info.grid == total + info.front
    assert np.array_equal(do.download(), raw_want)
    full = st.counters().reshape(G, 16).copy()
    popcount = lambda a: int(np.unpackbits(np.ascontiguousarray(a).view(np.uint8)).sum())
    assert full[:, 0].sum() == total and popcount(full[:, 1:]) == total
    bits = np.unpackbits(np.ascontiguousarray(full[:, 1:]).view(np.uint8).reshape(G, -1), axis=1)
    keep_mask = (rng.random(bits.shape) < 0.5).astype(np.uint8)
    def relaunch_with(made):
        state = np.zeros_like(full)
        state[:, 1:] = np.packbits(made, axis=1).view(np.int32).reshape(G, 15)
        state[:, 0] = made.sum(axis=1)
        st.executed.upload(state.reshape(-1))
        gp.launch("gp_launch_conv2d", p, st.ctx())
        sync(gp)
        assert np.array_equal(st.counters().reshape(G, 16), full)

    do.fill32(0xFFFFFFFF)
    relaunch_with(bits & keep_mask)          # a random half marked as made: the other half runs
    assert not np.array_equal(do.download(), raw_want)
    relaunch_with(bits & (1 - keep_mask))    # the complement fills in the rest
    assert np.array_equal(do.download(), raw_want)


@pytest.mark.parametrize("dt", ["f16", "f32"])
def test_conv2d_long_tiles_left_mid_k_and_resumed_bit_exact(gp, dt):
    """A deep 3x3 convolution on the 128 x 128 body (K = 9 * Cin): with the checkpoint workspace the
    stop request is honoured between two K-steps, and the resumed result (bias, residual and ReLU
    included) is bit-identical to the uninterrupted one."""
    rng = np.random.default_rng(21)
    N, H, Cin, Cout = 4, 16, 512 if dt == "f16" else 256, 256
    x = rnd(rng, (N, Cin, H, H), dt)
    w = rnd(rng, (Cout, Cin, 3, 3), dt, -0.05, 0.05)
    b = rnd(rng, (Cout,), dt, -0.1, 0.1)
    res = rnd(rng, (N, Cout, H, H), dt)
    want, info0, (p, do, keep) = gpu_conv2d(gp, dt, x, w, b, 1, 1, res, gp.ACT_RELU, tile=128, variant=2)
    ref = O.conv2d(x, w, b, 1, 1, residual=res, act=O.ACT_RELU) if hasattr(O, "ACT_RELU") else None
    if ref is not None:
        assert rel_err(want, O.round_to(ref, dt)) < TOL[dt]
    raw_want = do.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    assert st.enable_checkpoints(p) > 0
    stream = gp.Stream(1)
    tiles = info0.total_tiles
    stopped = 0
    for inject in (0, tiles // 2):
        do.fill32(0)
        st.reset(); st.clear_stop(); flag.set(0)
        gp.check(gp.lib().gp_ckpt_reset_async(gp.vp(st.ckpt.ptr), None))
        info = gp.launch("gp_launch_conv2d", p, st.ctx(kernel_id=0, inject_at=inject), stream)
        stream.sync()
        assert flag.get() == 1
        hdr = st.checkpoint_headers(info.grid)
        if st.stop_index() == 0 and hdr[:, 0].sum() > 0:
            stopped += 1
            live = hdr[hdr[:, 0] == 1]
            assert (live[:, 3] > 0).all() and len(set(live[:, 2].tolist())) == len(live)
            assert not np.array_equal(do.download(), raw_want)
        flag.set(0); st.clear_stop()
        gp.launch("gp_launch_conv2d", p, st.ctx(kernel_id=0), stream)
        stream.sync()
        assert st.stop_index() == -1
        assert int(st.checkpoint_headers(info.grid)[:, 0].sum()) == 0
        assert np.array_equal(do.download(), raw_want), (dt, inject)
    assert stopped >= 1, "the stop request was never seen inside a tile"


@pytest.mark.parametrize("dt", ["f16", "bf16"])
@pytest.mark.parametrize("shape", [(1, 12, 128), (2, 3, 77), (1, 2, 384), (1, 1, 512), (1, 4, 33), (1, 2, 129), (2, 2, 200), (1, 3, 257), (1, 2, 300), (1, 1, 385), (1, 1, 450)])
def test_fused_attention_matches_composed_oracle(gp, dt, shape):
    """softmax(Q K^T / sqrt(d)) V over the heads of a packed QKV buffer, against the oracle's
    batched-matmul / softmax / batched-matmul composition (fp64 softmax on unrounded scores)."""
    B, Hh, S = shape
    d, Hd = 64, Hh * 64
    rng = np.random.default_rng(S * 7 + Hh)
    qkv = rnd(rng, (B * S, 3 * Hd), dt, -1.5, 1.5)
    dtype = gp.DTYPE_BY_NAME[dt]
    es = gp.DTYPE_SIZE[dtype]
    dq = gp.DevBuf.from_array(qkv, dtype)
    do = gp.DevBuf(B * S * Hd * es)
    do.fill32(0x7E007E00)
    p = gp.AttentionParams(dtype=dtype, batch=B, heads=Hh, seq=S, head_dim=d, q=dq.ptr, k=dq.ptr + Hd * es, v=dq.ptr + 2 * Hd * es,
                           ld_qkv=3 * Hd, out=do.ptr, ld_out=Hd, scale=1.0 / np.sqrt(d))
    info = gp.launch("gp_launch_attention", p)
    sync(gp)
    got = do.download(dtype, (B, S, Hh, d))
    x = qkv.astype(np.float64).reshape(B, S, 3, Hh, d)
    q, k, v = x[:, :, 0], x[:, :, 1], x[:, :, 2]
    sc = np.einsum("bihd,bjhd->bhij", q, k) / np.sqrt(d)
    sc -= sc.max(-1, keepdims=True)
    pr = np.exp(sc)
    pr /= pr.sum(-1, keepdims=True)
    ref = np.einsum("bhij,bjhd->bihd", pr, v)
    assert info.total_tiles == -(-S // 64) * B * Hh  # 64 queries per tile, the keys split over two wavefronts
    assert np.isfinite(got).all()
    assert rel_err(got, ref) < TOL[dt], (dt, shape)


def test_fused_attention_preempt_resume_bit_exact(gp):
    B, Hh, S, d = 4, 12, 128, 64
    Hd = Hh * d
    rng = np.random.default_rng(3)
    qkv = rnd(rng, (B * S, 3 * Hd), "f16", -1, 1)
    dq = gp.DevBuf.from_array(qkv, gp.F16)
    do = gp.DevBuf(B * S * Hd * 2)
    p = gp.AttentionParams(dtype=gp.F16, batch=B, heads=Hh, seq=S, head_dim=d, q=dq.ptr, k=dq.ptr + Hd * 2, v=dq.ptr + 2 * Hd * 2,
                           ld_qkv=3 * Hd, out=do.ptr, ld_out=Hd, scale=0.125)
    gp.launch("gp_launch_attention", p)
    sync(gp)
    want = do.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag)
    do.fill32(0)
    gp.launch("gp_launch_attention", p, st.ctx(inject_at=10, max_workgroups=4))
    sync(gp)
    assert flag.get() == 1 and st.stop_index() == 0 and st.counters()[0] < B * Hh
    flag.set(0)
    st.clear_stop()
    gp.launch("gp_launch_attention", p, st.ctx(max_workgroups=4))
    sync(gp)
    assert np.array_equal(do.download(), want)


def test_deep_preemptible_convolution_takes_small_tiles_with_the_same_bits(gp):
    """A preemptible launch finishes the tiles it holds before it leaves: where the rule would run 128 x 128 tiles
    over K >= 2304 (VGG-16's 256 -> 256 layers at 56 x 56), a launch with claim counters takes 64 x 64 tiles,
    and the result has the bits of the plain launch; stopped and resumed, still the same.  A tile chosen by
    the caller is respected."""
    rng = np.random.default_rng(11)
    N, H, Cc = 16, 56, 256
    x = O.round_to(rng.normal(0, 1, (N, Cc, H, H)).astype(np.float32), "f16")
    w = O.round_to((rng.normal(0, 1, (Cc, Cc, 3, 3)) * 0.03).astype(np.float32), "f16")
    bias = O.round_to(rng.normal(0, 0.1, Cc).astype(np.float32), "f16")
    plain, info, (p, do, keep) = gpu_conv2d(gp, "f16", x, w, bias, 1, 1, act=gp.ACT_RELU)
    M = N * H * H
    assert info.total_tiles == (M // 128) * (Cc // 128)
    base = do.download().copy()
    flag = gp.Flag()
    st = gp.BlpState(1, flag, 32)
    do.fill32(0)
    info = gp.launch("gp_launch_conv2d", p, st.ctx(fresh=1))
    sync(gp)
    assert info.total_tiles == (M // 64) * (Cc // 64)
    assert np.array_equal(do.download(), base)
    for frac in (0.2, 0.7):
        st.reset(); st.clear_stop(); flag.set(0)
        do.fill32(0)
        gp.launch("gp_launch_conv2d", p, st.ctx(inject_at=int(frac * info.total_tiles), fresh=1))
        sync(gp)
        assert flag.get() == 1 and not np.array_equal(do.download(), base)
        flag.set(0); st.clear_stop()
        gp.launch("gp_launch_conv2d", p, st.ctx())
        sync(gp)
        assert np.array_equal(do.download(), base), frac
    p.tile_m = p.tile_n = 128
    st.reset(); st.clear_stop()
    info = gp.launch("gp_launch_conv2d", p, st.ctx(fresh=1))
    sync(gp)
    assert info.total_tiles == (M // 128) * (Cc // 128) and np.array_equal(do.download(), base)


def test_launches_report_their_start_and_a_marker_reports_the_end(gp):
    """gp_preempt_ctx::started_host: the first workgroup of every preemptible launch stores the launch's number in
    a word of host memory, in stream order, whichever dispatcher loop the kernel is built around; a
    gp_store_word_async marker behind them says that all of them have left.  (What a host that submits kernel by
    kernel polls instead of events and stream queries.)"""
    import time
    started, left = gp.Flag(), gp.Flag()
    started.set(0); left.set(0)
    flag = gp.Flag()
    st = gp.BlpState(4, flag, 32)
    stream = gp.Stream(1)
    rng = np.random.default_rng(5)
    M, N, K = 512, 512, 256
    A = O.round_to(rng.uniform(-1, 1, (M, K)).astype(np.float32), "f16")
    B = O.round_to(rng.uniform(-1, 1, (N, K)).astype(np.float32), "f16")
    dA, dB, dC = gp.DevBuf.from_array(A, gp.F16), gp.DevBuf.from_array(B, gp.F16), gp.DevBuf(M * N * 2)
    g = gp.GemmParams(dtype=gp.F16, M=M, N=N, K=K, A=dA.ptr, lda=K, B=dB.ptr, ldb=K, b_is_nk=1, C=dC.ptr, ldc=N, alpha=1.0, act=gp.ACT_NONE, batch=1)
    dX, dY = gp.DevBuf.from_array(A[:, :1].repeat(N, 1).copy(), gp.F16), gp.DevBuf(M * N * 2)
    e = gp.EltwiseParams(dtype=gp.F16, rows=M, cols=N, a=dC.ptr, a_stride=N, b=dX.ptr, b_stride=N, scale=None, shift=None, out=dY.ptr, out_stride=N, act=gp.ACT_RELU)
    seen = []
    for seq, (fn, p, kid) in enumerate([("gp_launch_gemm", g, 0), ("gp_launch_eltwise", e, 1), ("gp_launch_gemm", g, 2), ("gp_launch_eltwise", e, 3)], start=1):
        gp.launch(fn, p, st.ctx(kernel_id=kid, fresh=1, started=started, started_seq=seq), stream)
    gp.check(gp.lib().gp_store_word_async(stream.h, gp.vp(left.dev), 77))
    t0 = time.perf_counter()
    while left.get() != 77 and time.perf_counter() - t0 < 5.0:
        seen.append(started.get())
    assert left.get() == 77, "the marker never ran"
    # by the time the marker has run every launch before it has started (and left): the word holds the last number
    assert started.get() == 4
    assert seen == sorted(seen), "launch numbers went backwards"
    stream.sync()
    want = np.maximum(O.gemm_bias_act(A, B, None, None, gp.ACT_NONE, b_is_nk=True) + A[:, :1], 0)
    assert rel_err(dY.download(gp.F16, (M, N)), want) < TOL["f16"]
