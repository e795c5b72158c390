"""Seeded random operators: HIP C ABI vs the CPU oracle, bit-exact for integer
tensors, rel 1e-2 for floating point (the tolerance the path's contract states)."""
import numpy as np
import pytest

import tvx_case as TC

pytestmark = pytest.mark.gpu

FLOAT_RTOL = 1e-2


def rand_q(rng, shape, dtype):
    if dtype == 0:
        return rng.integers(0, 256, shape).astype(np.uint8)
    return rng.integers(-128, 128, shape).astype(np.int8)


def conv_case(rng, *, n, c, h, w, oc, kh, kw, stride, dil, pad, mult, mode, groups=0):
    """mode: 'u8' (per-tensor), 'i8pc' (int8 per-channel), 'u8pc' (u8 act, i8 pc weights), 'f32', 'f16'."""
    icg = 1 if mult > 0 else c // max(groups, 1)
    if mult > 0:
        oc = c * mult
    out_w = (w + pad[0] + pad[1] - ((kw - 1) * dil[0] + 1)) // stride[0] + 1
    out_h = (h + pad[2] + pad[3] - ((kh - 1) * dil[1] + 1)) // stride[1] + 1
    kws = dict(in_shape=[w, h, c, n], w_shape=[kw, kh, icg, oc], out_shape=[out_w, out_h, oc, n],
               stride=stride, dilation=dil, pad_left=pad[0], pad_top=pad[2], multiplier=mult)
    if groups:
        kws["groups"] = groups
    if mode in ("f32", "f16"):
        npd = np.float32 if mode == "f32" else np.float16
        dt = 3 if mode == "f32" else 2
        x = rng.standard_normal(n * c * h * w).astype(npd)
        wt = (rng.standard_normal(oc * icg * kh * kw) * 0.2).astype(npd)
        b = rng.standard_normal(oc).astype(np.float32)
        kws.update(in_dtype=dt, w_dtype=dt, out_dtype=dt)
        return x, wt, b, kws
    in_dt = 0 if mode.startswith("u8") else 1
    w_dt = 0 if mode == "u8" else 1
    x = rand_q(rng, n * c * h * w, in_dt)
    wt = rand_q(rng, oc * icg * kh * kw, w_dt)
    b = rng.integers(-4096, 4097, oc).astype(np.int32)
    zx = 128 if in_dt == 0 else int(rng.integers(-10, 10))
    kmacs = icg * kh * kw
    s_out = float(np.float32(0.05 * 0.01 * 40 * np.sqrt(kmacs)))
    if mode == "u8":
        wq = (0.01, 120, None)
    else:
        wq = (1.0, 0, np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32))
    kws.update(in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt, in_q=(0.05, zx), w_q=wq,
               out_q=(s_out, 3 if in_dt == 0 else -3))
    return x, wt, b, kws


CONV_GRID = [
    dict(n=2, c=8, h=9, w=11, oc=6, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 1, 1], mult=0),
    dict(n=1, c=3, h=17, w=15, oc=16, kh=3, kw=3, stride=[2, 2], dil=[1, 1], pad=[0, 1, 0, 1], mult=0),
    dict(n=3, c=16, h=7, w=7, oc=32, kh=1, kw=1, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0),
    dict(n=2, c=5, h=12, w=10, oc=4, kh=5, kw=3, stride=[1, 2], dil=[2, 1], pad=[2, 2, 3, 3], mult=0),
    dict(n=2, c=6, h=10, w=10, oc=0, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 1, 1], mult=1),
    dict(n=1, c=4, h=9, w=13, oc=0, kh=3, kw=3, stride=[2, 2], dil=[1, 1], pad=[1, 1, 1, 1], mult=2),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc", "f32", "f16"])
@pytest.mark.parametrize("gi", range(len(CONV_GRID)))
@pytest.mark.parametrize("act", [0, 2])
def test_conv2d_random(oracle, gi, mode, act):
    rng = np.random.default_rng(1000 + gi * 10 + act)
    x, w, b, kws = conv_case(rng, mode=mode, **CONV_GRID[gi])
    want = oracle.conv2d(x, w, b, act=act, **kws)
    got = TC.gpu_conv2d(x, w, b, act=act, **kws)
    if mode in ("f32", "f16"):
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=2e-2)
    else:
        assert np.array_equal(got, want)
        assert len(np.unique(want)) > 4  # the case exercises more than saturation


def test_conv2d_without_bias_and_runtime_weights(oracle):
    rng = np.random.default_rng(5)
    x, w, b, kws = conv_case(rng, mode="u8", **CONV_GRID[0])
    want = oracle.conv2d(x, w, None, **kws)
    assert np.array_equal(TC.gpu_conv2d(x, w, None, **kws), want)
    assert np.array_equal(TC.gpu_conv2d(x, w, None, const_weights=False, **kws), want)


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc", "f32", "f16"])
@pytest.mark.parametrize("shape", [(5, 37, 11), (64, 256, 48), (1, 800, 500), (33, 130, 70), (7, 500, 10), (3, 1283, 200)])
def test_fully_connected_random(oracle, mode, shape):
    m, k, n = shape
    rng = np.random.default_rng(m * 7 + k)
    if mode in ("f32", "f16"):
        npd, dt = (np.float32, 3) if mode == "f32" else (np.float16, 2)
        x = rng.standard_normal(m * k).astype(npd)
        w = (rng.standard_normal(n * k) * 0.02).astype(npd)
        b = rng.standard_normal(n).astype(np.float32)
        kws = dict(m=m, k=k, n=n, in_dtype=dt, w_dtype=dt, out_dtype=dt)
        want = oracle.fully_connected(x, w, b, **kws)
        got = TC.gpu_fully_connected(x, w, b, **kws)
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=2e-2)
        return
    in_dt = 0 if mode.startswith("u8") else 1
    w_dt = 0 if mode == "u8" else 1
    x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    wq = (0.01, 120, None) if mode == "u8" else \
        (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
    kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
               in_q=(0.02, 128 if in_dt == 0 else 0), w_q=wq,
               out_q=(float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else 0))
    for act in (0, 1):
        want = oracle.fully_connected(x, w, b, act=act, **kws)
        got = TC.gpu_fully_connected(x, w, b, act=act, **kws)
        assert np.array_equal(got, want)
    assert len(np.unique(want)) > 4


POOLS = [
    dict(in_shape=[24, 24, 20, 3], ksize=[2, 2], stride=[2, 2], pad=[0, 0, 0, 0]),
    dict(in_shape=[7, 7, 64, 2], ksize=[7, 7], stride=[7, 7], pad=[0, 0, 0, 0]),
    dict(in_shape=[13, 9, 5, 2], ksize=[3, 3], stride=[2, 2], pad=[1, 1, 0, 1]),
    dict(in_shape=[10, 10, 3, 1], ksize=[3, 2], stride=[1, 3], pad=[1, 0, 1, 1]),
]


@pytest.mark.parametrize("dtype", [0, 1, 2, 3])
@pytest.mark.parametrize("ptype", [0, 1, 2, 3])   # MAX, AVG, L2, AVG_ANDROID
@pytest.mark.parametrize("pi", range(len(POOLS)))
def test_pool2d_random(oracle, pi, ptype, dtype):
    p = POOLS[pi]
    rng = np.random.default_rng(pi * 100 + ptype * 10 + dtype)
    w, h, c, n = p["in_shape"]
    out_w = (w + p["pad"][0] + p["pad"][1] - p["ksize"][0]) // p["stride"][0] + 1
    out_h = (h + p["pad"][2] + p["pad"][3] - p["ksize"][1]) // p["stride"][1] + 1
    kws = dict(in_shape=p["in_shape"], out_shape=[out_w, out_h, c, n], ksize=p["ksize"],
               stride=p["stride"], pad_left=p["pad"][0], pad_top=p["pad"][2], pool_type=ptype, dtype=dtype)
    if dtype < 2:
        x = rand_q(rng, w * h * c * n, dtype)
        for in_q, out_q in (((0.1, 7), (0.1, 7)), ((0.1, 7), (0.07, -2 if dtype else 9))):
            want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
            got = TC.gpu_pool2d(x, in_q=in_q, out_q=out_q, **kws)
            assert np.array_equal(got, want)
    else:
        x = rng.standard_normal(w * h * c * n).astype(np.float32 if dtype == 3 else np.float16)
        want = oracle.pool2d(x, **kws)
        got = TC.gpu_pool2d(x, **kws)
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=1e-3)


POOL_ROWS = [
    # in_shape {W, H, C, N}, ksize, stride, pad {l, r, t, b}: windows two or three taps wide (pool2d_rows_i8)
    dict(in_shape=[24, 24, 20, 5], ksize=[2, 2], stride=[2, 2], pad=[0, 0, 0, 0]),      # LeNet: several planes per workgroup
    dict(in_shape=[8, 8, 50, 3], ksize=[2, 2], stride=[2, 2], pad=[0, 0, 0, 0]),
    dict(in_shape=[112, 112, 8, 2], ksize=[3, 3], stride=[2, 2], pad=[0, 1, 0, 1]),    # SAME at stride 2: right / bottom padding
    dict(in_shape=[112, 112, 6, 1], ksize=[3, 3], stride=[2, 2], pad=[1, 1, 1, 1]),
    dict(in_shape=[13, 9, 5, 2], ksize=[3, 3], stride=[2, 2], pad=[1, 1, 0, 1]),        # odd widths: planes that do not start on a dword
    dict(in_shape=[10, 10, 3, 1], ksize=[3, 2], stride=[1, 3], pad=[1, 0, 1, 1]),
    dict(in_shape=[15, 7, 9, 3], ksize=[2, 5], stride=[1, 2], pad=[1, 1, 2, 2]),        # tall window, output width not a multiple of 4
    dict(in_shape=[230, 190, 2, 2], ksize=[3, 3], stride=[2, 2], pad=[1, 1, 1, 1]),     # planes in several row bands
    dict(in_shape=[301, 77, 3, 1], ksize=[2, 2], stride=[1, 1], pad=[0, 1, 0, 1]),
    dict(in_shape=[5, 4, 70, 4], ksize=[3, 3], stride=[1, 1], pad=[2, 2, 2, 2]),        # more padding than image in places
    dict(in_shape=[3, 3, 5, 2], ksize=[2, 2], stride=[2, 2], pad=[1, 1, 1, 1]),
]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("ptype", [0, 1, 3])
@pytest.mark.parametrize("pi", range(len(POOL_ROWS)))
def test_pool2d_rows(oracle, pi, ptype, dtype, monkeypatch):
    monkeypatch.setenv("TVX_POOL_STENCIL", "0")   # (the register stencil would take the stride-2 MAX shapes of this grid)
    p = POOL_ROWS[pi]
    rng = np.random.default_rng(600 + pi * 10 + ptype)
    w, h, c, n = p["in_shape"]
    out_w = (w + p["pad"][0] + p["pad"][1] - p["ksize"][0]) // p["stride"][0] + 1
    out_h = (h + p["pad"][2] + p["pad"][3] - p["ksize"][1]) // p["stride"][1] + 1
    kws = dict(in_shape=p["in_shape"], out_shape=[out_w, out_h, c, n], ksize=p["ksize"],
               stride=p["stride"], pad_left=p["pad"][0], pad_top=p["pad"][2], pool_type=ptype, dtype=dtype)
    x = rand_q(rng, w * h * c * n, dtype)
    zi = 7 if dtype else 120
    for in_q, out_q in (((0.1, zi), (0.1, zi)), ((0.1, zi), (0.07, -2 if dtype else 9)), ((0.5, zi), (0.25, zi))):
        want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
        got = TC.gpu_pool2d(x, in_q=in_q, out_q=out_q, want_kernel="pool2d_rows_i8", **kws)
        assert np.array_equal(got, want), (int((got != want).sum()), np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("band_kb", ["8", "33", "60"])
def test_pool2d_rows_band_budgets(oracle, band_kb, monkeypatch):
    """LDS budgets below and above what two images of the pipelined form may take (64 KiB together): where the
    pipelined plan falls through, the plain plan's grid and LDS size must be the ones launched - every plane of
    1024 plane groups written."""
    monkeypatch.setenv("TVX_POOL_BAND_KB", band_kb)
    monkeypatch.setenv("TVX_POOL_STENCIL", "0")
    rng = np.random.default_rng(650)
    w, h, c, n = 24, 24, 64, 40   # 2560 planes: enough plane groups for the pipelined form at every budget
    x = rng.integers(0, 256, w * h * c * n, dtype=np.uint8)
    kws = dict(in_shape=[w, h, c, n], out_shape=[12, 12, c, n], ksize=[2, 2], stride=[2, 2], pad_left=0, pad_top=0,
               pool_type=0, dtype=0, in_q=(0.1, 120), out_q=(0.1, 120))
    want = oracle.pool2d(x, **kws)
    got = TC.gpu_pool2d(x, want_kernel="pool2d_rows_i8", **kws)
    assert np.array_equal(got, want), int((got != want).sum())


def test_pool2d_full_size_max_3x3_stride2(oracle, monkeypatch):
    """3x3 stride 2 MAX on 112x112x64 at batch 32 (25.7 MB in, 6.4 MB out): whole output against the oracle."""
    rng = np.random.default_rng(0x74)
    w, h, c, n = 112, 112, 64, 32
    x = rng.integers(0, 256, w * h * c * n, dtype=np.uint8)
    kws = dict(in_shape=[w, h, c, n], out_shape=[56, 56, c, n], ksize=[3, 3], stride=[2, 2], pad_left=0, pad_top=0,
               pool_type=0, dtype=0, in_q=(0.05, 3), out_q=(0.05, 3))
    want = oracle.pool2d(x, **kws)
    got = TC.gpu_pool2d(x, want_kernel="pool2d_stencil_i8", **kws)
    assert np.array_equal(got, want)
    monkeypatch.setenv("TVX_POOL_STENCIL", "0")
    got = TC.gpu_pool2d(x, want_kernel="pool2d_rows_i8", **kws)
    assert np.array_equal(got, want)


POOL_STENCIL = [
    # in_shape {W, H, C, N}, ksize, pad {l, r, t, b}: MAX pooling at stride 2 on rows of whole 8-byte units (pool2d_stencil_i8)
    dict(in_shape=[112, 112, 6, 2], ksize=[3, 3], pad=[0, 1, 0, 1]),     # SAME at stride 2: the padding column and row behind
    dict(in_shape=[112, 112, 5, 1], ksize=[3, 3], pad=[1, 1, 1, 1]),     # ... in front: the left neighbour's last column
    dict(in_shape=[24, 24, 20, 5], ksize=[2, 2], pad=[0, 0, 0, 0]),      # LeNet
    dict(in_shape=[8, 8, 50, 3], ksize=[2, 2], pad=[0, 0, 0, 0]),        # one lane per row
    dict(in_shape=[56, 31, 7, 2], ksize=[3, 2], pad=[1, 0, 0, 0]),       # seven lanes per row (eight with the idle one), an odd height
    dict(in_shape=[40, 13, 3, 3], ksize=[2, 3], pad=[1, 0, 1, 1]),       # two taps across with left padding, three down
    dict(in_shape=[64, 9, 4, 2], ksize=[3, 3], pad=[0, 1, 1, 0]),        # row groups that end inside a thread's four rows
    dict(in_shape=[512, 6, 2, 1], ksize=[3, 3], pad=[1, 0, 1, 0]),       # the widest row: a wavefront per image row
    dict(in_shape=[16, 1100, 3, 1], ksize=[2, 2], pad=[0, 0, 1, 0]),     # tall planes: several workgroups per plane
    dict(in_shape=[112, 112, 4, 2], ksize=[3, 3], pad=[0, 0, 0, 0]),     # VALID: 55 x 55, rows that end inside a lane's four outputs
    dict(in_shape=[48, 20, 5, 2], ksize=[3, 2], pad=[0, 0, 1, 0]),       # 23 columns
    dict(in_shape=[32, 11, 3, 2], ksize=[2, 2], pad=[0, 0, 0, 0], out_w=13),  # a declared output narrower than the input allows
]


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("pi", range(len(POOL_STENCIL)))
def test_pool2d_stencil(oracle, pi, dtype):
    """The register-stencil MAX pooling against the oracle, with equal quantization on both sides (the maximum is the
    result), with a moved zero point and with a rescale (the generic requantization of the maximum)."""
    p = POOL_STENCIL[pi]
    rng = np.random.default_rng(900 + pi * 10 + dtype)
    w, h, c, n = p["in_shape"]
    out_w = p.get("out_w", (w + p["pad"][0] + p["pad"][1] - p["ksize"][0]) // 2 + 1)
    out_h = (h + p["pad"][2] + p["pad"][3] - p["ksize"][1]) // 2 + 1
    assert out_w <= w // 2
    kws = dict(in_shape=p["in_shape"], out_shape=[out_w, out_h, c, n], ksize=p["ksize"], stride=[2, 2],
               pad_left=p["pad"][0], pad_top=p["pad"][2], pool_type=0, dtype=dtype)
    x = rand_q(rng, w * h * c * n, dtype)
    # (low codes everywhere but in a few places: a padding tap that took part would show)
    x = np.where(rng.random(x.size) < 0.7, x.min(), x).astype(x.dtype)
    zi = 7 if dtype else 120
    import torch
    for in_q, out_q in (((0.1, zi), (0.1, zi)), ((0.1, zi), (0.1, zi + 5)), ((0.5, zi), (0.25, zi))):
        want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
        T = TC.tvx()
        d = T.Pool2dDesc()
        d.in_w, d.in_h, d.channels, d.batch = p["in_shape"]
        d.out_w, d.out_h = out_w, out_h
        d.k_w, d.k_h = p["ksize"]
        d.stride_w = d.stride_h = 2
        d.pad_left, d.pad_top, d.pool_type, d.dtype = p["pad"][0], p["pad"][2], 0, dtype
        d.in_scale, d.in_zp = in_q
        d.out_scale, d.out_zp = out_q
        op = T.pool2d_create(d)
        assert op.kernel_name == "pool2d_stencil_i8", op.kernel_name
        xd = TC.to_device(x)
        yd = TC.device_out(want.size + 32, TC.NP_OF[dtype])
        yd.fill_(99)
        op.run(xd, None, yd)
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        op.close()
        assert np.array_equal(got[:want.size], want), (int((got[:want.size] != want).sum()), np.flatnonzero(got[:want.size] != want)[:8])
        assert np.all(got[want.size:] == 99), "wrote past the tensor"
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("shape", [(7, 7, 1280, 3), (2, 2, 5, 1), (5, 3, 9, 2), (17, 19, 6, 2), (33, 31, 3, 1)], ids=str)
@pytest.mark.parametrize("ptype", [1, 3])
@pytest.mark.parametrize("dtype", [0, 1])
def test_global_average_pool(oracle, shape, ptype, dtype):
    """Quantized average over the whole plane: its own kernel (4, 16 or 64 lanes per plane, planes that do
    not end on a dword), the oracle's arithmetic."""
    w, h, c, n = shape
    rng = np.random.default_rng(w * 100 + h + dtype)
    x = rand_q(rng, w * h * c * n, dtype)
    kws = dict(in_shape=list(shape), out_shape=[1, 1, c, n], ksize=[w, h], stride=[1, 1], pad_left=0, pad_top=0,
               pool_type=ptype, dtype=dtype)
    zp = 7 if dtype else 120  # near the mean of the data, so that the finer output scale does not saturate
    for in_q, out_q in (((0.1, zp), (0.1, zp)), ((0.1, zp), (0.013, -2 if dtype else 9))):
        want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
        got = TC.gpu_pool2d(x, in_q=in_q, out_q=out_q, want_kernel="avgpool_plane_i8", **kws)
        assert np.array_equal(got, want)
        assert out_q[0] != in_q[0] or len(np.unique(want)) > 2


@pytest.mark.parametrize("dtype", [0, 1])
def test_eltwise_quantized(oracle, dtype):
    rng = np.random.default_rng(dtype)
    a, b = rand_q(rng, 100003, dtype), rand_q(rng, 100003, dtype)
    za, zb, zo = (120, 110, 128) if dtype == 0 else (3, -4, 5)
    for act in (1, 2):
        for out_q in ((0.05, za), (0.031, zo)):
            want = oracle.activation(act, dtype, a, (0.05, za), out_q)
            assert np.array_equal(TC.gpu_activation(act, dtype, a, (0.05, za), out_q), want)
    want = oracle.add(dtype, a, (0.03, za), b, (0.05, zb), (0.07, zo))
    assert np.array_equal(TC.gpu_add(dtype, a, (0.03, za), b, (0.05, zb), (0.07, zo)), want)
    sm_want = oracle.softmax(dtype, a[:100000], 10, 1.0, (0.1, za))
    sm_got = TC.gpu_softmax(dtype, a[:100000], 10, 1.0, (0.1, za))
    assert np.allclose(sm_got, sm_want, rtol=1e-4, atol=1e-7)


@pytest.mark.parametrize("c", [1, 3, 4, 5, 16, 17, 64, 65, 1000, 1001, 1024, 1025, 3000])
def test_softmax_group_sizes(oracle, c):
    # every lanes-per-group choice of the register-resident kernel, its upper limit and the strided
    # kernel past it; a row count that leaves the last wavefront partly empty
    rng = np.random.default_rng(c)
    rows = 37
    x = rand_q(rng, rows * c, 0)
    want = oracle.softmax(0, x, c, 0.7, (0.05, 131))
    got = TC.gpu_softmax(0, x, c, 0.7, (0.05, 131))
    assert np.allclose(got, want, rtol=1e-4, atol=1e-9)
    assert np.allclose(got.reshape(rows, c).sum(axis=1), 1.0, atol=1e-5)
    f = (rng.standard_normal(rows * c) * 3).astype(np.float32)
    for beta in (1.0, -0.5):
        want = oracle.softmax(3, f, c, beta, (1.0, 0))
        assert np.allclose(TC.gpu_softmax(3, f, c, beta, (1.0, 0)), want, rtol=1e-4, atol=1e-9)


def test_eltwise_float(oracle):
    rng = np.random.default_rng(3)
    a = (rng.standard_normal(5000) * 4).astype(np.float32)
    b = rng.standard_normal(5000).astype(np.float32)
    assert np.array_equal(TC.gpu_activation(2, 3, a, (1.0, 0), (1.0, 0)), np.clip(a, 0, 6))
    assert np.array_equal(TC.gpu_add(3, a, (1.0, 0), b, (1.0, 0), (1.0, 0)), a + b)
    h = a.astype(np.float16)
    assert np.array_equal(TC.gpu_activation(1, 2, h, (1.0, 0), (1.0, 0)), np.maximum(h, 0))


FC_EDGE_SHAPES = [
    # 256 x 256 tiles: M, N not multiples of the tile, K not of the 128-byte step
    ((600, 512, 528), "fc_mfma_i8_256x256x128"), ((513, 144, 769), "fc_mfma_i8_256x256x128"),
    # few outputs -> 16 x 16 tiles with the reduction split over four wavefronts: ragged M / N, N not a
    # multiple of 4 (byte stores), K with a 16 / 32 / 48-byte tail and shorter than one 64-byte step,
    # more k-steps than one batch of loads, the MobileNetV2 and LeNet classifier shapes
    ((300, 512, 272), "fc_mfma_i8_16x16_splitk"), ((257, 144, 513), "fc_mfma_i8_16x16_splitk"),
    ((12, 1280, 1000), "fc_mfma_i8_16x16_splitk"), ((64, 1280, 1000), "fc_mfma_i8_16x16_splitk"),
    ((256, 800, 500), "fc_mfma_i8_16x16_splitk"), ((17, 48, 1001), "fc_mfma_i8_16x16_splitk"),
    ((1000, 16, 9), "fc_mfma_i8_16x16_splitk"), ((33, 4112, 250), "fc_mfma_i8_16x16_splitk"),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("shape,kernel", FC_EDGE_SHAPES)
def test_fully_connected_mfma_edges(oracle, mode, shape, kernel):
    """Tile and reduction edges of the two MFMA variants."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n)
    in_dt = 0 if mode.startswith("u8") else 1
    w_dt = 0 if mode == "u8" else 1
    x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    wq = (0.01, 117, None) if mode == "u8" else \
        (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
    kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
               in_q=(0.02, 131 if in_dt == 0 else -2), w_q=wq,
               out_q=(float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else 0))
    for act in (0, 2):
        want = oracle.fully_connected(x, w, b, act=act, **kws)
        got = TC.gpu_fully_connected(x, w, b, act=act, want_kernel=kernel, **kws)
        assert np.array_equal(got, want), int((got != want).sum())
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("mode", ["i8pc", "u8", "u8pc", "i8zp"])
@pytest.mark.parametrize("shape", [(600, 512, 528), (513, 144, 769), (1025, 16, 300), (130, 336, 2050), (385, 1040, 700)])
def test_fully_connected_128_row_tiles(oracle, shape, mode, monkeypatch):
    """The 128 x 256 tile form of the quantized kernel (its own choice from 1024 tiles up) on small ragged shapes: M, N
    not multiples of the tile, reductions of one 16-byte chunk, with a tail, of an odd and an even count of k-tiles
    (its weight slots come in pairs); int8 and uint8 activations, per-channel weights and a uniform weight zero point
    (re-bias and row sums one piece at a time). The same shapes on 256-row tiles give the same bytes."""
    m, k, n = shape
    rng = np.random.default_rng(m * 7 + k + n)
    in_dt = 0 if mode.startswith("u8") else 1
    w_dt = 0 if mode == "u8" else 1
    x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    if mode == "u8":
        wq = (0.01, 117, None)
    elif mode == "i8zp":
        wq = (0.01, -9, None)
    else:
        wq = (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
    kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt, in_q=(0.02, 131 if in_dt == 0 else -2), w_q=wq,
               out_q=(float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else 3))
    for act in (0, 1, 2):
        want = oracle.fully_connected(x, w, b, act=act, **kws)
        monkeypatch.setenv("TVX_FC_TILE_M", "128")
        got = TC.gpu_fully_connected(x, w, b, act=act, want_kernel="fc_mfma_i8_128x256x128", **kws)
        assert np.array_equal(got, want), (mode, act, int((got != want).sum()))
        monkeypatch.setenv("TVX_FC_TILE_M", "256")
        assert np.array_equal(TC.gpu_fully_connected(x, w, b, act=act, want_kernel="fc_mfma_i8_256x256x128", **kws), want)
    assert len(np.unique(want)) > 4


def test_fully_connected_full_size_uint8_asymmetric(oracle):
    """M=8192, K=4096, N=4096 uint8 with a uniform weight zero point: the variant whose activations are re-biased
    and summed per row inside the kernel, one k-tile ahead of the multiplications, over all 32 k-tiles, on 128-row
    tiles (two workgroups per CU). A seeded sample of rows against the oracle, every one of the 64 tile rows covered."""
    m, k, n = 8192, 4096, 4096
    rng = np.random.default_rng(0x76)
    x = rng.integers(0, 256, m * k, dtype=np.uint8)
    w = rng.integers(0, 256, n * k, dtype=np.uint8)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    kws = dict(k=k, n=n, in_dtype=0, w_dtype=0, out_dtype=0, in_q=(0.02, 121), w_q=(0.01, 131, None),
               out_q=(1.2, 128))
    got = TC.gpu_fully_connected(x, w, b, m=m, want_kernel="fc_mfma_i8_128x256x128", **kws).reshape(m, n)
    rows = np.sort(np.concatenate([np.arange(64) * 128 + rng.integers(0, 128, 64), rng.choice(m, 8, replace=False)]))
    want = oracle.fully_connected(np.ascontiguousarray(x.reshape(m, k)[rows]).ravel(), w, b, m=len(rows), **kws)
    assert np.array_equal(got[rows], want.reshape(len(rows), n))
    assert len(np.unique(got)) > 100


def test_fully_connected_full_size_int8_per_channel(oracle):
    """M=8192, K=4096, N=4096 int8 per-channel (128 x 256 tiles, two workgroups per CU): the whole problem on the
    GPU, a seeded sample of rows recomputed by the oracle - one in every one of the 64 tile rows (all output
    columns: every tile of the launch is touched) and 8 anywhere -, plus independence of the rows."""
    m, k, n = 8192, 4096, 4096
    rng = np.random.default_rng(0x75)
    x = rng.integers(-128, 128, m * k, dtype=np.int8)
    w = rng.integers(-128, 128, n * k, dtype=np.int8)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    ws = np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32)
    kws = dict(k=k, n=n, in_dtype=1, w_dtype=1, out_dtype=1, in_q=(0.02, 0), w_q=(1.0, 0, ws),
               out_q=(0.05, 0))
    got = TC.gpu_fully_connected(x, w, b, m=m, want_kernel="fc_mfma_i8_128x256x128", **kws).reshape(m, n)
    rows = np.unique(np.concatenate([np.arange(64) * 128 + rng.integers(0, 128, 64), rng.choice(m, 8, replace=False)]))
    assert set(rows // 128) == set(range(64))
    want = oracle.fully_connected(np.ascontiguousarray(x.reshape(m, k)[rows]).ravel(), w, b, m=len(rows), **kws)
    assert np.array_equal(got[rows], want.reshape(len(rows), n))
    assert len(np.unique(got)) > 100
    # rows are independent: permuting input rows permutes output rows
    perm = rng.permutation(m)
    got_p = TC.gpu_fully_connected(np.ascontiguousarray(x.reshape(m, k)[perm]).ravel(), w, b, m=m, **kws)
    assert np.array_equal(got_p.reshape(m, n), got[perm])


@pytest.mark.parametrize("shape", [(300, 200, 260), (256, 64, 256), (1, 8, 3), (517, 1032, 40)])
@pytest.mark.parametrize("act", [0, 1, 2])
def test_fully_connected_float16_mfma_edges(oracle, shape, act):
    """float16 FC on the matrix cores: ragged M / N tiles, K tails (K % 64 != 0), fused
    ReLU / ReLU6. fp32 accumulation on both sides; tolerance 1e-2 relative."""
    m, k, n = shape
    rng = np.random.default_rng(m + k + n)
    x = rng.standard_normal(m * k).astype(np.float16)
    w = (rng.standard_normal(n * k) * 0.05).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float32)
    kws = dict(m=m, k=k, n=n, in_dtype=2, w_dtype=2, out_dtype=2)
    want = oracle.fully_connected(x, w, b, act=act, **kws)
    got = TC.gpu_fully_connected(x, w, b, act=act, want_kernel="fc_mfma_f16_256x256x64", **kws)
    assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-2)
    if act == 2:
        assert got.max() <= 6.0 and got.min() >= 0.0


def test_fully_connected_full_size_float16(oracle):
    """M=8192, K=4096, N=4096 float16 (inputs N(0,1), weights N(0,0.02)): the whole problem on
    the GPU, a seeded sample of 32 rows recomputed by the oracle in fp32, within 1e-2."""
    m, k, n = 8192, 4096, 4096
    rng = np.random.default_rng(0x76)
    x = rng.standard_normal(m * k, dtype=np.float32).astype(np.float16)
    w = (rng.standard_normal(n * k, dtype=np.float32) * 0.02).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float32)
    kws = dict(k=k, n=n, in_dtype=2, w_dtype=2, out_dtype=2)
    got = TC.gpu_fully_connected(x, w, b, m=m, want_kernel="fc_mfma_f16_256x256x64", **kws).reshape(m, n)
    rows = np.sort(rng.choice(m, 32, replace=False))
    want = oracle.fully_connected(np.ascontiguousarray(x.reshape(m, k)[rows]).ravel(), w, b, m=len(rows), **kws)
    want = want.reshape(len(rows), n).astype(np.float32)
    assert np.allclose(got[rows].astype(np.float32), want, rtol=1e-2, atol=1e-2)
    assert np.isfinite(got.astype(np.float32)).all()


def test_conv2d_cfg2_full_size(oracle):
    """uint8 3x3 64->64 on 56x56x64 at batch 32, SAME, fused ReLU6: whole output vs the oracle."""
    rng = np.random.default_rng(0x72)
    n, c, h, w, oc = 32, 64, 56, 56, 64
    x = rng.integers(0, 256, n * c * h * w, dtype=np.uint8)
    wt = rng.integers(0, 256, oc * c * 9, dtype=np.uint8)
    b = rng.integers(-4096, 4097, oc).astype(np.int32)
    kws = dict(in_shape=[w, h, c, n], w_shape=[3, 3, c, oc], out_shape=[w, h, oc, n], stride=[1, 1],
               dilation=[1, 1], pad_left=1, pad_top=1, multiplier=0, in_dtype=0, w_dtype=0, out_dtype=0,
               in_q=(0.05, 128), w_q=(0.01, 120, None), out_q=(0.1, 0), act=2)
    want = oracle.conv2d(x, wt, b, **kws)
    got = TC.gpu_conv2d(x, wt, b, want_kernel="conv2d_band_i8", **kws)
    assert np.array_equal(got, want)
    assert got.max() == 60 and len(np.unique(got)) == 61  # ReLU6 at scale 0.1: q in [0, 60]


IGEMM_KERNELS = ("conv2d_igemm_i8", "conv2d_igemm_i8_persistent", "conv2d_band_i8")

IGEMM_GRID = [
    # (n, c, h, w, oc, kh, kw, stride, dil, pad[l,r,t,b])
    (2, 32, 28, 28, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (1, 12, 32, 32, 32, 3, 3, [2, 2], [1, 1], [0, 1, 0, 1]),   # channels padded to 16 (C = 3 would be im2col's)
    (2, 16, 14, 14, 96, 1, 1, [1, 1], [1, 1], [0, 0, 0, 0]),
    (1, 64, 9, 7, 40, 3, 3, [1, 1], [2, 2], [2, 2, 2, 2]),
    (1, 20, 8, 8, 50, 5, 5, [1, 1], [1, 1], [0, 0, 0, 0]),
    (3, 64, 7, 7, 160, 3, 3, [2, 1], [1, 1], [1, 1, 1, 1]),
    (1, 24, 13, 20, 144, 1, 1, [1, 1], [1, 1], [0, 0, 0, 0]),
    # weights + halo beyond one LDS load: the reduction runs in channel groups
    (1, 128, 14, 14, 160, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (2, 256, 7, 7, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (1, 200, 9, 9, 40, 3, 3, [2, 2], [1, 1], [1, 1, 1, 1]),
    (1, 96, 10, 12, 256, 5, 5, [1, 1], [1, 1], [2, 2, 2, 2]),
    (1, 528, 6, 6, 32, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(IGEMM_GRID)))
def test_conv2d_igemm_shapes(oracle, gi, mode):
    n, c, h, w, oc, kh, kw, stride, dil, pad = IGEMM_GRID[gi]
    rng = np.random.default_rng(2000 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=stride, dil=dil,
                              pad=pad, mult=0, mode=mode)
    want = oracle.conv2d(x, wt, b, act=1, **kws)
    pointwise = kh == 1 and kw == 1 and stride == [1, 1] and pad == [0, 0, 0, 0]
    got = TC.gpu_conv2d(x, wt, b, act=1, want_kernel="pwconv_i8" if pointwise else IGEMM_KERNELS, **kws)
    assert np.array_equal(got, want)
    assert len(np.unique(want)) > 4


PERSIST_GRID = [
    # (n, c, h, w, oc, kh, kw, stride, dil, pad[l,r,t,b]): shapes of the persistent variant (weights in registers:
    # 32 or 64 input channels under a 3x3 kernel, 33..64 output channels, width a multiple of 4)
    (5, 64, 56, 56, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (3, 32, 28, 28, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (4, 64, 20, 24, 40, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),     # 40 output channels: the second channel tile is ragged
    (3, 32, 17, 40, 33, 3, 3, [2, 2], [1, 1], [0, 1, 0, 1]),     # stride 2: five halo rows for two output rows
    (2, 64, 14, 20, 64, 3, 3, [1, 1], [1, 1], [0, 0, 0, 0]),     # VALID: no padding columns, 18-pixel rows
    (2, 64, 12, 12, 48, 3, 3, [1, 1], [2, 2], [2, 2, 2, 2]),     # dilation 2: five halo rows per output row
    (9, 64, 8, 8, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),       # whole images smaller than one tile
    (2, 32, 9, 64, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),      # 64 columns: the widest single patch row
]


@pytest.mark.parametrize("knobs", [{}, {"TVX_IGEMM_WGS": "8"}, {"TVX_IGEMM_WGS": "16", "TVX_IGEMM_TILE_ROWS": "2"},
                                   {"TVX_IGEMM_WGS": "8", "TVX_IGEMM_TILE_ROWS": "1"}], ids=lambda k: "-".join(k.values()) or "default")
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(PERSIST_GRID)))
def test_conv2d_igemm_persistent(oracle, gi, mode, knobs, monkeypatch):
    """The persistent variant with its default launch and with few workgroups / small tiles forced, so that
    every workgroup walks many tiles through both halo buffers (tiles of one, two and more output rows)."""
    n, c, h, w, oc, kh, kw, stride, dil, pad = PERSIST_GRID[gi]
    monkeypatch.setenv("TVX_IGEMM_PERSIST", "1")   # also where the heuristic would take the one-tile-per-workgroup kernel
    monkeypatch.setenv("TVX_CONV_BAND", "0")       # (the kernel that is asked first)
    for k, v in knobs.items():
        monkeypatch.setenv(k, v)
    rng = np.random.default_rng(2500 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=stride, dil=dil,
                              pad=pad, mult=0, mode=mode)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="conv2d_igemm_i8_persistent", **kws)
        assert np.array_equal(got, want), (int((got != want).sum()), np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 4


BAND_GRID = [
    # (n, c, h, w, oc, kh, kw, stride, dil, pad[l,r,t,b]): shapes of the one-workgroup-per-CU kernel (weights in LDS:
    # 32 or 64 input channels under a 3x3 kernel, 33..64 output channels, input and output rows of whole 8-byte units)
    (5, 64, 56, 56, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (3, 32, 28, 24, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (4, 64, 20, 24, 40, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),     # 40 output channels: the second channel tile is ragged
    (3, 32, 17, 32, 33, 3, 3, [2, 2], [1, 1], [0, 1, 0, 1]),     # stride 2
    (2, 64, 16, 16, 48, 3, 3, [1, 1], [2, 2], [2, 2, 2, 2]),     # dilation 2: five halo rows per output row
    (9, 64, 8, 8, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),       # whole images smaller than one band
    (2, 32, 9, 64, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),      # 64 columns
    (2, 64, 11, 16, 64, 3, 3, [1, 1], [1, 1], [1, 1, 0, 2]),     # all vertical padding below
    (2, 64, 13, 16, 56, 3, 3, [1, 1], [1, 1], [0, 2, 1, 1]),     # all horizontal padding on the right
    (3, 64, 23, 40, 64, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),     # 23 rows: the last band of an image is short
]


@pytest.mark.parametrize("knobs", [{}, {"TVX_BAND_WGS": "8"}, {"TVX_BAND_WGS": "16", "TVX_BAND_ROWS": "2"},
                                   {"TVX_BAND_WGS": "8", "TVX_BAND_ROWS": "1"}, {"TVX_BAND_ROWS": "3"}],
                         ids=lambda k: "-".join(k.values()) or "default")
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(BAND_GRID)))
def test_conv2d_band(oracle, gi, mode, knobs, monkeypatch):
    """The band kernel with its default launch and with few workgroups / short bands forced, so that every
    workgroup walks many bands through both halo buffers (bands of one, two, three and more output rows)."""
    n, c, h, w, oc, kh, kw, stride, dil, pad = BAND_GRID[gi]
    monkeypatch.setenv("TVX_CONV_BAND", "1")   # also where few bands make the one-tile-per-workgroup kernel the choice
    for k, v in knobs.items():
        monkeypatch.setenv(k, v)
    rng = np.random.default_rng(2600 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=stride, dil=dil,
                              pad=pad, mult=0, mode=mode)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="conv2d_band_i8", **kws)
        assert np.array_equal(got, want), (int((got != want).sum()), np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 4


PW_GRID = [
    # (n, c, h, w, oc): 1x1 stride 1; HW % 16 == 0, % 4 == 0 and odd sizes; channel tails;
    # few and many output tiles; a tile that straddles images; images of fewer than four pixels
    (2, 32, 16, 16, 64),
    (3, 16, 14, 14, 96),
    (5, 24, 7, 7, 144),
    (2, 96, 14, 14, 576),
    (3, 960, 7, 7, 320),
    (1, 5, 3, 5, 7),
    (2, 576, 14, 14, 96),
    (1, 40, 20, 13, 33),
    (2, 130, 6, 6, 200),
    (4, 33, 1, 1, 40),
    (3, 8, 1, 3, 9),
    (2, 70, 2, 1, 5),
    (1, 2, 1, 2, 3),
]


@pytest.mark.parametrize("shape", [None, "128,1", "128,4", "32,1", "32,4"])
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(PW_GRID)))
def test_pointwise_conv_shapes(oracle, gi, mode, shape, monkeypatch):
    """Every workgroup shape of the kernel (pixels per workgroup, wavefronts) on every case,
    not only the one the heuristic would pick."""
    n, c, h, w, oc = PW_GRID[gi]
    if shape is not None:
        monkeypatch.setenv("TVX_PWCONV_SHAPE", shape)
    rng = np.random.default_rng(4000 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="pwconv_i8", **kws)
        assert np.array_equal(got, want), int((got != want).sum())
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("shape", ["128,1", "128,4", "32,1", "32,4"])
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", [0, 2, 3, 4, 8])
def test_pointwise_conv_walks_several_output_tiles_per_wavefront(oracle, gi, mode, shape, monkeypatch):
    """One workgroup per pixel tile (the launch the heuristic picks when pixel tiles alone fill the chip, as in
    a batch-64 network): every wavefront then walks several output tiles in sequence, re-using its input tile
    and - with per-tensor uint8 weights whose zero point is not 128 - the zero-point sums it computed once."""
    n, c, h, w, oc = PW_GRID[gi]
    monkeypatch.setenv("TVX_PWCONV_SHAPE", shape)
    monkeypatch.setenv("TVX_PWCONV_WGS", "1")
    rng = np.random.default_rng(4100 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    assert kws["w_q"][2] is not None or kws["w_q"][1] != 128
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="pwconv_i8", **kws)
        assert np.array_equal(got, want), int((got != want).sum())
    assert len(np.unique(want)) > 4


STREAM_GRID = [
    # (n, c, h, w, oc): shallow inputs, pixel groups of sixteen inside one image
    (3, 32, 16, 48, 64),    # 18 pixel tiles, whole output tiles
    (2, 24, 20, 36, 40),    # padded input channels, a partial output tile, a ragged last pixel tile (1440 pixels)
    (5, 7, 4, 12, 100),     # 48-pixel images: pixel tiles straddle images; four output tiles
    (1, 16, 8, 16, 33),     # one pixel tile
]


@pytest.mark.parametrize("tiles", [1, 2, 5])
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(STREAM_GRID)))
def test_pointwise_conv_streaming_form(oracle, gi, mode, tiles, monkeypatch):
    """The form for shallow inputs in which a wavefront walks several pixel tiles with the next tile's rows in
    flight: forced onto small cases (it is chosen from 1024 pixel tiles up), 1, 2 and 5 tiles per wavefront."""
    n, c, h, w, oc = STREAM_GRID[gi]
    monkeypatch.setenv("TVX_PWCONV_STREAM_MIN_TILES", "1")
    monkeypatch.setenv("TVX_PWCONV_STREAM", str(tiles))
    monkeypatch.setenv("TVX_PWCONV_SHAPE", "128,1")
    rng = np.random.default_rng(4300 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="pwconv_i8_stream", **kws)
        assert np.array_equal(got, want), int((got != want).sum())
    assert len(np.unique(want)) > 4


DW_GRID = [
    # (n, c, h, w, stride, pad[l,r,t,b])
    (2, 8, 16, 16, 1, [1, 1, 1, 1]),
    (1, 5, 9, 12, 1, [1, 1, 1, 1]),
    (3, 4, 17, 20, 2, [0, 1, 0, 1]),
    (2, 6, 16, 24, 2, [1, 1, 1, 1]),
    (1, 3, 10, 8, 1, [0, 0, 0, 0]),
    (1, 7, 33, 40, 1, [1, 1, 2, 2]),
    # rows of whole 8-byte units at stride 1: eight columns per thread
    (2, 4, 12, 16, 1, [0, 2, 0, 2]),     # no left padding
    (1, 3, 100, 24, 1, [1, 1, 1, 1]),    # three patches on four lanes, a tall plane (several workgroups per plane)
    (2, 5, 7, 64, 1, [1, 1, 1, 1]),      # eight patches per row, fewer rows than a patch is tall in the last group
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(DW_GRID)))
def test_depthwise3x3_shapes(oracle, gi, mode):
    n, c, h, w, s, pad = DW_GRID[gi]
    rng = np.random.default_rng(3000 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[s, s], dil=[1, 1],
                              pad=pad, mult=1, mode=mode)
    fast = kws["out_shape"][0] % 4 == 0
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="dwconv3x3_i8" if fast else "dwconv_planes_i8", **kws)
        assert np.array_equal(got, want)


@pytest.mark.parametrize("gi", [0, 6, 7, 8])
def test_depthwise3x3_four_columns_per_thread_on_wide_rows(oracle, gi, monkeypatch):
    """The four-column form on shapes that would take the eight-column one (it is what runs there when a tensor
    is not 8-byte aligned)."""
    n, c, h, w, s, pad = DW_GRID[gi]
    monkeypatch.setenv("TVX_DWCONV_COLS", "4")
    rng = np.random.default_rng(3100 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[s, s], dil=[1, 1],
                              pad=pad, mult=1, mode="u8")
    want = oracle.conv2d(x, wt, b, act=2, **kws)
    got = TC.gpu_conv2d(x, wt, b, act=2, want_kernel="dwconv3x3_i8", **kws)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("gi", [0, 6, 8])
def test_depthwise3x3_tensors_off_the_eight_byte_grid(oracle, gi):
    """Tensors that start four bytes into their allocations: the operator planned for 64-bit row loads has to
    take its four-column form at run time."""
    n, c, h, w, s, pad = DW_GRID[gi]
    rng = np.random.default_rng(3200 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[s, s], dil=[1, 1],
                              pad=pad, mult=1, mode="u8")
    want = oracle.conv2d(x, wt, b, act=0, **kws)
    got = TC.gpu_conv2d(x, wt, b, act=0, want_kernel="dwconv3x3_i8", misalign=4, **kws)
    assert np.array_equal(got, want)
    assert len(np.unique(want)) > 4


GROUPED_GRID = [
    # (n, c, oc, groups, h, w, k, stride, pad): the reference's shapes (groupedconv2d_test.cc) scaled up;
    # groups == c is a depthwise convolution in disguise and must reach the depthwise kernels
    (2, 6, 4, 2, 9, 9, 3, [1, 1], [0, 0, 0, 0], "conv2d_generic"),
    (1, 12, 9, 3, 7, 10, 3, [2, 1], [1, 1, 1, 1], "conv2d_generic"),
    (3, 8, 8, 4, 6, 6, 1, [1, 1], [0, 0, 0, 0], "conv2d_generic"),
    (2, 16, 16, 16, 12, 12, 3, [1, 1], [1, 1, 1, 1], None),
    (2, 6, 12, 6, 8, 8, 2, [2, 2], [0, 1, 0, 1], None),
    (1, 5, 7, 1, 6, 6, 3, [1, 1], [1, 1, 1, 1], None),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc", "f32", "f16"])
@pytest.mark.parametrize("gi", range(len(GROUPED_GRID)))
def test_grouped_conv2d(oracle, gi, mode):
    n, c, oc, groups, h, w, k, stride, pad, kernel = GROUPED_GRID[gi]
    rng = np.random.default_rng(7000 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=k, kw=k, stride=stride, dil=[1, 1],
                              pad=pad, mult=0, mode=mode, groups=groups)
    want = oracle.conv2d(x, wt, b, **kws)
    quant = mode not in ("f32", "f16")
    got = TC.gpu_conv2d(x, wt, b, want_kernel=kernel if quant else None, **kws)
    if quant:
        assert np.array_equal(got, want), int((got != want).sum())
        assert len(np.unique(want)) > 4
    else:
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=2e-2)
    if groups == c and quant and oc == c and k == 3:
        # the same numbers as the depthwise spelling of the operator
        dw = dict(kws, multiplier=1)
        dw.pop("groups")
        assert np.array_equal(TC.gpu_conv2d(x, wt, b, **dw), got)


GEMM_GRID = [
    # (n, c, oc, groups, h, w, kh, kw, stride, dil, pad[l,r,t,b]): groups worth a matrix tile (at least 8 output
    # channels and 32 window bytes each), one and two 32-channel tiles per workgroup, ragged last tiles, pixel
    # counts that are no multiple of four (element stores) and of 128 (ragged pixel tile), dilation, strides
    (2, 32, 48, 2, 13, 11, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (2, 64, 256, 4, 16, 16, 3, 3, [2, 2], [1, 1], [0, 1, 0, 1]),
    (1, 40, 40, 2, 15, 14, 5, 5, [1, 1], [2, 2], [4, 4, 4, 4]),
    (3, 48, 200, 2, 12, 20, 3, 1, [1, 2], [1, 1], [0, 0, 1, 1]),
    (2, 36, 27, 3, 9, 9, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (1, 40, 72, 1, 24, 24, 1, 1, [1, 1], [1, 1], [0, 0, 0, 0]),
    # unit column stride and output rows of whole pixel quads (the gather by quads): windows that leave the image
    # on the left and right by 1, 2 and 3 columns, the narrowest row (4 columns: every load is clamped), groups
    # whose channels do not fill a chunk half, row stride 2, as much padding as the window reaches
    (2, 32, 48, 2, 12, 16, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (1, 24, 24, 3, 10, 12, 3, 3, [1, 1], [2, 2], [2, 2, 2, 2]),
    (2, 64, 64, 2, 8, 4, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (1, 80, 40, 2, 9, 8, 3, 3, [1, 1], [3, 3], [3, 3, 3, 3]),
    (2, 36, 96, 3, 15, 20, 3, 5, [1, 2], [1, 1], [2, 2, 1, 1]),
    (1, 32, 32, 2, 6, 10, 3, 3, [1, 1], [1, 1], [2, 2, 2, 2]),
    (1, 64, 64, 2, 35, 32, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc", "f16"])
@pytest.mark.parametrize("gi", range(len(GEMM_GRID)))
def test_conv2d_gemm(oracle, gi, mode):
    """conv2d_gemm_i8 / conv2d_gemm_f16: windows gathered into LDS, MFMA over 64-byte chunks of the reduction."""
    n, c, oc, groups, h, w, kh, kw, stride, dil, pad = GEMM_GRID[gi]
    rng = np.random.default_rng(7300 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=stride, dil=dil,
                              pad=pad, mult=0, mode=mode, groups=groups if groups > 1 else 0)
    quant = mode != "f16"
    if quant and groups == 1 and kh == 1 and kw == 1:
        pytest.skip("the pointwise kernel takes the quantized 1x1 case")
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="conv2d_gemm_i8" if quant else "conv2d_gemm_f16", **kws)
        if quant:
            assert np.array_equal(got, want), int((got != want).sum())
        else:
            assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=2e-2)
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("kernel", ["conv2d_gemm_f16", "conv2d_igemm_f16"])
def test_conv2d_f16_kernels_match_float32_arithmetic(oracle, kernel, monkeypatch):
    """The float16 kernels accumulate in float32 and round once: against a float64 convolution of the same
    float16 operands the error stays within one float16 rounding of the result (plus the accumulation's)."""
    import torch
    import torch.nn.functional as F
    if kernel == "conv2d_gemm_f16":
        monkeypatch.setenv("TVX_NO_CONV_IGEMM_F16", "1")
    rng = np.random.default_rng(7400)
    n, c, oc, h, w = 2, 48, 64, 20, 20
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=3, kw=3, stride=[1, 1], dil=[1, 1],
                              pad=[1, 1, 1, 1], mult=0, mode="f16")
    got = TC.gpu_conv2d(x, wt, b, want_kernel=kernel, **kws).astype(np.float64)
    ref = F.conv2d(torch.from_numpy(x.astype(np.float64).reshape(n, c, h, w)),
                   torch.from_numpy(wt.astype(np.float64).reshape(oc, c, 3, 3)),
                   torch.from_numpy(b.astype(np.float64)), padding=1).numpy().reshape(-1)
    assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -10 + 2e-3)


IGEMM_F16_GRID = [
    # (n, c, oc, h, w, kh, kw, stride, pad[l,r,t,b]): the headline shape's layout in small; one and two channel tiles and a
    # ragged third; 2 / 4 / 8 channel steps; pixel counts that are no multiple of 128 (ragged last tile) or of four
    # (element stores); tiles that start in the middle of a row; strides 1 and 2; windows 1x1 .. 5x3; uneven pads
    (2, 64, 64, 14, 14, 3, 3, 1, [1, 1, 1, 1]),
    (1, 32, 40, 9, 10, 3, 3, 1, [1, 1, 1, 1]),
    (2, 16, 100, 12, 20, 1, 1, 1, [0, 0, 0, 0]),
    (1, 128, 32, 7, 6, 3, 3, 1, [1, 1, 1, 1]),
    (2, 48, 64, 20, 20, 3, 3, 2, [0, 1, 0, 1]),
    (1, 80, 48, 11, 14, 5, 3, 1, [2, 2, 1, 1]),
    (3, 32, 33, 13, 16, 3, 3, 1, [0, 2, 2, 0]),
    (1, 64, 64, 30, 56, 3, 3, 1, [1, 1, 1, 1]),
    (2, 16, 16, 5, 2, 2, 2, 1, [1, 0, 0, 1]),
    (1, 96, 70, 16, 12, 3, 3, 3, [1, 1, 1, 1]),
]


@pytest.mark.parametrize("pixel_tiles", [1, 2])
@pytest.mark.parametrize("gi", range(len(IGEMM_F16_GRID)))
def test_conv2d_igemm_f16(oracle, gi, pixel_tiles, monkeypatch):
    """conv2d_igemm_f16 (halo rows transposed into LDS once, implicit GEMM on the matrix cores) against the oracle within
    the float16 tolerance and, within float32 accumulation noise, against conv2d_gemm_f16 on the same operands."""
    import os
    n, c, oc, h, w, kh, kw, stride, pad = IGEMM_F16_GRID[gi]
    monkeypatch.setenv("TVX_CONV_F16_PIXEL_TILES", str(pixel_tiles))   # 128- and 256-pixel workgroups
    rng = np.random.default_rng(7600 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=[stride, stride], dil=[1, 1],
                              pad=pad, mult=0, mode="f16")
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="conv2d_igemm_f16", **kws)
        assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=FLOAT_RTOL, atol=2e-2)
        os.environ["TVX_NO_CONV_IGEMM_F16"] = "1"
        try:
            other = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="conv2d_gemm_f16", **kws)
        finally:
            del os.environ["TVX_NO_CONV_IGEMM_F16"]
        # two float32 accumulation orders of the same products, each rounded once to float16
        assert np.allclose(got.astype(np.float32), other.astype(np.float32), rtol=2e-3, atol=2e-3)
    assert len(np.unique(want)) > 4


DWP_GRID = [
    # (n, c, h, w, kh, kw, stride, dil, pad[l,r,t,b]): widths 14 / 7 / odd, 5x5 and 1x3 kernels,
    # dilation, asymmetric padding, a plane count that leaves a ragged last workgroup
    (4, 24, 14, 14, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (3, 40, 7, 7, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    (2, 19, 14, 14, 3, 3, [2, 2], [1, 1], [0, 1, 0, 1]),
    (1, 7, 9, 11, 5, 5, [1, 1], [1, 1], [2, 2, 2, 2]),
    (2, 5, 13, 6, 3, 3, [1, 2], [2, 2], [2, 2, 2, 2]),
    (1, 3, 5, 9, 1, 3, [1, 1], [1, 1], [1, 1, 0, 0]),
    (70, 33, 7, 7, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
    # 3x3 dword form: left padding 0 / 2 / 3, widths 4 / 5 / 6 / 13, stride 2 on odd widths, rows
    # of padding only at the top, more right padding than the kernel reaches
    (3, 11, 6, 5, 3, 3, [1, 1], [1, 1], [0, 0, 0, 0]),
    (2, 9, 8, 13, 3, 3, [1, 1], [1, 1], [2, 1, 2, 0]),
    (2, 6, 5, 6, 3, 3, [1, 1], [1, 1], [3, 2, 1, 2]),
    (5, 17, 13, 13, 3, 3, [2, 2], [1, 1], [1, 1, 1, 1]),
    (3, 8, 9, 4, 3, 3, [2, 2], [1, 1], [0, 1, 1, 0]),
    (2, 12, 7, 28, 3, 3, [1, 1], [1, 1], [2, 2, 1, 1]),
    (64, 96, 14, 14, 3, 3, [1, 1], [1, 1], [1, 1, 1, 1]),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(DWP_GRID)))
def test_depthwise_planes_shapes(oracle, gi, mode):
    n, c, h, w, kh, kw, stride, dil, pad = DWP_GRID[gi]
    rng = np.random.default_rng(5000 + gi)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=kh, kw=kw, stride=stride, dil=dil,
                              pad=pad, mult=1, mode=mode)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="dwconv_planes_i8", **kws)
        assert np.array_equal(got, want), int((got != want).sum())
    assert len(np.unique(want)) > 4


def test_depthwise_then_pointwise_full_size(oracle):
    """int8 per-channel block: depthwise 3x3 on 112x112x32 at batch 32, then pointwise 1x1 32->64
    with fused ReLU6; both stages whole-tensor against the oracle."""
    rng = np.random.default_rng(0x73)
    n, c, h, w, oc = 32, 32, 112, 112, 64
    x = rng.integers(-128, 128, n * c * h * w, dtype=np.int8)
    wd = rng.integers(-128, 128, c * 9, dtype=np.int8)
    bd = rng.integers(-4096, 4097, c).astype(np.int32)
    sd = np.exp(rng.uniform(np.log(0.002), np.log(0.05), c)).astype(np.float32)
    kd = dict(in_shape=[w, h, c, n], w_shape=[3, 3, c, 1], out_shape=[w, h, c, n], stride=[1, 1],
              dilation=[1, 1], pad_left=1, pad_top=1, multiplier=1, in_dtype=1, w_dtype=1, out_dtype=1,
              in_q=(0.03, 0), w_q=(1.0, 0, sd), out_q=(0.08, 0))
    mid_want = oracle.conv2d(x, wd, bd, **kd)
    mid = TC.gpu_conv2d(x, wd, bd, want_kernel="dwconv3x3_i8", **kd)
    assert np.array_equal(mid, mid_want)
    assert len(np.unique(mid)) > 100
    wp = rng.integers(-128, 128, oc * c, dtype=np.int8)
    bp = rng.integers(-4096, 4097, oc).astype(np.int32)
    sp = np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32)
    kp = dict(in_shape=[w, h, c, n], w_shape=[1, 1, c, oc], out_shape=[w, h, oc, n], stride=[1, 1],
              dilation=[1, 1], pad_left=0, pad_top=0, multiplier=0, in_dtype=1, w_dtype=1, out_dtype=1,
              in_q=(0.08, 0), w_q=(1.0, 0, sp), out_q=(0.05, 0), act=2)
    out_want = oracle.conv2d(mid, wp, bp, **kp)
    out = TC.gpu_conv2d(mid, wp, bp, want_kernel=("pwconv_i8", "pwconv_i8_stream"), **kp)
    assert np.array_equal(out, out_want)
    assert out.min() == 0 and out.max() == 120  # ReLU6 at scale 0.05


@pytest.mark.parametrize("in_dims,perm", [
    ((5, 3), (1, 0)), ((4, 3, 2), (2, 0, 1)), ((4, 3, 2), (1, 2, 0)), ((56, 56, 24, 3), (2, 0, 1, 3)),
    ((24, 56, 56, 3), (1, 2, 0, 3)), ((7, 5, 3, 2), (0, 1, 2, 3)), ((3, 1, 4, 1, 5, 2), (5, 4, 3, 2, 1, 0)), ((6,), (0,))])
def test_transpose(oracle, in_dims, perm):
    # (2,0,1,3) / (1,2,0,3) are the WHCN <-> CWHN conversions layout inference inserts around NHWC models
    for dt in (np.uint8, np.float16, np.int32):
        x = ((np.arange(int(np.prod(in_dims))) * 7 + 3) % 60000).astype(np.uint32).astype(dt)
        assert np.array_equal(TC.gpu_transpose(x, in_dims, perm), oracle.transpose(x, in_dims, perm))


def test_transpose_rejects_bad_descriptors():
    T = TC.tvx()
    for rank, perm, eb in ((0, (0,), 1), (7, (0,) * 6, 1), (2, (0, 0), 1), (2, (0, 2), 1), (2, (1, 0), 3)):
        d = T.TransposeDesc()
        d.rank, d.elem_bytes = rank, eb
        for i in range(min(rank, 6)):
            d.in_dims[i], d.perm[i] = 2, perm[i]
        with pytest.raises(T.TvxError):
            T.transpose_create(d)


@pytest.mark.parametrize("in_dtype,out_dtype", [(i, o) for i in range(4) for o in range(4)])
def test_dataconvert(oracle, in_dtype, out_dtype):
    # every pair of the four tensor types, 100003 elements incl. ties, saturation and all 8-bit codes
    rng = np.random.default_rng(in_dtype * 4 + out_dtype)
    n = 100003
    in_q = (0.037, 121 if in_dtype == 0 else -5) if in_dtype < 2 else (1.0, 0)
    out_q = (0.052, 117 if out_dtype == 0 else 9) if out_dtype < 2 else (1.0, 0)
    if in_dtype < 2:
        x = rand_q(rng, n, in_dtype)
    else:
        x = (rng.standard_normal(n) * 4).astype(np.float32)
        x[:64] = (np.arange(64) - 32) * np.float32(0.026)   # exact half-steps of the output scale
        x[64:68] = [1e6, -1e6, 0.0, -0.0]
        with np.errstate(over="ignore"):
            x = x.astype(TC.NP_OF[in_dtype])   # 1e6 becomes inf in float16, on purpose
    want = oracle.convert(x, in_dtype, in_q, out_dtype, out_q)
    got = TC.gpu_convert(x, in_dtype, in_q, out_dtype, out_q)
    assert np.array_equal(got.view(np.uint8), want.view(np.uint8))   # bit-exact, floats included


DECONV_GRID = [
    # n, c, h, w, oc, kh, kw, stride, pad(l, t), output_padding, groups, mode
    (2, 8, 7, 9, 12, 3, 3, (2, 2), (1, 1), (1, 1), 1, "u8"),        # the usual 2x upsampling
    (1, 16, 14, 14, 16, 4, 4, (2, 2), (1, 1), (0, 0), 1, "i8pc"),
    (3, 6, 5, 4, 6, 3, 3, (1, 1), (0, 0), (0, 0), 6, "u8"),          # depthwise form {Kw, Kh, C, 1}
    (2, 6, 5, 4, 9, 2, 3, (3, 2), (0, 1), (2, 1), 3, "u8pc"),        # grouped, stride > kernel along W
    (2, 5, 6, 6, 7, 3, 2, (2, 3), (2, 0), (1, 2), 1, "f32"),
    (1, 4, 9, 8, 4, 5, 5, (2, 2), (2, 2), (1, 1), 1, "f16"),
    (1, 3, 33, 31, 5, 3, 3, (2, 2), (1, 1), (1, 1), 1, "u8"),
]


@pytest.mark.parametrize("cfg", DECONV_GRID, ids=lambda c: "n%dc%d_%dx%d_oc%d_k%dx%d_s%s_p%s_op%s_g%d_%s" % (
    c[0], c[1], c[2], c[3], c[4], c[5], c[6], "x".join(map(str, c[7])), "x".join(map(str, c[8])),
    "x".join(map(str, c[9])), c[10], c[11]))
def test_deconv2d(oracle, cfg):
    n, c, h, w, oc, kh, kw, stride, pad, opad, groups, mode = cfg
    rng = np.random.default_rng(DECONV_GRID.index(cfg) + 77)
    ow = (w - 1) * stride[0] + kw - 2 * pad[0] + opad[0]
    oh = (h - 1) * stride[1] + kh - 2 * pad[1] + opad[1]
    depthwise = groups == c == oc
    ws = [kw, kh, c, 1] if depthwise else [kw, kh, c // groups, oc]
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=kh, kw=kw, stride=list(stride), dil=[1, 1],
                              pad=[pad[0], pad[0], pad[1], pad[1]], mult=0, mode=mode, groups=groups)
    kw_args = dict(kws)
    kw_args.update(out_shape=[ow, oh, oc, n], w_shape=ws, groups=groups, transposed=True)
    want = oracle.conv2d(x, wt, b, **kw_args)
    for const_weights in (True, False):
        got = TC.gpu_conv2d(x, wt, b, const_weights=const_weights, want_kernel="deconv2d_generic", **kw_args)
        if mode in ("f32", "f16"):
            assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=1e-2)  # tolerance of the path
        else:
            assert np.array_equal(got, want)
            assert 0.02 < np.mean((want > want.min()) & (want < want.max())), "saturated test data"


IM2COL_GRID = [
    # short windows (C * Kh * Kw <= 64, C not a multiple of 16): conv2d_im2col_i8
    dict(n=3, c=3, h=33, w=31, oc=32, kh=3, kw=3, stride=[2, 2], dil=[1, 1], pad=[0, 1, 0, 1], mult=0),   # MobileNet conv1 form
    dict(n=2, c=1, h=28, w=28, oc=20, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0),   # LeNet conv1
    dict(n=2, c=4, h=19, w=23, oc=50, kh=4, kw=4, stride=[1, 2], dil=[1, 1], pad=[2, 1, 1, 2], mult=0),   # K = 64 exactly
    dict(n=1, c=7, h=20, w=20, oc=100, kh=3, kw=3, stride=[1, 1], dil=[2, 2], pad=[2, 2, 2, 2], mult=0),  # K = 63, dilated, 4 channel tiles
    dict(n=5, c=2, h=9, w=7, oc=5, kh=1, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 0, 0], mult=0),      # tiny, hw % 4 != 0
    dict(n=2, c=3, h=64, w=64, oc=64, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 1, 1], mult=0),   # several workgroups per image
    dict(n=1, c=5, h=10, w=6, oc=40, kh=2, kw=3, stride=[1, 1], dil=[1, 3], pad=[2, 2, 1, 1], mult=0),    # rows as dwords that begin two bytes in front of the tensor / end behind it
    dict(n=1, c=1, h=1, w=4, oc=3, kh=1, kw=3, stride=[1, 1], dil=[1, 1], pad=[2, 2, 0, 0], mult=0),      # a four-byte tensor
    # kernel rows five taps wide: two dwords per row
    dict(n=1, c=1, h=1, w=5, oc=4, kh=1, kw=5, stride=[1, 1], dil=[1, 1], pad=[2, 2, 0, 0], mult=0),      # a five-byte tensor: both dwords moved inside
    dict(n=1, c=1, h=2, w=4, oc=3, kh=1, kw=5, stride=[1, 1], dil=[1, 1], pad=[2, 2, 0, 0], mult=0),      # eight bytes: the second dword of the last windows lies behind the tensor
    dict(n=2, c=2, h=7, w=9, oc=33, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[2, 2, 2, 2], mult=0),     # SAME 5 x 5, K = 50, two channel tiles
    dict(n=3, c=1, h=11, w=13, oc=7, kh=3, kw=5, stride=[2, 1], dil=[1, 1], pad=[1, 3, 1, 1], mult=0),    # uneven pads, strides
    dict(n=1, c=4, h=6, w=6, oc=9, kh=3, kw=5, stride=[1, 1], dil=[2, 1], pad=[4, 4, 2, 2], mult=0),      # K = 60, left padding as wide as the window reaches
    # wavefronts whose windows all lie inside the image's rows (no dword moved, the column border as one mask per
    # thread) next to wavefronts on the first / last rows
    dict(n=2, c=3, h=40, w=72, oc=32, kh=3, kw=3, stride=[2, 2], dil=[1, 1], pad=[1, 1, 1, 1], mult=0),
    dict(n=2, c=1, h=40, w=44, oc=12, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[2, 2, 2, 2], mult=0),
    dict(n=2, c=2, h=30, w=50, oc=16, kh=3, kw=3, stride=[1, 1], dil=[2, 1], pad=[0, 2, 2, 2], mult=0),   # dilated rows: window rows 0, 2, 4
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(IM2COL_GRID)))
def test_conv2d_im2col(oracle, gi, mode):
    rng = np.random.default_rng(3000 + gi)
    x, w, b, kws = conv_case(rng, mode=mode, **IM2COL_GRID[gi])
    for act in (0, 2):
        want = oracle.conv2d(x, w, b, act=act, **kws)
        got = TC.gpu_conv2d(x, w, b, act=act, want_kernel="conv2d_im2col_i8", **kws)
        assert np.array_equal(got, want), (gi, mode, act, np.flatnonzero(got != want)[:8])
    assert 0.02 < np.mean((want > want.min()) & (want < want.max())), "saturated test data"


@pytest.mark.parametrize("side,n", [(16, 2), (14, 3), (7, 5), (5, 1), (3, 2), (1, 6)], ids=lambda v: str(v))   # hw % 16 == 0, % 4 == 0, odd, below 4
@pytest.mark.parametrize("mode", ["u8", "i8pc"])
@pytest.mark.parametrize("conv_operand", [1, 2])
def test_pointwise_conv_with_fused_add(oracle, side, n, mode, conv_operand):
    """tvx_conv2d_add_create against the two operators it stands for: the oracle's convolution, quantized to
    the convolution's own output tensor, then the oracle's Add with the other operand."""
    rng = np.random.default_rng(side * 10 + conv_operand)
    c, oc = 48, 40
    x, w, b, kws = conv_case(rng, n=n, c=c, h=side, w=side, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                             pad=[0, 0, 0, 0], mult=0, mode=mode)
    dt = kws["out_dtype"]
    conv_q = kws["out_q"]
    other = rand_q(rng, n * oc * side * side, dt)
    other_q = (0.037, 121 if dt == 0 else -7)
    sum_q = (float(np.float32(conv_q[0] * 1.3)), 119 if dt == 0 else 5)
    t = oracle.conv2d(x, w, b, **kws)
    a, aq, bb, bq = (t, conv_q, other, other_q) if conv_operand == 1 else (other, other_q, t, conv_q)
    want = oracle.add(dt, a, aq, bb, bq, sum_q)
    T = TC.tvx()
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = kws["in_shape"]
    d.k_w = d.k_h = 1
    d.out_w, d.out_h, d.out_c = side, side, oc
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.in_dtype, d.w_dtype, d.out_dtype = kws["in_dtype"], kws["w_dtype"], dt
    d.in_scale, d.in_zp = kws["in_q"]
    keep = []
    TC._wq(d, kws["w_q"], keep)
    d.out_scale, d.out_zp = conv_q
    e = T.EltwiseDesc()
    e.count, e.dtype = want.size, dt
    e.a_scale, e.a_zp = aq
    e.b_scale, e.b_zp = bq
    e.out_scale, e.out_zp = sum_q
    op = T.conv2d_add_create(d, e, conv_operand, w, b)
    assert op.kernel_name == "pwconv_add_i8"
    import torch
    xd, od = TC.to_device(x), TC.to_device(other)
    yd = TC.device_out(want.size, TC.NP_OF[dt])
    op.run(xd, od, yd)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:8]
    assert 0.05 < np.mean((want > want.min()) & (want < want.max()))
    # a convolution no fused kernel takes: the caller is told so and creates the two operators
    d.k_w = d.k_h = 3
    d.pad_left = d.pad_top = 1
    w3 = rand_q(rng, oc * c * 9, kws["w_dtype"])
    with pytest.raises(T.TvxError) as err:
        T.conv2d_add_create(d, e, conv_operand, w3, b)
    assert err.value.status == T.E_UNSUPPORTED


def test_page_locked_host_memory_round_trip():
    """tvx_host_malloc memory as source and target of the library's copies."""
    import ctypes as C
    T = TC.tvx()
    L = T.lib()
    vp = C.c_void_p
    L.tvx_host_malloc.argtypes = [C.POINTER(vp), C.c_size_t]
    L.tvx_host_free.argtypes = [vp]
    L.tvx_malloc.argtypes = [C.POINTER(vp), C.c_size_t]
    L.tvx_free.argtypes = [vp]
    for f in (L.tvx_memcpy_h2d, L.tvx_memcpy_d2h):
        f.argtypes = [vp, vp, C.c_size_t, vp]
    L.tvx_stream_synchronize.argtypes = [vp]
    n = 1 << 20
    src, dst, dev = vp(), vp(), vp()
    assert L.tvx_host_malloc(C.byref(src), n) == 0 and L.tvx_host_malloc(C.byref(dst), n) == 0
    assert L.tvx_malloc(C.byref(dev), n) == 0
    data = np.random.default_rng(5).integers(0, 256, n, dtype=np.uint8)
    C.memmove(src, data.ctypes.data, n)
    assert L.tvx_memcpy_h2d(dev, src, n, None) == 0 and L.tvx_memcpy_d2h(dst, dev, n, None) == 0
    assert L.tvx_stream_synchronize(None) == 0
    back = np.frombuffer((C.c_uint8 * n).from_address(dst.value), dtype=np.uint8)
    assert np.array_equal(back, data)
    assert L.tvx_host_free(src) == 0 and L.tvx_host_free(dst) == 0 and L.tvx_free(dev) == 0
    empty = vp(1)
    assert L.tvx_host_malloc(C.byref(empty), 0) == 0 and not empty.value
