"""Seeded differential sweep: random operator configurations, HIP result vs oracle, bit for bit.
The shapes are drawn so that every kernel variant is reached many times (dense 3x3 / 5x5 /
strided / dilated, pointwise with every pixel-count residue, depthwise on aligned and odd
widths, FullyConnected around the tile and K-chunk edges, pooling of every type)."""
import collections

import numpy as np
import pytest

import tvx_case as TC
from test_gpu_parity import conv_case, rand_q

pytestmark = pytest.mark.gpu


def _conv_config(rng):
    kind = rng.choice(["dense", "pointwise", "depthwise", "depthwise_mobile"])
    n = int(rng.integers(1, 4))
    if kind == "depthwise_mobile":
        # the MobileNet shape: 3x3, one stride for both axes, SAME padding, rows of whole dwords
        st = int(rng.choice([1, 2]))
        w, h = 4 * st * int(rng.integers(1, 9)), int(rng.integers(3, 24))
        pl, pt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        return dict(n=n, c=int(rng.integers(1, 70)), h=h, w=w, oc=0, kh=3, kw=3, stride=[st, st], dil=[1, 1],
                    pad=[pl, 2 - pl if st == 1 else 1 - pl, pt, 1], mult=1)
    if kind == "pointwise":
        c, oc = int(rng.integers(1, 200)), int(rng.integers(1, 200))
        h, w = int(rng.integers(1, 20)), int(rng.integers(2, 20))
        if h * w < 4:
            h = 2
        return dict(n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0)
    kh, kw = (int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 3, 5]))) if rng.random() < 0.3 else (3, 3)
    s = [int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))]
    d = [int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2]))]
    # padding never exceeds the kernel's reach: every window touches the image
    pad = [int(min(rng.integers(0, 3), (kw - 1) * d[0])) for _ in range(2)] + \
          [int(min(rng.integers(0, 3), (kh - 1) * d[1])) for _ in range(2)]
    h = int(rng.integers((kh - 1) * d[1] + 1, 24))
    w = int(rng.choice([4, 8, 12, 16, 20, 28])) if rng.random() < 0.5 else int(rng.integers((kw - 1) * d[0] + 1, 24))
    w = max(w, (kw - 1) * d[0] + 1)
    if kind == "depthwise":
        return dict(n=n, c=int(rng.integers(1, 40)), h=h, w=w, oc=0, kh=kh, kw=kw, stride=s, dil=d, pad=pad,
                    mult=int(rng.choice([1, 1, 1, 2])))
    return dict(n=n, c=int(rng.integers(1, 150)), h=h, w=w, oc=int(rng.integers(1, 150)), kh=kh, kw=kw,
                stride=s, dil=d, pad=pad, mult=0)


def test_conv2d_sweep(oracle, tvx):
    rng = np.random.default_rng(0xC0)
    seen = collections.Counter()
    for i in range(240):
        cfg = _conv_config(rng)
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        act = int(rng.integers(0, 3))
        x, wt, b, kws = conv_case(rng, mode=mode, **cfg)
        if min(kws["out_shape"][:2]) < 1:
            continue
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        d_kernel = []
        got = _run_conv(tvx, x, wt, b, act, kws, d_kernel)
        seen[d_kernel[0]] += 1
        assert np.array_equal(got, want), (i, cfg, mode, act, d_kernel[0], int((got != want).sum()))
    # the sweep is only worth its name if it reaches every convolution kernel
    for k in ("conv2d_igemm_i8", "pwconv_i8", "dwconv3x3_i8", "dwconv_planes_i8", "conv2d_generic"):
        assert seen[k] >= 5, seen


def test_grouped_and_float16_conv2d_sweep(oracle):
    """Random grouped convolutions (quantized, bit for bit) and float16 convolutions (1e-2) on the GEMM-over-windows
    kernels: group counts 2-4, channel counts per group around the 32-channel tile edges, any kernel / stride /
    dilation / padding, pixel counts that leave ragged tiles."""
    rng = np.random.default_rng(0x6E)
    seen = collections.Counter()
    for i in range(90):
        kh, kw = (int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 3, 5]))) if rng.random() < 0.4 else (3, 3)
        s = [int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))]
        d = [int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2]))]
        pad = [int(min(rng.integers(0, 3), (kw - 1) * d[0])) for _ in range(2)] + \
              [int(min(rng.integers(0, 3), (kh - 1) * d[1])) for _ in range(2)]
        h = int(rng.integers((kh - 1) * d[1] + 1, 26))
        w = int(rng.integers((kw - 1) * d[0] + 1, 26))
        f16 = i % 3 == 2
        groups = 1 if f16 and rng.random() < 0.5 else int(rng.integers(2, 5))
        icg = int(rng.choice([4, 8, 12, 16, 20, 31, 32, 33, 48]))
        ocg = int(rng.choice([8, 9, 16, 31, 32, 33, 40, 64, 70]))
        if icg * kh * kw * (2 if f16 else 1) < 32:
            icg = 32
        mode = "f16" if f16 else str(rng.choice(["u8", "i8pc", "u8pc"]))
        x, wt, b, kws = conv_case(rng, n=int(rng.integers(1, 4)), c=groups * icg, h=h, w=w, oc=groups * ocg, kh=kh, kw=kw,
                                  stride=s, dil=d, pad=pad, mult=0, mode=mode, groups=groups if groups > 1 else 0)
        if min(kws["out_shape"][:2]) < 1:
            continue
        act = int(rng.integers(0, 3))
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        T = TC.tvx()
        got = TC.gpu_conv2d(x, wt, b, act=act, **kws)
        if f16:
            assert np.allclose(got.astype(np.float32), want.astype(np.float32), rtol=1e-2, atol=2e-2), (i, kws)
            seen["f16"] += 1
        else:
            assert np.array_equal(got, want), (i, kws["in_shape"], kws["w_shape"], groups, mode, act, int((got != want).sum()))
            seen["q"] += 1
    assert seen["f16"] >= 20 and seen["q"] >= 40, seen


def _run_conv(tvx, x, wt, b, act, kws, kernel_out):
    """gpu_conv2d, also reporting which kernel ran."""
    import ctypes as C
    import torch
    d = tvx.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = kws["in_shape"]
    d.k_w, d.k_h = kws["w_shape"][0], kws["w_shape"][1]
    d.out_w, d.out_h, d.out_c = kws["out_shape"][:3]
    d.stride_w, d.stride_h = kws["stride"]
    d.dilation_w, d.dilation_h = kws["dilation"]
    d.pad_left, d.pad_top, d.multiplier = kws["pad_left"], kws["pad_top"], kws["multiplier"]
    d.in_dtype, d.w_dtype, d.out_dtype = kws["in_dtype"], kws["w_dtype"], kws["out_dtype"]
    d.in_scale, d.in_zp = kws["in_q"]
    d.w_scale, d.w_zp = kws["w_q"][0], kws["w_q"][1]
    keep = None
    if kws["w_q"][2] is not None:
        keep = np.ascontiguousarray(kws["w_q"][2], dtype=np.float32)
        d.w_scales = keep.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = kws["out_q"]
    d.activation = act
    op = tvx.conv2d_create(d, wt, b)
    kernel_out.append(op.kernel_name)
    xd = TC.to_device(x)
    yd = TC.device_out(int(np.prod(kws["out_shape"])), TC.NP_OF[kws["out_dtype"]])
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    out = yd.cpu().numpy()
    op.close()
    return out


def test_fully_connected_sweep(oracle):
    rng = np.random.default_rng(0xFC)
    for i in range(60):
        m = int(rng.choice([1, 2, 7, 33, 255, 256, 257, 300]))
        k = int(rng.choice([16, 48, 112, 128, 144, 500, 512, 800, 1000]))
        n = int(rng.choice([1, 10, 31, 64, 255, 256, 257, 500]))
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        in_dt = 0 if mode.startswith("u8") else 1
        w_dt = 0 if mode == "u8" else 1
        x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
        b = rng.integers(-16384, 16385, n).astype(np.int32)
        wq = (0.01, int(rng.integers(100, 157)), None) if mode == "u8" else \
            (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
        kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
                   in_q=(0.02, int(rng.integers(100, 157)) if in_dt == 0 else int(rng.integers(-9, 10))), w_q=wq,
                   out_q=(float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else -3))
        act = int(rng.integers(0, 3))
        want = oracle.fully_connected(x, w, b, act=act, **kws)
        got = TC.gpu_fully_connected(x, w, b, act=act, **kws)
        assert np.array_equal(got, want), (i, m, k, n, mode, act)


def test_fully_connected_tiled_sweep(oracle, monkeypatch):
    """The tiled kernel (more than 2^18 outputs), 256- and 128-row tiles in turn: ragged last tiles in both directions, reductions from
    one 16-byte chunk to nine k-tiles with every tail, uint8 and int8 activations with and without a uniform weight
    zero point (re-bias and row sums inside the kernel), per-channel weights."""
    rng = np.random.default_rng(0xFD)
    for i in range(24):
        m, n = int(rng.integers(513, 1100)), int(rng.integers(513, 1100))
        k = 16 * int(rng.integers(1, 80))
        mode = str(rng.choice(["u8", "i8pc", "u8pc", "i8zp"]))
        in_dt = 0 if mode.startswith("u8") else 1
        w_dt = 0 if mode == "u8" else 1
        x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
        b = rng.integers(-16384, 16385, n).astype(np.int32)
        if mode == "u8":
            wq = (0.01, int(rng.integers(100, 157)), None)
        elif mode == "i8zp":
            wq = (0.01, int(rng.integers(-20, 21)), None)
        else:
            wq = (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
        kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
                   in_q=(0.02, int(rng.integers(100, 157)) if in_dt == 0 else int(rng.integers(-9, 10))), w_q=wq,
                   out_q=(float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else -3))
        act = int(rng.integers(0, 3))
        want = oracle.fully_connected(x, w, b, act=act, **kws)
        tile_m = "128" if i % 2 else "256"   # (its own choice here is 256: fewer than 1024 tiles)
        monkeypatch.setenv("TVX_FC_TILE_M", tile_m)
        got = TC.gpu_fully_connected(x, w, b, act=act, want_kernel="fc_mfma_i8_%sx256x128" % tile_m, **kws)
        assert np.array_equal(got, want), (i, m, k, n, mode, act, tile_m, int((got != want).sum()))


def test_pool2d_sweep(oracle):
    rng = np.random.default_rng(0xB0)
    for i in range(80):
        w, h = int(rng.integers(1, 30)), int(rng.integers(1, 30))
        kw, kh = int(rng.integers(1, min(w, 7) + 1)), int(rng.integers(1, min(h, 7) + 1))
        s = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
        pad = [int(rng.integers(0, kw)), int(rng.integers(0, kw)), int(rng.integers(0, kh)), int(rng.integers(0, kh))]
        c, n = int(rng.integers(1, 9)), int(rng.integers(1, 4))
        out_w = (w + pad[0] + pad[1] - kw) // s[0] + 1
        out_h = (h + pad[2] + pad[3] - kh) // s[1] + 1
        if out_w < 1 or out_h < 1:
            continue
        dtype = int(rng.integers(0, 2))
        ptype = int(rng.choice([0, 1, 3]))
        kws = dict(in_shape=[w, h, c, n], out_shape=[out_w, out_h, c, n], ksize=[kw, kh], stride=s,
                   pad_left=pad[0], pad_top=pad[2], pool_type=ptype, dtype=dtype)
        x = rand_q(rng, w * h * c * n, dtype)
        in_q = (0.1, 7)
        out_q = (0.1, 7) if rng.random() < 0.5 else (0.07, 9 if dtype == 0 else -2)
        want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
        got = TC.gpu_pool2d(x, in_q=in_q, out_q=out_q, **kws)
        assert np.array_equal(got, want), (i, kws)


def test_depthwise_eight_column_form_sweep(oracle):
    """Stride-1 depthwise 3x3 on rows of whole 8-byte units (the form with 64-bit row loads): random plane sizes up
    to several workgroups per plane, left / top padding 0 or 1, and tensors 0, 4 or 8 bytes off their allocations
    (4: the four-column form has to take over at run time)."""
    rng = np.random.default_rng(77)
    for i in range(60):
        n, c = int(rng.integers(1, 4)), int(rng.integers(1, 20))
        h, w = int(rng.integers(3, 120)), 8 * int(rng.integers(1, 33))
        pl, pt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[1, 1], dil=[1, 1],
                                  pad=[pl, 2 - pl, pt, 2 - pt], mult=1, mode=mode)
        act, mis = int(rng.integers(0, 3)), int(rng.choice([0, 0, 4, 8]))
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="dwconv3x3_i8", misalign=mis, **kws)
        assert np.array_equal(got, want), (i, n, c, h, w, pl, pt, mode, act, mis, int((got != want).sum()))


def test_pointwise_streaming_form_sweep(oracle, monkeypatch):
    """The streaming pointwise form forced onto random small cases: 1 to 32 input channels, pixel counts that are
    multiples of 16 in several ways, partial output tiles, 1 to 5 pixel tiles per wavefront."""
    monkeypatch.setenv("TVX_PWCONV_STREAM_MIN_TILES", "1")
    monkeypatch.setenv("TVX_PWCONV_SHAPE", "128,1")
    rng = np.random.default_rng(78)
    for i in range(60):
        n, c, oc = int(rng.integers(1, 6)), int(rng.integers(1, 33)), int(rng.integers(1, 200))
        w, h = 16, int(rng.integers(1, 40))
        if rng.integers(0, 2):
            w, h = 4 * int(rng.integers(1, 9)), 4 * int(rng.integers(1, 9))
        monkeypatch.setenv("TVX_PWCONV_STREAM", str(int(rng.integers(1, 6))))
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                                  pad=[0, 0, 0, 0], mult=0, mode=mode)
        act = int(rng.integers(0, 3))
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel="pwconv_i8_stream", **kws)
        assert np.array_equal(got, want), (i, n, c, h, w, oc, mode, act, int((got != want).sum()))


def test_conv2d_with_max_pool_sweep(oracle, tvx):
    """Random convolutions with even output extents + the 2x2 / stride-2 max pooling behind them through
    tvx_conv2d_pool_create, against the oracle's two operators; both fused kernels must be reached."""
    import torch
    from test_gpu_fused_small_nets import _descs
    rng = np.random.default_rng(0x9001)
    seen = collections.Counter()
    done = 0
    for i in range(400):
        if done >= 120:
            break
        kh, kw = (int(rng.choice([1, 2, 3, 5])), int(rng.choice([1, 3, 5]))) if rng.random() < 0.5 else (3, 3)
        s = [int(rng.choice([1, 1, 2])), int(rng.choice([1, 1, 2]))]
        d = [int(rng.choice([1, 1, 1, 2])), int(rng.choice([1, 1, 1, 2]))]
        pad = [int(min(rng.integers(0, 3), (kw - 1) * d[0])) for _ in range(2)] + \
              [int(min(rng.integers(0, 3), (kh - 1) * d[1])) for _ in range(2)]
        h = int(rng.integers((kh - 1) * d[1] + 2, 30))
        w = int(rng.integers((kw - 1) * d[0] + 2, 30))
        c = int(rng.choice([1, 2, 3, 4])) if rng.random() < 0.4 else int(rng.integers(5, 80))
        cfg = dict(n=int(rng.integers(1, 4)), c=c, h=h, w=w, oc=int(rng.integers(1, 140)), kh=kh, kw=kw, stride=s, dil=d, pad=pad, mult=0)
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        act = int(rng.integers(0, 3))
        x, wt, b, kws = conv_case(rng, mode=mode, **cfg)
        ow, oh, oc, n = kws["out_shape"]
        if ow < 2 or oh < 2 or ow % 2 or oh % 2:
            continue
        keep = []
        dd, pp = _descs(tvx, kws, act, keep)
        try:
            op = tvx.conv2d_pool_create(dd, pp, wt, b)
        except tvx.TvxError as e:
            assert e.status == tvx.E_UNSUPPORTED, (i, cfg)
            seen["declined"] += 1
            continue
        t = oracle.conv2d(x, wt, b, act=act, **kws)
        want = oracle.pool2d(t, in_shape=[ow, oh, oc, n], out_shape=[ow // 2, oh // 2, oc, n], ksize=[2, 2], stride=[2, 2],
                             pad_left=0, pad_top=0, pool_type=0, dtype=kws["out_dtype"], in_q=kws["out_q"], out_q=kws["out_q"])
        seen[op.kernel_name] += 1
        xd = TC.to_device(x)
        yd = TC.device_out(want.size, TC.NP_OF[kws["out_dtype"]])
        op.run(xd, None, yd)
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        op.close()
        assert np.array_equal(got, want), (i, cfg, mode, act, op.kernel_name, int((got != want).sum()))
        done += 1
    assert seen["conv2d_im2col_maxpool_i8"] >= 10 and seen["conv2d_igemm_maxpool_i8"] >= 30, seen


def test_conv2d_band_sweep(oracle, tvx, monkeypatch):
    """Random 3x3 convolutions of the shapes the one-workgroup-per-CU band kernel takes (32 or 64 input channels,
    33..64 output channels, rows of whole 8-byte units, stride 1 or 2, any padding up to one), forced onto it at
    small batches, with random band heights and grid sizes."""
    rng = np.random.default_rng(0xBA2D)
    ran = 0
    for i in range(60):
        st = int(rng.choice([1, 1, 2]))
        w = 8 * int(rng.integers(1, 9))
        if st == 2:
            w = 16 * int(rng.integers(1, 5))
        h = int(rng.integers(3, 40))
        pad = [int(rng.integers(0, 2)) for _ in range(4)]
        cfg = dict(n=int(rng.integers(1, 4)), c=int(rng.choice([32, 64])), h=h, w=w, oc=int(rng.integers(33, 65)), kh=3, kw=3,
                   stride=[st, st], dil=[1, 1], pad=pad, mult=0)
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        act = int(rng.integers(0, 3))
        x, wt, b, kws = conv_case(rng, mode=mode, **cfg)
        if min(kws["out_shape"][:2]) < 1 or kws["out_shape"][0] % 8:
            continue
        monkeypatch.setenv("TVX_CONV_BAND", "1")
        monkeypatch.setenv("TVX_BAND_WGS", str(int(rng.choice([8, 16, 64]))))
        if rng.random() < 0.5:
            monkeypatch.setenv("TVX_BAND_ROWS", str(int(rng.integers(1, 6))))
        else:
            monkeypatch.delenv("TVX_BAND_ROWS", raising=False)
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        d_kernel = []
        got = _run_conv(tvx, x, wt, b, act, kws, d_kernel)
        if d_kernel[0] != "conv2d_band_i8":
            continue
        ran += 1
        assert np.array_equal(got, want), (i, cfg, mode, act, int((got != want).sum()))
    assert ran >= 25, ran


def test_max_pool_register_stencil_sweep(oracle):
    """Stride-2 max pooling with 2- and 3-tap windows on rows of whole 8-byte units (the register-stencil kernel): random
    plane sizes from one lane to a whole wavefront per row and from one to hundreds of rows, pads 0 / 1 in front, output
    widths from as wide as the input allows down to narrower declared ones (rows that end inside a lane's four outputs),
    both code types, equal and different quantization on the two sides."""
    rng = np.random.default_rng(0x57E)
    for i in range(80):
        w, h = 8 * int(rng.integers(1, 65)), int(rng.integers(2, 140 if i % 4 else 700))
        kw, kh = int(rng.integers(2, 4)), int(rng.integers(2, 4))
        pl, pt = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        pr, pb = int(rng.integers(0, 2)), int(rng.integers(0, 2))
        out_w = min((w + pl + pr - kw) // 2 + 1, w // 2) - int(rng.integers(0, 3)) * int(rng.random() < 0.3)
        out_h = (h + pt + pb - kh) // 2 + 1
        if out_w < 1 or out_h < 1 or (out_h - 1) * 2 - pt > h - 1:
            continue
        c, n = int(rng.integers(1, 7)), int(rng.integers(1, 4))
        dtype = int(rng.integers(0, 2))
        kws = dict(in_shape=[w, h, c, n], out_shape=[out_w, out_h, c, n], ksize=[kw, kh], stride=[2, 2],
                   pad_left=pl, pad_top=pt, pool_type=0, dtype=dtype)
        x = rand_q(rng, w * h * c * n, dtype)
        in_q = (0.1, 7)
        out_q = (0.1, 7) if rng.random() < 0.6 else (0.07, 9 if dtype == 0 else -2)
        want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
        got = TC.gpu_pool2d(x, in_q=in_q, out_q=out_q, want_kernel="pool2d_stencil_i8", **kws)
        assert np.array_equal(got, want), (i, kws, out_q, int((got != want).sum()))


def test_channel_blocked_operators_sweep(oracle):
    """The operators between channel-blocked tensors on random shapes: pointwise convolutions (with and without the Add,
    every kernel shape reached through the reduction length and the channel-tile count), depthwise 3x3 at stride 1 with
    random pads, the depthwise kernel that reads WHCN and writes blocked (strides 1 and 2), the whole-plane average."""
    from test_gpu_blocked import _conv_desc, _run, from_blocked, to_blocked
    T = TC.tvx()
    rng = np.random.default_rng(0xB10C)
    seen = collections.Counter()
    for i in range(90):
        kind = ["pw", "pw_add", "dw", "dw_writer", "avg"][i % 5]
        mode = str(rng.choice(["u8", "i8pc", "u8pc"]))
        n = int(rng.integers(1, 5))
        h, w = int(rng.integers(1, 12)), int(rng.integers(1, 12))
        hw = h * w
        act = int(rng.choice([0, 1, 2]))
        keep = []
        if kind in ("pw", "pw_add"):
            c, oc = 32 * int(rng.integers(1, 18)), 32 * int(rng.integers(1, 14))
            x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0],
                                      mult=0, mode=mode)
            dt = kws["out_dtype"]
            if kind == "pw":
                want = oracle.conv2d(x, wt, b, act=act, **kws)
                op = T.conv2d_blocked_create(_conv_desc(T, kws, act, keep), wt, b)
                got = _run(op, to_blocked(x, n, c, hw), want.size, dt)
            else:
                operand = int(rng.integers(1, 3))
                other = rand_q(rng, n * oc * hw, dt)
                other_q, sum_q = (0.037, 121 if dt == 0 else -7), (float(np.float32(kws["out_q"][0] * 1.3)), 119 if dt == 0 else 5)
                t = oracle.conv2d(x, wt, b, **kws)
                a, aq, bb, bq = (t, kws["out_q"], other, other_q) if operand == 1 else (other, other_q, t, kws["out_q"])
                want = oracle.add(dt, a, aq, bb, bq, sum_q)
                e = T.EltwiseDesc()
                e.count, e.dtype = want.size, dt
                e.a_scale, e.a_zp = aq
                e.b_scale, e.b_zp = bq
                e.out_scale, e.out_zp = sum_q
                op = T.conv2d_blocked_create(_conv_desc(T, kws, 0, keep), wt, b, add_desc=e, conv_operand=operand)
                got = _run(op, to_blocked(x, n, c, hw), want.size, dt, other=to_blocked(other, n, oc, hw))
            got = from_blocked(got, n, oc, hw)
        elif kind == "dw":
            c = 16 * int(rng.integers(1, 12))
            pad = [int(rng.integers(0, 2)) for _ in range(4)]
            if h + pad[2] + pad[3] < 3 or w + pad[0] + pad[1] < 3:
                pad = [1, 1, 1, 1]
            x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=pad, mult=1, mode=mode)
            want = oracle.conv2d(x, wt, b, act=act, **kws)
            op = T.conv2d_blocked_create(_conv_desc(T, kws, act, keep), wt, b)
            got = from_blocked(_run(op, to_blocked(x, n, c, hw), want.size, kws["out_dtype"]), n, c,
                               kws["out_shape"][0] * kws["out_shape"][1])
        elif kind == "dw_writer":
            c, st = 16 * int(rng.integers(1, 8)), int(rng.choice([1, 2]))
            h, w = int(rng.integers(3, 30)), int(rng.integers(4, 30))
            pad = [1, 1, 1, 1] if st == 1 else [int(rng.integers(0, 2)), 1, int(rng.integers(0, 2)), 1]
            x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[st, st], dil=[1, 1], pad=pad, mult=1, mode=mode)
            want = oracle.conv2d(x, wt, b, act=act, **kws)
            op = T.conv2d_to_blocked_create(_conv_desc(T, kws, act, keep), wt, b)
            got = from_blocked(_run(op, x, want.size, kws["out_dtype"]), n, c, kws["out_shape"][0] * kws["out_shape"][1])
        else:
            c, dt = 16 * int(rng.integers(1, 40)), int(rng.integers(0, 2))
            x = rand_q(rng, n * c * hw, dt)
            in_q = (0.1, 7 if dt == 0 else -3)
            out_q = in_q if rng.random() < 0.5 else (0.07, 9 if dt == 0 else 2)
            kws = dict(in_shape=[w, h, c, n], out_shape=[1, 1, c, n], ksize=[w, h], stride=[1, 1], pad_left=0, pad_top=0,
                       pool_type=int(rng.choice([1, 3])), dtype=dt)
            want = oracle.pool2d(x, in_q=in_q, out_q=out_q, **kws)
            d = T.Pool2dDesc()
            d.in_w, d.in_h, d.channels, d.batch = w, h, c, n
            d.out_w = d.out_h = 1
            d.k_w, d.k_h, d.stride_w, d.stride_h = w, h, 1, 1
            d.pool_type, d.dtype = kws["pool_type"], dt
            d.in_scale, d.in_zp = in_q
            d.out_scale, d.out_zp = out_q
            op = T.pool2d_blocked_create(d)
            got = _run(op, to_blocked(x, n, c, hw), want.size, dt)
        seen[kind] += 1
        assert np.array_equal(got, want), (i, kind, mode, n, h, w, int((got != want).sum()), np.flatnonzero(got != want)[:6])
    assert min(seen.values()) == 18
