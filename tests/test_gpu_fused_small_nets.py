"""tvx_conv2d_pool_create and tvx_fully_connected_softmax_create (the pairs LeNet is made of) against the two
operators each stands for: the oracle's convolution quantized to its own output tensor, then the oracle's max
pooling - bit-exact; the oracle's FullyConnected codes, then its Softmax - within the Softmax tolerance, and
bit for bit what the library's own two kernels give."""
import numpy as np
import pytest

import tvx_case as TC
from test_gpu_parity import conv_case, rand_q

pytestmark = pytest.mark.gpu

# convolutions with even output extents; `kernel` is the fused kernel that must take the pair
CONV_POOL = [
    dict(n=3, c=1, h=28, w=28, oc=20, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], kernel="conv2d_im2col_maxpool_i8"),   # LeNet conv1: 576 pixels, three tiles
    dict(n=2, c=20, h=12, w=12, oc=50, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], kernel="conv2d_igemm_maxpool_i8"),   # LeNet conv2
    dict(n=2, c=3, h=31, w=27, oc=24, kh=3, kw=3, stride=[2, 2], dil=[1, 1], pad=[1, 1, 1, 1], kernel="conv2d_im2col_maxpool_i8"),   # stride 2, padding: 16 x 14
    dict(n=1, c=2, h=9, w=13, oc=70, kh=3, kw=2, stride=[1, 1], dil=[1, 2], pad=[1, 1, 2, 1], kernel="conv2d_im2col_maxpool_i8"),    # byte gather, three channel tiles
    dict(n=2, c=16, h=32, w=32, oc=40, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 1, 1], kernel="conv2d_igemm_maxpool_i8"),   # 1024 pixels: tiles of eight rows
    dict(n=3, c=24, h=14, w=14, oc=96, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], kernel="conv2d_igemm_maxpool_i8"),   # 12 x 12: tiles of 48 pixels, three channel tiles
    dict(n=1, c=40, h=8, w=12, oc=130, kh=1, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 0, 0], kernel="conv2d_igemm_maxpool_i8"),   # 8 x 12, two channel blocks
    dict(n=2, c=32, h=6, w=21, oc=32, kh=3, kw=3, stride=[2, 1], dil=[1, 1], pad=[0, 1, 1, 1], kernel="conv2d_igemm_maxpool_i8"),    # 6 x 10 from rows that are no whole dwords
]


def _descs(T, kws, act, keep):
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = kws["in_shape"]
    d.k_w, d.k_h = kws["w_shape"][0], kws["w_shape"][1]
    d.out_w, d.out_h, d.out_c = kws["out_shape"][:3]
    d.stride_w, d.stride_h = kws["stride"]
    d.dilation_w, d.dilation_h = kws["dilation"]
    d.pad_left, d.pad_top, d.multiplier = kws["pad_left"], kws["pad_top"], 0
    d.in_dtype, d.w_dtype, d.out_dtype = kws["in_dtype"], kws["w_dtype"], kws["out_dtype"]
    d.in_scale, d.in_zp = kws["in_q"]
    TC._wq(d, kws["w_q"], keep)
    d.out_scale, d.out_zp = kws["out_q"]
    d.activation = act
    p = T.Pool2dDesc()
    p.in_w, p.in_h, p.channels, p.batch = d.out_w, d.out_h, d.out_c, d.batch
    p.out_w, p.out_h = d.out_w // 2, d.out_h // 2
    p.k_w = p.k_h = p.stride_w = p.stride_h = 2
    p.pool_type, p.dtype = 0, d.out_dtype
    p.in_scale, p.in_zp = kws["out_q"]
    p.out_scale, p.out_zp = kws["out_q"]
    return d, p


@pytest.mark.parametrize("tile", [0, 32])   # 32: pixel tiles of eight pooled pixels, which end inside pooled rows
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("gi", range(len(CONV_POOL)))
def test_conv2d_with_fused_max_pool(oracle, gi, mode, tile, monkeypatch):
    if tile:
        if CONV_POOL[gi]["kernel"] != "conv2d_igemm_maxpool_i8" or mode == "u8pc":
            pytest.skip("the tile size is a lever of the implicit-GEMM kernel")
        monkeypatch.setenv("TVX_IGEMM_P", str(tile))
    g = dict(CONV_POOL[gi])
    kernel = g.pop("kernel")
    rng = np.random.default_rng(4000 + gi)
    x, w, b, kws = conv_case(rng, mult=0, mode=mode, **g)
    ow, oh, oc, n = kws["out_shape"]
    assert ow % 2 == 0 and oh % 2 == 0
    T = TC.tvx()
    import torch
    for act in (0, 2):
        t = oracle.conv2d(x, w, b, act=act, **kws)
        want = oracle.pool2d(t, in_shape=[ow, oh, oc, n], out_shape=[ow // 2, oh // 2, oc, n], ksize=[2, 2], stride=[2, 2],
                             pad_left=0, pad_top=0, pool_type=0, dtype=kws["out_dtype"], in_q=kws["out_q"], out_q=kws["out_q"])
        keep = []
        d, p = _descs(T, kws, act, keep)
        op = T.conv2d_pool_create(d, p, w, b)
        assert op.kernel_name == kernel, op.kernel_name
        xd = TC.to_device(x)
        yd = TC.device_out(want.size + 64, TC.NP_OF[kws["out_dtype"]])
        yd.fill_(77)
        op.run(xd, None, yd)
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        op.close()
        assert np.array_equal(got[:want.size], want), (gi, mode, act, np.flatnonzero(got[:want.size] != want)[:8])
        assert np.all(got[want.size:] == 77), "wrote past the pooled tensor"
    assert 0.02 < np.mean((want > want.min()) & (want < want.max())), "saturated test data"


def test_conv2d_pool_create_declines_what_it_does_not_fuse(oracle):
    rng = np.random.default_rng(7)
    T = TC.tvx()
    x, w, b, kws = conv_case(rng, n=1, c=1, h=28, w=28, oc=20, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0, mode="u8")
    keep = []
    d, p = _descs(T, kws, 0, keep)
    for field, value in (("pool_type", 1), ("k_w", 3), ("stride_h", 1), ("pad_left", 1), ("out_scale", 0.5), ("in_zp", 9)):
        d2, p2 = _descs(T, kws, 0, keep)
        setattr(p2, field, value)
        with pytest.raises(T.TvxError) as err:
            T.conv2d_pool_create(d2, p2, w, b)
        assert err.value.status == T.E_UNSUPPORTED, field
    # a pooling that does not read the convolution's output is a caller's mistake
    p.channels = 19
    with pytest.raises(T.TvxError) as err:
        T.conv2d_pool_create(d, p, w, b)
    assert err.value.status == T.E_INVALID
    # odd output extents (27 x 27), and a convolution neither fused kernel takes (depthwise)
    x, w, b, kws = conv_case(rng, n=1, c=1, h=31, w=31, oc=20, kh=5, kw=5, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0, mode="u8")
    d, p = _descs(T, kws, 0, keep)
    with pytest.raises(T.TvxError) as err:
        T.conv2d_pool_create(d, p, w, b)
    assert err.value.status == T.E_UNSUPPORTED
    x, w, b, kws = conv_case(rng, n=1, c=8, h=10, w=10, oc=0, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=[1, 1, 1, 1], mult=1, mode="u8")
    d, p = _descs(T, kws, 0, keep)
    d.multiplier = 1
    with pytest.raises(T.TvxError) as err:
        T.conv2d_pool_create(d, p, w, b)
    assert err.value.status == T.E_UNSUPPORTED


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("shape", [(1, 500, 10), (256, 500, 10), (7, 37, 3), (5, 1283, 16), (130, 64, 4), (3, 9, 1), (9, 130, 5)])
def test_fully_connected_with_fused_softmax(oracle, mode, shape):
    m, k, n = shape
    rng = np.random.default_rng(m * 11 + k)
    in_dt = 0 if mode.startswith("u8") else 1
    w_dt = 0 if mode == "u8" else 1
    x, w = rand_q(rng, m * k, in_dt), rand_q(rng, n * k, w_dt)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    wq = (0.01, 120, None) if mode == "u8" else \
        (1.0, 0, np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32))
    out_q = (float(np.float32(0.02 * 0.01 * 40 * np.sqrt(k))), 5 if in_dt == 0 else 0)
    kws = dict(m=m, k=k, n=n, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
               in_q=(0.02, 128 if in_dt == 0 else 0), w_q=wq, out_q=out_q)
    T = TC.tvx()
    import torch
    for act, beta in ((0, 1.0), (1, 0.3)):
        codes = oracle.fully_connected(x, w, b, act=act, **kws)
        if act == 0:
            assert len(np.unique(codes)) >= min(4, n), "saturated test data"
        want = oracle.softmax(in_dt, codes, n, beta, out_q)
        # the library's own two kernels
        two = TC.gpu_softmax(in_dt, TC.gpu_fully_connected(x, w, b, act=act, **kws), n, beta, out_q)
        d = T.FcDesc()
        d.m, d.k, d.n = m, k, n
        d.in_dtype, d.w_dtype, d.out_dtype = in_dt, w_dt, in_dt
        d.in_scale, d.in_zp = kws["in_q"]
        keep = []
        TC._wq(d, wq, keep)
        d.out_scale, d.out_zp = out_q
        d.activation = act
        s = T.SoftmaxDesc()
        s.channels, s.rows, s.beta, s.in_dtype, s.inner = n, m, beta, in_dt, 1
        s.in_scale, s.in_zp = out_q
        op = T.fully_connected_softmax_create(d, s, w, b)
        assert op.kernel_name == "fc_softmax_i8"
        xd = TC.to_device(x)
        yd = TC.device_out(m * n + 16, np.float32)
        yd.fill_(-5.0)
        op.run(xd, None, yd)
        torch.cuda.synchronize()
        got = yd.cpu().numpy()
        op.close()
        assert np.all(got[m * n:] == -5.0), "wrote past the result"
        got = got[:m * n]
        assert np.allclose(got, want, rtol=1e-4, atol=1e-9)
        assert np.array_equal(got, two), np.flatnonzero(got != two)[:8]
        assert np.allclose(got.reshape(m, n).sum(axis=1), 1.0, atol=1e-5)


def test_fully_connected_softmax_create_declines_what_it_does_not_fuse():
    T = TC.tvx()
    rng = np.random.default_rng(3)

    def descs(n=10, m=4, k=64):
        d = T.FcDesc()
        d.m, d.k, d.n = m, k, n
        d.in_dtype = d.w_dtype = d.out_dtype = 0
        d.in_scale, d.in_zp, d.w_scale, d.w_zp, d.out_scale, d.out_zp = 0.02, 128, 0.01, 120, 0.3, 5
        s = T.SoftmaxDesc()
        s.channels, s.rows, s.beta, s.in_dtype, s.inner = n, m, 1.0, 0, 1
        s.in_scale, s.in_zp = 0.3, 5
        return d, s

    w = rand_q(rng, 17 * 64, 0)
    d, s = descs(n=17)
    with pytest.raises(T.TvxError) as err:   # more outputs than the kernel keeps in a wavefront
        T.fully_connected_softmax_create(d, s, w, None)
    assert err.value.status == T.E_UNSUPPORTED
    d, s = descs()
    s.in_scale = 0.25
    with pytest.raises(T.TvxError) as err:   # the Softmax reads the codes under another scale
        T.fully_connected_softmax_create(d, s, w, None)
    assert err.value.status == T.E_UNSUPPORTED
    d, s = descs()
    s.rows = 5
    with pytest.raises(T.TvxError) as err:
        T.fully_connected_softmax_create(d, s, w, None)
    assert err.value.status == T.E_INVALID
    d, s = descs()
    with pytest.raises(T.TvxError) as err:   # weights that arrive at run time
        T.fully_connected_softmax_create(d, s, None, None)
    assert err.value.status == T.E_UNSUPPORTED
