"""Operators on channel-blocked tensors (tvx_conv2d_blocked_create, tvx_pool2d_blocked_create, tvx_layout_create)
against the oracle: the blocked order is built and undone in numpy here, so that every kernel is checked on its own."""
import numpy as np
import pytest

import tvx_case as TC
from test_gpu_parity import conv_case, rand_q

pytestmark = pytest.mark.gpu


def to_blocked(x, n, c, hw):
    """[n][c][hw] codes -> [c / 16][n * hw][16]"""
    return np.ascontiguousarray(x.reshape(n, c // 16, 16, hw).transpose(1, 0, 3, 2)).ravel()


def from_blocked(y, n, c, hw):
    return np.ascontiguousarray(y.reshape(c // 16, n, hw, 16).transpose(1, 0, 3, 2)).ravel()


def _conv_desc(T, kws, act, keep):
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = kws["in_shape"]
    d.k_w, d.k_h = kws["w_shape"][0], kws["w_shape"][1]
    d.out_w, d.out_h, d.out_c = kws["out_shape"][:3]
    d.stride_w, d.stride_h = kws["stride"]
    d.dilation_w, d.dilation_h = kws["dilation"]
    d.pad_left, d.pad_top, d.multiplier = kws["pad_left"], kws["pad_top"], kws["multiplier"]
    d.in_dtype, d.w_dtype, d.out_dtype = kws["in_dtype"], kws["w_dtype"], kws["out_dtype"]
    d.in_scale, d.in_zp = kws["in_q"]
    TC._wq(d, kws["w_q"], keep)
    d.out_scale, d.out_zp = kws["out_q"]
    d.activation = act
    return d


def _run(op, x, out_elems, dtype, other=None):
    import torch
    xd = TC.to_device(x)
    od = TC.to_device(other) if other is not None else None
    yd = TC.device_out(out_elems, TC.NP_OF[dtype])
    op.run(xd, od, yd)
    torch.cuda.synchronize()
    out = yd.cpu().numpy()
    op.close()
    return out


@pytest.mark.parametrize("shape", [(3, 32, 7, 7), (2, 48, 5, 3), (1, 16, 1, 1), (5, 160, 7, 7), (1, 64, 14, 14)])
def test_layout_round_trip(shape):
    n, c, h, w = shape
    T = TC.tvx()
    rng = np.random.default_rng(c + h)
    x = rng.integers(0, 256, n * c * h * w, dtype=np.uint8)
    blocked = _run(T.layout_create(w, h, c, n, True), x, x.size, 0)
    assert np.array_equal(blocked, to_blocked(x, n, c, h * w))
    back = _run(T.layout_create(w, h, c, n, False), blocked, x.size, 0)
    assert np.array_equal(back, x)


PW_SHAPES = [
    # (n, c, side, oc): MobileNetV2's 7 x 7 stage and its edges
    (3, 160, 7, 960),    # expansion: short reduction, many channels (four pixel tiles a workgroup)
    (3, 960, 7, 160),    # projection: long reduction, few channels (the reduction split four ways)
    (2, 320, 7, 1280),
    (1, 32, 3, 32),      # nine pixels: less than a tile
    (5, 64, 5, 96),      # 125 pixels: a ragged last tile; three channel tiles in a group of four
    (2, 576, 7, 160),
    (1, 416, 4, 64),     # thirteen k-steps: wavefronts of the split form with four and with three of them
]


@pytest.mark.parametrize("form", [None, (0, 1), (0, 2), (0, 4), (1, 1), "records"], ids=str)
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("shape", PW_SHAPES, ids=lambda s: "x".join(map(str, s)))
def test_pointwise_conv_blocked(oracle, shape, mode, form, monkeypatch):
    n, c, side, oc = shape
    if form == "records":  # per-tensor quantization without the one-record-for-all-channels epilogue
        if mode != "u8":
            pytest.skip("per-channel scales never share a record")
        monkeypatch.setenv("TVX_BLOCKED_UNIFORM_RQ", "0")
    elif form is not None:   # (form, channel tiles per wavefront): every kernel shape on every problem
        monkeypatch.setenv("TVX_BLOCKED_PW_FORM", str(form[0]))
        monkeypatch.setenv("TVX_BLOCKED_PW_TILES", str(form[1]))
    rng = np.random.default_rng(c + oc + side)
    x, w, b, kws = conv_case(rng, n=n, c=c, h=side, w=side, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                             pad=[0, 0, 0, 0], mult=0, mode=mode)
    T = TC.tvx()
    hw = side * side
    for act in (0, 2):
        want = oracle.conv2d(x, w, b, act=act, **kws)
        keep = []
        op = T.conv2d_blocked_create(_conv_desc(T, kws, act, keep), w, b)
        assert op.kernel_name == "pwconv_blocked_i8"
        got = from_blocked(_run(op, to_blocked(x, n, c, hw), want.size, kws["out_dtype"]), n, oc, hw)
        assert np.array_equal(got, want), (shape, mode, act, np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("conv_operand", [1, 2])
@pytest.mark.parametrize("mode", ["u8", "i8pc"])
@pytest.mark.parametrize("shape", [(3, 960, 7, 160), (2, 64, 5, 96), (3, 160, 7, 960)], ids=lambda s: "x".join(map(str, s)))
def test_pointwise_conv_blocked_with_add(oracle, shape, mode, conv_operand):
    n, c, side, oc = shape
    rng = np.random.default_rng(c + oc + conv_operand)
    x, w, b, kws = conv_case(rng, n=n, c=c, h=side, w=side, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                             pad=[0, 0, 0, 0], mult=0, mode=mode)
    dt, conv_q, hw = kws["out_dtype"], kws["out_q"], side * side
    other = rand_q(rng, n * oc * hw, dt)
    other_q = (0.037, 121 if dt == 0 else -7)
    sum_q = (float(np.float32(conv_q[0] * 1.3)), 119 if dt == 0 else 5)
    t = oracle.conv2d(x, w, b, **kws)
    a, aq, bb, bq = (t, conv_q, other, other_q) if conv_operand == 1 else (other, other_q, t, conv_q)
    want = oracle.add(dt, a, aq, bb, bq, sum_q)
    T = TC.tvx()
    keep = []
    e = T.EltwiseDesc()
    e.count, e.dtype = want.size, dt
    e.a_scale, e.a_zp = aq
    e.b_scale, e.b_zp = bq
    e.out_scale, e.out_zp = sum_q
    op = T.conv2d_blocked_create(_conv_desc(T, kws, 0, keep), w, b, add_desc=e, conv_operand=conv_operand)
    assert op.kernel_name == "pwconv_add_blocked_i8"
    got = from_blocked(_run(op, to_blocked(x, n, c, hw), want.size, dt, other=to_blocked(other, n, oc, hw)), n, oc, hw)
    assert np.array_equal(got, want), np.flatnonzero(got != want)[:8]
    assert 0.05 < np.mean((want > want.min()) & (want < want.max()))


DW_SHAPES = [
    # (n, c, h, w, pad[l,r,t,b])
    (3, 960, 7, 7, [1, 1, 1, 1]),
    (2, 32, 7, 7, [1, 1, 1, 1]),
    (1, 16, 1, 1, [1, 1, 1, 1]),     # a single pixel: eight of nine taps are padding
    (2, 48, 5, 9, [0, 0, 0, 0]),     # VALID
    (1, 64, 14, 14, [1, 1, 1, 1]),
    (3, 16, 6, 4, [1, 2, 0, 1]),     # uneven pads: the output is wider than the input
]


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("shape", DW_SHAPES, ids=lambda s: "x".join(map(str, s[:4])))
def test_depthwise_conv_blocked(oracle, shape, mode):
    n, c, h, w, pad = shape
    rng = np.random.default_rng(c + h * w)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[1, 1], dil=[1, 1], pad=pad, mult=1, mode=mode)
    T = TC.tvx()
    ow, oh = kws["out_shape"][0], kws["out_shape"][1]
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        keep = []
        op = T.conv2d_blocked_create(_conv_desc(T, kws, act, keep), wt, b)
        assert op.kernel_name == "dwconv3x3_blocked_i8"
        got = from_blocked(_run(op, to_blocked(x, n, c, h * w), want.size, kws["out_dtype"]), n, c, ow * oh)
        assert np.array_equal(got, want), (shape, mode, act, np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 3


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("shape", [(4, 1280, 7, 7), (3, 32, 16, 16), (2, 48, 3, 5), (65, 16, 2, 2)], ids=lambda s: "x".join(map(str, s)))
def test_global_average_pool_blocked(oracle, shape, dtype):
    n, c, h, w = shape
    rng = np.random.default_rng(c + h)
    x = rand_q(rng, n * c * h * w, dtype)
    T = TC.tvx()
    for out_q in ((0.1, 7), (0.07, 9 if dtype == 0 else -2)):
        kws = dict(in_shape=[w, h, c, n], out_shape=[1, 1, c, n], ksize=[w, h], stride=[1, 1], pad_left=0, pad_top=0,
                   pool_type=1, dtype=dtype)
        want = oracle.pool2d(x, in_q=(0.1, 7), out_q=out_q, **kws)
        d = T.Pool2dDesc()
        d.in_w, d.in_h, d.channels, d.batch = w, h, c, n
        d.out_w = d.out_h = 1
        d.k_w, d.k_h = w, h
        d.stride_w = d.stride_h = 1
        d.pool_type, d.dtype = 1, dtype
        d.in_scale, d.in_zp = 0.1, 7
        d.out_scale, d.out_zp = out_q
        op = T.pool2d_blocked_create(d)
        assert op.kernel_name == "avgpool_blocked_i8"
        got = _run(op, to_blocked(x, n, c, h * w), want.size, dtype)
        assert np.array_equal(got, want), np.flatnonzero(got != want)[:8]


def test_blocked_operators_decline_what_they_do_not_cover():
    T = TC.tvx()
    rng = np.random.default_rng(5)
    x, w, b, kws = conv_case(rng, n=1, c=24, h=7, w=7, oc=32, kh=1, kw=1, stride=[1, 1], dil=[1, 1], pad=[0, 0, 0, 0], mult=0, mode="u8")
    keep = []
    with pytest.raises(T.TvxError) as err:   # 24 input channels
        T.conv2d_blocked_create(_conv_desc(T, kws, 0, keep), w, b)
    assert err.value.status == T.E_UNSUPPORTED
    with pytest.raises(T.TvxError) as err:   # 24 channels
        T.layout_create(7, 7, 24, 1, True)
    assert err.value.status == T.E_UNSUPPORTED


@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("shape", [(3, 576, 14, 14, 2, [0, 1, 0, 1]), (2, 32, 7, 7, 1, [1, 1, 1, 1]), (1, 48, 9, 6, 2, [1, 1, 1, 1]),
                                   (2, 16, 5, 13, 1, [1, 1, 1, 1]), (1, 64, 28, 28, 2, [0, 1, 0, 1])],
                         ids=lambda s: "x".join(map(str, s[:5])))
def test_depthwise_conv_writing_blocked(oracle, shape, mode):
    """tvx_conv2d_to_blocked_create: WHCN in, blocked out - the way into a run of blocked operators."""
    n, c, h, w, stride, pad = shape
    rng = np.random.default_rng(c * 3 + h + stride)
    x, wt, b, kws = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[stride, stride], dil=[1, 1], pad=pad,
                              mult=1, mode=mode)
    T = TC.tvx()
    ohw = kws["out_shape"][0] * kws["out_shape"][1]
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        keep = []
        op = T.conv2d_to_blocked_create(_conv_desc(T, kws, act, keep), wt, b)
        assert op.kernel_name == "dwconv_planes_to_blocked_i8"
        got = from_blocked(_run(op, x, want.size, kws["out_dtype"]), n, c, ohw)
        assert np.array_equal(got, want), (shape, mode, act, np.flatnonzero(got != want)[:8])
    assert len(np.unique(want)) > 4


def test_conv2d_to_blocked_create_declines_other_convolutions():
    T = TC.tvx()
    rng = np.random.default_rng(6)
    for kw in (dict(c=24, oc=0, kh=3, kw=3, mult=1, pad=[1, 1, 1, 1]),     # channels that do not fill 16-channel blocks
               dict(c=32, oc=0, kh=5, kw=5, mult=1, pad=[2, 2, 2, 2]),     # another window
               dict(c=32, oc=32, kh=1, kw=1, mult=0, pad=[0, 0, 0, 0])):  # not depthwise
        x, wt, b, kws = conv_case(rng, n=1, h=7, w=7, stride=[1, 1], dil=[1, 1], mode="u8", **kw)
        keep = []
        with pytest.raises(T.TvxError) as err:
            T.conv2d_to_blocked_create(_conv_desc(T, kws, 0, keep), wt, b)
        assert err.value.status == T.E_UNSUPPORTED
