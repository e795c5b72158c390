"""tvx_conv2d_dw_pw_create: a depthwise 3x3 convolution and the 1x1 convolution behind it in one kernel, against
the oracle's two operators one after the other (the depthwise result quantized to its own tensor first), with
and without the residual Add behind the pointwise convolution."""
import numpy as np
import pytest

import tvx_case as TC
from test_gpu_parity import conv_case, rand_q

pytestmark = pytest.mark.gpu

CASES = [
    # n, c, h, w, oc, stride: tiles of 1, 2 and 4 output rows, channel counts that are no multiples of 32 / 16,
    # output channels that leave a ragged last tile, one and several output tiles per wavefront
    (2, 32, 16, 16, 64, 1),
    (2, 16, 112, 112, 24, 1),
    (1, 96, 112, 112, 24, 2),
    (2, 144, 56, 56, 24, 1),
    (1, 144, 56, 56, 32, 2),
    (2, 192, 28, 28, 32, 1),
    (3, 40, 8, 8, 200, 1),
    (2, 24, 32, 64, 40, 2),
    (1, 5, 4, 4, 3, 1),
]


def _desc(T, kws, act, keep):
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = kws["in_shape"]
    d.k_w, d.k_h = kws["w_shape"][0], kws["w_shape"][1]
    d.out_w, d.out_h, d.out_c = kws["out_shape"][:3]
    d.stride_w, d.stride_h = kws["stride"]
    d.dilation_w = d.dilation_h = 1
    d.pad_left, d.pad_top, d.multiplier = kws["pad_left"], kws["pad_top"], kws["multiplier"]
    d.in_dtype, d.w_dtype, d.out_dtype = kws["in_dtype"], kws["w_dtype"], kws["out_dtype"]
    d.in_scale, d.in_zp = kws["in_q"]
    TC._wq(d, kws["w_q"], keep)
    d.out_scale, d.out_zp = kws["out_q"]
    d.activation = act
    return d


def _pair(rng, n, c, h, w, oc, stride, mode):
    pad = [1, 1, 1, 1] if stride == 1 else [0, 1, 0, 1]   # SAME
    x, wd, bd, kd = conv_case(rng, n=n, c=c, h=h, w=w, oc=0, kh=3, kw=3, stride=[stride, stride], dil=[1, 1],
                              pad=pad, mult=1, mode=mode)
    oh, ow = kd["out_shape"][1], kd["out_shape"][0]
    _, wp, bp, kp = conv_case(rng, n=n, c=c, h=oh, w=ow, oc=oc, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    kp["in_q"] = kd["out_q"]   # the pointwise convolution reads the depthwise result
    return x, wd, bd, kd, wp, bp, kp


@pytest.mark.parametrize("with_add", [0, 1, 2], ids=["plain", "add_first", "add_second"])
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("ci", range(len(CASES)))
def test_depthwise_pointwise_fused(oracle, ci, mode, with_add):
    import torch
    n, c, h, w, oc, stride = CASES[ci]
    rng = np.random.default_rng(8000 + ci)
    x, wd, bd, kd, wp, bp, kp = _pair(rng, n, c, h, w, oc, stride, mode)
    dw_act, pw_act = 2, (0 if with_add else 2)
    mid = oracle.conv2d(x, wd, bd, act=dw_act, **kd)
    want = oracle.conv2d(mid, wp, bp, act=pw_act, **kp)
    T = TC.tvx()
    keep = []
    ddw, dpw = _desc(T, kd, dw_act, keep), _desc(T, kp, pw_act, keep)
    dt = kp["out_dtype"]
    e, other = None, None
    if with_add:
        other = rand_q(rng, want.size, dt)
        other_q = (0.037, 121 if dt == 0 else -7)
        sum_q = (float(np.float32(kp["out_q"][0] * 1.3)), 119 if dt == 0 else 5)
        a, aq, b, bq = (want, kp["out_q"], other, other_q) if with_add == 1 else (other, other_q, want, kp["out_q"])
        want = oracle.add(dt, a, aq, b, bq, sum_q)
        e = T.EltwiseDesc()
        e.count, e.dtype = want.size, dt
        e.a_scale, e.a_zp = aq
        e.b_scale, e.b_zp = bq
        e.out_scale, e.out_zp = sum_q
    op = T.conv2d_dw_pw_create(ddw, wd, bd, dpw, wp, bp, e, with_add)
    assert op.kernel_name == ("dwconv3x3_pwconv_add_i8" if with_add else "dwconv3x3_pwconv_i8")
    xd = TC.to_device(x)
    od = TC.to_device(other) if with_add else None
    yd = TC.device_out(want.size, TC.NP_OF[dt])
    op.run(xd, od, yd)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    op.close()
    assert np.array_equal(got, want), (int((got != want).sum()), np.flatnonzero(got != want)[:8])
    assert 0.02 < np.mean((want > want.min()) & (want < want.max())), "saturated test data"


def test_depthwise_pointwise_fused_full_size(oracle):
    """The int8 per-channel block at its full size: depthwise 3x3 on 112x112x32 at batch 32, pointwise 32 -> 64
    with ReLU6, one kernel, whole output against the oracle's two operators."""
    import torch
    rng = np.random.default_rng(0x73)
    n, c, h, w, oc = 32, 32, 112, 112, 64
    x = rng.integers(-128, 128, n * c * h * w, dtype=np.int8)
    wd = rng.integers(-128, 128, c * 9, dtype=np.int8)
    bd = rng.integers(-4096, 4097, c).astype(np.int32)
    sd = np.exp(rng.uniform(np.log(0.002), np.log(0.05), c)).astype(np.float32)
    kd = dict(in_shape=[w, h, c, n], w_shape=[3, 3, c, 1], out_shape=[w, h, c, n], stride=[1, 1],
              dilation=[1, 1], pad_left=1, pad_top=1, multiplier=1, in_dtype=1, w_dtype=1, out_dtype=1,
              in_q=(0.03, 0), w_q=(1.0, 0, sd), out_q=(0.08, 0))
    wp = rng.integers(-128, 128, oc * c, dtype=np.int8)
    bp = rng.integers(-4096, 4097, oc).astype(np.int32)
    sp = np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32)
    kp = dict(in_shape=[w, h, c, n], w_shape=[1, 1, c, oc], out_shape=[w, h, oc, n], stride=[1, 1],
              dilation=[1, 1], pad_left=0, pad_top=0, multiplier=0, in_dtype=1, w_dtype=1, out_dtype=1,
              in_q=(0.08, 0), w_q=(1.0, 0, sp), out_q=(0.05, 0))
    want = oracle.conv2d(oracle.conv2d(x, wd, bd, **kd), wp, bp, act=2, **kp)
    T = TC.tvx()
    keep = []
    op = T.conv2d_dw_pw_create(_desc(T, kd, 0, keep), wd, bd, _desc(T, kp, 2, keep), wp, bp)
    assert op.kernel_name == "dwconv3x3_pwconv_i8"
    xd = TC.to_device(x)
    yd = TC.device_out(want.size, np.int8)
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    op.close()
    assert np.array_equal(got, want), int((got != want).sum())
    assert want.min() == 0 and want.max() == 120


@pytest.mark.parametrize("mode", ["u8", "i8pc"])
def test_fused_pair_rounds_ties_to_even(oracle, mode):
    """Both requantizations of the fused kernel on exact .5 cases: multipliers odd * 2^-e, ties counted from the
    accumulators themselves (as the tie tests of the single operators do)."""
    import torch
    import torch.nn.functional as F
    from test_gpu_ties import _count_ties, _multipliers, _operands
    rng = np.random.default_rng(8100)
    u8 = mode == "u8"
    n, c, h, w, oc = 2, 32, 16, 16, 64
    zx, zw, zm, zo = (128, 120, 101, 99) if u8 else (-3, 0, 7, -5)
    dt = 0 if u8 else 1
    x, wd = _operands(rng, u8, 15, 7, n * c * h * w, c * 9, zx, zw)
    bd = rng.integers(-300, 301, c).astype(np.int32)
    acc_d = F.conv2d(torch.from_numpy(x.reshape(n, c, h, w).astype(np.float64) - zx),
                     torch.from_numpy(wd.reshape(c, 1, 3, 3).astype(np.float64) - zw),
                     torch.from_numpy(bd.astype(np.float64)), padding=1, groups=c).numpy().astype(np.int64)
    ed = max(3, int(np.round(np.log2(max(acc_d.std(), 1.0) / 12.0))))
    md = _multipliers(not u8, c, ed)
    kd = dict(in_shape=[w, h, c, n], w_shape=[3, 3, 1, c], out_shape=[w, h, c, n], stride=[1, 1], dilation=[1, 1],
              pad_left=1, pad_top=1, multiplier=1, in_dtype=dt, w_dtype=dt, out_dtype=dt, in_q=(0.5, zx),
              w_q=(float(2 * md[0]), zw, None) if u8 else (1.0, 0, (2 * md).astype(np.float32)), out_q=(1.0, zm))
    qlo, qhi = (0, 255) if u8 else (-128, 127)
    ties_d = sum(_count_ties(oracle, acc_d[:, ch], float(md[ch]), qlo, qhi, zm) for ch in range(c))
    mid = oracle.conv2d(x, wd, bd, act=0, **kd)
    _, wp = _operands(rng, u8, 1, 7, 1, oc * c, zx, zw)
    bp = rng.integers(-300, 301, oc).astype(np.int32)
    acc_p = np.einsum("nchw,oc->nohw", mid.reshape(n, c, h, w).astype(np.int64) - zm,
                      wp.reshape(oc, c).astype(np.int64) - zw) + bp[None, :, None, None]
    ep = max(3, int(np.round(np.log2(max(acc_p.std(), 1.0) / 12.0))))
    mp = _multipliers(not u8, oc, ep)
    kp = dict(in_shape=[w, h, c, n], w_shape=[1, 1, c, oc], out_shape=[w, h, oc, n], stride=[1, 1], dilation=[1, 1],
              pad_left=0, pad_top=0, multiplier=0, in_dtype=dt, w_dtype=dt, out_dtype=dt, in_q=(1.0, zm),
              w_q=(float(mp[0]), zw, None) if u8 else (1.0, 0, mp.astype(np.float32)), out_q=(1.0, zo))
    ties_p = sum(_count_ties(oracle, acc_p[:, ch], float(mp[ch]), qlo, qhi, zo) for ch in range(oc))
    assert ties_d >= 10 and ties_p >= 10, (ties_d, ties_p)
    want = oracle.conv2d(mid, wp, bp, act=0, **kp)
    T = TC.tvx()
    keep = []
    op = T.conv2d_dw_pw_create(_desc(T, kd, 0, keep), wd, bd, _desc(T, kp, 0, keep), wp, bp)
    assert op.kernel_name == "dwconv3x3_pwconv_i8"
    xd = TC.to_device(x)
    yd = TC.device_out(want.size, TC.NP_OF[dt])
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    op.close()
    assert np.array_equal(got, want), (int((got != want).sum()), ties_d, ties_p)
    assert len(np.unique(want)) > 4


def test_pairs_without_a_fused_kernel_are_declined():
    T = TC.tvx()
    rng = np.random.default_rng(1)
    x, wd, bd, kd, wp, bp, kp = _pair(rng, 1, 16, 14, 14, 32, 1, "u8")   # 14 columns: rows are no whole dwords
    keep = []
    with pytest.raises(T.TvxError) as err:
        T.conv2d_dw_pw_create(_desc(T, kd, 2, keep), wd, bd, _desc(T, kp, 0, keep), wp, bp)
    assert err.value.status == T.E_UNSUPPORTED
