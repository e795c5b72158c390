"""tvx_mbconv_create: an inverted-residual block (1x1 expansion, depthwise 3x3, 1x1 projection, residual Add) in
one kernel, against the oracle's operators one after the other, every intermediate quantized to its own tensor."""
import numpy as np
import pytest

import tvx_case as TC
from test_gpu_dwpw import _desc
from test_gpu_parity import conv_case, rand_q

pytestmark = pytest.mark.gpu

CASES = [
    # n, cin, cexp, cout, h, w, stride: the kernel's five plane shapes; chunk counts below, at and above the four
    # wavefronts; channel counts that are no multiples of 32; one, several and ten output tiles; heights that leave
    # a short last band
    (2, 64, 384, 64, 14, 14, 1),
    (3, 96, 576, 96, 14, 14, 1),
    (2, 64, 384, 96, 14, 14, 1),
    (2, 160, 960, 160, 7, 7, 1),
    (1, 160, 960, 320, 7, 7, 1),
    (2, 32, 192, 32, 28, 28, 1),
    (2, 32, 192, 64, 28, 28, 2),
    (2, 96, 576, 160, 14, 14, 2),
    (1, 24, 144, 40, 9, 14, 1),
    (2, 20, 72, 24, 5, 7, 1),
    (1, 16, 48, 16, 11, 28, 1),
    (2, 40, 100, 50, 10, 28, 2),
]


def _block(rng, n, cin, cexp, cout, h, w, stride, mode):
    x, w1, b1, k1 = conv_case(rng, n=n, c=cin, h=h, w=w, oc=cexp, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    pad = [1, 1, 1, 1] if stride == 1 else [0, 1, 0, 1]
    _, wd, bd, kd = conv_case(rng, n=n, c=cexp, h=h, w=w, oc=0, kh=3, kw=3, stride=[stride, stride], dil=[1, 1],
                              pad=pad, mult=1, mode=mode)
    oh, ow = kd["out_shape"][1], kd["out_shape"][0]
    _, w3, b3, k3 = conv_case(rng, n=n, c=cexp, h=oh, w=ow, oc=cout, kh=1, kw=1, stride=[1, 1], dil=[1, 1],
                              pad=[0, 0, 0, 0], mult=0, mode=mode)
    kd["in_q"] = k1["out_q"]
    k3["in_q"] = kd["out_q"]
    return x, (w1, b1, k1), (wd, bd, kd), (w3, b3, k3)


@pytest.mark.parametrize("with_add", [0, 1, 2], ids=["plain", "add_first", "add_second"])
@pytest.mark.parametrize("mode", ["u8", "i8pc", "u8pc"])
@pytest.mark.parametrize("ci", range(len(CASES)))
def test_inverted_residual_block(oracle, ci, mode, with_add, monkeypatch):
    import torch
    n, cin, cexp, cout, h, w, stride = CASES[ci]
    monkeypatch.setenv("TVX_MBCONV_ALL", "1")   # by default only the 14-column stride-1 blocks are taken
    rng = np.random.default_rng(8200 + ci)
    x, (w1, b1, k1), (wd, bd, kd), (w3, b3, k3) = _block(rng, n, cin, cexp, cout, h, w, stride, mode)
    e = oracle.conv2d(x, w1, b1, act=2, **k1)
    m = oracle.conv2d(e, wd, bd, act=2, **kd)
    want = oracle.conv2d(m, w3, b3, act=0, **k3)
    assert 0.02 < np.mean((e > e.min()) & (e < e.max())) and 0.02 < np.mean((m > m.min()) & (m < m.max()))
    T = TC.tvx()
    keep = []
    d1, d2, d3 = _desc(T, k1, 2, keep), _desc(T, kd, 2, keep), _desc(T, k3, 0, keep)
    dt = k3["out_dtype"]
    add, other = None, None
    if with_add:
        other = rand_q(rng, want.size, dt)
        other_q = (0.037, 121 if dt == 0 else -7)
        sum_q = (float(np.float32(k3["out_q"][0] * 1.3)), 119 if dt == 0 else 5)
        a, aq, b, bq = (want, k3["out_q"], other, other_q) if with_add == 1 else (other, other_q, want, k3["out_q"])
        want = oracle.add(dt, a, aq, b, bq, sum_q)
        add = T.EltwiseDesc()
        add.count, add.dtype = want.size, dt
        add.a_scale, add.a_zp = aq
        add.b_scale, add.b_zp = bq
        add.out_scale, add.out_zp = sum_q
    op = T.mbconv_create(d1, w1, b1, d2, wd, bd, d3, w3, b3, add, with_add)
    assert op.kernel_name == ("pwconv_dwconv3x3_pwconv_add_i8" if with_add else "pwconv_dwconv3x3_pwconv_i8")
    xd = TC.to_device(x)
    od = TC.to_device(other) if with_add else None
    yd = TC.device_out(want.size, TC.NP_OF[dt])
    op.run(xd, od, yd)
    torch.cuda.synchronize()
    got = yd.cpu().numpy()
    op.close()
    assert np.array_equal(got, want), (int((got != want).sum()), np.flatnonzero(got != want)[:8])
    assert 0.02 < np.mean((want > want.min()) & (want < want.max())), "saturated test data"


def test_blocks_without_a_fused_kernel_are_declined():
    T = TC.tvx()
    rng = np.random.default_rng(2)
    x, (w1, b1, k1), (wd, bd, kd), (w3, b3, k3) = _block(rng, 1, 16, 32, 16, 12, 12, 1, "u8")   # 12 columns
    keep = []
    with pytest.raises(T.TvxError) as err:
        T.mbconv_create(_desc(T, k1, 2, keep), w1, b1, _desc(T, kd, 2, keep), wd, bd, _desc(T, k3, 0, keep), w3, b3)
    assert err.value.status == T.E_UNSUPPORTED
