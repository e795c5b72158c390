"""Independent checks that pin what the golden vectors leave open: the fixed-point
requantization against exact rational arithmetic, ties, and the conv / FC / pool
restatement against brute-force numpy on random tensors."""
from fractions import Fraction

import numpy as np
import pytest


def rne_fraction(fr):
    fl = fr.numerator // fr.denominator
    rem = fr - fl
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and fl % 2 == 1):
        fl += 1
    return fl


def test_quantize_multiplier_is_within_2_pow_minus_31(oracle):
    rng = np.random.default_rng(1)
    for m in list(10.0 ** rng.uniform(-9, 2, 300)) + [0.25, 0.5, 1.0, 2.0, 3.0, 4.0, 1.0058823529]:
        mult, shift = oracle.quantize_multiplier(float(m))
        assert 2 ** 30 <= mult < 2 ** 31
        approx = Fraction(mult, 2 ** shift) if shift >= 0 else Fraction(mult * 2 ** (-shift))
        assert abs(approx / Fraction(float(m)) - 1) <= Fraction(1, 2 ** 31)


def test_requant_is_exact_rne_of_the_fixed_point_product(oracle):
    rng = np.random.default_rng(2)
    for _ in range(2000):
        acc = int(rng.integers(-2 ** 31, 2 ** 31))
        mult = int(rng.integers(2 ** 30, 2 ** 31))
        shift = int(rng.integers(1, 63))
        assert oracle.requant(acc, mult, shift) == rne_fraction(Fraction(acc * mult, 2 ** shift))


def test_requant_ties_go_to_even(oracle):
    # M = 0.5 exactly: odd accumulators land on .5
    mult, shift = oracle.quantize_multiplier(0.5)
    got = [oracle.requant(a, mult, shift) for a in (-5, -3, -1, 1, 3, 5, 7)]
    assert got == [-2, -2, 0, 0, 2, 2, 4]
    # powers of two are exact
    for m in (0.25, 1.0, 2.0, 4.0):
        mult, shift = oracle.quantize_multiplier(m)
        for a in (-1000, -7, 0, 4, 12345):
            assert oracle.requant(a, mult, shift) == rne_fraction(Fraction(a) * Fraction(m))


def brute_conv(x, w, bias, stride, dil, pad_l, pad_t, out_w, out_h, multiplier):
    """x [N,C,H,W], w [Oc,Icg,Kh,Kw] integer arrays -> int64 accumulators [N,Oc,Ho,Wo]."""
    n, c, h, wd = x.shape
    oc, icg, kh, kw = w.shape
    acc = np.zeros((n, oc, out_h, out_w), dtype=np.int64)
    for o in range(oc):
        for ci in range(icg):
            ic = (o // multiplier) if multiplier > 0 else ci
            for ky in range(kh):
                for kx in range(kw):
                    for oh in range(out_h):
                        ih = oh * stride[1] - pad_t + ky * dil[1]
                        if ih < 0 or ih >= h:
                            continue
                        for ow in range(out_w):
                            iw = ow * stride[0] - pad_l + kx * dil[0]
                            if iw < 0 or iw >= wd:
                                continue
                            acc[:, o, oh, ow] += x[:, ic, ih, iw] * w[o, ci, ky, kx]
    if bias is not None:
        acc += bias[None, :, None, None]
    return acc


@pytest.mark.parametrize("seed", range(6))
def test_conv_restatement_vs_bruteforce(oracle, seed):
    rng = np.random.default_rng(100 + seed)
    u8 = seed % 2 == 0
    depthwise = seed % 3 == 2
    n, c, h, wd = 2, 4, int(rng.integers(5, 9)), int(rng.integers(5, 9))
    kh, kw = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    stride = [int(rng.integers(1, 3)), int(rng.integers(1, 3))]
    dil = [int(rng.integers(1, 3)), int(rng.integers(1, 3))]
    pad_l, pad_t = int(rng.integers(0, 3)), int(rng.integers(0, 3))
    mult = 2 if depthwise else 0
    oc = c * mult if depthwise else 5
    icg = 1 if depthwise else c
    out_w = (wd + 2 * pad_l - ((kw - 1) * dil[0] + 1)) // stride[0] + 1
    out_h = (h + 2 * pad_t - ((kh - 1) * dil[1] + 1)) // stride[1] + 1
    if u8:
        x = rng.integers(0, 256, (n, c, h, wd)).astype(np.uint8)
        w = rng.integers(0, 256, (oc, icg, kh, kw)).astype(np.uint8)
        zx, zw, zo = 128, 120, 3
        w_scales = None
        in_dt = w_dt = oracle.U8
    else:
        x = rng.integers(-128, 128, (n, c, h, wd)).astype(np.int8)
        w = rng.integers(-128, 128, (oc, icg, kh, kw)).astype(np.int8)
        zx, zw, zo = -5, 0, -7
        w_scales = np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32)
        in_dt = w_dt = oracle.I8
    bias = rng.integers(-4096, 4097, oc).astype(np.int32)
    s_in, s_w, s_out = np.float32(0.05), np.float32(0.01), np.float32(0.11)
    acc = brute_conv(x.astype(np.int64) - zx, w.astype(np.int64) - zw, bias.astype(np.int64),
                     stride, dil, pad_l, pad_t, out_w, out_h, mult)
    qmin, qmax = (0, 255) if u8 else (-128, 127)
    want = np.zeros_like(acc)
    for o in range(oc):
        sw = float(w_scales[o]) if w_scales is not None else float(s_w)
        m, sh = oracle.quantize_multiplier(float(s_in) * sw / float(s_out))
        flat = [min(qmax, max(qmin, rne_fraction(Fraction(int(a) * m, 2 ** sh)) + zo))
                for a in acc[:, o].ravel()]
        want[:, o] = np.asarray(flat).reshape(acc[:, o].shape)
    got = oracle.conv2d(x.ravel(), w.ravel(), bias, in_shape=[wd, h, c, n], w_shape=[kw, kh, icg, oc],
                        out_shape=[out_w, out_h, oc, n], stride=stride, dilation=dil, pad_left=pad_l,
                        pad_top=pad_t, multiplier=mult, in_dtype=in_dt, w_dtype=w_dt, out_dtype=in_dt,
                        in_q=(float(s_in), zx), w_q=(float(s_w), zw, w_scales), out_q=(float(s_out), zo))
    assert np.array_equal(got.astype(np.int64), want.ravel())


def test_conv_matches_torch_conv2d_on_dequantized_integers(oracle):
    # textbook reduction: the int32 accumulator equals F.conv2d on (x - zx), (w - zw)
    import torch
    import torch.nn.functional as F
    rng = np.random.default_rng(7)
    n, c, h, wd, oc, k = 2, 8, 9, 10, 6, 3
    x = rng.integers(0, 256, (n, c, h, wd)).astype(np.uint8)
    w = rng.integers(0, 256, (oc, c, k, k)).astype(np.uint8)
    bias = rng.integers(-500, 500, oc).astype(np.int32)
    zx, zw = 128, 120
    acc = F.conv2d(torch.from_numpy(x.astype(np.float64) - zx), torch.from_numpy(w.astype(np.float64) - zw),
                   torch.from_numpy(bias.astype(np.float64)), stride=1, padding=1).numpy()
    # scale chosen so requant is the identity: out = acc (then clamp)
    got = oracle.conv2d(x.ravel(), w.ravel(), bias, in_shape=[wd, h, c, n], w_shape=[k, k, c, oc],
                        out_shape=[wd, h, oc, n], stride=[1, 1], dilation=[1, 1], pad_left=1, pad_top=1,
                        multiplier=0, in_dtype=oracle.U8, w_dtype=oracle.U8, out_dtype=oracle.U8,
                        in_q=(1.0, zx), w_q=(2.0 ** -12, zw, None), out_q=(1.0, 100))
    want = np.clip(np.array([rne_fraction(Fraction(int(a), 4096)) for a in acc.ravel()]) + 100, 0, 255)
    assert np.array_equal(got.astype(np.int64), want)


def test_fc_restatement_vs_numpy(oracle):
    rng = np.random.default_rng(11)
    m, k, n = 7, 33, 9
    x = rng.integers(-128, 128, (m, k)).astype(np.int8)
    w = rng.integers(-128, 128, (n, k)).astype(np.int8)
    bias = rng.integers(-16384, 16385, n).astype(np.int32)
    ws = np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32)
    s_in, s_out, zx, zo = np.float32(0.02), np.float32(0.05), 3, -4
    acc = (x.astype(np.int64) - zx) @ w.astype(np.int64).T + bias
    want = np.zeros((m, n), dtype=np.int64)
    for j in range(n):
        mu, sh = oracle.quantize_multiplier(float(s_in) * float(ws[j]) / float(s_out))
        want[:, j] = [min(127, max(-128, rne_fraction(Fraction(int(a) * mu, 2 ** sh)) + zo)) for a in acc[:, j]]
    got = oracle.fully_connected(x.ravel(), w.ravel(), bias, m=m, k=k, n=n, in_dtype=oracle.I8,
                                 w_dtype=oracle.I8, out_dtype=oracle.I8, in_q=(float(s_in), zx),
                                 w_q=(1.0, 0, ws), out_q=(float(s_out), zo))
    assert np.array_equal(got.astype(np.int64), want.ravel())


def _f32(v):
    """The exact rational value of a float32 number (scales travel as float32)."""
    return Fraction(float(np.float32(v)))


def _closed_form_activation(q, act, qmin, qmax, s_in, z_in, s_out, z_out, oracle):
    """Textbook definition, exact: dequantize, clamp to [0, inf) or [0, 6] in the real domain, divide by the
    output scale, round half to even, add the zero point, saturate. The only thing taken from the oracle is the
    Q31 image of s_in / s_out (pinned on its own above): the real value is (q - z_in) * mult * 2^-shift output
    quanta, six real units are 6 / s_out of them."""
    mult, shift = oracle.quantize_multiplier(float(np.float32(s_in)) / float(np.float32(s_out)))
    v = Fraction((int(q) - z_in) * mult, 2 ** shift)
    if act in ("RELU", "RELU6"):
        v = max(v, Fraction(0))
    if act == "RELU6":
        v = min(v, Fraction(6) / _f32(s_out))
    return min(qmax, max(qmin, rne_fraction(v) + z_out))


@pytest.mark.parametrize("dtype_name,z_in,z_out", [("U8", 117, 9), ("U8", 3, 131), ("I8", -11, -100), ("I8", 20, 5)])
@pytest.mark.parametrize("s_in,s_out", [(0.07, 0.07), (0.05, 0.023), (0.023, 0.07), (0.11, 0.047), (0.5, 0.25),
                                         (0.25, 0.5), (3.0, 4.0)])
@pytest.mark.parametrize("act", ["RELU", "RELU6"])
def test_activation_restatement_vs_closed_form(oracle, dtype_name, z_in, z_out, s_in, s_out, act):
    # 6 / 0.07 = 85.71, 6 / 0.023 = 260.87, 6 / 0.047 = 127.66, 6 / 4 = 1.5 (a tie: half-even gives 2):
    # floor instead of round-to-nearest, a bound at zero instead of the zero point, or clamping the rounded
    # value to the wrong side of the requantization all change codes here. 0.25 -> 0.5 and 3 -> 4 put odd
    # inputs on exact .5 ties.
    u8 = dtype_name == "U8"
    dt = oracle.U8 if u8 else oracle.I8
    qmin, qmax = (0, 255) if u8 else (-128, 127)
    q = np.arange(qmin, qmax + 1).astype(np.uint8 if u8 else np.int8)
    got = oracle.activation(oracle.ACT_RELU if act == "RELU" else oracle.ACT_RELU6, dt, q,
                            (s_in, z_in), (s_out, z_out))
    want = [_closed_form_activation(v, act, qmin, qmax, s_in, z_in, s_out, z_out, oracle) for v in q]
    assert got.astype(np.int64).tolist() == want
    assert len(set(want)) > 2  # the case is not saturated flat


def test_activation_ties_and_bounds_by_hand(oracle):
    # s_in 0.25 -> s_out 0.5, zero points 10 -> 3: real = (q - 10) / 4, quanta = (q - 10) / 2
    q = np.array([10, 11, 12, 13, 15, 9, 0, 34, 35, 36, 255], dtype=np.uint8)
    # quanta:      0  .5   1  1.5 2.5 -.5 -5  12 12.5 13  122.5 ; six real units = 12 quanta
    relu = oracle.activation(oracle.ACT_RELU, oracle.U8, q, (0.25, 10), (0.5, 3))
    assert relu.tolist() == [3, 3, 4, 5, 5, 3, 3, 15, 15, 16, 125]      # .5 -> 0, 1.5 -> 2, 2.5 -> 2, 12.5 -> 12, 122.5 -> 122
    relu6 = oracle.activation(oracle.ACT_RELU6, oracle.U8, q, (0.25, 10), (0.5, 3))
    assert relu6.tolist() == [3, 3, 4, 5, 5, 3, 3, 15, 15, 15, 15]
    # int8, negative zero point, upper bound beyond the type: 6 / 0.02 = 300 quanta -> saturates at 127
    qi = np.array([-128, -101, -100, -99, 0, 127], dtype=np.int8)
    r6 = oracle.activation(oracle.ACT_RELU6, oracle.I8, qi, (0.02, -100), (0.02, -100))
    assert r6.tolist() == [-100, -100, -100, -99, 0, 127]
    # upper bound inside the type with a non-integer quotient: 6 / 0.07 = 85.71 -> 86 quanta above the zero point
    r6 = oracle.activation(oracle.ACT_RELU6, oracle.I8, qi, (0.07, -100), (0.07, -100))
    assert r6.tolist() == [-100, -100, -100, -99, -14, -14]


@pytest.mark.parametrize("seed", range(4))
def test_fused_activation_on_conv_vs_closed_form(oracle, seed):
    # the fused epilogue, output zero point != 0, checked through brute-force accumulators and exact rationals
    rng = np.random.default_rng(500 + seed)
    u8 = seed % 2 == 0
    n, c, h, wd, oc = 1, 5, 6, 7, 4
    qmin, qmax = (0, 255) if u8 else (-128, 127)
    npdt = np.uint8 if u8 else np.int8
    x = rng.integers(qmin, qmax + 1, (n, c, h, wd)).astype(npdt)
    w = rng.integers(qmin, qmax + 1, (oc, c, 3, 3)).astype(npdt)
    bias = rng.integers(-4096, 4097, oc).astype(np.int32)
    zx, zw, zo = (128, 120, 17) if u8 else (-5, 0, -90)
    s_in, s_w, s_out = 0.05, 0.01, [0.07, 0.023, 0.047, 0.11][seed]
    acc = brute_conv(x.astype(np.int64) - zx, w.astype(np.int64) - zw, bias.astype(np.int64),
                     [1, 1], [1, 1], 1, 1, wd, h, 0)
    mult, shift = oracle.quantize_multiplier(float(np.float32(s_in)) * float(np.float32(s_w)) / float(np.float32(s_out)))
    for act_name, act in (("RELU", oracle.ACT_RELU), ("RELU6", oracle.ACT_RELU6)):
        want = []
        for a in acc.ravel():
            v = max(Fraction(int(a) * mult, 2 ** shift), Fraction(0))
            if act_name == "RELU6":
                v = min(v, Fraction(6) / _f32(s_out))
            want.append(min(qmax, max(qmin, rne_fraction(v) + zo)))
        dt = oracle.U8 if u8 else oracle.I8
        got = oracle.conv2d(x.ravel(), w.ravel(), bias, in_shape=[wd, h, c, n], w_shape=[3, 3, c, oc],
                            out_shape=[wd, h, oc, n], stride=[1, 1], dilation=[1, 1], pad_left=1, pad_top=1,
                            multiplier=0, in_dtype=dt, w_dtype=dt, out_dtype=dt, in_q=(s_in, zx),
                            w_q=(s_w, zw, None), out_q=(s_out, zo), act=act)
        assert got.astype(np.int64).tolist() == want
        assert min(want) == max(qmin, zo) and len(set(want)) > 3   # both the lower bound and the interior occur
    # and the same on FullyConnected (int8 per-channel)
    if not u8:
        m, k, nn = 5, 19, 6
        xf = rng.integers(-128, 128, (m, k)).astype(np.int8)
        wf = rng.integers(-128, 128, (nn, k)).astype(np.int8)
        bf = rng.integers(-3000, 3000, nn).astype(np.int32)
        ws = np.exp(rng.uniform(np.log(0.001), np.log(0.02), nn)).astype(np.float32)
        accf = (xf.astype(np.int64) - 4) @ wf.astype(np.int64).T + bf
        got = oracle.fully_connected(xf.ravel(), wf.ravel(), bf, m=m, k=k, n=nn, in_dtype=oracle.I8, w_dtype=oracle.I8,
                                     out_dtype=oracle.I8, in_q=(0.02, 4), w_q=(1.0, 0, ws), out_q=(0.047, -90),
                                     act=oracle.ACT_RELU6)
        want = np.zeros((m, nn), dtype=np.int64)
        for j in range(nn):
            mu, sh = oracle.quantize_multiplier(float(np.float32(0.02)) * float(ws[j]) / float(np.float32(0.047)))
            for i in range(m):
                v = min(max(Fraction(int(accf[i, j]) * mu, 2 ** sh), Fraction(0)), Fraction(6) / _f32(0.047))
                want[i, j] = min(127, max(-128, rne_fraction(v) - 90))
        assert np.array_equal(got.astype(np.int64), want.ravel())


def test_fused_relu6_equals_conv_then_relu6_when_quant_is_shared(oracle):
    # consistency of the two forms (each is pinned by closed form above): fusing is legal when the tensor
    # between the operators and the output share their quantization
    rng = np.random.default_rng(13)
    n, c, h, wd, oc = 1, 8, 6, 6, 4
    x = rng.integers(0, 256, (n, c, h, wd)).astype(np.uint8)
    w = rng.integers(0, 256, (oc, c, 3, 3)).astype(np.uint8)
    bias = rng.integers(-4096, 4097, oc).astype(np.int32)
    for out_q in ((0.1, 0), (0.07, 23)):
        kw = dict(in_shape=[wd, h, c, n], w_shape=[3, 3, c, oc], out_shape=[wd, h, oc, n], stride=[1, 1],
                  dilation=[1, 1], pad_left=1, pad_top=1, multiplier=0, in_dtype=oracle.U8,
                  w_dtype=oracle.U8, out_dtype=oracle.U8, in_q=(0.05, 128), w_q=(0.01, 120, None),
                  out_q=out_q)
        fused = oracle.conv2d(x.ravel(), w.ravel(), bias, act=oracle.ACT_RELU6, **kw)
        plain = oracle.conv2d(x.ravel(), w.ravel(), bias, **kw)
        two_step = oracle.activation(oracle.ACT_RELU6, oracle.U8, plain, out_q, out_q)
        assert np.array_equal(fused, two_step)


def test_pool_avg_divisors(oracle):
    # AVG divides by the window area, AVG_ANDROID by the in-bounds count
    x = np.arange(1, 10, dtype=np.float32)
    kw = dict(in_shape=[3, 3, 1, 1], out_shape=[2, 2, 1, 1], ksize=[2, 2], stride=[2, 2],
              pad_left=0, pad_top=0, dtype=oracle.F32)
    avg = oracle.pool2d(x, pool_type=oracle.POOL["AVG"], **kw)
    android = oracle.pool2d(x, pool_type=oracle.POOL["AVG_ANDROID"], **kw)
    assert np.allclose(avg, [(1 + 2 + 4 + 5) / 4, (3 + 6) / 4, (7 + 8) / 4, 9 / 4])
    assert np.allclose(android, [(1 + 2 + 4 + 5) / 4, (3 + 6) / 2, (7 + 8) / 2, 9])


def test_pool_l2_closed_forms(oracle):
    """L2 pooling = root of the mean of the squares over the window area. Pinned by cases with known answers: a
    3-4 pair (sqrt(12.5)), a constant plane (its absolute value), a one-tap window (|x|), homogeneity (scaling the
    input scales the result), padding that counts as zeros, and numpy on random planes."""
    f32 = oracle.F32
    l2 = oracle.POOL["L2"]
    got = oracle.pool2d(np.array([3, 4], np.float32), in_shape=[2, 1, 1, 1], out_shape=[1, 1, 1, 1], ksize=[2, 1],
                        stride=[1, 1], pad_left=0, pad_top=0, pool_type=l2, dtype=f32)
    assert np.allclose(got, [np.sqrt(12.5)], rtol=1e-6)
    x = np.full(5 * 4, -2.5, np.float32)
    got = oracle.pool2d(x, in_shape=[5, 4, 1, 1], out_shape=[3, 2, 1, 1], ksize=[3, 3], stride=[1, 1], pad_left=0,
                        pad_top=0, pool_type=l2, dtype=f32)
    assert np.allclose(got, 2.5, rtol=1e-6)
    rng = np.random.default_rng(77)
    x = rng.standard_normal(6 * 7 * 2).astype(np.float32)
    one = oracle.pool2d(x, in_shape=[6, 7, 2, 1], out_shape=[6, 7, 2, 1], ksize=[1, 1], stride=[1, 1], pad_left=0,
                        pad_top=0, pool_type=l2, dtype=f32)
    assert np.allclose(one, np.abs(x), rtol=1e-6)
    kw = dict(in_shape=[6, 7, 2, 1], out_shape=[3, 4, 2, 1], ksize=[3, 3], stride=[2, 2], pad_left=1, pad_top=1,
              pool_type=l2, dtype=f32)
    base = oracle.pool2d(x, **kw)
    assert np.allclose(oracle.pool2d(-3 * x, **kw), 3 * base, rtol=1e-5)
    # numpy: zero-padded plane, mean of squares over all nine taps
    xp = np.pad(x.reshape(2, 7, 6).astype(np.float64), ((0, 0), (1, 1), (1, 1)))
    want = np.array([[[np.sqrt(np.mean(xp[c, 2 * oh:2 * oh + 3, 2 * ow:2 * ow + 3] ** 2)) for ow in range(3)]
                      for oh in range(4)] for c in range(2)])
    assert np.allclose(base.reshape(2, 4, 3), want, rtol=1e-5)
    # the corner window holds four real taps of nine: smaller than the mean over the taps alone
    corner = x.reshape(2, 7, 6)[0, :2, :2].astype(np.float64)
    assert np.isclose(base[0], np.sqrt((corner ** 2).sum() / 9), rtol=1e-5)


@pytest.mark.parametrize("dtype_name", ["U8", "I8"])
@pytest.mark.parametrize("s_in,s_out", [(0.05, 0.05), (0.05, 0.023), (0.5, 0.25), (1.0, 1.0)])
def test_quantized_pool_l2_is_exact(oracle, dtype_name, s_in, s_out):
    """Quantized L2 pooling against exact rational arithmetic: the code q with (q - 1/2)^2 <= V < (q + 1/2)^2 for
    V = (s_in / s_out)^2 * sum (x - z_in)^2 / area - no square root is taken on this side."""
    rng = np.random.default_rng(60 + (dtype_name == "U8"))
    u8 = dtype_name == "U8"
    qmin, qmax = (0, 255) if u8 else (-128, 127)
    z_in, z_out = (101, 7) if u8 else (-9, -100)
    W, H, C, N = 7, 6, 3, 2
    k, stride, pad = [3, 3], [2, 2], [1, 1]
    ow, oh = (W + 2 * pad[0] - k[0]) // stride[0] + 1, (H + 2 * pad[1] - k[1]) // stride[1] + 1
    x = rng.integers(qmin, qmax + 1, (N * C, H, W)).astype(np.uint8 if u8 else np.int8)
    got = oracle.pool2d(x.ravel(), in_shape=[W, H, C, N], out_shape=[ow, oh, C, N], ksize=k, stride=stride,
                        pad_left=pad[0], pad_top=pad[1], pool_type=oracle.POOL["L2"],
                        dtype=oracle.U8 if u8 else oracle.I8, in_q=(s_in, z_in), out_q=(s_out, z_out))
    ratio = _f32(s_in) / _f32(s_out)
    want = []
    for p in range(N * C):
        for taps in _pool_windows(x[p], k, stride, pad, (ow, oh)):
            v4 = 4 * ratio * ratio * sum((t - z_in) ** 2 for t in taps) / (k[0] * k[1])   # (2 sqrt(V))^2
            q = 0
            while (2 * q + 1) ** 2 <= v4:   # smallest q with (2q + 1)^2 > 4V, i.e. sqrt(V) < q + 1/2
                q += 1
            assert (2 * q + 1) ** 2 != v4 and (q == 0 or (2 * q - 1) ** 2 != v4)   # (no exact tie in this data)
            want.append(min(qmax, max(qmin, q + z_out)))
    assert got.astype(np.int64).tolist() == want
    assert len(set(want)) > 8


def _pool_windows(xr, k, stride, pad, out_wh):
    """In-bounds taps of every window of one plane xr[H][W] (plain Python)."""
    H, W = xr.shape
    for oh in range(out_wh[1]):
        for ow in range(out_wh[0]):
            taps = [int(xr[ih, iw])
                    for ih in range(oh * stride[1] - pad[1], oh * stride[1] - pad[1] + k[1]) if 0 <= ih < H
                    for iw in range(ow * stride[0] - pad[0], ow * stride[0] - pad[0] + k[0]) if 0 <= iw < W]
            yield taps


@pytest.mark.parametrize("dtype_name", ["U8", "I8"])
@pytest.mark.parametrize("s_in,s_out", [(0.05, 0.05), (0.05, 0.023), (0.07, 0.11), (0.5, 0.25), (0.25, 0.5), (1.0, 1.0)])
@pytest.mark.parametrize("pool", ["MAX", "AVG", "AVG_ANDROID"])
def test_quantized_pool_requantization_is_exact(oracle, dtype_name, s_in, s_out, pool):
    # in != out quantization, padded 3x3 stride-2 windows on 7x6 planes. MAX: the largest code, dequantized and
    # requantized by the Q31 rule; averages: exact rational mean of (x - z_in) * s_in / s_out, half to even.
    # (1.0 -> 1.0 and 0.25 -> 0.5 land sums on exact .5 ties.)
    rng = np.random.default_rng(40 + 3 * (dtype_name == "U8") + ["MAX", "AVG", "AVG_ANDROID"].index(pool))
    u8 = dtype_name == "U8"
    qmin, qmax = (0, 255) if u8 else (-128, 127)
    z_in, z_out = (101, 7) if u8 else (-9, 12)
    W, H, C, N = 7, 6, 3, 2
    k, stride, pad = [3, 3], [2, 2], [1, 1]
    ow, oh = (W + 2 * pad[0] - k[0]) // stride[0] + 1, (H + 2 * pad[1] - k[1]) // stride[1] + 1
    x = rng.integers(qmin, qmax + 1, (N * C, H, W)).astype(np.uint8 if u8 else np.int8)
    got = oracle.pool2d(x.ravel(), in_shape=[W, H, C, N], out_shape=[ow, oh, C, N], ksize=k, stride=stride,
                        pad_left=pad[0], pad_top=pad[1], pool_type=oracle.POOL[pool],
                        dtype=oracle.U8 if u8 else oracle.I8, in_q=(s_in, z_in), out_q=(s_out, z_out))
    ratio = _f32(s_in) / _f32(s_out)
    mult, shift = oracle.quantize_multiplier(float(np.float32(s_in)) / float(np.float32(s_out)))
    want, ties = [], 0
    for p in range(N * C):
        for taps in _pool_windows(x[p], k, stride, pad, (ow, oh)):
            if pool == "MAX":
                v = Fraction((max(taps) - z_in) * mult, 2 ** shift)
            else:
                div = k[0] * k[1] if pool == "AVG" else len(taps)
                v = Fraction(sum(t - z_in for t in taps)) * ratio / div
            ties += (v - (v.numerator // v.denominator)) == Fraction(1, 2)
            want.append(min(qmax, max(qmin, rne_fraction(v) + z_out)))
    assert got.astype(np.int64).tolist() == want
    if pool == "AVG_ANDROID" and s_in == s_out:
        assert ties > 0   # window sums over 4 / 6 taps hit .5 often: the tie rule is exercised


def test_quantized_add_is_exact(oracle):
    # exact rational value of (a - za) * sa / so + (b - zb) * sb / so with the float32 scales, half to even
    rng = np.random.default_rng(17)
    for dt_name, sa, za, sb, zb, so, zo in (("U8", 0.03, 120, 0.05, 110, 0.07, 128), ("I8", 0.011, -3, 0.2, 7, 0.09, -20),
                                            ("U8", 0.5, 3, 0.25, 200, 1.0, 100), ("I8", 0.25, 1, 0.25, 0, 0.5, 0)):
        u8 = dt_name == "U8"
        qmin, qmax = (0, 255) if u8 else (-128, 127)
        a = rng.integers(qmin, qmax + 1, 1500).astype(np.uint8 if u8 else np.int8)
        b = rng.integers(qmin, qmax + 1, 1500).astype(np.uint8 if u8 else np.int8)
        got = oracle.add(oracle.U8 if u8 else oracle.I8, a, (sa, za), b, (sb, zb), (so, zo))
        ra, rb = _f32(sa) / _f32(so), _f32(sb) / _f32(so)
        want, ties = [], 0
        for p, q in zip(a.tolist(), b.tolist()):
            v = (p - za) * ra + (q - zb) * rb
            ties += (v - (v.numerator // v.denominator)) == Fraction(1, 2)
            want.append(min(qmax, max(qmin, rne_fraction(v) + zo)))
        assert got.astype(np.int64).tolist() == want
        if so in (1.0, 0.5):
            assert ties > 100  # power-of-two ratios: a quarter or half of the sums sit on .5


def test_quantized_softmax(oracle):
    rng = np.random.default_rng(17)
    x = rng.integers(0, 256, 40).astype(np.uint8)
    sm = oracle.softmax(oracle.U8, x, 10, 1.0, (0.1, 128))
    ref = np.exp((x.reshape(4, 10).astype(np.float64) - 128) * np.float32(0.1))
    ref /= ref.sum(axis=1, keepdims=True)
    assert np.allclose(sm.reshape(4, 10), ref, rtol=1e-5, atol=1e-7)


def _np_transpose(x, in_dims, perm):
    # numpy's axes run slowest first, the tensors here fastest first: dimension d is numpy axis r-1-d.
    r = len(in_dims)
    a = x.reshape(tuple(reversed(in_dims)))
    return np.transpose(a, axes=[r - 1 - perm[r - 1 - j] for j in range(r)]).reshape(-1)


@pytest.mark.parametrize("in_dims,perm", [
    ((5, 3), (1, 0)), ((4, 3, 2), (2, 0, 1)), ((4, 3, 2), (1, 2, 0)), ((7, 5, 3, 2), (2, 0, 1, 3)),
    ((7, 5, 3, 2), (0, 1, 2, 3)), ((3, 1, 4, 1, 5), (4, 3, 2, 1, 0)), ((6,), (0,))])
def test_transpose_restatement_vs_numpy(oracle, in_dims, perm):
    # A non-involutive perm ((2,0,1) vs (1,2,0)) tells out[i] = in[perm[i]] from its inverse reading.
    for dt in (np.uint8, np.float16, np.int32):
        x = np.arange(int(np.prod(in_dims))).astype(dt)
        got = oracle.transpose(x, in_dims, perm)
        assert got.dtype == x.dtype
        assert np.array_equal(got, _np_transpose(x, in_dims, perm))
    # the extent rule of the reference: out.size[i] = in.size[perm[i]]; element at input coordinate c lands
    # at output coordinate o with o[i] = c[perm[i]] -- checked by hand on one element of (4,3,2)/(2,0,1)
    if in_dims == (4, 3, 2) and perm == (2, 0, 1):
        x = np.arange(24, dtype=np.int32)
        y = oracle.transpose(x, in_dims, perm)            # out dims (2, 4, 3)
        c = (3, 1, 1)                                     # input offset 3 + 4*1 + 12*1 = 19
        o = (c[2], c[0], c[1])                            # output offset 1 + 2*3 + 8*1 = 15
        assert y[o[0] + 2 * o[1] + 8 * o[2]] == 19


def test_convert_restatement_vs_numpy(oracle):
    # quantize: rint(f / scale) + zp with round-half-even and saturation (vsi_nn_dtype_util_prv.h:228-252)
    f = np.array([0.0, 0.25, 0.75, 1.25, -0.25, -0.75, 63.0, 1000.0, -1000.0, 0.1, np.float32(0.3)], dtype=np.float32)
    want = np.clip(np.rint(f / np.float32(0.5)) + 3, 0, 255).astype(np.uint8)          # numpy rint = half to even
    assert list(want[:6]) == [3, 3, 5, 5, 3, 1]                                       # ties 0.5, 1.5, 2.5, -0.5, -1.5
    assert np.array_equal(oracle.convert(f, 3, (1.0, 0), 0, (0.5, 3)), want)
    want_i8 = np.clip(np.rint(f / np.float32(0.5)) - 3, -128, 127).astype(np.int8)
    assert np.array_equal(oracle.convert(f, 3, (1.0, 0), 1, (0.5, -3)), want_i8)
    # dequantize: (q - zp) * scale in float32, all 256 codes
    q = np.arange(256, dtype=np.uint8)
    got = oracle.convert(q, 0, (np.float32(0.0036), 7), 3, (1.0, 0))
    assert np.array_equal(got, (q.astype(np.float32) - np.float32(7)) * np.float32(0.0036))
    # requantize with equal scales is a shift of the zero point with saturation
    assert np.array_equal(oracle.convert(q, 0, (0.25, 0), 0, (0.25, 10)), np.minimum(q.astype(np.int32) + 10, 255))
    # uint8 <-> int8 with the zero point moved by 128 is the identity on the real values
    i8 = oracle.convert(q, 0, (0.1, 128), 1, (0.1, 0))
    assert np.array_equal(i8.astype(np.int32), q.astype(np.int32) - 128)
    # float16 output rounds to nearest even like numpy's cast; float16 input widens exactly
    h = oracle.convert(f, 3, (1.0, 0), 2, (1.0, 0))
    assert np.array_equal(h.view(np.uint16), f.astype(np.float16).view(np.uint16))
    assert np.array_equal(oracle.convert(h, 2, (1.0, 0), 3, (1.0, 0)), h.astype(np.float32))


def _deconv_bruteforce(x, w, bias, xs, ws, os_, stride, pad, groups):
    """Pure-Python gather form on integers: out(ox, oy) sums in(ix, iy) * w(kx, ky) over ix * s - pad + kx == ox."""
    W, H, C, N = xs
    KW, KH, ICG, OC = ws
    OW, OH = os_[0], os_[1]
    y = np.zeros((N, OC, OH, OW), dtype=np.int64)
    xr = x.reshape(N, C, H, W).astype(np.int64)
    wr = w.reshape(OC, ICG, KH, KW).astype(np.int64)
    for n in range(N):
        for oc in range(OC):
            ic0 = (oc // (OC // groups)) * ICG
            for oy in range(OH):
                for ox in range(OW):
                    acc = int(bias[oc]) if bias is not None else 0
                    for ci in range(ICG):
                        for ky in range(KH):
                            ty = oy + pad[1] - ky
                            if ty < 0 or ty % stride[1] or ty // stride[1] >= H:
                                continue
                            for kx in range(KW):
                                tx = ox + pad[0] - kx
                                if tx < 0 or tx % stride[0] or tx // stride[0] >= W:
                                    continue
                                acc += xr[n, ic0 + ci, ty // stride[1], tx // stride[0]] * wr[oc, ci, ky, kx]
                    y[n, oc, oy, ox] = acc
    return y.reshape(-1)


@pytest.mark.parametrize("seed", range(6))
def test_deconv_restatement_vs_bruteforce_and_adjoint(oracle, seed):
    rng = np.random.default_rng(100 + seed)
    groups = [1, 1, 2, 1, 3, 1][seed]
    icg, ocg = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    C, OC = icg * groups, ocg * groups
    W, H, N = int(rng.integers(2, 6)), int(rng.integers(2, 6)), int(rng.integers(1, 3))
    KW, KH = int(rng.integers(1, 4)), int(rng.integers(1, 4))
    stride = [int(rng.integers(1, 4)), int(rng.integers(1, 4))]
    pad = [int(rng.integers(0, KW)), int(rng.integers(0, KH))]
    opad = [int(rng.integers(0, stride[0])), int(rng.integers(0, stride[1]))]
    OW = (W - 1) * stride[0] + KW - pad[0] - int(rng.integers(0, 2)) + opad[0]
    OH = (H - 1) * stride[1] + KH - pad[1] - int(rng.integers(0, 2)) + opad[1]
    if OW < 1 or OH < 1:
        pytest.skip("empty output")
    xs, ws, os_ = [W, H, C, N], [KW, KH, icg, OC], [OW, OH, OC, N]
    # (1) float32 operands holding small integers, unit scales: the oracle's scatter against a gather in Python
    x = rng.integers(-5, 6, int(np.prod(xs))).astype(np.float32)
    w = rng.integers(-4, 5, int(np.prod(ws))).astype(np.float32)
    b = rng.integers(-9, 10, OC).astype(np.float32)
    got = oracle.conv2d(x, w, b, in_shape=xs, w_shape=ws, out_shape=os_, stride=stride, dilation=[1, 1],
                        pad_left=pad[0], pad_top=pad[1], multiplier=0, groups=groups, in_dtype=3, w_dtype=3,
                        out_dtype=3, transposed=True)
    want = _deconv_bruteforce(x, w, b, xs, ws, os_, stride, pad, groups)
    assert np.array_equal(got.astype(np.int64), want)
    # (2) adjoint of the (separately pinned) convolution: <conv(u), v> == <u, deconv(v)> when the extents are
    # the exact ones; the convolution's weights are the same numbers with the channel roles swapped
    if groups == 1 and opad == [0, 0]:
        OWf, OHf = (W - 1) * stride[0] + KW - 2 * pad[0], (H - 1) * stride[1] + KH - 2 * pad[1]
        if OWf >= KW and OHf >= KH and pad[0] < KW and pad[1] < KH and OWf > 0 and OHf > 0:
            v = x                                             # deconv input  {W, H, C, N}
            u = rng.integers(-5, 6, OWf * OHf * OC * N).astype(np.float32)   # conv input {OWf, OHf, OC, N}
            dv = oracle.conv2d(v, w, None, in_shape=xs, w_shape=ws, out_shape=[OWf, OHf, OC, N], stride=stride,
                               dilation=[1, 1], pad_left=pad[0], pad_top=pad[1], multiplier=0, in_dtype=3, w_dtype=3,
                               out_dtype=3, transposed=True)
            w_conv = np.ascontiguousarray(w.reshape(OC, icg, KH, KW).transpose(1, 0, 2, 3)).reshape(-1)  # [C][OC]
            cu = oracle.conv2d(u, w_conv, None, in_shape=[OWf, OHf, OC, N], w_shape=[KW, KH, OC, C],
                               out_shape=xs, stride=stride, dilation=[1, 1], pad_left=pad[0], pad_top=pad[1],
                               multiplier=0, in_dtype=3, w_dtype=3, out_dtype=3)
            assert float(np.dot(cu.astype(np.float64), v)) == float(np.dot(u, dv.astype(np.float64)))
    # (3) quantized: requantization and zero points as for Conv2d, checked through the integer accumulators
    xq = rng.integers(0, 256, int(np.prod(xs)), dtype=np.uint8)
    wq = rng.integers(0, 256, int(np.prod(ws)), dtype=np.uint8)
    bq = rng.integers(-300, 300, OC).astype(np.int32)
    acc = _deconv_bruteforce(xq.astype(np.int64) - 121, wq.astype(np.int64) - 130, bq, xs, ws, os_, stride, pad, groups)
    mult, shift = oracle.quantize_multiplier(0.5 * 0.25 / 37.0)
    want_q = np.clip(np.array([oracle.requant(int(a), mult, shift) for a in acc]) + 100, 0, 255)
    got_q = oracle.conv2d(xq, wq, bq, in_shape=xs, w_shape=ws, out_shape=os_, stride=stride, dilation=[1, 1],
                          pad_left=pad[0], pad_top=pad[1], multiplier=0, groups=groups, in_dtype=0, w_dtype=0,
                          out_dtype=0, in_q=(0.5, 121), w_q=(0.25, 130, None), out_q=(37.0, 100), transposed=True)
    assert np.array_equal(got_q, want_q)
