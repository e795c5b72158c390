"""Round-half-to-even at exact ties, per fast epilogue. Random float scales essentially never
land an accumulator on a .5, so each case here uses requantization multipliers of the form
odd * 2^-e (exact in float32) and checks from the accumulators themselves - recomputed with
plain integer arithmetic - that the case really holds ties that are not clamped away, that the
intended kernel took the operator, and that its output equals the oracle's bit for bit."""
import numpy as np
import pytest

import tvx_case as TC

pytestmark = pytest.mark.gpu


def _count_ties(oracle, acc, m_real, lo, hi, zo):
    """Accumulators whose exact product with the Q31 multiplier ends in .5 and whose result is not clamped."""
    mult, shift = oracle.quantize_multiplier(m_real)
    p = acc.astype(np.int64) * mult
    tie = (p & ((1 << shift) - 1)) == (1 << (shift - 1))
    q = (p >> shift) + zo
    return int(np.sum(tie & (q > lo) & (q < hi - 1)))


def _operands(rng, u8, amp_x, amp_w, nx, nw, zx, zw):
    """amp = None: the full range of the type; else codes within +-amp of the zero point."""
    lo, hi = (0, 256) if u8 else (-128, 128)
    npd = np.uint8 if u8 else np.int8
    x = (rng.integers(lo, hi, nx) if amp_x is None else zx + rng.integers(-amp_x, amp_x + 1, nx)).astype(npd)
    w = (rng.integers(lo, hi, nw) if amp_w is None else zw + rng.integers(-amp_w, amp_w + 1, nw)).astype(npd)
    return x, w


def _multipliers(per_channel, channels, e):
    """Real multipliers odd * 2^-k around 2^-e: one for per-tensor weights, a cycle of four (plus an
    ordinary inexact one) for per-channel weights. Input scale 0.5, output scale 1: w_scale = 2 * M."""
    if not per_channel:
        return np.full(channels, 3.0 * 2.0 ** -(e + 1))
    cyc = [3.0 * 2.0 ** -(e + 1), 2.0 ** -e, 5.0 * 2.0 ** -(e + 2), 2.0 ** -(e + 1), 0.0131 * 2.0 ** (6 - e)]
    return np.array([cyc[c % len(cyc)] for c in range(channels)])


CONV_TIE_CASES = [
    # kernel, dict(n, c, h, w, oc, k, stride, pad, mult), amplitude of (x, w) codes or None = full range (ties then
    # need accumulators of 2^10 .. 2^14 and are rare: those cases are sized for a few dozen of them)
    ("pwconv_i8", dict(n=2, c=32, h=16, w=16, oc=64, k=1, stride=1, pad=0, mult=0), (15, 7)),
    ("pwconv_i8", dict(n=8, c=96, h=14, w=14, oc=160, k=1, stride=1, pad=0, mult=0), None),
    ("pwconv_i8_stream", dict(n=2, c=32, h=16, w=16, oc=64, k=1, stride=1, pad=0, mult=0), (15, 7)),
    ("pwconv_i8_stream", dict(n=24, c=24, h=16, w=32, oc=72, k=1, stride=1, pad=0, mult=0), None),
    ("conv2d_igemm_i8_persistent", dict(n=2, c=32, h=28, w=28, oc=64, k=3, stride=1, pad=1, mult=0), (15, 7)),
    ("conv2d_band_i8", dict(n=2, c=32, h=24, w=24, oc=64, k=3, stride=1, pad=1, mult=0), (15, 7)),
    ("conv2d_band_i8", dict(n=10, c=64, h=28, w=24, oc=64, k=3, stride=1, pad=1, mult=0), None),
    ("conv2d_igemm_i8", dict(n=2, c=48, h=28, w=28, oc=96, k=3, stride=1, pad=1, mult=0), (15, 7)),
    ("conv2d_igemm_i8", dict(n=8, c=64, h=28, w=28, oc=80, k=3, stride=1, pad=1, mult=0), None),
    ("conv2d_igemm_i8_persistent", dict(n=10, c=64, h=28, w=28, oc=64, k=3, stride=1, pad=1, mult=0), None),
    ("conv2d_gemm_i8", dict(n=2, c=40, h=16, w=16, oc=40, k=3, stride=1, pad=1, mult=0, groups=2), (15, 7)),
    ("conv2d_gemm_i8", dict(n=16, c=48, h=48, w=48, oc=48, k=3, stride=2, pad=1, mult=0, groups=2), None),
    ("conv2d_im2col_i8", dict(n=3, c=3, h=33, w=31, oc=32, k=3, stride=2, pad=1, mult=0), (15, 7)),
    ("conv2d_im2col_i8", dict(n=12, c=1, h=28, w=28, oc=20, k=5, stride=1, pad=0, mult=0), None),
    ("dwconv3x3_i8", dict(n=2, c=8, h=16, w=16, oc=8, k=3, stride=1, pad=1, mult=1), (15, 7)),
    ("dwconv3x3_i8", dict(n=10, c=16, h=32, w=48, oc=16, k=3, stride=2, pad=1, mult=1), None),
    ("dwconv_planes_i8", dict(n=4, c=24, h=14, w=14, oc=24, k=3, stride=1, pad=1, mult=1), (15, 7)),
    ("dwconv_planes_i8", dict(n=32, c=40, h=9, w=11, oc=40, k=5, stride=1, pad=2, mult=1), None),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc"])
@pytest.mark.parametrize("ci", range(len(CONV_TIE_CASES)))
def test_conv_epilogues_round_ties_to_even(oracle, ci, mode, monkeypatch):
    import torch
    import torch.nn.functional as F
    kernel, g, amp = CONV_TIE_CASES[ci]
    if kernel.endswith("_persistent"):
        monkeypatch.setenv("TVX_IGEMM_PERSIST", "1")
        monkeypatch.setenv("TVX_CONV_BAND", "0")
    if kernel == "conv2d_band_i8":
        monkeypatch.setenv("TVX_CONV_BAND", "1")
    if kernel.endswith("_stream"):  # (the form is chosen from 1024 pixel tiles up)
        monkeypatch.setenv("TVX_PWCONV_STREAM_MIN_TILES", "1")
        monkeypatch.setenv("TVX_PWCONV_SHAPE", "128,1")
    rng = np.random.default_rng(9000 + ci)
    u8 = mode == "u8"
    n, c, h, w, oc, k, stride, pad, dm = (g[key] for key in ("n", "c", "h", "w", "oc", "k", "stride", "pad", "mult"))
    groups = g.get("groups", 0)
    icg = 1 if dm else c // max(groups, 1)
    zx, zw, zo = (128, 120, 101) if u8 else (-3, 0, 7)
    ax, aw = amp if amp else (None, None)
    x, wt = _operands(rng, u8, ax, aw, n * c * h * w, oc * icg * k * k, zx, zw)
    b = rng.integers(-300, 301, oc).astype(np.int32)
    # exact accumulators: float64 convolution of small integers
    acc = F.conv2d(torch.from_numpy(x.reshape(n, c, h, w).astype(np.float64) - zx),
                   torch.from_numpy(wt.reshape(oc, icg, k, k).astype(np.float64) - zw),
                   torch.from_numpy(b.astype(np.float64)), stride=stride, padding=pad,
                   groups=c if dm else max(groups, 1)).numpy().astype(np.int64)
    e = max(3, int(np.round(np.log2(max(acc.std(), 1.0) / 12.0))))   # ~12 output codes of spread
    m = _multipliers(not u8, oc, e)
    out_h, out_w = acc.shape[2], acc.shape[3]
    kws = dict(in_shape=[w, h, c, n], w_shape=[k, k, icg, oc], out_shape=[out_w, out_h, oc, n],
               stride=[stride, stride], dilation=[1, 1], pad_left=pad, pad_top=pad, multiplier=dm,
               in_dtype=0 if u8 else 1, w_dtype=0 if u8 else 1, out_dtype=0 if u8 else 1, in_q=(0.5, zx),
               w_q=(float(2 * m[0]), zw, None) if u8 else (1.0, 0, (2 * m).astype(np.float32)), out_q=(1.0, zo))
    if groups:
        kws["groups"] = groups
    qlo, qhi = (0, 255) if u8 else (-128, 127)
    ties = sum(_count_ties(oracle, acc[:, ch], float(m[ch]), qlo, qhi, zo) for ch in range(oc))
    assert ties >= 10, (ties, e)
    for act in (0, 2):
        want = oracle.conv2d(x, wt, b, act=act, **kws)
        got = TC.gpu_conv2d(x, wt, b, act=act, want_kernel=kernel, **kws)
        assert np.array_equal(got, want), (int((got != want).sum()), ties)
    assert len(np.unique(want)) > 4


FC_TIE_CASES = [
    ("fc_mfma_i8_256x256x128", (600, 512, 528), (15, 7)),
    ("fc_mfma_i8_256x256x128", (1025, 144, 769), None),
    ("fc_mfma_i8_16x16_splitk", (300, 512, 272), (15, 7)),
    ("fc_mfma_i8_16x16_splitk", (64, 1280, 1000), (None, 7)),
]


@pytest.mark.parametrize("mode", ["u8", "i8pc"])
@pytest.mark.parametrize("ci", range(len(FC_TIE_CASES)))
def test_fully_connected_epilogues_round_ties_to_even(oracle, ci, mode):
    kernel, (mm, k, n), amp = FC_TIE_CASES[ci]
    rng = np.random.default_rng(9100 + ci)
    u8 = mode == "u8"
    zx, zw, zo = (131, 117, 99) if u8 else (-2, 0, -9)
    ax, aw = amp if amp else (None, None)
    x, wt = _operands(rng, u8, ax, aw, mm * k, n * k, zx, zw)
    b = rng.integers(-300, 301, n).astype(np.int32)
    acc = (x.reshape(mm, k).astype(np.int64) - zx) @ (wt.reshape(n, k).astype(np.int64) - zw).T + b
    e = max(3, int(np.round(np.log2(max(acc.std(), 1.0) / 12.0))))
    m = _multipliers(not u8, n, e)
    kws = dict(m=mm, k=k, n=n, in_dtype=0 if u8 else 1, w_dtype=0 if u8 else 1, out_dtype=0 if u8 else 1,
               in_q=(0.5, zx), w_q=(float(2 * m[0]), zw, None) if u8 else (1.0, 0, (2 * m).astype(np.float32)),
               out_q=(1.0, zo))
    qlo, qhi = (0, 255) if u8 else (-128, 127)
    ties = sum(_count_ties(oracle, acc[:, j], float(m[j]), qlo, qhi, zo) for j in range(n))
    assert ties >= 10, (ties, e)
    for act in (0, 1):
        want = oracle.fully_connected(x, wt, b, act=act, **kws)
        got = TC.gpu_fully_connected(x, wt, b, act=act, want_kernel=kernel, **kws)
        assert np.array_equal(got, want), (int((got != want).sum()), ties)
    assert len(np.unique(want)) > 4


def test_zero_points_outside_the_type_are_rejected():
    T = TC.tvx()
    d = T.Conv2dDesc()
    d.in_w = d.in_h = d.out_w = d.out_h = 4
    d.in_c = d.out_c = 16
    d.batch = d.k_w = d.k_h = d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.U8
    d.in_scale = d.w_scale = d.out_scale = 0.5
    w = np.zeros(256, dtype=np.uint8)
    for field, bad in (("in_zp", 256), ("w_zp", -1), ("out_zp", 300)):
        setattr(d, field, bad)
        with pytest.raises(T.TvxError) as err:
            T.conv2d_create(d, w, None)
        assert err.value.status == T.E_INVALID and "zero point" in str(err.value)
        setattr(d, field, 0)
    T.conv2d_create(d, w, None).close()
