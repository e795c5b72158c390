"""Whole-network graph descriptions (see graphfile.py for the format): the LeNet of the
reference's sample and a MobileNetV2-1.0 with synthetic parameters. They describe graphs
only; running them is the C++ runtime's business."""
import importlib

import numpy as np

_gf = importlib.import_module(__name__.rsplit(".", 1)[0] + ".graphfile")
asym, tensor, op = _gf.asym, _gf.tensor, _gf.op


def same_pad(size, k, s, d=1):
    """TensorFlow-style SAME padding of one axis -> (out, front, back); the rule of
    vsi_nn_compute_padding (reference: src/tim/vx/internal/src/utils/vsi_nn_util.c:483-588)."""
    out = (size + s - 1) // s
    total = max((out - 1) * s + (k - 1) * d + 1 - size, 0)
    return out, total // 2, total - total // 2


def lenet_asymu8(weights, image, batch=1):
    """uint8 LeNet exactly as samples/lenet/lenet_asymu8.cc:113-290 of the reference builds
    it: conv 5x5x20 - maxpool 2 - conv 5x5x50 - maxpool 2 - FC 500 - ReLU - FC 10 - softmax.
    `weights` is that sample's 432820-byte parameter blob, `image` 28*28 uint8 (tiled over
    the batch). Scales and zero points are the sample's."""
    w = np.asarray(weights, dtype=np.uint8)
    assert w.size == 432820
    i32 = lambda a, b: w[a:b].view(np.int32)
    x = np.tile(np.asarray(image, dtype=np.uint8).reshape(-1), batch)
    b = batch
    T = [
        tensor(0, "UINT8", "INPUT", [28, 28, 1, b], asym(0.00390625, 0), x),
        tensor(1, "UINT8", "CONSTANT", [5, 5, 1, 20], asym(0.00336234, 119), w[0:500]),
        tensor(2, "INT32", "CONSTANT", [20], asym(1.313e-05, 0), i32(500, 580)),
        tensor(3, "UINT8", "TRANSIENT", [24, 24, 20, b], asym(0.01928069, 140)),
        tensor(4, "UINT8", "TRANSIENT", [12, 12, 20, b], asym(0.01928069, 140)),
        tensor(5, "UINT8", "CONSTANT", [5, 5, 20, 50], asym(0.0011482, 128), w[580:25580]),
        tensor(6, "INT32", "CONSTANT", [50], asym(2.214e-05, 0), i32(25580, 25780)),
        tensor(7, "UINT8", "TRANSIENT", [8, 8, 50, b], asym(0.04075872, 141)),
        tensor(8, "UINT8", "TRANSIENT", [4, 4, 50, b], asym(0.04075872, 141)),
        tensor(9, "UINT8", "CONSTANT", [800, 500], asym(0.00073548, 130), w[25780:425780]),
        tensor(10, "INT32", "CONSTANT", [500], asym(2.998e-05, 0), i32(425780, 427780)),
        tensor(11, "UINT8", "TRANSIENT", [500, b], asym(0.01992089, 0)),
        tensor(12, "UINT8", "TRANSIENT", [500, b], asym(0.01992089, 0)),
        tensor(13, "UINT8", "CONSTANT", [500, 10], asym(0.00158043, 135), w[427780:432780]),
        tensor(14, "INT32", "CONSTANT", [10], asym(3.148e-05, 0), i32(432780, 432820)),
        tensor(15, "UINT8", "TRANSIENT", [10, b], asym(0.06251489, 80)),
        tensor(16, "FLOAT32", "OUTPUT", [10, b]),
    ]
    P = [
        op("CONV2D", [0, 1, 2], [3], pad_type="VALID", ksize=[5, 5], weights=20),
        op("POOL", [3], [4], pad_type="NONE", pool_type="MAX", ksize=[2, 2], stride=[2, 2]),
        op("CONV2D", [4, 5, 6], [7], pad_type="VALID", ksize=[5, 5], weights=50),
        op("POOL", [7], [8], pad_type="NONE", pool_type="MAX", ksize=[2, 2], stride=[2, 2]),
        op("FCL", [8, 9, 10], [11], axis=2, weights=500),
        op("RELU", [11], [12]),
        op("FCL", [12, 13, 14], [15], axis=0, weights=10),
        op("SOFTMAX", [15], [16], beta=1.0, sm_axis=0),
    ]
    return {"test": "lenet_asymu8_b%d" % batch, "tensors": T, "ops": P, "output": 16}


def lenet_random(batch=1, seed=0x71):
    """The same LeNet topology with seeded synthetic parameters: input uint8 uniform [0, 255] at
    scale 1/255, zero point 0; weights uint8 uniform at scale 0.02 with a zero point drawn from
    [100, 156] per tensor; int32 biases uniform in [-1024, 1024] at scale s_in * s_w. Activation
    scales and zero points come from a calibration pass in floating point over the first images
    of the batch (each layer's output range between its 0.1 % and 99.9 % quantiles, widened to hold
    zero, mapped onto the 256 codes), so that no layer collapses or saturates; they are part of the description."""
    rng = np.random.default_rng(seed)
    b = batch
    u8 = lambda n: rng.integers(0, 256, n, dtype=np.uint8)
    s_w = 0.02
    T, P = [], []
    nb = min(b, 4)  # images of the calibration pass

    def t(dtype, attr, shape, quant=None, data=None):
        T.append(tensor(len(T), dtype, attr, shape, quant, data))
        return T[-1]

    def quantize(real, relu):
        # the range always holds the real value 0: the zero point has to be one of the 256 codes
        lo = 0.0 if relu else min(float(np.quantile(real, 0.001)), 0.0)
        hi = max(float(np.quantile(real, 0.999)), 0.0)
        s_out = float(np.float32(max(hi - lo, 1e-6) / 255.0))
        zp = int(np.clip(np.rint(-lo / s_out), 0, 255))
        codes = np.clip(np.rint(real / s_out) + zp, zp if relu else 0, 255)
        return asym(s_out, zp), (codes - zp) * s_out

    def layer(kind, x, real_in, w_shape, out_shape, relu=False, **attrs):
        """real_in: the calibration images' activations as real numbers, [nb, C, H, W] or [nb, K]."""
        s_in = x["quant"]["scales"][0]
        oc = w_shape[-1]
        w_zp = int(rng.integers(100, 157))
        wq = u8(int(np.prod(w_shape)))
        bq = rng.integers(-1024, 1025, oc).astype(np.int32)
        w = t("UINT8", "CONSTANT", w_shape, asym(s_w, w_zp), wq)
        bias = t("INT32", "CONSTANT", [oc], asym(float(np.float32(s_in) * np.float32(s_w)), 0), bq)
        wr = (wq.astype(np.float64) - w_zp) * s_w
        if kind == "CONV2D":
            k = w_shape[0]
            win = np.lib.stride_tricks.sliding_window_view(real_in, (k, k), axis=(2, 3))  # [n, c, oh, ow, k, k]
            real = np.einsum("nchwyx,ocyx->nohw", win, wr.reshape(oc, w_shape[2], k, k))
            real += (bq * s_in * s_w)[None, :, None, None]
        else:
            real = real_in.reshape(nb, -1) @ wr.reshape(oc, -1).T + bq * s_in * s_w
        q, real = quantize(real, relu)
        y = t("UINT8", "TRANSIENT", out_shape, q)
        P.append(op(kind, [x["id"], w["id"], bias["id"]], [y["id"]], weights=oc, **attrs))
        return y, real

    def pool(x, real):
        w_, h_, c_, _ = x["shape"]
        y = t("UINT8", "TRANSIENT", [w_ // 2, h_ // 2, c_, b], x["quant"])
        P.append(op("POOL", [x["id"]], [y["id"]], pad_type="NONE", pool_type="MAX", ksize=[2, 2], stride=[2, 2]))
        return y, real.reshape(nb, c_, h_ // 2, 2, w_ // 2, 2).max(axis=(3, 5))

    img = u8(28 * 28 * b)
    x = t("UINT8", "INPUT", [28, 28, 1, b], asym(1.0 / 255.0, 0), img)
    real = img[:nb * 784].reshape(nb, 1, 28, 28).astype(np.float64) / 255.0
    h, real = layer("CONV2D", x, real, [5, 5, 1, 20], [24, 24, 20, b], pad_type="VALID", ksize=[5, 5])
    h, real = pool(h, real)
    h, real = layer("CONV2D", h, real, [5, 5, 20, 50], [8, 8, 50, b], pad_type="VALID", ksize=[5, 5])
    h, real = pool(h, real)
    h, real = layer("FCL", h, real, [800, 500], [500, b], relu=True, axis=2)
    r = t("UINT8", "TRANSIENT", [500, b], h["quant"])
    P.append(op("RELU", [h["id"]], [r["id"]]))
    logits, real = layer("FCL", r, real, [500, 10], [10, b], axis=0)
    out = t("FLOAT32", "OUTPUT", [10, b])
    P.append(op("SOFTMAX", [logits["id"]], [out["id"]], beta=1.0, sm_axis=0))
    return {"test": "lenet_random_b%d" % batch, "tensors": T, "ops": P, "output": out["id"],
            "logits": logits["id"]}


def cut_at(graph, tensor_id, name=None):
    """The graph up to the operator that produces `tensor_id`, with that tensor as the OUTPUT."""
    import copy
    last = next(i for i, o in enumerate(graph["ops"]) if tensor_id in o["outputs"])
    g = {k: v for k, v in graph.items() if k not in ("tensors", "ops")}
    g["ops"] = copy.deepcopy(graph["ops"][:last + 1])
    used = {i for o in g["ops"] for i in o["inputs"] + o["outputs"]}
    g["tensors"] = [dict(t) for t in graph["tensors"] if t["id"] in used]
    for t in g["tensors"]:
        if t["id"] == tensor_id:
            t["attr"] = "OUTPUT"
    g["output"] = tensor_id
    g["test"] = name or "%s_cut%d" % (graph["test"], tensor_id)
    return g


# (expansion, output channels, repeats, first stride) of the MobileNetV2 bottleneck stages
_MBV2_STAGES = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1),
                (6, 160, 3, 2), (6, 320, 1, 1)]


class _Builder:
    def __init__(self, seed):
        self.rng = np.random.default_rng(seed)
        self.tensors, self.ops = [], []

    def new(self, dtype, attr, shape, quant=None, data=None):
        t = tensor(len(self.tensors), dtype, attr, shape, quant, data)
        self.tensors.append(t)
        return t

    def conv(self, x, oc, k, stride, act, depthwise=False, out_attr="TRANSIENT"):
        """uint8 conv with synthetic weights. Scales are chosen from a running estimate of
        the activations' spread (`_rms`, in quantization steps about the zero point) so that
        every layer's output fills the uint8 range instead of collapsing or saturating:
        Relu6 outputs use the scale that maps 6.0 to 255, linear ones a spread of ~38 steps."""
        w_in, h_in, c_in, b = x["shape"]
        ow, pl, pr = same_pad(w_in, k, stride)
        oh, pt, pb = same_pad(h_in, k, stride)
        fan = k * k * (1 if depthwise else c_in)
        w_shape = [k, k, c_in, 1] if depthwise else [k, k, c_in, oc]
        w_zp = int(self.rng.integers(124, 132))
        wq = self.rng.integers(0, 256, size=int(np.prod(w_shape)), dtype=np.uint8)
        s_in = x["quant"]["scales"][0]
        target = 100.0 if act else 38.0
        m = target / (np.sqrt(fan) * 74.0 * x["_rms"])  # accumulator spread -> output steps
        if act:
            s_out = float(np.float32(6.0 / 255.0))
            s_w = float(np.float32(m * s_out / s_in))
        else:
            s_w = float(np.float32(0.002 + 0.002 * self.rng.random()))
            s_out = float(np.float32(s_in * s_w / m))
        out_zp = 0 if act else int(self.rng.integers(118, 138))
        bias = self.rng.integers(-2000, 2000, size=oc, dtype=np.int32)
        wt = self.new("UINT8", "CONSTANT", w_shape, asym(s_w, w_zp), wq)
        bt = self.new("INT32", "CONSTANT", [oc], asym(float(np.float32(s_in) * np.float32(s_w)), 0), bias)
        q_out = asym(s_out, out_zp)
        attrs = dict(pad_type="AUTO", pad=[pl, pr, pt, pb], ksize=[k, k], stride=[stride, stride],
                     weights=oc, multiplier=1 if depthwise else 0)
        if not act:
            y = self.new("UINT8", out_attr, [ow, oh, oc, b], q_out)
            y["_rms"] = target
            self.ops.append(op("CONV2D", [x["id"], wt["id"], bt["id"]], [y["id"]], **attrs))
            return y
        mid = self.new("UINT8", "TRANSIENT", [ow, oh, oc, b], q_out)
        y = self.new("UINT8", out_attr, [ow, oh, oc, b], q_out)
        y["_rms"] = 0.7 * target
        self.ops.append(op("CONV2D", [x["id"], wt["id"], bt["id"]], [mid["id"]], **attrs))
        self.ops.append(op(act, [mid["id"]], [y["id"]]))
        return y

    def add(self, a, b):
        sa, sb = a["quant"]["scales"][0], b["quant"]["scales"][0]
        real = float(np.hypot(sa * a["_rms"], sb * b["_rms"]))
        y = self.new("UINT8", "TRANSIENT", a["shape"],
                     asym(float(np.float32(real / 38.0)), int(self.rng.integers(118, 138))))
        y["_rms"] = 38.0
        self.ops.append(op("ADD", [a["id"], b["id"]], [y["id"]]))
        return y


def mobilenet_v2(batch=1, res=224, classes=1000, seed=0):
    """MobileNetV2-1.0, uint8 asymmetric per-tensor throughout, synthetic parameters:
    conv3x3/2 - 17 inverted-residual blocks - conv1x1x1280 - global average pool - FC.
    Activations are Relu6 operators behind TRANSIENT tensors of identical quantization (what
    a converter emits and the runtime fuses); residuals are quantized Adds. The graph's
    output is the uint8 logits tensor {classes, batch}."""
    g = _Builder(seed)
    x = g.new("UINT8", "INPUT", [res, res, 3, batch], asym(1.0 / 128, 128),
              g.rng.integers(0, 256, size=res * res * 3 * batch, dtype=np.uint8))
    x["_rms"] = 74.0
    x = g.conv(x, 32, 3, 2, "RELU6")
    c_in = 32
    for t, c, n, s in _MBV2_STAGES:
        for i in range(n):
            stride = s if i == 0 else 1
            block_in = x
            h = x
            if t != 1:
                h = g.conv(h, c_in * t, 1, 1, "RELU6")
            h = g.conv(h, c_in * t, 3, stride, "RELU6", depthwise=True)
            h = g.conv(h, c, 1, 1, None)
            if stride == 1 and c_in == c:
                h = g.add(block_in, h)
            x = h
            c_in = c
    x = g.conv(x, 1280, 1, 1, "RELU6")
    w_in, h_in, c, b = x["shape"]
    pooled = g.new("UINT8", "TRANSIENT", [1, 1, c, b], x["quant"])
    g.ops.append(op("POOL", [x["id"]], [pooled["id"]], pad_type="VALID", pool_type="AVG",
                    ksize=[w_in, h_in], stride=[w_in, h_in]))
    s_in = pooled["quant"]["scales"][0]
    s_w = float(np.float32(0.003))
    wt = g.new("UINT8", "CONSTANT", [c, classes], asym(s_w, 128),
               g.rng.integers(0, 256, size=c * classes, dtype=np.uint8))
    bt = g.new("INT32", "CONSTANT", [classes], asym(float(np.float32(s_in) * np.float32(s_w)), 0),
               g.rng.integers(-4000, 4000, size=classes, dtype=np.int32))
    m = 38.0 / (np.sqrt(c) * 74.0 * 60.0)
    logits = g.new("UINT8", "OUTPUT", [classes, b], asym(float(np.float32(s_in * s_w / m)), 128))
    g.ops.append(op("FCL", [pooled["id"], wt["id"], bt["id"]], [logits["id"]], axis=2, weights=classes))
    return {"test": "mobilenet_v2_u8_b%d_r%d" % (batch, res), "tensors": g.tensors, "ops": g.ops,
            "output": logits["id"]}


def conv3x3_same_relu6(batch=32, channels=64, side=56, seed=0x71):
    """One uint8 per-tensor 3x3 convolution with SAME padding and a Relu6 behind it (fused by the runtime):
    the single-operator benchmark configuration as an application would build it."""
    rng = np.random.default_rng(seed)
    c, s, n = channels, side, batch
    q = asym
    return {"test": "conv3x3_u8_%dto%d_%dx%d_b%d" % (c, c, s, s, n), "output": 4, "tensors": [
        tensor(0, "UINT8", "INPUT", [s, s, c, n], q(0.05, 128), rng.integers(0, 256, n * c * s * s, dtype=np.uint8)),
        tensor(1, "UINT8", "CONSTANT", [3, 3, c, c], q(0.01, 120), rng.integers(0, 256, c * c * 9, dtype=np.uint8)),
        tensor(2, "INT32", "CONSTANT", [c], q(0.0005, 0), rng.integers(-4096, 4097, c).astype(np.int32)),
        tensor(3, "UINT8", "TRANSIENT", [s, s, c, n], q(0.1, 0)),
        tensor(4, "UINT8", "OUTPUT", [s, s, c, n], q(0.1, 0))],
        "ops": [op("CONV2D", [0, 1, 2], [3], pad_type="SAME", ksize=[3, 3], weights=c),
                op("RELU6", [3], [4])]}


def mac_count(graph):
    """Multiply-accumulates of every CONV2D / FCL of a graph description."""
    ts = {t["id"]: t for t in graph["tensors"]}
    total = 0
    for o in graph["ops"]:
        if o["kind"] == "CONV2D":
            w, y = ts[o["inputs"][1]]["shape"], ts[o["outputs"][0]]["shape"]
            per_out = w[0] * w[1] * (1 if o["attrs"]["multiplier"] else w[2])
            total += per_out * int(np.prod(y))
        elif o["kind"] == "FCL":
            w, y = ts[o["inputs"][1]]["shape"], ts[o["outputs"][0]]["shape"]
            total += w[0] * int(np.prod(y))
    return total
