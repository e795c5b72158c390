"""ctypes front of oracle/tvx_oracle.c (the CPU restatement; test infrastructure).

`run_case(case)` executes one recorded graph from tests/golden/*.json through
the oracle and returns the output tensor as a numpy array.
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "_build", "libtvx_oracle.so")

U8, I8, F16, F32 = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_RELU6 = 0, 1, 2
POOL = {"MAX": 0, "AVG": 1, "L2": 2, "AVG_ANDROID": 3}
DTYPE_CODE = {"UINT8": U8, "INT8": I8, "FLOAT16": F16, "FLOAT32": F32}
NP_DTYPE = {"UINT8": np.uint8, "INT8": np.int8, "FLOAT16": np.float16,
            "FLOAT32": np.float32, "INT32": np.int32}


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "in_c", "batch", "k_w", "k_h", "out_c", "out_w", "out_h",
        "stride_w", "stride_h", "dil_w", "dil_h", "pad_left", "pad_top", "multiplier",
        "in_dtype", "w_dtype", "out_dtype")] + [
        ("in_scale", C.c_float), ("in_zp", C.c_int32), ("w_scale", C.c_float),
        ("w_zp", C.c_int32), ("w_scales", C.POINTER(C.c_float)),
        ("out_scale", C.c_float), ("out_zp", C.c_int32), ("act", C.c_int32), ("groups", C.c_int32)]


class FcDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in ("m", "k", "n", "in_dtype", "w_dtype", "out_dtype")] + [
        ("in_scale", C.c_float), ("in_zp", C.c_int32), ("w_scale", C.c_float),
        ("w_zp", C.c_int32), ("w_scales", C.POINTER(C.c_float)),
        ("out_scale", C.c_float), ("out_zp", C.c_int32), ("act", C.c_int32)]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "in_w", "in_h", "channels", "batch", "out_w", "out_h", "k_w", "k_h",
        "stride_w", "stride_h", "pad_left", "pad_top", "pool_type", "dtype")] + [
        ("in_scale", C.c_float), ("in_zp", C.c_int32),
        ("out_scale", C.c_float), ("out_zp", C.c_int32)]


_lib = None


def build(force=False):
    if force or not os.path.exists(LIB_PATH) or \
            os.path.getmtime(LIB_PATH) < os.path.getmtime(os.path.join(HERE, "tvx_oracle.c")):
        subprocess.check_call(["make", "-s", "-B", "-C", HERE])
    return LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        _lib = C.CDLL(LIB_PATH)
        _lib.tvxo_requant.restype = C.c_int64
        _lib.tvxo_requant.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        _lib.tvxo_quantize_multiplier.argtypes = [C.c_double, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        _lib.tvxo_activation.argtypes = [C.c_int, C.c_int, C.c_int64, C.c_void_p, C.c_float, C.c_int32,
                                         C.c_void_p, C.c_float, C.c_int32]
        _lib.tvxo_add.argtypes = [C.c_int, C.c_int64, C.c_void_p, C.c_float, C.c_int32, C.c_void_p,
                                  C.c_float, C.c_int32, C.c_void_p, C.c_float, C.c_int32]
        _lib.tvxo_convert.argtypes = [C.c_int, C.c_int64, C.c_void_p, C.c_float, C.c_int32, C.c_int, C.c_void_p,
                                      C.c_float, C.c_int32]
        _lib.tvxo_convert.restype = None
        _lib.tvxo_transpose.argtypes = [C.c_int32, C.POINTER(C.c_uint32), C.POINTER(C.c_uint32), C.c_int32,
                                        C.c_void_p, C.c_void_p]
        _lib.tvxo_transpose.restype = None
        _lib.tvxo_softmax.argtypes = [C.c_int, C.c_int32, C.c_int64, C.c_int64, C.c_float, C.c_void_p, C.c_float,
                                      C.c_int32, C.c_void_p]
        _lib.tvxo_conv2d.argtypes = [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.tvxo_deconv2d.argtypes = [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.tvxo_fully_connected.argtypes = [C.POINTER(FcDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        _lib.tvxo_pool2d.argtypes = [C.POINTER(PoolDesc), C.c_void_p, C.c_void_p]
    return _lib


def _ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def quantize_multiplier(m):
    mult, shift = C.c_int32(), C.c_int32()
    lib().tvxo_quantize_multiplier(m, C.byref(mult), C.byref(shift))
    return mult.value, shift.value


def requant(acc, mult, shift):
    return lib().tvxo_requant(int(acc), int(mult), int(shift))


def _q(quant):
    """(scale, zp, per_channel_scales or None) of a fixture quant record."""
    if quant["type"] == "SYMMETRIC_PER_CHANNEL":
        return 1.0, 0, np.asarray(quant["scales"], dtype=np.float32)
    if quant["type"] == "ASYMMETRIC":
        return float(np.float32(quant["scales"][0])), int(quant["zero_points"][0]), None
    return 1.0, 0, None


def _conv_shapes(a, x_shape, w_shape, out_shape):
    """(in, weight, out) shapes in the 2-D operator's terms; Conv1d tensors {W, C, N} / {Kw, Ic, Oc}
    are rows of height one."""
    if a.get("conv_1d"):
        return ([x_shape[0], 1, x_shape[1], x_shape[2]], [w_shape[0], 1, w_shape[1], w_shape[2]],
                [out_shape[0], 1, out_shape[1], out_shape[2]])
    return x_shape, w_shape, out_shape



ACT_TO_WHCN = {"CWHN": [1, 2, 0, 3]}                      # activation layouts other than WHCN
ACT_FROM_WHCN = {"CWHN": [2, 0, 1, 3]}
KERNEL_TO_WHICOC = {"IcWHOc": [1, 2, 0, 3], "OcIcWH": [2, 3, 1, 0], "IcOcWH": [2, 3, 0, 1]}


def _permuted(shape, perm):
    return [shape[p] for p in perm]


def _resolved_pad(a, in_shape, w_shape):
    """Explicit {left, right, top, bottom} of a conv / pool: AUTO keeps the operator's own numbers,
    VALID pads nothing, SAME makes out = ceil(in / stride) with the smaller half in front
    (src/tim/vx/internal/src/utils/vsi_nn_util.c:221-235, 513-553)."""
    if a["pad_type"] in ("AUTO", "NONE"):
        return list(a["pad"])
    if a["pad_type"] == "VALID":
        return [0, 0, 0, 0]
    pad = []
    for ax in (0, 1):
        dil = a["dilation"][ax] or 1
        ke = (w_shape[ax] - 1) * dil + 1
        out = -(-in_shape[ax] // a["stride"][ax])
        total = max((out - 1) * a["stride"][ax] + ke - in_shape[ax], 0)
        pad += [total // 2, total - total // 2]
    return pad


def conv2d(x, w, bias, *, in_shape, w_shape, out_shape, stride, dilation, pad_left, pad_top,
           multiplier, in_dtype, w_dtype, out_dtype, in_q=(1.0, 0), w_q=(1.0, 0, None),
           out_q=(1.0, 0), act=ACT_NONE, groups=0, transposed=False):
    """Shapes are WHCN / WHIcOc lists (dim 0 fastest); arrays are flat, C-contiguous.
    transposed: DeConv2d (same descriptor, read the other way round)."""
    d = ConvDesc()
    d.groups = groups
    d.in_w, d.in_h, d.in_c, d.batch = in_shape
    d.k_w, d.k_h = w_shape[0], w_shape[1]
    d.out_w, d.out_h, d.out_c = out_shape[0], out_shape[1], out_shape[2]
    d.stride_w, d.stride_h = stride
    d.dil_w, d.dil_h = dilation
    d.pad_left, d.pad_top, d.multiplier = pad_left, pad_top, multiplier
    d.in_dtype, d.w_dtype, d.out_dtype = in_dtype, w_dtype, out_dtype
    d.in_scale, d.in_zp = in_q
    d.w_scale, d.w_zp = w_q[0], w_q[1]
    ws = None
    if w_q[2] is not None:
        ws = np.ascontiguousarray(w_q[2], dtype=np.float32)
        d.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = out_q
    d.act = act
    np_out = {U8: np.uint8, I8: np.int8, F16: np.float16, F32: np.float32}[out_dtype]
    y = np.zeros(int(np.prod(out_shape)), dtype=np_out)
    (lib().tvxo_deconv2d if transposed else lib().tvxo_conv2d)(C.byref(d), _ptr(x), _ptr(w), _ptr(bias), _ptr(y))
    return y


def fully_connected(x, w, bias, *, m, k, n, in_dtype, w_dtype, out_dtype, in_q=(1.0, 0),
                    w_q=(1.0, 0, None), out_q=(1.0, 0), act=ACT_NONE):
    d = FcDesc()
    d.m, d.k, d.n = m, k, n
    d.in_dtype, d.w_dtype, d.out_dtype = in_dtype, w_dtype, out_dtype
    d.in_scale, d.in_zp = in_q
    d.w_scale, d.w_zp = w_q[0], w_q[1]
    ws = None
    if w_q[2] is not None:
        ws = np.ascontiguousarray(w_q[2], dtype=np.float32)
        d.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = out_q
    d.act = act
    np_out = {U8: np.uint8, I8: np.int8, F16: np.float16, F32: np.float32}[out_dtype]
    y = np.zeros(m * n, dtype=np_out)
    lib().tvxo_fully_connected(C.byref(d), _ptr(x), _ptr(w), _ptr(bias), _ptr(y))
    return y


def pool2d(x, *, in_shape, out_shape, ksize, stride, pad_left, pad_top, pool_type, dtype,
           in_q=(1.0, 0), out_q=(1.0, 0)):
    """in_shape / out_shape are {W, H, C, N}."""
    d = PoolDesc()
    d.in_w, d.in_h, d.channels, d.batch = in_shape
    d.out_w, d.out_h = out_shape[0], out_shape[1]
    d.k_w, d.k_h = ksize
    d.stride_w, d.stride_h = stride
    d.pad_left, d.pad_top = pad_left, pad_top
    d.pool_type, d.dtype = pool_type, dtype
    d.in_scale, d.in_zp = in_q
    d.out_scale, d.out_zp = out_q
    np_out = {U8: np.uint8, I8: np.int8, F16: np.float16, F32: np.float32}[dtype]
    y = np.zeros(int(np.prod(out_shape)), dtype=np_out)
    lib().tvxo_pool2d(C.byref(d), _ptr(x), _ptr(y))
    return y


def activation(act, dtype, x, in_q, out_q):
    y = np.zeros_like(x)
    lib().tvxo_activation(act, dtype, x.size, _ptr(x), in_q[0], in_q[1], _ptr(y), out_q[0], out_q[1])
    return y


def add(dtype, a, a_q, b, b_q, out_q):
    y = np.zeros_like(a)
    lib().tvxo_add(dtype, a.size, _ptr(a), a_q[0], a_q[1], _ptr(b), b_q[0], b_q[1], _ptr(y),
                   out_q[0], out_q[1])
    return y


def softmax(dtype, x, c, beta, in_q, inner=1):
    """Softmax along an axis of `c` elements that are `inner` apart (inner = product of the dimensions below it)."""
    y = np.zeros(x.size, dtype=np.float32)
    lib().tvxo_softmax(dtype, c, x.size // (c * inner), inner, beta, _ptr(x), in_q[0], in_q[1], _ptr(y))
    return y


# --------------------------------------------------------------------------
# fixture cases
# --------------------------------------------------------------------------
NP_OF_CODE = {U8: np.uint8, I8: np.int8, F16: np.float16, F32: np.float32}


def convert(x, in_dtype, in_q, out_dtype, out_q):
    """DataConvert: element -> float32 -> output type (quantize / dequantize / requantize)."""
    x = np.ascontiguousarray(x).reshape(-1)
    y = np.zeros(x.size, dtype=NP_OF_CODE[out_dtype])
    lib().tvxo_convert(in_dtype, x.size, _ptr(x), in_q[0], in_q[1], out_dtype, _ptr(y), out_q[0], out_q[1])
    return y


def transpose(x, in_dims, perm):
    """Output dimension i is input dimension perm[i] (dimension 0 fastest); x is the flat input."""
    x = np.ascontiguousarray(x).reshape(-1)
    y = np.empty_like(x)
    dims = (C.c_uint32 * len(in_dims))(*in_dims)
    pm = (C.c_uint32 * len(perm))(*perm)
    lib().tvxo_transpose(len(in_dims), dims, pm, x.dtype.itemsize, _ptr(x), _ptr(y))
    return y


def expand(data, dtype_name):
    """Fixture 'data' field (list, or {'fill': v, 'n': count}) -> flat numpy array."""
    npd = NP_DTYPE[dtype_name]
    if isinstance(data, dict):
        return np.full(data["n"], data["fill"], dtype=npd)
    return np.asarray(data, dtype=npd)


def _softmax_view(shape, axis):
    """(elements along the axis, their distance) for a softmax along `axis` (dimension 0 is the fastest)."""
    axis = axis % len(shape)
    return shape[axis], int(np.prod(shape[:axis])) if axis else 1


def pad4(shape):
    """Pool1d tensors are {W, C, N}: view them as {W, 1, C, N}."""
    return [shape[0], 1, shape[1], shape[2]] if len(shape) == 3 else list(shape)


def run_case(case):
    """Run a one-operator fixture graph through the oracle; returns the flat output array."""
    if case.get("layout_inference") or len(case["ops"]) > 1:
        return run_graph(case)  # a source graph as the front end states it: layouts, unresolved pads
    tensors = {t["id"]: t for t in case["tensors"]}
    op = case["ops"][0]
    a = op["attrs"]
    ins = [tensors[i] for i in op["inputs"]]
    out = tensors[op["outputs"][0]]
    arr = [expand(t["data"], t["dtype"]) if t["data"] is not None else None for t in ins]
    if op["kind"] == "CONV2D":
        x, w = ins[0], ins[1]
        bias = arr[2] if len(ins) > 2 else None
        s, z, _ = _q(x["quant"])
        so, zo, _ = _q(out["quant"])
        xs, wsh, osh = _conv_shapes(a, x["shape"], w["shape"], out["shape"])
        return conv2d(arr[0], arr[1], bias, in_shape=xs, w_shape=wsh,
                      out_shape=osh, stride=a["stride"], dilation=a["dilation"],
                      pad_left=a["pad"][0], pad_top=a["pad"][2], multiplier=a["multiplier"], groups=a.get("groups", 0),
                      in_dtype=DTYPE_CODE[x["dtype"]], w_dtype=DTYPE_CODE[w["dtype"]],
                      out_dtype=DTYPE_CODE[out["dtype"]], in_q=(s, z), w_q=_q(w["quant"]),
                      out_q=(so, zo))
    if op["kind"] == "DECONV2D":
        x, w = ins[0], ins[1]
        s, z, _ = _q(x["quant"])
        so, zo, _ = _q(out["quant"])
        xs, wsh, osh = _conv_shapes(a, x["shape"], w["shape"], out["shape"])  # DeConv1d: rows of height one
        return conv2d(arr[0], arr[1], arr[2] if len(ins) > 2 else None, in_shape=xs, w_shape=wsh,
                      out_shape=osh, stride=a["stride"], dilation=[1, 1], pad_left=a["pad"][0],
                      pad_top=a["pad"][2], multiplier=0, groups=a.get("groups", 0), in_dtype=DTYPE_CODE[x["dtype"]],
                      w_dtype=DTYPE_CODE[w["dtype"]], out_dtype=DTYPE_CODE[out["dtype"]], in_q=(s, z),
                      w_q=_q(w["quant"]), out_q=(so, zo), transposed=True)
    if op["kind"] == "FCL":
        x, w = ins[0], ins[1]
        bias = arr[2] if len(ins) > 2 else None
        k = int(np.prod(x["shape"][:a["axis"] + 1]))
        m = int(np.prod(x["shape"][a["axis"] + 1:]))
        n = w["shape"][-1]
        s, z, _ = _q(x["quant"])
        so, zo, _ = _q(out["quant"])
        return fully_connected(arr[0], arr[1], bias, m=m, k=k, n=n,
                               in_dtype=DTYPE_CODE[x["dtype"]], w_dtype=DTYPE_CODE[w["dtype"]],
                               out_dtype=DTYPE_CODE[out["dtype"]], in_q=(s, z),
                               w_q=_q(w["quant"]), out_q=(so, zo))
    if op["kind"] == "POOL":
        x = ins[0]
        s, z, _ = _q(x["quant"])
        so, zo, _ = _q(out["quant"])
        return pool2d(arr[0], in_shape=pad4(x["shape"]), out_shape=pad4(out["shape"]),
                      ksize=a["ksize"], stride=a["stride"], pad_left=a["pad"][0],
                      pad_top=a["pad"][2], pool_type=POOL[a["pool_type"]],
                      dtype=DTYPE_CODE[x["dtype"]], in_q=(s, z), out_q=(so, zo))
    if op["kind"] == "SOFTMAX":
        x = ins[0]
        s, z, _ = _q(x["quant"])
        c, inner = _softmax_view(x["shape"], a.get("sm_axis", 0))
        return softmax(DTYPE_CODE[x["dtype"]], arr[0], c, a.get("beta", 1.0), (s, z), inner)
    if op["kind"] == "TRANSPOSE":
        return transpose(arr[0], ins[0]["shape"], a["perm"])
    if op["kind"] == "DATACONVERT":
        s, z, _ = _q(ins[0]["quant"])
        so, zo, _ = _q(out["quant"])
        return convert(arr[0], DTYPE_CODE[ins[0]["dtype"]], (s, z), DTYPE_CODE[out["dtype"]], (so, zo))
    raise NotImplementedError(op["kind"])


def run_graph(graph, keep_all=False):
    """Interpret a multi-operator graph description operator by operator (no fusion): every
    operator's result is quantized to its own output tensor before the next one reads it,
    which is what the reference's graph semantics prescribe (each vx node writes a tensor).
    Tensors need resolved shapes and explicit pads. Returns the flat output array (or the
    dict of all tensors' values)."""
    ts = {t["id"]: t for t in graph["tensors"]}
    val = {}
    for t in graph["tensors"]:
        if t["data"] is not None:
            d = t["data"]
            val[t["id"]] = (expand(d, t["dtype"]) if isinstance(d, (list, dict))
                            else np.ascontiguousarray(np.asarray(d), dtype=NP_DTYPE[t["dtype"]]).reshape(-1))
    for o in graph["ops"]:
        a = o["attrs"]
        ins = [ts[i] if i >= 0 else None for i in o["inputs"]]
        out = ts[o["outputs"][0]]
        k = o["kind"]
        x = ins[0]
        s, z, _ = _q(x["quant"])
        so, zo, _ = _q(out["quant"])
        xv = val[x["id"]]
        if k == "CONV2D":
            w = ins[1]
            bias = val[ins[2]["id"]] if len(ins) > 2 and ins[2] is not None else None
            # operands in another layout are brought to WHCN / WHIcOc, the result is taken back
            lay, klay = a.get("layout", "ANY"), a.get("kernel_layout", "ANY")
            xshape, wshape, oshape, wv = x["shape"], w["shape"], out["shape"], val[w["id"]]
            if lay in ACT_TO_WHCN:
                xv = transpose(xv, xshape, ACT_TO_WHCN[lay])
                xshape, oshape = _permuted(xshape, ACT_TO_WHCN[lay]), _permuted(oshape, ACT_TO_WHCN[lay])
            if klay in KERNEL_TO_WHICOC:
                wv = transpose(wv, wshape, KERNEL_TO_WHICOC[klay])
                wshape = _permuted(wshape, KERNEL_TO_WHICOC[klay])
            xs, wsh, osh = _conv_shapes(a, xshape, wshape, oshape)
            pad = _resolved_pad(a, xs, wsh)
            y = conv2d(xv, wv, bias, in_shape=xs, w_shape=wsh,
                       out_shape=osh, stride=a["stride"], dilation=[d or 1 for d in a["dilation"]],
                       pad_left=pad[0], pad_top=pad[2], multiplier=a["multiplier"], groups=a.get("groups", 0),
                       in_dtype=DTYPE_CODE[x["dtype"]], w_dtype=DTYPE_CODE[w["dtype"]],
                       out_dtype=DTYPE_CODE[out["dtype"]], in_q=(s, z), w_q=_q(w["quant"]),
                       out_q=(so, zo))
            if lay in ACT_FROM_WHCN:
                y = transpose(y, oshape, ACT_FROM_WHCN[lay])
        elif k == "FCL":
            w = ins[1]
            bias = val[ins[2]["id"]] if len(ins) > 2 and ins[2] is not None else None
            kk = int(np.prod(x["shape"][:a["axis"] + 1]))
            m = int(np.prod(x["shape"][a["axis"] + 1:]))
            y = fully_connected(xv, val[w["id"]], bias, m=m, k=kk, n=w["shape"][-1],
                                in_dtype=DTYPE_CODE[x["dtype"]], w_dtype=DTYPE_CODE[w["dtype"]],
                                out_dtype=DTYPE_CODE[out["dtype"]], in_q=(s, z),
                                w_q=_q(w["quant"]), out_q=(so, zo))
        elif k == "POOL":
            lay = a.get("layout", "ANY")
            xshape, oshape = x["shape"], out["shape"]
            if lay in ACT_TO_WHCN:
                xv = transpose(xv, xshape, ACT_TO_WHCN[lay])
                xshape, oshape = _permuted(xshape, ACT_TO_WHCN[lay]), _permuted(oshape, ACT_TO_WHCN[lay])
            pad = _resolved_pad(dict(a, dilation=[1, 1]), pad4(xshape), a["ksize"])
            y = pool2d(xv, in_shape=pad4(xshape), out_shape=pad4(oshape),
                       ksize=a["ksize"], stride=a["stride"], pad_left=pad[0],
                       pad_top=pad[2], pool_type=POOL[a["pool_type"]],
                       dtype=DTYPE_CODE[x["dtype"]], in_q=(s, z), out_q=(so, zo))
            if lay in ACT_FROM_WHCN:
                y = transpose(y, oshape, ACT_FROM_WHCN[lay])
        elif k in ("RELU", "RELU6"):
            y = activation(ACT_RELU if k == "RELU" else ACT_RELU6, DTYPE_CODE[x["dtype"]], xv,
                           (s, z), (so, zo))
        elif k == "ADD":
            b = ins[1]
            sb, zb, _ = _q(b["quant"])
            y = add(DTYPE_CODE[x["dtype"]], xv, (s, z), val[b["id"]], (sb, zb), (so, zo))
        elif k == "SOFTMAX":
            c, inner = _softmax_view(x["shape"], a.get("sm_axis", 0))
            y = softmax(DTYPE_CODE[x["dtype"]], xv, c, a.get("beta", 1.0), (s, z), inner)
        elif k == "RESHAPE":
            y = xv
        elif k == "TRANSPOSE":
            y = transpose(xv, x["shape"], a["perm"])
        elif k == "DATACONVERT":
            y = convert(xv, DTYPE_CODE[x["dtype"]], (s, z), DTYPE_CODE[out["dtype"]], (so, zo))
        else:
            raise NotImplementedError(k)
        val[out["id"]] = y
    return val if keep_all else val[graph["output"]]
