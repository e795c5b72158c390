"""Shared helpers: fixture loading, and running one operator through the C ABI
with torch tensors as device memory (plumbing only: torch computes nothing)."""
import ctypes as C
import importlib
import json
import os

import numpy as np

import tvx_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
GOLDEN_FILES = ["conv2d", "depthwise_conv", "grouped_conv2d", "conv1d", "fullyconnected", "max_pool", "avg_pool", "softmax",
                "transpose", "dataconvert", "layout_inference",
                "deconv2d", "grouped_conv1d", "deconv1d"]


def load_cases(name):
    with open(os.path.join(HERE, "golden", name + ".json")) as f:
        return json.load(f)


def all_cases():
    out = []
    for n in GOLDEN_FILES:
        for c in load_cases(n):
            out.append((n, c))
    return out


def case_id(item):
    n, c = item
    return "%s::%s[%d]" % (n, c["test"], c["index"])


def golden_of(case):
    t = {t["id"]: t for t in case["tensors"]}[case["output"]]
    return O.expand(case["golden"], t["dtype"])


def matches(case, out):
    g = golden_of(case)
    if case["compare"] == "eq":
        if np.issubdtype(np.asarray(g).dtype, np.floating):
            # EXPECT_EQ on float vectors (the reference's Softmax tests, which fall back to 1e-3 on
            # hardware with a different exp unit): equal up to the last bit or two - expf and the
            # division of another maths library round the odd result the other way
            g32 = np.asarray(g, dtype=np.float32)
            return bool(np.all(np.abs(np.asarray(out, dtype=np.float32) - g32) <= 2 * np.spacing(np.abs(g32))))
        return np.array_equal(out, g)
    return bool(np.all(np.abs(out.astype(np.float64) - g.astype(np.float64)) <= case["tol"] + 1e-12))


def tvx():
    return importlib.import_module("tim-vx_amd")


def to_device(arr):
    import torch
    return torch.from_numpy(np.ascontiguousarray(arr)).cuda()


def device_out(n, np_dtype):
    import torch
    tdt = {np.uint8: torch.uint8, np.int8: torch.int8, np.float16: torch.float16,
           np.float32: torch.float32}[np_dtype]
    return torch.empty(int(n), dtype=tdt, device="cuda")


NP_OF = {0: np.uint8, 1: np.int8, 2: np.float16, 3: np.float32}


def _wq(desc, w_q, keep):
    desc.w_scale, desc.w_zp = w_q[0], w_q[1]
    if w_q[2] is not None:
        ws = np.ascontiguousarray(w_q[2], dtype=np.float32)
        keep.append(ws)
        desc.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))


def gpu_conv2d(x, w, bias, *, in_shape, w_shape, out_shape, stride, dilation, pad_left, pad_top,
               multiplier, in_dtype, w_dtype, out_dtype, in_q=(1.0, 0), w_q=(1.0, 0, None),
               out_q=(1.0, 0), act=0, const_weights=True, want_kernel=None, groups=0, transposed=False, misalign=0):
    """misalign: byte offset of the activation and result tensors from their (256-byte aligned) allocations."""
    T = tvx()
    d = T.Conv2dDesc()
    d.groups = groups
    d.in_w, d.in_h, d.in_c, d.batch = in_shape
    d.k_w, d.k_h = w_shape[0], w_shape[1]
    d.out_w, d.out_h, d.out_c = out_shape[0], out_shape[1], out_shape[2]
    d.stride_w, d.stride_h = stride
    d.dilation_w, d.dilation_h = dilation
    d.pad_left, d.pad_top, d.multiplier = pad_left, pad_top, multiplier
    d.in_dtype, d.w_dtype, d.out_dtype = in_dtype, w_dtype, out_dtype
    d.in_scale, d.in_zp = in_q
    keep = []
    _wq(d, w_q, keep)
    d.out_scale, d.out_zp = out_q
    d.activation = act
    op = (T.deconv2d_create if transposed else T.conv2d_create)(d, w if const_weights else None, bias)
    if want_kernel is not None:
        assert op.kernel_name in ((want_kernel,) if isinstance(want_kernel, str) else want_kernel), op.kernel_name
    import torch
    xd = to_device(x)
    wd = None if const_weights else to_device(w)
    yd = device_out(np.prod(out_shape), NP_OF[out_dtype])
    if misalign:
        assert x.dtype.itemsize == 1 and NP_OF[out_dtype]().itemsize == 1
        xd = to_device(np.concatenate([np.zeros(misalign, x.dtype), x.reshape(-1)]))[misalign:]
        yd = device_out(np.prod(out_shape) + misalign, NP_OF[out_dtype])[misalign:]
        assert xd.data_ptr() % 256 == misalign and yd.data_ptr() % 256 == misalign
    op.run(xd, wd, yd)
    torch.cuda.synchronize()
    out = yd.cpu().numpy()
    op.close()
    return out


def gpu_fully_connected(x, w, bias, *, m, k, n, in_dtype, w_dtype, out_dtype, in_q=(1.0, 0),
                        w_q=(1.0, 0, None), out_q=(1.0, 0), act=0, const_weights=True,
                        want_kernel=None):
    T = tvx()
    d = T.FcDesc()
    d.m, d.k, d.n = m, k, n
    d.in_dtype, d.w_dtype, d.out_dtype = in_dtype, w_dtype, out_dtype
    d.in_scale, d.in_zp = in_q
    keep = []
    _wq(d, w_q, keep)
    d.out_scale, d.out_zp = out_q
    d.activation = act
    op = T.fully_connected_create(d, w if const_weights else None, bias)
    if want_kernel is not None:
        assert op.kernel_name == want_kernel, op.kernel_name
    import torch
    xd = to_device(x)
    wd = None if const_weights else to_device(w)
    yd = device_out(m * n, NP_OF[out_dtype])
    op.run(xd, wd, yd)
    torch.cuda.synchronize()
    out = yd.cpu().numpy()
    op.close()
    return out


def gpu_pool2d(x, *, in_shape, out_shape, ksize, stride, pad_left, pad_top, pool_type, dtype,
               in_q=(1.0, 0), out_q=(1.0, 0), want_kernel=None):
    T = tvx()
    d = T.Pool2dDesc()
    d.in_w, d.in_h, d.channels, d.batch = in_shape
    d.out_w, d.out_h = out_shape[0], out_shape[1]
    d.k_w, d.k_h = ksize
    d.stride_w, d.stride_h = stride
    d.pad_left, d.pad_top = pad_left, pad_top
    d.pool_type, d.dtype = pool_type, dtype
    d.in_scale, d.in_zp = in_q
    d.out_scale, d.out_zp = out_q
    op = T.pool2d_create(d)
    if want_kernel is not None:
        assert op.kernel_name == want_kernel, op.kernel_name
    import torch
    xd = to_device(x)
    yd = device_out(np.prod(out_shape), NP_OF[dtype])
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    out = yd.cpu().numpy()
    op.close()
    return out


def gpu_activation(act, dtype, x, in_q, out_q):
    T = tvx()
    d = T.EltwiseDesc()
    d.count, d.dtype, d.activation = x.size, dtype, act
    d.a_scale, d.a_zp = in_q
    d.out_scale, d.out_zp = out_q
    op = T.activation_create(d)
    import torch
    xd = to_device(x)
    yd = device_out(x.size, NP_OF[dtype])
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def gpu_add(dtype, a, a_q, b, b_q, out_q):
    T = tvx()
    d = T.EltwiseDesc()
    d.count, d.dtype = a.size, dtype
    d.a_scale, d.a_zp = a_q
    d.b_scale, d.b_zp = b_q
    d.out_scale, d.out_zp = out_q
    op = T.add_create(d)
    import torch
    ad, bd = to_device(a), to_device(b)
    yd = device_out(a.size, NP_OF[dtype])
    op.run(ad, bd, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def gpu_softmax(dtype, x, c, beta, in_q, inner=1):
    T = tvx()
    d = T.SoftmaxDesc()
    d.channels, d.rows, d.beta, d.in_dtype, d.inner = c, x.size // (c * inner), beta, dtype, inner
    d.in_scale, d.in_zp = in_q
    op = T.softmax_create(d)
    import torch
    xd = to_device(x)
    yd = device_out(x.size, np.float32)
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def gpu_convert(x, in_dtype, in_q, out_dtype, out_q):
    T = tvx()
    d = T.ConvertDesc()
    d.count, d.in_dtype, d.out_dtype = x.size, in_dtype, out_dtype
    d.in_scale, d.in_zp = in_q
    d.out_scale, d.out_zp = out_q
    op = T.convert_create(d)
    import torch
    xd = to_device(x)
    yd = device_out(x.size, NP_OF[out_dtype])
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def gpu_transpose(x, in_dims, perm):
    T = tvx()
    d = T.TransposeDesc()
    d.rank, d.elem_bytes = len(in_dims), x.dtype.itemsize
    for i, (n, p) in enumerate(zip(in_dims, perm)):
        d.in_dims[i], d.perm[i] = n, p
    op = T.transpose_create(d)
    import torch
    xd = to_device(x)
    yd = torch.empty_like(xd)
    op.run(xd, None, yd)
    torch.cuda.synchronize()
    return yd.cpu().numpy()


def run_case_gpu(case):
    """One-operator fixture graph through the C ABI; mirrors tvx_oracle.run_case."""
    tensors = {t["id"]: t for t in case["tensors"]}
    op = case["ops"][0]
    a = op["attrs"]
    ins = [tensors[i] for i in op["inputs"]]
    out = tensors[op["outputs"][0]]
    arr = [O.expand(t["data"], t["dtype"]) if t["data"] is not None else None for t in ins]
    code = O.DTYPE_CODE
    if op["kind"] == "CONV2D":
        x, w = ins[0], ins[1]
        s, z, _ = O._q(x["quant"])
        so, zo, _ = O._q(out["quant"])
        xs, wsh, osh = O._conv_shapes(a, x["shape"], w["shape"], out["shape"])
        return gpu_conv2d(arr[0], arr[1], arr[2] if len(ins) > 2 else None, in_shape=xs,
                          w_shape=wsh, out_shape=osh, stride=a["stride"],
                          dilation=a["dilation"], pad_left=a["pad"][0], pad_top=a["pad"][2],
                          multiplier=a["multiplier"], groups=a.get("groups", 0), in_dtype=code[x["dtype"]],
                          w_dtype=code[w["dtype"]], out_dtype=code[out["dtype"]], in_q=(s, z),
                          w_q=O._q(w["quant"]), out_q=(so, zo),
                          const_weights=(w["attr"] == "CONSTANT"))
    if op["kind"] == "DECONV2D":
        x, w = ins[0], ins[1]
        s, z, _ = O._q(x["quant"])
        so, zo, _ = O._q(out["quant"])
        xs, wsh, osh = O._conv_shapes(a, x["shape"], w["shape"], out["shape"])  # DeConv1d: rows of height one
        return gpu_conv2d(arr[0], arr[1], arr[2] if len(ins) > 2 else None, in_shape=xs, w_shape=wsh,
                          out_shape=osh, stride=a["stride"], dilation=[1, 1], pad_left=a["pad"][0],
                          pad_top=a["pad"][2], multiplier=0, groups=a.get("groups", 0), in_dtype=code[x["dtype"]],
                          w_dtype=code[w["dtype"]], out_dtype=code[out["dtype"]], in_q=(s, z),
                          w_q=O._q(w["quant"]), out_q=(so, zo), const_weights=(w["attr"] == "CONSTANT"),
                          transposed=True)
    if op["kind"] == "FCL":
        x, w = ins[0], ins[1]
        k = int(np.prod(x["shape"][:a["axis"] + 1]))
        m = int(np.prod(x["shape"][a["axis"] + 1:]))
        s, z, _ = O._q(x["quant"])
        so, zo, _ = O._q(out["quant"])
        return gpu_fully_connected(arr[0], arr[1], arr[2] if len(ins) > 2 else None, m=m, k=k,
                                   n=w["shape"][-1], in_dtype=code[x["dtype"]],
                                   w_dtype=code[w["dtype"]], out_dtype=code[out["dtype"]],
                                   in_q=(s, z), w_q=O._q(w["quant"]), out_q=(so, zo))
    if op["kind"] == "POOL":
        x = ins[0]
        s, z, _ = O._q(x["quant"])
        so, zo, _ = O._q(out["quant"])
        return gpu_pool2d(arr[0], in_shape=O.pad4(x["shape"]), out_shape=O.pad4(out["shape"]),
                          ksize=a["ksize"], stride=a["stride"], pad_left=a["pad"][0],
                          pad_top=a["pad"][2], pool_type=O.POOL[a["pool_type"]],
                          dtype=code[x["dtype"]], in_q=(s, z), out_q=(so, zo))
    if op["kind"] == "SOFTMAX":
        x = ins[0]
        s, z, _ = O._q(x["quant"])
        c, inner = O._softmax_view(x["shape"], a.get("sm_axis", 0))
        return gpu_softmax(code[x["dtype"]], arr[0], c, a.get("beta", 1.0), (s, z), inner)
    if op["kind"] == "TRANSPOSE":
        return gpu_transpose(arr[0], ins[0]["shape"], a["perm"])
    if op["kind"] == "DATACONVERT":
        s, z, _ = O._q(ins[0]["quant"])
        so, zo, _ = O._q(out["quant"])
        return gpu_convert(arr[0], code[ins[0]["dtype"]], (s, z), code[out["dtype"]], (so, zo))
    raise NotImplementedError(op["kind"])
