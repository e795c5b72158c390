#!/usr/bin/env python3
"""Benchmark of the quantized convolution hot path on one MI355X.

A step = one pass of the hot path over one batch of synthetic input that is
already resident in HBM. The headline workload is the configuration the metric is quoted on:
one uint8 per-tensor Conv2d 3x3 64->64 on 56x56 at batch 32, SAME padding, fused
ReLU6. Prints ONE JSON line (metric: int8 conv TOPS) carrying the dominant
kernel's roofline and a CPU baseline timed on the host cores; `extra` holds the
same measurements for the other single-operator configurations.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

REPO = os.path.dirname(os.path.abspath(__file__))
for p in (REPO, os.path.join(REPO, "oracle"), os.path.join(REPO, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, 5.0 POP/s
PEAK_F16_TFLOPS = 2500.0  # MI355X dense fp16 MFMA, 2.5 PFLOP/s
PEAK_HBM_GBS = 8000.0     # HBM3E, 8 TB/s
SEED = 0x71


def _same(a, b, float_tol=None):
    if float_tol is None:
        return bool(np.array_equal(a, b))
    return bool(np.allclose(a.astype(np.float32), b.astype(np.float32), rtol=float_tol, atol=float_tol))


def conv_check(x, wt, b, kws, batch, float_tol=None):
    """The GPU result of the batch's first image against the CPU restatement of the same operator."""
    def check(gpu_out):
        import tvx_oracle as O
        k1 = dict(kws, in_shape=kws["in_shape"][:3] + [1], out_shape=kws["out_shape"][:3] + [1])
        ref = O.conv2d(np.ascontiguousarray(x[:x.size // batch]), wt, b, **k1)
        return _same(ref, gpu_out[:ref.size], float_tol)
    return check


def fc_check(x, wt, b, kws, rows=32, float_tol=None):
    """The first `rows` rows of the GPU result against the CPU restatement."""
    def check(gpu_out):
        import tvx_oracle as O
        ref = O.fully_connected(np.ascontiguousarray(x[:rows * kws["k"]]), wt, b, **dict(kws, m=rows))
        return _same(ref, gpu_out[:ref.size], float_tol)
    return check


def conv_cfg2(T, rng, batch=32):
    n, c, h, w, oc = batch, 64, 56, 56, 64
    x = rng.integers(0, 256, n * c * h * w, dtype=np.uint8)
    wt = rng.integers(0, 256, oc * c * 9, dtype=np.uint8)
    b = rng.integers(-4096, 4097, oc).astype(np.int32)
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 3
    d.out_w, d.out_h, d.out_c = w, h, oc
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.pad_left = d.pad_top = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.U8
    d.in_scale, d.in_zp, d.w_scale, d.w_zp = 0.05, 128, 0.01, 120
    d.out_scale, d.out_zp, d.activation = 0.1, 0, T.ACT_RELU6
    op = T.conv2d_create(d, wt, b)
    macs = n * h * w * oc * c * 9
    algo_bytes = x.size + n * oc * h * w + wt.size + 4 * oc
    oracle_kws = dict(in_shape=[w, h, c, n], w_shape=[3, 3, c, oc], out_shape=[w, h, oc, n],
                      stride=[1, 1], dilation=[1, 1], pad_left=1, pad_top=1, multiplier=0,
                      in_dtype=0, w_dtype=0, out_dtype=0, in_q=(0.05, 128), w_q=(0.01, 120, None),
                      out_q=(0.1, 0), act=2)
    return dict(name="conv2d_u8_3x3_64to64_56x56_b%d_same_relu6" % n, op=op, inputs=(x,), out_elems=n * oc * h * w,
                out_dtype=np.uint8, ops=2 * macs, algo_bytes=algo_bytes, bound="mfma",
                oracle=("conv2d", (x, wt, b), oracle_kws, n), check=conv_check(x, wt, b, oracle_kws, n))


def conv_cfg2_b256(T, rng):
    """The headline convolution at batch 256: eight times the work per launch, where the launch's fixed cost
    (about 4 us) and the pipeline's fill no longer dominate."""
    return conv_cfg2(T, rng, batch=256)


def conv_f16(T, rng):
    """The headline convolution's shape in float16 (float32 accumulation)."""
    n, c, h, w, oc = 32, 64, 56, 56, 64
    x = rng.standard_normal(n * c * h * w, dtype=np.float32).astype(np.float16)
    wt = (rng.standard_normal(oc * c * 9, dtype=np.float32) * 0.05).astype(np.float16)
    b = rng.standard_normal(oc).astype(np.float32)
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 3
    d.out_w, d.out_h, d.out_c = w, h, oc
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.pad_left = d.pad_top = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.F16
    d.activation = T.ACT_RELU6
    op = T.conv2d_create(d, wt, b)
    kws = dict(in_shape=[w, h, c, n], w_shape=[3, 3, c, oc], out_shape=[w, h, oc, n], stride=[1, 1], dilation=[1, 1],
               pad_left=1, pad_top=1, multiplier=0, in_dtype=2, w_dtype=2, out_dtype=2, act=2)
    return dict(name="conv2d_f16_3x3_64to64_56x56_b32_same_relu6", op=op, inputs=(x,), out_elems=n * oc * h * w,
                out_dtype=np.float16, ops=2 * n * h * w * oc * c * 9, algo_bytes=2 * (x.size + n * oc * h * w + wt.size) + 4 * oc,
                bound="mfma", peak=PEAK_F16_TFLOPS, oracle=None, check=conv_check(x, wt, b, kws, n, float_tol=1e-2))


def conv_grouped(T, rng):
    """A grouped convolution (4 groups of 32 -> 32 channels, 3x3, 28x28, batch 32), u8 per-tensor."""
    n, c, h, w, oc, groups = 32, 128, 28, 28, 128, 4
    x = rng.integers(0, 256, n * c * h * w, dtype=np.uint8)
    wt = rng.integers(0, 256, oc * (c // groups) * 9, dtype=np.uint8)
    b = rng.integers(-4096, 4097, oc).astype(np.int32)
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 3
    d.out_w, d.out_h, d.out_c = w, h, oc
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.pad_left = d.pad_top = 1
    d.groups = groups
    d.in_dtype = d.w_dtype = d.out_dtype = T.U8
    d.in_scale, d.in_zp, d.w_scale, d.w_zp = 0.05, 128, 0.01, 120
    d.out_scale, d.out_zp, d.activation = 0.1, 0, T.ACT_RELU6
    op = T.conv2d_create(d, wt, b)
    return dict(name="grouped_conv2d_u8_3x3_4x32to32_28x28_b32_same_relu6", op=op, inputs=(x,),
                out_elems=n * oc * h * w, out_dtype=np.uint8, ops=2 * n * h * w * oc * (c // groups) * 9,
                algo_bytes=x.size + n * oc * h * w + wt.size + 4 * oc, bound="mfma", oracle=None,
                check=conv_check(x, wt, b, dict(in_shape=[w, h, c, n], w_shape=[3, 3, c // groups, oc], out_shape=[w, h, oc, n],
                                                stride=[1, 1], dilation=[1, 1], pad_left=1, pad_top=1, multiplier=0, groups=groups,
                                                in_dtype=0, w_dtype=0, out_dtype=0, in_q=(0.05, 128), w_q=(0.01, 120, None),
                                                out_q=(0.1, 0), act=2), n))


def fc_cfg5(T, rng):
    m, k, n = 8192, 4096, 4096
    x = rng.integers(-128, 128, m * k, dtype=np.int8)
    wt = rng.integers(-128, 128, n * k, dtype=np.int8)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    ws = np.exp(rng.uniform(np.log(0.001), np.log(0.02), n)).astype(np.float32)
    d = T.FcDesc()
    d.m, d.k, d.n = m, k, n
    d.in_dtype = d.w_dtype = d.out_dtype = T.I8
    d.in_scale, d.in_zp = 0.02, 0
    import ctypes as C
    d.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = 0.05, 0
    op = T.fully_connected_create(d, wt, b)
    return dict(name="fc_i8_per_channel_m8192_k4096_n4096", op=op, inputs=(x,), out_elems=m * n,
                out_dtype=np.int8, ops=2 * m * k * n, algo_bytes=m * k + n * k + m * n + 4 * n,
                bound="mfma", oracle=None,
                check=fc_check(x, wt, b, dict(k=k, n=n, in_dtype=1, w_dtype=1, out_dtype=1, in_q=(0.02, 0), w_q=(1.0, 0, ws),
                                              out_q=(0.05, 0))))


def fc_cfg5_u8(T, rng):
    """The same shape with uint8 activations and uint8 weights under a uniform zero point: the operand kinds of
    the reference's own quantized tests (the kernel re-biases the activations and sums their rows on its way)."""
    m, k, n = 8192, 4096, 4096
    x = rng.integers(0, 256, m * k, dtype=np.uint8)
    wt = rng.integers(0, 256, n * k, dtype=np.uint8)
    b = rng.integers(-16384, 16385, n).astype(np.int32)
    d = T.FcDesc()
    d.m, d.k, d.n = m, k, n
    d.in_dtype = d.w_dtype = d.out_dtype = T.U8
    d.in_scale, d.in_zp = 0.02, 121
    d.w_scale, d.w_zp = 0.01, 131
    d.out_scale, d.out_zp = 1.2, 128
    op = T.fully_connected_create(d, wt, b)
    return dict(name="fc_u8_asymmetric_m8192_k4096_n4096", op=op, inputs=(x,), out_elems=m * n,
                out_dtype=np.uint8, ops=2 * m * k * n, algo_bytes=m * k + n * k + m * n + 4 * n,
                bound="mfma", oracle=None,
                check=fc_check(x, wt, b, dict(k=k, n=n, in_dtype=0, w_dtype=0, out_dtype=0, in_q=(0.02, 121), w_q=(0.01, 131, None),
                                              out_q=(1.2, 128))))


def fc_cfg5_f16(T, rng):
    m, k, n = 8192, 4096, 4096
    x = rng.standard_normal(m * k, dtype=np.float32).astype(np.float16)
    wt = (rng.standard_normal(n * k, dtype=np.float32) * 0.02).astype(np.float16)
    b = rng.standard_normal(n).astype(np.float32)
    d = T.FcDesc()
    d.m, d.k, d.n = m, k, n
    d.in_dtype = d.w_dtype = d.out_dtype = T.F16
    op = T.fully_connected_create(d, wt, b)
    return dict(name="fc_f16_m8192_k4096_n4096", op=op, inputs=(x,), out_elems=m * n,
                out_dtype=np.float16, ops=2 * m * k * n, algo_bytes=2 * (m * k + n * k + m * n) + 4 * n,
                bound="mfma", peak=PEAK_F16_TFLOPS, oracle=None,
                check=fc_check(x, wt, b, dict(k=k, n=n, in_dtype=2, w_dtype=2, out_dtype=2), float_tol=1e-2))


def dw_cfg3a(T, rng):
    n, c, h, w = 32, 32, 112, 112
    x = rng.integers(-128, 128, n * c * h * w, dtype=np.int8)
    wt = rng.integers(-128, 128, c * 9, dtype=np.int8)
    b = rng.integers(-4096, 4097, c).astype(np.int32)
    ws = np.exp(rng.uniform(np.log(0.002), np.log(0.05), c)).astype(np.float32)
    import ctypes as C
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 3
    d.out_w, d.out_h, d.out_c = w, h, c
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.pad_left = d.pad_top = 1
    d.multiplier = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.I8
    d.in_scale, d.in_zp = 0.03, 0
    d.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = 0.08, 0
    op = T.conv2d_create(d, wt, b)
    return dict(name="depthwise3x3_i8_per_channel_112x112x32_b32", op=op, inputs=(x,), out_elems=x.size,
                out_dtype=np.int8, ops=2 * x.size * 9, algo_bytes=2 * x.size + wt.size + 4 * c,
                bound="hbm", oracle=None,
                check=conv_check(x, wt, b, dict(in_shape=[w, h, c, n], w_shape=[3, 3, 1, c], out_shape=[w, h, c, n], stride=[1, 1],
                                                dilation=[1, 1], pad_left=1, pad_top=1, multiplier=1, in_dtype=1, w_dtype=1,
                                                out_dtype=1, in_q=(0.03, 0), w_q=(1.0, 0, ws), out_q=(0.08, 0)), n))


def pw_cfg3b(T, rng):
    n, c, h, w, oc = 32, 32, 112, 112, 64
    x = rng.integers(-128, 128, n * c * h * w, dtype=np.int8)
    wt = rng.integers(-128, 128, oc * c, dtype=np.int8)
    b = rng.integers(-4096, 4097, oc).astype(np.int32)
    ws = np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32)
    import ctypes as C
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 1
    d.out_w, d.out_h, d.out_c = w, h, oc
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.I8
    d.in_scale, d.in_zp = 0.08, 0
    d.w_scales = ws.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp, d.activation = 0.05, 0, T.ACT_RELU6
    op = T.conv2d_create(d, wt, b)
    return dict(name="pointwise1x1_i8_per_channel_32to64_112x112_b32_relu6", op=op, inputs=(x,),
                out_elems=n * oc * h * w, out_dtype=np.int8, ops=2 * n * h * w * c * oc,
                algo_bytes=x.size + n * oc * h * w + wt.size + 4 * oc, bound="hbm", oracle=None,
                check=conv_check(x, wt, b, dict(in_shape=[w, h, c, n], w_shape=[1, 1, c, oc], out_shape=[w, h, oc, n], stride=[1, 1],
                                                dilation=[1, 1], pad_left=0, pad_top=0, multiplier=0, in_dtype=1, w_dtype=1,
                                                out_dtype=1, in_q=(0.08, 0), w_q=(1.0, 0, ws), out_q=(0.05, 0), act=2), n))


def pool_workload(T, rng, name, in_shape, k, stride, pool_type, dtype=0):
    w, h, c, n = in_shape
    ow, oh = (w - k) // stride + 1, (h - k) // stride + 1
    x = rng.integers(0, 256, w * h * c * n, dtype=np.uint8)
    d = T.Pool2dDesc()
    d.in_w, d.in_h, d.channels, d.batch = w, h, c, n
    d.out_w, d.out_h = ow, oh
    d.k_w = d.k_h = k
    d.stride_w = d.stride_h = stride
    d.pool_type, d.dtype = pool_type, dtype
    d.in_scale, d.in_zp, d.out_scale, d.out_zp = 0.05, 3, 0.05, 3
    op = T.pool2d_create(d)

    def check(gpu_out):
        import tvx_oracle as O
        ref = O.pool2d(np.ascontiguousarray(x[:w * h * c]), in_shape=[w, h, c, 1], out_shape=[ow, oh, c, 1], ksize=[k, k],
                       stride=[stride, stride], pad_left=0, pad_top=0, pool_type=pool_type, dtype=dtype, in_q=(0.05, 3), out_q=(0.05, 3))
        return _same(ref, gpu_out[:ref.size])
    return dict(name=name, op=op, inputs=(x,), out_elems=ow * oh * c * n, out_dtype=np.uint8,
                ops=w * h * c * n, algo_bytes=x.size + ow * oh * c * n, bound="hbm", oracle=None, check=check)


def pool_lenet_b256(T, rng):
    return pool_workload(T, rng, "maxpool2x2_s2_u8_24x24x20_b256", [24, 24, 20, 256], 2, 2, T.POOL_MAX)


def pool_3x3_s2(T, rng):
    return pool_workload(T, rng, "maxpool3x3_s2_u8_112x112x64_b32", [112, 112, 64, 32], 3, 2, T.POOL_MAX)


def pool_global_avg(T, rng):
    return pool_workload(T, rng, "avgpool7x7_u8_7x7x1280_b64", [7, 7, 1280, 64], 7, 7, T.POOL_AVG)


def dwpw_cfg3(T, rng):
    """The depthwise 3x3 and the pointwise convolution behind it as one operator: the 112x112x32 tensor between them
    stays on the chip (38.54 MB of compulsory traffic instead of 64.2 MB for the two operators)."""
    import ctypes as C
    n, c, h, w, oc = 32, 32, 112, 112, 64
    x = rng.integers(-128, 128, n * c * h * w, dtype=np.int8)
    wd = rng.integers(-128, 128, c * 9, dtype=np.int8)
    bd = rng.integers(-4096, 4097, c).astype(np.int32)
    sd = np.exp(rng.uniform(np.log(0.002), np.log(0.05), c)).astype(np.float32)
    wp = rng.integers(-128, 128, oc * c, dtype=np.int8)
    bp = rng.integers(-4096, 4097, oc).astype(np.int32)
    sp = np.exp(rng.uniform(np.log(0.002), np.log(0.05), oc)).astype(np.float32)
    d = T.Conv2dDesc()
    d.in_w, d.in_h, d.in_c, d.batch = w, h, c, n
    d.k_w = d.k_h = 3
    d.out_w, d.out_h, d.out_c = w, h, c
    d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.pad_left = d.pad_top = 1
    d.multiplier = 1
    d.in_dtype = d.w_dtype = d.out_dtype = T.I8
    d.in_scale, d.in_zp = 0.03, 0
    d.w_scales = sd.ctypes.data_as(C.POINTER(C.c_float))
    d.out_scale, d.out_zp = 0.08, 0
    p = T.Conv2dDesc()
    p.in_w, p.in_h, p.in_c, p.batch = w, h, c, n
    p.k_w = p.k_h = 1
    p.out_w, p.out_h, p.out_c = w, h, oc
    p.stride_w = p.stride_h = p.dilation_w = p.dilation_h = 1
    p.in_dtype = p.w_dtype = p.out_dtype = T.I8
    p.in_scale, p.in_zp = 0.08, 0
    p.w_scales = sp.ctypes.data_as(C.POINTER(C.c_float))
    p.out_scale, p.out_zp, p.activation = 0.05, 0, T.ACT_RELU6
    op = T.conv2d_dw_pw_create(d, wd, bd, p, wp, bp)

    def check(gpu_out):
        import tvx_oracle as O
        common = dict(stride=[1, 1], dilation=[1, 1], in_dtype=1, w_dtype=1, out_dtype=1)
        mid = O.conv2d(np.ascontiguousarray(x[:c * h * w]), wd, bd, in_shape=[w, h, c, 1], w_shape=[3, 3, 1, c], out_shape=[w, h, c, 1],
                       pad_left=1, pad_top=1, multiplier=1, in_q=(0.03, 0), w_q=(1.0, 0, sd), out_q=(0.08, 0), **common)
        ref = O.conv2d(mid, wp, bp, in_shape=[w, h, c, 1], w_shape=[1, 1, c, oc], out_shape=[w, h, oc, 1], pad_left=0, pad_top=0,
                       multiplier=0, in_q=(0.08, 0), w_q=(1.0, 0, sp), out_q=(0.05, 0), act=2, **common)
        return _same(ref, gpu_out[:ref.size])
    return dict(check=check, name="depthwise3x3_then_pointwise1x1_i8_per_channel_112x112x32to64_b32_relu6", op=op, inputs=(x,),
                out_elems=n * oc * h * w, out_dtype=np.int8, ops=2 * n * h * w * c * (9 + oc),
                algo_bytes=x.size + n * oc * h * w + wd.size + wp.size + 4 * (c + oc), bound="hbm", oracle=None)


def time_workload(wl, steps, warmup, ring_bytes=0):
    """Returns (wall ms per step over exactly `steps` steps, mean kernel ms per launch). With ring_bytes the
    launches rotate over as many copies of the input and output tensors as make up that many bytes, so that
    no launch finds its operands in a cache (the memory-side cache holds 256 MB)."""
    import torch
    stream = torch.cuda.current_stream()
    dev_in = [torch.from_numpy(a).cuda() for a in wl["inputs"]]
    tdt = {np.uint8: torch.uint8, np.int8: torch.int8, np.float16: torch.float16}[wl["out_dtype"]]
    out = torch.empty(wl["out_elems"], dtype=tdt, device="cuda")
    op = wl["op"]
    in1 = dev_in[1] if len(dev_in) > 1 else None
    if ring_bytes:
        per = dev_in[0].numel() * dev_in[0].element_size() + out.numel() * out.element_size()
        copies = max(2, -(-ring_bytes // per))
        ins = [dev_in[0]] + [dev_in[0].clone() for _ in range(copies - 1)]
        outs = [out] + [torch.empty_like(out) for _ in range(copies - 1)]
        for i in range(max(warmup, copies)):
            op.run(ins[i % copies], in1, outs[i % copies], stream.cuda_stream)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0 = time.perf_counter()
        e0.record(stream)
        for i in range(steps):
            op.run(ins[i % copies], in1, outs[i % copies], stream.cuda_stream)
        e1.record(stream)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps, e0.elapsed_time(e1) / steps
    for _ in range(warmup):
        op.run(dev_in[0], in1, out, stream.cuda_stream)
    torch.cuda.synchronize()
    # The timed region: exactly `steps` launches, one kernel each, back to back on one
    # stream. Wall clock brackets it with synchronisation on both sides; a HIP event pair
    # recorded on the launch stream brackets the same region for the kernel's average
    # launch duration (per-launch event pairs would add their own ~2 us to each sample).
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record(stream)
    for _ in range(steps):
        op.run(dev_in[0], in1, out, stream.cuda_stream)
    e1.record(stream)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / steps
    kernel_ms = e0.elapsed_time(e1) / steps
    wl["device_out"] = out
    return wall_ms, kernel_ms


KERNEL_SOURCES = {"conv2d_igemm_i8": "conv_igemm_i8.hip", "conv2d_igemm_i8_persistent": "conv_igemm_i8.hip", "conv2d_band_i8": "conv_band_i8.hip",
                  "fc_mfma_i8_256x256x128": "fc_mfma_i8.hip", "fc_mfma_i8_128x256x128": "fc_mfma_i8.hip", "fc_mfma_f16_256x256x64": "fc_mfma_i8.hip",
                  "dwconv3x3_i8": "dwconv3x3_i8.hip", "pwconv_i8": "pwconv_i8.hip", "pwconv_i8_stream": "pwconv_i8.hip", "dwconv3x3_pwconv_i8": "dwpw_i8.hip", "pool2d_rows_i8": "pool2d_i8.hip", "pool2d_stencil_i8": "pool2d_stencil_i8.hip",
                  "conv2d_gemm_i8": "conv_gemm.hip", "conv2d_gemm_f16": "conv_gemm.hip", "conv2d_igemm_f16": "conv_igemm_f16.hip",
                  "avgpool_plane_i8": "kernels_generic.hip"}


def kernel_source_sha256(kernel_name):
    import hashlib
    f = KERNEL_SOURCES.get(kernel_name)
    path = os.path.join(REPO, "tim-vx_amd", "csrc", f) if f else None
    if not path or not os.path.exists(path):
        return None
    return hashlib.sha256(open(path, "rb").read()).hexdigest()


def roofline(wl, kernel_ms, traffic=None):
    if wl["bound"] == "mfma":
        achieved = wl["ops"] / (kernel_ms * 1e-3) / 1e12
        peak = wl.get("peak", PEAK_INT8_TOPS)
        return dict(bound="mfma", achieved=round(achieved, 3), peak=peak,
                    unit="TFLOP/s" if "peak" in wl else "TOP/s", frac=round(achieved / peak, 5), traffic=traffic)
    achieved = wl["algo_bytes"] / (kernel_ms * 1e-3) / 1e9
    return dict(bound="hbm", achieved=round(achieved, 2), peak=PEAK_HBM_GBS, unit="GB/s",
                frac=round(achieved / PEAK_HBM_GBS, 5), traffic=traffic)


def cpu_baseline(wl, gpu_out):
    """The CPU restatement (oracle, OpenMP) on a bounded sample of the same workload:
    the first `sample_n` images of the batch; also re-checks the GPU result on them."""
    import tvx_oracle as O
    kind, arrays, kws, batch = wl["oracle"]
    sample_n = batch  # the whole batch, repeated until about 10 s of CPU time have passed
    x, wt, b = arrays
    per_img = x.size // batch
    kws = dict(kws)
    O.conv2d(np.ascontiguousarray(x[:per_img]), wt, b,
             **dict(kws, in_shape=kws["in_shape"][:3] + [1], out_shape=kws["out_shape"][:3] + [1]))  # warm-up
    reps, dt = 0, 0.0
    while dt < 10.0 and reps < 50:
        t0 = time.perf_counter()
        ref = O.conv2d(x, wt, b, **kws)
        dt += time.perf_counter() - t0
        reps += 1
    dt /= reps
    ok = bool(np.array_equal(ref, gpu_out[:ref.size]))
    tops = wl["ops"] * sample_n / batch / dt / 1e12
    # the same code on one thread, on the first two images of the batch (about 5 s)
    threads = O.lib().tvxo_num_threads()
    O.lib().tvxo_set_num_threads(1)
    n1 = min(2, batch)
    k1 = dict(kws, in_shape=kws["in_shape"][:3] + [n1], out_shape=kws["out_shape"][:3] + [n1])
    x1 = np.ascontiguousarray(x[:per_img * n1])
    reps1, dt1 = 0, 0.0
    while dt1 < 5.0 and reps1 < 20:
        t0 = time.perf_counter()
        O.conv2d(x1, wt, b, **k1)
        dt1 += time.perf_counter() - t0
        reps1 += 1
    O.lib().tvxo_set_num_threads(threads)
    tops1 = wl["ops"] * n1 / batch / (dt1 / reps1) / 1e12
    return dict(value=round(tops, 5), unit="TOPS", cores=threads, kind="port",
                sample="the same %d-image conv, %d repetitions of %.3f s each; CPU restatement in C with OpenMP "
                       "(not the vendor simulator, which cannot run here); GPU output equal to it: %s"
                       % (batch, reps, dt, ok),
                one_thread=dict(value=round(tops1, 5), unit="TOPS", cores=1,
                                sample="the first %d images, %d repetitions of %.3f s each" % (n1, reps1, dt1 / reps1))), ok


def network_extras(steps, warmup):
    """LeNet (the reference's CPU-runnable sample) and MobileNetV2 at batch 64 through the
    tim::vx C++ API: images/s per Graph::Run(), whole call (host copies of the graph's input
    and output included) and operator sequence alone."""
    import tempfile
    GF = importlib.import_module("tim-vx_amd.graphfile")
    G = importlib.import_module("tim-vx_amd.graphs")
    z = np.load(os.path.join(REPO, "tests", "golden", "lenet_asymu8.npz"))
    nets = [("lenet_asymu8_b1", G.lenet_asymu8(z["weights"], z["input"], batch=1), 1),
            ("lenet_asymu8_b256", G.lenet_asymu8(z["weights"], z["input"], batch=256), 256),
            ("lenet_random_b256", G.lenet_random(batch=256), 256),   # seeded synthetic parameters instead of the sample's
            ("mobilenet_v2_u8_b64_224", G.mobilenet_v2(batch=64, res=224), 64),
            # the headline convolution as an application reaches it: through the C++ API, with the host copies
            # of its input and output (run_ms is the PCIe-inclusive time, device_ms the operator alone)
            ("conv3x3_u8_64to64_56x56_b32_cpp_api", G.conv3x3_same_relu6(), 32)]
    out = {}
    with tempfile.TemporaryDirectory() as d:
        _, info, _ = GF.run_graphs([g for _, g, _ in nets], d, bench=(warmup, steps))
    # LeNet layer by layer (device time stamps around every operator; a run of its own: the stamps cost time)
    with tempfile.TemporaryDirectory() as d:
        _, opinfo, _ = GF.run_graphs([g for _, g, _ in nets[:3]], d, bench=(warmup, steps), env={"TVX_RUNTIME_PROFILE": "ops"})
    for name, g, batch in nets:
        i = info.get(g["test"], {})
        if "run_ms" not in i:
            out[name] = {"error": i.get("fail", "no timing")}
            continue
        out[name] = {"images_per_s": round(batch / (i["run_ms"] * 1e-3), 1),
                     "images_per_s_device": round(batch / (i["device_ms"] * 1e-3), 1),
                     "run_ms": round(i["run_ms"], 4), "device_ms": round(i["device_ms"], 4),
                     "tops_device": round(2 * G.mac_count(g) / (i["device_ms"] * 1e-3) / 1e12, 2)}
        ops_us = opinfo.get(g["test"], {}).get("ops_us")
        if ops_us and name.startswith("lenet"):
            out[name]["per_layer_us"] = [[k, round(v, 2)] for k, v in ops_us]
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-extra", action="store_true", help="skip the non-headline workloads")
    ap.add_argument("--no-networks", action="store_true",
                    help="skip the LeNet / MobileNetV2 runs (child processes) and the device calibration")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="run only a plain 256 MiB device copy, 10 times (scales the HBM byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)")
    import torch
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU: the hot path has no CPU fallback")
    if args.copy_calibration:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda").fill_(3)
        dst = torch.empty_like(src)
        for _ in range(10):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"copy_bytes": 256 << 20, "repeats": 10}))
        return
    T = importlib.import_module("tim-vx_amd")
    rng = np.random.default_rng(SEED)

    wl = conv_cfg2(T, rng)
    wall_ms, kernel_ms = time_workload(wl, args.steps, args.warmup)
    gpu_out = wl["device_out"].cpu().numpy()
    cpu, parity_ok = cpu_baseline(wl, gpu_out)
    # measured HBM bytes per launch (scaled FETCH_SIZE + WRITE_SIZE), kept per kernel and workload
    tmap = {}
    tpath = os.path.join(REPO, "profiles", "traffic.json")
    if os.path.exists(tpath):
        tmap = json.load(open(tpath))

    stale = []

    def traffic_of(w):
        """Measured HBM bytes per launch of this kernel on this workload (profiles/traffic.json), or None. The
        record carries the hash of the kernel's source file at the time of the measurement: when the source has
        changed since, the figure is still reported but flagged (stderr and `traffic_stale`)."""
        rec = tmap.get(w["op"].kernel_name + "|" + w["name"]) or tmap.get(w["op"].kernel_name, {})
        if rec.get("workload") != w["name"]:
            return None
        if rec.get("source_sha256") != kernel_source_sha256(w["op"].kernel_name):
            stale.append(w["op"].kernel_name)
            sys.stderr.write("bench.py: profiles/traffic.json predates the current source of %s: re-measure\n"
                             % w["op"].kernel_name)
        return rec.get("bytes_per_launch")

    traffic = traffic_of(wl)
    line = {
        "metric": "int8 conv TOPS", "value": round(wl["ops"] / (wall_ms * 1e-3) / 1e12, 3), "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "u8",
        "data": "synthetic",
        "config": {"workload": wl["name"], "kernel": wl["op"].kernel_name, "batch": 32,
                   "parity_vs_oracle_on_sample": parity_ok},
        "roofline": dict(roofline(wl, kernel_ms, traffic), kernel=wl["op"].kernel_name,
                         kernel_ms=round(kernel_ms, 5)),
        "cpu_baseline": cpu,
    }
    if stale:
        line["roofline"]["traffic_stale"] = True
    if not args.no_extra:
        extra = {}
        for make in (fc_cfg5, fc_cfg5_u8, fc_cfg5_f16, dw_cfg3a, pw_cfg3b, dwpw_cfg3, conv_cfg2_b256, conv_f16, conv_grouped, pool_3x3_s2,
                     pool_lenet_b256, pool_global_avg):
            w2 = make(T, rng)
            steps2 = max(5, min(args.steps, 50))
            wall2, k2 = time_workload(w2, steps2, min(args.warmup, 5))
            # the first image (or rows) of the result against the CPU restatement, before any figure is reported
            checked = w2["check"](w2["device_out"].cpu().numpy()) if w2.get("check") else None
            rec = dict(kernel=w2["op"].kernel_name, parity_vs_oracle_on_sample=checked, ms_per_step=round(wall2, 5),
                       tops=round(w2["ops"] / (wall2 * 1e-3) / 1e12, 2),
                       gbs=round(w2["algo_bytes"] / (wall2 * 1e-3) / 1e9, 1),
                       roofline=dict(roofline(w2, k2, traffic_of(w2)), kernel_ms=round(k2, 5)))
            if w2["bound"] == "hbm":
                # The roofline of a bandwidth-bound kernel is quoted on launches that rotate over 640 MB of
                # operands: re-run in place, a 26 or 39 MB working set may be served by the memory-side cache.
                _, k3 = time_workload(w2, steps2, min(args.warmup, 5), ring_bytes=640 << 20)
                rec["roofline_in_place"] = rec["roofline"]
                rec["roofline"] = dict(roofline(w2, k3, traffic_of(w2)), kernel_ms=round(k3, 5),
                                       operands="rotating over 640 MB of input / output copies")
            extra[w2["name"]] = rec
        if args.no_networks:
            line["extra"] = extra
            line["children_at_exit"] = reap_children()
            print(json.dumps(line))
            return
        extra.update(network_extras(max(5, min(args.steps, 30)), 3))
        # what this very device sustains with the simplest kernels: the int8 matrix cores on
        # zeros (nominal clock) and on random bytes (the clock held under load), a streaming copy
        extra["device_calibration"] = {
            "mfma_i8_tops_zero_operands": round(T.calibrate_mfma_i8(False), 0),
            "mfma_i8_tops_random_operands": round(T.calibrate_mfma_i8(True), 0),
            "copy_read_plus_write_gbs": round(T.calibrate_copy(), 0),
            # the same copy kernel on the depthwise workload's bytes (12.8 MB in, 12.8 MB out), launched back to
            # back in place: what a launch of that size can reach with the per-launch floor under it
            "copy_12p8MB_read_plus_write_gbs": round(T.calibrate_copy(12845056, 50), 0),
        }
        line["extra"] = extra
    line["children_at_exit"] = reap_children()
    print(json.dumps(line))


def reap_children():
    """Nothing may outlive the benchmark: every child process this run started (the graph runner, a build step)
    has been waited for; whatever is still there is ended and counted."""
    try:
        import psutil
    except ImportError:
        return None
    left = psutil.Process().children(recursive=True)
    for p in left:
        try:
            p.kill()
        except psutil.Error:
            pass
    psutil.wait_procs(left, timeout=5)
    return len(left)


if __name__ == "__main__":
    main()
