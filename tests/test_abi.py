"""The C-ABI library loads, exports every symbol include/tvx_hip.h declares, and
its host-only entry points behave (no GPU needed, no compute calls)."""
import ctypes as C
import os
import re

import pytest

REPO = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(REPO, "include", "tvx_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tvx_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(tvx):
    L = tvx.lib()
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(L, n), n


def test_host_only_entry_points(tvx, oracle):
    L = tvx.lib()
    assert b"gfx950" in L.tvx_version()
    assert L.tvx_status_string(-2) == b"unsupported"
    for m in (0.25, 1.0, 0.00037, 3.0, 1.0058823529):
        mult, shift = C.c_int32(), C.c_int32()
        assert L.tvx_quantize_multiplier(m, C.byref(mult), C.byref(shift)) == 0
        assert (mult.value, shift.value) == oracle.quantize_multiplier(m)
        for acc in (-123456, -1, 0, 1, 77, 2 ** 31 - 1, -2 ** 31):
            assert L.tvx_requantize(acc, mult.value, shift.value) == oracle.requant(acc, mult.value, shift.value)


def test_descriptor_validation_needs_no_gpu(tvx):
    d = tvx.Conv2dDesc()
    with pytest.raises(tvx.TvxError) as e:
        tvx.conv2d_create(d)
    assert e.value.status == tvx.E_INVALID
    f = tvx.FcDesc()
    f.m, f.k, f.n = 2, 3, 4
    f.in_dtype, f.w_dtype, f.out_dtype = tvx.I8, tvx.U8, tvx.I8
    with pytest.raises(tvx.TvxError) as e:
        tvx.fully_connected_create(f)
    assert e.value.status == tvx.E_UNSUPPORTED


def test_zero_points_outside_the_type_are_invalid(tvx):
    """A zero point is a code of its tensor's type; checked before any device work."""
    import numpy as np
    d = tvx.Conv2dDesc()
    d.in_w = d.in_h = d.out_w = d.out_h = 4
    d.in_c = d.out_c = 16
    d.batch = d.k_w = d.k_h = d.stride_w = d.stride_h = d.dilation_w = d.dilation_h = 1
    d.in_dtype = d.w_dtype = d.out_dtype = tvx.U8
    d.in_scale = d.w_scale = d.out_scale = 0.5
    w = np.zeros(256, dtype=np.uint8)
    for field, bad in (("in_zp", 256), ("w_zp", -1), ("out_zp", 300)):
        setattr(d, field, bad)
        with pytest.raises(tvx.TvxError) as e:
            tvx.conv2d_create(d, w, None)
        assert e.value.status == tvx.E_INVALID and "zero point" in str(e.value)
        setattr(d, field, 0)
    f = tvx.FcDesc()
    f.m, f.k, f.n = 2, 16, 4
    f.in_dtype = f.w_dtype = f.out_dtype = tvx.I8
    f.in_scale = f.w_scale = f.out_scale = 0.5
    f.out_zp = -129
    with pytest.raises(tvx.TvxError) as e:
        tvx.fully_connected_create(f, np.zeros(64, dtype=np.int8), None)
    assert e.value.status == tvx.E_INVALID
    p = tvx.Pool2dDesc()
    p.in_w = p.in_h = p.out_w = p.out_h = 2
    p.channels = p.batch = p.k_w = p.k_h = p.stride_w = p.stride_h = 1
    p.dtype = tvx.U8
    p.in_scale = p.out_scale = 1.0
    p.in_zp = 256
    with pytest.raises(tvx.TvxError) as e:
        tvx.pool2d_create(p)
    assert e.value.status == tvx.E_INVALID


def test_compute_fails_loudly_without_a_gpu(tvx):
    if tvx.lib().tvx_device_count() > 0:
        pytest.skip("a GPU is present")
    p = tvx.Pool2dDesc()
    p.in_w = p.in_h = p.out_w = p.out_h = 2
    p.channels = p.batch = p.k_w = p.k_h = p.stride_w = p.stride_h = 1
    p.dtype = tvx.F32
    with pytest.raises(tvx.TvxError) as e:
        tvx.pool2d_create(p)
    assert e.value.status == tvx.E_DEVICE
    assert "no CPU path" in str(e.value)
