"""Python plumbing around libtvx_hip.so (the C ABI of include/tvx_hip.h).

The product is the shared library and the C++ tim::vx runtime built on it;
this module only (a) builds them with hipcc / g++ and (b) exposes the C ABI
through ctypes so tests and the benchmark can drive it with device memory
held in torch tensors. There is no CPU path: every compute call needs a GPU.
"""
import ctypes as C
import os

from . import build as _build

PKG_DIR = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG_DIR, "lib", "libtvx_hip.so")

OK, E_INVALID, E_UNSUPPORTED, E_DEVICE, E_NOMEM = 0, -1, -2, -3, -4
U8, I8, F16, F32 = 0, 1, 2, 3
ACT_NONE, ACT_RELU, ACT_RELU6 = 0, 1, 2
POOL_MAX, POOL_AVG, POOL_L2, POOL_AVG_ANDROID = 0, 1, 2, 3


class Conv2dDesc(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "in_w", "in_h", "in_c", "batch", "k_w", "k_h", "out_w", "out_h", "out_c",
        "stride_w", "stride_h", "dilation_w", "dilation_h", "pad_left", "pad_top")] + [
        ("multiplier", C.c_int32), ("in_dtype", C.c_int32), ("w_dtype", C.c_int32),
        ("out_dtype", C.c_int32), ("in_scale", C.c_float), ("in_zp", C.c_int32),
        ("w_scale", C.c_float), ("w_zp", C.c_int32), ("w_scales", C.POINTER(C.c_float)),
        ("out_scale", C.c_float), ("out_zp", C.c_int32), ("activation", C.c_int32), ("groups", C.c_int32)]


class FcDesc(C.Structure):
    _fields_ = [("m", C.c_uint32), ("k", C.c_uint32), ("n", C.c_uint32),
                ("in_dtype", C.c_int32), ("w_dtype", C.c_int32), ("out_dtype", C.c_int32),
                ("in_scale", C.c_float), ("in_zp", C.c_int32), ("w_scale", C.c_float),
                ("w_zp", C.c_int32), ("w_scales", C.POINTER(C.c_float)),
                ("out_scale", C.c_float), ("out_zp", C.c_int32), ("activation", C.c_int32)]


class Pool2dDesc(C.Structure):
    _fields_ = [(n, C.c_uint32) for n in (
        "in_w", "in_h", "channels", "batch", "out_w", "out_h", "k_w", "k_h",
        "stride_w", "stride_h", "pad_left", "pad_top")] + [
        ("pool_type", C.c_int32), ("dtype", C.c_int32), ("in_scale", C.c_float),
        ("in_zp", C.c_int32), ("out_scale", C.c_float), ("out_zp", C.c_int32)]


class EltwiseDesc(C.Structure):
    _fields_ = [("count", C.c_uint64), ("dtype", C.c_int32), ("activation", C.c_int32),
                ("a_scale", C.c_float), ("a_zp", C.c_int32), ("b_scale", C.c_float),
                ("b_zp", C.c_int32), ("out_scale", C.c_float), ("out_zp", C.c_int32)]


class SoftmaxDesc(C.Structure):
    _fields_ = [("channels", C.c_uint32), ("rows", C.c_uint64), ("beta", C.c_float),
                ("in_dtype", C.c_int32), ("in_scale", C.c_float), ("in_zp", C.c_int32), ("inner", C.c_uint64)]


class ConvertDesc(C.Structure):
    _fields_ = [("count", C.c_uint64), ("in_dtype", C.c_int32), ("in_scale", C.c_float), ("in_zp", C.c_int32),
                ("out_dtype", C.c_int32), ("out_scale", C.c_float), ("out_zp", C.c_int32)]


class TransposeDesc(C.Structure):
    _fields_ = [("rank", C.c_uint32), ("in_dims", C.c_uint32 * 6), ("perm", C.c_uint32 * 6),
                ("elem_bytes", C.c_uint32)]


class TvxError(RuntimeError):
    def __init__(self, status, message):
        super().__init__("tvx status %d: %s" % (status, message))
        self.status = status


_lib = None


def build(verbose=False):
    """Compile the HIP library and the C++ runtime in-tree (see build.py)."""
    _build.build_all(verbose=verbose)


def lib():
    """The loaded C ABI. Raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: run __graft_entry__.build() first" % LIB_PATH)
        # torch ships its own libamdhip64.so.7; two HIP runtimes in one process do
        # not both see the GPU. Loading torch's first makes the dynamic loader
        # resolve this library's libamdhip64.so.7 dependency to that same copy.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        L = C.CDLL(LIB_PATH)
        vp = C.c_void_p
        L.tvx_version.restype = C.c_char_p
        L.tvx_last_error.restype = C.c_char_p
        L.tvx_status_string.restype = C.c_char_p
        L.tvx_status_string.argtypes = [C.c_int]
        L.tvx_op_kernel_name.restype = C.c_char_p
        L.tvx_op_kernel_name.argtypes = [vp]
        L.tvx_malloc.argtypes = [C.POINTER(vp), C.c_size_t]
        L.tvx_free.argtypes = [vp]
        for f in (L.tvx_memcpy_h2d, L.tvx_memcpy_d2h, L.tvx_memcpy_d2d):
            f.argtypes = [vp, vp, C.c_size_t, vp]
        L.tvx_stream_create.argtypes = [C.POINTER(vp)]
        L.tvx_stream_destroy.argtypes = [vp]
        L.tvx_stream_synchronize.argtypes = [vp]
        L.tvx_quantize_multiplier.argtypes = [C.c_double, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]
        L.tvx_requantize.restype = C.c_int64
        L.tvx_requantize.argtypes = [C.c_int32, C.c_int32, C.c_int32]
        L.tvx_conv2d_create.argtypes = [C.POINTER(Conv2dDesc), vp, vp, C.POINTER(vp)]
        L.tvx_conv2d_add_create.argtypes = [C.POINTER(Conv2dDesc), C.POINTER(EltwiseDesc), C.c_int, vp, vp, C.POINTER(vp)]
        L.tvx_deconv2d_create.argtypes = [C.POINTER(Conv2dDesc), vp, vp, C.POINTER(vp)]
        L.tvx_conv2d_dw_pw_create.argtypes = [C.POINTER(Conv2dDesc), vp, vp, C.POINTER(Conv2dDesc), vp, vp,
                                              C.POINTER(EltwiseDesc), C.c_int, C.POINTER(vp)]
        L.tvx_mbconv_create.argtypes = [C.POINTER(Conv2dDesc), vp, vp, C.POINTER(Conv2dDesc), vp, vp, C.POINTER(Conv2dDesc), vp, vp,
                                        C.POINTER(EltwiseDesc), C.c_int, C.POINTER(vp)]
        L.tvx_conv2d_pool_create.argtypes = [C.POINTER(Conv2dDesc), C.POINTER(Pool2dDesc), vp, vp, C.POINTER(vp)]
        L.tvx_conv2d_blocked_create.argtypes = [C.POINTER(Conv2dDesc), C.POINTER(EltwiseDesc), C.c_int, vp, vp, C.POINTER(vp)]
        L.tvx_conv2d_to_blocked_create.argtypes = [C.POINTER(Conv2dDesc), vp, vp, C.POINTER(vp)]
        L.tvx_pool2d_blocked_create.argtypes = [C.POINTER(Pool2dDesc), C.POINTER(vp)]
        L.tvx_layout_create.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32, C.c_uint32, C.c_int, C.POINTER(vp)]
        L.tvx_fully_connected_softmax_create.argtypes = [C.POINTER(FcDesc), C.POINTER(SoftmaxDesc), vp, vp, C.POINTER(vp)]
        L.tvx_fully_connected_create.argtypes = [C.POINTER(FcDesc), vp, vp, C.POINTER(vp)]
        L.tvx_pool2d_create.argtypes = [C.POINTER(Pool2dDesc), C.POINTER(vp)]
        L.tvx_activation_create.argtypes = [C.POINTER(EltwiseDesc), C.POINTER(vp)]
        L.tvx_add_create.argtypes = [C.POINTER(EltwiseDesc), C.POINTER(vp)]
        L.tvx_op_run3.argtypes = [vp, vp, vp, vp, vp, vp]
        L.tvx_softmax_create.argtypes = [C.POINTER(SoftmaxDesc), C.POINTER(vp)]
        L.tvx_convert_create.argtypes = [C.POINTER(ConvertDesc), C.POINTER(vp)]
        L.tvx_transpose_create.argtypes = [C.POINTER(TransposeDesc), C.POINTER(vp)]
        L.tvx_op_run.argtypes = [vp, vp, vp, vp, vp]
        L.tvx_op_destroy.argtypes = [vp]
        L.tvx_op_destroy.restype = None
        _lib = L
    return _lib


def check(status):
    if status != OK:
        raise TvxError(status, lib().tvx_last_error().decode())


class Op:
    """Owns one tvx_op handle."""

    def __init__(self, handle):
        self.handle = handle

    @property
    def kernel_name(self):
        return lib().tvx_op_kernel_name(self.handle).decode()

    def run(self, in0, in1, out, stream=None):
        """in0 / in1 / out are device pointers (ints) or torch CUDA tensors."""
        def ptr(t):
            if t is None:
                return None
            return t if isinstance(t, int) else t.data_ptr()
        check(lib().tvx_op_run(self.handle, ptr(in0), ptr(in1), ptr(out), stream))

    def close(self):
        if self.handle:
            lib().tvx_op_destroy(self.handle)
            self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def _host_ptr(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def conv2d_create(desc, weights=None, bias=None):
    """weights / bias: C-contiguous numpy arrays (host) or None."""
    h = C.c_void_p()
    check(lib().tvx_conv2d_create(C.byref(desc), _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def conv2d_add_create(desc, add_desc, conv_operand, weights, bias=None):
    h = C.c_void_p()
    check(lib().tvx_conv2d_add_create(C.byref(desc), C.byref(add_desc), conv_operand, _host_ptr(weights),
                                      _host_ptr(bias), C.byref(h)))
    return Op(h)


def conv2d_dw_pw_create(dw_desc, dw_weights, dw_bias, pw_desc, pw_weights, pw_bias, add_desc=None, conv_operand=0):
    h = C.c_void_p()
    check(lib().tvx_conv2d_dw_pw_create(C.byref(dw_desc), _host_ptr(dw_weights), _host_ptr(dw_bias),
                                        C.byref(pw_desc), _host_ptr(pw_weights), _host_ptr(pw_bias),
                                        C.byref(add_desc) if add_desc is not None else None, conv_operand, C.byref(h)))
    return Op(h)


def mbconv_create(expand, expand_w, expand_b, dw, dw_w, dw_b, project, project_w, project_b, add_desc=None, conv_operand=0):
    """1x1 expansion, depthwise 3x3 and 1x1 projection (+ residual Add) as one operator."""
    h = C.c_void_p()
    check(lib().tvx_mbconv_create(C.byref(expand), _host_ptr(expand_w), _host_ptr(expand_b),
                                  C.byref(dw), _host_ptr(dw_w), _host_ptr(dw_b),
                                  C.byref(project), _host_ptr(project_w), _host_ptr(project_b),
                                  C.byref(add_desc) if add_desc is not None else None, conv_operand, C.byref(h)))
    return Op(h)


def conv2d_to_blocked_create(desc, weights, bias=None):
    """A depthwise 3x3 convolution that reads a WHCN tensor and writes its result channel-blocked."""
    h = C.c_void_p()
    check(lib().tvx_conv2d_to_blocked_create(C.byref(desc), _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def conv2d_blocked_create(desc, weights, bias=None, add_desc=None, conv_operand=0):
    """A 1x1 (optionally + Add) or depthwise 3x3 convolution between channel-blocked tensors."""
    h = C.c_void_p()
    check(lib().tvx_conv2d_blocked_create(C.byref(desc), C.byref(add_desc) if add_desc is not None else None, conv_operand,
                                          _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def pool2d_blocked_create(desc):
    """Whole-plane average pooling of a channel-blocked tensor."""
    h = C.c_void_p()
    check(lib().tvx_pool2d_blocked_create(C.byref(desc), C.byref(h)))
    return Op(h)


def layout_create(w, h, c, n, to_blocked):
    """WHCN planes -> channel-blocked order (to_blocked) or back."""
    hd = C.c_void_p()
    check(lib().tvx_layout_create(w, h, c, n, 1 if to_blocked else 0, C.byref(hd)))
    return Op(hd)


def conv2d_pool_create(desc, pool_desc, weights, bias=None):
    """A convolution and the 2x2 / stride-2 max pooling behind it as one operator."""
    h = C.c_void_p()
    check(lib().tvx_conv2d_pool_create(C.byref(desc), C.byref(pool_desc), _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def fully_connected_softmax_create(desc, softmax_desc, weights, bias=None):
    """A FullyConnected layer of at most 16 outputs and the Softmax over them as one operator (fp32 result)."""
    h = C.c_void_p()
    check(lib().tvx_fully_connected_softmax_create(C.byref(desc), C.byref(softmax_desc), _host_ptr(weights),
                                                   _host_ptr(bias), C.byref(h)))
    return Op(h)


def deconv2d_create(desc, weights=None, bias=None):
    h = C.c_void_p()
    check(lib().tvx_deconv2d_create(C.byref(desc), _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def fully_connected_create(desc, weights=None, bias=None):
    h = C.c_void_p()
    check(lib().tvx_fully_connected_create(C.byref(desc), _host_ptr(weights), _host_ptr(bias), C.byref(h)))
    return Op(h)


def pool2d_create(desc):
    h = C.c_void_p()
    check(lib().tvx_pool2d_create(C.byref(desc), C.byref(h)))
    return Op(h)


def activation_create(desc):
    h = C.c_void_p()
    check(lib().tvx_activation_create(C.byref(desc), C.byref(h)))
    return Op(h)


def add_create(desc):
    h = C.c_void_p()
    check(lib().tvx_add_create(C.byref(desc), C.byref(h)))
    return Op(h)


def softmax_create(desc):
    h = C.c_void_p()
    check(lib().tvx_softmax_create(C.byref(desc), C.byref(h)))
    return Op(h)


def convert_create(desc):
    h = C.c_void_p()
    check(lib().tvx_convert_create(C.byref(desc), C.byref(h)))
    return Op(h)


def transpose_create(desc):
    h = C.c_void_p()
    check(lib().tvx_transpose_create(C.byref(desc), C.byref(h)))
    return Op(h)


_calib = None


def _calibration_lib():
    """libtvx_calibrate.so: the benchmark's device-calibration kernels (not part of the C ABI)."""
    global _calib
    if _calib is None:
        L = C.CDLL(os.path.join(PKG_DIR, "lib", "libtvx_calibrate.so"))
        L.tvx_calibrate_mfma_i8.argtypes = [C.c_int, C.c_int, C.POINTER(C.c_double)]
        L.tvx_calibrate_copy.argtypes = [C.c_size_t, C.c_int, C.POINTER(C.c_double)]
        _calib = L
    return _calib


def calibrate_mfma_i8(random_operands, launches=5):
    """Sustained int8 matrix-core rate of this GPU in TOPS (zeros: nominal clock; random
    operands: the clock held under the multipliers' switching power)."""
    v = C.c_double()
    if _calibration_lib().tvx_calibrate_mfma_i8(int(bool(random_operands)), launches, C.byref(v)) != 0:
        raise RuntimeError("tvx_calibrate_mfma_i8 failed")
    return v.value


def calibrate_copy(nbytes=256 << 20, launches=10):
    """Read + write GB/s of a plain streaming device copy of `nbytes`."""
    v = C.c_double()
    if _calibration_lib().tvx_calibrate_copy(nbytes, launches, C.byref(v)) != 0:
        raise RuntimeError("tvx_calibrate_copy failed")
    return v.value
