"""ctypes front-end of the x86 VNNI kernels in oracle/cpu_vnni_gemm.c and oracle/cpu_vnni_conv.c: the benchmark's CPU baseline.

Test / benchmark infrastructure only; the product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcpubaseline.so")
_lib = None


def build(force=False):
    newest = max(os.path.getmtime(os.path.join(_HERE, s)) for s in ("cpu_vnni_gemm.c", "cpu_vnni_conv.c", "ncnn_int8_oracle.c"))
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < newest:
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcpubaseline.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.cpu_vnni_available.restype = C.c_int
        _lib.cpu_vnni_set_num_threads.restype = None
        _lib.cpu_vnni_set_num_threads.argtypes = [C.c_int]
        _lib.cpu_vnni_packed_bytes.restype = C.c_size_t
        _lib.cpu_vnni_packed_bytes.argtypes = [C.c_int, C.c_int]
        _lib.cpu_vnni_pack_b.restype = None
        _lib.cpu_vnni_pack_b.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
        _lib.cpu_vnni_gemm.restype = C.c_int
        _lib.cpu_vnni_gemm.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_size_t, C.c_void_p]
        vp, ci, cf = C.c_void_p, C.c_int, C.c_float
        _lib.cpu_vnni_conv_nhwc.restype = ci
        _lib.cpu_vnni_conv_nhwc.argtypes = [C.POINTER(ConvDesc), vp, ci, cf, vp, vp, vp, vp, ci, vp, vp]
        _lib.cpu_dwconv_nhwc.restype = ci
        _lib.cpu_dwconv_nhwc.argtypes = [C.POINTER(ConvDesc), vp, ci, vp, vp, vp, vp, vp, ci, vp, vp]
        _lib.cpu_add_f32.restype = None
        _lib.cpu_add_f32.argtypes = [vp, vp, vp, C.c_size_t]
        _lib.cpu_relu.restype = None
        _lib.cpu_relu.argtypes = [vp, ci, C.c_size_t]
        _lib.cpu_maxpool_nhwc.restype = None
        _lib.cpu_maxpool_nhwc.argtypes = [vp, ci, ci, ci, ci, ci, ci, ci, vp, ci, ci]
        _lib.cpu_global_avgpool_nhwc.restype = None
        _lib.cpu_global_avgpool_nhwc.argtypes = [vp, ci, ci, ci, vp]
    return _lib


class ConvDesc(C.Structure):
    """cpu_conv_desc of cpu_vnni_conv.c; the pads are explicit borders (resolve -233 / -234 before)."""
    _fields_ = [(n, C.c_int) for n in ("w", "h", "c", "n", "num_output", "kernel_w", "kernel_h", "dilation_w", "dilation_h", "stride_w", "stride_h",
                                       "pad_left", "pad_right", "pad_top", "pad_bottom")] + [("pad_value", C.c_float)]


def available():
    return bool(lib().cpu_vnni_available())


def set_num_threads(n):
    lib().cpu_vnni_set_num_threads(int(n))


def pack_b(bq):
    bq = np.ascontiguousarray(bq, np.int8)
    n, k = bq.shape
    packed = np.empty(lib().cpu_vnni_packed_bytes(n, k), np.uint8)
    lib().cpu_vnni_pack_b(bq.ctypes.data, k, n, k, packed.ctypes.data)
    return packed


def gemm(a, packed, n, b_scales, bias=None, want_acc=False):
    """a fp32 [M][K] quantised per row inside; returns fp32 [M][N] (and the int32 sums)."""
    a = np.ascontiguousarray(a, np.float32)
    m, k = a.shape
    b_scales = np.ascontiguousarray(np.atleast_1d(b_scales), np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
    out = np.empty((m, n), np.float32)
    acc = np.empty((m, n), np.int32) if want_acc else None
    rc = lib().cpu_vnni_gemm(a.ctypes.data, k, m, n, k, packed.ctypes.data, b_scales.ctypes.data, b_scales.size,
                             None if bias is None else bias.ctypes.data, out.ctypes.data, n, None if acc is None else acc.ctypes.data)
    if rc != 0:
        raise MemoryError("cpu_vnni_gemm")
    return (out, acc) if want_acc else out


def _ptr(a):
    return None if a is None else a.ctypes.data


def _out_hw(d):
    H, W = d.h + d.pad_top + d.pad_bottom, d.w + d.pad_left + d.pad_right
    return (H - (d.dilation_h * (d.kernel_h - 1) + 1)) // d.stride_h + 1, (W - (d.dilation_w * (d.kernel_w - 1) + 1)) // d.stride_w + 1


def fold_scales(w_scales, in_scales):
    """scale_in of the reference's epilogue: 0 where the weight scale is 0, else 1 / (input scale * weight scale), in binary32."""
    w = np.asarray(w_scales, np.float32)
    prod = (np.asarray(in_scales, np.float32) * w).astype(np.float32)
    with np.errstate(divide="ignore"):
        return np.where(w == 0, np.float32(0), np.float32(1) / prod).astype(np.float32)


def pack_conv_weights(wq):
    """int8 [num_output][c][kh][kw] -> packed for conv_nhwc (K runs ky, kx, c)."""
    wq = np.ascontiguousarray(wq, np.int8)
    return pack_b(np.ascontiguousarray(wq.transpose(0, 2, 3, 1)).reshape(wq.shape[0], -1))


def _like(out, shape, dtype):
    """`out` when it has this shape and type (a blob kept from an earlier pass, as a pool allocator hands out), else a new array."""
    if out is not None and out.shape == tuple(shape) and out.dtype == dtype and out.flags.c_contiguous:
        return out
    return np.empty(shape, dtype)


def conv_nhwc(d, x, in_scale, packed, scale_in, bias, scale_out, act_type=0, act_params=(0.0, 0.0), out=None):
    """x [n][h][w][c] fp32 or int8 -> [n][outh][outw][num_output] fp32, or int8 when scale_out is given."""
    x = np.ascontiguousarray(x)
    oh, ow = _out_hw(d)
    out = _like(out, (d.n, oh, ow, d.num_output), np.float32 if scale_out is None else np.int8)
    so = None if scale_out is None else np.ascontiguousarray(np.atleast_1d(scale_out), np.float32)
    ap = np.asarray(list(act_params)[:2], np.float32)
    rc = lib().cpu_vnni_conv_nhwc(C.byref(d), x.ctypes.data, x.dtype.itemsize, float(in_scale), packed.ctypes.data, scale_in.ctypes.data, _ptr(bias),
                                  _ptr(so), act_type, ap.ctypes.data, out.ctypes.data)
    if rc != 0:
        raise MemoryError("cpu_vnni_conv_nhwc")
    return out


def dwconv_nhwc(d, x, in_scales, weight_taps, scale_in, bias, scale_out, act_type=0, act_params=(0.0, 0.0), out=None):
    """Depthwise: weight_taps int8 [kh*kw][c]; in_scales / scale_in / scale_out one value per channel."""
    x = np.ascontiguousarray(x)
    oh, ow = _out_hw(d)
    out = _like(out, (d.n, oh, ow, d.c), np.float32 if scale_out is None else np.int8)
    ins = np.ascontiguousarray(in_scales, np.float32)
    so = None if scale_out is None else np.ascontiguousarray(scale_out, np.float32)
    ap = np.asarray(list(act_params)[:2], np.float32)
    rc = lib().cpu_dwconv_nhwc(C.byref(d), x.ctypes.data, x.dtype.itemsize, ins.ctypes.data, weight_taps.ctypes.data, scale_in.ctypes.data, _ptr(bias),
                               _ptr(so), act_type, ap.ctypes.data, out.ctypes.data)
    if rc != 0:
        raise MemoryError("cpu_dwconv_nhwc")
    return out


def add_f32(a, b, out=None):
    out = _like(out, a.shape, a.dtype)
    lib().cpu_add_f32(a.ctypes.data, b.ctypes.data, out.ctypes.data, a.size)
    return out


def relu_inplace(x):
    lib().cpu_relu(x.ctypes.data, x.dtype.itemsize, x.size)
    return x


def maxpool_nhwc(x, kernel, stride, out=None):
    n, h, w, c = x.shape
    ph, pw = (stride - (h - kernel) % stride) % stride, (stride - (w - kernel) % stride) % stride
    oh, ow = (h + ph - kernel) // stride + 1, (w + pw - kernel) // stride + 1
    out = _like(out, (n, oh, ow, c), x.dtype)
    lib().cpu_maxpool_nhwc(x.ctypes.data, x.dtype.itemsize, n, h, w, c, kernel, stride, out.ctypes.data, oh, ow)
    return out


def global_avgpool_nhwc(x):
    n, h, w, c = x.shape
    out = np.empty((n, 1, 1, c), np.float32)
    lib().cpu_global_avgpool_nhwc(x.ctypes.data, n, h * w, c, out.ctypes.data)
    return out
