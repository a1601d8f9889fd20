"""ctypes signatures for include/ncnnhip.h plus a thin numpy <-> device-buffer convenience layer."""
import ctypes as C
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
_LIB = os.path.join(_PKG, "lib", "libncnnhip.so")

c_void_pp = C.POINTER(C.c_void_p)


class NcnnHipError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("ncnnhip error %d: %s" % (code, text))
        self.code = code


class Activation(C.Structure):
    _fields_ = [("type", C.c_int), ("p0", C.c_float), ("p1", C.c_float)]

    @classmethod
    def make(cls, act_type=0, params=(0.0, 0.0)):
        p = list(params) + [0.0, 0.0]
        return cls(int(act_type), float(p[0]), float(p[1]))


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("w", "h", "c", "batch", "num_output", "kernel_w", "kernel_h", "dilation_w", "dilation_h",
                                       "stride_w", "stride_h", "pad_left", "pad_right", "pad_top", "pad_bottom")] + \
               [("pad_value", C.c_float), ("group", C.c_int)]


class ConvFusion(C.Structure):
    _fields_ = [("residual_dev", C.c_void_p), ("relu_after", C.c_int), ("quantised_out_dev", C.c_void_p), ("quantise_scale", C.c_float)]


class PoolDesc(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("w", "h", "c", "batch", "pooling_type", "kernel_w", "kernel_h", "stride_w", "stride_h", "pad_top", "pad_left",
                                       "outw", "outh", "global_pooling", "avgpool_count_include_pad", "count_x0", "count_x1", "count_y0", "count_y1")]


def library_path():
    return _LIB


_SIGNATURES = {
    "ncnnhip_init": [C.c_int],
    "ncnnhip_device_info": [C.c_char_p, C.c_size_t, C.POINTER(C.c_int), C.POINTER(C.c_size_t)],
    "ncnnhip_stream_create": [c_void_pp],
    "ncnnhip_stream_destroy": [C.c_void_p],
    "ncnnhip_stream_synchronize": [C.c_void_p],
    "ncnnhip_device_synchronize": [],
    "ncnnhip_copy2d": [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p],
    "ncnnhip_attention_workspace_bytes": [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t)],
    "ncnnhip_attention_f32": [C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t,
                              C.c_void_p],
    "ncnnhip_attention_f32_strided": [C.c_void_p, C.c_size_t, C.c_float, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                      C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_attention_f32_append": [C.c_void_p, C.c_size_t, C.c_float, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p,
                                     C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_stream_begin_capture": [C.c_void_p],
    "ncnnhip_stream_end_capture": [C.c_void_p, C.POINTER(C.c_void_p)],
    "ncnnhip_graph_launch": [C.c_void_p, C.c_void_p],
    "ncnnhip_graph_destroy": [C.c_void_p],
    "ncnnhip_set_device_allocator": [C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_default_device_malloc": [c_void_pp, C.c_size_t],
    "ncnnhip_default_device_free": [C.c_void_p],
    "ncnnhip_malloc": [c_void_pp, C.c_size_t],
    "ncnnhip_free": [C.c_void_p],
    "ncnnhip_memcpy_h2d": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_memcpy_d2h": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_memcpy_d2d": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_memset": [C.c_void_p, C.c_int, C.c_size_t, C.c_void_p],
    "ncnnhip_event_create": [c_void_pp],
    "ncnnhip_event_destroy": [C.c_void_p],
    "ncnnhip_event_record": [C.c_void_p, C.c_void_p],
    "ncnnhip_event_synchronize": [C.c_void_p],
    "ncnnhip_event_elapsed_ms": [C.c_void_p, C.c_void_p, C.POINTER(C.c_float)],
    "ncnnhip_quantize": [C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_int,
                         C.c_void_p, C.c_int, C.c_void_p],
    "ncnnhip_conv_out_shape": [C.POINTER(ConvDesc), C.POINTER(C.c_int), C.POINTER(C.c_int)],
    "ncnnhip_fold_input_scales": [C.c_void_p, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p],
    "ncnnhip_conv_int8": [C.POINTER(ConvDesc), C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                          Activation, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_conv_nhwc_sizes": [C.POINTER(ConvDesc), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "ncnnhip_conv_pack_weights": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p],
    "ncnnhip_to_nhwc_int8": [C.POINTER(ConvDesc), C.c_void_p, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_conv_int8_nhwc": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p, C.c_int,
                               C.c_size_t, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_conv_fusion_supported": [C.POINTER(ConvDesc)],
    "ncnnhip_conv_from_float_supported": [C.POINTER(ConvDesc)],
    "ncnnhip_conv_small_tile_selected": [C.POINTER(ConvDesc), C.c_int],
    "ncnnhip_conv_from_float_workspace_bytes": [C.POINTER(ConvDesc), C.POINTER(C.c_size_t)],
    "ncnnhip_conv_int8_nhwc_from_float": [C.POINTER(ConvDesc), C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p,
                                          C.POINTER(ConvFusion), C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_conv_int8_nhwc_fused": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p, C.POINTER(ConvFusion), C.c_void_p,
                                     C.c_size_t, C.c_void_p],
    "ncnnhip_conv_resolved_pads": [C.POINTER(ConvDesc), C.POINTER(C.c_int), C.POINTER(C.c_int)],
    "ncnnhip_padded_channels": [C.c_int],
    "ncnnhip_chw_to_nhwc": [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_nhwc_to_chw": [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_size_t, C.c_void_p],
    "ncnnhip_quantize_nhwc": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_int, C.c_void_p],
    "ncnnhip_int8_to_f32": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_dwconv_packed_bytes": [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t)],
    "ncnnhip_dwconv_pack_weights": [C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_dwconv_int8_nhwc": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p, C.c_void_p],
    "ncnnhip_relu": [C.c_void_p, C.c_void_p, C.c_int, C.c_size_t, C.c_float, C.c_void_p],
    "ncnnhip_scale": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_float, C.c_void_p],
    "ncnnhip_eltwise": [C.POINTER(C.c_void_p), C.c_int, C.c_int, C.POINTER(C.c_float), C.c_int, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_chw_to_nhwc4_f32": [C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_widen_nhwc4_f32": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_conv_stem_supported": [C.POINTER(ConvDesc)],
    "ncnnhip_conv_stem_sizes": [C.POINTER(ConvDesc), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "ncnnhip_conv_stem_pack_weights": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p],
    "ncnnhip_quantize_stem": [C.POINTER(ConvDesc), C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_conv_int8_stem": [C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p, C.POINTER(ConvFusion),
                               C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_pooling_nhwc": [C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_maxpool_nhwc_int8": [C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_global_pooling_nhwc_quantised": [C.POINTER(PoolDesc), C.c_void_p, C.c_float, C.c_void_p, C.c_void_p],
    "ncnnhip_softmax": [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p],
    "ncnnhip_innerproduct_int8": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, Activation,
                                  C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_innerproduct_workspace_bytes": [C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t)],
    "ncnnhip_innerproduct_int8_ws": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p, C.c_size_t,
                                     C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_innerproduct_int8_noalloc": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, Activation, C.c_void_p,
                                          C.c_size_t, C.c_void_p],
    "ncnnhip_gemm_quantize_rows": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_quantize_tensor": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_transpose_f32": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_transpose_pair_f32": [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_transpose_s8": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_gemm_int8": [C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int,
                          C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_int, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_int8_tile_operand": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_quantize_rows_tiled": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_int8_tiled": [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_int,
                                C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_gemm_blockquant": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                C.c_void_p, C.c_void_p, C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_blockquant_packed_size": [C.c_int, C.c_int, C.c_int, C.c_int, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "ncnnhip_blockquant_pack": [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_blockquant_packed_f16a": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                            C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_gemm_blockquant_packed_supported": [C.c_int],
    "ncnnhip_gemm_blockquant_packed": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_gemm_blockquant_packed_multi": [C.c_void_p, C.c_int, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int, C.c_int,
                                             C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_blockquant_packed_rows_workspace_bytes": [C.c_int, C.c_int, C.POINTER(C.c_size_t)],
    "ncnnhip_gemm_blockquant_packed_rows": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p,
                                            C.c_int, C.c_float, C.c_float, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p],
    "ncnnhip_peak_launch_chain": [C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_peak_mfma_i8": [C.c_int, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_peak_hbm_read": [C.c_void_p, C.c_size_t, C.c_int, C.c_void_p, C.c_void_p],
    "ncnnhip_gemm_blockquant_f16a": [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p,
                                     C.c_void_p, C.c_size_t, C.c_void_p],
}

EXPORTED_SYMBOLS = sorted(list(_SIGNATURES) + ["ncnnhip_last_error"])

_lib = None


def lib():
    """Loads libncnnhip.so.  Raises if it has not been built -- there is no fallback path."""
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise NcnnHipError(-1, "%s is missing: run `python -c 'import __graft_entry__ as g; g.build()'` "
                                   "(or python ncnn_amd/build.py) first" % _LIB)
        _lib = C.CDLL(_LIB)
        for name, argtypes in _SIGNATURES.items():
            fn = getattr(_lib, name)
            fn.argtypes = argtypes
            fn.restype = C.c_int
        _lib.ncnnhip_last_error.restype = C.c_char_p
        _lib.ncnnhip_last_error.argtypes = []
    return _lib


def check(code):
    if code != 0:
        raise NcnnHipError(code, lib().ncnnhip_last_error().decode("utf-8", "replace"))


class DeviceBuffer:
    """A hipMalloc'd buffer with the numpy shape/dtype it mirrors."""

    def __init__(self, nbytes, shape=None, dtype=np.uint8):
        self.ptr = C.c_void_p()
        self.nbytes = int(nbytes)
        self.shape = shape
        self.dtype = np.dtype(dtype)
        check(lib().ncnnhip_malloc(C.byref(self.ptr), self.nbytes))

    @classmethod
    def from_numpy(cls, arr, stream=None):
        arr = np.ascontiguousarray(arr)
        buf = cls(arr.nbytes, arr.shape, arr.dtype)
        check(lib().ncnnhip_memcpy_h2d(buf.ptr, arr.ctypes.data_as(C.c_void_p), arr.nbytes, stream))
        check(lib().ncnnhip_stream_synchronize(stream))
        return buf

    @classmethod
    def zeros(cls, nbytes, stream=None):
        """A zero-filled byte buffer (the convolution workspace must be cleared once after allocation)."""
        buf = cls(max(int(nbytes), 4))
        check(lib().ncnnhip_memset(buf.ptr, 0, buf.nbytes, stream))
        check(lib().ncnnhip_stream_synchronize(stream))
        return buf

    @classmethod
    def empty(cls, shape, dtype):
        shape = tuple(int(s) for s in np.atleast_1d(shape))
        return cls(int(np.prod(shape)) * np.dtype(dtype).itemsize, shape, dtype)

    def to_numpy(self, stream=None):
        out = np.empty(self.shape, self.dtype)
        check(lib().ncnnhip_memcpy_d2h(out.ctypes.data_as(C.c_void_p), self.ptr, out.nbytes, stream))
        check(lib().ncnnhip_stream_synchronize(stream))
        return out

    def fill_bytes(self, byte, stream=None):
        check(lib().ncnnhip_memset(self.ptr, int(byte), self.nbytes, stream))

    def free(self):
        if self.ptr:
            lib().ncnnhip_free(self.ptr)
            self.ptr = C.c_void_p()

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def _ptr(buf):
    if buf is None:
        return None
    return buf.ptr if isinstance(buf, DeviceBuffer) else buf


class Runtime:
    """Numpy-in / numpy-out convenience calls; each uploads its operands, launches on one stream and
    downloads the result.  Used by the tests and the smoke check; the benchmark drives the C ABI directly."""

    def __init__(self, device=0):
        check(lib().ncnnhip_init(device))
        self.stream = C.c_void_p()
        check(lib().ncnnhip_stream_create(C.byref(self.stream)))

    def sync(self):
        check(lib().ncnnhip_stream_synchronize(self.stream))

    def device_info(self):
        name = C.create_string_buffer(128)
        cu, mem = C.c_int(), C.c_size_t()
        check(lib().ncnnhip_device_info(name, 128, C.byref(cu), C.byref(mem)))
        return name.value.decode(), cu.value, mem.value

    def up(self, arr):
        return None if arr is None else DeviceBuffer.from_numpy(arr, self.stream)

    # -- Quantize -------------------------------------------------------------------------
    def quantize(self, x, scales):
        x = np.ascontiguousarray(x, np.float32)
        scales = np.ascontiguousarray(np.atleast_1d(scales), np.float32)
        rows, cols = x.shape
        dx, ds = self.up(x), self.up(scales)
        dy = DeviceBuffer.empty((rows, cols), np.int8)
        check(lib().ncnnhip_quantize(dx.ptr, cols, 0, dy.ptr, cols, 0, rows, cols, 1, ds.ptr, scales.size, self.stream))
        return dy.to_numpy(self.stream)

    # -- Convolution / ConvolutionDepthWise -------------------------------------------------
    def fold_input_scales(self, w_scales, in_scales, num_output):
        w_scales = np.ascontiguousarray(np.atleast_1d(w_scales), np.float32)
        in_scales = np.ascontiguousarray(np.atleast_1d(in_scales), np.float32)
        out = np.empty(num_output, np.float32)
        check(lib().ncnnhip_fold_input_scales(w_scales.ctypes.data, w_scales.size, in_scales.ctypes.data, in_scales.size,
                                              num_output, out.ctypes.data))
        return out

    def conv_layer(self, x, weight, bias, w_scales, in_scales, top_scales, num_output, kernel, dilation=(1, 1), stride=(1, 1),
                   pads=(0, 0, 0, 0), pad_value=0.0, group=1, term=1, act=0, act_params=(0.0, 0.0), want_acc=False, path="auto"):
        """Whole forward_int8 of Convolution (group == 1, per-output-channel weight scales) or
        ConvolutionDepthWise (scale tables with `group` entries): x is [c][h][w] or [n][c][h][w], fp32 or int8."""
        x = np.ascontiguousarray(x)
        if x.ndim == 3:
            x = x[None]
        n, c, h, w = x.shape
        d = ConvDesc(w, h, c, n, num_output, kernel[0], kernel[1], dilation[0], dilation[1], stride[0], stride[1],
                     pads[0], pads[1], pads[2], pads[3], float(pad_value), group)
        ow, oh = C.c_int(), C.c_int()
        check(lib().ncnnhip_conv_out_shape(C.byref(d), C.byref(ow), C.byref(oh)))
        ow, oh = ow.value, oh.value
        w_scales = np.atleast_1d(np.asarray(w_scales, np.float32))
        in_scales = np.atleast_1d(np.asarray(in_scales, np.float32))
        scale_in = self.fold_input_scales(w_scales, in_scales, num_output)
        cstep, nstep = h * w, c * h * w
        requant = term > 100
        if path == "auto":
            path = "nhwc" if (group == 1 and not want_acc) else "chw"
        if path == "nhwc":
            # channels-last fast path: quantise+transpose, packed weights, same epilogue
            nb, wb, sb_ = C.c_size_t(), C.c_size_t(), C.c_size_t()
            check(lib().ncnnhip_conv_nhwc_sizes(C.byref(d), C.byref(nb), C.byref(wb), C.byref(sb_)))
            wq = np.ascontiguousarray(weight, np.int8)
            pk = np.empty(wb.value, np.int8)
            check(lib().ncnnhip_conv_pack_weights(C.byref(d), wq.ctypes.data, pk.ctypes.data))
            dx = self.up(x if x.dtype == np.int8 else x.astype(np.float32))
            dsc = self.up(in_scales)
            dn = DeviceBuffer(nb.value)
            check(lib().ncnnhip_to_nhwc_int8(C.byref(d), dx.ptr, x.dtype.itemsize, cstep, nstep, dsc.ptr, in_scales.size, dn.ptr, self.stream))
            scale_out = None
            if requant:
                ts = np.atleast_1d(np.asarray(top_scales, np.float32))
                scale_out = np.repeat(ts, num_output // ts.size).astype(np.float32)
            dpk, dsi, db, dso = self.up(pk), self.up(scale_in), self.up(None if bias is None else np.asarray(bias, np.float32)), self.up(scale_out)
            dws = DeviceBuffer.zeros(sb_.value, self.stream)
            dout = DeviceBuffer.empty((n, num_output, oh, ow), np.int8 if requant else np.float32)
            check(lib().ncnnhip_conv_int8_nhwc(C.byref(d), dn.ptr, dpk.ptr, dsi.ptr, _ptr(db), _ptr(dso), Activation.make(act, act_params), dout.ptr,
                                               0, oh * ow, num_output * oh * ow, dws.ptr, sb_.value, self.stream))
            return dout.to_numpy(self.stream)
        if x.dtype == np.int8:
            dxq = self.up(x)
        else:
            per_channel = np.repeat(in_scales, c // in_scales.size).astype(np.float32) if in_scales.size > 1 else in_scales
            dx, dsc = self.up(x.astype(np.float32)), self.up(per_channel)
            dxq = DeviceBuffer.empty(x.shape, np.int8)
            check(lib().ncnnhip_quantize(dx.ptr, cstep, nstep, dxq.ptr, cstep, nstep, c, cstep, n, dsc.ptr, per_channel.size, self.stream))
        scale_out = None
        if requant:
            ts = np.atleast_1d(np.asarray(top_scales, np.float32))
            scale_out = np.repeat(ts, num_output // ts.size).astype(np.float32)
        dw_, dsi, db, dso = self.up(np.asarray(weight, np.int8)), self.up(scale_in), self.up(None if bias is None else np.asarray(bias, np.float32)), self.up(scale_out)
        dout = DeviceBuffer.empty((n, num_output, oh, ow), np.int8 if requant else np.float32)
        dacc = DeviceBuffer.empty((n, num_output, oh, ow), np.int32) if want_acc else None
        check(lib().ncnnhip_conv_int8(C.byref(d), dxq.ptr, cstep, nstep, dw_.ptr, dsi.ptr, _ptr(db), _ptr(dso), Activation.make(act, act_params),
                                      dout.ptr, oh * ow, num_output * oh * ow, _ptr(dacc), self.stream))
        out = dout.to_numpy(self.stream)
        if want_acc:
            return out, dacc.to_numpy(self.stream)
        return out

    # -- device-resident (channels-last) blobs and the fp32 layers between the int8 layers -----
    def to_channels_last(self, x):
        """[n][c][h][w] (or [c][h][w]) fp32 / int8 numpy -> device [n][h*w][Cp] buffer."""
        x = np.ascontiguousarray(x)
        if x.ndim == 3:
            x = x[None]
        n, c, h, w = x.shape
        cp = lib().ncnnhip_padded_channels(c)
        dx = self.up(x)
        out = DeviceBuffer.empty((n, h * w, cp), x.dtype)
        check(lib().ncnnhip_chw_to_nhwc(dx.ptr, x.dtype.itemsize, c, h * w, n, h * w, c * h * w, out.ptr, self.stream))
        return out

    def from_channels_last(self, buf, n, c, h, w):
        out = DeviceBuffer.empty((n, c, h, w), buf.dtype)
        check(lib().ncnnhip_nhwc_to_chw(buf.ptr, buf.dtype.itemsize, c, h * w, n, out.ptr, h * w, c * h * w, self.stream))
        return out.to_numpy(self.stream)

    def quantize_channels_last(self, buf, c, scales):
        n, hw, cp = buf.shape
        ds = self.up(np.atleast_1d(np.asarray(scales, np.float32)))
        out = DeviceBuffer.empty((n, hw, cp), np.int8)
        check(lib().ncnnhip_quantize_nhwc(buf.ptr, out.ptr, n * hw, c, ds.ptr, ds.shape[0], self.stream))
        return out

    def relu(self, x, slope=0.0):
        x = np.ascontiguousarray(x)
        dx = self.up(x)
        out = DeviceBuffer.empty(x.shape, x.dtype)
        check(lib().ncnnhip_relu(dx.ptr, out.ptr, x.dtype.itemsize, x.size, float(slope), self.stream))
        return out.to_numpy(self.stream)

    def eltwise(self, xs, op_type=1, coeffs=None):
        xs = [np.ascontiguousarray(x, np.float32) for x in xs]
        bufs = [self.up(x) for x in xs]
        ptrs = (C.c_void_p * len(bufs))(*[b.ptr for b in bufs])
        co = None if coeffs is None else (C.c_float * len(coeffs))(*[float(v) for v in coeffs])
        out = DeviceBuffer.empty(xs[0].shape, np.float32)
        check(lib().ncnnhip_eltwise(ptrs, len(bufs), int(op_type), co, 0 if coeffs is None else len(coeffs), out.ptr, xs[0].size, self.stream))
        return out.to_numpy(self.stream)

    def pooling(self, x, pooling_type, kernel, stride, pad_top_left, out_hw, global_pooling=False, count_include_pad=0, count_rect=(0, 0, 0, 0)):
        """x [n][c][h][w] fp32; the border is given resolved (head pads and output extent); count_rect = (x0, x1, y0, y1) in image
        coordinates is the region whose taps make up an average's divisor without count_include_pad (all zero: the image)."""
        x = np.ascontiguousarray(x, np.float32)
        n, c, h, w = x.shape
        src = self.to_channels_last(x)
        if global_pooling:
            d = PoolDesc(w, h, c, n, pooling_type, 0, 0, 1, 1, 0, 0, 1, 1, 1, 0)
            out = DeviceBuffer.empty((n, c), np.float32)
            check(lib().ncnnhip_pooling_nhwc(C.byref(d), src.ptr, out.ptr, self.stream))
            return out.to_numpy(self.stream)
        oh, ow = out_hw
        d = PoolDesc(w, h, c, n, pooling_type, kernel[0], kernel[1], stride[0], stride[1], pad_top_left[0], pad_top_left[1], ow, oh, 0, int(count_include_pad),
                     *count_rect)
        out = DeviceBuffer.empty((n, oh * ow, src.shape[2]), np.float32)
        check(lib().ncnnhip_pooling_nhwc(C.byref(d), src.ptr, out.ptr, self.stream))
        return self.from_channels_last(out, n, c, oh, ow)

    def maxpool_int8(self, xq, kernel, stride, pad_top_left, out_hw):
        """xq [n][c][h][w] int8 (quantised values); windowed max pooling on the int8 blob."""
        xq = np.ascontiguousarray(xq, np.int8)
        n, c, h, w = xq.shape
        src = self.to_channels_last(xq)
        oh, ow = out_hw
        d = PoolDesc(w, h, c, n, 0, kernel[0], kernel[1], stride[0], stride[1], pad_top_left[0], pad_top_left[1], ow, oh, 0, 0)
        out = DeviceBuffer.empty((n, oh * ow, src.shape[2]), np.int8)
        check(lib().ncnnhip_maxpool_nhwc_int8(C.byref(d), src.ptr, out.ptr, self.stream))
        return self.from_channels_last(out, n, c, oh, ow)

    def global_pooling_quantised(self, x, pooling_type, scale):
        """x [n][c][h][w] fp32 -> [n][c] int8 = float2int8(global pool * scale)."""
        x = np.ascontiguousarray(x, np.float32)
        n, c, h, w = x.shape
        src = self.to_channels_last(x)
        d = PoolDesc(w, h, c, n, pooling_type, 0, 0, 1, 1, 0, 0, 1, 1, 1, 0)
        out = DeviceBuffer.empty((n, c), np.int8)
        check(lib().ncnnhip_global_pooling_nhwc_quantised(C.byref(d), src.ptr, float(scale), out.ptr, self.stream))
        return out.to_numpy(self.stream)

    def attention(self, q, kt, vt, num_heads, mask=None, use_workspace=True, q_scale=None):
        """q [src][embed] (scaled), kt / vt [embed][dst], mask [src][dst] or [heads][src][dst] -> [src][embed].

        With q_scale, q may be wider than embed (its first embed columns are the queries, the row stride is its width) and
        every query value is multiplied by q_scale on load."""
        q, kt, vt = [np.ascontiguousarray(a, np.float32) for a in (q, kt, vt)]
        src, q_stride = q.shape
        embed, dst = kt.shape
        dq, dk, dv = self.up(q), self.up(kt), self.up(vt)
        dm = None if mask is None else self.up(np.ascontiguousarray(mask, np.float32))
        mask_heads = 0 if mask is None else (1 if mask.ndim == 2 else mask.shape[0])
        out = DeviceBuffer.empty((src, embed), np.float32)
        wsb = C.c_size_t()
        check(lib().ncnnhip_attention_workspace_bytes(num_heads, embed // num_heads, src, dst, C.byref(wsb)))
        ws = DeviceBuffer.empty((max(wsb.value, 4),), np.uint8) if use_workspace else None
        if q_scale is None:
            assert q_stride == embed
            check(lib().ncnnhip_attention_f32(dq.ptr, dk.ptr, dv.ptr, dst, _ptr(dm), mask_heads, num_heads, embed // num_heads, src, dst, out.ptr,
                                              _ptr(ws), wsb.value if use_workspace else 0, self.stream))
        else:
            check(lib().ncnnhip_attention_f32_strided(dq.ptr, q_stride, float(q_scale), dk.ptr, dv.ptr, dst, _ptr(dm), mask_heads, num_heads, embed // num_heads,
                                                      src, dst, out.ptr, _ptr(ws), wsb.value if use_workspace else 0, self.stream))
        return out.to_numpy(self.stream)

    def attention_append(self, qkv, kt, vt, num_heads, past, q_scale, mask=None):
        """qkv [src][>= 3*embed]; kt / vt [embed][past + src] with the cache in their first `past` columns.  Returns (out, kt, vt) after the call."""
        qkv, kt, vt = [np.ascontiguousarray(a, np.float32) for a in (qkv, kt, vt)]
        src, stride = qkv.shape
        embed, dst = kt.shape
        assert dst == past + src
        dq, dk, dv = self.up(qkv), self.up(kt), self.up(vt)
        dm = None if mask is None else self.up(np.ascontiguousarray(mask, np.float32))
        mask_heads = 0 if mask is None else (1 if mask.ndim == 2 else mask.shape[0])
        out = DeviceBuffer.empty((src, embed), np.float32)
        wsb = C.c_size_t()
        check(lib().ncnnhip_attention_workspace_bytes(num_heads, embed // num_heads, src, dst, C.byref(wsb)))
        ws = DeviceBuffer.empty((max(wsb.value, 4),), np.uint8)
        check(lib().ncnnhip_attention_f32_append(dq.ptr, stride, float(q_scale), dk.ptr, dv.ptr, dst, past, _ptr(dm), mask_heads, num_heads, embed // num_heads, src,
                                                 out.ptr, ws.ptr, wsb.value, self.stream))
        return out.to_numpy(self.stream), dk.to_numpy(self.stream), dv.to_numpy(self.stream)

    def softmax(self, x):
        x = np.ascontiguousarray(x, np.float32)
        n, count = x.shape
        dx = self.up(x)
        out = DeviceBuffer.empty(x.shape, np.float32)
        check(lib().ncnnhip_softmax(dx.ptr, out.ptr, count, n, self.stream))
        return out.to_numpy(self.stream)

    def conv_channels_last(self, x, weight, bias, w_scales, in_scales, top_scales, num_output, kernel, dilation=(1, 1), stride=(1, 1),
                           pads=(0, 0, 0, 0), pad_value=0.0, group=1, term=1, act=0, act_params=(0.0, 0.0), residual=None, relu_after=False,
                           quantise_scale=None, stem=False, from_float=None):
        """Convolution (group 1) or depthwise (group == c == num_output) entirely on channels-last device blobs:
        upload+convert, quantise if fp32, kernel writing channels-last, convert back.  x is [n][c][h][w].
        stem=True: the narrow-input form (at most 4 input channels, 4-byte pixels with a physical border).
        from_float=np.float32 / np.float16: one launch, the fp32 / fp16 blob quantised inside the kernel."""
        x = np.ascontiguousarray(x)
        if x.ndim == 3:
            x = x[None]
        n, c, h, w = x.shape
        d = ConvDesc(w, h, c, n, num_output, kernel[0], kernel[1], dilation[0], dilation[1], stride[0], stride[1],
                     pads[0], pads[1], pads[2], pads[3], float(pad_value), group)
        ow, oh = C.c_int(), C.c_int()
        check(lib().ncnnhip_conv_out_shape(C.byref(d), C.byref(ow), C.byref(oh)))
        ow, oh = ow.value, oh.value
        w_scales = np.atleast_1d(np.asarray(w_scales, np.float32))
        in_scales = np.atleast_1d(np.asarray(in_scales, np.float32))
        scale_in = self.fold_input_scales(w_scales, in_scales, num_output)
        requant = term > 100
        if from_float is not None:
            if not lib().ncnnhip_conv_from_float_supported(C.byref(d)):
                raise ValueError("this layer keeps its separate Quantize pass")
            if np.dtype(from_float) == np.float32:
                src = self.to_channels_last(x.astype(np.float32))
            else:  # fp16: the layout change on the host (the device converter moves 1- and 4-byte values)
                cp = lib().ncnnhip_padded_channels(c)
                xh = np.zeros((n, h * w, cp), np.float16)
                xh[:, :, :c] = x.astype(np.float16).reshape(n, c, h * w).transpose(0, 2, 1)
                src = self.up(xh)
            dsi, db = self.up(scale_in), self.up(None if bias is None else np.asarray(bias, np.float32))
            dso = None
            if requant:
                ts = np.atleast_1d(np.asarray(top_scales, np.float32))
                dso = self.up(np.repeat(ts, num_output // ts.size).astype(np.float32))
            pk_bytes = C.c_size_t()
            check(lib().ncnnhip_conv_nhwc_sizes(C.byref(d), None, C.byref(pk_bytes), None))
            pk = np.empty(pk_bytes.value, np.int8)
            check(lib().ncnnhip_conv_pack_weights(C.byref(d), np.ascontiguousarray(weight, np.int8).ctypes.data, pk.ctypes.data))
            dpk, dscale = self.up(pk), self.up(in_scales[:1])
            ocp = lib().ncnnhip_padded_channels(num_output)
            dout = DeviceBuffer.empty((n, oh * ow, ocp), np.int8 if requant else np.float32)
            fused = residual is not None or relu_after or quantise_scale is not None
            dres = None if residual is None else self.to_channels_last(np.asarray(residual, np.float32))
            dq8 = None if quantise_scale is None else DeviceBuffer.empty((n, oh * ow, ocp), np.int8)
            fu = ConvFusion(_ptr(dres), int(relu_after), _ptr(dq8), float(quantise_scale or 0.0))
            wsb = C.c_size_t()
            check(lib().ncnnhip_conv_from_float_workspace_bytes(C.byref(d), C.byref(wsb)))
            dws = DeviceBuffer.zeros(wsb.value, self.stream)
            for _ in range(2):  # twice: the second launch finds the workspace as the first one left it
                check(lib().ncnnhip_conv_int8_nhwc_from_float(C.byref(d), src.ptr, np.dtype(from_float).itemsize, dscale.ptr, dpk.ptr, dsi.ptr, _ptr(db), _ptr(dso),
                                                              Activation.make(act, act_params), dout.ptr, C.byref(fu) if fused else None, dws.ptr, wsb.value, self.stream))
            raw = dout.to_numpy(self.stream)
            assert not raw[:, :, num_output:].any(), "pad channels of a channels-last blob must be zero"
            if fused:
                q8 = None if dq8 is None else self.from_channels_last(dq8, n, num_output, oh, ow)
                return self.from_channels_last(dout, n, num_output, oh, ow), q8
            return self.from_channels_last(dout, n, num_output, oh, ow)
        src = self.to_channels_last(x)
        if stem:
            if not lib().ncnnhip_conv_stem_supported(C.byref(d)):
                raise ValueError("not a narrow-input convolution")
            ib, wb, sb_ = C.c_size_t(), C.c_size_t(), C.c_size_t()
            check(lib().ncnnhip_conv_stem_sizes(C.byref(d), C.byref(ib), C.byref(wb), C.byref(sb_)))
            image = DeviceBuffer.empty((ib.value,), np.int8)
            dscale = self.up(in_scales[:1])
            check(lib().ncnnhip_quantize_stem(C.byref(d), src.ptr, x.dtype.itemsize, src.shape[2], dscale.ptr, image.ptr, self.stream))
            src = image
        elif x.dtype != np.int8:
            per_channel = np.repeat(in_scales, c // in_scales.size).astype(np.float32) if in_scales.size > 1 else in_scales
            src = self.quantize_channels_last(src, c, per_channel)
        scale_out = None
        if requant:
            ts = np.atleast_1d(np.asarray(top_scales, np.float32))
            scale_out = np.repeat(ts, num_output // ts.size).astype(np.float32)
        dsi, db, dso = self.up(scale_in), self.up(None if bias is None else np.asarray(bias, np.float32)), self.up(scale_out)
        ocp = lib().ncnnhip_padded_channels(num_output)
        dout = DeviceBuffer.empty((n, oh * ow, ocp), np.int8 if requant else np.float32)
        wq = np.ascontiguousarray(weight, np.int8)
        if stem:
            pk = np.empty(wb.value, np.int8)
            check(lib().ncnnhip_conv_stem_pack_weights(C.byref(d), wq.ctypes.data, pk.ctypes.data))
            dpk, dws = self.up(pk), DeviceBuffer.zeros(sb_.value, self.stream)
            fused = residual is not None or relu_after or quantise_scale is not None
            dres = None if residual is None else self.to_channels_last(np.asarray(residual, np.float32))
            dq8 = None if quantise_scale is None else DeviceBuffer.empty((n, oh * ow, ocp), np.int8)
            fu = ConvFusion(_ptr(dres), int(relu_after), _ptr(dq8), float(quantise_scale or 0.0))
            check(lib().ncnnhip_conv_int8_stem(C.byref(d), src.ptr, dpk.ptr, dsi.ptr, _ptr(db), _ptr(dso), Activation.make(act, act_params), dout.ptr,
                                               C.byref(fu) if fused else None, dws.ptr, sb_.value, self.stream))
            if fused:
                q8 = None if dq8 is None else self.from_channels_last(dq8, n, num_output, oh, ow)
                return self.from_channels_last(dout, n, num_output, oh, ow), q8
        elif group == 1:
            nb, wb, sb_ = C.c_size_t(), C.c_size_t(), C.c_size_t()
            check(lib().ncnnhip_conv_nhwc_sizes(C.byref(d), C.byref(nb), C.byref(wb), C.byref(sb_)))
            pk = np.empty(wb.value, np.int8)
            check(lib().ncnnhip_conv_pack_weights(C.byref(d), wq.ctypes.data, pk.ctypes.data))
            dpk, dws = self.up(pk), DeviceBuffer.zeros(sb_.value, self.stream)
            if residual is not None or relu_after or quantise_scale is not None:
                # the layers after the convolution folded into its epilogue; returns (fp32 result, its quantised copy or None)
                dres = None if residual is None else self.to_channels_last(np.asarray(residual, np.float32))
                dq8 = None if quantise_scale is None else DeviceBuffer.empty((n, oh * ow, ocp), np.int8)
                fu = ConvFusion(_ptr(dres), int(relu_after), _ptr(dq8), float(quantise_scale or 0.0))
                check(lib().ncnnhip_conv_int8_nhwc_fused(C.byref(d), src.ptr, dpk.ptr, dsi.ptr, _ptr(db), Activation.make(act, act_params), dout.ptr, C.byref(fu),
                                                         dws.ptr, sb_.value, self.stream))
                q8 = None if dq8 is None else self.from_channels_last(dq8, n, num_output, oh, ow)
                return self.from_channels_last(dout, n, num_output, oh, ow), q8
            check(lib().ncnnhip_conv_int8_nhwc(C.byref(d), src.ptr, dpk.ptr, dsi.ptr, _ptr(db), _ptr(dso), Activation.make(act, act_params), dout.ptr,
                                               1, 0, 0, dws.ptr, sb_.value, self.stream))
        else:
            nbytes = C.c_size_t()
            check(lib().ncnnhip_dwconv_packed_bytes(c, kernel[0], kernel[1], C.byref(nbytes)))
            pk = np.empty(nbytes.value, np.int8)
            check(lib().ncnnhip_dwconv_pack_weights(c, kernel[0], kernel[1], wq.ctypes.data, pk.ctypes.data))
            dpk = self.up(pk)
            check(lib().ncnnhip_dwconv_int8_nhwc(C.byref(d), src.ptr, dpk.ptr, dsi.ptr, _ptr(db), _ptr(dso), Activation.make(act, act_params), dout.ptr, self.stream))
        raw = dout.to_numpy(self.stream)
        assert not raw[:, :, num_output:].any(), "pad channels of a channels-last blob must be zero"
        return self.from_channels_last(dout, n, num_output, oh, ow)

    # -- InnerProduct -------------------------------------------------------------------------
    def innerproduct_layer(self, x, weight, bias, w_scales, in_scale, act=0, act_params=(0.0, 0.0), want_acc=False):
        x = np.ascontiguousarray(x)
        rows, k = x.shape
        weight = np.ascontiguousarray(weight, np.int8)
        num_output = weight.shape[0]
        scale_in = self.fold_input_scales(w_scales, [in_scale], num_output)
        if x.dtype == np.int8:
            dxq = self.up(x)
        else:
            dx, dsc = self.up(x.astype(np.float32)), self.up(np.asarray([in_scale], np.float32))
            dxq = DeviceBuffer.empty((rows, k), np.int8)
            check(lib().ncnnhip_quantize(dx.ptr, k, 0, dxq.ptr, k, 0, rows, k, 1, dsc.ptr, 1, self.stream))
        dw_, dsi, db = self.up(weight), self.up(scale_in), self.up(None if bias is None else np.asarray(bias, np.float32))
        dout = DeviceBuffer.empty((rows, num_output), np.float32)
        dacc = DeviceBuffer.empty((rows, num_output), np.int32) if want_acc else None
        check(lib().ncnnhip_innerproduct_int8(dxq.ptr, k, rows, k, num_output, dw_.ptr, dsi.ptr, _ptr(db), Activation.make(act, act_params),
                                              dout.ptr, num_output, _ptr(dacc), self.stream))
        out = dout.to_numpy(self.stream)
        # the workspace form (matrix cores, split K) must give the same values
        wsb = C.c_size_t()
        check(lib().ncnnhip_innerproduct_workspace_bytes(rows, k, num_output, C.byref(wsb)))
        dws = DeviceBuffer.zeros(wsb.value, self.stream)
        dout2 = DeviceBuffer.empty((rows, num_output), np.float32)
        check(lib().ncnnhip_innerproduct_int8_ws(dxq.ptr, k, rows, k, num_output, dw_.ptr, dsi.ptr, _ptr(db), Activation.make(act, act_params),
                                                 dout2.ptr, num_output, dws.ptr, wsb.value, self.stream))
        if not np.array_equal(dout2.to_numpy(self.stream), out):
            raise AssertionError("ncnnhip_innerproduct_int8_ws differs from ncnnhip_innerproduct_int8")
        return (out, dacc.to_numpy(self.stream)) if want_acc else out

    # -- Gemm int8 ----------------------------------------------------------------------------
    def gemm_quantize_rows(self, a):
        a = np.ascontiguousarray(a, np.float32)
        m, k = a.shape
        da = self.up(a)
        daq, ds = DeviceBuffer.empty((m, k), np.int8), DeviceBuffer.empty((m,), np.float32)
        check(lib().ncnnhip_gemm_quantize_rows(da.ptr, k, m, k, daq.ptr, k, ds.ptr, self.stream))
        return daq.to_numpy(self.stream), ds.to_numpy(self.stream)

    def gemm_quantize_tensor(self, b):
        b = np.ascontiguousarray(b, np.float32)
        n, k = b.shape
        db = self.up(b)
        dbq, ds = DeviceBuffer.empty((n, k), np.int8), DeviceBuffer.empty((1,), np.float32)
        check(lib().ncnnhip_gemm_quantize_tensor(db.ptr, k, n, k, dbq.ptr, k, ds.ptr, self.stream))
        return dbq.to_numpy(self.stream), ds.to_numpy(self.stream)[0]

    def gemm_int8(self, aq, bq, a_scales, b_scales, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0, output_transpose=False,
                  want_acc=False):
        aq, bq = np.ascontiguousarray(aq, np.int8), np.ascontiguousarray(bq, np.int8)
        m, k = aq.shape
        n = bq.shape[0]
        b_scales = np.ascontiguousarray(np.atleast_1d(b_scales), np.float32)
        daq, dbq, dsa, dsb = self.up(aq), self.up(bq), self.up(np.asarray(a_scales, np.float32)), self.up(b_scales)
        dc = self.up(None if c is None else np.asarray(c, np.float32))
        oshape = (n, m) if output_transpose else (m, n)
        dout = DeviceBuffer.empty(oshape, np.float32)
        dacc = DeviceBuffer.empty((m, n), np.int32) if want_acc else None
        check(lib().ncnnhip_gemm_int8(daq.ptr, k, dbq.ptr, k, m, n, k, dsa.ptr, dsb.ptr, b_scales.size, _ptr(dc),
                                      broadcast_type_c if c is not None else -1, alpha, beta, int(output_transpose), dout.ptr,
                                      oshape[1], _ptr(dacc), self.stream))
        out = dout.to_numpy(self.stream)
        return (out, dacc.to_numpy(self.stream)) if want_acc else out

    def gemm_tile_operand(self, q, operand):
        """Row-major int8 [rows][K] -> the 256x256 Gemm kernel's tiled layout (operand 0 = A, 1 = B), as a flat array."""
        q = np.ascontiguousarray(q, np.int8)
        rows, k = q.shape
        dq = self.up(q)
        dt = DeviceBuffer.empty((rows * k,), np.int8)
        check(lib().ncnnhip_gemm_int8_tile_operand(dq.ptr, k, rows, k, operand, dt.ptr, self.stream))
        return dt.to_numpy(self.stream)

    def gemm_quantize_rows_tiled(self, a):
        a = np.ascontiguousarray(a, np.float32)
        m, k = a.shape
        da = self.up(a)
        dq = DeviceBuffer.empty((m * k,), np.int8)
        ds = DeviceBuffer.empty((m,), np.float32)
        check(lib().ncnnhip_gemm_quantize_rows_tiled(da.ptr, k, m, k, dq.ptr, ds.ptr, self.stream))
        return dq.to_numpy(self.stream), ds.to_numpy(self.stream)

    def gemm_int8_tiled(self, aq_tiled, bq_tiled, m, n, k, a_scales, b_scales, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0):
        b_scales = np.ascontiguousarray(np.atleast_1d(b_scales), np.float32)
        daq, dbq = self.up(np.ascontiguousarray(aq_tiled, np.int8)), self.up(np.ascontiguousarray(bq_tiled, np.int8))
        dsa, dsb = self.up(np.asarray(a_scales, np.float32)), self.up(b_scales)
        dc = self.up(None if c is None else np.asarray(c, np.float32))
        dout = DeviceBuffer.empty((m, n), np.float32)
        check(lib().ncnnhip_gemm_int8_tiled(daq.ptr, dbq.ptr, m, n, k, dsa.ptr, dsb.ptr, b_scales.size, _ptr(dc),
                                            broadcast_type_c if c is not None else -1, alpha, beta, dout.ptr, n, self.stream))
        return dout.to_numpy(self.stream)

    def transpose(self, a):
        a = np.ascontiguousarray(a)
        r, c_ = a.shape
        da = self.up(a)
        dt = DeviceBuffer.empty((c_, r), a.dtype)
        fn = lib().ncnnhip_transpose_f32 if a.dtype == np.float32 else lib().ncnnhip_transpose_s8
        check(fn(da.ptr, c_, r, c_, dt.ptr, r, self.stream))
        return dt.to_numpy(self.stream)

    def transpose_pair_into(self, wide, col_a, col_b, cols, dst_a, dst_b, past):
        """Columns [col_a, col_a+cols) and [col_b, col_b+cols) of the fp32 matrix `wide`, transposed, written as columns past.. of dst_a / dst_b
        ([cols][time], returned as new arrays)."""
        wide = np.ascontiguousarray(wide, np.float32)
        rows, stride = wide.shape
        dst_a, dst_b = [np.ascontiguousarray(d, np.float32) for d in (dst_a, dst_b)]
        time = dst_a.shape[1]
        dw, da, db = self.up(wide), self.up(dst_a), self.up(dst_b)
        check(lib().ncnnhip_transpose_pair_f32(C.c_void_p(dw.ptr.value + col_a * 4), C.c_void_p(dw.ptr.value + col_b * 4), stride, rows, cols,
                                               C.c_void_p(da.ptr.value + past * 4), C.c_void_p(db.ptr.value + past * 4), time, self.stream))
        return da.to_numpy(self.stream), db.to_numpy(self.stream)

    # -- block-quantised Gemm -----------------------------------------------------------------
    def gemm_blockquant(self, a, b_packed, scales, bits, block, in_scales=None, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0):
        m, k = a.shape
        b_packed = np.ascontiguousarray(b_packed, np.uint8)
        n = b_packed.shape[0]
        half = a.dtype == np.float16
        da = self.up(np.ascontiguousarray(a, np.float16 if half else np.float32))
        db, ds = self.up(b_packed), self.up(np.asarray(scales, np.float32))
        dout = DeviceBuffer.empty((m, n), np.float32)
        if half:
            check(lib().ncnnhip_gemm_blockquant_f16a(da.ptr, k, m, n, k, db.ptr, bits, block, ds.ptr, dout.ptr, n, self.stream))
        else:
            dis = self.up(None if in_scales is None else np.asarray(in_scales, np.float32))
            dc = self.up(None if c is None else np.asarray(c, np.float32))
            check(lib().ncnnhip_gemm_blockquant(da.ptr, k, m, n, k, db.ptr, bits, block, ds.ptr, _ptr(dis), _ptr(dc),
                                                broadcast_type_c if c is not None else -1, alpha, beta, dout.ptr, n, self.stream))
        return dout.to_numpy(self.stream)

    def blockquant_pack(self, b_packed, scales, block, bits=8, k=None):
        """Host-side repack of block-quantised weights (the .bin's field stream, [N][ceil(K*bits/8)] bytes) into matrix-core tiles."""
        b_packed = np.ascontiguousarray(b_packed, np.uint8)
        scales = np.ascontiguousarray(scales, np.float32)
        n = b_packed.shape[0]
        k = b_packed.shape[1] * 8 // bits if k is None else k
        wb, db = C.c_size_t(), C.c_size_t()
        check(lib().ncnnhip_blockquant_packed_size(n, k, bits, block, C.byref(wb), C.byref(db)))
        pw = np.empty(wb.value, np.uint8)
        pd = np.empty(db.value // 4, np.float32)
        check(lib().ncnnhip_blockquant_pack(b_packed.ctypes.data, scales.ctypes.data, n, k, bits, block, pw.ctypes.data, pd.ctypes.data))
        return pw, pd

    def blockquant_multi_args(self, mats, douts):
        """ctypes argument arrays of ncnnhip_gemm_blockquant_packed_multi for device-resident matrices:
        mats = [(dev packed weights, dev descales, n, dev c or None, broadcast type, alpha, beta)], douts = output buffers."""
        k = len(mats)
        PtrArr, IntArr, FloatArr, SizeArr = C.c_void_p * k, C.c_int * k, C.c_float * k, C.c_size_t * k
        return (IntArr(*[m[2] for m in mats]), PtrArr(*[m[0].ptr.value for m in mats]), PtrArr(*[m[1].ptr.value for m in mats]),
                PtrArr(*[(m[3].ptr.value if m[3] is not None else None) for m in mats]), IntArr(*[(m[4] if m[3] is not None else -1) for m in mats]),
                FloatArr(*[m[5] for m in mats]), FloatArr(*[m[6] for m in mats]), PtrArr(*[d.ptr.value for d in douts]), SizeArr(*[m[2] for m in mats]))

    def gemm_blockquant_packed_multi(self, a, mats, bits=8, block=64, in_scales=None):
        """Several packed matrices on the same activation rows in one launch.  mats = [(pw, pd, n, c or None, broadcast type, alpha, beta)];
        a fp16 or fp32.  Returns the list of outputs."""
        half = a.dtype == np.float16
        a = np.ascontiguousarray(a, np.float16 if half else np.float32)
        m, k = a.shape
        da = self.up(a)
        dis = self.up(None if in_scales is None else np.asarray(in_scales, np.float32))
        dev = [(self.up(pw), self.up(pd), n, self.up(None if c is None else np.asarray(c, np.float32)), bt, alpha, beta) for pw, pd, n, c, bt, alpha, beta in mats]
        douts = [DeviceBuffer.empty((m, mt[2]), np.float32) for mt in mats]
        ns, ws, ds, cs, bts, als, bes, outs, strides = self.blockquant_multi_args(dev, douts)
        check(lib().ncnnhip_gemm_blockquant_packed_multi(da.ptr, 2 if half else 4, k, m, k, len(mats), ns, ws, ds, bits, block, _ptr(dis), cs, bts, als, bes, outs, strides,
                                                         self.stream))
        return [d.to_numpy(self.stream) for d in douts]

    def gemm_blockquant_packed(self, a, pw, pd, n, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0, bits=8, block=64, in_scales=None, rows_kernel=False):
        """a fp16: the fp16-activation entry point; a fp32 (optionally with in_scales): the layer's contract, activations split into three bf16
        (rows_kernel: the tiled form for many rows, with its workspace)."""
        half = a.dtype == np.float16
        a = np.ascontiguousarray(a, np.float16 if half else np.float32)
        m, k = a.shape
        da, dw_, dd = self.up(a), self.up(pw), self.up(pd)
        dc = self.up(None if c is None else np.asarray(c, np.float32))
        dout = DeviceBuffer.empty((m, n), np.float32)
        bt = broadcast_type_c if c is not None else -1
        if half:
            assert in_scales is None
            check(lib().ncnnhip_gemm_blockquant_packed_f16a(da.ptr, k, m, n, k, dw_.ptr, dd.ptr, bits, block, _ptr(dc), bt, alpha, beta, dout.ptr, n, self.stream))
        elif rows_kernel:
            dis = self.up(None if in_scales is None else np.asarray(in_scales, np.float32))
            wsb = C.c_size_t()
            check(lib().ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(m, k, C.byref(wsb)))
            ws = DeviceBuffer.empty((wsb.value,), np.uint8)
            check(lib().ncnnhip_gemm_blockquant_packed_rows(da.ptr, k, m, n, k, dw_.ptr, dd.ptr, bits, block, _ptr(dis), _ptr(dc), bt, alpha, beta, dout.ptr, n,
                                                            ws.ptr, wsb.value, self.stream))
        else:
            dis = self.up(None if in_scales is None else np.asarray(in_scales, np.float32))
            check(lib().ncnnhip_gemm_blockquant_packed(da.ptr, k, m, n, k, dw_.ptr, dd.ptr, bits, block, _ptr(dis), _ptr(dc), bt, alpha, beta, dout.ptr, n,
                                                       self.stream))
        return dout.to_numpy(self.stream)
