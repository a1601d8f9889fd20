"""ctypes front-end of the CPU checker (oracle/ncnn_int8_oracle.c).

Test infrastructure only: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg.  The product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")


def build(force=False):
    src = os.path.join(_HERE, "ncnn_int8_oracle.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "liboracle.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


class ConvDesc(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("w", "h", "c", "num_output", "kernel_w", "kernel_h", "dilation_w", "dilation_h",
                                       "stride_w", "stride_h", "pad_left", "pad_right", "pad_top", "pad_bottom")] + \
               [("pad_value", C.c_float), ("bias_term", C.c_int), ("group", C.c_int), ("int8_scale_term", C.c_int),
                ("activation_type", C.c_int), ("activation_params", C.c_float * 2)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.oracle_float2int8.restype = C.c_int8
        _lib.oracle_float2int8.argtypes = [C.c_float]
        _lib.oracle_activation.restype = C.c_float
        _lib.oracle_activation.argtypes = [C.c_float, C.c_int, C.c_void_p]
        _lib.oracle_gemm_quantize_tensor.restype = C.c_float
        _lib.oracle_blockquant_unpack.restype = C.c_int
        _lib.oracle_num_threads.restype = C.c_int
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _f32(a):
    return None if a is None else np.ascontiguousarray(a, dtype=np.float32)


def set_num_threads(n):
    lib().oracle_set_num_threads(C.c_int(int(n)))


def num_threads():
    return int(lib().oracle_num_threads())


def float2int8(v):
    v = np.asarray(v, dtype=np.float32)
    out = np.empty(v.shape, np.int8)
    f = lib().oracle_float2int8
    flat_in, flat_out = v.reshape(-1), out.reshape(-1)
    for i in range(flat_in.size):
        flat_out[i] = f(C.c_float(float(flat_in[i])))
    return out


def activation(v, act_type, params=(0.0, 0.0)):
    p = np.zeros(2, np.float32)
    p[: len(params)] = params
    return float(lib().oracle_activation(C.c_float(float(v)), int(act_type), _p(p)))


def quantize(x, scales):
    """x [rows][cols] fp32, scales of length 1 or rows -> int8."""
    x = _f32(x)
    scales = _f32(np.atleast_1d(scales))
    rows, cols = x.shape
    y = np.empty((rows, cols), np.int8)
    lib().oracle_quantize(_p(x), C.c_size_t(cols), _p(y), C.c_size_t(cols), rows, cols, _p(scales), int(scales.size))
    return y


def make_desc(x_shape, num_output, kernel, dilation=(1, 1), stride=(1, 1), pads=(0, 0, 0, 0), pad_value=0.0, bias_term=0,
              group=1, int8_scale_term=1, activation_type=0, activation_params=(0.0, 0.0)):
    """kernel/dilation/stride are (w, h); pads are (left, right, top, bottom) as in the param ids 4,15,14,16."""
    c, h, w = x_shape
    d = ConvDesc()
    d.w, d.h, d.c = w, h, c
    d.num_output = num_output
    d.kernel_w, d.kernel_h = kernel
    d.dilation_w, d.dilation_h = dilation
    d.stride_w, d.stride_h = stride
    d.pad_left, d.pad_right, d.pad_top, d.pad_bottom = pads
    d.pad_value = pad_value
    d.bias_term = bias_term
    d.group = group
    d.int8_scale_term = int8_scale_term
    d.activation_type = activation_type
    ap = list(activation_params) + [0.0, 0.0]
    d.activation_params[0], d.activation_params[1] = ap[0], ap[1]
    return d


def resolve_padding(desc):
    """Explicit (top, bottom, left, right) borders of a layer description (-233 / -234 resolved as the reference does)."""
    out = (C.c_int * 4)()
    lib().oracle_resolve_padding(desc.w, desc.h, desc.kernel_w, desc.kernel_h, desc.dilation_w, desc.dilation_h, desc.stride_w, desc.stride_h,
                                 desc.pad_left, desc.pad_right, desc.pad_top, desc.pad_bottom, out)
    return tuple(out)


def conv_out_shape(desc):
    ow, oh = C.c_int(), C.c_int()
    lib().oracle_conv_out_shape(C.byref(desc), C.byref(ow), C.byref(oh))
    return oh.value, ow.value


def _conv_family(fn, desc, x, weight, bias, w_scales, in_scales, top_scales, want_acc):
    x = np.ascontiguousarray(x)
    assert x.dtype in (np.float32, np.int8) and x.ndim == 3
    weight = np.ascontiguousarray(weight, dtype=np.int8)
    oh, ow = conv_out_shape(desc)
    requant = desc.int8_scale_term > 100
    out = np.empty((desc.num_output, oh, ow), np.int8 if requant else np.float32)
    acc = np.empty((desc.num_output, oh, ow), np.int32) if want_acc else None
    bias, w_scales, in_scales, top_scales = _f32(bias), _f32(w_scales), _f32(in_scales), _f32(top_scales)
    ret = fn(C.byref(desc), _p(x), int(x.dtype.itemsize), C.c_size_t(x.shape[1] * x.shape[2]), _p(weight), _p(bias),
             _p(w_scales), _p(in_scales), _p(top_scales), _p(out), C.c_size_t(oh * ow), _p(acc))
    if ret != 0:
        raise RuntimeError("oracle returned %d" % ret)
    return (out, acc) if want_acc else out


def convolution_int8(desc, x, weight, bias, w_scales, in_scale, top_scale=None, want_acc=False):
    return _conv_family(lib().oracle_convolution_int8, desc, x, weight, bias, w_scales, np.atleast_1d(in_scale),
                        None if top_scale is None else np.atleast_1d(top_scale), want_acc)


def convolutiondepthwise_int8(desc, x, weight, bias, w_scales, in_scales, top_scales=None, want_acc=False):
    """Scale arrays must already have `group` entries, as the layer holds them after load_model."""
    return _conv_family(lib().oracle_convolutiondepthwise_int8, desc, x, weight, bias, w_scales, in_scales, top_scales,
                        want_acc)


def quantize_weights(w, scales):
    """w [rows][row_size] fp32, one scale per row."""
    w = _f32(w)
    scales = _f32(np.atleast_1d(scales))
    rows, rs = w.shape
    assert scales.size == rows
    out = np.empty((rows, rs), np.int8)
    lib().oracle_quantize_weights(_p(w), _p(out), rows, rs, _p(scales))
    return out


def innerproduct_int8(x, weight, bias, w_scales, in_scale, activation_type=0, activation_params=(0.0, 0.0), want_acc=False):
    """x [rows][num_input] fp32 or int8; weight int8 [num_output][num_input] -> fp32 [rows][num_output]."""
    x = np.ascontiguousarray(x)
    rows, num_input = x.shape
    weight = np.ascontiguousarray(weight, dtype=np.int8)
    num_output = weight.shape[0]
    out = np.empty((rows, num_output), np.float32)
    acc = np.empty((rows, num_output), np.int32) if want_acc else None
    ap = np.zeros(2, np.float32)
    ap[: len(activation_params)] = activation_params
    bias, w_scales, in_scale = _f32(bias), _f32(w_scales), _f32(np.atleast_1d(in_scale))
    ret = lib().oracle_innerproduct_int8(_p(x), int(x.dtype.itemsize), C.c_size_t(num_input), rows, num_input, num_output,
                                         _p(weight), _p(bias), _p(w_scales), _p(in_scale), int(activation_type), _p(ap),
                                         _p(out), C.c_size_t(num_output), _p(acc))
    if ret != 0:
        raise RuntimeError("oracle returned %d" % ret)
    return (out, acc) if want_acc else out


def gemm_quantize_rows(a):
    a = _f32(a)
    m, k = a.shape
    aq = np.empty((m, k), np.int8)
    s = np.empty(m, np.float32)
    lib().oracle_gemm_quantize_rows(_p(a), C.c_size_t(k), m, k, _p(aq), C.c_size_t(k), _p(s))
    return aq, s


def gemm_quantize_tensor(b):
    b = _f32(b)
    n, k = b.shape
    bq = np.empty((n, k), np.int8)
    s = lib().oracle_gemm_quantize_tensor(_p(b), C.c_size_t(k), n, k, _p(bq), C.c_size_t(k))
    return bq, np.float32(s)


def gemm_int8(aq, bq, a_scales, b_scales, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0, output_transpose=False,
              want_acc=False):
    aq = np.ascontiguousarray(aq, dtype=np.int8)
    bq = np.ascontiguousarray(bq, dtype=np.int8)
    m, k = aq.shape
    n = bq.shape[0]
    assert bq.shape[1] == k
    a_scales = _f32(a_scales)
    b_scales = _f32(np.atleast_1d(b_scales))
    c = _f32(c)
    out = np.empty((n, m) if output_transpose else (m, n), np.float32)
    acc = np.empty((m, n), np.int32) if want_acc else None
    lib().oracle_gemm_int8(_p(aq), C.c_size_t(k), _p(bq), C.c_size_t(k), m, n, k, _p(a_scales), _p(b_scales),
                           int(b_scales.size), _p(c), int(broadcast_type_c if c is not None else -1), C.c_float(alpha),
                           C.c_float(beta), int(bool(output_transpose)), _p(out), C.c_size_t(out.shape[1]), _p(acc))
    return (out, acc) if want_acc else out


def blockquant_pack(w, bits, block):
    w = _f32(w)
    n, k = w.shape
    packed = (k * bits + 7) // 8
    nblk = (k + block - 1) // block
    q = np.zeros((n, packed), np.uint8)
    s = np.empty((n, nblk), np.float32)
    lib().oracle_blockquant_pack(_p(w), n, k, int(bits), int(block), _p(q), _p(s))
    return q, s


def blockquant_unpack(row, k, bits):
    row = np.ascontiguousarray(row, dtype=np.uint8)
    return int(lib().oracle_blockquant_unpack(_p(row), int(k), int(bits), int(row.size)))


def gemm_blockquant(a, b_packed, scales, bits, block, in_scales=None, c=None, broadcast_type_c=-1, alpha=1.0, beta=1.0):
    a = _f32(a)
    m, k = a.shape
    b_packed = np.ascontiguousarray(b_packed, dtype=np.uint8)
    n = b_packed.shape[0]
    assert b_packed.shape[1] == (k * bits + 7) // 8
    scales = _f32(scales)
    in_scales, c = _f32(in_scales), _f32(c)
    out = np.empty((m, n), np.float32)
    lib().oracle_gemm_blockquant(_p(a), C.c_size_t(k), m, n, k, _p(b_packed), int(bits), int(block), _p(scales),
                                 _p(in_scales), _p(c), int(broadcast_type_c if c is not None else -1), C.c_float(alpha),
                                 C.c_float(beta), _p(out), C.c_size_t(n))
    return out


class MhaWeight(C.Structure):
    _fields_ = [("packed", C.c_void_p), ("scales", C.c_void_p), ("in_scales", C.c_void_p), ("bias", C.c_void_p)]


class MhaDesc(C.Structure):
    _fields_ = [(n, C.c_int) for n in ("embed_dim", "num_heads", "qdim", "kdim", "vdim", "src_seqlen", "cur_seqlen", "past_seqlen", "self_attention",
                                       "mask_heads")] + [("scale", C.c_float), ("bits", C.c_int), ("block", C.c_int)]


def mha_blockquant(q, k, v, weights, embed_dim, num_heads, scale, bits, block, mask=None, cached_k=None, cached_v=None, self_attention=True):
    """MultiHeadAttention with block-quantised weights.  q [src][qdim], k [cur][kdim], v [cur][vdim];
    weights = 4 x (packed uint8 [rows][..], scales [rows][nblk], in_scales [K] or None, bias [rows]) for q, k, v, out;
    mask [src][dst] or [heads][src][dst]; cached_k / cached_v [embed_dim][past].  Returns (out, k_cache, v_cache)."""
    q, k, v = _f32(q), _f32(k), _f32(v)
    src, qdim = q.shape
    cur = k.shape[0]
    past = 0 if cached_k is None else cached_k.shape[1]
    dst = (past + cur if self_attention else past) if past > 0 else cur
    keep, ws = [], (MhaWeight * 4)()
    for i, (packed, scales, in_scales, bias) in enumerate(weights):
        arrs = [np.ascontiguousarray(packed, np.uint8), _f32(scales), _f32(in_scales), _f32(bias)]
        keep.append(arrs)
        ws[i] = MhaWeight(*[None if a is None else a.ctypes.data for a in arrs])
    mask, cached_k, cached_v = _f32(mask), _f32(cached_k), _f32(cached_v)
    mask_heads = 0 if mask is None else (1 if mask.ndim == 2 else mask.shape[0])
    d = MhaDesc(embed_dim, num_heads, qdim, k.shape[1], v.shape[1], src, cur, past, int(bool(self_attention)), mask_heads, float(scale), bits, block)
    out = np.empty((src, qdim), np.float32)
    ko = np.empty((embed_dim, dst), np.float32)
    vo = np.empty((embed_dim, dst), np.float32)
    ret = lib().oracle_mha_blockquant(C.byref(d), _p(q), _p(k), _p(v), _p(mask), _p(cached_k), _p(cached_v), ws, _p(out), _p(ko), _p(vo))
    if ret != 0:
        raise RuntimeError("oracle_mha_blockquant returned %d" % ret)
    return out, ko, vo
