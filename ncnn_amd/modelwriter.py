"""Writer of ncnn .param text and .bin weight streams for the int8 / block-quant layers.

Byte layout follows what ncnn's loaders read (src/modelbin.cpp:82-338 and the layers' load_model): every weight
blob is a 4-byte tag + payload padded to 4 bytes (int8 tag 0x000D4B38, fp32 tag 0), bias and scale tables are raw
fp32.  Floats in .param text are always written with an exponent so the parser stores them as floats."""
import struct

import numpy as np

INT8_TAG = 0x000D4B38


def _pad4(b):
    return b + b"\0" * (-len(b) % 4)


def weight_blob(w):
    w = np.ascontiguousarray(w)
    if w.dtype == np.int8 or w.dtype == np.uint8:
        return struct.pack("<I", INT8_TAG) + _pad4(w.tobytes())
    return struct.pack("<I", 0) + w.astype(np.float32).tobytes()


def raw_f32(a):
    return np.ascontiguousarray(np.atleast_1d(a), np.float32).tobytes()


def conv_weights(weight, bias, w_scales, in_scale, top_scale):
    """Convolution / ConvolutionDepthWise / InnerProduct order: weights, bias, weight scales, input scale, top scale."""
    out = weight_blob(weight)
    if bias is not None:
        out += raw_f32(bias)
    out += raw_f32(w_scales) + raw_f32(in_scale)
    if top_scale is not None:
        out += raw_f32(top_scale)
    return out


def fmt(v):
    return "%e" % float(v)


def conv_param(name, bottom, top, num_output, kernel, stride=1, pad=0, dilation=1, bias=1, weight_size=0, term=1, act=0, act_params=(),
               group=None):
    kw, kh = (kernel, kernel) if np.isscalar(kernel) else kernel
    s = "%-24s %-24s 1 1 %s %s 0=%d 1=%d 11=%d 2=%d 3=%d 4=%d 5=%d 6=%d" % ("ConvolutionDepthWise" if group else "Convolution", name, bottom, top,
                                                                          num_output, kw, kh, dilation, stride, pad, bias, weight_size)
    if group:
        s += " 7=%d" % group
    s += " 8=%d" % term
    if act:
        s += " 9=%d" % act
    if len(act_params):
        s += " -23310=%d,%s" % (len(act_params), ",".join(fmt(v) for v in act_params))
    return s


def innerproduct_param(name, bottom, top, num_output, weight_size, bias=1, term=2, act=0):
    s = "%-24s %-24s 1 1 %s %s 0=%d 1=%d 2=%d 8=%d" % ("InnerProduct", name, bottom, top, num_output, bias, weight_size, term)
    if act:
        s += " 9=%d" % act
    return s


def gemm_param(name, bottoms, top, M=0, N=0, K=0, alpha=1.0, beta=1.0, transA=0, transB=1, constantA=0, constantB=1, constantC=0,
               broadcast_type_C=0, quantize_term=2, output_transpose=0, output_N1M=0):
    return ("%-24s %-24s %d 1 %s %s 0=%s 1=%s 2=%d 3=%d 4=%d 5=%d 6=%d 7=%d 8=%d 9=%d 10=%d 11=%d 14=%d 18=%d"
            % ("Gemm", name, len(bottoms), " ".join(bottoms), top, fmt(alpha), fmt(beta), transA, transB, constantA, constantB, constantC, M, N, K,
               broadcast_type_C, output_N1M, output_transpose, quantize_term))


def mha_param(name, bottoms, tops, embed_dim, num_heads, qdim, kdim=None, vdim=None, attn_mask=0, kv_cache=0, quantize_term=801, scale=None):
    """MultiHeadAttention (src/layer/multiheadattention.cpp:64-76): 2 = weight_data_size = embed_dim * qdim."""
    s = "%-24s %-24s %d %d %s %s 0=%d 1=%d 2=%d 3=%d 4=%d 5=%d" % ("MultiHeadAttention", name, len(bottoms), len(tops), " ".join(bottoms), " ".join(tops),
                                                                 embed_dim, num_heads, embed_dim * qdim, kdim or embed_dim, vdim or embed_dim, attn_mask)
    if scale is not None:
        s += " 6=%s" % fmt(scale)
    return s + " 7=%d 18=%d" % (kv_cache, quantize_term)


def mha_blockquant_weights(weights):
    """weights: 4 x (packed uint8 [rows][bytes], scales [rows][nblk], input scales [K] or None, bias [rows]) for q, k, v, out, in the order
    MultiHeadAttention::load_model reads them (src/layer/multiheadattention.cpp:137-184): weight+bias pairs, then the block scales,
    then the input scales."""
    out = b""
    for packed, scales, ins, bias in weights:
        out += weight_blob(np.ascontiguousarray(packed).view(np.int8)) + raw_f32(bias)
    for packed, scales, ins, bias in weights:
        out += raw_f32(scales)
    for packed, scales, ins, bias in weights:
        if ins is not None:
            out += raw_f32(ins)
    return out


def assemble_param(lines):
    """lines: layer lines in order; counts layers and distinct blobs for the header."""
    blobs = set()
    for ln in lines:
        tok = ln.split()
        nb, nt = int(tok[2]), int(tok[3])
        blobs.update(tok[4: 4 + nb + nt])
    return "7767517\n%d %d\n%s\n" % (len(lines), len(blobs), "\n".join(lines))
