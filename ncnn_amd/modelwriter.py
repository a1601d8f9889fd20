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


# The reference's number for a layer type: its place among the ncnn_add_layer calls of src/CMakeLists.txt:66-176 (the
# generated layer_type_enum.h); a .param.bin file names its layers by these numbers.
LAYER_TYPE_INDEX = {"Dropout": 9, "Eltwise": 10, "Flatten": 14, "InnerProduct": 15, "Input": 16, "Pooling": 21, "ReLU": 26, "Softmax": 32,
                    "Split": 33, "Convolution": 6, "ConvolutionDepthWise": 42, "Gemm": 74, "MultiHeadAttention": 79}


def _is_float_text(v):
    return "." in v or "e" in v.lower()


def assemble_param_bin(lines, custom_types=()):
    """The same net as assemble_param(lines) in the binary form Net::load_param_bin reads (src/net.cpp:1667-2018), as
    tools/ncnn2mem.cpp writes it: 32-bit little-endian words; magic, layer count, blob count; per layer the type number,
    bottom count, top count, the blob numbers (in order of first appearance in the text), then per parameter its id and
    value -- id as it is for a scalar (a value with '.' or 'e' in its text is a float, anything else an int), -23300 - id
    and a length before an array, -23400 - id, a length and the bytes padded to words before a string -- and -233 to end
    the layer.  custom_types: names of registered custom layers, numbered 256 + place."""
    number, out = {}, []
    for ln in lines:
        tok = ln.split()
        nb, nt = int(tok[2]), int(tok[3])
        for b in tok[4: 4 + nb + nt]:
            number.setdefault(b, len(number))
    out.append(struct.pack("<3i", 7767517, len(lines), len(number)))
    for ln in lines:
        tok = ln.split()
        nb, nt = int(tok[2]), int(tok[3])
        ti = LAYER_TYPE_INDEX[tok[0]] if tok[0] in LAYER_TYPE_INDEX else 256 + list(custom_types).index(tok[0])
        out.append(struct.pack("<3i", ti, nb, nt))
        out.append(struct.pack("<%di" % (nb + nt), *[number[b] for b in tok[4: 4 + nb + nt]]))
        for item in tok[4 + nb + nt:]:
            key, value = item.split("=", 1)
            pid = int(key)
            if pid <= -23300:
                vals = value.split(",")
                count = int(vals[0])
                out.append(struct.pack("<2i", pid, count))
                for v in vals[1: 1 + count]:
                    out.append(struct.pack("<f", float(v)) if _is_float_text(v) else struct.pack("<i", int(v)))
            elif value[:1] == '"' or value[:1].isalpha():
                text = value.strip('"').encode()
                out.append(struct.pack("<2i", -23400 - pid, len(text)) + _pad4(text))
            else:
                out.append(struct.pack("<i", pid) + (struct.pack("<f", float(value)) if _is_float_text(value) else struct.pack("<i", int(value))))
        out.append(struct.pack("<i", -233))
    return b"".join(out), number
