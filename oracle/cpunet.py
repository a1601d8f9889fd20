"""Whole-model CPU pass built from the VNNI kernels of oracle/cpu_vnni_conv.c: the benchmark's CPU baseline for the
network workloads (test / benchmark infrastructure; the product package never imports this module).

Reads the same .param text and .bin bytes as the runtime.  load() does what the reference does at load time (weights
repacked, scales folded); run() is the timed part: every layer on channels-last blobs, [n][h][w][c].  Results equal the
scalar oracle's executor bit for bit (tests/test_oracle_pins.py)."""
import struct

import numpy as np

from . import cpubaseline as cb
from . import oracle

F = np.float32


def _parse_param(text):
    lines = text.strip().split("\n")
    layers = []
    for ln in lines[2:]:
        tok = ln.split()
        nb, nt = int(tok[2]), int(tok[3])
        L = dict(type=tok[0], name=tok[1], bottoms=tok[4:4 + nb], tops=tok[4 + nb:4 + nb + nt], p={})
        for kv in tok[4 + nb + nt:]:
            k, v = kv.split("=")
            k = int(k)
            vals = v.split(",")
            if k <= -23300:
                k, vals = -k - 23300, vals[1:]
            conv = [float(x) if ("." in x or "e" in x.lower()) else int(x) for x in vals]
            L["p"][k] = conv if (len(conv) > 1 or kv.startswith("-233")) else conv[0]
        layers.append(L)
    return layers


class _Bin:
    def __init__(self, blob):
        self.b, self.pos = blob, 0

    def weights(self, n):
        tag = struct.unpack_from("<I", self.b, self.pos)[0]
        self.pos += 4
        assert tag == 0x000D4B38, "the CPU baseline runs int8 models only"
        a = np.frombuffer(self.b, np.int8, n, self.pos).copy()
        self.pos += (n + 3) // 4 * 4
        return a

    def raw(self, n):
        a = np.frombuffer(self.b, np.float32, n, self.pos).copy()
        self.pos += 4 * n
        return a


def load(param_text, bin_blob):
    """-> list of prepared layers (weights packed, scales folded)."""
    rd = _Bin(bin_blob)
    model = []
    for L in _parse_param(param_text):
        t, p = L["type"], L["p"]
        if t in ("Convolution", "ConvolutionDepthWise"):
            cout, kw = p[0], p[1]
            kh = p.get(11, kw)
            group = p.get(7, 1) if t == "ConvolutionDepthWise" else 1
            term = p[8]
            wq = rd.weights(p[6])
            L["bias"] = rd.raw(cout) if p.get(5, 0) else None
            if t == "Convolution":
                ws, ins, tops = rd.raw(cout), rd.raw(1), (rd.raw(1) if term > 100 else None)
                cin = p[6] // (cout * kw * kh)
                L["packed"] = cb.pack_conv_weights(wq.reshape(cout, cin, kh, kw))
                L["in_scale"], L["scale_in"], L["scale_out"] = float(ins[0]), cb.fold_scales(ws, ins[0]), tops
            else:
                assert group == cout and p[6] == cout * kw * kh, "the CPU baseline covers depthwise layers (group == channels)"
                per_group = term in (1, 101)
                ws = rd.raw(group if per_group else 1)
                ws = ws if per_group else np.full(group, ws[0], F)
                ins = np.full(group, rd.raw(1)[0], F)
                L["taps"] = np.ascontiguousarray(wq.reshape(cout, kh * kw).T)
                L["in_scales"], L["scale_in"] = ins, cb.fold_scales(ws, ins)
                L["scale_out"] = np.full(group, rd.raw(1)[0], F) if term > 100 else None
        elif t == "InnerProduct":
            cout = p[0]
            wq = rd.weights(p[2]).reshape(cout, -1)
            L["bias"] = rd.raw(cout) if p.get(1, 0) else None
            ws, ins = rd.raw(cout), rd.raw(1)
            L["packed"] = cb.pack_b(wq)  # a 1x1 convolution over a 1x1 image
            L["k"], L["in_scale"], L["scale_in"] = wq.shape[1], float(ins[0]), cb.fold_scales(ws, ins[0])
        model.append(L)
    return model


def _desc(L, x):
    p = L["p"]
    n, h, w, c = x.shape
    kw = p[1]
    kh = p.get(11, kw)
    pad = p.get(4, 0)
    group = p.get(7, 1) if L["type"] == "ConvolutionDepthWise" else 1
    od = oracle.make_desc((c, h, w), p[0], (kw, kh), (p.get(2, 1), p.get(12, p.get(2, 1))), (p.get(3, 1), p.get(13, p.get(3, 1))),
                          (pad, p.get(15, pad), p.get(14, pad), p.get(16, p.get(14, pad))), p.get(18, 0.0), p.get(5, 0), group, p[8], p.get(9, 0), (0.0, 0.0))
    top, bottom, left, right = oracle.resolve_padding(od)
    d = cb.ConvDesc(w, h, c, n, p[0], kw, kh, od.dilation_w, od.dilation_h, od.stride_w, od.stride_h, left, right, top, bottom, float(p.get(18, 0.0)))
    ap = list(p.get(10, [0.0, 0.0])) + [0.0, 0.0] if isinstance(p.get(10, 0), list) else [0.0, 0.0]
    return d, p.get(9, 0), ap[:2]


def run(model, x, want=None, keep=None):
    """x: [n][c][h][w] fp32 (planar, as a caller holds it).  Returns blob name -> channels-last array.
    keep: the dict an earlier pass over inputs of the same shape returned; its arrays are written again instead of
    allocating new ones (what the reference's pool allocators do between inferences)."""
    blobs = {}
    keep = keep or {}
    shared = set()  # blobs with more than one consumer: an in-place layer works on a copy of those
    for L in model:
        t, p = L["type"], L["p"]
        ins = [blobs[b] for b in L["bottoms"]]
        old = keep.get(L["tops"][0]) if L["tops"] else None
        if t == "Input":
            out = cb._like(old, (x.shape[0], x.shape[2], x.shape[3], x.shape[1]), F)
            out[...] = np.asarray(x, F).transpose(0, 2, 3, 1)
        elif t == "Convolution":
            d, act, ap = _desc(L, ins[0])
            out = cb.conv_nhwc(d, ins[0], L["in_scale"], L["packed"], L["scale_in"], L["bias"], L["scale_out"], act, ap, out=old)
        elif t == "ConvolutionDepthWise":
            d, act, ap = _desc(L, ins[0])
            out = cb.dwconv_nhwc(d, ins[0], L["in_scales"], L["taps"], L["scale_in"], L["bias"], L["scale_out"], act, ap, out=old)
        elif t == "InnerProduct":
            xin = ins[0]
            n = xin.shape[0]
            if xin.shape[1] * xin.shape[2] != 1:  # flatten in the planar order the weights expect
                xin = np.ascontiguousarray(xin.transpose(0, 3, 1, 2))
            xin = xin.reshape(n, 1, 1, L["k"])
            d = cb.ConvDesc(1, 1, L["k"], n, p[0], 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, 0.0)
            out = cb.conv_nhwc(d, xin, L["in_scale"], L["packed"], L["scale_in"], L["bias"], None, p.get(9, 0), (0.0, 0.0), out=old)
        elif t == "Pooling":
            if p.get(4, 0):
                assert p.get(0, 0) == 1, "global max pooling is not used by the benchmark models"
                xin = ins[0] if ins[0].dtype == np.float32 else ins[0].astype(F)
                out = cb.global_avgpool_nhwc(xin)
            else:
                assert p.get(0, 0) == 0 and p.get(3, 0) == 0 and p.get(5, 0) == 0
                out = cb.maxpool_nhwc(ins[0], p.get(1, 0), p.get(2, 1), out=old)
        elif t == "Split":
            for top in L["tops"]:
                blobs[top] = ins[0]
                shared.add(top)
            continue
        elif t == "Eltwise":
            out = cb.add_f32(ins[0], ins[1], out=old)
        elif t == "ReLU":
            out = cb.relu_inplace(ins[0].copy() if L["bottoms"][0] in shared else ins[0])
        elif t == "Softmax":
            v = ins[0].reshape(ins[0].shape[0], -1)
            e = np.exp(v - v.max(axis=1, keepdims=True)).astype(F)
            out = (e / np.cumsum(e, axis=1, dtype=F)[:, -1:]).astype(F).reshape(ins[0].shape)
        else:
            raise ValueError(t)
        blobs[L["tops"][0]] = out
        if want is not None and L["tops"][0] == want:
            break
    return blobs
