"""Reference executor for .param/.bin models built from the CPU oracle (test infrastructure).

Parses the same .param text and .bin bytes the runtime loads (its own tiny parser, written independently of the
C++ one) and runs every quantised layer through oracle/ncnn_int8_oracle.c; the fp32 glue layers are evaluated with
sequential float32 sums so that results are comparable bit for bit with ncnn's naive layers."""
import struct

import numpy as np

from oracle import oracle

F = np.float32


def parse_param(text):
    lines = [ln for ln in text.strip().split("\n")]
    assert lines[0].strip() == "7767517"
    layers = []
    for ln in lines[2:]:
        tok = ln.split()
        nb, nt = int(tok[2]), int(tok[3])
        L = dict(type=tok[0], name=tok[1], bottoms=tok[4:4 + nb], tops=tok[4 + nb:4 + nb + nt], p={})
        for kv in tok[4 + nb + nt:]:
            k, v = kv.split("=")
            k = int(k)
            if k <= -23300:
                k = -k - 23300
                vals = v.split(",")[1:]
            else:
                vals = v.split(",")
            conv = [float(x) if ("." in x or "e" in x.lower()) else int(x) for x in vals]
            L["p"][k] = conv if (len(conv) > 1 or kv.startswith("-233")) else conv[0]
        layers.append(L)
    return layers


class BinReader:
    def __init__(self, blob):
        self.b, self.pos = blob, 0

    def weights(self, n):
        tag = struct.unpack_from("<I", self.b, self.pos)[0]
        self.pos += 4
        if tag == 0x000D4B38:
            a = np.frombuffer(self.b, np.int8, n, self.pos).copy()
            self.pos += (n + 3) // 4 * 4
        else:
            assert tag == 0
            a = np.frombuffer(self.b, np.float32, n, self.pos).copy()
            self.pos += 4 * n
        return a

    def raw(self, n):
        a = np.frombuffer(self.b, np.float32, n, self.pos).copy()
        self.pos += 4 * n
        return a


def _seq_sum(v):
    """float32 sum in index order along the last axis (what a scalar C loop produces)."""
    return np.cumsum(v.astype(F), axis=-1, dtype=F)[..., -1] if v.shape[-1] else np.zeros(v.shape[:-1], F)


def _pool(x, p):
    kind = p.get(0, 0)
    if p.get(4, 0):
        flat = x.reshape(x.shape[0], -1)
        if kind == 0:
            return flat.max(axis=1).astype(F)
        return (_seq_sum(flat) / F(flat.shape[1])).astype(F)
    k, s = p.get(1, 0), p.get(2, 1)
    assert p.get(3, 0) == 0 and p.get(5, 0) == 0
    c, h, w = x.shape
    ph, pw = (s - (h - k) % s) % s, (s - (w - k) % s) % s
    oh, ow = (h + ph - k) // s + 1, (w + pw - k) // s + 1
    if kind == 1:
        # average without the border in the count (avgpool_count_include_pad = 0, src/layer/pooling.cpp:253-300): the taps of
        # a window that lie inside the image are added in float32, rows first, and divided by their number
        assert p.get(6, 0) == 0
        xp = np.pad(x, ((0, 0), (0, ph), (0, pw)))
        inside = np.pad(np.ones((h, w), bool), ((0, ph), (0, pw)))
        acc, area = np.zeros((c, oh, ow), F), np.zeros((oh, ow), F)
        for ky in range(k):
            for kx in range(k):
                sl = (slice(ky, ky + (oh - 1) * s + 1, s), slice(kx, kx + (ow - 1) * s + 1, s))
                acc = (acc + xp[(slice(None),) + sl]).astype(F)  # border taps are zeros: adding them changes nothing
                area += inside[sl]
        return (acc / area).astype(F)
    xp = np.pad(x, ((0, 0), (0, ph), (0, pw)), constant_values=-np.finfo(F).max)
    win = np.stack([xp[:, ky: ky + (oh - 1) * s + 1: s, kx: kx + (ow - 1) * s + 1: s] for ky in range(k) for kx in range(k)])
    return win.max(axis=0).astype(F)


def run(param_text, bin_blob, x, want=None):
    """x: [c][h][w] fp32.  Returns dict blob name -> array (int8 blobs stay int8)."""
    layers = parse_param(param_text)
    rd = BinReader(bin_blob)
    blobs = {}
    for L in layers:
        t, p = L["type"], L["p"]
        ins = [blobs[b] for b in L["bottoms"]]
        if t == "Input":
            blobs[L["tops"][0]] = x.astype(F)
        elif t in ("Convolution", "ConvolutionDepthWise"):
            cout, kw = p[0], p[1]
            kh = p.get(11, kw)
            group = p.get(7, 1) if t == "ConvolutionDepthWise" else 1
            term = p[8]
            wq = rd.weights(p[6])
            bias = rd.raw(cout) if p.get(5, 0) else None
            if t == "Convolution":
                ws, ins_, tops = rd.raw(cout), rd.raw(1), (rd.raw(1) if term > 100 else None)
            else:
                per_group = term in (1, 101)
                ws = rd.raw(group if per_group else 1)
                ws = ws if per_group else np.full(group, ws[0], F)
                ins_ = np.full(group, rd.raw(1)[0], F)
                tops = np.full(group, rd.raw(1)[0], F) if term > 100 else None
            xin = ins[0]
            pad = p.get(4, 0)
            ap = p.get(10, [0.0, 0.0])
            ap = list(ap) + [0.0, 0.0]
            d = oracle.make_desc(xin.shape, cout, (kw, kh), (p.get(2, 1), p.get(12, p.get(2, 1))), (p.get(3, 1), p.get(13, p.get(3, 1))),
                                 (pad, p.get(15, pad), p.get(14, pad), p.get(16, p.get(14, pad))), p.get(18, 0.0), p.get(5, 0), group, term, p.get(9, 0), ap[:2])
            cg = xin.shape[0] // group
            wq = wq.reshape(cout, cg, kh, kw)
            if t == "Convolution":
                out = oracle.convolution_int8(d, xin, wq, bias, ws, ins_[0], None if tops is None else tops[0])
            else:
                out = oracle.convolutiondepthwise_int8(d, xin, wq, bias, ws, ins_, tops)
            blobs[L["tops"][0]] = out
        elif t == "InnerProduct":
            cout = p[0]
            wq = rd.weights(p[2])
            bias = rd.raw(cout) if p.get(1, 0) else None
            ws, in_scale = rd.raw(cout), rd.raw(1)[0]
            xin = ins[0].reshape(1, -1)
            blobs[L["tops"][0]] = oracle.innerproduct_int8(xin, wq.reshape(cout, -1), bias, ws, in_scale, p.get(9, 0))[0]
        elif t == "Pooling":
            xin = ins[0].astype(F) if ins[0].dtype == np.int8 else ins[0]
            blobs[L["tops"][0]] = _pool(xin, p)
        elif t == "Split":
            for top in L["tops"]:
                blobs[top] = ins[0]
        elif t == "Eltwise":
            a, b = [v.astype(F) for v in ins]
            blobs[L["tops"][0]] = (a + b).astype(F)
        elif t == "ReLU":
            blobs[L["tops"][0]] = np.maximum(ins[0], 0)
        elif t == "Softmax":
            v = ins[0].astype(F)
            e = np.exp(v - v.max()).astype(F)
            blobs[L["tops"][0]] = (e / _seq_sum(e)).astype(F)
        else:
            raise ValueError(t)
        if want is not None and L["tops"] and L["tops"][0] == want:
            break
    return blobs
