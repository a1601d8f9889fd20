"""Builders of the two benchmark networks as ncnn int8 models (.param text + .bin bytes).

What ncnn's offline tools do for a real model (tools/quantize/ncnn2table.cpp + ncnn2int8.cpp: collect activation
ranges, write int8_scale_term and the scale tables, fuse requantisation between consecutive quantised layers) is
done here for seeded random-weight networks of the ResNet-50 and MobileNetV2 shapes:

  1. build the fp32 graph with random weights,
  2. run a seeded calibration set through a plain numpy fp32 forward and record max|blob| for every blob
     (absmax calibration: scale = 127 / max|blob|),
  3. quantise weights per output channel (per group for depthwise) with 127 / max|w| and emit the layers:
     a conv whose every consumer (looking through Split) is again a quantised layer gets int8_scale_term + 100
     and top_scale = the consumers' input scale, otherwise it dequantises to fp32.

Only numpy is used; nothing here touches the GPU or the CPU checker.
"""
import numpy as np

from . import modelwriter as mw

F = np.float32
QUANTISED = ("Convolution", "ConvolutionDepthWise", "InnerProduct")


def _round_half_away(v):
    v = np.asarray(v, np.float64)
    return np.sign(v) * np.floor(np.abs(v) + 0.5)


class Graph:
    def __init__(self, seed, input_shape):
        self.rng = np.random.default_rng(seed)
        self.layers = []  # dicts: type, name, bottoms, tops, plus per-type fields
        self.input_shape = input_shape  # (c, h, w)
        self.layers.append(dict(type="Input", name="data", bottoms=[], tops=["data"]))
        self._uid = 0

    def _add(self, **kw):
        self.layers.append(kw)
        return kw["tops"][0] if len(kw["tops"]) == 1 else kw["tops"]

    def conv(self, name, bottom, cin, cout, k, stride=1, pad=0, act=0, act_params=(), sigma=None, group=1, bias=True):
        cg = cin // group
        fan_in = cg * k * k
        sd = np.sqrt(2.0 / fan_in) if sigma is None else sigma
        w = (self.rng.standard_normal((cout, cg, k, k)) * sd).astype(F)
        b = self.rng.uniform(-0.1, 0.1, cout).astype(F) if bias else None
        return self._add(type="ConvolutionDepthWise" if group > 1 else "Convolution", name=name, bottoms=[bottom], tops=[name], w=w, b=b, k=k,
                         stride=stride, pad=pad, act=act, act_params=tuple(act_params), group=group, cout=cout)

    def fc(self, name, bottom, cin, cout, sigma=None):
        sd = np.sqrt(2.0 / cin) if sigma is None else sigma
        w = (self.rng.standard_normal((cout, cin)) * sd).astype(F)
        b = self.rng.uniform(-0.1, 0.1, cout).astype(F)
        return self._add(type="InnerProduct", name=name, bottoms=[bottom], tops=[name], w=w, b=b, cout=cout)

    def pool(self, name, bottom, kind, k=0, stride=1, global_pool=False):
        return self._add(type="Pooling", name=name, bottoms=[bottom], tops=[name], kind=kind, k=k, stride=stride, global_pool=global_pool)

    def split(self, bottom, n=2):
        self._uid += 1
        name = "splitncnn_%d" % self._uid
        return self._add(type="Split", name=name, bottoms=[bottom], tops=["%s_%s_%d" % (bottom, name, i) for i in range(n)])

    def add(self, name, a, b):
        return self._add(type="Eltwise", name=name, bottoms=[a, b], tops=[name])

    def relu(self, name, bottom):
        return self._add(type="ReLU", name=name, bottoms=[bottom], tops=[name])

    def softmax(self, name, bottom):
        return self._add(type="Softmax", name=name, bottoms=[bottom], tops=[name])


# ------------------------------------------------------------------------------- topologies
def resnet50(seed=50, input_hw=224, num_classes=1000):
    """Bottleneck stages 3/4/6/3, 64..2048 channels, 7x7/2 stem, stride-2 projection shortcuts, global average pool, FC."""
    g = Graph(seed, (3, input_hw, input_hw))
    x = g.conv("conv1", "data", 3, 64, 7, stride=2, pad=3, act=1)
    x = g.pool("pool1", x, "max", k=3, stride=2)
    cin = 64
    for stage, (blocks, mid) in enumerate(((3, 64), (4, 128), (6, 256), (3, 512)), start=2):
        cout = mid * 4
        for bi in range(blocks):
            tag = "res%d%s" % (stage, "abcdef"[bi])
            stride = 2 if (bi == 0 and stage > 2) else 1
            xa, xb = g.split(x)
            if bi == 0:
                short = g.conv(tag + "_branch1", xb, cin, cout, 1, stride=stride)
            else:
                short = xb
            y = g.conv(tag + "_branch2a", xa, cin, mid, 1, stride=stride, act=1)
            y = g.conv(tag + "_branch2b", y, mid, mid, 3, pad=1, act=1)
            y = g.conv(tag + "_branch2c", y, mid, cout, 1)
            x = g.add(tag, short, y)
            x = g.relu(tag + "_relu", x)
            cin = cout
    x = g.pool("pool5", x, "avg", global_pool=True)
    x = g.fc("fc1000", x, 2048, num_classes)
    g.softmax("prob", x)
    return g


def mobilenetv2(seed=2, input_hw=224, num_classes=1000, sigma=0.1):
    """Inverted residuals with expansion 6: 1x1 expand, 3x3 depthwise (stride 1/2), 1x1 project; ReLU6; widths 112 -> 7."""
    g = Graph(seed, (3, input_hw, input_hw))
    relu6 = dict(act=3, act_params=(0.0, 6.0))
    x = g.conv("conv1", "data", 3, 32, 3, stride=2, pad=1, sigma=sigma, **relu6)
    cin = 32
    cfg = ((1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1))
    bid = 0
    for t, c, n, s in cfg:
        for i in range(n):
            bid += 1
            stride = s if i == 0 else 1
            residual = stride == 1 and cin == c
            tag = "block%d" % bid
            if residual:
                xa, xb = g.split(x)
            else:
                xa, xb = x, None
            y = xa
            hidden = cin * t
            if t != 1:
                y = g.conv(tag + "_expand", y, cin, hidden, 1, sigma=sigma, **relu6)
            y = g.conv(tag + "_dw", y, hidden, hidden, 3, stride=stride, pad=1, sigma=sigma, group=hidden, **relu6)
            y = g.conv(tag + "_project", y, hidden, c, 1, sigma=sigma)
            x = g.add(tag + "_add", xb, y) if residual else y
            cin = c
    x = g.conv("conv_last", x, cin, 1280, 1, sigma=sigma, **relu6)
    x = g.pool("pool", x, "avg", global_pool=True)
    x = g.fc("fc", x, 1280, num_classes, sigma=sigma)
    g.softmax("prob", x)
    return g


def tiny_net(seed=7, input_hw=16):
    """A few layers of every kind, for fast tests."""
    g = Graph(seed, (4, input_hw, input_hw))
    x = g.conv("c1", "data", 4, 16, 3, pad=1, act=1)
    xa, xb = g.split(x)
    y = g.conv("dw", xa, 16, 16, 3, pad=1, group=16, act=3, act_params=(0.0, 6.0))
    y = g.conv("pw", y, 16, 16, 1)
    z = g.conv("c2", xb, 16, 16, 1)
    x = g.add("sum", z, y)
    x = g.relu("relu", x)
    x = g.conv("c3", x, 16, 24, 3, stride=2, pad=1, act=1)
    x = g.pool("gap", x, "avg", global_pool=True)
    x = g.fc("fc", x, 24, 10)
    g.softmax("prob", x)
    return g


# ------------------------------------------------------------------------------- fp32 forward (calibration)
def _act(x, act, params):
    if act == 1:
        return np.maximum(x, 0)
    if act == 3:
        return np.clip(x, params[0], params[1])
    return x


def _conv_fp32(x, L):
    c, h, w = x.shape
    k, s, p, group = L["k"], L["stride"], L["pad"], L["group"]
    xp = np.pad(x, ((0, 0), (p, p), (p, p)))
    oh, ow = (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1
    cols = np.empty((c, k, k, oh, ow), F)
    for ky in range(k):
        for kx in range(k):
            cols[:, ky, kx] = xp[:, ky: ky + (oh - 1) * s + 1: s, kx: kx + (ow - 1) * s + 1: s]
    wt = L["w"]
    cout = wt.shape[0]
    if group == 1:
        y = wt.reshape(cout, -1) @ cols.reshape(c * k * k, oh * ow)
    else:
        cg, og = c // group, cout // group
        y = np.einsum("gok,gkn->gon", wt.reshape(group, og, cg * k * k), cols.reshape(group, cg * k * k, oh * ow)).reshape(cout, oh * ow)
    y = y.reshape(cout, oh, ow).astype(F)
    if L["b"] is not None:
        y = y + L["b"][:, None, None]
    return _act(y, L["act"], L["act_params"]).astype(F)


def _pool_fp32(x, L):
    if L["global_pool"]:
        return (x.reshape(x.shape[0], -1).max(axis=1) if L["kind"] == "max" else x.reshape(x.shape[0], -1).mean(axis=1)).astype(F)
    k, s = L["k"], L["stride"]
    c, h, w = x.shape
    # "full" pad mode: keep the last partial window by padding the tail
    ph = (s - (h - k) % s) % s
    pw = (s - (w - k) % s) % s
    fill = -np.inf if L["kind"] == "max" else 0.0
    xp = np.pad(x, ((0, 0), (0, ph), (0, pw)), constant_values=fill)
    oh, ow = (h + ph - k) // s + 1, (w + pw - k) // s + 1
    win = np.stack([xp[:, ky: ky + (oh - 1) * s + 1: s, kx: kx + (ow - 1) * s + 1: s] for ky in range(k) for kx in range(k)])
    return (win.max(axis=0) if L["kind"] == "max" else win.mean(axis=0)).astype(F)


def forward_fp32(g, x):
    blobs = {"data": x.astype(F)}
    for L in g.layers:
        t = L["type"]
        if t == "Input":
            continue
        ins = [blobs[b] for b in L["bottoms"]]
        if t in ("Convolution", "ConvolutionDepthWise"):
            blobs[L["tops"][0]] = _conv_fp32(ins[0], L)
        elif t == "InnerProduct":
            blobs[L["tops"][0]] = (L["w"] @ ins[0].reshape(-1) + L["b"]).astype(F)
        elif t == "Pooling":
            blobs[L["tops"][0]] = _pool_fp32(ins[0], L)
        elif t == "Split":
            for top in L["tops"]:
                blobs[top] = ins[0]
        elif t == "Eltwise":
            blobs[L["tops"][0]] = (ins[0] + ins[1]).astype(F)
        elif t == "ReLU":
            blobs[L["tops"][0]] = np.maximum(ins[0], 0)
        elif t == "Softmax":
            e = np.exp(ins[0] - ins[0].max())
            blobs[L["tops"][0]] = (e / e.sum()).astype(F)
    return blobs


def calibrate(g, n_inputs=8, seed=1234, low=0.0, high=1.0):
    """max|blob| over a seeded set of uniform random inputs."""
    rng = np.random.default_rng(seed)
    absmax = {}
    for _ in range(n_inputs):
        x = rng.uniform(low, high, g.input_shape).astype(F)
        for name, v in forward_fp32(g, x).items():
            m = float(np.abs(v).max())
            absmax[name] = max(absmax.get(name, 0.0), m)
    return absmax


# ------------------------------------------------------------------------------- int8 model emission
def _consumers(g):
    cons = {}
    for L in g.layers:
        for b in L["bottoms"]:
            cons.setdefault(b, []).append(L)
    return cons


def _all_quantised_consumers(blob, cons):
    out = cons.get(blob, [])
    if not out:
        return False
    for L in out:
        if L["type"] == "Split":
            if not all(_all_quantised_consumers(t, cons) for t in L["tops"]):
                return False
        elif L["type"] not in QUANTISED:
            return False
    return True


def to_int8_model(g, absmax):
    """Returns (.param text, .bin bytes, info) where info maps layer name -> the quantised tables (for checkers)."""
    cons = _consumers(g)
    lines, blob, info = [], b"", {}
    c, h, w = g.input_shape
    for L in g.layers:
        t, name = L["type"], L["name"]
        if t == "Input":
            lines.append("%-24s %-24s 0 1 data 0=%d 1=%d 2=%d" % ("Input", name, w, h, c))
        elif t in ("Convolution", "ConvolutionDepthWise"):
            wt = L["w"]
            cout, group = wt.shape[0], L["group"]
            depthwise = t == "ConvolutionDepthWise"
            rows = wt.reshape(group if depthwise else cout, -1)
            am = np.abs(rows).max(axis=1)
            w_scales = np.where(am == 0, F(1), F(127) / am).astype(F)
            wq = np.clip(_round_half_away((rows * w_scales[:, None]).astype(F)), -127, 127).astype(np.int8)
            in_scale = F(127) / F(absmax[L["bottoms"][0]])
            requant = _all_quantised_consumers(L["tops"][0], cons)
            top_scale = F(127) / F(absmax[L["tops"][0]]) if requant else None
            term = (1 if True else 2) + (100 if requant else 0)
            lines.append(mw.conv_param(name, L["bottoms"][0], L["tops"][0], cout, L["k"], L["stride"], L["pad"], 1, int(L["b"] is not None),
                                       wq.size, term, L["act"], L["act_params"], group if depthwise else None))
            blob += mw.conv_weights(wq.reshape(-1), L["b"], w_scales, in_scale, top_scale)
            info[name] = dict(wq=wq.reshape(wt.shape), w_scales=w_scales, in_scale=in_scale, top_scale=top_scale, term=term)
        elif t == "InnerProduct":
            wt = L["w"]
            am = np.abs(wt).max(axis=1)
            w_scales = np.where(am == 0, F(1), F(127) / am).astype(F)
            wq = np.clip(_round_half_away((wt * w_scales[:, None]).astype(F)), -127, 127).astype(np.int8)
            in_scale = F(127) / F(absmax[L["bottoms"][0]])
            lines.append(mw.innerproduct_param(name, L["bottoms"][0], L["tops"][0], wt.shape[0], wq.size, 1, 2))
            blob += mw.conv_weights(wq.reshape(-1), L["b"], w_scales, in_scale, None)
            info[name] = dict(wq=wq, w_scales=w_scales, in_scale=in_scale)
        elif t == "Pooling":
            if L["global_pool"]:
                lines.append("%-24s %-24s 1 1 %s %s 0=%d 4=1" % ("Pooling", name, L["bottoms"][0], L["tops"][0], 0 if L["kind"] == "max" else 1))
            else:
                lines.append("%-24s %-24s 1 1 %s %s 0=%d 1=%d 2=%d" % ("Pooling", name, L["bottoms"][0], L["tops"][0], 0 if L["kind"] == "max" else 1,
                                                                      L["k"], L["stride"]))
        elif t == "Split":
            lines.append("%-24s %-24s 1 %d %s %s" % ("Split", name, len(L["tops"]), L["bottoms"][0], " ".join(L["tops"])))
        elif t == "Eltwise":
            lines.append("%-24s %-24s 2 1 %s %s 0=1" % ("Eltwise", name, " ".join(L["bottoms"]), L["tops"][0]))
        elif t == "ReLU":
            lines.append("%-24s %-24s 1 1 %s %s" % ("ReLU", name, L["bottoms"][0], L["tops"][0]))
        elif t == "Softmax":
            lines.append("%-24s %-24s 1 1 %s %s" % ("Softmax", name, L["bottoms"][0], L["tops"][0]))
        else:
            raise ValueError(t)
    return mw.assemble_param(lines), blob, info


def infer_shapes(g):
    """blob name -> (c, h, w) or (n,) for vectors, by walking the graph"""
    shp = {"data": tuple(g.input_shape)}
    for L in g.layers:
        t = L["type"]
        if t == "Input":
            continue
        i0 = shp[L["bottoms"][0]]
        if t in ("Convolution", "ConvolutionDepthWise"):
            c, h, w = i0
            k, s, p = L["k"], L["stride"], L["pad"]
            shp[L["tops"][0]] = (L["cout"], (h + 2 * p - k) // s + 1, (w + 2 * p - k) // s + 1)
        elif t == "InnerProduct":
            shp[L["tops"][0]] = (L["cout"],)
        elif t == "Pooling":
            c, h, w = i0
            if L["global_pool"]:
                shp[L["tops"][0]] = (c,)
            else:
                k, s = L["k"], L["stride"]
                ph, pw = (s - (h - k) % s) % s, (s - (w - k) % s) % s
                shp[L["tops"][0]] = (c, (h + ph - k) // s + 1, (w + pw - k) // s + 1)
        elif t == "Split":
            for top in L["tops"]:
                shp[top] = i0
        else:
            shp[L["tops"][0]] = i0
    return shp


def quantised_layer_table(g):
    """One row per quantised layer: what the hot path has to compute (shapes, MACs, whether input / output are int8)."""
    shp = infer_shapes(g)
    cons = _consumers(g)
    producer = {}
    for L in g.layers:
        for top in L["tops"]:
            producer[top] = L
    rows = []
    for L in g.layers:
        if L["type"] not in QUANTISED:
            continue
        bottom, top = L["bottoms"][0], L["tops"][0]
        src = producer[bottom]
        while src["type"] == "Split":
            src = producer[src["bottoms"][0]]
        int8_in = src["type"] in QUANTISED and _all_quantised_consumers(src["tops"][0], cons)
        row = dict(name=L["name"], type=L["type"], in_shape=shp[bottom], out_shape=shp[top], int8_in=int8_in)
        if L["type"] == "InnerProduct":
            row.update(macs=int(np.prod(L["w"].shape)), int8_out=False, k=1, stride=1, pad=0, group=1, act=0, act_params=())
        else:
            cout, oh, ow = shp[top]
            row.update(macs=int(cout * oh * ow * L["w"].shape[1] * L["k"] * L["k"]), int8_out=_all_quantised_consumers(top, cons), k=L["k"],
                       stride=L["stride"], pad=L["pad"], group=L["group"], act=L["act"], act_params=L["act_params"])
        rows.append(row)
    return rows


def build(which, seed=None, input_hw=None, n_calib=8):
    make = {"resnet50": resnet50, "mobilenetv2": mobilenetv2, "tiny": tiny_net}[which]
    kw = {}
    if seed is not None:
        kw["seed"] = seed
    if input_hw is not None:
        kw["input_hw"] = input_hw
    g = make(**kw)
    absmax = calibrate(g, n_calib)
    param, binblob, info = to_int8_model(g, absmax)
    return g, param, binblob, info
