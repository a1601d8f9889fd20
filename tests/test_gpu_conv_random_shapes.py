"""Convolution layers of seeded random shapes through whichever kernel the library picks for them, against the oracle.

The other convolution tests walk each kernel's own shapes; this one draws shapes, strides, dilations, borders, batch,
output form (fp32 / requantised), activation, input blob type (int8, fp32 / fp16 quantised inside the launch where the
layer has that form, else by a Quantize pass of its own) and now and then a fused tail without looking at which kernel
takes the layer, so that the rules that send a layer to a kernel are crossed wherever they lie.  Bit for bit.
Semantics: Convolution::forward_int8 (src/layer/convolution.cpp:383-508), ConvolutionDepthWise::forward_int8
(src/layer/convolutiondepthwise.cpp:305-520) per sample, batch as src/net.cpp:654-700."""
import ctypes as C
import os

import numpy as np
import pytest

from tests import cases
from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


def _draw(seed):
    """One layer: sizes bounded so that the oracle's scalar loops take well under a second."""
    rng = np.random.default_rng(1000 + seed)
    depthwise = rng.random() < 0.15
    batch = _pick(rng, [1, 1, 1, 2, 3, 5])
    kernel = _pick(rng, [(1, 1), (1, 1), (1, 1), (3, 3), (3, 3), (3, 3), (2, 2), (5, 5), (3, 1), (1, 3), (5, 3), (7, 7), (4, 4)])
    dilation = _pick(rng, [(1, 1), (1, 1), (1, 1), (1, 1), (2, 2), (1, 2), (3, 1)])
    stride = _pick(rng, [(1, 1), (1, 1), (1, 1), (2, 2), (2, 2), (2, 1), (3, 3), (1, 2)])
    if depthwise:
        c = outc = _pick(rng, [5, 8, 16, 32, 40, 64, 96, 144])
        if kernel == (7, 7):
            kernel = (3, 3)
    else:
        c = _pick(rng, [1, 3, 4, 8, 16, 20, 32, 48, 64, 64, 96, 128, 128, 160, 256, 512])
        outc = _pick(rng, [1, 4, 7, 16, 24, 40, 64, 64, 72, 100, 128, 130, 200, 256, 300, 512])
    ext_w, ext_h = (kernel[0] - 1) * dilation[0] + 1, (kernel[1] - 1) * dilation[1] + 1
    mode = rng.random()
    if mode < 0.25:
        pads = (-233,) * 4 if rng.random() < 0.5 else (-234,) * 4
        h, w = int(rng.integers(1, 41)), int(rng.integers(1, 41))
    else:
        pads = tuple(int(v) for v in rng.integers(0, 4, 4)) if mode < 0.75 else (0, 0, 0, 0)
        h = int(rng.integers(max(1, ext_h - pads[2] - pads[3]), 41))
        w = int(rng.integers(max(1, ext_w - pads[0] - pads[1]), 41))
    if rng.random() < 0.12:  # now and then a map large enough for the kernels built for many pixels
        h, w = (h + 60, w + 70) if c <= 64 else (h + 30, w + 20)
    term = _pick(rng, [1, 2, 101, 102])
    act, ap = _pick(rng, [(0, (0.0, 0.0)), (1, (0.0, 0.0)), (1, (0.0, 0.0)), (2, (0.1, 0.0)), (3, (0.0, 6.0)), (3, (-0.3, 0.4)), (6, (0.2, 0.5))])
    dtype = _pick(rng, [np.int8, np.int8, np.float32, np.float32, np.float16])
    bias = rng.random() < 0.8
    pad_value = 0.0
    tail = (not depthwise) and term < 100 and act == 0 and rng.random() < 0.5
    # bound the oracle's work (multiply-adds over the whole batch)
    def macs():
        ow = (w + 2 - ext_w) // stride[0] + 1
        oh = (h + 2 - ext_h) // stride[1] + 1
        return batch * max(ow, 1) * max(oh, 1) * outc * (1 if depthwise else c) * kernel[0] * kernel[1]
    while macs() > 6e7 and (h > 8 or w > 8):
        h, w = max(h * 3 // 4, 1), max(w * 3 // 4, 1)
        if pads[0] >= 0:
            h, w = max(h, ext_h), max(w, ext_w)
            if h == ext_h and w == ext_w:
                break
    return dict(depthwise=depthwise, batch=batch, c=c, h=h, w=w, outc=outc, kernel=kernel, dilation=dilation, stride=stride, pads=pads, term=term,
                act=act, ap=ap, dtype=dtype, bias=bias, pad_value=pad_value, tail=tail)


def _float_edges(x, dtype, in_scale):
    """Values that sit on float2int8's ties and beyond its range, in the blob's own type."""
    x = x.astype(dtype).astype(F)
    edge = (np.array([0.5, -0.5, 1.5, -2.5, 126.5, -126.5, 127.49, 300.0, -300.0, 0.49999997, -0.49999997], F) / in_scale).astype(dtype).astype(F)
    flat = x.reshape(-1)
    n = min(edge.size, flat.size)
    flat[:n] = edge[:n]
    return x


def _draw_large(seed):
    """A layer of 30 to 400 thousand output pixels (a batch of mid-sized maps): the kernels built for many pixels."""
    rng = np.random.default_rng(50000 + seed)
    depthwise = rng.random() < 0.2
    batch = _pick(rng, [2, 4, 8, 16])
    kernel, stride = _pick(rng, [((1, 1), (1, 1)), ((1, 1), (1, 1)), ((3, 3), (1, 1)), ((3, 3), (1, 1)), ((3, 3), (2, 2)), ((1, 1), (2, 2)), ((5, 5), (1, 1)),
                                 ((3, 1), (1, 1))])
    if depthwise:
        c = outc = _pick(rng, [16, 32, 64, 96, 144])
        if kernel[0] == 1:
            kernel = (3, 3)
    else:
        c = _pick(rng, [8, 16, 32, 64, 64, 128])
        outc = _pick(rng, [16, 24, 64, 64, 100, 128, 256])
    pads = _pick(rng, [(kernel[0] // 2, kernel[0] // 2, kernel[1] // 2, kernel[1] // 2), (-233,) * 4, (0, 0, 0, 0)])
    lo = 30000 * stride[0] * stride[1]
    for _ in range(100):
        h, w = int(rng.integers(24, 161)), int(rng.integers(24, 161))
        if lo <= batch * h * w <= 400000 * stride[0] * stride[1]:
            break
    per_px = outc * (1 if depthwise else c) * kernel[0] * kernel[1]
    while batch * h * w // (stride[0] * stride[1]) * per_px > 4e9 and h > 24:
        h = h * 3 // 4
    term = _pick(rng, [1, 2, 101, 102])
    act, ap = _pick(rng, [(0, (0.0, 0.0)), (1, (0.0, 0.0)), (1, (0.0, 0.0)), (3, (0.0, 6.0)), (2, (0.1, 0.0))])
    dtype = _pick(rng, [np.int8, np.int8, np.float32, np.float16])
    tail = (not depthwise) and term < 100 and act == 0 and rng.random() < 0.6
    return dict(depthwise=depthwise, batch=batch, c=c, h=h, w=w, outc=outc, kernel=kernel, dilation=(1, 1), stride=stride, pads=pads, term=term, act=act,
                ap=ap, dtype=dtype, bias=rng.random() < 0.8, pad_value=0.0, tail=tail)


# NCNN_RANDOM_LAYERS=<count> widens the walk (5000 layers take about a minute)
@pytest.mark.parametrize("seed", range(int(os.environ.get("NCNN_RANDOM_LAYERS", "400"))))
def test_random_layer_matches_oracle(rt, seed):
    _check(rt, seed, _draw(seed))


@pytest.mark.parametrize("seed", range(int(os.environ.get("NCNN_RANDOM_LARGE_LAYERS", "32"))))
def test_random_large_layer_matches_oracle(rt, seed):
    _check(rt, seed, _draw_large(seed))


def _check(rt, seed, p):
    from ncnn_amd.hip import ConvDesc, lib
    print("[case] random layer", seed, {k: (np.dtype(v).name if k == "dtype" else v) for k, v in p.items()}, flush=True)
    c, h, w, outc, batch, term = p["c"], p["h"], p["w"], p["outc"], p["batch"], p["term"]
    kernel, dilation, stride, pads, act, ap = p["kernel"], p["dilation"], p["stride"], p["pads"], p["act"], p["ap"]
    int8_in = p["dtype"] == np.int8
    group = c if p["depthwise"] else 1
    if min(oracle.resolve_padding(oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, group, term, act, ap))) < 0:
        # a SAME mode with a negative border: the reference's border copy runs out of bounds, oracle and library refuse the layer
        from ncnn_amd.hip import NcnnHipError
        x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, outc, kernel, group, term, True, True, by_group=p["depthwise"], batch=batch)
        with pytest.raises(NcnnHipError, match="negative border"):
            rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, group, term, act, ap)
        d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, group, term, act, ap)
        with pytest.raises(RuntimeError, match="-1"):
            (oracle.convolutiondepthwise_int8 if p["depthwise"] else oracle.convolution_int8)(d, x[0], wq, b, ws, ins if p["depthwise"] else ins[0], tops if p["depthwise"] else (None if tops is None else tops[0]))
        return
    if p["depthwise"]:
        by_group = term in (1, 101)
        x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, c, kernel, c, term, True, int8_in, by_group=True, batch=batch)
        if not by_group:
            ws = np.full(c, ws[0], F)
        # a scale of its own for every channel, so that a table read with the wrong index shows
        vary = np.random.default_rng(seed + 77)
        ins = (ins * vary.uniform(0.6, 1.0, c)).astype(F)
        tops = None if tops is None else (tops * vary.uniform(0.6, 1.4, c)).astype(F)
        if not int8_in:
            x = _float_edges(x, np.float32, ins[0])
        d = oracle.make_desc((c, h, w), c, kernel, dilation, stride, pads, 0.0, 1, c, term, act, ap)
        got = rt.conv_channels_last(x, wq, b, ws, ins, tops, c, kernel, dilation, stride, pads, 0.0, c, term, act, ap)
        for i in range(batch):
            want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
            assert got.dtype == want.dtype and np.array_equal(got[i], want), "sample %d" % i
        return
    x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, outc, kernel, 1, term, p["bias"], int8_in, batch=batch)
    from_float = None
    if not int8_in:
        x = _float_edges(x, p["dtype"], ins[0])
        dd = ConvDesc(w, h, c, batch, outc, kernel[0], kernel[1], dilation[0], dilation[1], stride[0], stride[1], pads[0], pads[1], pads[2], pads[3], 0.0, 1)
        if lib().ncnnhip_conv_from_float_supported(C.byref(dd)):
            from_float = p["dtype"]
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1 if p["bias"] else 0, 1, term, act, ap)
    want = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0]) for i in range(batch)])
    if p["tail"]:
        rng = np.random.default_rng(seed)
        res = rng.normal(0, 1, want.shape).astype(F)
        relu = bool(seed & 1)
        want = (want + res).astype(F)
        if relu:
            want = np.maximum(want, 0)
        next_scale = F(127) / max(np.abs(want).max(), F(1e-3))
        want_q = oracle.quantize(want.reshape(batch * outc, -1), [next_scale]).reshape(want.shape)
        got, got_q = rt.conv_channels_last(x, wq, b, ws, ins, None, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, ap, residual=res,
                                           relu_after=relu, quantise_scale=next_scale, from_float=from_float)
        assert np.array_equal(got, want) and np.array_equal(got_q, want_q)
        return
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, ap, from_float=from_float)
    assert got.dtype == want.dtype and np.array_equal(got, want, equal_nan=True)


@pytest.mark.parametrize("seed", range(int(os.environ.get("NCNN_RANDOM_LAYERS", "400")) // 2))
def test_random_planar_and_grouped_layer_matches_oracle(rt, seed):
    """The entry point on planar [c][h][w] blobs (ncnn's own layout: the path of host Mats): dense, depthwise and grouped
    layers (1 < group < channels, src/layer/convolutiondepthwise.cpp:515-636), with the int32 accumulators dumped beside the
    result, and the dense ones again through the channels-last kernels behind a layout change."""
    rng = np.random.default_rng(21000 + seed)
    group = _pick(rng, [1, 1, 2, 3, 4, 8, 0, 0])  # 0: depthwise
    if group == 0:
        c = outc = group = _pick(rng, [3, 8, 16, 24, 40])
    else:
        c = group * int(rng.integers(1, 9))
        outc = group * int(rng.integers(1, 13))
    batch = _pick(rng, [1, 1, 2, 3])
    kernel = _pick(rng, [(1, 1), (3, 3), (3, 3), (2, 2), (5, 3), (1, 3)])
    dilation = _pick(rng, [(1, 1), (1, 1), (2, 1), (2, 2)])
    stride = _pick(rng, [(1, 1), (1, 1), (2, 2), (1, 2)])
    ext_w, ext_h = (kernel[0] - 1) * dilation[0] + 1, (kernel[1] - 1) * dilation[1] + 1
    pads = _pick(rng, [(0, 0, 0, 0), tuple(int(v) for v in rng.integers(0, 3, 4)), (-233,) * 4, (-234,) * 4])
    grow = 0 if pads[0] < 0 else pads[0] + pads[1]
    w = int(rng.integers(max(1, ext_w - grow), 25))
    grow = 0 if pads[0] < 0 else pads[2] + pads[3]
    h = int(rng.integers(max(1, ext_h - grow), 25))
    term = _pick(rng, [1, 2, 101, 102])
    act, ap = _pick(rng, [(0, (0.0, 0.0)), (1, (0.0, 0.0)), (2, (0.1, 0.0)), (3, (0.0, 6.0)), (6, (0.2, 0.5))])
    int8_in = bool(rng.integers(2))
    pad_value = float(_pick(rng, [0.0, 0.0, -2.2, 3.7]))
    print("[case] random planar layer", seed, dict(batch=batch, c=c, h=h, w=w, outc=outc, group=group, kernel=kernel, dilation=dilation, stride=stride, pads=pads,
                                                 term=term, act=act, int8_in=int8_in, pad_value=pad_value), flush=True)
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, pad_value, 1, group, term, act, ap)
    if min(oracle.resolve_padding(d)) < 0:
        return  # (the refused SAME layers are walked by the first test of this file)
    x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, outc, kernel, group, term, True, int8_in, by_group=group > 1, batch=batch)
    if group > 1 and term in (2, 102):
        ws[:] = ws[0]
    if group > 1:
        # a scale of its own for every group, so that a table read with the wrong index shows
        ins = (ins * rng.uniform(0.6, 1.0, group)).astype(F)
        tops = None if tops is None else (tops * rng.uniform(0.6, 1.4, group)).astype(F)
        if int8_in:
            x = np.clip(np.round(x.astype(F) * rng.uniform(0.5, 1.0)), -127, 127).astype(np.int8)
    got, gacc = rt.conv_layer(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, pad_value, group, term, act, ap, want_acc=True)
    for i in range(batch):
        if group > 1:
            want, wacc = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops, want_acc=True)
        else:
            want, wacc = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0], want_acc=True)
        assert np.array_equal(gacc[i], wacc) and got.dtype == want.dtype and np.array_equal(got[i], want), "sample %d" % i
    if group == 1:
        again = rt.conv_layer(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, pad_value, 1, term, act, ap)
        assert np.array_equal(again, got)
