"""Convolution and ConvolutionDepthWise as layers -- load_param / load_model / extract -- at seeded random parameters, against
the oracle: every parameter id the layers read (kernel, dilation, stride as w / h pairs, the four pads or a SAME mode, pad_value,
bias_term, int8_scale_term 1 / 2 / 101 / 102, activation and its parameters, group for depthwise and grouped layers), fp32 input
blobs of any shape, a batch.  Bit for bit on host Mats, on blobs resident in HBM and through the plug-in
(src/layer/convolution.cpp:25-120 / 383-508, src/layer/convolutiondepthwise.cpp:25-140 / 305-640)."""
import os

import numpy as np
import pytest

from ncnn_amd import host, modelwriter as mw
from oracle import oracle
from tests import cases
from test_gpu_gemm_layer_random import _plugin

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "150"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


@pytest.mark.parametrize("route", ["host-blobs", "device-resident", "plug-in"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_convolution_layer_matches_oracle(seed, route):
    rng = np.random.default_rng(29000 + seed)
    group = _pick(rng, [1, 1, 1, 1, 0, 0, 2, 4])  # 0: depthwise
    if group == 0:
        c = outc = group = int(_pick(rng, [3, 8, 16, 24, 40, 96]))
    elif group > 1:
        c, outc = group * int(rng.integers(1, 9)), group * int(rng.integers(1, 9))
    else:
        c, outc = int(_pick(rng, [1, 3, 4, 5, 16, 20, 32, 64, 100])), int(_pick(rng, [1, 7, 16, 24, 40, 64, 100, 130]))
    batch = 1 if route == "plug-in" else _pick(rng, [1, 1, 2, 3])
    kernel = _pick(rng, [(1, 1), (3, 3), (3, 3), (2, 2), (5, 3), (1, 3), (7, 7), (3, 1)])
    dilation = _pick(rng, [(1, 1), (1, 1), (2, 1), (2, 2)])
    stride = _pick(rng, [(1, 1), (1, 1), (2, 2), (1, 2), (3, 3)])
    ext_w, ext_h = (kernel[0] - 1) * dilation[0] + 1, (kernel[1] - 1) * dilation[1] + 1
    pads = _pick(rng, [(0, 0, 0, 0), tuple(int(v) for v in rng.integers(0, 4, 4)), (1, 1, 1, 1), (-233,) * 4, (-234,) * 4])
    w = int(rng.integers(max(1, ext_w - (0 if pads[0] < 0 else pads[0] + pads[1])), 30))
    h = int(rng.integers(max(1, ext_h - (0 if pads[0] < 0 else pads[2] + pads[3])), 30))
    term = _pick(rng, [1, 2, 101, 102])
    act, ap = _pick(rng, [(0, ()), (1, ()), (2, (0.1,)), (3, (0.0, 6.0)), (3, (-0.3, 0.4)), (6, (0.2, 0.5))])
    bias = rng.random() < 0.8
    pad_value = float(_pick(rng, [0.0, 0.0, 0.0, -2.2, 3.7]))
    print("[case] random convolution layer", seed, route, dict(batch=batch, c=c, h=h, w=w, outc=outc, group=group, kernel=kernel, dilation=dilation, stride=stride,
                                                              pads=pads, term=term, act=act, bias=bias, pad_value=pad_value), flush=True)
    x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, outc, kernel, group, term, bias, False, by_group=group > 1, batch=batch)
    one_weight_scale = group > 1 and term in (2, 102)
    if one_weight_scale:
        ws[:] = ws[0]
    x.reshape(-1)[: min(x.size, 8)] = (np.array([0.5, -0.5, 1.5, -2.5, 126.5, 127.49, 300.0, -300.0], F) / ins[0])[: min(x.size, 8)]
    line = "%-24s %-24s 1 1 data out 0=%d 1=%d 11=%d 2=%d 12=%d 3=%d 13=%d 4=%d 15=%d 14=%d 16=%d 18=%s 5=%d 6=%d" % (
        "ConvolutionDepthWise" if group > 1 else "Convolution", "g", outc, kernel[0], kernel[1], dilation[0], dilation[1], stride[0], stride[1],
        pads[0], pads[1], pads[2], pads[3], mw.fmt(pad_value), int(bias), wq.size)
    if group > 1:
        line += " 7=%d" % group
    line += " 8=%d" % term
    if act:
        line += " 9=%d" % act
    if len(ap):
        line += " -23310=%d,%s" % (len(ap), ",".join(mw.fmt(v) for v in ap))
    lines = ["Input in0 0 1 data 0=%d 1=%d 2=%d" % (w, h, c), line]
    # (the model file holds ONE input scale and one top scale for a depthwise layer too: load_model spreads them over the groups,
    # src/layer/convolutiondepthwise.cpp:118-140)
    blob = mw.conv_weights(wq, b, ws[:1] if one_weight_scale else ws, ins[0], None if tops is None else tops[0])
    net = host.Net()
    if route == "plug-in":
        assert _plugin().ncnnhip_plugin_register(net.h_) == 0
    else:
        assert net.register_int8_layers() == 0
        net.set_use_hip_compute(route == "device-resident")
    assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(blob) == 0
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, pad_value, int(bias), group, term, act, tuple(ap) + (0.0, 0.0))
    ex = net.create_extractor()
    ex.input("data", x if batch > 1 else x[0])
    if min(oracle.resolve_padding(d)) < 0:
        with pytest.raises(RuntimeError):  # a SAME mode with a negative border: refused as the reference's border copy runs out of bounds
            ex.extract("out")
        return
    got = np.asarray(ex.extract("out"))
    for i in range(batch):
        if group > 1:
            want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
        else:
            want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0])
        gi = got[i] if batch > 1 else got
        assert gi.shape == want.shape and np.array_equal(gi, want.astype(F)), "sample %d" % i  # (extract hands int8 blobs over as fp32 values)
