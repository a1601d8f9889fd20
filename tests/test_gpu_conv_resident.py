"""The weights-resident convolution kernel (kernels with taps on layers with many output pixels: the batched nets)
against the oracle.

The kernel is chosen by the layer's shape (taps, 40000 output pixels and more); the environment variables
NCNNHIP_RESIDENT_MIN (pixel threshold) and NCNNHIP_RESIDENT_CFG (tile configuration 0..7) are read at every launch, so
the small cases here lower the threshold and walk every tile configuration, and the large ones run as a net would.
Semantics: Convolution::forward_int8 (src/layer/convolution.cpp:383-508) per sample, batch as src/net.cpp:654-700."""
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


@pytest.fixture
def resident_env():
    """Lowers the pixel threshold for a test and restores the environment afterwards."""
    saved = {k: os.environ.get(k) for k in ("NCNNHIP_RESIDENT_MIN", "NCNNHIP_RESIDENT_CFG", "NCNNHIP_RESIDENT_OFF")}

    def set_env(min_pixels=None, cfg=None):
        for k, v in (("NCNNHIP_RESIDENT_MIN", min_pixels), ("NCNNHIP_RESIDENT_CFG", cfg)):
            if v is None:
                os.environ.pop(k, None)
            else:
                os.environ[k] = str(v)
    yield set_env
    for k, v in saved.items():
        if v is None:
            os.environ.pop(k, None)
        else:
            os.environ[k] = v


def _say(*a):
    print("[case]", *a, flush=True)


def _check(rt, seed, batch, c, h, w, outc, kernel, dilation, stride, pads, term, act, act_params, bias=True, flip=False):
    x, wq, b, ws, ins, tops = cases.conv_case(seed, c, h, w, outc, kernel, 1, term, bias, True, batch=batch)
    if tops is not None and flip:
        tops = -tops
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1 if bias else 0, 1, term, act, act_params)
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, act_params)
    for i in range(batch):
        want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0])
        assert got.dtype == want.dtype and np.array_equal(got[i], want), "sample %d" % i


SMALL = [
    # batch, c, h, w, outc, kernel, dilation, stride, pads
    (3, 64, 13, 11, 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),     # tiles that cross rows and images, ragged last tile
    (2, 64, 9, 10, 40, (3, 3), (1, 1), (2, 2), (1, 1, 1, 1)),      # stride 2, channel tail (40 of 48 stored)
    (2, 128, 7, 7, 96, (3, 3), (2, 2), (1, 1), (2, 2, 2, 2)),      # dilation 2, two K steps per tap
    (1, 64, 12, 9, 70, (5, 3), (1, 1), (1, 2), (-233, -233, -233, -233)),  # SAME pads, 15 taps, uneven strides
    (2, 64, 10, 10, 32, (2, 2), (1, 1), (1, 1), (0, 0, 0, 0)),     # no padding, even kernel
    (5, 64, 7, 7, 100, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),      # small maps: tiles that hold several images
    (2, 192, 8, 8, 200, (3, 1), (1, 1), (1, 1), (1, 0, 1, 0)),     # several channel blocks, the last one partly padding; a column kernel
    (3, 64, 6, 40, 24, (1, 3), (1, 1), (1, 1), (0, 1, 0, 1)),      # a row kernel on a wide, low image
    (2, 256, 11, 13, 64, (2, 2), (1, 1), (2, 2), (0, 0, 0, 0)),    # non-overlapping 2x2 patches, four K pieces per tap
]


@pytest.mark.parametrize("cfg", range(8))
@pytest.mark.parametrize("shape", SMALL)
def test_every_tile_configuration_on_small_layers(rt, resident_env, cfg, shape):
    batch, c, h, w, outc, kernel, dilation, stride, pads = shape
    _say("resident small", cfg, shape)
    resident_env(min_pixels=1, cfg=cfg)
    for term, act, act_params in [(102, 1, (0.0, 0.0)), (2, 0, (0.0, 0.0))]:
        _check(rt, c + outc + cfg, batch, c, h, w, outc, kernel, dilation, stride, pads, term, act, act_params)


@pytest.mark.parametrize("act,act_params,flip,bias", [(0, (0.0, 0.0), False, True), (1, (0.0, 0.0), True, True), (3, (0.0, 6.0), False, False),
                                                      (3, (0.3, -0.2), False, True), (3, (-1e30, 1e30), False, True), (3, (float("-inf"), 0.5), False, True),
                                                      (3, (-0.4, 0.4), True, True)])
def test_activations_folded_into_the_clamp_or_taken_literally(rt, resident_env, act, act_params, flip, bias):
    """ReLU and clip fold into the requantising clamp when the tables allow it; negative output scales (flip), reversed,
    huge and infinite bounds take the literal path.  On a 3x3 and a 2x2 layer, per-channel and per-tensor output scales."""
    _say("resident activations", act, act_params, flip, bias)
    resident_env(min_pixels=1)
    _check(rt, 5, 2, 64, 12, 11, 48, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 102, act, act_params, bias, flip)
    _check(rt, 6, 2, 64, 12, 11, 80, (2, 2), (1, 1), (1, 1), (0, 0, 0, 0), 101, act, act_params, bias, flip)


@pytest.mark.parametrize("c,h,w,outc,kernel,pads,relu", [(64, 14, 14, 256, (3, 3), (1, 1, 1, 1), True), (64, 20, 18, 40, (3, 3), (1, 1, 1, 1), False),
                                                           (128, 7, 7, 200, (2, 2), (0, 0, 0, 0), True)])
@pytest.mark.parametrize("cfg", [0, 3, 4, 7])
def test_fused_tail_residual_relu_quantised_copy(rt, resident_env, c, h, w, outc, kernel, pads, relu, cfg):
    _say("resident fused tail", c, h, w, outc, kernel, relu, cfg)
    resident_env(min_pixels=1, cfg=cfg)
    rng = np.random.default_rng(c + outc)
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc, c, h, w, outc, kernel, 1, 2, True, True, batch=3)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), (1, 1), pads, 0.0, 1, 1, 2, 0, (0.0, 0.0))
    conv = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None) for i in range(3)])
    res = rng.normal(0, 1, conv.shape).astype(F)
    want = (conv + res).astype(F)
    if relu:
        want = np.maximum(want, 0)
    next_scale = F(127) / np.abs(want).max()
    want_q = oracle.quantize(want.reshape(-1, want.shape[-1]), [next_scale]).reshape(want.shape)
    got, got_q = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, (1, 1), (1, 1), pads, 0.0, 1, 2, 0, (0.0, 0.0),
                                       residual=res, relu_after=relu, quantise_scale=next_scale)
    assert np.array_equal(got, want)
    assert np.array_equal(got_q, want_q)


@pytest.mark.parametrize("batch,c,h,w,outc,kernel,stride,pads,term,act", [
    (20, 64, 56, 56, 64, (3, 3), (1, 1), (1, 1, 1, 1), 102, 1),    # ResNet-50 res2 branch2b: more tiles than the chip holds workgroups
    (24, 128, 28, 28, 128, (3, 3), (1, 1), (1, 1, 1, 1), 102, 1),  # res3 branch2b
    (9, 256, 14, 14, 256, (3, 3), (1, 1), (1, 1, 1, 1), 102, 1),   # res4 branch2b: tiles run from one image into the next
    (5, 64, 57, 57, 96, (3, 3), (2, 2), (0, 0, 0, 0), 2, 0),       # stride 2 without padding, fp32 out
    (3, 64, 40, 40, 48, (3, 3), (1, 1), (1, 1, 1, 1), 102, 3),     # clip
])
def test_benchmark_layer_shapes_as_a_net_runs_them(rt, resident_env, batch, c, h, w, outc, kernel, stride, pads, term, act):
    """The first shape is large enough for the shape rule to pick the kernel by itself (no environment override); the others run
    with the threshold lowered to 1536 pixels, the tile configuration still chosen by the kernel's own cost estimate."""
    _say("resident at size", batch, c, h, w, outc, kernel)
    if batch * h * w < 40000 * stride[0] * stride[1]:
        resident_env(min_pixels=1536)
    _check(rt, 11, batch, c, h, w, outc, kernel, (1, 1), stride, pads, term, act, (0.0, 6.0))
