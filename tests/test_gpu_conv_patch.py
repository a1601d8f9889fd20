"""The small-tile convolution kernel (two-dimensional tiles of 32 output pixels whose input patch is quantised into LDS:
layers with few output pixels) against the oracle.

The kernel is chosen by the layer's shape; the environment variable NCNNHIP_PATCH (0: never, 1: whenever the layer fits)
is read at every launch, so the cases here force it and ask ncnnhip_conv_small_tile_selected that it was taken.
Input blobs: fp32 and fp16 (the layer's Quantize pass inside the kernel, src/layer/quantize.cpp:48-111) and int8.
Semantics: Convolution::forward_int8 (src/layer/convolution.cpp:383-508) per sample, batch as src/net.cpp:654-700."""
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


@pytest.fixture
def forced():
    saved = os.environ.get("NCNNHIP_PATCH")
    os.environ["NCNNHIP_PATCH"] = "1"
    yield
    if saved is None:
        os.environ.pop("NCNNHIP_PATCH", None)
    else:
        os.environ["NCNNHIP_PATCH"] = saved


def _say(*a):
    print("[case]", *a, flush=True)


def _selected(batch, c, h, w, outc, kernel, dilation, stride, pads, elemsize):
    from ncnn_amd.hip import ConvDesc, lib
    d = ConvDesc(w, h, c, batch, outc, kernel[0], kernel[1], dilation[0], dilation[1], stride[0], stride[1], pads[0], pads[1], pads[2], pads[3], 0.0, 1)
    return lib().ncnnhip_conv_small_tile_selected(C.byref(d), elemsize)


SHAPES = [
    # name, batch, c, h, w, outc, kernel, dilation, stride, pads
    ("single-layer configuration 3x3 64->64 @56 (8x4 tiles, 9 steps per wavefront)", 1, 64, 56, 56, 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    ("3x3 64->64 @20x13 batch 3 (ragged tiles right and below)", 3, 64, 13, 20, 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    ("1x1 256->128 @28 batch 2 (two channel tiles, 32x1 tiles)", 2, 256, 28, 28, 128, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    ("1x1/2 96->100 @28 (three steps per tap, channel tail)", 1, 96, 28, 28, 100, (1, 1), (1, 1), (2, 2), (0, 0, 0, 0)),
    ("3x3/2 20->48 @33 SAME_UPPER batch 2 (20 channels in 32: one step per tap)", 2, 20, 33, 33, 48, (3, 3), (1, 1), (2, 2), (-233, -233, -233, -233)),
    ("5x3 dilated 2 32->64 @40x30", 1, 32, 30, 40, 64, (5, 3), (2, 2), (1, 1), (4, 4, 2, 2)),
    ("3x3 128->128 @28 (18 steps per wavefront)", 1, 128, 28, 28, 128, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    ("3x3 256->256 @14 (36 steps per wavefront)", 1, 256, 14, 14, 256, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    ("3x3 64->40 @7 batch 5 (one tile and a sliver per image)", 5, 64, 7, 7, 40, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    ("2x2/2 64->64 @10 no padding", 2, 64, 10, 10, 64, (2, 2), (1, 1), (2, 2), (0, 0, 0, 0)),
    ("1x3 row kernel 64->24 on 6x40, uneven strides", 3, 64, 6, 40, 24, (3, 1), (1, 1), (2, 1), (1, 1, 0, 0)),
    ("3x1 column kernel 192->200 @8 (four channel tiles, the last mostly padding)", 2, 192, 8, 8, 200, (1, 3), (1, 1), (1, 1), (0, 0, 1, 1)),
]


@pytest.mark.parametrize("shape", SHAPES, ids=[s[0] for s in SHAPES])
@pytest.mark.parametrize("dtype", [np.float32, np.float16, np.int8], ids=["fp32", "fp16", "int8"])
def test_small_tile_kernel_matches_oracle(rt, forced, shape, dtype):
    """Every output bit for bit the oracle's quantise-then-convolve, fp32 and requantised int8 output, with inputs that
    meet float2int8's ties and its out-of-range rule."""
    name, batch, c, h, w, outc, kernel, dilation, stride, pads = shape
    _say("conv small tile", name, np.dtype(dtype).name)
    assert _selected(batch, c, h, w, outc, kernel, dilation, stride, pads, np.dtype(dtype).itemsize) == 1
    for term, act, ap in [(1, 1, (0.0, 0.0)), (102, 3, (0.0, 6.0)), (2, 2, (0.1, 0.0)), (101, 0, (0.0, 0.0))]:
        x, wq, b, ws, ins, tops = cases.conv_case(len(name) + batch + term, c, h, w, outc, kernel, 1, term, True, dtype == np.int8, batch=batch)
        if dtype != np.int8:
            x = x.astype(dtype).astype(F)  # the values the device will see
            edge = np.array([0.5, -0.5, 1.5, -2.5, 126.5, -126.5, 127.49, 300.0, -300.0, 0.49999997, -0.49999997], F) / ins[0]
            x.reshape(-1)[: edge.size] = edge.astype(dtype).astype(F)
            if dtype == np.float32:
                x.reshape(-1)[edge.size: edge.size + 4] = [np.inf, -np.inf, np.nan, 3e38]
        d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, 1, term, act, ap)
        want = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0]) for i in range(batch)])
        got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, ap,
                                    from_float=None if dtype == np.int8 else dtype)
        assert got.dtype == want.dtype and np.array_equal(got, want, equal_nan=True), (term, act)


@pytest.mark.parametrize("act,act_params,flip,bias", [(1, (0.0, 0.0), True, True), (3, (0.0, 6.0), False, False), (3, (0.3, -0.2), False, True),
                                                      (3, (float("-inf"), 0.5), False, True), (3, (-0.4, 0.4), True, True), (4, (0.0, 0.0), False, True),
                                                      (5, (0.0, 0.0), False, False), (6, (0.2, 0.5), False, True)])
def test_small_tile_kernel_activations(rt, forced, act, act_params, flip, bias):
    """The reference's activations taken literally (src/layer/fused_activation.h:25-74): negative output scales (flip),
    reversed and infinite clip bounds, the transcendental ones; pad channels of the blob stay zero behind all of them."""
    _say("conv small tile activations", act, act_params, flip, bias)
    c, h, w, outc = 64, 12, 11, 40
    x, wq, b, ws, ins, tops = cases.conv_case(act + 7, c, h, w, outc, (3, 3), 1, 102, bias, True, batch=2)
    if flip:
        tops = -tops
    d = oracle.make_desc((c, h, w), outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1 if bias else 0, 1, 102, act, act_params)
    got = rt.conv_channels_last(x, wq, b if bias else None, ws, ins, tops, outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 102, act, act_params)
    for i in range(2):
        want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], tops[0])
        if act in (4, 5):  # expf / tanhf / logf of the device's library: one step at most, where the value sits at a tie
            assert np.abs(got[i].astype(np.int32) - want).max() <= 1 and np.mean(got[i] != want) < 1e-3
        else:
            assert np.array_equal(got[i], want)
    dq = oracle.make_desc((c, h, w), outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1 if bias else 0, 1, 2, act, act_params)
    gotf = rt.conv_channels_last(x, wq, b if bias else None, ws, ins, None, outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 2, act, act_params)
    for i in range(2):
        wantf = oracle.convolution_int8(dq, x[i], wq, b, ws, ins[0], None)
        if act in (4, 5):
            before = oracle.convolution_int8(oracle.make_desc((c, h, w), outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1 if bias else 0, 1, 2, 0, (0, 0)),
                                             x[i], wq, b, ws, ins[0], None)
            assert np.all(np.abs(gotf[i].astype(np.float64) - wantf) <= 1e-5 * np.maximum(np.abs(wantf), np.abs(before)))
        else:
            assert np.array_equal(gotf[i], wantf)


@pytest.mark.parametrize("from_float", [None, np.float32], ids=["int8", "fp32"])
@pytest.mark.parametrize("c,h,w,outc,kernel,pads,relu", [(64, 14, 14, 256, (3, 3), (1, 1, 1, 1), True), (64, 20, 18, 40, (3, 3), (1, 1, 1, 1), False),
                                                           (128, 7, 7, 200, (1, 1), (0, 0, 0, 0), True)])
def test_small_tile_kernel_fused_tail(rt, forced, c, h, w, outc, kernel, pads, relu, from_float):
    """Residual, ReLU layer and the quantised copy for the next convolution in the epilogue, as the pipelined kernel has them."""
    _say("conv small tile fused tail", c, h, w, outc, kernel, relu, from_float)
    rng = np.random.default_rng(c + outc)
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc, c, h, w, outc, kernel, 1, 2, True, from_float is None, batch=3)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), (1, 1), pads, 0.0, 1, 1, 2, 0, (0.0, 0.0))
    conv = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None) for i in range(3)])
    res = rng.normal(0, 1, conv.shape).astype(F)
    want = (conv + res).astype(F)
    if relu:
        want = np.maximum(want, 0)
    next_scale = F(127) / np.abs(want).max()
    want_q = oracle.quantize(want.reshape(3 * outc, -1), [next_scale]).reshape(want.shape)
    got, got_q = rt.conv_channels_last(x, wq, b, ws, ins, None, outc, kernel, (1, 1), (1, 1), pads, 0.0, 1, 2, 0, (0.0, 0.0), residual=res,
                                       relu_after=relu, quantise_scale=next_scale, from_float=from_float)
    assert np.array_equal(got, want) and np.array_equal(got_q, want_q)


def test_small_tile_kernel_is_chosen_by_shape_and_refuses_what_does_not_fit(rt):
    saved = os.environ.pop("NCNNHIP_PATCH", None)
    try:
        one = ((1, 1), (1, 1))
        # the single-layer configuration from an fp32 blob: 49 tiles of 64 pixels -> taken
        assert _selected(1, 64, 56, 56, 64, (3, 3), *one, (1, 1, 1, 1), 4) == 1
        # the same layer at batch 16 fills the chip with 64-pixel tiles
        assert _selected(16, 64, 56, 56, 64, (3, 3), *one, (1, 1, 1, 1), 4) == 0
        os.environ["NCNNHIP_PATCH"] = "1"
        # 16 channels per pixel: a 32-byte step would straddle two taps; K beyond the registers; a patch beyond LDS
        assert _selected(1, 16, 30, 40, 64, (5, 3), (2, 2), (1, 1), (4, 4, 2, 2), 4) == 0
        assert _selected(1, 512, 7, 7, 512, (3, 3), *one, (1, 1, 1, 1), 1) == 0
        assert _selected(1, 1024, 80, 80, 64, (3, 3), (9, 9), (1, 1), (9, 9, 9, 9), 1) == 0
        os.environ["NCNNHIP_PATCH"] = "0"
        assert _selected(1, 64, 56, 56, 64, (3, 3), *one, (1, 1, 1, 1), 4) == 0
    finally:
        if saved is None:
            os.environ.pop("NCNNHIP_PATCH", None)
        else:
            os.environ["NCNNHIP_PATCH"] = saved
