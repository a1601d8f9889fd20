"""Device-resident (channels-last) blobs: layout round trips, the quantise pass, both convolution kernels writing
channels-last, and the fp32 layers between them -- each against the oracle or a scalar restatement of the
reference loop (pooling.cpp, eltwise.cpp, relu.cpp, softmax.cpp) on the same seeded inputs."""
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


def _say(*a):
    print("[case]", *a, flush=True)


@pytest.mark.parametrize("n,c,h,w", [(1, 3, 5, 7), (2, 16, 9, 9), (3, 70, 13, 11), (1, 130, 1, 1)])
@pytest.mark.parametrize("dtype", [np.float32, np.int8])
def test_layout_round_trip_and_zero_padding(rt, n, c, h, w, dtype):
    _say("layout", n, c, h, w, dtype)
    rng = np.random.default_rng(c * h)
    x = rng.integers(-127, 128, (n, c, h, w)).astype(dtype)
    buf = rt.to_channels_last(x)
    raw = buf.to_numpy(rt.stream)
    assert raw.shape == (n, h * w, (c + 15) // 16 * 16)
    assert np.array_equal(raw[:, :, :c], x.reshape(n, c, h * w).transpose(0, 2, 1))
    assert not raw[:, :, c:].any()
    assert np.array_equal(rt.from_channels_last(buf, n, c, h, w), x)


@pytest.mark.parametrize("c,per_channel", [(3, False), (24, True), (64, False), (100, True)])
def test_quantize_channels_last_matches_oracle(rt, c, per_channel):
    rng = np.random.default_rng(c)
    x = rng.uniform(-3, 3, (2, c, 6, 5)).astype(F)
    x.flat[::97] = np.array([0.5, -0.5, 126.5, -126.5, 127.49, 200, -200, 1.5], F)[np.arange(x.flat[::97].size) % 8]
    scales = rng.uniform(20, 60, c if per_channel else 1).astype(F)
    want = oracle.quantize(x.transpose(1, 0, 2, 3).reshape(c, -1), scales).reshape(c, 2, 6, 5).transpose(1, 0, 2, 3)
    q = rt.quantize_channels_last(rt.to_channels_last(x), c, scales)
    raw = q.to_numpy(rt.stream)
    assert not raw[:, :, c:].any()
    assert np.array_equal(rt.from_channels_last(q, 2, c, 6, 5), want)


CONV_CASES = [
    # c, h, w, outc, kernel, dilation, stride, pads
    (3, 9, 11, 4, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (5, 8, 7, 6, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (4, 12, 10, 8, (3, 2), (2, 1), (2, 1), (2, 1, 0, 1)),
    (2, 13, 13, 3, (5, 5), (1, 1), (2, 2), (-233, -233, -233, -233)),
    (16, 20, 20, 130, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (64, 14, 14, 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (96, 7, 7, 200, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (512, 7, 7, 72, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),   # K split over workgroups
    (32, 150, 150, 136, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),  # 128-row tiles with a ragged last tile
]


@pytest.mark.parametrize("shape", CONV_CASES)
@pytest.mark.parametrize("term,act,act_params,int8_in", [(2, 1, (0, 0), False), (102, 3, (0.0, 6.0), True), (101, 0, (0, 0), False)])
def test_convolution_channels_last_bit_exact(rt, shape, term, act, act_params, int8_in):
    c, h, w, outc, kernel, dilation, stride, pads = shape
    _say("conv channels-last", shape, term, act, int8_in)
    x, wq, b, ws, ins, tops = cases.conv_case(c * 10 + outc + term, c, h, w, outc, kernel, 1, term, True, int8_in)
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, 1, term, act, act_params)
    want = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0], None if tops is None else tops[0])
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, act_params)
    assert got.dtype == want.dtype and np.array_equal(got[0], want)


@pytest.mark.parametrize("act_params", [(-0.37, 0.41), (0.013, 0.02), (0.3, -0.2), (-1e30, 1e30), (float("-inf"), 0.5)])
@pytest.mark.parametrize("term,bias,flip", [(102, True, False), (101, False, False), (102, True, True), (2, False, False)])
def test_clip_is_the_reference_clip_whatever_its_bounds(rt, act_params, term, bias, flip):
    """The kernels fold a clip into the requantising clamp when that is provably the same (bounds in order, finite
    tables, output scales not negative) and take the literal compare-and-select path otherwise: both bounds active,
    bounds that are no integers in the output scale, reversed bounds, huge and infinite bounds, negative output scales
    (flip), no bias, fp32 output."""
    _say("clip variants", act_params, term, bias, flip)
    for group, c, outc, kernel, pads in [(1, 24, 40, (1, 1), (0, 0, 0, 0)), (1, 16, 16, (3, 3), (1, 1, 1, 1)), (48, 48, 48, (3, 3), (1, 1, 1, 1))]:
        x, wq, b, ws, ins, tops = cases.conv_case(7 + term, c, 12, 11, outc, kernel, group, term, bias, term > 100, by_group=group > 1, batch=2)
        if group > 1 and term in (2, 102):
            ws = np.full(c, ws[0], F)
        if tops is not None and flip:
            tops = tops.copy()
            tops[:] = -tops
        d = oracle.make_desc((c, 12, 11), outc, kernel, (1, 1), (1, 1), pads, 0.0, 1 if bias else 0, group, term, 3, act_params)
        got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, (1, 1), (1, 1), pads, 0.0, group, term, 3, act_params)
        for i in range(2):
            if group > 1:
                want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
            else:
                want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0])
            assert got.dtype == want.dtype and np.array_equal(got[i], want), (group, kernel)


@pytest.mark.parametrize("c,outc,act,act_params,flip,hw", [
    (16, 24, 3, (0.0, 6.0), False, 257),     # clip folded into the clamp; second 16-channel block half padding
    (40, 8, 0, (0.0, 0.0), False, 257),      # 48 bytes per pixel: the last lane row reads bytes the zero weights cancel
    (64, 100, 1, (0.0, 0.0), False, 257),    # the full K, ReLU, channel count not a multiple of 16
    (24, 32, 3, (-0.2, 0.3), True, 257),     # negative output scales: the literal clip
    (8, 16, 2, (0.1, 0.0), False, 257),      # leaky ReLU: the general activation path
    (16, 96, 3, (0.0, 6.0), False, 365),     # MobileNetV2's first expansion: six channel blocks, three per wavefront pair
    (32, 144, 3, (0.5, 4.0), False, 257),    # a clip with a positive lower bound; nine channel blocks over two wavefronts
    (24, 40, 3, (-1.0, 2.0), False, 257),    # a clip with a negative lower bound: folded, rounded the general way
])
def test_pointwise_small_k_kernel_matches_oracle(rt, c, outc, act, act_params, flip, hw):
    """1x1 layers with at most 64 input channels, int8 output and 2^16 pixels or more take a kernel of their own
    (MFMA fed weights-first, tables in LDS, lane-row transposes before the store; a workgroup owns whole pixel rows of the
    output): ragged pixel count, batch 2."""
    _say("pointwise small-K", c, outc, act, act_params, flip, hw)
    h = w = hw
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc, c, h, w, outc, (1, 1), 1, 102, True, True, batch=2)
    if flip:
        tops = -tops
    d = oracle.make_desc((c, h, w), outc, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), 0.0, 1, 1, 102, act, act_params)
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), 0.0, 1, 102, act, act_params)
    for i in range(2):
        want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], tops[0])
        assert got.dtype == want.dtype and np.array_equal(got[i], want)


def test_convolution_channels_last_batch_and_pad_value(rt):
    x, wq, b, ws, ins, tops = cases.conv_case(21, 20, 10, 9, 24, (3, 3), 1, 101, True, False, batch=3)
    d = oracle.make_desc((20, 10, 9), 24, (3, 3), pads=(1, 1, 1, 1), pad_value=-2.2, bias_term=1, int8_scale_term=101, activation_type=1)
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, 24, (3, 3), pads=(1, 1, 1, 1), pad_value=-2.2, term=101, act=1)
    for i in range(3):
        assert np.array_equal(got[i], oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], tops[0]))


@pytest.mark.parametrize("c,h,w,kernel,stride,dilation,pads", [
    (6, 9, 10, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)), (32, 56, 56, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (96, 28, 28, (3, 3), (2, 2), (1, 1), (1, 1, 1, 1)), (40, 15, 17, (5, 5), (1, 1), (2, 2), (-233, -233, -233, -233)),
    (144, 14, 14, (3, 3), (2, 2), (1, 1), (0, 1, 0, 1))])
@pytest.mark.parametrize("term,act,int8_in", [(1, 0, False), (101, 3, True), (102, 1, False), (2, 3, False)])
def test_depthwise_channels_last_bit_exact(rt, c, h, w, kernel, stride, dilation, pads, term, act, int8_in):
    _say("depthwise channels-last", c, h, w, kernel, stride, term, act, int8_in)
    by_group = term in (1, 101)
    x, wq, b, ws, ins, tops = cases.conv_case(c + term, c, h, w, c, kernel, c, term, True, int8_in, by_group=True, batch=2)
    if not by_group:
        ws = np.full(c, ws[0], F)
    d = oracle.make_desc((c, h, w), c, kernel, dilation, stride, pads, 0.0, 1, c, term, act, (0.0, 6.0))
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, c, kernel, dilation, stride, pads, 0.0, c, term, act, (0.0, 6.0))
    for i in range(2):
        want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
        assert got.dtype == want.dtype and np.array_equal(got[i], want)


# ---- fp32 layers between the int8 layers --------------------------------------------------------------------
def _pool_ref(x, kind, k, s, pt, pl, oh, ow, include_pad):
    """Scalar restatement of Pooling::forward on one [c][h][w] sample with the border already resolved
    (src/layer/pooling.cpp:150-330): windows anchored at (i*s - pad), taps outside the image are -FLT_MAX for max,
    skipped (count_include_pad=0) or zero (=1) for average; sums run ky-major in float32."""
    c, h, w = x.shape
    out = np.zeros((c, oh, ow), F)
    for q in range(c):
        for i in range(oh):
            for j in range(ow):
                vals = []
                for ky in range(k[1]):
                    for kx in range(k[0]):
                        y, xx = i * s[1] - pt + ky, j * s[0] - pl + kx
                        vals.append(x[q, y, xx] if 0 <= y < h and 0 <= xx < w else None)
                inside = [v for v in vals if v is not None]
                if kind == 0:
                    out[q, i, j] = max(inside) if inside else -np.finfo(F).max
                else:
                    acc = F(0)
                    for v in inside:
                        acc = F(acc + v)
                    out[q, i, j] = F(acc / F(len(vals) if include_pad else len(inside)))
    return out


@pytest.mark.parametrize("c,h,w,stride,pads,term,act", [
    (64, 113, 112, 1, (1, 1, 1, 1), 101, 3),    # four output rows per thread, 113 rows: the last group has one
    (128, 45, 64, 1, (1, 1, 1, 1), 101, 1),     # two output rows per thread, odd row count
    (128, 91, 128, 2, (1, 1, 1, 1), 101, 3),    # stride 2, four rows per thread, 46 rows
    (96, 50, 128, 2, (0, 1, 0, 1), 1, 0),       # stride 2, two rows per thread, fp32 output
])
def test_depthwise_several_output_rows_per_thread(rt, c, h, w, stride, pads, term, act):
    """The 3x3 depthwise kernel gives a thread 1, 2 or 4 output rows depending on how many threads that leaves; the
    small shapes above all take one row, these (batch 8) take two and four, with row counts that do not divide."""
    _say("depthwise rows per thread", c, h, w, stride, term, act)
    x, wq, b, ws, ins, tops = cases.conv_case(c + h, c, h, w, c, (3, 3), c, term, True, term > 100, by_group=True, batch=8)
    d = oracle.make_desc((c, h, w), c, (3, 3), (1, 1), (stride, stride), pads, 0.0, 1, c, term, act, (0.0, 6.0))
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, c, (3, 3), (1, 1), (stride, stride), pads, 0.0, c, term, act, (0.0, 6.0))
    for i in (0, 3, 7):
        want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
        assert got.dtype == want.dtype and np.array_equal(got[i], want)


@pytest.mark.parametrize("kind,k,s,pt,pl,include_pad", [(0, (3, 3), (2, 2), 0, 0, 0), (0, (3, 3), (2, 2), 1, 1, 0), (0, (2, 3), (1, 2), 0, 1, 0),
                                                         (1, (3, 3), (2, 2), 1, 1, 0), (1, (3, 3), (1, 1), 1, 1, 1), (1, (2, 2), (2, 2), 0, 0, 0)])
def test_pooling_matches_scalar_restatement(rt, kind, k, s, pt, pl, include_pad):
    rng = np.random.default_rng(kind * 10 + k[0])
    n, c, h, w = 2, 20, 11, 12
    x = rng.normal(0, 1, (n, c, h, w)).astype(F)
    # tail pads of "full" mode: the last partial window is kept
    oh = -(-(h + pt - k[1]) // s[1]) + 1
    ow = -(-(w + pl - k[0]) // s[0]) + 1
    got = rt.pooling(x, kind, k, s, (pt, pl), (oh, ow), count_include_pad=include_pad)
    for i in range(n):
        assert np.array_equal(got[i], _pool_ref(x[i], kind, k, s, pt, pl, oh, ow, include_pad))


@pytest.mark.parametrize("k,s,pt,pl", [((3, 3), (2, 2), 0, 0), ((3, 3), (2, 2), 1, 1), ((2, 3), (1, 2), 0, 1), ((3, 3), (2, 2), 2, 2)])
def test_int8_max_pooling_is_the_quantised_fp32_max_pooling(rt, k, s, pt, pl):
    """Quantize is monotonic while value * scale stays inside the int32 range (beyond it the reference's float2int8
    wraps to -127): pooling the quantised blob == quantising the pooled blob (the oracle's float2int8)."""
    rng = np.random.default_rng(k[0] * 7 + pt)
    n, c, h, w = 2, 37, 11, 12
    x = rng.normal(0, 1, (n, c, h, w)).astype(F)
    x[0, 0, 0, 0] = 1e6   # clamps to 127
    x[0, 1, 0, 0] = -1e6  # clamps to -127
    scale = F(50.0)
    oh = -(-(h + pt - k[1]) // s[1]) + 1
    ow = -(-(w + pl - k[0]) // s[0]) + 1
    xq = oracle.quantize(x.reshape(1, -1), scale).reshape(x.shape)
    got = rt.maxpool_int8(xq, k, s, (pt, pl), (oh, ow))
    for i in range(n):
        pooled = _pool_ref(x[i], 0, k, s, pt, pl, oh, ow, 0)
        assert np.array_equal(got[i], oracle.quantize(pooled.reshape(1, -1), scale).reshape(pooled.shape))


@pytest.mark.parametrize("kind", [0, 1])
def test_global_pooling(rt, kind):
    rng = np.random.default_rng(kind)
    x = rng.normal(0, 1, (3, 70, 7, 7)).astype(F)
    got = rt.pooling(x, kind, None, None, None, None, global_pooling=True)
    flat = x.reshape(3, 70, 49)
    want = flat.max(axis=2) if kind == 0 else (np.cumsum(flat, axis=2, dtype=F)[..., -1] / F(49)).astype(F)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("kind", [0, 1])
def test_global_pooling_quantised_is_quantize_of_the_pooled_vector(rt, kind):
    """Global pooling that hands an int8 InnerProduct its input: float2int8(pool(x) * scale), the pooled value computed
    as the fp32 entry point computes it (sequential sum, one division), quantised as Quantize would (the oracle)."""
    rng = np.random.default_rng(10 + kind)
    x = rng.normal(0, 1, (3, 70, 7, 7)).astype(F)
    x[0, 0] = 1e9       # beyond the clamp
    x[1, 3] = -0.0131   # a small negative mean
    scale = F(37.3)
    flat = x.reshape(3, 70, 49)
    pooled = flat.max(axis=2) if kind == 0 else (np.cumsum(flat, axis=2, dtype=F)[..., -1] / F(49)).astype(F)
    want = oracle.quantize(pooled.reshape(1, -1), np.array([scale], F)).reshape(3, 70)
    got = rt.global_pooling_quantised(x, kind, scale)
    assert got.dtype == np.int8 and np.array_equal(got, want)


def test_relu_and_leaky_relu(rt):
    rng = np.random.default_rng(3)
    x = rng.normal(0, 1, 4096).astype(F)
    assert np.array_equal(rt.relu(x), np.maximum(x, 0))
    assert np.array_equal(rt.relu(x, 0.1), np.where(x < 0, (x * F(0.1)).astype(F), x))
    q = rng.integers(-127, 128, 1000).astype(np.int8)
    assert np.array_equal(rt.relu(q), np.maximum(q, 0))


def test_eltwise_all_modes(rt):
    rng = np.random.default_rng(4)
    a, b, c = [rng.normal(0, 1, 2048).astype(F) for _ in range(3)]
    assert np.array_equal(rt.eltwise([a, b], 1), a + b)
    assert np.array_equal(rt.eltwise([a, b, c], 1), (a + b) + c)
    assert np.array_equal(rt.eltwise([a, b, c], 0), (a * b) * c)
    assert np.array_equal(rt.eltwise([a, b, c], 2), np.maximum(np.maximum(a, b), c))
    co = [F(0.5), F(-1.25), F(3.0)]
    want = ((a * co[0]).astype(F) + (b * co[1]).astype(F)).astype(F) + (c * co[2]).astype(F)
    assert np.array_equal(rt.eltwise([a, b, c], 1, co), want.astype(F))


def test_softmax_within_1e_6(rt):
    # the device expf and a tree reduction replace libm expf and the sequential sum: tolerance, not bit parity
    rng = np.random.default_rng(5)
    x = rng.normal(0, 3, (4, 1000)).astype(F)
    got = rt.softmax(x)
    e = np.exp(x.astype(np.float64) - x.max(axis=1, keepdims=True))
    want = e / e.sum(axis=1, keepdims=True)
    assert np.allclose(got, want, rtol=1e-5, atol=1e-9)
    assert np.allclose(got.sum(axis=1), 1.0, atol=1e-5)


@pytest.mark.parametrize("c,h,w,outc,kernel,pads", [(64, 14, 14, 256, (1, 1), (0, 0, 0, 0)), (24, 20, 18, 40, (3, 3), (1, 1, 1, 1)),
                                                     (512, 7, 7, 200, (1, 1), (0, 0, 0, 0)), (2048, 7, 7, 48, (1, 1), (0, 0, 0, 0))])
@pytest.mark.parametrize("relu", [False, True])
def test_convolution_with_residual_relu_and_quantised_copy_in_the_epilogue(rt, c, h, w, outc, kernel, pads, relu):
    """conv -> Eltwise sum -> ReLU -> Quantize folded into one kernel equals the four layers run one by one."""
    _say("fused epilogue", c, h, w, outc, kernel, relu)
    rng = np.random.default_rng(c + outc)
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc, c, h, w, outc, kernel, 1, 2, True, False, batch=2)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), (1, 1), pads, 0.0, 1, 1, 2, 0, (0.0, 0.0))
    conv = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None) for i in range(2)])
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


# ---- narrow-input ("stem") convolution: 4-byte pixels with a physical border, 4 neighbouring pixels per K chunk ---------

@pytest.mark.parametrize("c,h,w,outc,kernel,stride,pads,dil_h,term,act", [
    (3, 32, 32, 64, (7, 7), (2, 2), (3, 3, 3, 3), 1, 2, 1),      # the ResNet stem, small
    (3, 33, 29, 32, (3, 3), (2, 2), (1, 1, 1, 1), 1, 101, 3),    # MobileNetV2's first layer: requantised output, clip
    (1, 17, 40, 20, (5, 3), (1, 1), (0, 4, 2, 0), 1, 1, 0),      # one channel, uneven pads, stride 1 (4-byte aligned gathers)
    (4, 20, 21, 70, (1, 1), (1, 2), (0, 0, 0, 0), 1, 2, 2),      # 1x1, leaky
    (2, 25, 25, 16, (9, 2), (3, 1), (-233, -233, -233, -233), 2, 2, 1),  # SAME pads, two groups of taps + a partial one, dilated rows
    (3, 16, 16, 130, (4, 4), (4, 4), (0, 0, 0, 0), 1, 102, 0),   # patch embedding, more output channels than one tile
])
def test_stem_convolution_matches_oracle(rt, c, h, w, outc, kernel, stride, pads, dil_h, term, act):
    x, wq, b, ws, ins, tops = cases.conv_case(c * 1000 + h + outc, c, h, w, outc, kernel, 1, term, True)
    act_params = {0: (0.0, 0.0), 1: (0.0, 0.0), 2: (0.1, 0.0), 3: (0.0, 3.0)}[act]
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, (1, dil_h), stride, pads, 0.0, 1, term, act, act_params, stem=True)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, dil_h), stride, pads, 0.0, 1, 1, term, act, act_params)
    want = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0], None if tops is None else tops[0])
    assert got.dtype == want.dtype and np.array_equal(got[0], want)


@pytest.mark.parametrize("batch,c,h,w,outc,kernel,stride,pads,term,act,act_params,flip", [
    (1, 3, 514, 514, 32, (3, 3), (2, 2), (1, 1, 1, 1), 101, 3, (0.0, 6.0), False),     # MobileNetV2's first layer: one K step, two channel blocks
    (1, 3, 520, 518, 64, (7, 7), (2, 2), (3, 3, 3, 3), 102, 1, (0.0, 0.0), False),     # ResNet-50's at the same size: 14 chunks, stays on the pipelined kernel
    (3, 3, 300, 302, 24, (3, 3), (2, 2), (-233, -233, -233, -233), 101, 0, (0.0, 0.0), False),  # pixel blocks that cross rows and images; 24 channels in 32
    (2, 4, 186, 190, 40, (3, 3), (1, 1), (1, 1, 1, 1), 102, 3, (-1.0, 2.0), False),    # stride 1: chunks on 4-byte boundaries; a negative clip bound
    (1, 1, 260, 259, 16, (4, 4), (1, 1), (0, 0, 0, 0), 101, 1, (0.0, 0.0), True),      # all four rows of a step in use; negative output scales
    (2, 3, 372, 370, 100, (4, 4), (2, 2), (1, 1, 1, 1), 102, 2, (0.1, 0.0), False),    # seven channel blocks, the last partly padding
])
def test_stem_convolution_on_the_pointwise_kernel(rt, batch, c, h, w, outc, kernel, stride, pads, term, act, act_params, flip):
    """A first layer of up to 4 x 4 taps with 65536 output pixels and more and an int8 output runs on the pointwise kernel's
    narrow-input form (operands straight from the bordered image): bit for bit the oracle's, as is the 7 x 7 layer of the
    same size beside it."""
    _say("stem on the pointwise kernel", batch, c, h, w, outc, kernel, stride, term, act)
    x, wq, b, ws, ins, tops = cases.conv_case(c * 100 + outc + kernel[0], c, h, w, outc, kernel, 1, term, True, False, batch=batch)
    if flip:
        tops = -tops
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), stride, pads, 0.0, 1, 1, term, act, act_params)
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, (1, 1), stride, pads, 0.0, 1, term, act, act_params, stem=True)
    assert got.shape[2] * got.shape[3] * batch >= 65536
    for i in range(batch):
        want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], tops[0])
        assert got.dtype == want.dtype and np.array_equal(got[i], want), "sample %d" % i


def test_stem_convolution_of_a_million_output_pixels(rt):
    """From 2^20 output pixels up the narrow-input layer runs on 128-pixel tiles of the pipelined kernel (fp32 output here, so
    the pointwise form does not take it): bit for bit the oracle's, batch of two, a last tile that is partly empty."""
    c, h, w, outc, kernel = 3, 1450, 1454, 16, (3, 3)
    x, wq, b, ws, ins, tops = cases.conv_case(123, c, h, w, outc, kernel, 1, 2, True, False, batch=2)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), (2, 2), (1, 1, 1, 1), 0.0, 1, 1, 2, 1)
    got = rt.conv_channels_last(x, wq, b, ws, ins, None, outc, kernel, (1, 1), (2, 2), (1, 1, 1, 1), 0.0, 1, 2, 1, (0.0, 0.0), stem=True)
    assert got.shape[0] * got.shape[2] * got.shape[3] >= (1 << 20)
    for i in range(2):
        assert np.array_equal(got[i], oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None))


def test_stem_convolution_batch_int8_input_and_fused_tail(rt):
    """Batch of 3, an int8 input blob (already quantised upstream), and the fused tail (residual, ReLU, quantised copy)."""
    c, h, w, outc, kernel = 3, 18, 22, 48, (3, 3)
    x, wq, b, ws, ins, tops = cases.conv_case(77, c, h, w, outc, kernel, 1, 2, True, False, batch=3)
    rng = np.random.default_rng(78)
    xq = oracle.quantize(x.reshape(3 * c, -1), ins[:1]).reshape(x.shape)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 1, 2, 1)
    plain = rt.conv_channels_last(xq, wq, b, ws, ins, None, outc, kernel, pads=(1, 1, 1, 1), term=2, act=1, stem=True)
    res = rng.normal(0, 1, plain.shape).astype(F)
    got, q8 = rt.conv_channels_last(x, wq, b, ws, ins, None, outc, kernel, pads=(1, 1, 1, 1), term=2, act=1, residual=res, relu_after=True,
                                    quantise_scale=21.5, stem=True)
    for i in range(3):
        want = oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None)
        assert np.array_equal(plain[i], want)
        fused = np.maximum((want + res[i]).astype(F), 0)
        assert np.array_equal(got[i], fused)
        assert np.array_equal(q8[i], oracle.quantize(fused.reshape(1, -1), F(21.5)).reshape(fused.shape))
