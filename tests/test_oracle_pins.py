"""Pins the C oracle (oracle/ncnn_int8_oracle.c) without running ncnn.

ncnn's own tests for this path are differential (naive vs optimised, no literal vectors), so the
oracle is pinned by what the mathematics fixes: hand-listed rounding cases, an independent numpy
int64/float32 statement (tests/npref.py), brute force on tiny inputs, and structural identities.
"""
import itertools

import numpy as np
import pytest

import cases
import npref
from oracle import oracle

F = np.float32


# ----------------------------------------------------------------------------- float2int8
def test_float2int8_special_cases():
    below_half = np.nextafter(F(0.5), F(0))  # 0.49999997: trunc(v+0.5) implementations give 1 here
    cases = [
        (0.0, 0), (-0.0, 0), (0.5, 1), (-0.5, -1), (1.5, 2), (-1.5, -2), (2.5, 3), (-2.5, -3),
        (float(below_half), 0), (-float(below_half), 0), (0.4999, 0), (126.5, 127), (-126.5, -127),
        (126.49999, 126), (127.49, 127), (127.5, 127), (-127.5, -127), (128.0, 127), (-128.0, -127),
        (200.0, 127), (-200.0, -127), (1e9, 127), (-1e9, -127), (3e9, -127), (-3e9, -127),
        (float("inf"), -127), (float("-inf"), -127), (float("nan"), -127),
    ]
    for v, want in cases:
        assert int(oracle.float2int8(F(v))) == want, v


def test_float2int8_matches_float64_rounding_on_grid():
    rng = np.random.default_rng(1)
    v = np.concatenate([rng.uniform(-140, 140, 4000), np.arange(-130, 130) + 0.5, np.arange(-130, 130) - 0.5]).astype(F)
    v = np.concatenate([v, np.nextafter(v, F(np.inf)), np.nextafter(v, F(-np.inf))])
    got = oracle.quantize(v[None, :], [1.0])[0]
    assert np.array_equal(got, npref.float2int8(v))
    assert got.min() >= -127 and got.max() <= 127


def test_float2int8_out_of_range_is_what_the_x86_conversion_gives():
    """`static_cast<int>(round(v))` (src/layer/convolution.cpp:375-381) is undefined in C++ for NaN and |v| >= 2^31; the
    reference's x86 builds get cvttss2si's "integer indefinite" 0x80000000, which the clamp turns into -127.  numpy's
    float32 -> int32 cast executes that very instruction on an x86 host, so the pin is the hardware's own answer."""
    import platform
    if platform.machine() not in ("x86_64", "AMD64"):
        pytest.skip("pins the x86 conversion")
    v = np.array([np.nan, np.inf, -np.inf, 3e9, -3e9, 2147483648.0, -2147483904.0, 1e30, -1e30], F)
    with np.errstate(invalid="ignore"):
        as_int = np.round(v).astype(np.int32)
    assert np.all(as_int == np.iinfo(np.int32).min)
    want = np.clip(as_int, -127, 127).astype(np.int8)
    assert np.array_equal(oracle.quantize(v[None, :], [1.0])[0], want)


def test_activation_closed_forms():
    assert oracle.activation(-1.0, 1) == 0.0 and oracle.activation(2.0, 1) == 2.0
    assert oracle.activation(-2.0, 2, (0.25,)) == -0.5
    assert oracle.activation(7.0, 3, (0.0, 6.0)) == 6.0 and oracle.activation(-1.0, 3, (0.0, 6.0)) == 0.0
    a, b = 1.0 / 6.0, 0.5  # hardswish
    assert oracle.activation(-4.0, 6, (a, b)) == 0.0
    assert oracle.activation(5.0, 6, (a, b)) == 5.0
    x = F(1.25)
    assert oracle.activation(float(x), 6, (a, b)) == float(x * (x * F(a) + F(b)))
    rng = np.random.default_rng(0)
    v = rng.uniform(-8, 8, 200).astype(F)
    for t, p in ((0, (0, 0)), (1, (0, 0)), (2, (0.1, 0)), (3, (0.0, 6.0)), (6, (a, b))):
        want = npref.activation(v, t, p)
        got = np.array([oracle.activation(float(z), t, p) for z in v], F)
        assert np.array_equal(got, want), t


def test_sigmoid_and_mish_against_float64_closed_forms():
    """Activation types 4 and 5 (src/layer/fused_activation.h:34-45) call the host's expf / logf / tanhf, so the pin is a
    tolerance, not a bit pattern: sigmoid against 1 / (1 + exp(-v)) in float64 to 4 units in the last place of a value
    in (0, 1] (plus 2e-44 where the result is denormal); mish against v * tanh(log1p(exp(v))) in float64 to 1e-6 * |v| (the fp32 formula rounds exp(v) + 1, which
    costs up to 6e-8 in the logarithm whatever its size, and the product scales that by |v|).  Known answers and the
    clamp of the sigmoid's argument at +-88.376 are checked exactly.  A dropped term, a flipped sign or the clamp on the
    wrong side fails these."""
    sig = lambda z: oracle.activation(float(z), 4)
    mish = lambda z: oracle.activation(float(z), 5)
    assert sig(0.0) == 0.5 and mish(0.0) == 0.0
    assert sig(100.0) == sig(88.3762626647949) and sig(-100.0) == sig(-88.3762626647949)
    assert sig(100.0) == 1.0 and 0.0 < sig(-100.0) < 1e-37
    assert abs(mish(1.0) - 0.8650983882673103) < 2e-7      # v * tanh(ln(1 + e)), 16 digits from the closed form
    assert abs(mish(-1.0) + 0.30340146137410895) < 2e-7
    assert mish(50.0) == 50.0 and mish(1000.0) == 1000.0    # tanh saturates; exp overflows to inf, log(inf) = inf, tanh = 1
    assert abs(mish(-20.0) + 20.0 * np.exp(-20.0)) < 20 * 1.3e-7
    rng = np.random.default_rng(45)
    v = np.concatenate([rng.uniform(-12, 12, 4000), rng.uniform(-90, 90, 1000), rng.uniform(-0.01, 0.01, 200)]).astype(F)
    v64 = v.astype(np.float64)
    s_got = np.array([sig(z) for z in v], np.float64)
    s_want = 1.0 / (1.0 + np.exp(-np.clip(v64, -88.3762626647949, 88.3762626647949)))
    assert np.all(np.abs(s_got - s_want) <= 4 * np.spacing(s_want.astype(F)).astype(np.float64) + 2e-44)  # (+ a few denormal steps at the clamp)
    assert np.all((s_got > 0) & (s_got <= 1))
    # sigmoid(-v) = 1 - sigmoid(v)
    s_neg = np.array([sig(-z) for z in v], np.float64)
    assert np.all(np.abs(s_got + s_neg - 1.0) <= 3e-7)
    m_got = np.array([mish(z) for z in v], np.float64)
    with np.errstate(over="ignore"):
        m_want = v64 * np.tanh(np.where(v64 > 40, v64, np.log1p(np.exp(np.minimum(v64, 40)))))
    assert np.all(np.abs(m_got - m_want) <= 1e-6 * np.abs(v64) + 1e-12), np.abs(m_got - m_want).max()
    # mish has one minimum, -0.308841 near v = -1.1924
    assert m_got.min() > -0.30885 and abs(min(mish(z) for z in np.arange(-1.3, -1.1, 0.001)) + 0.308841) < 1e-5


# ----------------------------------------------------------------------------- quantize
def test_quantize_per_row_and_single_scale():
    rng = np.random.default_rng(2)
    x = rng.uniform(-3, 3, (5, 37)).astype(F)
    s = rng.uniform(10, 60, 5).astype(F)
    assert np.array_equal(oracle.quantize(x, s), npref.float2int8(x * s[:, None]))
    assert np.array_equal(oracle.quantize(x, s[:1]), npref.float2int8(x * s[0]))


# ----------------------------------------------------------------------------- convolution
def _conv_case(rng, c, h, w, outc, kernel, dilation, stride, pads, group, term, act, act_params, bias, int8_in,
               by_group, pad_value=0.0):
    cg = c // group
    kw, kh = kernel
    x = rng.uniform(-1, 1, (c, h, w)).astype(F)
    wt = rng.integers(-127, 128, (outc, cg, kh, kw)).astype(np.int8)
    nws = group if by_group else outc
    w_scales = rng.uniform(20, 200, nws).astype(F)
    nas = group if by_group else 1
    in_scales = np.full(nas, F(127) / np.abs(x).max(), F)
    top_scales = np.full(nas, F(rng.uniform(5, 40)), F)
    b = rng.uniform(-0.1, 0.1, outc).astype(F) if bias else None
    if int8_in:
        x = npref.float2int8(x * in_scales[0])
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, pad_value, int(bias), group, term, act, act_params)
    return d, x, wt, b, w_scales, in_scales, top_scales


CONV_SHAPES = [
    # c, h, w, outc, kernel(w,h), dilation, stride, pads(l,r,t,b)
    (3, 9, 11, 4, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (5, 8, 7, 6, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (4, 12, 10, 8, (3, 2), (2, 1), (2, 1), (2, 1, 0, 1)),
    (2, 13, 13, 3, (5, 5), (1, 1), (2, 2), (-233, -233, -233, -233)),
    (2, 10, 9, 3, (4, 3), (1, 2), (3, 2), (-234, -234, -234, -234)),
    (7, 6, 6, 5, (3, 3), (1, 1), (1, 1), (0, 0, 0, 0)),
]


@pytest.mark.parametrize("shape", CONV_SHAPES)
@pytest.mark.parametrize("term,act,act_params,bias,int8_in", [
    (1, 0, (0, 0), False, False), (2, 1, (0, 0), True, False), (101, 3, (0.0, 6.0), True, True),
    (102, 2, (0.1, 0), True, False), (1, 6, (1 / 6.0, 0.5), True, True)])
def test_convolution_matches_numpy(shape, term, act, act_params, bias, int8_in):
    rng = np.random.default_rng(hash((shape, term, act)) % (2 ** 32))
    c, h, w, outc, kernel, dilation, stride, pads = shape
    d, x, wt, b, ws, ins, tops = _conv_case(rng, c, h, w, outc, kernel, dilation, stride, pads, 1, term, act, act_params,
                                           bias, int8_in, False)
    got, gacc = oracle.convolution_int8(d, x, wt, b, ws, ins[0], tops[0], want_acc=True)
    want, wacc = npref.conv_family(x, wt, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act,
                                   act_params, False)
    assert np.array_equal(gacc, wacc)
    assert got.dtype == want.dtype and np.array_equal(got, want)


def test_convolution_brute_force_tiny():
    # literal definition, python loops, no shared code with either implementation
    rng = np.random.default_rng(5)
    c, h, w, outc = 2, 4, 5, 3
    xq = rng.integers(-127, 128, (c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (outc, c, 3, 3)).astype(np.int8)
    d = oracle.make_desc((c, h, w), outc, (3, 3), pads=(1, 1, 1, 1), int8_scale_term=1)
    _, acc = oracle.convolution_int8(d, xq, wt, None, np.ones(outc, F), 1.0, want_acc=True)
    for p, i, j in itertools.product(range(outc), range(h), range(w)):
        s = 0
        for q, ky, kx in itertools.product(range(c), range(3), range(3)):
            y, x_ = i + ky - 1, j + kx - 1
            if 0 <= y < h and 0 <= x_ < w:
                s += int(xq[q, y, x_]) * int(wt[p, q, ky, kx])
        assert acc[p, i, j] == s


def test_convolution_nonzero_pad_value_is_cast_to_int8_after_quantisation():
    rng = np.random.default_rng(6)
    d, x, wt, b, ws, ins, tops = _conv_case(rng, 3, 6, 6, 4, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 1, 1, 0, (0, 0), False,
                                           False, False, pad_value=3.7)
    got, acc = oracle.convolution_int8(d, x, wt, b, ws, ins[0], want_acc=True)
    want, wacc = npref.conv_family(x, wt, b, ws, ins, tops, 4, (3, 3), pads=(1, 1, 1, 1), pad_value=3.7)
    assert np.array_equal(acc, wacc) and np.array_equal(got, want)
    # border byte is 3 (C cast), not quantize(3.7*scale)
    assert acc[0, 0, 0] != npref.conv_family(x, wt, b, ws, ins, tops, 4, (3, 3), pads=(1, 1, 1, 1), pad_value=0.0)[1][0, 0, 0]


def test_zero_weight_scale_gives_activation_of_bias():
    rng = np.random.default_rng(7)
    d, x, wt, b, ws, ins, tops = _conv_case(rng, 3, 5, 5, 4, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 1, 1, 1, (0, 0), True,
                                           False, False)
    ws[2] = 0
    got = oracle.convolution_int8(d, x, wt, b, ws, ins[0])
    assert np.all(got[2] == max(b[2], 0))


def test_1x1_convolution_equals_gemm_rows():
    rng = np.random.default_rng(8)
    c, h, w, outc = 16, 5, 7, 6
    xq = rng.integers(-127, 128, (c, h, w)).astype(np.int8)
    wt = rng.integers(-127, 128, (outc, c, 1, 1)).astype(np.int8)
    d = oracle.make_desc((c, h, w), outc, (1, 1))
    _, acc = oracle.convolution_int8(d, xq, wt, None, np.ones(outc, F), 1.0, want_acc=True)
    _, gacc = oracle.gemm_int8(wt.reshape(outc, c), xq.reshape(c, h * w).T.copy(), np.ones(outc, F), [1.0], want_acc=True)
    assert np.array_equal(acc.reshape(outc, h * w), gacc)


# ----------------------------------------------------------------------------- depthwise / group
@pytest.mark.parametrize("c,outc,group", [(6, 6, 6), (8, 8, 8), (6, 12, 3), (8, 4, 2), (4, 4, 1)])
@pytest.mark.parametrize("term,act,act_params,stride,int8_in", [
    (1, 0, (0, 0), (1, 1), False), (101, 3, (0.0, 6.0), (2, 2), True), (102, 1, (0, 0), (1, 1), False),
    (2, 3, (0.0, 6.0), (2, 2), False)])
def test_depthwise_and_group_match_numpy(c, outc, group, term, act, act_params, stride, int8_in):
    rng = np.random.default_rng(hash((c, outc, group, term)) % (2 ** 32))
    d, x, wt, b, ws, ins, tops = _conv_case(rng, c, 9, 10, outc, (3, 3), (1, 1), stride, (1, 1, 1, 1), group, term, act,
                                           act_params, True, int8_in, True)
    if term in (2, 102):
        ws[:] = ws[0]  # the layer broadcasts a single weight scale to every group
    got, gacc = oracle.convolutiondepthwise_int8(d, x, wt, b, ws, ins, tops, want_acc=True)
    want, wacc = npref.conv_family(x, wt, b, ws, ins, tops, outc, (3, 3), (1, 1), stride, (1, 1, 1, 1), 0.0, group, term,
                                   act, act_params, True)
    assert np.array_equal(gacc, wacc)
    assert got.dtype == want.dtype and np.array_equal(got, want)


def test_depthwise_equals_group_conv_with_group_equal_channels_and_group1_equals_conv():
    rng = np.random.default_rng(9)
    d, x, wt, b, ws, ins, tops = _conv_case(rng, 4, 7, 7, 8, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 1, 1, 1, (0, 0), True,
                                           True, True)
    # group == 1: depthwise layer arithmetic with one scale per group must equal Convolution with that scale everywhere
    got_dw = oracle.convolutiondepthwise_int8(d, x, wt, b, ws[:1], ins[:1], None)
    got_cv = oracle.convolution_int8(d, x, wt, b, np.full(8, ws[0], F), ins[0])
    assert np.array_equal(got_dw, got_cv)


def test_invalid_group_is_rejected_with_minus_100():
    rng = np.random.default_rng(10)
    d, x, wt, b, ws, ins, tops = _conv_case(rng, 6, 5, 5, 6, (3, 3), (1, 1), (1, 1), (0, 0, 0, 0), 1, 1, 0, (0, 0), False,
                                           True, True)
    d.group = 4
    with pytest.raises(RuntimeError, match="-100"):
        oracle.convolutiondepthwise_int8(d, x, wt, b, np.ones(4, F), np.ones(4, F), None)


@pytest.mark.parametrize("mode", [-233, -234])
@pytest.mark.parametrize("h,w,kernel,stride,resolved_upper", [
    (20, 37, (3, 1), (3, 3), (0, -1, 1, 1)),   # hpad = 1 + 18 - 20 = -1, wpad = 3 + 36 - 37 = 2
    (21, 37, (3, 1), (3, 3), (-1, -1, 1, 1)),  # hpad = -2: a negative border on both sides
    (10, 12, (1, 3), (2, 2), (0, 1, 0, -1)),   # the same across: wpad = 1 + 10 - 12 = -1, hpad = 3 + 8 - 10 = 1
])
def test_same_padding_with_a_negative_border_is_refused_by_oracle_and_library(mode, h, w, kernel, stride, resolved_upper):
    """src/layer/convolution.cpp:328-372 pads when wpad > 0 OR hpad > 0, with both values as they come: a kernel extent
    below the stride in one dimension gives a negative border there, and src/layer/padding.cpp:62-87 then copies all
    source rows into a smaller blob.  The reference has no defined result; the oracle returns -1, the library an error
    from the one call every entry point sizes its output with.  SAME layers whose two values are both <= 0 get no
    border at all and stay accepted."""
    import ctypes as C
    from ncnn_amd.hip import ConvDesc, lib
    rng = np.random.default_rng(h + w)
    d, x, wt, b, ws, ins, tops = _conv_case(rng, 8, h, w, 4, kernel, (1, 1), stride, (mode,) * 4, 1, 1, 0, (0, 0), False, True, False)
    t, bo, l, r = oracle.resolve_padding(d)
    if mode == -233:
        assert (t, bo, l, r) == resolved_upper
    assert min(t, bo, l, r) < 0 and max(t, bo, l, r) > 0
    with pytest.raises(RuntimeError, match="-1"):
        oracle.convolution_int8(d, x, wt, b, ws, ins[0], None)
    cd = ConvDesc(w, h, 8, 1, 4, kernel[0], kernel[1], 1, 1, stride[0], stride[1], mode, mode, mode, mode, 0.0, 1)
    ow, oh = C.c_int(), C.c_int()
    assert lib().ncnnhip_conv_out_shape(C.byref(cd), C.byref(ow), C.byref(oh)) == -1
    assert b"negative border" in lib().ncnnhip_last_error()
    assert lib().ncnnhip_conv_from_float_supported(C.byref(cd)) == 0
    # 1 x 1 at stride 2: both values are <= 0, no border is made, the layer runs
    d1, x1, w1, b1, ws1, ins1, _ = _conv_case(rng, 8, h, w, 4, (1, 1), (1, 1), (2, 2), (mode,) * 4, 1, 1, 0, (0, 0), False, True, False)
    assert oracle.resolve_padding(d1) == (0, 0, 0, 0)
    assert oracle.convolution_int8(d1, x1, w1, b1, ws1, ins1[0], None).shape == (4, (h - 1) // 2 + 1, (w - 1) // 2 + 1)
    cd1 = ConvDesc(w, h, 8, 1, 4, 1, 1, 1, 1, 2, 2, mode, mode, mode, mode, 0.0, 1)
    assert lib().ncnnhip_conv_out_shape(C.byref(cd1), C.byref(ow), C.byref(oh)) == 0 and (oh.value, ow.value) == ((h - 1) // 2 + 1, (w - 1) // 2 + 1)


# ----------------------------------------------------------------------------- inner product
@pytest.mark.parametrize("rows,num_input,num_output,act,bias,int8_in", [
    (1, 64, 10, 0, False, False), (1, 2048, 100, 1, True, False), (5, 33, 7, 3, True, False), (3, 16, 4, 0, True, True)])
def test_innerproduct_matches_numpy(rows, num_input, num_output, act, bias, int8_in):
    rng = np.random.default_rng(rows * 1000 + num_input)
    x = rng.uniform(-1, 1, (rows, num_input)).astype(F)
    in_scale = F(127) / np.abs(x).max()
    wt = rng.integers(-127, 128, (num_output, num_input)).astype(np.int8)
    ws = rng.uniform(10, 20, num_output).astype(F)
    ws[0] = 0 if num_output > 4 else ws[0]
    b = rng.uniform(-1, 1, num_output).astype(F) if bias else None
    if int8_in:
        x = npref.float2int8(x * in_scale)
    got, gacc = oracle.innerproduct_int8(x, wt, b, ws, in_scale, act, (0.0, 6.0), want_acc=True)
    want, wacc = npref.innerproduct(x, wt, b, ws, in_scale, act, (0.0, 6.0))
    assert np.array_equal(gacc, wacc) and np.array_equal(got, want)


# ----------------------------------------------------------------------------- gemm int8
def test_gemm_quantize_rows_matches_numpy_and_zero_row_scale_is_one():
    rng = np.random.default_rng(11)
    a = rng.normal(0, 1, (9, 77)).astype(F)
    a[4] = 0
    aq, s = oracle.gemm_quantize_rows(a)
    wq, wsc = npref.gemm_quantize_rows(a)
    assert np.array_equal(s, wsc) and np.array_equal(aq, wq)
    assert s[4] == 1.0 and not aq[4].any()
    assert np.abs(aq).max(axis=1)[np.arange(9) != 4].min() == 127  # absmax element maps to +-127


def test_gemm_quantize_tensor():
    rng = np.random.default_rng(12)
    b = rng.normal(0, 0.02, (6, 40)).astype(F)
    bq, s = oracle.gemm_quantize_tensor(b)
    assert s == F(127) / np.abs(b).max()
    assert np.array_equal(bq, npref.float2int8(b * s))


@pytest.mark.parametrize("bt", [-1, 0, 1, 2, 3, 4])
@pytest.mark.parametrize("alpha,beta,transpose,per_col", [(1.0, 1.0, False, False), (0.5, 2.0, True, False),
                                                          (1.0, 1.0, False, True), (1.7, 0.3, False, True)])
def test_gemm_int8_matches_numpy(bt, alpha, beta, transpose, per_col):
    rng = np.random.default_rng(100 + bt)
    m, n, k = 13, 17, 96
    a = rng.normal(0, 1, (m, k)).astype(F)
    aq, sa = oracle.gemm_quantize_rows(a)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = rng.uniform(50, 500, n if per_col else 1).astype(F)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    got, gacc = oracle.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose, want_acc=True)
    want, wacc = npref.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose)
    assert np.array_equal(gacc, wacc) and np.array_equal(got, want)


@pytest.mark.parametrize("bt", [-1, 0, 1, 4])
@pytest.mark.parametrize("per_col", [False, True])
@pytest.mark.parametrize("scale_span", [(50.0, 500.0), (1e-3, 1e3)])
def test_gemm_int8_dequantisation_is_the_closed_form_to_a_few_ulp(bt, per_col, scale_span):
    """What the mathematics fixes for the Gemm epilogue, independent of any restatement of its formula: the result is
    alpha * (acc / (sA_i * sB_j) + beta * c) evaluated in float64, and the fp32 statements of the reference
    (src/layer/gemm.cpp:509-555: one division for the descale, one multiply by it, the C term, the multiply by alpha; with
    one B scale per column two divisions and two multiplies) round at most five times on the way, so every output lies
    within 4 ulp of the float64 value's magnitude (measured on the larger of the result and its two addends: the sum may
    cancel).  A transposed operand, a scale applied to the wrong axis, a dropped beta or alpha miss this by orders of
    magnitude on scales that span six decades."""
    rng = np.random.default_rng(7 + bt + 10 * per_col)
    m, n, k = 13, 17, 96
    a = rng.normal(0, 1, (m, k)).astype(F) * np.exp(rng.uniform(np.log(scale_span[0]), np.log(scale_span[1]), (m, 1))).astype(F)
    aq, sa = oracle.gemm_quantize_rows(a)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = np.exp(rng.uniform(np.log(scale_span[0]), np.log(scale_span[1]), n if per_col else 1)).astype(F)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    alpha, beta = 1.7, 0.3
    got = oracle.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, False).astype(np.float64)
    acc = aq.astype(np.int64) @ bq.astype(np.int64).T
    scale = sa.astype(np.float64)[:, None] * (sb.astype(np.float64)[None, :] if per_col else float(sb[0]))
    deq = acc / scale
    cterm = np.zeros((m, n))
    if bt == 0:
        cterm[:] = float(c[0])
    elif bt == 1:
        cterm[:] = c.astype(np.float64)[:, None]
    elif bt == 4:
        cterm[:] = c.astype(np.float64).reshape(1, n)
    want = float(F(alpha)) * (deq + float(F(beta)) * cterm)
    magnitude = float(F(alpha)) * np.maximum(np.abs(deq), np.abs(float(F(beta)) * cterm))
    ulp = np.maximum(magnitude, 1e-300) * 2.0 ** -23
    assert got.shape == want.shape
    assert np.all(np.abs(got - want) <= 4 * ulp), float(np.max(np.abs(got - want) / ulp))


def test_gemm_operands_are_not_transposed():
    # asymmetric one-hot probes: acc[i][j] must be sum_k A[i][k]*B[j][k]
    aq = np.zeros((2, 4), np.int8)
    bq = np.zeros((3, 4), np.int8)
    aq[1, 2] = 5
    bq[2, 2] = -7
    _, acc = oracle.gemm_int8(aq, bq, np.ones(2, F), [1.0], want_acc=True)
    want = np.zeros((2, 3), np.int32)
    want[1, 2] = -35
    assert np.array_equal(acc, want)


# ----------------------------------------------------------------------------- block quant
@pytest.mark.parametrize("bits", [4, 6, 8])
@pytest.mark.parametrize("block", [32, 64, 128])
def test_blockquant_pack_unpack_inverse(bits, block):
    rng = np.random.default_rng(bits * 10 + block)
    n, k = 5, 200  # k not a multiple of any block size
    w = rng.normal(0, 0.02, (n, k)).astype(F)
    w[1, 64:128] = 0  # an all-zero block -> scale 1
    packed, scales = oracle.blockquant_pack(w, bits, block)
    q_np = npref.blockquant_unpack_all(packed, k, bits)
    q_c = np.array([[oracle.blockquant_unpack(packed[j], kk, bits) for kk in range(k)] for j in range(n)])
    assert np.array_equal(q_np, q_c)
    qmax = (1 << (bits - 1)) - 1
    assert q_c.max() <= qmax and q_c.min() >= -qmax
    # re-deriving q from the definition (scale = qmax/absmax per block, round half away)
    for j in range(n):
        for bi in range((k + block - 1) // block):
            blk = w[j, bi * block: (bi + 1) * block]
            am = np.abs(blk).max()
            s = F(1) if am == 0 else F(qmax) / am
            assert scales[j, bi] == s
            want = np.clip(npref.float2int8(blk * s).astype(int), -qmax, qmax)
            assert np.array_equal(q_c[j, bi * block: (bi + 1) * block], want)


def test_blockquant_unpack_known_bit_patterns():
    # 4-bit: byte 0xF1 -> low nibble 1, high nibble -1 ; 6-bit stream 0b11_111110, 0b0000_0001 -> -2, 7
    assert [oracle.blockquant_unpack(np.array([0xF1], np.uint8), k, 4) for k in range(2)] == [1, -1]
    row = np.array([0b11111110, 0b00000001, 0x00], np.uint8)
    assert [oracle.blockquant_unpack(row, k, 6) for k in range(2)] == [-2, 7]
    assert oracle.blockquant_unpack(np.array([0x80, 0x7F], np.uint8), 0, 8) == -128
    assert oracle.blockquant_unpack(np.array([0x80, 0x7F], np.uint8), 1, 8) == 127


@pytest.mark.parametrize("bits,block,m,n,k,bt,in_sc", [
    (8, 64, 1, 24, 256, -1, False), (8, 64, 4, 16, 200, 4, False), (4, 32, 3, 9, 100, 3, True),
    (6, 128, 2, 7, 300, 1, True), (8, 32, 16, 8, 64, 0, False), (4, 64, 1, 5, 65, 2, False)])
def test_blockquant_gemm_matches_float64_within_sequential_sum_error(bits, block, m, n, k, bt, in_sc):
    rng = np.random.default_rng(bits + block + m + n + k)
    a = rng.normal(0, 1, (m, k)).astype(F)
    w = rng.normal(0, 0.02, (n, k)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    ins = (0.75 + (np.arange(k) % 5) * 0.15).astype(F) if in_sc else None
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    got = oracle.gemm_blockquant(a, packed, scales, bits, block, ins, c, bt, 1.25, 0.5)
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins, c, bt, 1.25, 0.5)
    # sequential binary32 summation of k terms: |err| <= k * 2^-24 * sum|terms| (first-order bound)
    assert np.all(np.abs(got - val) <= (k + 4) * 2.0 ** -24 * floor + 1e-30)


def test_blockquant_gemm_exact_on_power_of_two_data():
    # every product and partial sum exactly representable -> the sequential fp32 sum has no rounding
    k, n, m = 128, 6, 2
    rng = np.random.default_rng(3)
    q = rng.integers(-127, 128, (n, k)).astype(np.int8)
    scales = np.full((n, k // 64), F(4.0), F)  # descale 0.25 exact
    a = rng.integers(-8, 9, (m, k)).astype(F)
    got = oracle.gemm_blockquant(a, q.view(np.uint8), scales, 8, 64)
    want = (a.astype(np.int64) @ q.astype(np.int64).T) * 0.25
    assert np.array_equal(got, want.astype(F))


# ----------------------------------------------------------------------------- the benchmark's x86 baseline
@pytest.mark.parametrize("m,n,k,per_col", [(7, 50, 96, False), (33, 130, 1000, True), (4, 64, 64, False), (9, 17, 5, True)])
def test_vnni_cpu_baseline_equals_the_scalar_oracle(m, n, k, per_col):
    """The VNNI Gemm timed beside the GPU computes the same function as the scalar restatement: same int32 sums,
    same fp32 results, including rows that quantise through the +-0.5 edge cases."""
    from oracle import cpubaseline
    if not cpubaseline.available():
        pytest.skip("host CPU has no AVX512-VNNI")
    rng = np.random.default_rng(m * n + k)
    a = rng.standard_normal((m, k)).astype(F)
    a[0, :] = 0                                   # zero row: scale 1
    a[1, : min(k, 4)] = np.array([0.49999997, -0.49999997, 0.5, -0.5], F)[: min(k, 4)]
    a[1, -1] = F(127.0) if k > 4 else a[1, -1]    # absmax 127 -> scale exactly 1: the values above meet float2int8 raw
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = rng.uniform(20, 90, n if per_col else 1).astype(F)
    bias = rng.standard_normal(n).astype(F)
    aq, sa = oracle.gemm_quantize_rows(a)
    want, wacc = oracle.gemm_int8(aq, bq, sa, sb, bias, 4, want_acc=True)
    got, gacc = cpubaseline.gemm(a, cpubaseline.pack_b(bq), n, sb, bias, want_acc=True)
    assert np.array_equal(gacc, wacc)
    assert np.array_equal(got, want)


def _cpu_conv_desc(cb, d, n):
    top, bottom, left, right = oracle.resolve_padding(d)
    return cb.ConvDesc(d.w, d.h, d.c, n, d.num_output, d.kernel_w, d.kernel_h, d.dilation_w, d.dilation_h, d.stride_w, d.stride_h,
                       left, right, top, bottom, d.pad_value)


_EDGE_VALUES = np.array([0.49999997, -0.49999997, 0.5, -0.5, 1.5, -2.5, 126.5, -126.5, 127.49, 300.0, -300.0, 3e9, -3e9, np.inf, -np.inf, np.nan], F)


@pytest.mark.parametrize("c,h,w,outc,kernel,dilation,stride,pads,pad_value,term,act,int8_in", [
    (16, 9, 11, 32, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 1, False),
    (3, 20, 20, 20, (7, 7), (1, 1), (2, 2), (3, 3, 3, 3), 0.0, 2, 0, False),        # K = 147: a tail of 3 bytes; 20 channels: a tail of 4 lanes
    (64, 8, 8, 64, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0), 0.0, 101, 1, True),        # rows are the pixels themselves
    (24, 7, 7, 130, (1, 1), (1, 1), (2, 2), (0, 0, 0, 0), 0.0, 102, 3, True),
    (8, 10, 9, 17, (3, 2), (2, 1), (1, 2), (-233, -233, -233, -233), 3.0, 1, 2, False),   # SAME_UPPER, a border value, dilation
    (8, 6, 6, 16, (3, 3), (1, 1), (1, 1), (-234, -234, -234, -234), 0.0, 101, 4, True),
    (12, 5, 5, 10, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 5, False),
    (12, 5, 5, 10, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 101, 6, False),
])
def test_vnni_convolution_baseline_equals_the_scalar_oracle(c, h, w, outc, kernel, dilation, stride, pads, pad_value, term, act, int8_in):
    """The im2col + VNNI convolution timed beside the GPU is the oracle's function: fp32 and int8 outputs bit for bit, over
    batches, every activation type, borders, strides, dilation, channel and K tails, a zero weight scale, and inputs that
    quantise through float2int8's edge cases."""
    from oracle import cpubaseline as cb
    if not cb.available():
        pytest.skip("host CPU has no AVX512-VNNI")
    n = 3
    rng = np.random.default_rng(c * h + outc)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(F)
    in_scale = F(127.0)
    x.reshape(-1)[: _EDGE_VALUES.size] = _EDGE_VALUES / in_scale if not int8_in else 0
    if int8_in:
        x = rng.integers(-127, 128, (n, c, h, w)).astype(np.int8)
    wq = rng.integers(-127, 128, (outc, c, kernel[1], kernel[0])).astype(np.int8)
    ws = rng.uniform(50, 200, outc).astype(F)
    ws[1] = 0
    bias = rng.uniform(-1, 1, outc).astype(F)
    bias[2] = np.nan if act == 1 else bias[2]
    top = np.array([F(20.0)], F) if term > 100 else None
    ap = (0.1, 0.0) if act == 2 else (-0.5, 2.0) if act == 3 else (0.2, 0.5) if act == 6 else (0.0, 0.0)
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, pad_value, 1, 1, term, act, ap)
    want = np.stack([oracle.convolution_int8(d, x[i], wq, bias, ws, in_scale, None if top is None else top[0]) for i in range(n)])
    got = cb.conv_nhwc(_cpu_conv_desc(cb, d, n), np.ascontiguousarray(x.transpose(0, 2, 3, 1)), in_scale, cb.pack_conv_weights(wq),
                       cb.fold_scales(ws, in_scale), bias, top, act, ap)
    assert np.array_equal(got.transpose(0, 3, 1, 2), want, equal_nan=True)


@pytest.mark.parametrize("c,h,w,kernel,stride,pads,term,act,int8_in", [
    (32, 9, 9, (3, 3), (1, 1), (1, 1, 1, 1), 1, 3, False),
    (20, 8, 10, (3, 3), (2, 2), (-233, -233, -233, -233), 101, 1, True),
    (7, 6, 6, (5, 5), (1, 1), (2, 2, 2, 2), 102, 0, False),
    (48, 7, 7, (3, 3), (1, 1), (1, 1, 1, 1), 2, 2, True),
])
def test_depthwise_baseline_equals_the_scalar_oracle(c, h, w, kernel, stride, pads, term, act, int8_in):
    from oracle import cpubaseline as cb
    if not cb.available():
        pytest.skip("host CPU has no AVX512-VNNI")
    n = 2
    rng = np.random.default_rng(c + h)
    x = rng.uniform(-1, 1, (n, c, h, w)).astype(F)
    x.reshape(-1)[: _EDGE_VALUES.size] = _EDGE_VALUES / F(100.0)
    if int8_in:
        x = rng.integers(-127, 128, (n, c, h, w)).astype(np.int8)
    wq = rng.integers(-127, 128, (c, 1, kernel[1], kernel[0])).astype(np.int8)
    per_group = term in (1, 101)
    ws = rng.uniform(50, 200, c).astype(F) if per_group else np.full(c, F(77.0), F)
    if per_group:
        ws[1] = 0
    ins = np.full(c, F(100.0), F)
    tops = np.full(c, F(15.0), F) if term > 100 else None
    bias = rng.uniform(-1, 1, c).astype(F)
    ap = (0.1, 0.0) if act == 2 else (0.0, 6.0)
    d = oracle.make_desc((c, h, w), c, kernel, (1, 1), stride, pads, 0.0, 1, c, term, act, ap)
    want = np.stack([oracle.convolutiondepthwise_int8(d, x[i], wq, bias, ws, ins, tops) for i in range(n)])
    taps = np.ascontiguousarray(wq.reshape(c, -1).T)
    got = cb.dwconv_nhwc(_cpu_conv_desc(cb, d, n), np.ascontiguousarray(x.transpose(0, 2, 3, 1)), ins, taps, cb.fold_scales(ws, ins), bias, tops, act, ap)
    assert np.array_equal(got.transpose(0, 3, 1, 2), want, equal_nan=True)


@pytest.mark.parametrize("which,kw", [("tiny", {}), ("mobilenetv2", dict(input_hw=64, n_calib=1)), ("resnet50", dict(input_hw=64, n_calib=1))])
def test_cpu_baseline_model_pass_equals_the_oracle_executor(which, kw):
    """The whole-model CPU pass timed beside the GPU (VNNI layers + the glue loops, channels-last) gives the blobs of the
    scalar oracle's executor bit for bit, for a batch, and again when it writes into the arrays of the pass before."""
    from ncnn_amd import zoo
    from oracle import cpubaseline as cb, cpunet
    import refnet
    if not cb.available():
        pytest.skip("host CPU has no AVX512-VNNI")
    g, param, blob, info = zoo.build(which, **kw)
    x = np.random.default_rng(4).uniform(0, 1, (2,) + tuple(g.input_shape)).astype(F)
    model = cpunet.load(param, blob)
    first = cpunet.run(model, x)
    again = cpunet.run(model, x[::-1].copy(), keep=first)
    again = cpunet.run(model, x, keep=again)
    layers = refnet.parse_param(param)
    overwritten = {L["bottoms"][0] for L in layers if L["type"] == "ReLU"}  # in-place layers leave their result in the bottom blob
    for i in range(2):
        ref = refnet.run(param, blob, x[i])
        checked = 0
        for name, v in ref.items():
            if name in overwritten or name not in again:
                continue
            want = v if v.ndim != 3 else v.transpose(1, 2, 0)
            assert np.array_equal(again[name][i].reshape(want.shape), want), name
            checked += 1
        assert checked >= 8


def test_float_pipe_formulation_of_float2int8_equals_the_oracle():
    """The device rounds without leaving the float pipe: clamp to [-127, 127], add copysign(0.5) with the add rounded
    TOWARD ZERO, truncate; one compare-select for NaN and |v| >= 2^31.  The same operations evaluated here (the add
    exactly in float64, then rounded toward zero to float32) must give float2int8's value on ties, near-ties, the clamp
    edges, huge values, infinities and NaN, and on a dense random sample -- and the nearest-even add it replaces must
    fail on 0.49999997, which is why the rounding mode matters."""
    rng = np.random.default_rng(7)
    ks = np.arange(-300, 301, dtype=np.float64)
    ties = np.concatenate([ks + 0.5, np.nextafter((ks + 0.5).astype(F), F(np.inf)), np.nextafter((ks + 0.5).astype(F), F(-np.inf))]).astype(F)
    special = np.array([0.0, -0.0, 0.49999997, -0.49999997, 126.5, -126.5, 127.49, -127.49, 127.5, -127.5, 200, -200, 2147483520.0, 2147483648.0,
                        -2147483648.0, 4e9, -4e9, 1e30, -1e30, np.inf, -np.inf, np.nan, 8388607.5, -8388607.5, 1e-40, -1e-40], F)
    v = np.concatenate([ties, special, rng.normal(0, 60, 200000).astype(F), rng.uniform(-130, 130, 200000).astype(F)])

    def formulation(toward_zero):
        with np.errstate(invalid="ignore"):
            c = np.where(np.isnan(v), F(0), np.clip(v, F(-127), F(127))).astype(F)  # a NaN is overridden below
            exact = c.astype(np.float64) + np.copysign(0.5, c.astype(np.float64))   # exact: both fit in 53 bits
            y = exact.astype(F)                                                     # nearest even
            if toward_zero:
                y = np.where(np.abs(y.astype(np.float64)) > np.abs(exact), np.nextafter(y, F(0)), y).astype(F)
            r = np.trunc(y)
            return np.where(np.abs(v) < F(2147483648.0), r, F(-127))

    want = oracle.float2int8(v).astype(F)
    assert np.array_equal(formulation(True), want)
    wrong = formulation(False) != want
    assert wrong.any() and wrong[np.flatnonzero(v == F(0.49999997))[0]]


def test_clip_folded_into_the_requantising_clamp_equals_clip_then_requantise():
    """The device replaces  float2int8(clip(f, p0, p1) * s)  by  float2int8 of  clamp(f * s, lo, hi)  with
    lo = clamp(p0 * s, -127, 127), hi = clamp(p1 * s, -127, 127)  when p0 <= p1, s >= 0 and everything is finite (the
    multiplication is monotone, so it commutes with min and max; nested clamps are one clamp).  Both sides evaluated in
    float32 here, the left one by the oracle's float2int8: equal on values at and around the clip bounds, around the
    images of the bounds, on ties, and on a dense sample, for scales that make the bounds' images integers, half
    integers, tiny, beyond 127, and zero -- and NOT equal once the scale is negative or the clipped value times the
    scale can reach 2^31 (where float2int8 answers -127), which is why the device tests both before folding."""
    rng = np.random.default_rng(11)
    differs_for_negative_scale = differs_for_huge_bounds = False
    for p0, p1 in [(0.0, 6.0), (-0.37, 0.41), (0.013, 0.02), (-1e30, 1e30), (-3.0, -1.0), (2.5, 2.5)]:
        for s in [21.166666, 127.0 / 6.0, 0.25, 1e-3, 300.0, 0.0, 63.5 / 0.41, -21.0]:
            p0f, p1f, sf = F(p0), F(p1), F(s)
            around = [np.nextafter(b, d) for b in (p0f, p1f) for d in (F(-np.inf), F(np.inf))] + [p0f, p1f]
            ties = ((np.arange(-140, 141) + 0.5) / s).astype(F) if s != 0 else np.zeros(1, F)
            f = np.concatenate([np.array(around, F), ties, np.nextafter(ties, F(np.inf)), np.nextafter(ties, F(-np.inf)),
                                rng.normal(0, 3, 20000).astype(F), rng.uniform(-8, 8, 20000).astype(F), np.array([0.0, -0.0, 1e20, -1e20], F)])
            with np.errstate(over="ignore"):
                want = oracle.float2int8((np.minimum(np.maximum(f, p0f), p1f) * sf).astype(F))
                lo = np.clip(F(p0f * sf), F(-127), F(127))
                hi = np.clip(F(p1f * sf), F(-127), F(127))
                got = oracle.float2int8(np.clip((f * sf).astype(F), min(lo, hi), max(lo, hi)).astype(F))
            if s >= 0 and max(abs(p0), abs(p1)) * s < 2.0 ** 31:
                assert np.array_equal(got, want), (p0, p1, s)
            elif s < 0:
                differs_for_negative_scale |= not np.array_equal(got, want)
            else:
                differs_for_huge_bounds |= not np.array_equal(got, want)
    assert differs_for_negative_scale and differs_for_huge_bounds


def test_float_quotient_is_within_one_of_the_integer_quotient_below_2_to_20():
    """The convolution kernel splits a pixel index into (sample, row, column) with a float reciprocal instead of an
    integer division when the index is below 2^20: trunc(float(n) * rcp(float(d))) is then off by at most one, which
    the remainder corrects.  Checked here for reciprocals up to two ulps off in either direction (the hardware's is
    good to one), over random and extreme operands."""
    rng = np.random.default_rng(3)
    n = np.concatenate([rng.integers(0, 1 << 20, 400000), np.array([0, 1, (1 << 20) - 1, (1 << 20) - 2, 1 << 19])]).astype(np.int64)
    d = np.concatenate([rng.integers(1, 1 << 20, 200000), rng.integers(1, 300, 200000), np.array([1, 1, 2, 3, (1 << 20) - 1])]).astype(np.int64)
    rcp = (F(1) / d.astype(F)).astype(F)
    for ulps in (-2, -1, 0, 1, 2):
        r = rcp.copy()
        for _ in range(abs(ulps)):
            r = np.nextafter(r, F(np.inf) if ulps > 0 else F(0))
        q = np.trunc(n.astype(F) * r).astype(np.int64)
        assert np.abs(q - n // d).max() <= 1, ulps


# ---- attention with block-quantised weights (src/layer/multiheadattention.cpp:561-912) ---------------------------------

def _mha_tolerance(case):
    """|error| allowed per output: fp32 sequential sums over <= max(K, dst) terms of O(1) values."""
    return 2e-4


@pytest.mark.parametrize("spec", cases.MHA_CASES, ids=[str(c[0]) for c in cases.MHA_CASES])
def test_mha_blockquant_matches_float64_attention(spec):
    case = cases.mha_case(*spec)
    out, ko, vo = oracle.mha_blockquant(**case)
    want, kw, vw = npref.mha_f64(**case)
    assert out.shape == want.shape and ko.shape == kw.shape
    assert np.abs(out - want).max() <= _mha_tolerance(case) * max(1.0, np.abs(want).max())
    assert np.abs(ko - kw).max() <= 1e-4 * max(1.0, np.abs(kw).max())
    assert np.abs(vo - vw).max() <= 1e-4 * max(1.0, np.abs(vw).max())


def test_mha_blockquant_matches_torch_multi_head_attention():
    """The layer follows torch.nn.MultiheadAttention (multiheadattention.cpp:234): with the dequantised weights as
    its projection matrices torch's own routine must give the same numbers."""
    torch = pytest.importorskip("torch")
    case = cases.mha_case(21, 64, 4, 64, 48, 40, 6, 8, 8, 32, False, 0, True, "2d")
    out, _, _ = oracle.mha_blockquant(**case)
    wq, wk, wv, wo = [npref.blockquant_dequantise(w[0], w[1], k, 8, 32) for w, k in zip(case["weights"], (64, 48, 40, 64))]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a, np.float32))
    bias = np.concatenate([case["weights"][i][3] for i in range(3)])
    got, _ = torch.nn.functional.multi_head_attention_forward(
        t(case["q"])[:, None], t(case["k"])[:, None], t(case["v"])[:, None], 64, 4, None, t(bias), None, None, False, 0.0, t(wo), t(case["weights"][3][3]),
        training=False, need_weights=False, attn_mask=t(case["mask"]), use_separate_proj_weight=True, q_proj_weight=t(wq), k_proj_weight=t(wk),
        v_proj_weight=t(wv))
    assert np.abs(got[:, 0].numpy() - out).max() <= 2e-5 * max(1.0, np.abs(out).max())


def test_mha_blockquant_cache_identity():
    """Causal self-attention over n tokens == n one-token calls that hand their keys / values back as the cache;
    masked-out keys contribute exact zeros, so the two evaluations agree bit for bit."""
    n, e = 6, 64
    case = cases.mha_case(31, e, 4, e, e, e, n, n, 8, 64, False, 0, True, None)
    causal = np.where(np.arange(n)[None, :] <= np.arange(n)[:, None], 0.0, -1e30).astype(F)
    full, kfull, vfull = oracle.mha_blockquant(**dict(case, mask=causal))
    ck = cv = None
    for i in range(n):
        x = case["q"][i:i + 1]
        step, ck, cv = oracle.mha_blockquant(**dict(case, q=x, k=x, v=x, cached_k=ck, cached_v=cv))
        assert np.array_equal(step[0], full[i]), i
    assert np.array_equal(ck, kfull) and np.array_equal(cv, vfull)


@pytest.mark.parametrize("bits,block", [(4, 32), (6, 128), (8, 64), (4, 64), (6, 32)])
def test_product_side_block_quantiser_equals_the_oracles(bits, block):
    """ncnn_amd.synth.blockquant_weights (numpy; feeds the benchmark and the model writer) against the oracle's packer."""
    from ncnn_amd import synth
    rng = np.random.default_rng(bits * block)
    w = (rng.standard_normal((13, 200)) * 0.02).astype(F)
    w[3, :64] = 0
    p1, s1 = synth.blockquant_weights(w, bits, block)
    p2, s2 = oracle.blockquant_pack(w, bits, block)
    assert np.array_equal(p1, p2) and np.array_equal(s1, s2)
