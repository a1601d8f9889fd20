"""GPU parity: every C-ABI launch against the CPU oracle on identical seeded inputs.

int32 accumulators and requantised int8 outputs must be bit-exact.  fp32 outputs of the integer
layers are produced by the same sequence of single fp32 operations as the reference, so they are
required to be bit-exact too (stricter than the 1e-5 relative the task allows).  The block-quant
Gemm accumulates in a different order than the reference's sequential sum and is held to
|gpu - ref| <= 1e-5 * sum_k |a_k * w_k|.
"""
import ctypes as C

import os

import numpy as np
import pytest

import cases
import npref
from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


def _say(*a):
    print(*a, flush=True)


# ----------------------------------------------------------------------------- quantize
def test_quantize_matches_oracle(rt):
    rng = np.random.default_rng(0)
    for rows, cols in ((1, 5), (3, 1024), (7, 1031), (64, 3136)):
        _say("quantize", rows, cols)
        x = rng.uniform(-3, 3, (rows, cols)).astype(F)
        x.flat[:8] = [0.5, -0.5, 1.5, -1.5, 0.49999997, 126.5, 1e9, -1e9][: min(8, x.size)]
        for scales in (rng.uniform(5, 60, rows).astype(F), np.array([F(42.3)])):
            assert np.array_equal(rt.quantize(x, scales), oracle.quantize(x, scales))
    special = np.array([[np.nan, np.inf, -np.inf, 3e9, -3e9, 127.5, -127.5, 0.0]], F)
    assert np.array_equal(rt.quantize(special, [1.0]), oracle.quantize(special, [1.0]))


# ----------------------------------------------------------------------------- gemm
@pytest.mark.parametrize("m,k", [(5, 77), (9, 4096), (16, 4100), (33, 513), (8200, 4096)])  # the last one is above 128 MB: non-temporal loads
def test_gemm_quantize_rows(rt, m, k):
    _say("gemm_quantize_rows", m, k)
    a = np.random.default_rng(m * k).standard_normal((m, k), dtype=F)
    a[m // 2] = 0
    gq, gs = rt.gemm_quantize_rows(a)
    oq, os_ = oracle.gemm_quantize_rows(a)
    assert np.array_equal(gs, os_) and np.array_equal(gq, oq)


def test_gemm_quantize_tensor(rt):
    b = (np.random.default_rng(3).standard_normal((37, 129), dtype=F) * F(0.02)).astype(F)
    gq, gs = rt.gemm_quantize_tensor(b)
    oq, os_ = oracle.gemm_quantize_tensor(b)
    assert gs == os_ and np.array_equal(gq, oq)


def test_transposes(rt):
    rng = np.random.default_rng(4)
    a = rng.standard_normal((45, 70), dtype=F)
    assert np.array_equal(rt.transpose(a), a.T)
    q = rng.integers(-127, 128, (33, 129)).astype(np.int8)
    assert np.array_equal(rt.transpose(q), q.T)


GEMM_SHAPES = [(13, 17, 96), (1, 1, 1), (128, 128, 64), (130, 257, 100), (64, 300, 77), (256, 512, 1024), (300, 200, 4100),
               # one to four rows of A on 64 columns and more: one wavefront per row of B (aligned rows, ragged K, K below a vector)
               (1, 4096, 4096), (4, 1000, 2048), (3, 64, 100), (2, 333, 8),
               # up to 48 rows on the matrix cores, 16 rows of A per group: ragged last group, ragged last tile of B, one K step
               (16, 256, 64), (17, 1000, 1024), (48, 70, 2048), (33, 4096, 128)]


@pytest.mark.parametrize("shape", GEMM_SHAPES)
@pytest.mark.parametrize("bt,alpha,beta,transpose,per_col", [(-1, 1.0, 1.0, False, False), (4, 1.0, 1.0, False, False),
                                                             (3, 0.5, 2.0, True, False), (1, 1.7, 0.3, False, True),
                                                             (0, 1.0, 1.0, False, True), (2, 1.0, -1.0, True, True)])
def test_gemm_int8_bit_exact(rt, shape, bt, alpha, beta, transpose, per_col):
    m, n, k = shape
    _say("gemm_int8", shape, bt, alpha, beta, transpose, per_col)
    a, bq, sb, _ = cases.gemm_case(m * 31 + n * 7 + k, m, n, k, per_col)
    rng = np.random.default_rng(bt + 10)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    aq, sa = oracle.gemm_quantize_rows(a)
    want, wacc = oracle.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose, want_acc=True)
    got, gacc = rt.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose, want_acc=True)
    assert np.array_equal(gacc, wacc)
    assert np.array_equal(got, want)
    # without the accumulator dump the launcher may pick a pipelined kernel: same answer
    assert np.array_equal(rt.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose), want)


@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1024), (100, 64, 64), (333, 260, 192), (64, 1000, 2048), (2048, 2048, 512)])
@pytest.mark.parametrize("bt,alpha,beta,per_col", [(4, 1.0, 1.0, True), (-1, 1.0, 1.0, False), (1, 0.5, 2.0, False), (0, 1.0, 1.5, True)])
def test_gemm_int8_mid_sizes_through_the_pipelined_kernels(rt, m, n, k, bt, alpha, beta, per_col):
    """K % 64 == 0 shapes below the 256x256 kernel's range run as a 1x1 convolution over the rows of A."""
    _say("gemm_int8 mid", m, n, k, bt, per_col)
    a, bq, sb, _ = cases.gemm_case(m + n + k + bt, m, n, k, per_col)
    rng = np.random.default_rng(bt + 20)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    aq, sa = oracle.gemm_quantize_rows(a)
    want, _ = npref.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta)
    assert np.array_equal(rt.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta), want)


def test_gemm_int8_1024_cube_against_numpy_int_matmul(rt):
    # one of the benchmark's own sizes; the accumulators are checked against an exact integer matmul
    m = n = k = 1024
    _say("gemm_int8 1024^3")
    a, bq, sb, bias = cases.gemm_case(1024, m, n, k)
    aq, sa = rt.gemm_quantize_rows(a)
    oq, os_ = oracle.gemm_quantize_rows(a)
    assert np.array_equal(aq, oq) and np.array_equal(sa, os_)
    got, gacc = rt.gemm_int8(aq, bq, sa, sb, bias, 4, want_acc=True)
    want, wacc = npref.gemm_int8(aq, bq, sa, sb, bias, 4)
    assert np.array_equal(gacc, wacc)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("m,n,k", [(2048, 4096, 64), (4096, 2048, 192), (2304, 3840, 320), (4096, 4096, 4096)])
@pytest.mark.parametrize("bt,per_col", [(4, True), (-1, False)])
def test_gemm_int8_256x256_kernel_sizes(rt, m, n, k, bt, per_col):
    """From 128 tiles of 256 x 256 up (K % 64 == 0) the Gemm runs on the 256x256 ring kernel: one, three and five K steps
    (shorter than, equal to and longer than the ring's prologue), a tile count that is not a multiple of 8 with a ragged last
    row group, and the benchmark's own 4096 cube.  Every output element is compared; the accumulators come from a float64
    matmul, which is exact here, and the 2048 x 4096 x 64 case is also checked against the scalar oracle."""
    _say("gemm_int8 256x256", m, n, k, bt, per_col)
    a, bq, sb, bias = cases.gemm_case(m + 3 * n + 7 * k, m, n, k, per_col)
    c = bias.reshape(1, n) if bt == 4 else None
    aq, sa = rt.gemm_quantize_rows(a)
    oq, os_ = oracle.gemm_quantize_rows(a)
    assert np.array_equal(aq, oq) and np.array_equal(sa, os_)
    acc = npref.gemm_acc_exact(aq, bq)
    want, _ = npref.gemm_int8(aq, bq, sa, sb, c, bt, acc=acc)
    got = rt.gemm_int8(aq, bq, sa, sb, c, bt)
    assert np.array_equal(got, want)
    if k == 64 and not per_col:
        assert np.array_equal(got, oracle.gemm_int8(aq, bq, sa, sb, c, bt))
    # the same Gemm on operands in the kernel's tiled layout: the quantiser writes A tiled, B is tiled once
    atq, ats = rt.gemm_quantize_rows_tiled(a)
    assert np.array_equal(ats, sa)
    assert np.array_equal(atq, _tiled(aq, False))
    btq = rt.gemm_tile_operand(bq, 1)
    assert np.array_equal(btq, _tiled(bq, True))
    assert np.array_equal(rt.gemm_tile_operand(aq, 0), atq)
    assert np.array_equal(rt.gemm_int8_tiled(atq, btq, m, n, k, sa, sb, c, bt), want)


@pytest.mark.parametrize("depth", [64, 128])
@pytest.mark.parametrize("m,n,k", [(1024, 1024, 64), (1024, 1024, 128), (1024, 1024, 192), (896, 1024, 384), (896, 1024, 448), (1152, 768, 512), (1024, 1024, 576),
                                   (1024, 1024, 640), (1024, 1024, 1024), (1280, 1408, 1280), (2048, 2048, 2048)])
@pytest.mark.parametrize("bt,per_col", [(4, True), (-1, False)])
def test_gemm_int8_128x128_kernel_sizes(rt, m, n, k, bt, per_col, depth):
    """Between 48 tiles of 128 x 128 and 128 tiles of 256 x 256 the Gemm runs on the 128x128 ring kernels: K steps of 128 bytes
    where K allows, of 64 bytes otherwise or when NCNNHIP_GEMM_RING128=64 (read at every call) forces them.  K steps fewer than,
    equal to and more than the ring's four stages in either form, tile counts that are not a multiple of 8 with a ragged last row
    group, the 1024 and 2048 cubes of the benchmark's grid.  Every output element
    against the epilogue op by op on exact accumulators; the 1024 x 1024 x 64 case also against the scalar oracle; and the same
    call with the kernel switched off (the 64-row tiles of the convolution kernel) gives the same bits."""
    _say("gemm_int8 128x128", m, n, k, bt, per_col, depth)
    a, bq, sb, bias = cases.gemm_case(m + 3 * n + 7 * k, m, n, k, per_col)
    c = bias.reshape(1, n) if bt == 4 else None
    aq, sa = oracle.gemm_quantize_rows(a)
    want, _ = npref.gemm_int8(aq, bq, sa, sb, c, bt, acc=npref.gemm_acc_exact(aq, bq))
    saved = os.environ.get("NCNNHIP_GEMM_RING128")
    try:
        os.environ["NCNNHIP_GEMM_RING128"] = str(depth)
        got = rt.gemm_int8(aq, bq, sa, sb, c, bt)
        os.environ["NCNNHIP_GEMM_RING128"] = "0"
        other = rt.gemm_int8(aq, bq, sa, sb, c, bt) if depth == 128 else got
    finally:
        if saved is None:
            os.environ.pop("NCNNHIP_GEMM_RING128", None)
        else:
            os.environ["NCNNHIP_GEMM_RING128"] = saved
    assert np.array_equal(got, want)
    assert np.array_equal(other, want)
    if k == 64 and not per_col:
        assert np.array_equal(got, oracle.gemm_int8(aq, bq, sa, sb, c, bt))


def test_gemm_int8_8192_cube(rt):
    """The largest size of the standalone Gemm configuration, M = N = K = 8192 (4 tiles of 256 x 256 per compute unit, 128 K
    steps), every output element: row quantisation against the scalar oracle, accumulators from a float64 matmul (exact:
    8192 * 127 * 127 < 2^53), the fp32 epilogue op by op; row-major operands and the tiled operands the benchmark uses."""
    m = n = k = 8192
    _say("gemm_int8 8192 cube")
    a, bq, sb, bias = cases.gemm_case(8192, m, n, k, True)
    c = bias.reshape(1, n)
    oq, os_ = oracle.gemm_quantize_rows(a)
    atq, ats = rt.gemm_quantize_rows_tiled(a)
    assert np.array_equal(ats, os_) and np.array_equal(atq, _tiled(oq, False))
    del a
    _say("  exact accumulators")
    acc = npref.gemm_acc_exact(oq, bq)
    want, _ = npref.gemm_int8(oq, bq, os_, sb, c, 4, acc=acc)
    del acc
    _say("  tiled launch")
    got = rt.gemm_int8_tiled(atq, rt.gemm_tile_operand(bq, 1), m, n, k, os_, sb, c, 4)
    assert np.array_equal(got, want)
    _say("  row-major launch")
    got = rt.gemm_int8(oq, bq, os_, sb, c, 4)
    assert np.array_equal(got, want)
    # 64 rows spread over the matrix against the scalar oracle itself (the whole cube would take it minutes)
    rows = np.arange(64) * 128 + 77
    assert np.array_equal(want[rows], oracle.gemm_int8(oq[rows], bq, os_[rows], sb, c, 4))


@pytest.mark.parametrize("m,n,k", [(256, 256, 8192), (512, 256, 64), (256, 768, 1088)])
def test_gemm_int8_tiled_entry_few_tiles(rt, m, n, k):
    """The tiled entry points take any whole number of tiles: one tile with the longest rows the tiled quantiser accepts
    (8192, eight 16-byte loads per thread), two tiles with a single K step, three tiles with 17 steps."""
    _say("gemm_int8 tiled, few tiles", m, n, k)
    a, bq, sb, bias = cases.gemm_case(5 * m + n + k, m, n, k, True)
    aq, sa = oracle.gemm_quantize_rows(a)
    atq, ats = rt.gemm_quantize_rows_tiled(a)
    assert np.array_equal(ats, sa) and np.array_equal(atq, _tiled(aq, False))
    want = oracle.gemm_int8(aq, bq, sa, sb, bias.reshape(1, n), 4, 0.75, 1.5)
    got = rt.gemm_int8_tiled(atq, rt.gemm_tile_operand(bq, 1), m, n, k, sa, sb, bias.reshape(1, n), 4, 0.75, 1.5)
    assert np.array_equal(got, want)


def _tiled(q, operand_b):
    """numpy statement of the tiled operand layout: [r / 256][k / 64][r % 256][k % 64]; for B, position p of a tile holds row
    (p >> 7) * 128 + 4 * (p & 31) + ((p >> 5) & 3)."""
    rows, k = q.shape
    t = q.reshape(rows // 256, 256, k // 64, 64)
    if operand_b:
        p = np.arange(256)
        t = t[:, (p >> 7) * 128 + 4 * (p & 31) + ((p >> 5) & 3)]
    return np.ascontiguousarray(t.transpose(0, 2, 1, 3)).reshape(-1)


def test_gemm_int8_tiled_rejects_what_it_cannot_run(rt):
    from ncnn_amd.hip import NcnnHipError
    q = np.zeros((256, 64), np.int8)
    for bad in (lambda: rt.gemm_tile_operand(np.zeros((255, 64), np.int8), 0), lambda: rt.gemm_tile_operand(np.zeros((256, 48), np.int8), 1),
                lambda: rt.gemm_quantize_rows_tiled(np.zeros((256, 100), F)),
                lambda: rt.gemm_int8_tiled(q.reshape(-1), q.reshape(-1), 256, 256, 64, np.ones(256, F), [1.0], np.zeros(256, F), 1)):
        with pytest.raises(NcnnHipError):
            bad()


# ----------------------------------------------------------------------------- convolution
CONV_CASES = [
    # c, h, w, outc, kernel, dilation, stride, pads
    (3, 9, 11, 4, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (5, 8, 7, 6, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
    (4, 12, 10, 8, (3, 2), (2, 1), (2, 1), (2, 1, 0, 1)),
    (2, 13, 13, 3, (5, 5), (1, 1), (2, 2), (-233, -233, -233, -233)),
    (2, 10, 9, 3, (4, 3), (1, 2), (3, 2), (-234, -234, -234, -234)),
    (16, 20, 20, 130, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (64, 14, 14, 64, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1)),
    (96, 7, 7, 200, (1, 1), (1, 1), (1, 1), (0, 0, 0, 0)),
]


@pytest.mark.parametrize("shape", CONV_CASES)
@pytest.mark.parametrize("term,act,act_params,bias,int8_in", [
    (1, 1, (0, 0), True, False), (2, 0, (0, 0), False, False), (101, 3, (0.0, 6.0), True, True), (102, 2, (0.1, 0), True, False),
    (1, 6, (1 / 6.0, 0.5), True, True)])
def test_convolution_bit_exact(rt, shape, term, act, act_params, bias, int8_in):
    c, h, w, outc, kernel, dilation, stride, pads = shape
    _say("conv", shape, term, act, bias, int8_in)
    x, wq, b, ws, ins, tops = cases.conv_case(c * 100 + outc + term, c, h, w, outc, kernel, 1, term, bias, int8_in)
    d = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, int(bias), 1, term, act, act_params)
    want, wacc = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0], None if tops is None else tops[0], want_acc=True)
    got, gacc = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, act_params, want_acc=True)
    assert np.array_equal(gacc[0], wacc)
    assert got.dtype == want.dtype and np.array_equal(got[0], want)
    fast = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, term, act, act_params, path="nhwc")
    assert fast.dtype == want.dtype and np.array_equal(fast[0], want)


@pytest.mark.parametrize("act", [4, 5])
@pytest.mark.parametrize("shape", [CONV_CASES[0], CONV_CASES[5], CONV_CASES[7]])
def test_convolution_sigmoid_and_mish(rt, shape, act):
    """Activation types 4 (sigmoid) and 5 (mish), src/layer/fused_activation.h:34-45, call expf / logf / tanhf: the device's
    are not the host libm's bit for bit, so these two are held to the tolerance stated for fp32 outputs,
    |gpu - ref| <= 1e-5 * max(|ref|, |value before the activation|), and a requantised int8 output may differ by one step
    only where the oracle's own value lies within that tolerance of a rounding tie.  Accumulators stay bit-exact."""
    c, h, w, outc, kernel, dilation, stride, pads = shape
    _say("conv sigmoid/mish", shape, act)
    for path in ("chw", "nhwc"):
        # fp32 output
        x, wq, b, ws, ins, _ = cases.conv_case(c + outc + act, c, h, w, outc, kernel, 1, 1, True, False, w_sigma=0.3)
        d0 = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, 1, 1, 0, (0, 0))
        da = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, 1, 1, act, (0, 0))
        before = oracle.convolution_int8(d0, x[0], wq, b, ws, ins[0])
        want = oracle.convolution_int8(da, x[0], wq, b, ws, ins[0])
        assert np.abs(before).max() > 2, "the case should reach both tails of the activation"
        got = rt.conv_layer(x[0], wq, b, ws, ins, None, outc, kernel, dilation, stride, pads, 0.0, 1, 1, act, (0, 0), path=path)[0]
        tol = 1e-5 * np.maximum(np.abs(want), np.abs(before))
        assert np.all(np.abs(got.astype(np.float64) - want) <= tol), (path, np.abs(got - want).max())
        # requantised output
        x, wq, b, ws, ins, tops = cases.conv_case(c + outc + act, c, h, w, outc, kernel, 1, 101, True, False, w_sigma=0.3)
        tops[:] = F(127) / F(4.0 if act == 5 else 1.0)
        d8 = oracle.make_desc((c, h, w), outc, kernel, dilation, stride, pads, 0.0, 1, 1, 101, act, (0, 0))
        want8 = oracle.convolution_int8(d8, x[0], wq, b, ws, ins[0], tops[0])
        got8 = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, kernel, dilation, stride, pads, 0.0, 1, 101, act, (0, 0), path=path)[0]
        diff = got8.astype(np.int32) - want8
        assert np.abs(diff).max() <= 1
        scaled = want.astype(np.float64) * float(tops[0])
        tie_distance = np.abs(np.abs(scaled - np.floor(scaled)) - 0.5)
        assert np.all(tie_distance[diff != 0] <= (tol * float(tops[0]) + 1e-6)[diff != 0]), path
        assert (diff != 0).mean() < 1e-3


def test_convolution_nonzero_pad_value(rt):
    x, wq, b, ws, ins, tops = cases.conv_case(5, 3, 6, 6, 4, (3, 3))
    d = oracle.make_desc((3, 6, 6), 4, (3, 3), pads=(1, 1, 1, 1), pad_value=3.7, bias_term=1)
    want = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0])
    for path in ("chw", "nhwc"):
        got = rt.conv_layer(x[0], wq, b, ws, ins, None, 4, (3, 3), pads=(1, 1, 1, 1), pad_value=3.7, path=path)
        assert np.array_equal(got[0], want), path


def test_convolution_zero_weight_scale(rt):
    x, wq, b, ws, ins, tops = cases.conv_case(6, 8, 6, 6, 5, (3, 3))
    ws[3] = 0
    got = rt.conv_layer(x[0], wq, b, ws, ins, None, 5, (3, 3), pads=(1, 1, 1, 1), act=1)
    assert np.all(got[0, 3] == max(b[3], 0))


@pytest.mark.parametrize("name,c,h,w,outc,kernel,stride,pads,term,act", [
    ("single-layer config 3x3 64->64 @56", 64, 56, 56, 64, (3, 3), (1, 1), (1, 1, 1, 1), 1, 1),
    ("resnet stem 7x7/2 3->64 @112 (reduced from 224)", 3, 112, 112, 64, (7, 7), (2, 2), (3, 3, 3, 3), 2, 0),
    ("resnet 1x1 256->64 @28 requant", 256, 28, 28, 64, (1, 1), (1, 1), (0, 0, 0, 0), 102, 1),
    ("resnet 1x1/2 256->512 @28 fp32 out", 256, 28, 28, 512, (1, 1), (2, 2), (0, 0, 0, 0), 2, 0),
    ("resnet 3x3 512->512 @7 requant", 512, 7, 7, 512, (3, 3), (1, 1), (1, 1, 1, 1), 102, 1),
    ("mobilenetv2 pointwise 96->24 @56 relu6", 96, 56, 56, 24, (1, 1), (1, 1), (0, 0, 0, 0), 101, 3),
    ("wide plane 3x3 20->130 @180 (channel count off the 16 grid, 128x128 tiles)", 20, 180, 180, 130, (3, 3), (1, 1), (1, 1, 1, 1), 101, 1),
    ("wide plane 1x1 40->48 @190 (64x128 tiles)", 40, 190, 190, 48, (1, 1), (1, 1), (0, 0, 0, 0), 1, 0),
    ("resnet 3x3 512->512 @7 fp32 out (K split over workgroups)", 512, 7, 7, 512, (3, 3), (1, 1), (1, 1, 1, 1), 1, 0),
])
def test_convolution_network_shapes(rt, name, c, h, w, outc, kernel, stride, pads, term, act):
    _say("conv net-shape", name)
    int8_in = term > 100
    x, wq, b, ws, ins, tops = cases.conv_case(len(name), c, h, w, outc, kernel, 1, term, True, int8_in)
    d = oracle.make_desc((c, h, w), outc, kernel, (1, 1), stride, pads, 0.0, 1, 1, term, act, (0.0, 6.0))
    want, wacc = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0], None if tops is None else tops[0], want_acc=True)
    got, gacc = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, kernel, (1, 1), stride, pads, 0.0, 1, term, act, (0.0, 6.0), want_acc=True)
    assert np.array_equal(gacc[0], wacc)
    assert np.array_equal(got[0], want)
    fast = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, kernel, (1, 1), stride, pads, 0.0, 1, term, act, (0.0, 6.0), path="nhwc")
    assert np.array_equal(fast[0], want)
    if act in (1, 3):
        assert got.min() >= 0


@pytest.mark.parametrize("name,c,h,w,outc,kernel,stride,pads,term,act,batch", [
    ("single-layer config 3x3 64->64 @56", 64, 56, 56, 64, (3, 3), (1, 1), (1, 1, 1, 1), 1, 1, 1),
    ("same, batch 3, requantised output", 64, 20, 20, 64, (3, 3), (1, 1), (1, 1, 1, 1), 101, 3, 3),
    ("1x1 256->128 @28 (rows are the pixels themselves)", 256, 28, 28, 128, (1, 1), (1, 1), (0, 0, 0, 0), 2, 0, 2),
    ("1x1/2 96->100 @28 (channel tails on both sides)", 96, 28, 28, 100, (1, 1), (2, 2), (0, 0, 0, 0), 1, 2, 1),
    ("3x3/2 20->48 @33 SAME_UPPER (20 channels in 32)", 20, 33, 33, 48, (3, 3), (2, 2), (-233, -233, -233, -233), 1, 1, 2),
    ("5x3 dilated 16->64 @40x30", 16, 30, 40, 64, (5, 3), (1, 1), (4, 4, 2, 2), 1, 0, 1),
    ("3x3 512->512 @7 (K split over workgroups)", 512, 7, 7, 512, (3, 3), (1, 1), (1, 1, 1, 1), 1, 1, 1),
    ("3x3 64->96 @12 requantised, batch 2 (K split three ways, a partly filled last tile)", 64, 12, 12, 96, (3, 3), (1, 1), (1, 1, 1, 1), 101, 1, 2),
    ("1x1 512->64 @9 (rows are the pixels, K split)", 512, 9, 9, 64, (1, 1), (1, 1), (0, 0, 0, 0), 1, 0, 1),
])
@pytest.mark.parametrize("dtype", [np.float32, np.float16], ids=["fp32", "fp16"])
def test_convolution_one_launch_from_float_blob(rt, name, c, h, w, outc, kernel, stride, pads, term, act, batch, dtype):
    """The layer's Quantize pass inside the convolution kernel (fp32 and fp16 blobs): every output bit for bit the oracle's
    quantise-then-convolve, including inputs that meet float2int8's ties and the out-of-range rule."""
    _say("conv from float", name, np.dtype(dtype).name)
    dil = (2, 2) if "dilated" in name else (1, 1)
    x, wq, b, ws, ins, tops = cases.conv_case(len(name) + batch, c, h, w, outc, kernel, 1, term, True, False, batch=batch)
    x = x.astype(dtype).astype(F)  # the values the device will see
    edge = np.array([0.5, -0.5, 1.5, -2.5, 126.5, -126.5, 127.49, 300.0, -300.0, 0.49999997, -0.49999997], F) / ins[0]
    x.reshape(-1)[: edge.size] = edge.astype(dtype).astype(F)
    if dtype == np.float32:
        x.reshape(-1)[edge.size: edge.size + 4] = [np.inf, -np.inf, np.nan, 3e38]
    ap = (0.1, 0.0) if act == 2 else (0.0, 6.0)
    d = oracle.make_desc((c, h, w), outc, kernel, dil, stride, pads, 0.0, 1, 1, term, act, ap)
    want = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None if tops is None else tops[0]) for i in range(batch)])
    got = rt.conv_channels_last(x, wq, b, ws, ins, tops, outc, kernel, dil, stride, pads, 0.0, 1, term, act, ap, from_float=dtype)
    assert np.array_equal(got, want, equal_nan=True)


def test_convolution_one_launch_from_float_blob_with_the_fused_tail(rt):
    c, hw, outc = 64, 14, 64
    x, wq, b, ws, ins, tops = cases.conv_case(5, c, hw, hw, outc, (3, 3), 1, 1, True, False, batch=2)
    rng = np.random.default_rng(6)
    res = rng.uniform(-1, 1, (2, outc, hw, hw)).astype(F)
    d = oracle.make_desc((c, hw, hw), outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 1, 1, 0, (0.0, 0.0))
    conv = np.stack([oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], None) for i in range(2)])
    want = np.maximum(conv + res, 0).astype(F)
    q_scale = F(9.5)
    want_q = oracle.quantize(want.reshape(2 * outc, -1), [q_scale]).reshape(want.shape)
    got, got_q = rt.conv_channels_last(x, wq, b, ws, ins, None, outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 1, 0, (0.0, 0.0),
                                       residual=res, relu_after=True, quantise_scale=q_scale, from_float=np.float32)
    assert np.array_equal(got, want) and np.array_equal(got_q, want_q)


def test_convolution_from_float_refuses_what_needs_its_own_quantize_pass(rt):
    import ctypes as C
    import ncnn_amd
    from ncnn_amd.hip import ConvDesc, lib
    # a non-zero border value, a workgroup's share of the operands beyond the LDS budget, a grouped layer
    border = ConvDesc(56, 56, 64, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 3.0, 1)
    deep = ConvDesc(112, 112, 2048, 1, 64, 1, 1, 1, 1, 1, 1, 0, 0, 0, 0, 0.0, 1)
    grouped = ConvDesc(56, 56, 64, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0.0, 2)
    ok = ConvDesc(56, 56, 64, 1, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0.0, 1)
    split = ConvDesc(7, 7, 512, 1, 512, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0.0, 1)
    assert [lib().ncnnhip_conv_from_float_supported(C.byref(d)) for d in (border, deep, grouped, ok, split)] == [0, 0, 0, 1, 1]
    need = C.c_size_t()
    assert lib().ncnnhip_conv_from_float_workspace_bytes(C.byref(split), C.byref(need)) == 0 and need.value > 0
    assert lib().ncnnhip_conv_from_float_workspace_bytes(C.byref(border), C.byref(need)) != 0
    x, wq, b, ws, ins, tops = cases.conv_case(1, 64, 56, 56, 64, (3, 3), 1, 1, True, False)
    with pytest.raises(ValueError):
        rt.conv_channels_last(x, wq, b, ws, ins, None, 64, (3, 3), pads=(1, 1, 1, 1), pad_value=3.0, from_float=np.float32)


def test_convolution_batch_equals_per_sample_loop(rt):
    # ncnn runs a batch as a per-sample loop (src/net.cpp:654-700); the folded launch must match it
    x, wq, b, ws, ins, tops = cases.conv_case(77, 16, 14, 14, 40, (3, 3), 1, 101, True, False, batch=3)
    d = oracle.make_desc((16, 14, 14), 40, (3, 3), pads=(1, 1, 1, 1), bias_term=1, int8_scale_term=101, activation_type=1)
    got = rt.conv_layer(x, wq, b, ws, ins, tops, 40, (3, 3), pads=(1, 1, 1, 1), term=101, act=1)
    for i in range(3):
        assert np.array_equal(got[i], oracle.convolution_int8(d, x[i], wq, b, ws, ins[0], tops[0]))


# ----------------------------------------------------------------------------- depthwise / group
@pytest.mark.parametrize("c,outc,group,h,w,stride", [(6, 6, 6, 9, 10, (1, 1)), (32, 32, 32, 56, 56, (1, 1)), (96, 96, 96, 28, 28, (2, 2)),
                                                      (6, 12, 3, 9, 10, (1, 1)), (8, 4, 2, 12, 12, (2, 2)), (64, 64, 4, 14, 14, (1, 1))])
@pytest.mark.parametrize("term,act,int8_in", [(1, 0, False), (101, 3, True), (102, 1, False), (2, 3, False)])
def test_depthwise_and_group_bit_exact(rt, c, outc, group, h, w, stride, term, act, int8_in):
    _say("dw/group", c, outc, group, h, w, stride, term, act, int8_in)
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc + group + term, c, h, w, outc, (3, 3), group, term, True, int8_in, by_group=True)
    if term in (2, 102):
        ws[:] = ws[0]
    d = oracle.make_desc((c, h, w), outc, (3, 3), (1, 1), stride, (1, 1, 1, 1), 0.0, 1, group, term, act, (0.0, 6.0))
    want, wacc = oracle.convolutiondepthwise_int8(d, x[0], wq, b, ws, ins, tops, want_acc=True)
    got, gacc = rt.conv_layer(x[0], wq, b, ws, ins, tops, outc, (3, 3), (1, 1), stride, (1, 1, 1, 1), 0.0, group, term, act, (0.0, 6.0), want_acc=True)
    assert np.array_equal(gacc[0], wacc)
    assert got.dtype == want.dtype and np.array_equal(got[0], want)


def test_depthwise_5x5_dilated_generic_kernel(rt):
    x, wq, b, ws, ins, tops = cases.conv_case(91, 8, 15, 13, 8, (5, 3), 8, 101, True, True, by_group=True)
    d = oracle.make_desc((8, 15, 13), 8, (5, 3), (2, 1), (1, 2), (-233,) * 4, 0.0, 1, 8, 101, 1)
    want = oracle.convolutiondepthwise_int8(d, x[0], wq, b, ws, ins, tops)
    got = rt.conv_layer(x[0], wq, b, ws, ins, tops, 8, (5, 3), (2, 1), (1, 2), (-233,) * 4, 0.0, 8, 101, 1)
    assert np.array_equal(got[0], want)


def test_invalid_group_returns_minus_100(rt):
    """6 channels in 4 groups: ConvolutionDepthWise::forward_int8 returns -100 (src/layer/convolutiondepthwise.cpp:433-437),
    and so does the launch (the scale tables are given per output channel, so that folding them is not what fails)."""
    import ncnn_amd
    x, wq, b, ws, ins, tops = cases.conv_case(1, 6, 5, 5, 6, (3, 3), 6, 1, False, True, by_group=True)
    with pytest.raises(ncnn_amd.NcnnHipError) as e:
        rt.conv_layer(x[0], wq, b, np.ones(6, F), np.ones(1, F), None, 6, (3, 3), group=4)
    assert e.value.code == -100


# ----------------------------------------------------------------------------- inner product
@pytest.mark.parametrize("rows,k,n,act,bias,int8_in", [(1, 2048, 1000, 0, True, False), (1, 1280, 1000, 0, True, True), (1, 33, 7, 1, False, False),
                                                        (5, 64, 10, 3, True, False), (16, 512, 300, 0, True, False), (32, 2048, 1000, 0, True, False), (13, 520, 37, 1, True, True), (70, 100, 130, 1, True, True)])
def test_innerproduct_bit_exact(rt, rows, k, n, act, bias, int8_in):
    _say("innerproduct", rows, k, n, act, bias, int8_in)
    rng = np.random.default_rng(rows + k + n)
    x = rng.uniform(-1, 1, (rows, k)).astype(F)
    in_scale = F(127) / np.abs(x).max()
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(10, 20, n).astype(F)
    ws[1 % n] = 0
    b = rng.uniform(-1, 1, n).astype(F) if bias else None
    if int8_in:
        x = oracle.quantize(x, [in_scale])
    want, wacc = oracle.innerproduct_int8(x, wq, b, ws, in_scale, act, (0.0, 6.0), want_acc=True)
    got, gacc = rt.innerproduct_layer(x, wq, b, ws, in_scale, act, (0.0, 6.0), want_acc=True)
    assert np.array_equal(gacc, wacc) and np.array_equal(got, want)


# ----------------------------------------------------------------------------- block quant
def _bq_check(got, a, packed, scales, bits, block, ins=None, c=None, bt=-1, alpha=1.0, beta=1.0):
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins, c, bt, alpha, beta)
    ref = oracle.gemm_blockquant(a, packed, scales, bits, block, ins, c, bt, alpha, beta)
    tol = 1e-5 * floor + 1e-30
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) / tol))
    assert np.all(np.abs(got - val) <= tol), float(np.max(np.abs(got - val) / tol))


@pytest.mark.parametrize("bits,block,m,n,k,bt,in_sc", [
    (8, 64, 1, 24, 256, -1, False), (8, 64, 4, 16, 200, 4, False), (4, 32, 3, 9, 100, 3, True), (6, 128, 2, 7, 300, 1, True),
    (8, 32, 16, 8, 64, 0, False), (4, 64, 1, 5, 65, 2, False), (8, 128, 5, 33, 1024, 4, True), (8, 64, 3, 10, 4096 + 16, -1, False),
    # 32 rows and more: the fp32 matrix-core kernel (ragged tiles in both directions, every C broadcast, input scales)
    (8, 64, 32, 64, 64, -1, False), (8, 64, 70, 100, 256, 4, True), (8, 32, 129, 65, 96, 3, False), (8, 128, 64, 31, 1024, 1, True),
    (8, 64, 200, 130, 2048, 0, False), (8, 64, 33, 8, 4096 + 32, 2, False),
    # 4- and 6-bit fields with K % 16 == 0: the streaming kernel (8 / 12 bytes per 16 weights) and the matrix-core kernel
    (4, 32, 1, 24, 256, -1, False), (4, 64, 4, 40, 1024, 4, True), (6, 64, 3, 17, 512, 1, False), (6, 128, 2, 33, 4096 + 16, -1, True),
    (4, 128, 70, 100, 256, 3, True), (6, 32, 40, 65, 96, 0, False), (4, 32, 16, 8, 11008, -1, False), (6, 64, 129, 31, 1024, 4, False)])
def test_blockquant_small(rt, bits, block, m, n, k, bt, in_sc):
    _say("blockquant", bits, block, m, n, k, bt, in_sc)
    rng = np.random.default_rng(bits + block + m + n + k)
    a = rng.standard_normal((m, k), dtype=F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    ins = (0.75 + (np.arange(k) % 5) * 0.15).astype(F) if in_sc else None
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    got = rt.gemm_blockquant(a, packed, scales, bits, block, ins, c, bt, 1.25, 0.5)
    _bq_check(got, a, packed, scales, bits, block, ins, c, bt, 1.25, 0.5)


@pytest.mark.parametrize("m", [1, 4, 16])
@pytest.mark.parametrize("n,k", [(512, 4096), (256, 11008)])
def test_blockquant_decode_shapes_fp32_and_fp16_activations(rt, m, n, k):
    # the decode configuration's K with a reduced N (rows are independent, so N only scales the work)
    _say("blockquant decode", m, n, k)
    a, packed, scales = cases.blockquant_case(m * 7 + n + k, m, n, k)
    got32 = rt.gemm_blockquant(a, packed, scales, 8, 64)
    _bq_check(got32, a, packed, scales, 8, 64)
    got16 = rt.gemm_blockquant(a.astype(np.float16), packed, scales, 8, 64)
    assert np.array_equal(got16, got32)  # fp16-representable activations: both entry points see the same numbers


@pytest.mark.parametrize("bits", [4, 6])
def test_blockquant_low_bit_decode_shape_fp16_activations(rt, bits):
    _say("blockquant decode", bits)
    m, n, k = 4, 256, 4096
    rng = np.random.default_rng(bits)
    a = rng.standard_normal((m, k)).astype(np.float16).astype(F)  # fp16-representable: both entry points see the same numbers
    packed, scales = oracle.blockquant_pack((rng.standard_normal((n, k)) * 0.02).astype(F), bits, 32)
    got32 = rt.gemm_blockquant(a, packed, scales, bits, 32)
    _bq_check(got32, a, packed, scales, bits, 32)
    got16 = rt.gemm_blockquant(a.astype(np.float16), packed, scales, bits, 32)
    assert np.array_equal(got16, got32)


@pytest.mark.parametrize("m,n,k,block,bt", [(1, 512, 4096, 64, -1), (4, 256, 4096, 64, 4), (16, 256, 4096, 64, 3), (16, 250, 11008, 64, -1),
                                            (3, 37, 208, 64, 1), (1, 16, 64, 64, 0), (20, 64, 1024, 128, 2), (7, 100, 4096 + 48, 128, -1),
                                            # more than 512 tiles of 16 rows: workgroups stay and walk the tiles (ragged last tile, odd K blocks)
                                            (1, 11008, 4096, 64, -1), (4, 8200 + 8, 4096, 64, -1), (4, 8200 + 5, 1024 + 64, 64, 4), (16, 9000, 512, 128, 3), (2, 16400, 192, 64, 1),
                                            # every wavefront count of the kernel that requests a wavefront's whole share at once (8, 15 and 16 wavefronts of 16 / 12 /
                                            # 16 K blocks, a last wavefront with a single block and with none), rows through LDS (up to 4) and in registers (5 to 16),
                                            # and K beyond its reach (the ring kernel takes over)
                                            (2, 48, 8192, 64, -1), (1, 33, 12288, 64, 4), (3, 40, 11008 + 16, 64, 1), (4, 32, 16384, 128, -1), (1, 32, 16384 + 64, 64, -1),
                                            (9, 40, 8192, 64, 1), (5, 24, 4096 + 64, 64, -1), (12, 40, 12288, 64, -1), (16, 4096, 4096, 64, 4), (2, 20, 1024 + 16, 64, 3),
                                            # from 1024 tiles up, 5 to 16 rows take two tiles per workgroup: an odd tile count with a ragged last tile, an even one, K inside a step
                                            (16, 16384 + 11, 512, 64, 3), (9, 16384 + 32, 1024 + 48, 128, 4), (5, 16400, 4096, 64, -1)])
def test_blockquant_packed_matrix_core_path(rt, m, n, k, block, bt):
    _say("blockquant packed", m, n, k, block, bt)
    a, packed, scales = cases.blockquant_case(m + n + k + block, m, n, k, 8, block)
    rng = np.random.default_rng(bt + 50)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    pw, pd = rt.blockquant_pack(packed, scales, block)
    got = rt.gemm_blockquant_packed(a.astype(np.float16), pw, pd, n, c, bt, 0.75, 1.5, bits=8, block=block)
    _bq_check(got, a, packed, scales, 8, block, None, c, bt, 0.75, 1.5)


@pytest.mark.parametrize("bits,block,m,n,k,bt", [
    # every field width and block size of the layout whose steps are split in two halves, at one, few (through LDS) and up to 16 (registers) activation rows
    (4, 64, 1, 512, 4096, -1), (4, 32, 1, 256, 4096, 4), (4, 128, 1, 256, 4096, -1), (6, 64, 1, 512, 4096, -1), (6, 32, 1, 256, 4096, 0), (6, 128, 1, 100, 4096, -1),
    (8, 32, 1, 512, 4096, -1), (4, 64, 2, 48, 4096, 1), (6, 32, 3, 40, 4096, 2), (8, 32, 4, 256, 4096, 4), (4, 32, 4, 250, 4096, 3), (6, 64, 4, 64, 4096, -1),
    (4, 64, 16, 256, 4096, 3), (4, 32, 16, 250, 4096, -1), (6, 64, 16, 128, 4096, 4), (6, 32, 9, 40, 4096, 1), (8, 32, 16, 256, 4096, -1), (4, 128, 5, 24, 4096 + 64, -1),
    # 8, 15 and 16 wavefronts; a last wavefront with one step and with none; K that ends inside a step and inside a block
    (4, 64, 1, 40, 8192, -1), (6, 64, 2, 33, 12288, 4), (4, 32, 3, 40, 11008 + 16, 1), (8, 32, 4, 32, 16384, -1), (6, 128, 1, 32, 16384, -1), (4, 64, 1, 250, 11008, -1),
    (4, 64, 3, 37, 208, 1), (6, 32, 1, 16, 64, 0), (8, 32, 2, 20, 1024 + 16, 3), (4, 128, 7, 100, 4096 + 48, -1), (6, 64, 12, 40, 8192, -1), (4, 32, 16, 64, 96, 2),
    # more than 16 rows (one pass per 16), and more than 4 rows with K beyond 8192 (four at a time)
    (4, 64, 20, 64, 1024, 2), (6, 32, 33, 40, 512, 3), (4, 64, 9, 40, 12288, 1), (6, 64, 16, 24, 16384, 3), (8, 32, 7, 40, 11008, 4),
    # many tiles; from 1024 up two tiles per workgroup at 5 to 16 rows
    (4, 64, 1, 11008, 4096, -1), (6, 64, 4, 8200 + 5, 1024 + 64, 4), (4, 32, 16, 9000, 512, 3), (4, 64, 16, 16384 + 11, 512, -1), (6, 32, 7, 16400, 256 + 16, 3),
    (8, 32, 12, 16384 + 40, 1024, 4)])
def test_blockquant_packed_low_bit_widths_and_blocks_of_32(rt, bits, block, m, n, k, bt):
    _say("blockquant packed", bits, block, m, n, k, bt)
    from ncnn_amd import synth
    a, packed, scales = synth.blockquant_operands(bits + block + m + n + k, m, n, k, bits, block)  # activations are fp16-representable
    rng = np.random.default_rng(bt + 51)
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
    got = rt.gemm_blockquant_packed(a.astype(np.float16), pw, pd, n, c, bt, 0.75, 1.5, bits=bits, block=block)
    _bq_check(got, a, packed, scales, bits, block, None, c, bt, 0.75, 1.5)


@pytest.mark.parametrize("bits,block,m,n,k,bt,in_sc", [
    # fp32 activations on the packed weights (three bf16 planes): one, two and four rows per pass, more rows in several passes
    (8, 64, 1, 512, 4096, -1, False), (8, 64, 2, 100, 4096, 4, True), (8, 64, 4, 256, 4096, 3, False), (8, 128, 3, 40, 4096, 1, True), (8, 64, 16, 64, 4096, 3, False),
    (4, 64, 1, 256, 4096, -1, False), (4, 32, 4, 250, 4096, 4, True), (6, 64, 1, 128, 4096, -1, True), (6, 32, 3, 40, 4096, 2, False), (8, 32, 4, 64, 4096, -1, False),
    (4, 128, 7, 40, 2048 + 48, 0, True),
    # K up to 8192: two rows per pass; beyond: one; K that ends inside a step; a last wavefront without work
    (8, 64, 4, 48, 8192, -1, False), (4, 64, 3, 33, 8192, 1, True), (8, 64, 2, 40, 11008, -1, False), (4, 32, 1, 40, 11008 + 16, 4, False), (6, 64, 4, 32, 12288, 3, True),
    (8, 64, 1, 32, 16384, -1, False), (6, 128, 2, 20, 16384, 1, False), (8, 64, 3, 37, 208, 1, True), (4, 64, 1, 16, 64, 0, False), (8, 32, 2, 20, 1024 + 16, 3, False),
    # many tiles
    (8, 64, 1, 11008, 4096, -1, False), (4, 64, 4, 8200 + 5, 1024 + 64, 4, True)])
def test_blockquant_packed_fp32_activations(rt, bits, block, m, n, k, bt, in_sc):
    _say("blockquant packed fp32", bits, block, m, n, k, bt, in_sc)
    from ncnn_amd import synth
    a, packed, scales = synth.blockquant_operands(bits + block + m + n + k + 1, m, n, k, bits, block, half_exact=False)  # full fp32 mantissas
    a[0, : min(k, 8)] = [3.0e-30, -1.5e30, 1.0, -1.0, 1.0 + 2.0 ** -23, 2.0 ** -100, 0.0, -7.25e12][: min(k, 8)]  # the far ends of the exponent range
    rng = np.random.default_rng(bt + 52)
    ins = rng.uniform(0.5, 1.5, k).astype(F) if in_sc else None
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
    got = rt.gemm_blockquant_packed(a, pw, pd, n, c, bt, 0.75, 1.5, bits=bits, block=block, in_scales=ins)
    _bq_check(got, a, packed, scales, bits, block, ins, c, bt, 0.75, 1.5)


@pytest.mark.parametrize("act,bits,block,m,k,ns,in_sc", [
    # the decode shapes' siblings: gate + up, q + k + v; fp16 and fp32 activations; every layout; ragged N; one matrix; eight
    ("fp16", 8, 64, 1, 4096, (176, 160), False), ("fp16", 8, 64, 16, 1024, (64, 100, 37), False), ("fp16", 4, 32, 4, 2048 + 16, (48, 16, 250), False),
    ("fp16", 6, 128, 7, 512, (33,), False), ("fp32", 8, 64, 1, 4096, (176, 160), False), ("fp32", 8, 64, 4, 4096, (40, 256, 100), True),
    ("fp32", 4, 64, 2, 1024, (16,) * 8, True), ("fp32", 6, 32, 3, 256, (300, 20), False),
    # shapes the one-pass kernel does not take: matrix by matrix behind the same call
    ("fp16", 8, 64, 20, 1024, (64, 48), False), ("fp32", 8, 64, 4, 8192, (32, 48), False)])
def test_blockquant_packed_multi_equals_the_single_calls_and_the_oracle(rt, act, bits, block, m, k, ns, in_sc):
    """Several weight matrices on the same activation rows in one launch: each output is bit for bit what the single-matrix entry
    gives (same kernel, same order of additions; the workgroup only finds its matrix differently), and within the usual bound of the
    oracle's Gemm::forward_weight_block_quantize (src/layer/gemm.cpp:425-483) per matrix -- with a different C, alpha and beta each."""
    _say("blockquant multi", act, bits, block, m, k, ns, in_sc)
    from ncnn_amd import synth
    rng = np.random.default_rng(len(ns) + m + k)
    a = None
    mats, refs = [], []
    for i, n in enumerate(ns):
        ai, packed, scales = synth.blockquant_operands(bits + block + m + n + k + i, m, n, k, bits, block, half_exact=(act == "fp16"))
        a = ai if a is None else a
        bt = (-1, 4, 0, 3, 1, 2)[i % 6]
        c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)), 4: rng.normal(size=(1, n))}[bt]
        c = None if c is None else c.astype(F)
        alpha, beta = float(F(0.5 + 0.25 * i)), float(F(1.5 - 0.125 * i))
        pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
        mats.append((pw, pd, n, c, bt, alpha, beta))
        refs.append((packed, scales, c, bt, alpha, beta))
    ins = rng.uniform(0.5, 1.5, k).astype(F) if in_sc else None
    x = a.astype(np.float16) if act == "fp16" else a
    got = rt.gemm_blockquant_packed_multi(x, mats, bits=bits, block=block, in_scales=ins)
    for i, (pw, pd, n, c, bt, alpha, beta) in enumerate(mats):
        single = rt.gemm_blockquant_packed(x, pw, pd, n, c, bt, alpha, beta, bits=bits, block=block, in_scales=ins)
        assert np.array_equal(got[i], single), "matrix %d differs from the single-matrix call" % i
        packed, scales = refs[i][0], refs[i][1]
        _bq_check(got[i], a, packed, scales, bits, block, ins, c, bt, alpha, beta)


@pytest.mark.parametrize("bits,block,m,n,k,bt,in_sc", [
    # the tiled form for many rows: ragged in rows (64), weight rows (128 per workgroup, 16 per tile) and K (64); every layout; C broadcasts; input scales
    (8, 64, 64, 128, 64, -1, False), (8, 64, 70, 100, 256, 4, True), (8, 32, 129, 65, 96, 3, False), (8, 128, 64, 31, 1024, 1, True), (8, 64, 200, 130, 2048, 0, False),
    (8, 64, 33, 8, 4096 + 32, 2, False), (4, 128, 70, 100, 256, 3, True), (6, 32, 40, 65, 96, 0, False), (6, 64, 129, 31, 1024, 4, False), (4, 64, 1, 300, 208, -1, False),
    (4, 32, 300, 260, 1024 + 16, 4, True), (8, 64, 1500, 1024, 1024, 4, False),
    # up to 48 rows (96 over many weight rows): the weight-streaming form on pre-split operand fragments, 16 rows per pass (one and two passes, ragged rows,
    # 1 to 8 wavefronts, a last wavefront with fewer steps, K that ends inside a step)
    (8, 64, 5, 100, 256, -1, False), (8, 64, 16, 256, 4096, 3, False), (4, 32, 9, 40, 1024 + 16, 1, True), (6, 64, 31, 33, 512, 4, False), (8, 32, 17, 20, 96, 2, False),
    (8, 128, 12, 24, 4096, -1, True), (4, 64, 16, 4100, 2048 + 48, 4, False), (6, 128, 8, 16, 64, 0, False), (8, 64, 20, 40, 3072 + 64, 3, True), (8, 64, 16, 24, 4096 + 64, -1, False),
    # K beyond 4096: rounds of 8 wavefronts x 8 steps (a last round with idle wavefronts, with a ragged wavefront)
    (4, 64, 9, 40, 11008, 1, False), (8, 64, 20, 33, 8192 + 16, 4, True), (6, 64, 5, 20, 12288, -1, False), (8, 128, 16, 250, 11008, 3, False)])
def test_blockquant_packed_rows_kernel(rt, bits, block, m, n, k, bt, in_sc):
    _say("blockquant packed rows", bits, block, m, n, k, bt, in_sc)
    from ncnn_amd import synth
    a, packed, scales = synth.blockquant_operands(bits + block + m + n + k + 2, m, n, k, bits, block, half_exact=False)
    rng = np.random.default_rng(bt + 53)
    ins = rng.uniform(0.5, 1.5, k).astype(F) if in_sc else None
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)),
         4: rng.normal(size=(1, n))}[bt]
    c = None if c is None else c.astype(F)
    pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
    got = rt.gemm_blockquant_packed(a, pw, pd, n, c, bt, 0.75, 1.5, bits=bits, block=block, in_scales=ins, rows_kernel=True)
    _bq_check(got, a, packed, scales, bits, block, ins, c, bt, 0.75, 1.5)


@pytest.mark.parametrize("bits,block", [(8, 64), (8, 32), (6, 64), (4, 128)])
def test_blockquant_packed_fp32_split_keeps_all_24_bits(rt, bits, block):
    """One non-zero activation per row, power-of-two scales: an output is a single product x * q * 2^-2, known to float64
    exactly, and the three partial products of the bf16 split add up with at most two roundings.  A split that lost its
    lowest plane would be off by up to 2^-16, one that lost the middle plane by 2^-8; the sum's tolerance of the other
    tests (1e-5 of sum |a w|) would not notice the former."""
    k, n, m = 256, 48, 4
    rng = np.random.default_rng(bits * 10 + block)
    qmax = (1 << (bits - 1)) - 1
    q = rng.integers(-qmax, qmax + 1, (n, k))
    w = (q * 0.25).astype(F)  # quantises back to q with scale 4 when a block holds +-qmax; force that
    w[:, ::block] = qmax * 0.25
    packed, scales = oracle.blockquant_pack(w, bits, block)
    assert np.all(scales == F(4.0))
    qq = npref.blockquant_unpack_all(packed, k, bits)
    a = np.zeros((m, k), F)
    pos = [5, 64 + 40, 128 + 17, 255]
    vals = [F(1.0) + F(2.0 ** -23), F(-3.1415927e-20), F(16777215.0 * 2.0 ** 40), F(0.7071068)]
    for i in range(m):
        a[i, pos[i]] = vals[i]
    pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
    want = np.stack([float(vals[i]) * qq[:, pos[i]].astype(np.float64) * 0.25 for i in range(m)])
    for rows_kernel in (False, True):  # the few-row kernel (split while staging in LDS) and the tiled one (split by a pass of its own)
        got = rt.gemm_blockquant_packed(a, pw, pd, n, bits=bits, block=block, rows_kernel=rows_kernel).astype(np.float64)
        assert np.all(np.abs(got - want) <= np.abs(want) * 2.0 ** -22), (rows_kernel, float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-300))))


@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (4096, 11008)])
@pytest.mark.parametrize("m,act", [(1, "fp16"), (4, "fp16"), (16, "fp16"), (1, "fp32"), (4, "fp32"), (16, "fp32"), (64, "fp32"), (200, "fp32")])
def test_blockquant_full_size_properties(rt, n, k, m, act):
    """The decode configuration at its full sizes, through size-independent properties (no oracle pass over 45 M weights per case):
    doubling the activations doubles every output exactly (a power of two commutes with the split, the products and the sums);
    permuting the activation rows permutes the output rows bit for bit (a row's result does not depend on its neighbours or on its
    position modulo the kernel's row grouping... only on which kernel runs, which the row count fixes); and 48 sampled weight rows agree
    with the float64 value within the usual 1e-5 of sum |a w|."""
    _say("blockquant full size", n, k, m, act)
    import ncnn_amd
    from ncnn_amd import hip, synth
    a, packed, scales = synth.blockquant_operands(n + k + m, m, n, k, 8, 64, half_exact=(act == "fp16"))
    pw, pd = rt.blockquant_pack(packed, scales, 64)
    dw_, dd = rt.up(pw), rt.up(pd)

    def run(x):
        x = x.astype(np.float16) if act == "fp16" else x
        # the weights stay on the device between the calls; only the activations change
        m_, k_ = x.shape
        da = rt.up(np.ascontiguousarray(x))
        dout = ncnn_amd.DeviceBuffer.empty((m_, n), np.float32)
        lib = hip.lib()
        if act == "fp16":
            hip.check(lib.ncnnhip_gemm_blockquant_packed_f16a(da.ptr, k_, m_, n, k_, dw_.ptr, dd.ptr, 8, 64, None, -1, 1.0, 1.0, dout.ptr, n, rt.stream))
        elif m_ >= 5:
            wsb = C.c_size_t()
            hip.check(lib.ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(m_, k_, C.byref(wsb)))
            ws = ncnn_amd.DeviceBuffer.empty((wsb.value,), np.uint8)
            hip.check(lib.ncnnhip_gemm_blockquant_packed_rows(da.ptr, k_, m_, n, k_, dw_.ptr, dd.ptr, 8, 64, None, None, -1, 1.0, 1.0, dout.ptr, n, ws.ptr, wsb.value,
                                                              rt.stream))
        else:
            hip.check(lib.ncnnhip_gemm_blockquant_packed(da.ptr, k_, m_, n, k_, dw_.ptr, dd.ptr, 8, 64, None, None, -1, 1.0, 1.0, dout.ptr, n, rt.stream))
        return dout.to_numpy(rt.stream)

    out = run(a)
    assert np.array_equal(run(a * F(2)), out * F(2))
    if m > 1:
        perm = np.random.default_rng(m).permutation(m)
        if m > 16:  # 16-row groups share a pass / a tile: keep rows inside their group of 16 so that the same lanes' sums are compared
            perm = np.concatenate([g0 + np.random.default_rng(g0).permutation(min(16, m - g0)) for g0 in range(0, m, 16)])
        assert np.array_equal(run(a[perm]), out[perm])
    cols = np.random.default_rng(n).choice(n, 48, replace=False)
    val, floor = npref.blockquant_gemm_f64(a, packed[cols], scales[cols], 8, 64)
    assert np.all(np.abs(out[:, cols] - val) <= 1e-5 * floor + 1e-30)


def test_blockquant_exact_on_power_of_two_data(rt):
    k, n, m = 128, 6, 2
    rng = np.random.default_rng(3)
    q = rng.integers(-127, 128, (n, k)).astype(np.int8)
    scales = np.full((n, k // 64), F(4.0), F)
    a = rng.integers(-8, 9, (m, k)).astype(F)
    got = rt.gemm_blockquant(a, q.view(np.uint8), scales, 8, 64)
    assert np.array_equal(got, ((a.astype(np.int64) @ q.astype(np.int64).T) * 0.25).astype(F))


# ---- attention core (src/layer/multiheadattention.cpp:776-866) ----------------------------------------------------------

@pytest.mark.parametrize("heads,hd,src,dst,mask", [(4, 16, 9, 9, None), (3, 24, 7, 130, "2d"), (8, 64, 5, 300, "3d"), (2, 32, 1, 1, None), (1, 8, 70, 3, "2d"),
                                                    # head dimensions of the matrix-core kernel: ragged query blocks and key tiles, one to many tiles per wavefront
                                                    (2, 96, 40, 70, "2d"), (1, 128, 33, 257, None), (4, 64, 100, 129, "3d"), (2, 64, 64, 1024, None), (3, 32, 1, 515, "2d"), (16, 64, 1, 1500, None), (2, 128, 33, 4100, "3d"),
                                                    # many workgroups (two and a half per compute unit)
                                                    (16, 64, 1500, 1500, None), (16, 32, 1920, 300, "2d"),
                                                    # one to four queries on 256 keys and more: the streaming kernels (64 keys per workgroup + merge), head
                                                    # dimensions of any size, partial last chunks, rows that are / are not 16-byte aligned
                                                    (4, 40, 3, 700, "3d"), (2, 200, 4, 260, None), (5, 64, 2, 1024, "2d"), (1, 256, 4, 301, None), (3, 7, 1, 257, "2d")])
def test_attention_core_matches_float64(rt, heads, hd, src, dst, mask):
    rng = np.random.default_rng(heads * 100 + dst)
    e = heads * hd
    q = (rng.normal(0, 1, (src, e)) / np.sqrt(hd)).astype(F)
    kt = rng.normal(0, 1, (e, dst)).astype(F)
    vt = rng.normal(0, 1, (e, dst)).astype(F)
    m = None
    if mask:
        shape = (src, dst) if mask == "2d" else (heads, src, dst)
        m = rng.normal(0, 1, shape).astype(F)
        drop = rng.random(shape) < 0.3
        drop[..., 0] = False
        m[drop] = F(-1e30)
    got = rt.attention(q, kt, vt, heads, m)
    assert np.array_equal(got.shape, (src, e))
    plain = rt.attention(q, kt, vt, heads, m, use_workspace=False)  # without the scratch the keys are not split over workgroups
    want = np.empty((src, e))
    for h in range(heads):
        sl = slice(h * hd, (h + 1) * hd)
        s = q[:, sl].astype(np.float64) @ kt[sl].astype(np.float64)
        if m is not None:
            s = s + (m if m.ndim == 2 else m[h]).astype(np.float64)
        s = np.exp(s - s.max(axis=1, keepdims=True))
        want[:, sl] = (s / s.sum(axis=1, keepdims=True)) @ vt[sl].astype(np.float64).T
    # fp32 sums over head_dim and dst terms of O(1) values, device expf
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    assert np.abs(plain - want).max() <= 2e-5 * max(1.0, np.abs(want).max())


@pytest.mark.parametrize("heads,hd,src,dst", [(4, 64, 37, 200), (2, 32, 1, 300), (3, 24, 5, 40)])
def test_attention_reads_strided_queries_and_scales_them_on_load(rt, heads, hd, src, dst):
    """Queries taken out of a wider row (q, k and v made by one Gemm) and multiplied by the layer's scale where they are read:
    bit for bit what the plain entry gives on the scaled queries (src/layer/multiheadattention.cpp:634 rounds the same product)."""
    rng = np.random.default_rng(heads + dst)
    e = heads * hd
    wide = rng.normal(0, 1, (src, 3 * e)).astype(F)
    kt = rng.normal(0, 1, (e, dst)).astype(F)
    vt = rng.normal(0, 1, (e, dst)).astype(F)
    scale = F(1.0 / np.sqrt(hd))
    want = rt.attention(wide[:, :e] * scale, kt, vt, heads)
    got = rt.attention(wide, kt, vt, heads, q_scale=scale)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("rows,cols,past", [(1, 64, 13), (37, 96, 0), (70, 33, 5)])
def test_transpose_pair_appends_key_and_value_columns(rt, rows, cols, past):
    rng = np.random.default_rng(rows + cols)
    wide = rng.normal(0, 1, (rows, 3 * cols)).astype(F)
    ka = rng.normal(0, 1, (cols, past + rows)).astype(F)
    va = rng.normal(0, 1, (cols, past + rows)).astype(F)
    got_k, got_v = rt.transpose_pair_into(wide, cols, 2 * cols, cols, ka, va, past)
    want_k, want_v = ka.copy(), va.copy()
    want_k[:, past:] = wide[:, cols:2 * cols].T
    want_v[:, past:] = wide[:, 2 * cols:].T
    assert np.array_equal(got_k, want_k) and np.array_equal(got_v, want_v)


@pytest.mark.parametrize("heads,hd,src,past,mask", [(4, 64, 1, 299, None), (2, 40, 3, 318, "2d"), (3, 32, 4, 255, None), (2, 64, 2, 62, "3d"), (2, 64, 40, 100, None), (3, 24, 1, 7, None)])
def test_attention_appends_the_new_keys_and_values_itself(rt, heads, hd, src, past, mask):
    """q, k and v side by side in one row per token: the call writes the new key / value columns behind the cache and attends over
    all of them - bit for bit what the separate append and the strided call give, and the cache columns stay as they were."""
    rng = np.random.default_rng(heads * 1000 + past)
    e, dst = heads * hd, past + src
    qkv = rng.normal(0, 1, (src, 3 * e + 5)).astype(F)
    kt = rng.normal(0, 1, (e, dst)).astype(F)
    vt = rng.normal(0, 1, (e, dst)).astype(F)
    m = None
    if mask:
        m = rng.normal(0, 1, (src, dst) if mask == "2d" else (heads, src, dst)).astype(F)
    scale = F(1.0 / np.sqrt(hd))
    want_kt, want_vt = kt.copy(), vt.copy()
    want_kt[:, past:] = qkv[:, e:2 * e].T
    want_vt[:, past:] = qkv[:, 2 * e:3 * e].T
    want = rt.attention(qkv, want_kt, want_vt, heads, m, q_scale=scale)
    got, got_kt, got_vt = rt.attention_append(qkv, kt, vt, heads, past, scale, m)
    assert np.array_equal(got_kt, want_kt) and np.array_equal(got_vt, want_vt)
    assert np.array_equal(got, want)
