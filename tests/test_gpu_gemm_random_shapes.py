"""Gemm, InnerProduct and block-quantised Gemm at seeded random shapes through whichever kernel the library picks, against
the oracle.

The other tests walk each kernel's own shapes; here M, N, K, the C broadcast, alpha / beta, the output transposition, the
scale form of B, the activation and the input type are drawn without looking at the kernel that takes the call (one
wavefront per row of B, the few-row kernels, the 64 / 128 / 256 wide tiles, K split over workgroups, ragged last tiles,
K below a vector), so that the rules between the kernels are crossed wherever they lie.
Int8 Gemm and InnerProduct: bit for bit (src/layer/gemm.cpp:745-966, src/layer/innerproduct.cpp:147-230).
Block-quantised Gemm: |got - ref| <= 1e-5 * sum |a * w| against the oracle and a float64 value (src/layer/gemm.cpp:339-483)."""
import os

import numpy as np
import pytest

from tests import cases, npref
from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "300"))  # NCNN_RANDOM_LAYERS=<count> widens every walk of this file


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


def _dim(rng, small, large):
    """A size: mostly small and odd, sometimes a multiple of 64, now and then large."""
    r = rng.random()
    if r < 0.45:
        return int(rng.integers(1, small + 1))
    if r < 0.75:
        return 64 * int(rng.integers(1, max(small // 64, 1) + 1))
    if r < 0.9:
        return int(rng.integers(small, large + 1))
    return 64 * int(rng.integers(max(small // 64, 1), large // 64 + 1))


def _c_operand(rng, bt, m, n):
    c = {-1: None, 0: rng.normal(size=1), 1: rng.normal(size=m), 2: rng.normal(size=(m, 1)), 3: rng.normal(size=(m, n)), 4: rng.normal(size=(1, n))}[bt]
    return None if c is None else c.astype(F)


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_gemm_int8_matches_oracle(rt, seed):
    rng = np.random.default_rng(5000 + seed)
    m, n, k = _dim(rng, 200, 1500), _dim(rng, 300, 2500), _dim(rng, 300, 4500)
    while m * n * k > 4e8:
        m, n, k = max(m * 2 // 3, 1), max(n * 2 // 3, 1), max(k * 3 // 4, 1)
    bt = _pick(rng, [-1, -1, 0, 1, 2, 3, 4, 4])
    alpha, beta = _pick(rng, [1.0, 1.0, 0.5, 1.7, -1.0]), _pick(rng, [1.0, 1.0, 2.0, 0.3, -1.0, 0.0])
    transpose, per_col = bool(rng.integers(2)), bool(rng.integers(2))
    print("[case] random gemm", seed, (m, n, k), bt, alpha, beta, transpose, per_col, flush=True)
    a, bq, sb, _ = cases.gemm_case(seed, m, n, k, per_col)
    c = _c_operand(rng, bt, m, n)
    aq, sa = oracle.gemm_quantize_rows(a)
    gq, gs = rt.gemm_quantize_rows(a)
    assert np.array_equal(gq, aq) and np.array_equal(gs, sa)
    want, wacc = oracle.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose, want_acc=True)
    got, gacc = rt.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose, want_acc=True)
    assert np.array_equal(gacc, wacc) and np.array_equal(got, want)
    # without the accumulator dump the launcher may pick another kernel: same answer
    assert np.array_equal(rt.gemm_int8(aq, bq, sa, sb, c, bt, alpha, beta, transpose), want)


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_innerproduct_matches_oracle(rt, seed):
    rng = np.random.default_rng(7000 + seed)
    rows = _pick(rng, [1, 1, 2, 3, 4, 5, 8, 16, 17, 32, 48, 49, 64, 70, 128, 200])
    k, n = _dim(rng, 300, 4500), _dim(rng, 300, 2500)
    while rows * n * k > 3e8:
        n, k = max(n * 2 // 3, 1), max(k * 3 // 4, 1)
    act, ap = _pick(rng, [(0, (0.0, 0.0)), (1, (0.0, 0.0)), (2, (0.1, 0.0)), (3, (0.0, 6.0)), (3, (-0.3, 0.4)), (6, (0.2, 0.5))])
    bias, int8_in = rng.random() < 0.8, bool(rng.integers(2))
    print("[case] random innerproduct", seed, rows, k, n, act, ap, bias, int8_in, flush=True)
    x = rng.uniform(-1, 1, (rows, k)).astype(F)
    in_scale = F(127) / np.abs(x).max()
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(10, 20, n).astype(F) * F(np.sqrt(k))
    if rng.random() < 0.3:
        ws[int(rng.integers(n))] = 0  # a zero weight scale: the reference's dequantisation scale is then 0
    b = rng.uniform(-1, 1, n).astype(F) if bias else None
    if int8_in:
        x = oracle.quantize(x, [in_scale])
    want, wacc = oracle.innerproduct_int8(x, wq, b, ws, in_scale, act, ap, want_acc=True)
    got, gacc = rt.innerproduct_layer(x, wq, b, ws, in_scale, act, ap, want_acc=True)
    assert np.array_equal(gacc, wacc) and np.array_equal(got, want)


@pytest.mark.parametrize("seed", range(COUNT // 2))
def test_random_blockquant_gemm_matches_oracle_and_float64(rt, seed):
    from ncnn_amd import synth
    rng = np.random.default_rng(9000 + seed)
    bits, block = _pick(rng, [8, 8, 4, 6]), _pick(rng, [64, 64, 32, 128])
    m = _pick(rng, [1, 1, 1, 2, 3, 4, 5, 8, 16, 17, 33, 48, 64, 100])
    n = _dim(rng, 300, 9000)
    k = 16 * int(rng.integers(1, 40)) if rng.random() < 0.4 else 64 * int(rng.integers(1, 200))  # the packed layout takes K in whole 16s
    while m * n * k > 2.5e8 or n * k > 4e7:
        n = max(n * 2 // 3, 1)
    bt = _pick(rng, [-1, -1, 0, 1, 2, 3, 4])
    half = bool(rng.integers(2))
    plain = (not half) and rng.random() < 0.35  # the entry that reads the .bin layout as it is: any K
    if plain:
        k = int(rng.integers(1, 3000))
    in_sc = (not half) and rng.random() < 0.4
    print("[case] random blockquant", seed, bits, block, (m, n, k), bt, "fp16" if half else "fp32", in_sc, "bin layout" if plain else "packed", flush=True)
    a, packed, scales = synth.blockquant_operands(seed, m, n, k, bits, block, half_exact=half)
    ins = rng.uniform(0.5, 1.5, k).astype(F) if in_sc else None
    c = _c_operand(rng, bt, m, n)
    if plain:
        got = rt.gemm_blockquant(a, packed, scales, bits, block, ins, c, bt, 0.75, 1.5)
    else:
        pw, pd = rt.blockquant_pack(packed, scales, block, bits=bits, k=k)
        got = rt.gemm_blockquant_packed(a.astype(np.float16) if half else a, pw, pd, n, c, bt, 0.75, 1.5, bits=bits, block=block, in_scales=ins)
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins, c, bt, 0.75, 1.5)
    ref = oracle.gemm_blockquant(a, packed, scales, bits, block, ins, c, bt, 0.75, 1.5)
    tol = 1e-5 * floor + 1e-30
    assert np.all(np.abs(got - ref) <= tol), float(np.max(np.abs(got - ref) / tol))
    assert np.all(np.abs(got - val) <= tol), float(np.max(np.abs(got - val) / tol))
