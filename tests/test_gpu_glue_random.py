"""The kernels between the int8 layers at seeded random sizes, through the C ABI: the layout changes (planar <-> channels
last, fp32 and int8, any channel count), Quantize on channels-last blobs (one scale or one per channel,
src/layer/quantize.cpp:48-111), ReLU / leaky ReLU, Eltwise (product, sum with and without coefficients, max; two to five
inputs, src/layer/eltwise.cpp:30-160), Softmax, windowed max pooling on int8 blobs and the global poolings with their
quantised form.  Sizes from one element to a few hundred thousand, odd ones above all.  Bit for bit except Softmax (the
device's expf and a tree sum: 1e-5 relative)."""
import os

import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "100"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


def _size(rng):
    return int(_pick(rng, [1, 2, 3, 5, 17, 63, 64, 65, 255, 1000, 4097, int(rng.integers(1, 300000))]))


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_layout_round_trip_and_quantize(rt, seed):
    rng = np.random.default_rng(23000 + seed)
    n, c = _pick(rng, [1, 1, 2, 5]), int(_pick(rng, [1, 2, 3, 4, 5, 15, 16, 17, 31, 33, 64, 100, 257, int(rng.integers(1, 600))]))
    h, w = int(rng.integers(1, 40)), int(rng.integers(1, 40))
    print("[case] random layout", seed, (n, c, h, w), flush=True)
    x = rng.normal(0, 2, (n, c, h, w)).astype(F)
    buf = rt.to_channels_last(x)
    raw = buf.to_numpy(rt.stream)
    assert raw.shape[2] % 16 == 0 and not raw[:, :, c:].any()
    assert np.array_equal(raw[:, :, :c], x.reshape(n, c, h * w).transpose(0, 2, 1))
    assert np.array_equal(rt.from_channels_last(buf, n, c, h, w), x)
    q8 = rng.integers(-128, 128, (n, c, h, w)).astype(np.int8)
    b8 = rt.to_channels_last(q8)
    assert not b8.to_numpy(rt.stream)[:, :, c:].any() and np.array_equal(rt.from_channels_last(b8, n, c, h, w), q8)
    per_channel = bool(rng.integers(2))
    scales = rng.uniform(5, 80, c if per_channel else 1).astype(F)
    x.reshape(-1)[: min(x.size, 8)] = (np.array([0.5, -0.5, 1.5, -2.5, 126.5, 127.49, 300.0, -300.0], F) / scales[0])[: min(x.size, 8)]
    want = oracle.quantize(x.transpose(1, 0, 2, 3).reshape(c, -1), scales).reshape(c, n, h, w).transpose(1, 0, 2, 3)
    q = rt.quantize_channels_last(rt.to_channels_last(x), c, scales)
    assert not q.to_numpy(rt.stream)[:, :, c:].any() and np.array_equal(rt.from_channels_last(q, n, c, h, w), want)


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_relu_eltwise_softmax(rt, seed):
    rng = np.random.default_rng(25000 + seed)
    size = (_size(rng) + 3) // 4 * 4  # fp32 blobs on the device hold whole groups of four values (channels padded to 16)
    print("[case] random elementwise", seed, size, flush=True)
    x = rng.normal(0, 1, size).astype(F)
    slope = F(_pick(rng, [0.0, 0.1, 0.25, -0.5]))
    assert np.array_equal(rt.relu(x, float(slope)), np.where(x < 0, (x * slope).astype(F), x) if slope != 0 else np.maximum(x, 0))
    q = rng.integers(-128, 128, size - int(rng.integers(4))).astype(np.int8)
    assert np.array_equal(rt.relu(q), np.maximum(q, 0))
    if seed % 10 == 0:
        from ncnn_amd.hip import NcnnHipError
        with pytest.raises(NcnnHipError, match="multiple of 4"):
            rt.relu(np.zeros(size + 1, F))
        with pytest.raises(NcnnHipError, match="multiple of 4"):
            rt.eltwise([np.zeros(size + 2, F), np.zeros(size + 2, F)], 1)
    k = int(rng.integers(2, 6))
    xs = [rng.normal(0, 1, size).astype(F) for _ in range(k)]
    acc_sum, acc_prod, acc_max = xs[0], xs[0], xs[0]
    for v in xs[1:]:
        acc_sum, acc_prod, acc_max = (acc_sum + v).astype(F), (acc_prod * v).astype(F), np.maximum(acc_max, v)
    assert np.array_equal(rt.eltwise(xs, 1), acc_sum) and np.array_equal(rt.eltwise(xs, 0), acc_prod) and np.array_equal(rt.eltwise(xs, 2), acc_max)
    co = rng.uniform(-2, 2, k).astype(F)
    want = (xs[0] * co[0]).astype(F)
    for v, cc in zip(xs[1:], co[1:]):
        want = (want + (v * cc).astype(F)).astype(F)
    assert np.array_equal(rt.eltwise(xs, 1, list(co)), want)
    rows, cols = int(_pick(rng, [1, 2, 7])), int(_pick(rng, [1, 2, 10, 100, 1000, 1001, int(rng.integers(1, 5000))]))
    s = rng.normal(0, 3, (rows, cols)).astype(F)
    got = rt.softmax(s)
    e = np.exp(s.astype(np.float64) - s.max(axis=1, keepdims=True))
    assert np.allclose(got, e / e.sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-9)


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_int8_max_pooling_and_global_pooling(rt, seed):
    rng = np.random.default_rng(27000 + seed)
    n, c = _pick(rng, [1, 2, 3]), int(_pick(rng, [1, 3, 16, 17, 40, 64, 100]))
    k, s = (int(rng.integers(1, 5)), int(rng.integers(1, 5))), (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    pt, pl = int(rng.integers(0, k[1])), int(rng.integers(0, k[0]))
    h, w = int(rng.integers(k[1], 30)), int(rng.integers(k[0], 30))
    oh, ow = (h + pt - k[1]) // s[1] + 1 + int(rng.integers(2)), (w + pl - k[0]) // s[0] + 1 + int(rng.integers(2))  # now and then a tail window
    oh, ow = min(oh, (h + pt - 1) // s[1] + 1), min(ow, (w + pl - 1) // s[0] + 1)  # every window starts inside the image
    print("[case] random int8 pooling", seed, (n, c, h, w), k, s, (pt, pl), (oh, ow), flush=True)
    xq = rng.integers(-127, 128, (n, c, h, w)).astype(np.int8)
    xb = np.full((n, c, pt + h + k[1] + s[1] * oh, pl + w + k[0] + s[0] * ow), -128, np.int16)
    xb[:, :, pt:pt + h, pl:pl + w] = xq
    win = np.stack([xb[:, :, ky: ky + (oh - 1) * s[1] + 1: s[1], kx: kx + (ow - 1) * s[0] + 1: s[0]] for ky in range(k[1]) for kx in range(k[0])])
    assert np.array_equal(rt.maxpool_int8(xq, k, s, (pt, pl), (oh, ow)), win.max(axis=0).astype(np.int8))
    x = rng.normal(0, 1, (n, c, h, w)).astype(F)
    flat = x.reshape(n, c, -1)
    avg = (np.cumsum(flat, axis=2, dtype=F)[..., -1] / F(h * w)).astype(F)
    assert np.array_equal(rt.pooling(x, 0, None, None, None, None, global_pooling=True), flat.max(axis=2))
    assert np.array_equal(rt.pooling(x, 1, None, None, None, None, global_pooling=True), avg)
    scale = F(rng.uniform(20, 200))
    assert np.array_equal(rt.global_pooling_quantised(x, 1, scale), oracle.quantize(avg, [scale]))
    assert np.array_equal(rt.global_pooling_quantised(x, 0, scale), oracle.quantize(flat.max(axis=2), [scale]))
