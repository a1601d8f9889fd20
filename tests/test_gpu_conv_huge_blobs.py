"""Convolution layers whose output blob is larger than 2^32 bytes or 2^31 elements (a batch of more than a thousand
mid-sized maps): offsets into such a blob need 64 bits everywhere.  The folded batch is compared with runs of single
samples (the reference's batch is a per-sample loop, src/net.cpp:654-700; the single-sample path is held to the oracle
by the other tests), first, middle and last ones, bit for bit."""
import numpy as np
import pytest

from tests import cases

pytestmark = pytest.mark.gpu
F = np.float32


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


@pytest.mark.parametrize("batch,c,hw,outc,kernel,group,term,act", [
    (1400, 16, 112, 64, (1, 1), 1, 2, 1),     # pointwise kernel, 4.5e9 bytes of fp32
    (1400, 16, 112, 128, (1, 1), 1, 1, 0),    # 2.2e9 elements, 9e9 bytes
    (900, 32, 112, 96, (3, 3), 1, 2, 1),      # kernels with taps, 4.3e9 bytes
    (1400, 16, 112, 64, (1, 1), 1, 102, 3),   # requantised output, 1.1e9 elements
    (1200, 96, 112, 96, (3, 3), 96, 1, 3),    # depthwise, 5.8e9 bytes
])
def test_output_blobs_beyond_32_bit_offsets(rt, batch, c, hw, outc, kernel, group, term, act):
    print("[case] huge blob", batch, c, hw, outc, kernel, group, term, "output elements %.2e" % (batch * hw * hw * outc), flush=True)
    x, wq, b, ws, ins, tops = cases.conv_case(5, c, hw, hw, outc, kernel, group, term, True, True, by_group=group > 1, batch=4)
    xb = np.concatenate([np.roll(x, i, axis=3) for i in range(batch // 4)])  # every group of four samples shifted differently
    pads = (kernel[0] // 2,) * 4
    args = (wq, b, ws, ins, tops, outc, kernel, (1, 1), (1, 1), pads, 0.0, group, term, act, (0.0, 6.0))
    got = rt.conv_channels_last(xb, *args)
    assert got.shape == (batch, outc, hw, hw)
    for i in (0, 1, batch // 2, batch - 2, batch - 1):
        one = rt.conv_channels_last(xb[i:i + 1], *args)
        assert np.array_equal(got[i], one[0]), "sample %d" % i


@pytest.mark.parametrize("which,out", [("resnet50", "fc1000"), ("mobilenetv2", "fc")])
def test_benchmark_network_at_batch_1500(which, out):
    """The whole networks at 224 x 224 and batch 1500, device resident: the fp32 shortcut blobs of ResNet-50's second stage
    are 4.8e9 bytes each, MobileNetV2's widest int8 blob 1.8e9 elements.  Class scores of the first, middle and last
    samples against single-sample passes, bit for bit."""
    from ncnn_amd import host, zoo
    batch = 1500
    print("[case] huge net", which, batch, flush=True)
    g, param, blob, info = zoo.build(which, input_hw=224, n_calib=1)
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(True)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    base = np.random.default_rng(1).uniform(0, 1, (8,) + tuple(g.input_shape)).astype(F)
    xs = np.concatenate([np.roll(base, i, axis=3) for i in range((batch + 7) // 8)])[:batch]
    ex = net.create_extractor()
    ex.input("data", xs)
    got = np.asarray(ex.extract(out)).reshape(batch, -1)
    for i in (0, 1, batch // 2, batch - 2, batch - 1):
        one = net.create_extractor()
        one.input("data", xs[i])
        assert np.array_equal(got[i], np.asarray(one.extract(out)).reshape(-1)), "sample %d" % i
