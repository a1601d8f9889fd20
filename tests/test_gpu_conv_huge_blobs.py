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
