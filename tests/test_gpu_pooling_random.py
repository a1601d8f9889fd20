"""The Pooling layer between the int8 layers at seeded random geometries, through load_param / extract in both execution
modes, against a scalar restatement of Pooling::forward (src/layer/pooling.cpp:150-330 with make_padding, :347-414): max
and average, rectangular windows and strides, the four pad modes (full with its tail pad, valid, SAME_UPPER, SAME_LOWER),
pad parameters, avgpool_count_include_pad, a batch.  fp32 in, fp32 out, bit for bit (the average adds the taps of a window
rows first in float32 and divides by the reference's count)."""
import os

import numpy as np
import pytest

from ncnn_amd import host, modelwriter as mw
from test_gpu_net import _avgpool_reference

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "150"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


def _border(w, h, k, s, pads, pad_mode):
    """(top, bottom, left, right) of the bordered image the reference builds."""
    pl, pr, pt, pb = pads
    if pad_mode == 0:
        wtail, htail = (w + pl + pr - k[0]) % s[0], (h + pt + pb - k[1]) % s[1]
        return pt, pb + (s[1] - htail if htail else 0), pl, pr + (s[0] - wtail if wtail else 0)
    if pad_mode == 1:
        return pt, pb, pl, pr
    wpad = k[0] + (w - 1) // s[0] * s[0] - w
    hpad = k[1] + (h - 1) // s[1] * s[1] - h
    if not (wpad > 0 or hpad > 0):
        return 0, 0, 0, 0
    if pad_mode == 2:
        return int(hpad / 2), hpad - int(hpad / 2), int(wpad / 2), wpad - int(wpad / 2)  # C division: towards zero
    return hpad - int(hpad / 2), int(hpad / 2), wpad - int(wpad / 2), int(wpad / 2)


def _maxpool_reference(x, k, s, pads, pad_mode):
    c, h, w = x.shape
    t, b, l, r = _border(w, h, k, s, pads, pad_mode)
    xb = np.full((c, h + t + b, w + l + r), -np.finfo(F).max, F)
    xb[:, t:t + h, l:l + w] = x
    oh, ow = (xb.shape[1] - k[1]) // s[1] + 1, (xb.shape[2] - k[0]) // s[0] + 1
    win = np.stack([xb[:, ky: ky + (oh - 1) * s[1] + 1: s[1], kx: kx + (ow - 1) * s[0] + 1: s[0]] for ky in range(k[1]) for kx in range(k[0])])
    return win.max(axis=0).astype(F)


@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_pooling_layer_matches_reference_restatement(seed, resident):
    rng = np.random.default_rng(13000 + seed)
    kind = int(rng.integers(2))
    c, batch = int(rng.integers(1, 21)), int(rng.choice([1, 1, 2, 3]))
    k = (int(rng.integers(1, 6)), int(rng.integers(1, 6)))
    s = (int(rng.integers(1, 4)), int(rng.integers(1, 4)))
    pad_mode = int(rng.integers(4))
    pads = tuple(int(min(v, kk - 1)) for v, kk in zip(rng.integers(0, 3, 4), (k[0], k[0], k[1], k[1]))) if rng.random() < 0.6 else (0, 0, 0, 0)
    include_pad = int(rng.integers(2))
    w = int(rng.integers(max(1, k[0] - pads[0] - pads[1]), 19))
    h = int(rng.integers(max(1, k[1] - pads[2] - pads[3]), 15))
    x = rng.normal(0, 1, (batch, c, h, w)).astype(F)
    print("[case] random pooling", seed, "resident" if resident else "host", ["max", "avg"][kind], (batch, c, h, w), "k", k, "s", s, "pads", pads,
          "pad_mode", pad_mode, "include_pad", include_pad, flush=True)
    lines = ["Input in0 0 1 data 0=%d 1=%d 2=%d" % (w, h, c),
             "Pooling pool 1 1 data out 0=%d 1=%d 11=%d 2=%d 12=%d 3=%d 14=%d 13=%d 15=%d 5=%d 6=%d"
             % (kind, k[0], k[1], s[0], s[1], pads[0], pads[1], pads[2], pads[3], pad_mode, include_pad)]
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(b"") == 0
    ex = net.create_extractor()
    ex.input("data", x if batch > 1 else x[0])
    if min(_border(w, h, k, s, pads, pad_mode)) < 0:
        # a SAME mode with the window below the stride in one dimension and a border needed in the other: the reference's
        # border copy writes out of bounds (src/layer/padding.cpp:62-87 with a negative border); refused here
        with pytest.raises(RuntimeError):
            ex.extract("out")
        return
    got = ex.extract("out")
    for i in range(batch):
        with np.errstate(invalid="ignore", divide="ignore"):
            want = _avgpool_reference(x[i], k, s, pads, pad_mode, include_pad) if kind == 1 else _maxpool_reference(x[i], k, s, pads, pad_mode)
        gi = got[i] if batch > 1 else got
        # (a window with no tap inside the counted rectangle is 0 / 0 in the reference: NaN on both sides)
        assert gi.shape == want.shape and np.array_equal(gi, want, equal_nan=True), "sample %d" % i
