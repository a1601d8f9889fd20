"""The InnerProduct layer through load_param / load_model / extract at seeded random input forms, against the oracle:
a vector, rows of num_input values (each row a product of its own, src/layer/innerproduct.cpp:56-107 / 147-230), a two-
or three-dimensional blob that is flattened in ncnn's planar order (on the device the blob is channels-last, or the narrow
four-channel image of an uploaded input), a batch; int8 or fp32 weights in the model file, every activation, with and
without bias.  Bit for bit on host Mats, on blobs resident in HBM and through the plug-in."""
import os

import numpy as np
import pytest

from ncnn_amd import host, modelwriter as mw
from oracle import oracle
from test_gpu_gemm_layer_random import _plugin

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "150"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


@pytest.mark.parametrize("route", ["host-blobs", "device-resident", "plug-in"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_innerproduct_layer_matches_oracle(seed, route):
    rng = np.random.default_rng(19000 + seed)
    form = _pick(rng, ["vector", "rows", "rows", "2-D flattened", "3-D flattened", "3-D flattened", "3-D of one pixel"])
    batch = 1 if route == "plug-in" else _pick(rng, [1, 1, 2, 3])
    n = int(rng.integers(1, 150))
    if form == "vector":
        shape = (int(rng.integers(1, 700)),)
    elif form == "rows":
        shape = (int(_pick(rng, [1, 2, 5, 9, 33, 50, 70])), int(rng.integers(1, 400)))
    elif form == "2-D flattened":
        shape = (int(rng.integers(2, 12)), int(rng.integers(1, 60)))
    elif form == "3-D of one pixel":
        shape = (int(rng.integers(1, 300)), 1, 1)
    else:
        shape = (int(_pick(rng, [1, 2, 3, 4, 5, 16, 20, 33])), int(rng.integers(1, 9)), int(rng.integers(1, 9)))
    k = shape[1] if form == "rows" else int(np.prod(shape))
    if form == "2-D flattened" and shape[1] == k:
        form = "rows"
    act, ap = _pick(rng, [(0, ()), (1, ()), (2, (0.1,)), (3, (0.0, 6.0)), (4, ()), (0, ())])
    bias, fp32_weights = rng.random() < 0.8, rng.random() < 0.3
    print("[case] random innerproduct layer", seed, route, form, "batch", batch, shape, "->", n, "act", act, bias, "fp32 weights" if fp32_weights else "", flush=True)
    x = rng.uniform(-1, 1, (batch,) + shape).astype(F)
    in_scale = F(127) / np.abs(x).max()
    wf = rng.normal(0, 0.1, (n, k)).astype(F)
    ws = (F(127) / np.maximum(np.abs(wf).max(axis=1), F(1e-6))).astype(F)
    wq = oracle.quantize_weights(wf, ws)
    b = rng.normal(size=n).astype(F) if bias else None
    dims = "0=%d" % shape[0] if len(shape) == 1 else "0=%d 1=%d" % (shape[1], shape[0]) if len(shape) == 2 else "0=%d 1=%d 2=%d" % (shape[2], shape[1], shape[0])
    line = mw.innerproduct_param("fc", "x", "out", n, n * k, int(bias), 2, act)
    if len(ap):
        line += " -23310=%d,%s" % (len(ap), ",".join(mw.fmt(v) for v in ap))
    lines = ["Input in0 0 1 x " + dims, line]
    blob = mw.conv_weights(wf.reshape(-1) if fp32_weights else wq, b, ws, in_scale, None)
    net = host.Net()
    if route == "plug-in":
        assert _plugin().ncnnhip_plugin_register(net.h_) == 0
    else:
        assert net.register_int8_layers() == 0
        net.set_use_hip_compute(route == "device-resident")
    assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(blob) == 0
    ex = net.create_extractor()
    # (a batch is a 4-D array of 3-D blobs: lower-dimensional samples are fed one by one)
    samples = [x] if (batch > 1 and len(shape) == 3) else list(x)
    got = []
    for s in samples:
        e = net.create_extractor()
        e.input("x", s)
        got.append(np.asarray(e.extract("out")))
    got = got[0] if (batch > 1 and len(shape) == 3) else np.stack(got)
    params = tuple(ap) + (0.0, 0.0)
    for i in range(batch):
        rows = x[i] if form == "rows" else x[i].reshape(1, -1)
        want = oracle.innerproduct_int8(rows, wq, b, ws, in_scale, act, params[:2])
        gi = got[i].reshape(want.shape)
        if act == 4:  # the device's expf: one unit in the last place of the sigmoid at most
            assert np.allclose(gi, want, rtol=1e-6, atol=1e-7), "sample %d" % i
        else:
            assert np.array_equal(gi, want), "sample %d" % i
