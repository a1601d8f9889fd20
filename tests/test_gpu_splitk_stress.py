"""The K-split kernels hand partial sums from workgroup to workgroup through device memory (partials, an arrival counter
per output tile, the last arriver reduces and leaves the counter at zero).  A mistake in that hand-off's ordering shows as
a rare wrong value, so each layer runs 200 times on each of two streams that overlap on the GPU, every launch writing
its own output slice, and every slice must hold the oracle's bytes."""
import ctypes as C

import numpy as np
import pytest

import cases
from oracle import oracle
from ncnn_amd.hip import Activation, ConvDesc, DeviceBuffer, check, lib

pytestmark = pytest.mark.gpu
F = np.float32
ROUNDS = 200


@pytest.fixture(scope="module")
def rt():
    import ncnn_amd
    return ncnn_amd.Runtime(0)


def _at(buf, offset):
    return C.c_void_p(buf.ptr.value + offset)


def _two_streams():
    out = []
    for _ in range(2):
        s = C.c_void_p()
        check(lib().ncnnhip_stream_create(C.byref(s)))
        out.append(s)
    return out


def test_k_split_convolution_200_launches_on_two_streams(rt):
    c, hw, outc = 512, 7, 512
    x, wq, b, ws, ins, tops = cases.conv_case(77, c, hw, hw, outc, (3, 3), 1, 1, True, True)
    d = oracle.make_desc((c, hw, hw), outc, (3, 3), (1, 1), (1, 1), (1, 1, 1, 1), 0.0, 1, 1, 1, 1, (0.0, 0.0))
    want = oracle.convolution_int8(d, x[0], wq, b, ws, ins[0], None)            # [outc][h][w] fp32
    want_cl = np.ascontiguousarray(want.reshape(outc, hw * hw).T)               # channels-last, outc is a multiple of 16

    desc = ConvDesc(hw, hw, c, 1, outc, 3, 3, 1, 1, 1, 1, 1, 1, 1, 1, 0.0, 1)
    nb, wb, sb = C.c_size_t(), C.c_size_t(), C.c_size_t()
    check(lib().ncnnhip_conv_nhwc_sizes(C.byref(desc), C.byref(nb), C.byref(wb), C.byref(sb)))
    assert sb.value > 0, "this shape is meant to take the K-split path"
    src = rt.to_channels_last(x[0])                                              # int8 [1][49][512]
    pk = np.empty(wb.value, np.int8)
    check(lib().ncnnhip_conv_pack_weights(C.byref(desc), np.ascontiguousarray(wq, np.int8).ctypes.data, pk.ctypes.data))
    dpk, dsi, db = rt.up(pk), rt.up(rt.fold_input_scales(ws, ins, outc)), rt.up(np.asarray(b, F))
    rt.sync()
    out_bytes = hw * hw * outc * 4
    streams = _two_streams()
    outs = [DeviceBuffer.empty((ROUNDS, hw * hw, outc), F) for _ in streams]
    wss = [DeviceBuffer.zeros(sb.value, s) for s in streams]                    # one workspace per stream: calls that share one race
    act = Activation.make(1, (0.0, 0.0))
    try:
        for i in range(ROUNDS):
            for s, o, w in zip(streams, outs, wss):
                check(lib().ncnnhip_conv_int8_nhwc(C.byref(desc), src.ptr, dpk.ptr, dsi.ptr, db.ptr, None, act, _at(o, i * out_bytes),
                                                   1, 0, 0, w.ptr, sb.value, s))
        for k, (s, o) in enumerate(zip(streams, outs)):
            got = o.to_numpy(s)
            bad = [i for i in range(ROUNDS) if not np.array_equal(got[i], want_cl)]
            assert not bad, "stream %d: launches %s differ from the oracle" % (k, bad[:10])
    finally:
        for s in streams:
            lib().ncnnhip_stream_synchronize(s)
            lib().ncnnhip_stream_destroy(s)


def test_k_split_innerproduct_200_launches_on_two_streams(rt):
    rows, k, n = 64, 2048, 1000  # beyond the few-row kernel's 48 rows: 16 tiles of 64 x 64, K split over workgroups
    rng = np.random.default_rng(5)
    xq = rng.integers(-127, 128, (rows, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    ws = rng.uniform(10, 20, n).astype(F)
    b = rng.uniform(-1, 1, n).astype(F)
    in_scale = F(31.75)
    want = oracle.innerproduct_int8(xq, wq, b, ws, in_scale, 0, (0.0, 0.0))

    wsb = C.c_size_t()
    check(lib().ncnnhip_innerproduct_workspace_bytes(rows, k, n, C.byref(wsb)))
    assert wsb.value > 0, "this shape is meant to take the K-split path (the few-row kernel, which hands nothing over, reports no workspace)"
    dx, dw, dsi, db = rt.up(xq), rt.up(wq), rt.up(rt.fold_input_scales(ws, [in_scale], n)), rt.up(b)
    rt.sync()
    out_bytes = rows * n * 4
    streams = _two_streams()
    outs = [DeviceBuffer.empty((ROUNDS, rows, n), F) for _ in streams]
    wss = [DeviceBuffer.zeros(wsb.value, s) for s in streams]
    act = Activation.make(0, (0.0, 0.0))
    try:
        for i in range(ROUNDS):
            for s, o, w in zip(streams, outs, wss):
                check(lib().ncnnhip_innerproduct_int8_ws(dx.ptr, k, rows, k, n, dw.ptr, dsi.ptr, db.ptr, act, _at(o, i * out_bytes), n,
                                                         w.ptr, wsb.value, s))
        for j, (s, o) in enumerate(zip(streams, outs)):
            got = o.to_numpy(s)
            bad = [i for i in range(ROUNDS) if not np.array_equal(got[i], want)]
            assert not bad, "stream %d: launches %s differ from the oracle" % (j, bad[:10])
    finally:
        for s in streams:
            lib().ncnnhip_stream_synchronize(s)
            lib().ncnnhip_stream_destroy(s)
