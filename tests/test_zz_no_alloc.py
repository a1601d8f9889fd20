"""The InnerProduct entry point that allocates nothing (ncnnhip_innerproduct_int8_noalloc): through the C ABI, against
the workspace form (ncnnhip_innerproduct_int8_ws) and the oracle, bit for bit, on calls in a row that share the
library-held scratch -- a large one first, then smaller ones, then one the scratch cannot hold."""
import ctypes as C

import numpy as np
import pytest

from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32


def _case(seed, rows, k, n):
    rng = np.random.default_rng(seed)
    xq = rng.integers(-127, 128, (rows, k)).astype(np.int8)
    wq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    w_scales = rng.uniform(20, 90, n).astype(F)
    in_scale = F(rng.uniform(10, 40))
    bias = rng.uniform(-0.5, 0.5, n).astype(F)
    return xq, wq, w_scales, in_scale, bias


def _both_forms(rt, hip, xq, wq, w_scales, in_scale, bias, act):
    lib = hip.lib()
    rows, k = xq.shape
    n = wq.shape[0]
    scale_in = rt.fold_input_scales(w_scales, [in_scale], n)
    dx, dw, dsi, db = rt.up(xq), rt.up(wq), rt.up(scale_in), rt.up(bias)
    a = hip.Activation.make(act, (0.0, 0.0))
    wsb = C.c_size_t()
    hip.check(lib.ncnnhip_innerproduct_workspace_bytes(rows, k, n, C.byref(wsb)))
    dws = hip.DeviceBuffer.zeros(max(wsb.value, 16), rt.stream)
    want = hip.DeviceBuffer.empty((rows, n), F)
    hip.check(lib.ncnnhip_innerproduct_int8_ws(dx.ptr, k, rows, k, n, dw.ptr, dsi.ptr, db.ptr, a, want.ptr, n, dws.ptr, wsb.value, rt.stream))
    got = hip.DeviceBuffer.empty((rows, n), F)
    got.fill_bytes(0xFF, rt.stream)
    hip.check(lib.ncnnhip_innerproduct_int8_noalloc(dx.ptr, k, rows, k, n, dw.ptr, dsi.ptr, db.ptr, a, got.ptr, n, rt.stream))
    return got.to_numpy(rt.stream), want.to_numpy(rt.stream), wsb.value


def test_noalloc_innerproduct_equals_the_workspace_form_on_calls_in_a_row():
    import ncnn_amd
    from ncnn_amd import hip
    rt = ncnn_amd.Runtime(0)
    # K-split shapes first (FC 2048 -> 1000 is the ResNet-50 head, at a batch beyond the few-row kernel's 48 rows), each
    # smaller than the one before, then shapes without a split: the few-row kernel's, a tiled one, the gemv kernel's; all
    # share the one scratch
    shapes = [(64, 2048, 1000), (56, 1536, 1000), (50, 3072, 256), (16, 2048, 1000), (64, 512, 128), (300, 256, 64), (3, 100, 10)]
    used_scratch = 0
    for i, (rows, k, n) in enumerate(shapes):
        print("noalloc innerproduct", rows, k, n, flush=True)
        xq, wq, w_scales, in_scale, bias = _case(100 + i, rows, k, n)
        got, want, ws = _both_forms(rt, hip, xq, wq, w_scales, in_scale, bias, act=1 if i % 2 else 0)
        used_scratch += ws > 0
        assert np.array_equal(got, want), "no-alloc form differs from the workspace form at %s" % ((rows, k, n),)
        ref = oracle.innerproduct_int8(xq, wq, bias, w_scales, in_scale, activation_type=1 if i % 2 else 0)
        assert np.array_equal(got, ref), "no-alloc form differs from the oracle at %s" % ((rows, k, n),)
    assert used_scratch >= 3, "the shapes were meant to exercise the K split"
    # the same large shape again after the small ones: whatever they left in the scratch must not matter
    xq, wq, w_scales, in_scale, bias = _case(7, 64, 2048, 1000)
    got, want, _ = _both_forms(rt, hip, xq, wq, w_scales, in_scale, bias, act=0)
    assert np.array_equal(got, want)


def test_noalloc_innerproduct_refuses_what_its_scratch_cannot_hold():
    import ncnn_amd
    from ncnn_amd import hip
    rt = ncnn_amd.Runtime(0)
    lib = hip.lib()
    # 5 x 40 tiles of 64 x 64, each split in two: 400 accumulator dumps of 16 KB, more than the 4 MiB the library holds
    rows, k, n = 320, 2048, 2560
    wsb = C.c_size_t()
    hip.check(lib.ncnnhip_innerproduct_workspace_bytes(rows, k, n, C.byref(wsb)))
    if wsb.value <= (4 << 20) + 4096:
        pytest.skip("no shape found that needs more scratch than the library holds (%d bytes)" % wsb.value)
    dx = hip.DeviceBuffer.zeros(rows * k, rt.stream)
    dw = hip.DeviceBuffer.zeros(n * k, rt.stream)
    dsi = rt.up(np.ones(n, F))
    out = hip.DeviceBuffer.empty((rows, n), F)
    rc = lib.ncnnhip_innerproduct_int8_noalloc(dx.ptr, k, rows, k, n, dw.ptr, dsi.ptr, None, hip.Activation.make(0, (0.0, 0.0)), out.ptr, n, rt.stream)
    assert rc == -1
    assert b"ncnnhip_innerproduct_int8_ws" in lib.ncnnhip_last_error()
    rt.sync()
