"""Out-of-memory behaviour at the boundary (the reference's tests/test_convolution_oom.cpp and tests/test_gemm_oom.cpp
through tests/testutil.cpp:2111-2340): an allocator that returns NULL at its N-th call, for every N up to the number of
calls a clean pass makes, must make the pass return -100 -- no crash, nothing left behind that spoils the next pass.
On the host the NULL comes from a replaced entry of the allocator's function-pointer table; on the device from a device
allocator installed with ncnnhip_set_device_allocator that refuses from its N-th call on."""
import ctypes as C

import numpy as np
import pytest

import refnet
from ncnn_amd import hip, host, zoo

pytestmark = pytest.mark.gpu
F = np.float32
MALLOC_FN = C.CFUNCTYPE(C.c_int, C.POINTER(C.c_void_p), C.c_size_t, C.c_void_p)
FREE_FN = C.CFUNCTYPE(C.c_int, C.c_void_p, C.c_void_p)


class FailingAllocator:
    """ncnn_allocator_create_pool_allocator() with fast_malloc replaced: the fail_at-th call (from 0) returns NULL."""

    def __init__(self):
        L = host.lib()
        self.a = L.ncnn_allocator_create_pool_allocator()
        self.count, self.fail_at = 0, -1
        original = self.a.contents.fast_malloc
        self._original = C.cast(original, C.c_void_p).value
        proto = host.AllocatorTable._fields_[1][1]
        self._real = proto(self._original)

        def fast_malloc(allocator, size):
            i = self.count
            self.count += 1
            return None if i == self.fail_at else self._real(allocator, size)

        self._thunk = proto(fast_malloc)
        self.a.contents.fast_malloc = self._thunk

    def close(self):
        host.lib().ncnn_allocator_destroy(self.a)


def _net(resident):
    g, param, blob, info = zoo.build("tiny", seed=21)
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    x = np.random.default_rng(22).uniform(0, 1, g.input_shape).astype(F)
    return net, x, refnet.run(param, blob, x)["fc"]


def _extract_code(ex, name):
    """(status, values or None); the values are copied out while the extractor, whose allocator owns them, is alive."""
    out = C.c_void_p()
    ret = host.lib().ncnn_extractor_extract(ex.h_, name.encode(), C.byref(out))
    m = host.Mat(out.value)
    got = m.to_numpy().copy() if ret == 0 else None
    del m
    return ret, got


@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
def test_host_allocator_returning_null_gives_minus_100(resident):
    L = host.lib()
    net, x, want = _net(resident)
    fa = FailingAllocator()
    opt = L.ncnn_option_create()
    base = L.ncnn_net_get_option(net.h_)
    L.ncnn_option_set_use_hip_compute(opt, L.ncnn_option_get_use_hip_compute(base))
    L.ncnn_option_set_blob_allocator(opt, fa.a)
    L.ncnn_option_set_workspace_allocator(opt, fa.a)
    L.ncnn_net_set_option(net.h_, opt)  # extractors created from now on allocate their blobs through the failing allocator

    def one_pass():
        ex = net.create_extractor(own_stream=False)
        ex.input("data", x)
        return _extract_code(ex, "fc")

    fa.count, fa.fail_at = 0, -1
    ret, got = one_pass()
    assert ret == 0 and np.array_equal(got, want)
    calls = fa.count
    assert calls >= (1 if resident else 5)
    for n in range(calls):
        print("host allocation", n, "of", calls, "fails", flush=True)
        fa.count, fa.fail_at = 0, n
        ret, _ = one_pass()
        assert ret == -100, (n, ret)
    fa.count, fa.fail_at = 0, -1
    ret, got = one_pass()
    assert ret == 0 and np.array_equal(got, want)
    L.ncnn_option_destroy(opt)


@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
def test_device_allocation_failing_gives_minus_100(resident):
    K = hip.lib()
    net, x, want = _net(resident)

    def one_pass():
        # a fresh net per pass would hide pool reuse; a fresh extractor takes an idle command whose pool is warm, so the
        # injected limit only bites where a pass really allocates
        ex = net.create_extractor(own_stream=not resident)
        ex.input("data", x)
        return _extract_code(ex, "fc")

    # a device allocator that wraps the default one and refuses from the n-th call on (the reference's test allocator
    # returns NULL the same way: tests/testutil.cpp:2111-2156)
    left = [0]

    @MALLOC_FN
    def counting_malloc(dev, nbytes, user):
        if left[0] <= 0:
            return -100
        left[0] -= 1
        return K.ncnnhip_default_device_malloc(dev, nbytes)

    @FREE_FN
    def plain_free(dev, user):
        return K.ncnnhip_default_device_free(dev)

    def restore():
        hip.check(K.ncnnhip_set_device_allocator(None, None, None))

    try:
        failures = 0
        for n in range(0, 200):
            print("device allocation limit", n, flush=True)
            left[0] = n
            hip.check(K.ncnnhip_set_device_allocator(C.cast(counting_malloc, C.c_void_p), C.cast(plain_free, C.c_void_p), None))
            ret, got = one_pass()
            restore()
            if ret == 0:
                assert np.array_equal(got, want)
                break
            assert ret == -100, (n, ret)
            failures += 1
        else:
            pytest.fail("a pass still ran out of device memory with 200 allocations allowed")
        assert failures >= 1, "the first pass of a net allocates device buffers: a limit of 0 must fail"
    finally:
        restore()
    ret, got = one_pass()
    assert ret == 0 and np.array_equal(got, want)
