"""The layer half of the C API (src/c_api.h:196-352): parameter dictionaries, model readers, layers as tables of function
pointers and their registration on a net -- first with a layer written against the table (host only), then, on the GPU,
with the four MI355X layers plugged into a net through ncnn_net_register_custom_layer_by_type instead of the one-call
ncnnhip_register_int8_layers."""
import ctypes as C

import numpy as np
import pytest

from ncnn_amd import host, modelwriter as mw

F = np.float32


def test_paramdict_handles():
    L = host.lib()
    pd = L.ncnn_paramdict_create()
    assert L.ncnn_paramdict_get_type(pd, 3) == 0 and L.ncnn_paramdict_get_int(pd, 3, 77) == 77
    L.ncnn_paramdict_set_int(pd, 3, 5)
    L.ncnn_paramdict_set_float(pd, 4, 2.5)
    arr = host.Mat.from_numpy(np.array([1.5, -2.0, 4.0], F))
    L.ncnn_paramdict_set_array(pd, 5, arr.h_)
    assert L.ncnn_paramdict_get_type(pd, 3) == 2 and L.ncnn_paramdict_get_int(pd, 3, 0) == 5
    assert L.ncnn_paramdict_get_type(pd, 4) == 3 and L.ncnn_paramdict_get_float(pd, 4, 0.0) == 2.5
    got = host.Mat(L.ncnn_paramdict_get_array(pd, 5, None))
    assert np.array_equal(got.to_numpy(), [1.5, -2.0, 4.0])
    L.ncnn_paramdict_destroy(pd)


def test_modelbin_from_mat_array_hands_out_the_mats_in_order():
    L = host.lib()
    a, b = np.arange(6, dtype=F), np.arange(4, dtype=F) * 2
    mats = [host.Mat.from_numpy(a), host.Mat.from_numpy(b)]
    handles = (C.c_void_p * 2)(mats[0].h_, mats[1].h_)
    mb = L.ncnn_modelbin_create_from_mat_array(handles, 2)
    first = host.Mat(mb.contents.load_1d(mb, 6, 1))
    second = host.Mat(mb.contents.load_2d(mb, 2, 2, 1))
    assert np.array_equal(first.to_numpy(), a) and np.array_equal(second.to_numpy().reshape(-1), b)
    L.ncnn_modelbin_destroy(mb)


def test_builtin_layer_through_its_table():
    L = host.lib()
    assert not L.ncnn_layer_create_by_type(b"Convolution")  # known type, but no host implementation: the HIP layer must be registered
    relu = L.ncnn_layer_create_by_type(b"ReLU")
    assert relu and L.ncnn_layer_get_type(relu) in (b"ReLU", b"") and L.ncnn_layer_get_typeindex(relu) == L.ncnn_layer_type_to_index(b"ReLU")
    assert L.ncnn_layer_get_one_blob_only(relu) == 1 and L.ncnn_layer_get_support_inplace(relu) == 1
    pd = L.ncnn_paramdict_create()
    L.ncnn_paramdict_set_float(pd, 0, 0.25)  # slope
    assert relu.contents.load_param(relu, pd) == 0
    opt = L.ncnn_option_create()
    x = np.array([-4.0, 2.0, -1.0, 0.0], F)
    m = host.Mat.from_numpy(x.copy())
    assert relu.contents.forward_inplace_1(relu, m.h_, opt) == 0
    assert np.array_equal(m.to_numpy(), [-1.0, 2.0, -0.25, 0.0])
    L.ncnn_option_destroy(opt)
    L.ncnn_paramdict_destroy(pd)
    L.ncnn_layer_destroy(relu)


def test_custom_layer_written_against_the_table_runs_inside_a_net():
    """A layer type the library has never heard of, implemented by overwriting entries of ncnn_layer_create()'s table:
    load_param reads a factor (id 0) and an offset array (id 1), forward_inplace_1 computes x * factor + offset[channel]."""
    L = host.lib()
    state = {"created": 0, "destroyed": 0, "params": None}
    keep = []

    def creator():
        layer = L.ncnn_layer_create()
        L.ncnn_layer_set_one_blob_only(layer, 1)
        L.ncnn_layer_set_support_inplace(layer, 1)

        def load_param(self, pd):
            off = host.Mat(L.ncnn_paramdict_get_array(pd, 1, None))
            state["params"] = (L.ncnn_paramdict_get_float(pd, 0, 1.0), off.to_numpy().copy())
            return 0

        def forward_inplace_1(self, mat, opt):
            m = host.Mat(mat)
            try:
                factor, off = state["params"]
                c, h, w, cstep = m.c, m.h, m.w, m.cstep
                base = L.ncnn_mat_get_data(mat)
                buf = np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_float)), shape=(c, cstep))
                buf[:, : h * w] = buf[:, : h * w] * F(factor) + off[:, None]
                return 0
            finally:
                m.h_ = None  # borrowed handle: the net owns the blob

        fns = (host.LayerTable._fields_[1][1](load_param), host.LayerTable._fields_[7][1](forward_inplace_1))
        keep.append(fns)
        layer.contents.load_param, layer.contents.forward_inplace_1 = fns
        state["created"] += 1
        return layer

    def destroyer(layer):
        state["destroyed"] += 1
        L.ncnn_layer_destroy(layer)

    net = host.Net()
    net.register_custom_layer("ScaleShift", creator, destroyer)
    lines = ["Input in0 0 1 data 0=4 1=3 2=2", "ScaleShift ss 1 1 data out 0=2.5 -23301=2,1.0,-3.0", "ReLU relu 1 1 out act"]
    assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(b"") == 0
    x = np.random.default_rng(0).normal(0, 1, (2, 3, 4)).astype(F)
    ex = net.create_extractor()
    ex.input("data", x)
    want = np.maximum(x * F(2.5) + np.array([1.0, -3.0], F)[:, None, None], 0)
    assert np.array_equal(ex.extract("act"), want)
    assert state["created"] == 1
    del ex, net
    import gc
    gc.collect()
    assert state["destroyed"] == 1


@pytest.mark.gpu
@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
def test_hip_layers_registered_through_function_pointers(resident):
    """The drop-in route of a C program: ncnn_net_register_custom_layer_by_type for "Convolution", "ConvolutionDepthWise" and
    "InnerProduct" with creators that return the MI355X layers as ncnn_layer_t tables, then load_param / load_model /
    extract.  Same blobs as the oracle executor, bit for bit."""
    import refnet
    from ncnn_amd import zoo
    L = host.lib()
    made = []

    def creator_of(type_name):
        def creator():
            layer = L.ncnnhip_layer_create_by_type(type_name.encode())
            assert layer and L.ncnn_layer_get_type(layer) == type_name.encode()
            made.append(type_name)
            return layer
        return creator

    g, param, blob, info = zoo.build("tiny", seed=11)
    net = host.Net()
    for t in ("Convolution", "ConvolutionDepthWise", "InnerProduct", "Gemm"):
        net.register_custom_layer(t, creator_of(t), L.ncnn_layer_destroy)
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    assert {"Convolution", "ConvolutionDepthWise", "InnerProduct"} <= set(made)
    x = np.random.default_rng(12).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    for name in ("dw", "c3", "fc"):
        ex = net.create_extractor()
        ex.input("data", x)
        want = ref[name].astype(F) if ref[name].dtype == np.int8 else ref[name]
        assert np.array_equal(ex.extract(name), want), name
