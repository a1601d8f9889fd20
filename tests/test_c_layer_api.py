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


def test_mat_constructors_clone_and_reshape_as_the_references_c_api_test_uses_them():
    """tests/test_c_api.cpp:407-480 (test_c_api_batch) step by step: a batch of 3-D blobs written through
    ncnn_mat_get_batch_data, its deep copy, its reshape to vectors (the batch kept), a 2-D batch of 2-byte elements; then the
    remaining constructors of src/c_api.h:110-137, ncnn_mat_fill_float and ncnn_mat_get_channel_data."""
    import ctypes as C
    L = host.lib()
    W, H, Cc, B = 4, 3, 2, 3
    a = L.ncnn_mat_create_3d_batch(W, H, Cc, B, None)
    assert (L.ncnn_mat_get_dims(a), L.ncnn_mat_get_w(a), L.ncnn_mat_get_h(a), L.ncnn_mat_get_c(a), L.ncnn_mat_get_n(a)) == (3, W, H, Cc, B)
    assert L.ncnn_mat_get_nstep(a) != 0

    def floats(ptr, count):
        return np.ctypeslib.as_array(C.cast(ptr, C.POINTER(C.c_float)), (count,))

    cstep = L.ncnn_mat_get_cstep(a)
    for bi in range(B):
        data = floats(L.ncnn_mat_get_batch_data(a, bi), cstep * Cc)
        for q in range(Cc):
            data[q * cstep: q * cstep + W * H] = [bi * 100 + q * 10 + i for i in range(W * H)]
    b = L.ncnn_mat_clone(a, None)
    assert L.ncnn_mat_get_n(b) == B and L.ncnn_mat_get_data(b) != L.ncnn_mat_get_data(a)
    c = L.ncnn_mat_reshape_1d(a, W * H * Cc, None)
    assert (L.ncnn_mat_get_dims(c), L.ncnn_mat_get_w(c), L.ncnn_mat_get_n(c)) == (1, W * H * Cc, B)
    bstep = L.ncnn_mat_get_cstep(b)
    for bi in range(B):
        bdata = floats(L.ncnn_mat_get_batch_data(b, bi), bstep * Cc)
        cdata = floats(L.ncnn_mat_get_batch_data(c, bi), W * H * Cc)
        for q in range(Cc):
            want = np.array([bi * 100 + q * 10 + i for i in range(W * H)], np.float32)
            assert np.array_equal(bdata[q * bstep: q * bstep + W * H], want) and np.array_equal(cdata[q * W * H: (q + 1) * W * H], want)
    d = L.ncnn_mat_create_2d_elem_batch(5, 6, 2, 1, 2, None)
    assert (L.ncnn_mat_get_dims(d), L.ncnn_mat_get_w(d), L.ncnn_mat_get_h(d), L.ncnn_mat_get_n(d), L.ncnn_mat_get_elemsize(d)) == (2, 5, 6, 2, 2)
    for m in (a, b, c, d):
        L.ncnn_mat_destroy(m)

    shapes = {L.ncnn_mat_create_1d(7, None): (1, 7, 1, 1, 1, 1), L.ncnn_mat_create_2d(7, 5, None): (2, 7, 5, 1, 1, 1), L.ncnn_mat_create_3d(7, 5, 3, None): (3, 7, 5, 1, 3, 1),
              L.ncnn_mat_create_4d(7, 5, 2, 3, None): (4, 7, 5, 2, 3, 1), L.ncnn_mat_create_1d_batch(7, 4, None): (1, 7, 1, 1, 1, 4),
              L.ncnn_mat_create_2d_batch(7, 5, 4, None): (2, 7, 5, 1, 1, 4), L.ncnn_mat_create_4d_batch(7, 5, 2, 3, 4, None): (4, 7, 5, 2, 3, 4),
              L.ncnn_mat_create_4d_elem(7, 5, 2, 3, 1, 1, None): (4, 7, 5, 2, 3, 1), L.ncnn_mat_create_1d_elem_batch(7, 1, 1, 2, None): (1, 7, 1, 1, 1, 2),
              L.ncnn_mat_create_4d_elem_batch(7, 5, 2, 3, 4, 1, 2, None): (4, 7, 5, 2, 3, 2)}
    for m, want in shapes.items():
        assert (L.ncnn_mat_get_dims(m), L.ncnn_mat_get_w(m), L.ncnn_mat_get_h(m), L.ncnn_mat_get_d(m), L.ncnn_mat_get_c(m), L.ncnn_mat_get_n(m)) == want
        L.ncnn_mat_destroy(m)
    backing = np.arange(7 * 5 * 3, dtype=np.float32)
    for m, dims in ((L.ncnn_mat_create_external_1d(105, backing.ctypes.data, None), 1), (L.ncnn_mat_create_external_2d(21, 5, backing.ctypes.data, None), 2),
                    (L.ncnn_mat_create_external_4d(7, 5, 1, 3, backing.ctypes.data, None), 4), (L.ncnn_mat_create_external_4d_elem(7, 5, 1, 3, backing.ctypes.data, 4, 1, None), 4)):
        assert L.ncnn_mat_get_dims(m) == dims and L.ncnn_mat_get_data(m) == backing.ctypes.data
        L.ncnn_mat_destroy(m)
    m = L.ncnn_mat_create_3d(4, 3, 2, None)
    L.ncnn_mat_fill_float(m, 2.5)
    step = L.ncnn_mat_get_cstep(m)
    assert L.ncnn_mat_get_channel_data(m, 1) == L.ncnn_mat_get_data(m) + step * 4
    assert np.all(floats(L.ncnn_mat_get_channel_data(m, 1), 12) == 2.5)
    r = L.ncnn_mat_reshape_2d(m, 6, 4, None)
    assert (L.ncnn_mat_get_dims(r), L.ncnn_mat_get_w(r), L.ncnn_mat_get_h(r)) == (2, 6, 4) and np.all(floats(L.ncnn_mat_get_data(r), 24) == 2.5)
    r3 = L.ncnn_mat_reshape_3d(r, 2, 3, 4, None)
    assert (L.ncnn_mat_get_dims(r3), L.ncnn_mat_get_c(r3)) == (3, 4)
    for x in (m, r, r3):
        L.ncnn_mat_destroy(x)


def test_option_switches_net_indices_and_clear():
    """src/c_api.h:61-99 (the Option switches this runtime holds: set, read back), :382-391 (ncnn_net_clear, the blob indices of
    a net's inputs and outputs)."""
    L = host.lib()
    opt = L.ncnn_option_create()
    for f in host.OPTION_SWITCHES:
        for v in (1, 0, 1):
            getattr(L, "ncnn_option_set_" + f)(opt, v)
            assert getattr(L, "ncnn_option_get_" + f)(opt) == v, f
    L.ncnn_option_set_num_threads(opt, 3)
    assert L.ncnn_option_get_num_threads(opt) == 3
    L.ncnn_option_destroy(opt)
    net = host.Net()
    text = "7767517\n3 3\nInput in0 0 1 data 0=4 1=4 2=2\nReLU r 1 1 data mid\nReLU r2 1 1 mid out\n"
    assert net.load_param_mem(text) == 0
    blobs = net.blobs()
    assert L.ncnn_net_get_input_index(net.h_, 0) == list(blobs).index("data") and L.ncnn_net_get_output_index(net.h_, 0) == list(blobs).index("out")
    assert L.ncnn_net_get_input_index(net.h_, 5) == -1
    L.ncnn_net_clear(net.h_)
    assert L.ncnn_net_get_layer_count(net.h_) == 0 and L.ncnn_net_get_input_count(net.h_) == 0
    assert net.load_param_mem(text) == 0 and L.ncnn_net_get_layer_count(net.h_) == 3  # a cleared net loads again
