"""Seeded random int8 networks through load_param -> load_model -> create_extractor -> extract, against the oracle-based
executor on the same .param/.bin bytes, with blobs crossing the host per layer and with blobs resident in HBM.

The topologies are drawn from the blocks the two benchmark networks are made of -- plain and strided convolutions,
depthwise + pointwise pairs with and without a shortcut, bottlenecks with identity and projection shortcuts, max / average
pooling, global pooling, InnerProduct, Softmax -- in random order, widths, map sizes and batch, so that the executor's
fusion rules (Eltwise / ReLU / the next layer's Quantize inside a convolution's epilogue, sibling layers behind a Split,
int8 blobs between requantising layers) meet combinations the two fixed networks do not contain.
Every blob of every layer is compared bit for bit (Softmax to 1e-6); batch is the reference's per-sample loop
(src/net.cpp:654-700)."""
import os

import numpy as np
import pytest

import refnet
from ncnn_amd import host, modelwriter as mw, zoo

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_NETS", "40"))  # NCNN_RANDOM_NETS=<count> widens the walk


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


def random_net(seed, wide=1):
    """wide = 4: four times the channels on maps of 48 to 112 pixels (the kernels built for many pixels and channels)."""
    rng = np.random.default_rng(300 + seed + 100000 * (wide - 1))
    cin = _pick(rng, [1, 3, 3, 4])
    hw = int(rng.integers(14, 49)) if wide == 1 else int(rng.integers(48, 113))
    g = zoo.Graph(seed, (cin, hw, hw))
    relu6 = dict(act=3, act_params=(0.0, 6.0))
    acts = [dict(act=0), dict(act=1), dict(act=1), relu6]
    k = _pick(rng, [3, 3, 5, 7])
    c = _pick(rng, [8, 16, 24, 32]) * (2 if wide > 1 else 1)
    stride = _pick(rng, [1, 2])
    x = g.conv("stem", "data", cin, c, k, stride=stride, pad=k // 2, **_pick(rng, acts))
    size = (hw + 2 * (k // 2) - k) // stride + 1
    for bi in range(int(rng.integers(2, 6))):
        tag = "b%d" % bi
        kind = _pick(rng, ["conv", "conv", "dwpw", "dwpw", "bottleneck", "bottleneck", "pool"])
        if kind == "pool" and size >= 6:
            pk = _pick(rng, [2, 3])
            x = g.pool(tag + "_pool", x, _pick(rng, ["max", "avg"]), k=pk, stride=2)
            size = -(-(size - pk) // 2) + 1
        elif kind == "conv" or kind == "pool":
            cout = _pick(rng, [8, 16, 20, 32, 48, 64]) * wide
            ck = _pick(rng, [1, 3, 3])
            cs = 2 if (size >= 8 and rng.random() < 0.3) else 1
            x = g.conv(tag + "_conv", x, c, cout, ck, stride=cs, pad=ck // 2, bias=rng.random() < 0.8, **_pick(rng, acts))
            size = (size + 2 * (ck // 2) - ck) // cs + 1
            c = cout
        elif kind == "dwpw":
            t = _pick(rng, [1, 2, 6])
            cout = _pick(rng, [c, c, 16 * wide, 24 * wide, 40 * wide])
            cs = 2 if (size >= 8 and rng.random() < 0.3) else 1
            residual = cs == 1 and cout == c
            xa, xb = g.split(x) if residual else (x, None)
            y = xa
            hidden = c * t
            if t != 1:
                y = g.conv(tag + "_expand", y, c, hidden, 1, **relu6)
            y = g.conv(tag + "_dw", y, hidden, hidden, 3, stride=cs, pad=1, group=hidden, **relu6)
            y = g.conv(tag + "_project", y, hidden, cout, 1)
            x = g.add(tag + "_add", xb, y) if residual else y
            size = (size + 2 - 3) // cs + 1
            c = cout
        else:
            mid = _pick(rng, [8, 16, 32]) * wide
            cout = _pick(rng, [c, c, 32 * wide, 64 * wide, 96 * wide])
            cs = 2 if (size >= 8 and rng.random() < 0.3) else 1
            xa, xb = g.split(x)
            short = g.conv(tag + "_branch1", xb, c, cout, 1, stride=cs) if (cout != c or cs != 1 or rng.random() < 0.2) else xb
            y = g.conv(tag + "_2a", xa, c, mid, 1, stride=cs, act=1)
            y = g.conv(tag + "_2b", y, mid, mid, 3, pad=1, act=1)
            y = g.conv(tag + "_2c", y, mid, cout, 1)
            x = g.add(tag + "_sum", short, y)
            if rng.random() < 0.8:
                x = g.relu(tag + "_relu", x)
            size = (size - 1) // cs + 1
            c = cout
    x = g.pool("gap", x, _pick(rng, ["avg", "avg", "max"]), global_pool=True)
    n_out = _pick(rng, [5, 10, 37, 100])
    x = g.fc("fc", x, c, n_out)
    g.softmax("prob", x)
    absmax = zoo.calibrate(g, 2 if wide == 1 else 1)
    param, blob, _ = zoo.to_int8_model(g, absmax)
    return g, param, blob


@pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_net_every_blob_matches(seed, resident):
    g, param, blob = random_net(seed)
    rng = np.random.default_rng(seed)
    batch = _pick(rng, [1, 1, 2, 3])
    xs = rng.uniform(0, 1, (batch,) + tuple(g.input_shape)).astype(F)
    print("[case] random net", seed, "resident" if resident else "host", "batch", batch, "input", g.input_shape,
          [L["name"] for L in g.layers if L["type"] not in ("Input", "Split")], flush=True)
    refs = [refnet.run(param, blob, xs[i]) for i in range(batch)]
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    names = [t for L in g.layers if L["type"] not in ("Input", "Split", "Softmax") for t in L["tops"]]
    # one extractor per blob: each pass may fuse what the blob asked for allows; then all of them from one extractor, in
    # the network's order (in light mode a pass releases what it has consumed, the input included: asking one extractor for
    # an earlier blob after a later one is an error here as in the reference)
    for name in names:
        ex = net.create_extractor()
        ex.input("data", xs if batch > 1 else xs[0])
        got = ex.extract(name)
        for i in range(batch):
            want = refs[i][name]
            want = want.astype(F) if want.dtype == np.int8 else want
            gi = got[i] if batch > 1 else got
            assert gi.reshape(want.shape).shape == want.shape and np.array_equal(gi.reshape(want.shape), want), (name, i)
    ex = net.create_extractor()
    ex.input("data", xs if batch > 1 else xs[0])
    for name in names:
        got = ex.extract(name)
        for i in range(batch):
            want = refs[i][name]
            want = want.astype(F) if want.dtype == np.int8 else want
            gi = got[i] if batch > 1 else got
            assert np.array_equal(gi.reshape(want.shape), want), ("one extractor", name, i)
    prob = ex.extract("prob")
    for i in range(batch):
        assert np.allclose((prob[i] if batch > 1 else prob).reshape(-1), refs[i]["prob"].reshape(-1), rtol=1e-6, atol=1e-7)


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_net_recorded_pass_replays_like_the_oracle(seed):
    """The same networks recorded into a graph once and replayed with new input values: every replay gives the oracle
    executor's logits bit for bit (replays with eager passes and synchronisations in between)."""
    g, param, blob = random_net(seed)
    rng = np.random.default_rng(1000 + seed)
    batch = _pick(rng, [1, 1, 2, 3])
    shape = (batch,) + tuple(g.input_shape)
    print("[case] random net, recorded", seed, "batch", batch, "input", g.input_shape, flush=True)
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(True)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    x0 = rng.uniform(0, 1, shape).astype(F)
    graph = net.record("data", net.upload(x0 if batch > 1 else x0[0]), "fc")
    for i in range(3):
        x = x0 if i == 0 else rng.uniform(0, 1, shape).astype(F)
        want = np.stack([refnet.run(param, blob, x[j], want="fc")["fc"].reshape(-1) for j in range(batch)])
        if i:
            graph.update_input(x if batch > 1 else x[0])
            ex = net.create_extractor()  # eager work on the same net between the replays
            ex.input("data", x[0])
            assert np.array_equal(np.asarray(ex.extract("fc")).reshape(-1), want[0])
        graph.launch()
        if i == 1:
            graph.launch()  # back-to-back replays of the same values
        graph.synchronize()
        assert np.array_equal(graph.output().to_numpy().reshape(batch, -1), want), i


@pytest.mark.parametrize("seed", range(COUNT))
def test_random_net_through_the_plugin_matches_the_oracle(seed):
    """The same networks with their Convolution / ConvolutionDepthWise / InnerProduct layers supplied by the plug-in, the C
    shim written against nothing but the reference's c_api.h (function-pointer layer tables registered by type): every blob
    bit for bit, from one extractor in the network's order."""
    import ctypes as C
    from ncnn_amd import build
    host.lib()
    if not os.path.exists(build.LIBPLUGIN):
        raise RuntimeError("%s is missing: build it with python ncnn_amd/build.py" % build.LIBPLUGIN)
    plugin = C.CDLL(build.LIBPLUGIN)
    plugin.ncnnhip_plugin_register.restype = C.c_int
    plugin.ncnnhip_plugin_register.argtypes = [C.c_void_p]
    g, param, blob = random_net(seed)
    x = np.random.default_rng(2000 + seed).uniform(0, 1, g.input_shape).astype(F)
    print("[case] random net through the plug-in", seed, "input", g.input_shape, flush=True)
    ref = refnet.run(param, blob, x)
    net = host.Net()
    assert plugin.ncnnhip_plugin_register(net.h_) == 0
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    ex = net.create_extractor()
    ex.input("data", x)
    for name in [t for L in g.layers if L["type"] not in ("Input", "Split", "Softmax") for t in L["tops"]]:
        want = ref[name].astype(F) if ref[name].dtype == np.int8 else ref[name]
        got = ex.extract(name)
        assert np.array_equal(np.asarray(got).reshape(want.shape), want), name


@pytest.mark.parametrize("resident", [False, True, "plugin"], ids=["host-blobs", "device-resident", "plug-in"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_net_from_the_binary_param_form_matches_the_oracle(seed, resident):
    """The same networks loaded from the binary form of their .param text (Net::load_param_bin, src/net.cpp:1667-2018, the
    file tools/ncnn2mem.cpp writes: layers by the reference's type numbers, blobs by number, no names), fed and read by blob
    number: every blob bit for bit.  Also with the layers supplied by the plug-in, which registers them by type name and is
    found by type number here."""
    g, param, blob = random_net(seed)
    x = np.random.default_rng(2000 + seed).uniform(0, 1, g.input_shape).astype(F)
    print("[case] random net from .param.bin", seed, resident if resident == "plugin" else "resident" if resident else "host", "input", g.input_shape, flush=True)
    ref = refnet.run(param, blob, x)
    data, number = mw.assemble_param_bin(param.splitlines()[2:])
    net = host.Net()
    if resident == "plugin":
        import ctypes as C
        from ncnn_amd import build
        host.lib()
        if not os.path.exists(build.LIBPLUGIN):
            raise RuntimeError("%s is missing: build it with python ncnn_amd/build.py" % build.LIBPLUGIN)
        plugin = C.CDLL(build.LIBPLUGIN)
        plugin.ncnnhip_plugin_register.restype = C.c_int
        plugin.ncnnhip_plugin_register.argtypes = [C.c_void_p]
        assert plugin.ncnnhip_plugin_register(net.h_) == 0
    else:
        assert net.register_int8_layers() == 0
        net.set_use_hip_compute(resident)
    assert net.load_param_bin_mem(data) == 0 and net.load_model_mem(blob) == 0
    ex = net.create_extractor()
    ex.input(number["data"], x)
    for name in [t for L in g.layers if L["type"] not in ("Input", "Split", "Softmax") for t in L["tops"]]:
        want = ref[name].astype(F) if ref[name].dtype == np.int8 else ref[name]
        got = ex.extract(number[name])
        assert np.array_equal(np.asarray(got).reshape(want.shape), want), name


@pytest.mark.parametrize("seed", range(int(os.environ.get("NCNN_RANDOM_WIDE_NETS", "10"))))
def test_random_wide_net_at_a_batch_matches_the_oracle(seed):
    """Networks of the same blocks with four times the channels on maps of 48 to 112 pixels, at batch 4 to 16, device
    resident: the class scores and the deepest blobs of every sample bit for bit the oracle executor's."""
    g, param, blob = random_net(seed, wide=4)
    rng = np.random.default_rng(3000 + seed)
    batch = _pick(rng, [4, 8, 16])
    xs = rng.uniform(0, 1, (batch,) + tuple(g.input_shape)).astype(F)
    names = [t for L in g.layers if L["type"] not in ("Input", "Split", "Softmax") for t in L["tops"]]
    probes = names[-4:]
    print("[case] random wide net", seed, "batch", batch, "input", g.input_shape, names, flush=True)
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(True)
    assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
    got = {}
    for name in probes:
        ex = net.create_extractor()
        ex.input("data", xs)
        got[name] = np.asarray(ex.extract(name))
    for i in (0, batch // 2, batch - 1):
        ref = refnet.run(param, blob, xs[i])
        for name in probes:
            want = ref[name].astype(F) if ref[name].dtype == np.int8 else ref[name]
            assert np.array_equal(got[name][i].reshape(want.shape), want), (name, i)


def test_random_nets_on_concurrent_threads():
    """Six threads at once, each with a network of its own (its own Net, layers, weights, streams and pools) plus one
    network they all share, pass after pass with new inputs: whatever the library keeps per process -- lazily built
    tables, the device allocator, the zero line of the convolution kernels -- serves them all.  Every result bit for
    bit the oracle executor's."""
    import threading

    def load(param, blob):
        net = host.Net()
        assert net.register_int8_layers() == 0
        net.set_use_hip_compute(True)
        assert net.load_param_mem(param) == 0 and net.load_model_mem(blob) == 0
        return net

    shared_g, shared_param, shared_blob = random_net(7000)
    shared = load(shared_param, shared_blob)
    errors = []

    def worker(t):
        try:
            g, param, blob = random_net(7001 + t, wide=4 if t % 2 else 1)
            net = load(param, blob)
            rng = np.random.default_rng(t)
            for it in range(6):
                for gg, pp, bb, nn in ((g, param, blob, net), (shared_g, shared_param, shared_blob, shared)):
                    x = rng.uniform(0, 1, gg.input_shape).astype(F)
                    ex = nn.create_extractor()
                    ex.input("data", x)
                    got = np.asarray(ex.extract("fc")).reshape(-1)
                    want = refnet.run(pp, bb, x, want="fc")["fc"].reshape(-1)
                    if not np.array_equal(got, want):
                        errors.append("thread %d pass %d: result differs" % (t, it))
                        return
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(6)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not errors, errors
