"""End-to-end parity through the drop-in boundary: register the HIP layers, load_param, load_model,
create_extractor, input, extract -- against the oracle-based executor on the same .param/.bin bytes."""
import numpy as np
import pytest

import cases
import refnet
from ncnn_amd import host, modelwriter as mw, zoo
from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32


def _say(*a):
    print(*a, flush=True)


RESIDENT = pytest.mark.parametrize("resident", [False, True], ids=["host-blobs", "device-resident"])


def _load(param, blob, resident=False):
    net = host.Net()
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(resident)  # blobs stay in HBM (channels-last) between layers, or cross the host per layer
    assert net.load_param_mem(param) == 0
    assert net.load_model_mem(blob) == 0
    return net


@RESIDENT
def test_tiny_net_every_blob_matches(resident):
    g, param, blob, info = zoo.build("tiny")
    x = np.random.default_rng(0).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    net = _load(param, blob, resident)
    for name in ("c1", "dw", "pw", "c2", "sum", "relu", "c3", "gap", "fc"):
        ex = net.create_extractor()
        ex.input("data", x)
        got = ex.extract(name)
        want = ref[name]
        want = want.astype(F) if want.dtype == np.int8 else want  # extract() expands int8 blobs to fp32
        assert got.shape == want.shape, name
        assert np.array_equal(got, want), name
    ex = net.create_extractor()
    ex.input("data", x)
    assert np.allclose(ex.extract("prob"), ref["prob"], rtol=1e-6, atol=1e-7)


@RESIDENT
def test_tiny_net_lightmode_off_and_shared_thread_stream(resident):
    g, param, blob, info = zoo.build("tiny", seed=3)
    x = np.random.default_rng(1).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    net = _load(param, blob, resident)
    net.set_lightmode(False)
    ex = net.create_extractor(own_stream=False)
    ex.input("data", x)
    assert np.array_equal(ex.extract("fc"), ref["fc"])
    assert np.array_equal(ex.extract("c3"), ref["c3"].astype(F))  # still held with light mode off


@RESIDENT
def test_batch_equals_per_sample(resident):
    g, param, blob, info = zoo.build("tiny", seed=5)
    xs = np.random.default_rng(2).uniform(0, 1, (3,) + g.input_shape).astype(F)
    net = _load(param, blob, resident)
    ex = net.create_extractor()
    ex.input("data", xs)
    got = ex.extract("fc")
    assert got.shape[0] == 3
    for i in range(3):
        assert np.array_equal(got[i].reshape(-1), refnet.run(param, blob, xs[i])["fc"])


@RESIDENT
def test_extractors_on_concurrent_threads_agree(resident):
    """forward is const and re-entrant (src/layer.h:95-101; one Extractor per thread is ncnn's threading model): four
    threads, each with its own Extractors and inputs, get what a single-threaded run gets."""
    import threading
    g, param, blob, info = zoo.build("mobilenetv2", input_hw=64, n_calib=1)
    net = _load(param, blob, resident)
    rng = np.random.default_rng(5)
    xs = [rng.uniform(0, 1, g.input_shape).astype(F) for _ in range(4)]

    def run(x):
        ex = net.create_extractor()
        ex.input("data", x)
        return ex.extract("fc")

    want = [run(x) for x in xs]
    errors = []

    def worker(i):
        try:
            for _ in range(6):
                if not np.array_equal(run(xs[i]), want[i]):
                    errors.append("thread %d: result differs" % i)
                    return
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (i, e))

    threads = [threading.Thread(target=worker, args=(i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


def test_narrow_input_image_reaches_layers_that_need_the_ordinary_layout():
    """A 3-channel input stays at 4 floats per pixel on the device; layers other than the first convolution get it
    widened, and extracting it gives back what went in."""
    lines = ["Input in0 0 1 data 0=12 1=10 2=3", "Split sp 1 3 data d1 d2 d3", "Pooling pool 1 1 d1 p 0=0 1=2 2=2", "ReLU relu 1 1 d2 r",
             "Pooling gap 1 1 d3 g 0=1 4=1"]
    net = _load(mw.assemble_param(lines), b"", True)
    x = np.random.default_rng(2).normal(0, 1, (2, 3, 10, 12)).astype(F)
    for name, want in (("p", x.reshape(2, 3, 5, 2, 6, 2).max(axis=(3, 5))), ("r", np.maximum(x, 0)), ("data", x)):
        ex = net.create_extractor()
        ex.input("data", x)
        assert np.array_equal(ex.extract(name), want), name
    ex = net.create_extractor()
    ex.input("data", x)
    flat = x.reshape(2, 3, -1)
    assert np.array_equal(ex.extract("g"), (np.cumsum(flat, axis=2, dtype=F)[..., -1] / F(120)).astype(F))


def _avgpool_reference(x, k, s, pads, pad_mode, include_pad):
    """Pooling::forward for average pooling as the reference computes it (src/layer/pooling.cpp:150-330 with make_padding,
    :347-414): build the bordered image, then per window skip taps by the LAYER'S pad parameters (tail pad only in pad_mode
    0), so a SAME border (pad_mode 2 / 3, pad parameters 0) is summed as zeros and counted."""
    c, h, w = x.shape
    pl, pr, pt, pb = pads
    wtailpad = htailpad = 0
    if pad_mode == 0:
        wtail, htail = (w + pl + pr - k[0]) % s[0], (h + pt + pb - k[1]) % s[1]
        wtailpad = s[0] - wtail if wtail else 0
        htailpad = s[1] - htail if htail else 0
        border = (pt, pb + htailpad, pl, pr + wtailpad)
    elif pad_mode == 1:
        border = (pt, pb, pl, pr)
    else:
        wpad = k[0] + (w - 1) // s[0] * s[0] - w
        hpad = k[1] + (h - 1) // s[1] * s[1] - h
        border = (0, 0, 0, 0)
        if wpad > 0 or hpad > 0:
            border = (hpad // 2, hpad - hpad // 2, wpad // 2, wpad - wpad // 2) if pad_mode == 2 else (hpad - hpad // 2, hpad // 2, wpad - wpad // 2, wpad // 2)
    xb = np.zeros((c, h + border[0] + border[1], w + border[2] + border[3]), F)
    xb[:, border[0]:border[0] + h, border[2]:border[2] + w] = x
    hb, wb = xb.shape[1:]
    oh, ow = (hb - k[1]) // s[1] + 1, (wb - k[0]) // s[0] + 1
    out = np.zeros((c, oh, ow), F)
    for q in range(c):
        for i in range(oh):
            for j in range(ow):
                acc, area = F(0), 0
                for ki in range(k[1]):
                    sy = i * s[1] + ki
                    if not include_pad and (sy < pt or sy >= hb - pb - htailpad):
                        continue
                    for kj in range(k[0]):
                        sx = j * s[0] + kj
                        if not include_pad and (sx < pl or sx >= wb - pr - wtailpad):
                            continue
                        acc = F(acc + xb[q, sy, sx])
                        area += 1
                out[q, i, j] = F(acc / F(k[0] * k[1] if include_pad else area))
    return out


@RESIDENT
@pytest.mark.parametrize("w,h,k,s,pads,pad_mode,include_pad", [
    (5, 5, (3, 3), (2, 2), (0, 0, 0, 0), 2, 0),      # SAME_UPPER: the border's zeros count (area 3 per row at the edge, not 2)
    (5, 7, (3, 3), (2, 2), (0, 0, 0, 0), 3, 0),      # SAME_LOWER
    (8, 6, (3, 2), (2, 1), (0, 0, 0, 0), 2, 0),
    (6, 6, (3, 3), (2, 2), (1, 0, 1, 0), 2, 0),      # SAME with non-zero pad parameters: they exclude taps of the SAME border
    (7, 6, (3, 3), (2, 2), (1, 1, 1, 1), 0, 0),      # full padding with a tail pad: neither pads nor tail count
    (7, 6, (3, 3), (2, 2), (1, 1, 1, 1), 1, 0),
    (7, 6, (3, 3), (2, 2), (1, 1, 1, 1), 0, 1),
    (5, 5, (3, 3), (2, 2), (0, 0, 0, 0), 2, 1),
])
def test_average_pooling_divisor_follows_the_reference_in_every_pad_mode(resident, w, h, k, s, pads, pad_mode, include_pad):
    c = 5
    x = np.random.default_rng(w * 10 + h + pad_mode).normal(0, 1, (c, h, w)).astype(F)
    lines = ["Input in0 0 1 data 0=%d 1=%d 2=%d" % (w, h, c),
             "Pooling pool 1 1 data out 0=1 1=%d 11=%d 2=%d 12=%d 3=%d 14=%d 13=%d 15=%d 5=%d 6=%d"
             % (k[0], k[1], s[0], s[1], pads[0], pads[1], pads[2], pads[3], pad_mode, include_pad)]
    got = _single(lines, b"", {"data": x}, "out", resident)
    want = _avgpool_reference(x, k, s, pads, pad_mode, include_pad)
    assert got.shape == want.shape and np.array_equal(got, want)


def test_resident_input_into_a_net_that_runs_on_host_blobs():
    """A blob fed as a HipMat when nothing of the Extractor has touched the device yet: a net with use_hip_compute off
    downloads it for its first layer, and extracting the fed blob itself gives back what went in."""
    g, param, blob, info = zoo.build("tiny")
    x = np.random.default_rng(3).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    net = _load(param, blob, False)
    xin = net.upload(x)
    ex = net.create_extractor()
    assert ex.input_resident("data", xin) == 0
    assert np.array_equal(ex.extract("data"), x)
    ex = net.create_extractor()
    assert ex.input_resident("data", xin) == 0
    assert np.array_equal(ex.extract("fc"), ref["fc"])


def test_resident_blob_outlives_its_extractor_and_its_net():
    """A HipMat shares the buffer pool it was cut from: it stays valid after the Extractor, the command and the Net that
    produced it are gone."""
    import gc
    g, param, blob, info = zoo.build("tiny", seed=2)
    x = np.random.default_rng(4).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    net = _load(param, blob, True)
    ex = net.create_extractor()
    ex.input("data", x)
    out = ex.extract_resident("fc")
    ex.synchronize()
    out.net = None
    del ex, net
    gc.collect()
    assert np.array_equal(out.to_numpy().reshape(-1), ref["fc"].reshape(-1))


def test_uploads_from_several_threads_and_reassigned_inputs():
    """Net::upload from four threads at once, each reassigning its input blob in a loop and extracting resident results
    without waiting in between: a buffer that returns to the upload pool is not refilled while a pass still reads it."""
    import threading
    g, param, blob, info = zoo.build("tiny", seed=7)
    net = _load(param, blob, True)
    rng = np.random.default_rng(8)
    xs = [rng.uniform(0, 1, g.input_shape).astype(F) for _ in range(6)]
    want = [refnet.run(param, blob, x)["fc"].reshape(-1) for x in xs]
    errors = []

    def worker(t):
        try:
            outs = []
            for i in range(12):
                xin = net.upload(xs[(t + i) % 6])  # the previous blob of this name goes back to the pool here
                ex = net.create_extractor()
                ex.input_resident("data", xin)
                outs.append(((t + i) % 6, ex, ex.extract_resident("fc")))
            for j, ex, o in outs:
                ex.synchronize()
                if not np.array_equal(o.to_numpy().reshape(-1), want[j]):
                    errors.append("thread %d: wrong result for input %d" % (t, j))
                    return
        except Exception as e:  # noqa: BLE001
            errors.append("thread %d: %r" % (t, e))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors


@RESIDENT
def test_featmask_switches_a_single_layer_to_host_blobs_and_one_thread(resident):
    """Param id 31 (featmask) applies at create_pipeline AND at forward time (src/net.cpp:100-121,163): bit 4 takes the
    layer off the device-resident path, bit 7 gives it one thread, bit 3 leaves use_int8_inference alone.  Results do not
    change."""
    g, param, blob, info = zoo.build("tiny", seed=9)
    x = np.random.default_rng(9).uniform(0, 1, g.input_shape).astype(F)
    ref = refnet.run(param, blob, x)
    lines = param.split("\n")
    masked, n = [], 0
    for ln in lines:
        if ln.startswith("Convolution ") and n < 2:
            ln = ln + " 31=%d" % (16 + 128 + 8 if n == 0 else 8)
            n += 1
        masked.append(ln)
    assert n == 2
    net = _load("\n".join(masked), blob, resident)
    ex = net.create_extractor()
    ex.input("data", x)
    assert np.array_equal(ex.extract("fc"), ref["fc"])


def test_int8_inference_switched_off_is_an_error_not_a_fallback():
    g, param, blob, info = zoo.build("tiny")
    net = _load(param, blob)
    net.set_use_int8_inference(False)
    ex = net.create_extractor()
    ex.input("data", np.zeros(g.input_shape, F))
    with pytest.raises(RuntimeError):
        ex.extract("fc")


# ----------------------------------------------------------------------------- single layers through the boundary
def _single(param_lines, blob, feeds, out, resident=False):
    net = _load(mw.assemble_param(param_lines), blob, resident)
    ex = net.create_extractor()
    for k, v in feeds.items():
        ex.input(k, v)
    return ex.extract(out)


@RESIDENT
def test_gemm_layer_int8_constant_b_with_bias(resident):
    rng = np.random.default_rng(4)
    m, n, k = 37, 50, 96
    a = rng.standard_normal((m, k), dtype=F)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = F(63.5)
    c = rng.standard_normal((1, n), dtype=F)
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m),
             mw.gemm_param("g", ["a"], "out", M=0, N=n, K=k, constantB=1, constantC=1, broadcast_type_C=4, quantize_term=2)]
    blob = mw.weight_blob(bq) + mw.weight_blob(c) + mw.raw_f32(sb)
    got = _single(lines, blob, {"a": a}, "out", resident)
    aq, sa = oracle.gemm_quantize_rows(a)
    assert np.array_equal(got, oracle.gemm_int8(aq, bq, sa, [sb], c, 4))


def test_gemm_layer_int8_constant_b_large_enough_for_the_tiled_operands():
    """From 128 output tiles of 256 x 256 the device-resident Gemm layer quantises A straight into the 256x256 kernel's tiled
    layout and multiplies it with the copy of B that create_pipeline tiled; the answer is the oracle's, bit for bit."""
    import npref
    rng = np.random.default_rng(5)
    m, n, k = 2048, 4096, 128
    a = rng.standard_normal((m, k), dtype=F)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = F(41.25)
    c = rng.standard_normal((1, n), dtype=F)
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m),
             mw.gemm_param("g", ["a"], "out", M=0, N=n, K=k, constantB=1, constantC=1, broadcast_type_C=4, quantize_term=2)]
    blob = mw.weight_blob(bq) + mw.weight_blob(c) + mw.raw_f32(sb)
    got = _single(lines, blob, {"a": a}, "out", True)
    aq, sa = oracle.gemm_quantize_rows(a)
    want, _ = npref.gemm_int8(aq, bq, sa, [sb], c, 4, acc=npref.gemm_acc_exact(aq, bq))
    assert np.array_equal(got, want)
    rows = np.arange(0, m, 97)
    assert np.array_equal(got[rows], oracle.gemm_int8(aq[rows], bq, sa[rows], [sb], c, 4))


def test_gemm_layer_int8_two_dynamic_operands_transposed_output():
    rng = np.random.default_rng(5)
    m, n, k = 20, 33, 64
    a = rng.standard_normal((m, k), dtype=F)
    b = (rng.standard_normal((k, n), dtype=F) * F(0.02)).astype(F)  # transB = 0: stored [K][N]
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), "Input in1 0 1 b 0=%d 1=%d" % (n, k),
             mw.gemm_param("g", ["a", "b"], "out", transB=0, constantB=0, quantize_term=2, output_transpose=1, alpha=0.5)]
    got = _single(lines, b"", {"a": a, "b": b}, "out")
    aq, sa = oracle.gemm_quantize_rows(a)
    bq, sb = oracle.gemm_quantize_tensor(b)
    want = oracle.gemm_int8(aq, bq.T.copy(), sa, [sb], None, -1, 0.5, 1.0, True)
    assert np.array_equal(got, want)


def _single_where(param_lines, blob, feeds, out, resident, layer="g"):
    """extract(out) and where the named layer ran ('device' | 'host')."""
    net = _load(mw.assemble_param(param_lines), blob, resident)
    ex = net.create_extractor()
    ex.set_layer_timing(True)
    for k, v in feeds.items():
        ex.input(k, v)
    got = ex.extract(out)
    where = {r[2]: r[3] for r in ex.layer_timing()}
    return got, where[layer]


@RESIDENT
@pytest.mark.parametrize("c,outc,group,h,w,stride,term,act", [(8, 4, 2, 12, 12, 2, 1, 1), (64, 64, 4, 14, 14, 1, 101, 3), (6, 12, 3, 9, 10, 1, 2, 0),
                                                              (32, 48, 8, 10, 7, 1, 102, 1)])
def test_grouped_convolution_layer_stays_on_the_device(c, outc, group, h, w, stride, term, act, resident):
    """ConvolutionDepthWise with 1 < group < channels (src/layer/convolutiondepthwise.cpp:515-636: group by group) through
    load_param / load_model / forward, batch of two: bit for bit the oracle's, on host Mats and as a device layer (the
    planar kernel between two layout changes in HBM)."""
    x, wq, b, ws, ins, tops = cases.conv_case(c + outc + group + term, c, h, w, outc, (3, 3), group, term, True, False, by_group=True, batch=2)
    one_weight_scale = term in (2, 102)
    if one_weight_scale:
        ws[:] = ws[0]
    ap = (0.0, 6.0) if act == 3 else ()
    lines = ["Input in0 0 1 data 0=%d 1=%d 2=%d" % (w, h, c),
             mw.conv_param("g", "data", "out", outc, 3, stride=stride, pad=1, weight_size=wq.size, term=term, act=act, act_params=ap, group=group)]
    blob = mw.conv_weights(wq, b, ws[:1] if one_weight_scale else ws, ins[0], None if tops is None else tops[0])
    got, where = _single_where(lines, blob, {"data": x}, "out", resident)
    d = oracle.make_desc((c, h, w), outc, (3, 3), (1, 1), (stride, stride), (1, 1, 1, 1), 0.0, 1, group, term, act, (0.0, 6.0))
    for i in range(2):
        want = oracle.convolutiondepthwise_int8(d, x[i], wq, b, ws, ins, tops)
        assert np.array_equal(got[i], want.astype(F)), "sample %d" % i  # (extract hands an int8 blob over as fp32 values, src/net.cpp:3007-3012)
    assert where == ("device" if resident else "host")


GEMM_FORMS = ["two dynamic operands, B stored [K][N], transposed output", "constant int8 A, dynamic B, dynamic per-column C",
              "transA, constant int8 B, constant per-row C", "3-D operands of height 1", "batch of three, two dynamic 3-D operands",
              "constant fp32 A stored transposed, dynamic B stored [K][N]", "both operands constant, dynamic full C, transposed output",
              "one row: 1-D A, dynamic B, scalar C", "N x 1 x M output, 20 channels in 32", "transposed N x 1 x M output"]


@RESIDENT
@pytest.mark.parametrize("form", range(len(GEMM_FORMS)), ids=GEMM_FORMS)
def test_gemm_layer_int8_every_form_stays_on_the_device(form, resident):
    """Gemm::forward_int8 (src/layer/gemm.cpp:745-966) beyond the network form: constant or dynamic A, B and C, transposed
    inputs and output, 3-D operands (c rows of w values), a batch.  Bit for bit the oracle's on host Mats and on blobs that
    stay in HBM -- where the layer must run as a device layer, not through host Mats."""
    rng = np.random.default_rng(40 + form)
    m, n, k = 24, 40, 96
    a = rng.standard_normal((m, k), dtype=F)
    b = (rng.standard_normal((n, k), dtype=F) * F(0.05)).astype(F)  # [N][K]
    aq, sa = oracle.gemm_quantize_rows(a)
    bq, sb = oracle.gemm_quantize_tensor(b)
    in_a, in_b = "Input in0 0 1 a 0=%d 1=%d" % (k, m), "Input in1 0 1 b 0=%d 1=%d" % (k, n)
    if form == 0:
        lines = [in_a, "Input in1 0 1 b 0=%d 1=%d" % (n, k), mw.gemm_param("g", ["a", "b"], "out", transB=0, constantB=0, output_transpose=1, alpha=0.5)]
        got, where = _single_where(lines, b"", {"a": a, "b": b.T.copy()}, "out", resident)
        want = oracle.gemm_int8(aq, bq, sa, [sb], None, -1, 0.5, 1.0, True)
    elif form == 1:
        c = rng.standard_normal(n, dtype=F)
        ca_scales = (F(127) / np.abs(a).max(axis=1)).astype(F)
        caq = oracle.quantize(a, ca_scales)  # one scale per row, as a constant int8 A carries them
        lines = [in_b, "Input in2 0 1 c 0=%d" % n, mw.gemm_param("g", ["b", "c"], "out", M=m, K=k, constantA=1, constantB=0, beta=0.25)]
        got, where = _single_where(lines, mw.weight_blob(caq) + mw.raw_f32(ca_scales), {"b": b, "c": c}, "out", resident)
        want = oracle.gemm_int8(caq, bq, ca_scales, [sb], c, 4, 1.0, 0.25)
    elif form == 2:
        c = rng.standard_normal((m, 1), dtype=F)
        cbq = rng.integers(-127, 128, (n, k)).astype(np.int8)
        csb = F(51.0)
        lines = ["Input in0 0 1 a 0=%d 1=%d" % (m, k), mw.gemm_param("g", ["a"], "out", N=n, K=k, M=m, transA=1, constantB=1, constantC=1, broadcast_type_C=2, beta=0.5)]
        got, where = _single_where(lines, mw.weight_blob(cbq) + mw.weight_blob(c) + mw.raw_f32(csb), {"a": a.T.copy()}, "out", resident)
        want = oracle.gemm_int8(aq, cbq, sa, [csb], c, 2, 1.0, 0.5)
    elif form == 3:
        lines = ["Input in0 0 1 a 0=%d 1=1 2=%d" % (k, m), "Input in1 0 1 b 0=%d 1=1 2=%d" % (k, n), mw.gemm_param("g", ["a", "b"], "out", constantB=0)]
        got, where = _single_where(lines, b"", {"a": a.reshape(m, 1, k), "b": b.reshape(n, 1, k)}, "out", resident)
        want = oracle.gemm_int8(aq, bq, sa, [sb], None, -1)
    elif form == 4:
        a3 = rng.standard_normal((3, m, k), dtype=F)
        b3 = (rng.standard_normal((3, n, k), dtype=F) * F(0.05)).astype(F)
        # (a batch is a 4-D array of 3-D blobs: the operands are 3-D blobs of height 1 here too)
        lines = ["Input in0 0 1 a 0=%d 1=1 2=%d" % (k, m), "Input in1 0 1 b 0=%d 1=1 2=%d" % (k, n), mw.gemm_param("g", ["a", "b"], "out", constantB=0, alpha=2.0)]
        got, where = _single_where(lines, b"", {"a": a3.reshape(3, m, 1, k), "b": b3.reshape(3, n, 1, k)}, "out", resident)
        want = []
        for i in range(3):
            qa, s_a = oracle.gemm_quantize_rows(a3[i])
            qb, s_b = oracle.gemm_quantize_tensor(b3[i])
            want.append(oracle.gemm_int8(qa, qb, s_a, [s_b], None, -1, 2.0))
        want = np.stack(want)
    elif form == 5:
        lines = ["Input in1 0 1 b 0=%d 1=%d" % (n, k), mw.gemm_param("g", ["b"], "out", M=m, K=k, transA=1, transB=0, constantA=1, constantB=0)]
        blob = mw.weight_blob(a.T.copy()) + mw.raw_f32(np.ones(m, F))  # fp32 A: quantised row by row at forward time; the scale table is read and not used
        got, where = _single_where(lines, blob, {"b": b.T.copy()}, "out", resident)
        want = oracle.gemm_int8(aq, bq, sa, [sb], None, -1)
    elif form == 6:
        c = rng.standard_normal((m, n), dtype=F)
        ca_scales = (F(127) / np.abs(a).max(axis=1)).astype(F)
        caq = oracle.quantize(a, ca_scales)
        cbq = rng.integers(-127, 128, (n, k)).astype(np.int8)
        csb = F(33.0)
        lines = ["Input in0 0 1 c 0=%d 1=%d" % (n, m), mw.gemm_param("g", ["c"], "out", M=m, N=n, K=k, constantA=1, constantB=1, output_transpose=1)]
        got, where = _single_where(lines, mw.weight_blob(caq) + mw.weight_blob(cbq) + mw.raw_f32(ca_scales) + mw.raw_f32(csb), {"c": c}, "out", resident)
        want = oracle.gemm_int8(caq, cbq, ca_scales, [csb], c, 3, 1.0, 1.0, True)
    elif form == 7:
        c = np.array([0.75], F)
        lines = ["Input in0 0 1 a 0=%d" % k, in_b, "Input in2 0 1 c 0=1", mw.gemm_param("g", ["a", "b", "c"], "out", constantB=0)]
        got, where = _single_where(lines, b"", {"a": a[0], "b": b, "c": c}, "out", resident)
        want = oracle.gemm_int8(aq[:1], bq, sa[:1], [sb], c, 0)
    elif form == 8:
        # output (w = N, h = 1, c = M) with M = 20 rows: a channels-last blob of 32 channels in HBM
        lines = ["Input in0 0 1 a 0=%d 1=20" % k, in_b, mw.gemm_param("g", ["a", "b"], "out", constantB=0, output_N1M=1)]
        got, where = _single_where(lines, b"", {"a": a[:20], "b": b}, "out", resident)
        want = oracle.gemm_int8(aq[:20], bq, sa[:20], [sb], None, -1).reshape(20, 1, n)
    else:
        cbq = rng.integers(-127, 128, (n, k)).astype(np.int8)
        csb = F(47.0)
        c = rng.standard_normal((1, n), dtype=F)
        lines = [in_a, mw.gemm_param("g", ["a"], "out", N=n, K=k, constantB=1, constantC=1, broadcast_type_C=4, output_N1M=1, output_transpose=1)]
        got, where = _single_where(lines, mw.weight_blob(cbq) + mw.weight_blob(c) + mw.raw_f32(csb), {"a": a}, "out", resident)
        want = oracle.gemm_int8(aq, cbq, sa, [csb], c, 4, 1.0, 1.0, True).reshape(n, 1, m)
    assert np.array_equal(np.asarray(got).reshape(want.shape), want)
    assert where == ("device" if resident else "host")


@RESIDENT
@pytest.mark.parametrize("bits,block,insc,m,n,k", [
    (8, 64, 0, 4, 24, 200), (4, 32, 1, 4, 24, 200), (6, 128, 0, 4, 24, 200),  # K % 16 != 0: the .bin layout as it is
    # K % 16 == 0: create_pipeline also uploads matrix-core tiles; few rows take them four per pass, 32 rows and more the tiled bf16 kernel
    (8, 64, 0, 1, 40, 256), (8, 64, 1, 4, 33, 256), (4, 32, 1, 3, 24, 512), (6, 128, 0, 16, 40, 1024), (8, 32, 0, 20, 24, 256),
    (8, 64, 0, 40, 100, 256), (4, 64, 1, 70, 33, 512), (6, 32, 0, 129, 40, 96), (8, 128, 1, 33, 130, 1024),
    # K beyond 4096: three and four rows take the pre-split kernels (the few-row kernel would stream the weights once per row), two rows do not
    (8, 64, 0, 4, 24, 4352), (4, 32, 1, 3, 40, 8192), (8, 64, 1, 2, 24, 4352)])
def test_gemm_layer_block_quant(bits, block, insc, m, n, k, resident):
    import npref
    rng = np.random.default_rng(bits + m + k)
    a = rng.standard_normal((m, k), dtype=F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    ins = (0.75 + (np.arange(k) % 5) * 0.15).astype(F) if insc else None
    term = bits * 100 + insc * 10 + {32: 0, 64: 1, 128: 2}[block]
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), mw.gemm_param("g", ["a"], "out", N=n, K=k, constantB=1, quantize_term=term)]
    blob = mw.weight_blob(packed.view(np.int8)) + mw.raw_f32(scales) + (mw.raw_f32(ins) if insc else b"")
    got = _single(lines, blob, {"a": a}, "out", resident)
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins)
    assert np.all(np.abs(got - val) <= 1e-5 * floor + 1e-30)


@RESIDENT
@pytest.mark.parametrize("m,n,k,c_shape,bt", [(4, 40, 256, (40,), 4), (20, 33, 512, (20, 33), 3), (3, 24, 200, (3, 1), 2), (1, 48, 256, (1,), 0)])
def test_gemm_layer_block_quant_with_c_as_the_second_bottom_blob(m, n, k, c_shape, bt, resident):
    """Gemm::forward_weight_block_quantize takes C from the second bottom blob when it is not a constant
    (src/layer/gemm.cpp:372-421): per column, full, per row, scalar -- on host Mats and as a device layer."""
    import npref
    rng = np.random.default_rng(m + n + k)
    a = rng.standard_normal((m, k), dtype=F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    c = rng.standard_normal(c_shape, dtype=F)
    packed, scales = oracle.blockquant_pack(w, 8, 64)
    c_in = "Input in1 0 1 c 0=%d" % c_shape[0] if len(c_shape) == 1 else "Input in1 0 1 c 0=%d 1=%d" % (c_shape[1], c_shape[0])
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), c_in, mw.gemm_param("g", ["a", "c"], "out", N=n, K=k, constantB=1, quantize_term=801, alpha=0.5, beta=2.0)]
    blob = mw.weight_blob(packed.view(np.int8)) + mw.raw_f32(scales)
    got, where = _single_where(lines, blob, {"a": a, "c": c}, "out", resident)
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, 8, 64, None, c, bt, 0.5, 2.0)
    assert np.all(np.abs(got - val) <= 1e-5 * floor + 1e-30)
    assert where == ("device" if resident else "host")


@pytest.mark.parametrize("m", [1, 4, 9])
def test_sibling_block_quant_gemms_behind_a_split_share_one_launch(m):
    """The gate / up pair of a decoder layer: block-quantised Gemm layers that read the outputs of one Split run as ONE launch
    on device-resident blobs (up to four activation rows), and every output is bit for bit what the layer gives in a net of
    its own; a sibling with per-layer input scales, and every sibling at nine rows, keeps its own launch.  The reference runs
    the layers one after the other (src/net.cpp:625-700 for the executor, src/layer/gemm.cpp:425-483 for each)."""
    import npref
    rng = np.random.default_rng(m)
    k, bits, block = 512, 8, 64
    a = rng.standard_normal((m, k), dtype=F)
    specs = [("gate", 176, False, False), ("up", 100, True, False), ("third", 48, False, True)]  # name, N, constant C per column, input scales
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), "Split sp 1 3 a a_g a_u a_t"]
    blob, parts = b"", {}
    for name, n, with_c, insc in specs:
        w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
        packed, scales = oracle.blockquant_pack(w, bits, block)
        c = rng.standard_normal((1, n), dtype=F) if with_c else None
        ins = (0.75 + (np.arange(k) % 5) * 0.15).astype(F) if insc else None
        term = bits * 100 + (10 if insc else 0) + 1
        kw = dict(N=n, K=k, constantB=1, quantize_term=term, alpha=0.5 if with_c else 1.0)
        if with_c:
            kw.update(constantC=1, broadcast_type_C=4)
        line = mw.gemm_param(name, ["a_" + name[0]], name + "_out", **kw)
        piece = mw.weight_blob(packed.view(np.int8)) + (mw.weight_blob(c) if with_c else b"") + mw.raw_f32(scales) + (mw.raw_f32(ins) if insc else b"")
        lines.append(line)
        blob += piece
        parts[name] = (line.replace("a_" + name[0], "a"), piece, packed, scales, c, ins, kw.get("alpha", 1.0))
    net = _load(mw.assemble_param(lines), blob, True)
    ex = net.create_extractor()
    ex.input("a", a)
    got = {name: ex.extract(name + "_out") for name, _, _, _ in specs}
    for name, n, with_c, insc in specs:
        line, piece, packed, scales, c, ins, alpha = parts[name]
        alone = _single(["Input in0 0 1 a 0=%d 1=%d" % (k, m), line], piece, {"a": a}, name + "_out", True)
        assert np.array_equal(got[name], alone), name
        val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins, c, 4 if with_c else -1, alpha, 1.0)
        assert np.all(np.abs(got[name] - val) <= 1e-5 * floor + 1e-30), name


@RESIDENT
@pytest.mark.parametrize("spec", cases.MHA_CASES, ids=[str(c[0]) for c in cases.MHA_CASES])
def test_multiheadattention_layer_block_quant(spec, resident):
    """MultiHeadAttention with block-quantised weights through load_param / load_model / forward, against the oracle:
    every arrangement of inputs the layer knows (self / cross attention, shared or per-head mask, cache in and out), on
    host blobs and with every blob (the caches and the per-head mask included) resident in HBM."""
    case = cases.mha_case(*spec)
    seed, e, heads, qdim, kdim, vdim, src, cur, bits, block, insc, past, self_att, mask = spec
    term = bits * 100 + int(insc) * 10 + {32: 0, 64: 1, 128: 2}[block]
    feeds, lines, bottoms = {"q": case["q"]}, ["Input in_q 0 1 q 0=%d 1=%d" % (qdim, src)], ["q"]
    if not self_att or case["k"] is not case["q"]:
        feeds["k"] = case["k"]
        lines.append("Input in_k 0 1 k 0=%d 1=%d" % (kdim, cur))
        bottoms.append("k")
        if case["v"] is not case["k"]:
            feeds["v"] = case["v"]
            lines.append("Input in_v 0 1 v 0=%d 1=%d" % (vdim, cur))
            bottoms.append("v")
    self_layout = len(bottoms) == 1  # the layer itself tells self from cross attention by the number of q/k/v blobs
    if case["mask"] is not None:
        feeds["m"] = case["mask"]
        lines.append("Input in_m 0 1 m")
        bottoms.append("m")
    tops = ["out"]
    if past:
        feeds["ck"], feeds["cv"] = case["cached_k"], case["cached_v"]
        lines += ["Input in_ck 0 1 ck", "Input in_cv 0 1 cv"]
        bottoms += ["ck", "cv"]
        tops += ["ko", "vo"]
    lines.append(mw.mha_param("mha", bottoms, tops, e, heads, qdim, kdim, vdim, attn_mask=int(case["mask"] is not None), kv_cache=int(bool(past)),
                              quantize_term=term))
    net = host.Net()
    assert net.register_attention_layer() == 0
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(mw.assemble_param(lines)) == 0
    assert net.load_model_mem(mw.mha_blockquant_weights(case["weights"])) == 0
    ex = net.create_extractor()
    for name, value in feeds.items():
        ex.input(name, value)
    got = ex.extract("out")
    want, kw, vw = oracle.mha_blockquant(**dict(case, self_attention=self_layout))
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= 2e-5 * max(1.0, np.abs(want).max())
    if past:
        assert np.abs(ex.extract("ko") - kw).max() <= 1e-5 * max(1.0, np.abs(kw).max())
        assert np.abs(ex.extract("vo") - vw).max() <= 1e-5 * max(1.0, np.abs(vw).max())


@RESIDENT
def test_per_layer_timing_lists_every_layer_that_ran(resident):
    """The executor's per-layer timing (the reference's NCNN_BENCHMARK output): one record per layer run, in execution order,
    device layers timed by events, host layers by the wall clock; results are unchanged and nothing is recorded when off."""
    g, param, blob, info = zoo.build("tiny", seed=11)
    net = _load(param, blob, resident)
    x = np.random.default_rng(12).uniform(0, 1, g.input_shape).astype(F)
    want = refnet.run(param, blob, x)["fc"]
    ex = net.create_extractor()
    ex.set_layer_timing(True)
    ex.input("data", x)
    assert np.array_equal(ex.extract("fc").reshape(-1), want.reshape(-1))
    rows = ex.layer_timing()
    names = [r[2] for r in rows]
    assert "c1" in names and "fc" in names and names.index("c1") < names.index("fc")
    assert all(r[4] >= 0.0 and r[4] < 1000.0 for r in rows)
    where = {r[2]: r[3] for r in rows}
    assert where["fc"] == ("device" if resident else "host")
    assert sum(r[4] for r in rows) > 0.0
    ex2 = net.create_extractor()
    ex2.input("data", x)
    ex2.extract("fc")
    assert ex2.layer_timing() == []


def test_multiheadattention_layer_rejects_other_weight_formats():
    net = host.Net()
    assert net.register_attention_layer() == 0
    lines = ["Input in_q 0 1 q 0=64 1=4", mw.mha_param("mha", ["q"], ["out"], 64, 4, 64, quantize_term=0)]
    assert net.load_param_mem(mw.assemble_param(lines)) != 0  # fp32 weights: no silent fallback, the load fails


def test_innerproduct_layer_2d_rows_and_fp32_weights_quantised_at_load():
    rng = np.random.default_rng(6)
    rows, k, n = 5, 48, 12
    x = rng.uniform(-1, 1, (rows, k)).astype(F)
    wf = rng.normal(0, 0.1, (n, k)).astype(F)
    ws = (F(127) / np.abs(wf).max(axis=1)).astype(F)
    in_scale = F(127) / np.abs(x).max()
    b = rng.normal(size=n).astype(F)
    lines = ["Input in0 0 1 x 0=%d 1=%d" % (k, rows), mw.innerproduct_param("fc", "x", "out", n, n * k, 1, 2, 1)]
    blob = mw.conv_weights(wf.reshape(-1), b, ws, in_scale, None)  # fp32 weights in the file
    got = _single(lines, blob, {"x": x}, "out")
    wq = oracle.quantize_weights(wf, ws)
    assert np.array_equal(got, oracle.innerproduct_int8(x, wq, b, ws, in_scale, 1))


# ----------------------------------------------------------------------------- the two benchmark networks
@pytest.mark.parametrize("which,hw", [("resnet50", 224), ("mobilenetv2", 224)])
def test_benchmark_network_batch1_matches_oracle_executor(which, hw):
    _say("building", which)
    g, param, blob, info = zoo.build(which, input_hw=hw, n_calib=2)
    x = np.random.default_rng(9).uniform(0, 1, g.input_shape).astype(F)
    last_fc = "fc1000" if which == "resnet50" else "fc"
    _say("oracle forward", which)
    ref = refnet.run(param, blob, x, want=last_fc)
    for resident in (False, True):
        _say("device forward", which, "device-resident" if resident else "host blobs")
        net = _load(param, blob, resident)
        ex = net.create_extractor()
        ex.input("data", x)
        got = ex.extract(last_fc)
        assert np.array_equal(got, ref[last_fc])
        # a requantised (int8) blob deep in the net, bit for bit
        probe = "res4c_branch2b" if which == "resnet50" else "block10_dw"
        ex = net.create_extractor()
        ex.input("data", x)
        assert np.array_equal(ex.extract(probe), ref[probe].astype(F))
        if which == "resnet50":
            # the stem's convolution -> max pooling -> two quantising convolutions runs on quantised values when the
            # whole net is asked for; asked for by name, its blobs still come out as the model defines them (fp32)
            for name in ("conv1", "pool1"):
                ex = net.create_extractor()
                ex.input("data", x)
                got = ex.extract(name)
                assert got.dtype == F and np.array_equal(got, ref[name]), name
    # batch 2, device-resident: the folded batch equals the per-sample result
    xs = np.stack([x, x[:, ::-1].copy()])
    ex = net.create_extractor()
    ex.input("data", xs)
    got = ex.extract(last_fc)
    assert np.array_equal(got[0].reshape(-1), ref[last_fc])
    ex1 = net.create_extractor()
    ex1.input("data", xs[1])
    assert np.array_equal(got[1].reshape(-1), ex1.extract(last_fc).reshape(-1))


@pytest.mark.parametrize("which,batch", [("mobilenetv2", 32), ("resnet50", 16)])
def test_benchmark_batch_equals_the_per_sample_passes(which, batch):
    """At the benchmark's batch sizes the kernels take other variants than at batch 1 (several output rows per
    depthwise thread, the pointwise small-K kernel, other tiles and K splits).  Batch 1 is pinned on the oracle
    executor above; here the folded batch must reproduce, bit for bit, the logits and a requantised blob deep in the
    net of single-sample passes (samples 0, a middle one, the last), and ONE sample of the batch (the last) is also run
    through the oracle executor: its logits and the deep int8 blob must equal the folded batch's bit for bit."""
    _say("building", which)
    g, param, blob, info = zoo.build(which, input_hw=224, n_calib=1)
    net = _load(param, blob, True)
    xs = np.random.default_rng(21).uniform(0, 1, (batch,) + tuple(g.input_shape)).astype(F)
    last_fc = "fc1000" if which == "resnet50" else "fc"
    probe = "res2b_branch2b" if which == "resnet50" else "block2_dw"
    _say("oracle forward of the last sample", which)
    ref = refnet.run(param, blob, xs[batch - 1], want=last_fc)
    for name in (last_fc, probe):
        ex = net.create_extractor()
        ex.input("data", xs)
        got = np.asarray(ex.extract(name))
        assert got.shape[0] == batch
        assert np.array_equal(got[batch - 1].reshape(-1), np.asarray(ref[name], F).reshape(-1)), (name, "oracle")
        for i in (0, batch // 2 - 1, batch - 1):
            ex1 = net.create_extractor()
            ex1.input("data", xs[i])
            assert np.array_equal(got[i].reshape(-1), np.asarray(ex1.extract(name)).reshape(-1)), (name, i)


@pytest.mark.parametrize("m", [3, 16, 70])
def test_recorded_block_quant_gemm_replays_like_the_eager_pass(m):
    """A block-quantised Gemm layer inside a recorded pass, at row counts that take its three forms (the few-row kernel; the split pass
    + the weight-streaming kernel; the split pass + the tiled kernel, each with scratch borrowed from the command the graph owns):
    replays with new inputs equal the eager Extractor bit for bit."""
    n, k, bits, block = 48, 256, 8, 64
    rng = np.random.default_rng(m)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    lines = ["Input data 0 1 data 0=%d 1=%d" % (k, m), mw.gemm_param("g", ["data"], "out", N=n, K=k, constantB=1, quantize_term=bits * 100 + 1)]
    blob = mw.weight_blob(packed.view(np.int8)) + mw.raw_f32(scales)
    net = _load(mw.assemble_param(lines), blob, True)

    def eager(x):
        ex = net.create_extractor()
        ex.input("data", x)
        return np.asarray(ex.extract("out"))

    x0 = rng.standard_normal((m, k), dtype=F)
    graph = net.record("data", net.upload(x0), "out")
    graph.launch()
    graph.synchronize()
    assert np.array_equal(graph.output().to_numpy().reshape(m, n), eager(x0))
    for i in range(3):
        x = rng.standard_normal((m, k), dtype=F)
        want = eager(x)
        graph.update_input(x)
        graph.launch()
        graph.launch()
        graph.synchronize()
        assert np.array_equal(graph.output().to_numpy().reshape(m, n), want), i


@pytest.mark.parametrize("which,batch", [("tiny", 1), ("tiny", 3), ("mobilenetv2", 1), ("resnet50", 2)])
def test_recorded_pass_replays_like_the_eager_pass(which, batch):
    """A pass recorded into a graph and replayed: every replay, with new input values and with eager work and
    synchronisations in between, gives the eager Extractor's result bit for bit."""
    _say("building", which)
    kw = {} if which == "tiny" else {"input_hw": 96, "n_calib": 1}
    g, param, blob, info = zoo.build(which, **kw)
    out_name = {"tiny": "fc", "mobilenetv2": "fc", "resnet50": "fc1000"}[which]
    net = _load(param, blob, True)
    rng = np.random.default_rng(11)
    shape = (batch,) + tuple(g.input_shape)
    x0 = rng.uniform(0, 1, shape).astype(F)

    def eager(x):
        ex = net.create_extractor()
        ex.input("data", x if batch > 1 else x[0])
        return np.asarray(ex.extract(out_name)).reshape(batch, -1)

    xin = net.upload(x0 if batch > 1 else x0[0])
    graph = net.record("data", xin, out_name)
    graph.launch()
    graph.synchronize()
    assert np.array_equal(graph.output().to_numpy().reshape(batch, -1), eager(x0))
    for i in range(4):
        x = rng.uniform(0, 1, shape).astype(F)
        want = eager(x)  # eager work on another stream of the same net between the replays
        graph.update_input(x if batch > 1 else x[0])
        graph.launch()
        if i % 2:
            graph.launch()  # back-to-back replays of the same values
        graph.synchronize()
        got = graph.output().to_numpy().reshape(batch, -1)
        assert np.array_equal(got, want), i
