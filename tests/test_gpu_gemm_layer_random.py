"""The int8 Gemm layer through load_param / load_model / extract at seeded random forms, against the oracle.

Gemm::forward_int8 (src/layer/gemm.cpp:745-966) takes A, B and C each as a constant of the model or as a bottom blob, A
and B stored either way round, C in one of five broadcast shapes (named by a parameter when constant, found from its shape
when it is a blob), the output plain, transposed and / or as an N x 1 x M blob.  The forms are drawn here instead of listed,
with odd M, N, K; every one has to come out bit for bit the oracle's, on host Mats, on blobs that stay in HBM (where the
layer has to run as a device layer) and through the plug-in written against the reference's c_api.h."""
import os

import numpy as np
import pytest

from ncnn_amd import host, modelwriter as mw
from oracle import oracle

pytestmark = pytest.mark.gpu
F = np.float32
COUNT = int(os.environ.get("NCNN_RANDOM_LAYERS", "150"))  # NCNN_RANDOM_LAYERS=<count> widens the walk


def _pick(rng, options):
    return options[int(rng.integers(len(options)))]


def _plugin():
    import ctypes as C
    from ncnn_amd import build
    host.lib()
    if not os.path.exists(build.LIBPLUGIN):
        raise RuntimeError("%s is missing: build it with python ncnn_amd/build.py" % build.LIBPLUGIN)
    p = C.CDLL(build.LIBPLUGIN)
    p.ncnnhip_plugin_register.restype = C.c_int
    p.ncnnhip_plugin_register.argtypes = [C.c_void_p]
    return p


def _run(lines, blob, feeds, resident):
    net = host.Net()
    if resident == "plugin":
        # the layer as the C shim written against the reference's c_api.h supplies it (function-pointer table, host Mats)
        assert _plugin().ncnnhip_plugin_register(net.h_) == 0
        assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(blob) == 0
        ex = net.create_extractor()
        for k, v in feeds.items():
            ex.input(k, v)
        return ex.extract("out"), "plugin"
    assert net.register_int8_layers() == 0
    net.set_use_hip_compute(resident)
    assert net.load_param_mem(mw.assemble_param(lines)) == 0 and net.load_model_mem(blob) == 0
    ex = net.create_extractor()
    ex.set_layer_timing(True)
    for k, v in feeds.items():
        ex.input(k, v)
    got = ex.extract("out")
    where = {r[2]: r[3] for r in ex.layer_timing()}
    return got, where["g"]


@pytest.mark.parametrize("resident", [False, True, "plugin"], ids=["host-blobs", "device-resident", "plug-in"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_gemm_layer_form_matches_oracle(seed, resident):
    rng = np.random.default_rng(11000 + seed)
    m, n, k = int(rng.integers(1, 71)), int(rng.integers(1, 131)), int(rng.integers(1, 301))
    if m == n:
        n += 1  # a one-dimensional C of M values is told from one of N values by its length
    form_a = _pick(rng, ["blob", "blob", "blob stored K x M", "constant int8"])
    form_b = _pick(rng, ["blob", "blob stored K x N", "constant int8", "constant int8"])
    form_c = _pick(rng, ["none", "none", "constant", "constant", "blob"])
    bt = _pick(rng, [0, 1, 2, 3, 4]) if form_c != "none" else -1
    alpha, beta = _pick(rng, [1.0, 1.0, 0.5, 1.7, -1.0]), _pick(rng, [1.0, 1.0, 0.25, 2.0, -1.0])
    transpose, n1m = bool(rng.integers(2)), rng.random() < 0.25
    print("[case] random gemm layer", seed, resident if resident == "plugin" else "resident" if resident else "host", (m, n, k), "A:", form_a, "B:", form_b, "C:", form_c, bt,
          alpha, beta, "transposed" if transpose else "", "N1M" if n1m else "", flush=True)

    a = rng.standard_normal((m, k), dtype=F)
    b = (rng.standard_normal((n, k), dtype=F) * F(0.05)).astype(F)
    lines, feeds, bottoms, blob, tail = [], {}, [], b"", b""
    kw = dict(alpha=alpha, beta=beta, output_transpose=int(transpose), output_N1M=int(n1m), constantA=0, constantB=0, constantC=0)
    if form_a == "constant int8":
        sa = (F(127) / np.maximum(np.abs(a).max(axis=1), F(1e-6))).astype(F)
        aq = oracle.quantize(a, sa)  # one scale per row, as a constant int8 A carries them
        blob += mw.weight_blob(aq)
        tail += mw.raw_f32(sa)
        kw.update(constantA=1, M=m, K=k)
    else:
        aq, sa = oracle.gemm_quantize_rows(a)
        stored = a.T.copy() if form_a == "blob stored K x M" else a
        lines.append("Input in0 0 1 a 0=%d 1=%d" % (stored.shape[1], stored.shape[0]))
        feeds["a"] = stored
        bottoms.append("a")
        kw.update(transA=int(form_a == "blob stored K x M"))
    if form_b == "constant int8":
        bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
        sb = F(rng.uniform(20, 60))
        blob += mw.weight_blob(bq)
        tail += mw.raw_f32(sb)
        kw.update(constantB=1, N=n, K=k)
    else:
        bq, sb = oracle.gemm_quantize_tensor(b)
        stored = b.T.copy() if form_b == "blob stored K x N" else b
        lines.append("Input in1 0 1 b 0=%d 1=%d" % (stored.shape[1], stored.shape[0]))
        feeds["b"] = stored
        bottoms.append("b")
        kw.update(transB=int(form_b != "blob stored K x N"))
    c = None
    if form_c != "none":
        c = {0: rng.standard_normal(1), 1: rng.standard_normal(m), 2: rng.standard_normal((m, 1)), 3: rng.standard_normal((m, n)),
             4: rng.standard_normal((1, n))}[bt].astype(F)
        if form_c == "constant":
            blob += mw.weight_blob(c)
            kw.update(constantC=1, broadcast_type_C=bt)
            if not kw.get("M"):
                kw.update(M=m)
            if not kw.get("N"):
                kw.update(N=n)
        else:
            if bt in (0, 1):
                lines.append("Input in2 0 1 c 0=%d" % c.size)
            elif bt == 4 and rng.random() < 0.5:
                c = c.reshape(n)  # one value per column as a one-dimensional blob
                lines.append("Input in2 0 1 c 0=%d" % n)
            else:
                lines.append("Input in2 0 1 c 0=%d 1=%d" % (c.shape[1], c.shape[0]))
            feeds["c"] = c
            bottoms.append("c")
    if not bottoms:
        # every operand a constant: the layer still needs a bottom blob; hand C over as the blob instead
        c = rng.standard_normal((m, n)).astype(F)
        bt = 3
        blob = mw.weight_blob(aq) + mw.weight_blob(bq)
        kw.update(constantC=0, broadcast_type_C=0)
        lines.append("Input in2 0 1 c 0=%d 1=%d" % (n, m))
        feeds["c"] = c
        bottoms.append("c")
    lines.append(mw.gemm_param("g", bottoms, "out", **kw))
    got, where = _run(lines, blob + tail, feeds, resident)
    want = oracle.gemm_int8(aq, bq, sa, [sb], None if c is None else c.reshape(-1) if c.ndim == 1 else c, bt, alpha, beta, transpose)
    if n1m:
        want = want.reshape(want.shape[0], 1, want.shape[1])
    assert np.asarray(got).size == want.size and np.array_equal(np.asarray(got).reshape(want.shape), want)
    assert where == ("plugin" if resident == "plugin" else "device" if resident else "host")


@pytest.mark.parametrize("resident", [False, True, "plugin"], ids=["host-blobs", "device-resident", "plug-in"])
@pytest.mark.parametrize("seed", range(COUNT))
def test_random_block_quantised_gemm_layer_matches_float64(seed, resident):
    """Gemm::forward_weight_block_quantize (src/layer/gemm.cpp:339-483) as a layer: 4 / 6 / 8-bit weights in blocks of 32 / 64
    / 128, with and without per-K input scales, C absent, a constant of the model or the second bottom blob in any of its
    shapes, 1 to 140 activation rows, K in whole 16s (the matrix-core layouts) and not.  |got - value| <= 1e-5 * sum |a * w|
    against float64."""
    from tests import npref
    rng = np.random.default_rng(15000 + seed)
    bits, block, insc = _pick(rng, [8, 8, 4, 6]), _pick(rng, [32, 64, 64, 128]), bool(rng.integers(2))
    m = int(_pick(rng, [1, 1, 2, 3, 4, 5, 9, 16, 20, 33, 70, 140]))
    n = int(rng.integers(1, 200))
    k = int(_pick(rng, [16 * int(rng.integers(1, 40)), 64 * int(rng.integers(1, 80)), int(rng.integers(1, 700)), 4096 + 64 * int(rng.integers(0, 70))]))
    form_c = _pick(rng, ["none", "none", "constant", "blob"])
    bt = _pick(rng, [0, 1, 2, 3, 4]) if form_c != "none" else -1
    if m == n:
        n += 1
    alpha, beta = _pick(rng, [1.0, 0.5, -1.0]), _pick(rng, [1.0, 2.0, 0.25])
    print("[case] random block-quantised gemm layer", seed, resident, bits, block, insc, (m, n, k), "C:", form_c, bt, alpha, beta, flush=True)
    a = rng.standard_normal((m, k), dtype=F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    ins = rng.uniform(0.5, 1.5, k).astype(F) if insc else None
    term = bits * 100 + int(insc) * 10 + {32: 0, 64: 1, 128: 2}[block]
    lines, feeds, bottoms = ["Input in0 0 1 a 0=%d 1=%d" % (k, m)], {"a": a}, ["a"]
    kw = dict(N=n, K=k, constantB=1, quantize_term=term, alpha=alpha, beta=beta)
    blob = mw.weight_blob(packed.view(np.int8))
    c = None
    if form_c != "none":
        c = {0: rng.standard_normal(1), 1: rng.standard_normal(m), 2: rng.standard_normal((m, 1)), 3: rng.standard_normal((m, n)),
             4: rng.standard_normal((1, n))}[bt].astype(F)
        if form_c == "constant":
            blob += mw.weight_blob(c)
            kw.update(constantC=1, broadcast_type_C=bt, M=m)
        else:
            lines.append("Input in1 0 1 c 0=%d" % c.size if c.ndim == 1 else "Input in1 0 1 c 0=%d 1=%d" % (c.shape[1], c.shape[0]))
            feeds["c"] = c
            bottoms.append("c")
    blob += mw.raw_f32(scales) + (mw.raw_f32(ins) if insc else b"")
    lines.append(mw.gemm_param("g", bottoms, "out", **kw))
    got, where = _run(lines, blob, feeds, resident)
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins, c, bt, alpha, beta)
    assert got.shape == val.shape and np.all(np.abs(got - val) <= 1e-5 * floor + 1e-30)
    assert where == ("plugin" if resident == "plugin" else "device" if resident else "host")
