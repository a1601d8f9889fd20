"""plugin/ncnnhip_plugin.c: the four int8 layers as a plug-in for an unmodified ncnn, written against ncnn's public C API
(src/c_api.h:196-352) and the kernel library's C ABI only.

On the CPU: the file compiles, with every warning an error, against the reference's own c_api.h (its two generated headers come
from a cmake configure step in a temporary directory; skipped where the reference or cmake is absent), and it names nothing of
ncnn beyond what that header declares.  On the GPU: the same file, compiled against this repository's copy of the C API, is
registered on nets through its one entry point and every layer type is compared with the oracle."""
import ctypes as C
import os
import re
import shutil
import subprocess

import numpy as np
import pytest

from ncnn_amd import build, host, modelwriter as mw
from oracle import oracle

F = np.float32
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SOURCE = os.path.join(ROOT, "plugin", "ncnnhip_plugin.c")
REFERENCE = "/root/reference"


def _say(*a):
    print(*a, flush=True)


def _ncnn_names(text):
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return set(re.findall(r"\b_*ncnn_[A-Za-z0-9_]+\b", text))


def test_plugin_names_nothing_outside_the_two_public_headers():
    """Every ncnn_* identifier of the source is declared by this repository's copy of the C API, which
    test_reference_interface.py holds against the reference's header; every ncnnhip_* one by ncnnhip.h (its own entry point
    aside)."""
    used = _ncnn_names(open(SOURCE).read())
    api = _ncnn_names(open(os.path.join(ROOT, "include", "ncnn_amd_c_api.h")).read())
    kernels = set(re.findall(r"\bncnnhip_[A-Za-z0-9_]+\b", open(os.path.join(ROOT, "include", "ncnnhip.h")).read()))
    mine = {"ncnnhip_plugin_register"}
    unknown = {n for n in used if n not in api and n not in kernels and n not in mine and n != "ncnn_amd_c_api"}
    assert not unknown, sorted(unknown)
    assert not re.search(r"\bncnnhip_(layer_create_by_type|register_int8_layers|net_upload|extractor_)", open(SOURCE).read()), \
        "the plug-in must not lean on this repository's extensions of the C API"


@pytest.mark.skipif(not os.path.isdir(os.path.join(REFERENCE, "src")), reason="the reference tree is not on this machine")
@pytest.mark.skipif(shutil.which("cmake") is None, reason="cmake is not installed")
def test_plugin_compiles_against_the_reference_c_api_header(tmp_path):
    cfg = str(tmp_path / "cfg")
    r = subprocess.run(["cmake", "-S", REFERENCE, "-B", cfg, "-DNCNN_VULKAN=OFF", "-DNCNN_BUILD_TOOLS=OFF", "-DNCNN_BUILD_EXAMPLES=OFF",
                        "-DNCNN_BUILD_BENCHMARK=OFF", "-DNCNN_BUILD_TESTS=OFF", "-DNCNN_PYTHON=OFF"], capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-2000:]
    assert os.path.exists(os.path.join(cfg, "src", "platform.h")) and os.path.exists(os.path.join(cfg, "src", "ncnn_export.h"))
    r = subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I", os.path.join(REFERENCE, "src"),
                        "-I", os.path.join(cfg, "src"), "-I", os.path.join(ROOT, "include"), SOURCE], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr[-4000:]
    # and every ncnn_* name it uses is one that header declares
    declared = _ncnn_names(open(os.path.join(REFERENCE, "src", "c_api.h")).read())
    kernels = set(re.findall(r"\bncnnhip_[A-Za-z0-9_]+\b", open(os.path.join(ROOT, "include", "ncnnhip.h")).read()))
    used = {n for n in _ncnn_names(open(SOURCE).read()) if not n.startswith("ncnnhip_") and n != "ncnn_amd_c_api"}
    assert used <= declared, sorted(used - declared)
    assert {n for n in _ncnn_names(open(SOURCE).read()) if n.startswith("ncnnhip_")} <= kernels | {"ncnnhip_plugin_register"}


def test_plugin_library_exports_its_entry_point():
    if not os.path.exists(build.LIBPLUGIN):
        build.build_plugin()
    out = subprocess.run(["nm", "-D", "--defined-only", build.LIBPLUGIN], capture_output=True, text=True, check=True).stdout
    assert [l.split()[-1] for l in out.splitlines() if " T " in l] == ["ncnnhip_plugin_register"]
    undefined = subprocess.run(["nm", "-D", "--undefined-only", build.LIBPLUGIN], capture_output=True, text=True, check=True).stdout
    assert "ncnn_net_register_custom_layer_by_type" in undefined and "ncnnhip_conv_int8_nhwc" in undefined


# ----------------------------------------------------------------------------- on the GPU
def _plugin():
    host.lib()
    if not os.path.exists(build.LIBPLUGIN):
        raise RuntimeError("%s is missing: build it with python ncnn_amd/build.py" % build.LIBPLUGIN)
    P = C.CDLL(build.LIBPLUGIN)
    P.ncnnhip_plugin_register.restype = C.c_int
    P.ncnnhip_plugin_register.argtypes = [C.c_void_p]
    return P


def _load(param, blob):
    net = host.Net()
    assert _plugin().ncnnhip_plugin_register(net.h_) == 0
    assert net.load_param_mem(param) == 0
    assert net.load_model_mem(blob) == 0
    return net


def _single(lines, blob, feeds, out):
    net = _load(mw.assemble_param(lines), blob)
    ex = net.create_extractor()
    for k, v in feeds.items():
        ex.input(k, v)
    return ex.extract(out)


@pytest.mark.gpu
def test_tiny_net_through_the_plugin_matches_the_oracle_executor():
    """Convolution (fp32 and requantised outputs, fused activations), ConvolutionDepthWise and InnerProduct inside a net whose
    other layers are the library's own; two extractors in a row on the same layers (their scratch is reused)."""
    import refnet
    from ncnn_amd import zoo
    _say("plugin tiny net")
    g, param, blob, info = zoo.build("tiny", seed=11)
    net = _load(param, blob)
    rng = np.random.default_rng(12)
    for trial in range(2):
        x = rng.uniform(0, 1, g.input_shape).astype(F)
        ref = refnet.run(param, blob, x)
        ex = net.create_extractor()
        ex.input("data", x)
        for name in ("dw", "c3", "fc"):
            want = ref[name].astype(F) if ref[name].dtype == np.int8 else ref[name]
            assert np.array_equal(ex.extract(name), want), (trial, name)


@pytest.mark.gpu
@pytest.mark.parametrize("which", ["mobilenetv2", "resnet50"])
def test_benchmark_network_through_the_plugin(which):
    """Every Convolution / ConvolutionDepthWise / InnerProduct of the benchmark nets (at a 96-pixel input) through the plug-in's
    tables: the class scores and a requantised blob deep in the net, bit for bit."""
    import refnet
    from ncnn_amd import zoo
    _say("plugin", which)
    g, param, blob, info = zoo.build(which, input_hw=96, n_calib=2)
    net = _load(param, blob)
    x = np.random.default_rng(3).uniform(0, 1, g.input_shape).astype(F)
    last_fc = "fc1000" if which == "resnet50" else "fc"
    probe = "res4c_branch2b" if which == "resnet50" else "block10_dw"
    ref = refnet.run(param, blob, x, want=last_fc)
    ex = net.create_extractor()
    ex.input("data", x)
    assert np.array_equal(ex.extract(probe), ref[probe].astype(F))
    assert np.array_equal(ex.extract(last_fc), ref[last_fc])


@pytest.mark.gpu
def test_innerproduct_rows_and_fp32_weights_quantised_at_load():
    _say("plugin innerproduct")
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


@pytest.mark.gpu
def test_gemm_int8_constant_b_with_bias():
    _say("plugin gemm constant B")
    rng = np.random.default_rng(4)
    m, n, k = 37, 50, 96
    a = rng.standard_normal((m, k), dtype=F)
    bq = rng.integers(-127, 128, (n, k)).astype(np.int8)
    sb = F(63.5)
    c = rng.standard_normal((1, n), dtype=F)
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m),
             mw.gemm_param("g", ["a"], "out", M=0, N=n, K=k, constantB=1, constantC=1, broadcast_type_C=4, quantize_term=2)]
    blob = mw.weight_blob(bq) + mw.weight_blob(c) + mw.raw_f32(sb)
    got = _single(lines, blob, {"a": a}, "out")
    aq, sa = oracle.gemm_quantize_rows(a)
    assert np.array_equal(got, oracle.gemm_int8(aq, bq, sa, [sb], c, 4))


@pytest.mark.gpu
def test_gemm_int8_two_dynamic_operands_transposed_output():
    _say("plugin gemm dynamic operands")
    rng = np.random.default_rng(5)
    m, n, k = 20, 33, 64
    a = rng.standard_normal((m, k), dtype=F)
    b = (rng.standard_normal((k, n), dtype=F) * F(0.02)).astype(F)  # transB = 0: stored [K][N]
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), "Input in1 0 1 b 0=%d 1=%d" % (n, k),
             mw.gemm_param("g", ["a", "b"], "out", transB=0, constantB=0, quantize_term=2, output_transpose=1, alpha=0.5)]
    got = _single(lines, b"", {"a": a, "b": b}, "out")
    aq, sa = oracle.gemm_quantize_rows(a)
    bq, sb = oracle.gemm_quantize_tensor(b)
    assert np.array_equal(got, oracle.gemm_int8(aq, bq.T.copy(), sa, [sb], None, -1, 0.5, 1.0, True))


@pytest.mark.gpu
@pytest.mark.parametrize("bits,block,insc,m,n,k", [(8, 64, 0, 4, 24, 200), (4, 32, 1, 3, 24, 512), (6, 128, 0, 16, 40, 1024), (8, 64, 1, 1, 33, 256)])
def test_gemm_block_quant(bits, block, insc, m, n, k):
    import npref
    _say("plugin gemm block quant", bits, block, insc, m, n, k)
    rng = np.random.default_rng(bits + m + k)
    a = rng.standard_normal((m, k), dtype=F)
    w = (rng.standard_normal((n, k), dtype=F) * F(0.02)).astype(F)
    packed, scales = oracle.blockquant_pack(w, bits, block)
    ins = (0.75 + (np.arange(k) % 5) * 0.15).astype(F) if insc else None
    term = bits * 100 + insc * 10 + {32: 0, 64: 1, 128: 2}[block]
    lines = ["Input in0 0 1 a 0=%d 1=%d" % (k, m), mw.gemm_param("g", ["a"], "out", N=n, K=k, constantB=1, quantize_term=term)]
    blob = mw.weight_blob(packed.view(np.int8)) + mw.raw_f32(scales) + (mw.raw_f32(ins) if insc else b"")
    got = _single(lines, blob, {"a": a}, "out")
    val, floor = npref.blockquant_gemm_f64(a, packed, scales, bits, block, ins)
    assert np.all(np.abs(got - val) <= 1e-5 * floor + 1e-30)


@pytest.mark.gpu
def test_layers_without_a_quantisation_term_are_refused_at_load():
    _say("plugin refusal")
    net = host.Net()
    assert _plugin().ncnnhip_plugin_register(net.h_) == 0
    lines = ["Input in0 0 1 x 0=8 1=8 2=4", mw.conv_param("c", "x", "out", 4, 3, weight_size=4 * 4 * 9, term=0)]
    assert net.load_param_mem(mw.assemble_param(lines)) != 0
