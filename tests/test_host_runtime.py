"""Host-side logic of the ncnn-API mirror (no GPU needed): .param parsing, .bin reading, Mat layout,
graph loading with the HIP layers registered, and the C-ABI symbol tables of both libraries."""
import ctypes as C
import os
import struct

import numpy as np
import pytest

import ncnn_amd
from ncnn_amd import hip, host

F = np.float32


def bits(f):
    return struct.unpack("<I", struct.pack("<f", f))[0]


# ----------------------------------------------------------------------------- symbols
def test_libncnnhip_exports_every_declared_symbol():
    lib = hip.lib()
    import re
    hdr = open(os.path.join(os.path.dirname(ncnn_amd.__file__), "..", "include", "ncnnhip.h")).read()
    declared = set(re.findall(r"\b(ncnnhip_[a-z0-9_]+)\s*\(", hdr))
    assert declared == set(hip.EXPORTED_SYMBOLS), declared ^ set(hip.EXPORTED_SYMBOLS)
    for name in declared:
        getattr(lib, name)


def test_libncnn_amd_exports_every_declared_symbol():
    lib = host.lib()
    import re
    hdr = open(os.path.join(os.path.dirname(ncnn_amd.__file__), "..", "include", "ncnn_amd_c_api.h")).read()
    declared = set(re.findall(r"\b(ncnn(?:hip)?_[a-z0-9_]+)\s*\((?!\*)", hdr))  # (not the return types of function-pointer members)
    assert len(declared) > 90
    for name in declared:
        getattr(lib, name)


# ----------------------------------------------------------------------------- ParamDict
def test_paramdict_ints_floats_arrays():
    t, v, arr = host.paramdict_probe("0=64 1=3 11=5 9=1 18=2.5 10=0.0,6.0 6=36864 -23303=3,1,2,3\n", 0)
    assert (t, v) == (2, 64)
    assert host.paramdict_probe("0=64 18=2.5\n", 18)[:2] == (3, bits(2.5))
    t, n, arr = host.paramdict_probe("10=0.0,6.0 0=1\n", 10)
    assert t == 6 and n == 2 and arr[:2] == [bits(0.0), bits(6.0)]
    t, n, arr = host.paramdict_probe("-23303=3,1,2,3 0=1\n", 3)
    assert t == 5 and n == 3 and arr[:3] == [1, 2, 3]
    t, n, arr = host.paramdict_probe("-23310=2,0.000000e+00,6.000000e+00\n", 10)
    assert t == 6 and arr[:2] == [bits(0.0), bits(6.0)]
    assert host.paramdict_probe("0=1\n", 5)[0] == 0  # unset


def test_paramdict_int_literal_read_as_float_is_the_bit_pattern():
    # "0=1" for a float parameter yields the int's bits (1.4e-45), as in the reference's union storage
    t, v, _ = host.paramdict_probe("0=1\n", 0)
    assert t == 2 and v == 1


@pytest.mark.parametrize("text,want", [("1.25", 1.25), ("-0.5", -0.5), ("6.000000e+00", 6.0), ("1.234567e-01", None), ("3.e2", 300.0),
                                         ("1e-3", None), ("+2.5E1", 25.0), ("0.1", None), ("123456.789", None), ("7.0e-10", None)])
def test_paramdict_float_parser_follows_the_reference_recipe(text, want):
    # recipe: uint digits -> double (whole + frac/10^n), scaled by repeated *1e8 / *10, then rounded to float
    def recipe(s):
        neg = s.startswith("-")
        s = s.lstrip("+-")
        mant, _, ex = s.lower().partition("e")
        whole, _, frac = mant.partition(".")
        v = float(int(whole or "0") & 0xffffffff)
        if frac:
            v += (int(frac) & 0xffffffff) / float((10 ** len(frac)) & 0xffffffff)
        if ex:
            eneg = ex.startswith("-")
            e = int(ex.lstrip("+-"))
            scale = 1.0
            while e >= 8:
                scale *= 1e8
                e -= 8
            while e > 0:
                scale *= 10.0
                e -= 1
            v = v / scale if eneg else v * scale
        return np.float32(-v if neg else v)
    t, v, _ = host.paramdict_probe("3=%s\n" % text, 3)
    assert t == 3 and v == bits(float(recipe(text)))
    if want is not None:
        assert v == bits(want)


def test_paramdict_rejects_id_out_of_range():
    assert host.paramdict_probe("40=1\n", 0)[0] == -1


# ----------------------------------------------------------------------------- ModelBin
def test_modelbin_tags():
    w = np.array([1.5, -2.0, 3.25], F)
    q = np.array([1, -2, 3, -127, 127], np.int8)
    assert np.array_equal(host.modelbin_probe(host.tagged_fp32(w), 3, 0)[0], w)
    got, used = host.modelbin_probe(host.tagged_int8(q), 5, 0)
    assert got.dtype == np.int8 and np.array_equal(got, q) and used == 4 + 8  # payload padded to 4 bytes
    h = np.array([0.5, -1.0, 65504.0], np.float16)
    got, used = host.modelbin_probe(host.tagged_fp16(h), 3, 0)
    assert np.array_equal(got, h.astype(F)) and used == 4 + 8
    got, used = host.modelbin_probe(w.tobytes(), 3, 1)
    assert np.array_equal(got, w) and used == 12
    raw = struct.pack("<I", 0x0002C056) + w.tobytes()
    assert np.array_equal(host.modelbin_probe(raw, 3, 0)[0], w)
    # table-coded weights: 256-entry fp32 table + one index byte per weight
    table = np.arange(256, dtype=F) * F(0.5)
    idx = np.array([3, 200, 7], np.uint8)
    blob = struct.pack("<I", 0x01020304) + table.tobytes() + idx.tobytes() + b"\0"
    assert np.array_equal(host.modelbin_probe(blob, 3, 0)[0], table[idx])


# ----------------------------------------------------------------------------- Mat layout
@pytest.mark.parametrize("w,h,c,es,n", [(56, 56, 64, 4, 1), (58, 58, 3, 1, 1), (7, 7, 5, 4, 3), (224, 224, 3, 4, 16), (3, 3, 2, 1, 2)])
def test_mat_cstep_and_nstep_rules(w, h, c, es, n):
    m = host.Mat.batch3d(w, h, c, es, n)
    cstep = ((w * h * es + 15) // 16) * 16 // es
    assert m.cstep == cstep
    if n > 1:
        assert m.nstep == ((cstep * c * es + 4095) // 4096) * 4096 // es
    else:
        assert m.nstep == cstep * c
    assert (m.dims, m.w, m.h, m.c, m.n, m.elemsize) == (3, w, h, c, n, es)


# ----------------------------------------------------------------------------- graph loading
PARAM = """7767517
7 8
Input            data    0 1 data 0=8 1=8 2=4
Convolution      c1      1 1 data c1 0=6 1=3 4=1 5=1 6=216 8=102 9=1
Split            sp      1 2 c1 c1a c1b
ConvolutionDepthWise dw  1 1 c1a dw 0=6 1=3 4=1 5=1 6=54 7=6 8=1 9=3 -23310=2,0.0,6.0
Convolution      c2      1 1 c1b c2 0=6 1=1 5=0 6=36 8=2
Eltwise          add     2 1 dw c2 sum 0=1
ReLU             relu    1 1 sum out
"""


def test_load_param_with_hip_layers_registered():
    net = host.Net()
    net.register_int8_layers()
    assert net.load_param_mem(PARAM) == 0
    assert net.layer_types() == ["Input", "Convolution", "Split", "ConvolutionDepthWise", "Convolution", "Eltwise", "ReLU"]
    flags = net.layer_flags()
    # Convolution: one_blob_only, not inplace, int8 storage, batch folding, no packing
    assert flags[1] == 1 | 4 | 8 and flags[3] == 1 | 4 | 8
    assert net.input_names() == ["data"] and net.output_names() == ["out"]
    blobs = net.blobs()
    assert blobs["c1"] == (1, 2) and blobs["c1a"] == (2, 3) and blobs["sum"] == (5, 6) and blobs["out"] == (6, -1)


def test_python_wrappers_destroy_extractors_before_their_net_whatever_the_finaliser_order():
    """Objects that die in one pass of the cyclic garbage collector (held, say, by the traceback of a failed test) are
    finalised in any order; an extractor destroyed after its net would hand its command back to freed memory.  The net's
    finaliser therefore destroys what lives on it first, and the extractor's own finaliser finds nothing left to do."""
    import gc
    net = host.Net()
    net.register_int8_layers()
    assert net.load_param_mem(PARAM) == 0
    exs = [net.create_extractor(), net.create_extractor(own_stream=False)]
    assert len(net._owned) == 2 and all(len(e._owned.pairs) >= 1 for e in exs)
    host.Net.__del__(net)  # the net first, as the collector may do
    assert net.h_ is None and not net._owned and all(e._owned.pairs == [] for e in exs)
    for e in exs:
        host.Extractor.__del__(e)  # nothing is destroyed twice
    # and the ordinary order: an extractor that goes first takes its record off the net
    net2 = host.Net()
    ex = net2.create_extractor()
    assert len(net2._owned) == 1
    del ex
    gc.collect()
    assert not net2._owned


def test_hot_layers_have_no_host_fallback():
    # without the HIP layers a net using Convolution cannot even be built
    net = host.Net()
    assert net.load_param_mem(PARAM) != 0


def test_non_quantised_convolution_is_refused():
    net = host.Net()
    net.register_int8_layers()
    bad = PARAM.replace("8=102 9=1", "9=1")
    assert net.load_param_mem(bad) != 0


@pytest.mark.skipif(os.path.exists("/dev/kfd"), reason="checks the failure mode on a machine without a GPU")
def test_load_model_fails_loudly_without_a_gpu():
    from ncnn_amd import modelwriter
    rng = np.random.default_rng(0)
    net = host.Net()
    net.register_int8_layers()
    assert net.load_param_mem(PARAM) == 0
    binimg = b"".join([
        modelwriter.conv_weights(rng.integers(-127, 128, 216).astype(np.int8), rng.normal(size=6).astype(F), np.full(6, 50, F), 20.0, 10.0),
        modelwriter.conv_weights(rng.integers(-127, 128, 54).astype(np.int8), rng.normal(size=6).astype(F), np.full(6, 50, F), 10.0, None),
        modelwriter.conv_weights(rng.integers(-127, 128, 36).astype(np.int8), None, np.full(6, 50, F), 10.0, None),
    ])
    assert net.load_model_mem(binimg) != 0  # create_pipeline needs the device


# ---- packed block-quant layouts: what the kernel's lanes load, undone in numpy -------------------------------------------

def _unpack_tiles(pw, n, k, bits, block):
    """Inverse of ncnnhip_blockquant_pack's weight layout, written from the layout's description in include/ncnnhip.h:
    int [tiles*16][steps*64], fields back to signed values."""
    tiles, steps = (n + 15) // 16, (k + 63) // 64
    halves = bits != 8 or block == 32
    chunk = np.asarray(pw, np.uint8).reshape(tiles, steps, 128 * bits)
    u = np.zeros((tiles, steps, 64, 16), np.int64)  # [lane][field]
    if bits == 8:
        u[:] = chunk.reshape(tiles, steps, 64, 16)
    elif bits == 4:
        d = chunk.reshape(tiles, steps, 64, 8).copy().view(np.uint32).astype(np.int64)  # [lane][2 dwords]
        for e in range(16):
            u[..., e] = (d[..., e >> 3] >> (4 * ((e & 7) >> 1) + 16 * (e & 1))) & 15
    else:
        d01 = chunk[..., :512].reshape(tiles, steps, 64, 8).copy().view(np.uint32).astype(np.int64)
        d2 = chunk[..., 512:].reshape(tiles, steps, 64, 4).copy().view(np.uint32).astype(np.int64)[..., 0]
        d = [d01[..., 0], d01[..., 1], d2]
        for pair in range(8):
            for hi in range(2):
                if pair < 6:
                    v = (d[pair >> 1] >> (6 * (pair & 1) + 16 * hi)) & 63
                else:
                    v = ((d[pair - 6] >> (12 + 16 * hi)) & 15) | (((d[2] >> (12 + 2 * (pair - 6) + 16 * hi)) & 3) << 4)
                u[..., 2 * pair + hi] = v
    q = np.zeros((tiles * 16, steps * 64), np.int64)
    for l in range(64):
        for e in range(16):
            kk = (e >> 3) * 32 + (l >> 4) * 8 + (e & 7) if halves else (l >> 4) * 16 + e
            q[(l & 15)::16, kk::64] = u[:, :, l, e]
    return q - (1 << (bits - 1))


@pytest.mark.parametrize("bits", [4, 6, 8])
@pytest.mark.parametrize("block", [32, 64, 128])
@pytest.mark.parametrize("n,k", [(16, 64), (37, 208), (5, 4096 + 48), (33, 96)])
def test_blockquant_pack_layouts_hold_every_field_and_descale(bits, block, n, k):
    from ncnn_amd import synth
    import npref
    rng = np.random.default_rng(bits * 1000 + block + n + k)
    packed, scales = synth.blockquant_weights(rng.standard_normal((n, k)).astype(np.float32), bits, block)
    lib = hip.lib()
    wb, db = C.c_size_t(), C.c_size_t()
    assert lib.ncnnhip_blockquant_packed_size(n, k, bits, block, C.byref(wb), C.byref(db)) == 0
    tiles, steps, nblk = (n + 15) // 16, (k + 63) // 64, (k + block - 1) // block
    per_step = 2 if block == 32 else 1
    assert wb.value == tiles * steps * 128 * bits and db.value == tiles * steps * 16 * 4 * per_step
    pw = np.full(wb.value, 0xA5, np.uint8)
    pd = np.full(db.value // 4, np.nan, np.float32)
    assert lib.ncnnhip_blockquant_pack(packed.ctypes.data, scales.ctypes.data, n, k, bits, block, pw.ctypes.data, pd.ctypes.data) == 0
    q = _unpack_tiles(pw, n, k, bits, block)
    want = np.zeros_like(q)
    want[:n, :k] = npref.blockquant_unpack_all(packed, k, bits)  # padding rows / K hold zeros
    assert np.array_equal(q, want)
    d = pd.reshape(tiles, steps, per_step, 16)
    with np.errstate(divide="ignore"):
        inv = (np.float32(1) / scales).astype(np.float32)
    for t in range(tiles):
        for s in range(steps):
            for h in range(per_step):
                blk = (s * 64 + h * 32) // block
                for r in range(16):
                    j = t * 16 + r
                    want_d = inv[j, blk] if (j < n and blk < nblk) else np.float32(0)
                    assert d[t, s, h, r] == want_d, (t, s, h, r)


def test_blockquant_pack_refuses_what_has_no_kernel():
    lib = hip.lib()
    wb, db = C.c_size_t(), C.c_size_t()
    assert lib.ncnnhip_blockquant_packed_size(16, 16384 + 64, 4, 64, C.byref(wb), C.byref(db)) != 0  # the halves layout stops at K = 16384
    assert lib.ncnnhip_blockquant_packed_size(16, 16384 + 64, 8, 64, C.byref(wb), C.byref(db)) == 0
    assert lib.ncnnhip_blockquant_packed_size(16, 64, 5, 64, C.byref(wb), C.byref(db)) != 0
    assert lib.ncnnhip_blockquant_packed_size(16, 64, 8, 48, C.byref(wb), C.byref(db)) != 0


def test_packed_blockquant_entry_points_refuse_bad_arguments_before_touching_the_device():
    """Argument checks come first, so they can be exercised without a GPU: every call below must return an error code
    (never crash, never report success)."""
    lib = hip.lib()
    fake = C.c_void_p(0x1000)  # never dereferenced: the calls stop at their checks
    wsb = C.c_size_t()
    assert lib.ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(70, 4096 + 16, C.byref(wsb)) == 0
    assert wsb.value == 3 * 128 * (4096 + 64) * 2  # rows and K rounded up to 64, three bf16 planes
    assert lib.ncnnhip_gemm_blockquant_packed_rows_workspace_bytes(0, 64, C.byref(wsb)) != 0
    rows = lib.ncnnhip_gemm_blockquant_packed_rows
    few = lib.ncnnhip_gemm_blockquant_packed
    half = lib.ncnnhip_gemm_blockquant_packed_f16a
    ok_rows = dict(a=fake, stride=64, m=8, n=16, k=64, w=fake, d=fake, bits=8, block=64, ins=None, c=None, bt=-1, out=fake, ostride=16, ws=fake, wsb=1 << 20)

    def call_rows(**kw):
        p = dict(ok_rows, **kw)
        return rows(p["a"], p["stride"], p["m"], p["n"], p["k"], p["w"], p["d"], p["bits"], p["block"], p["ins"], p["c"], p["bt"], 1.0, 1.0, p["out"], p["ostride"],
                    p["ws"], p["wsb"], None)

    assert call_rows(a=None) != 0 and call_rows(w=None) != 0 and call_rows(out=None) != 0 and call_rows(ws=None) != 0
    assert call_rows(k=72) != 0            # K % 16
    assert call_rows(bits=5) != 0 and call_rows(block=48) != 0
    assert call_rows(stride=32) != 0 and call_rows(ostride=8) != 0
    assert call_rows(wsb=1024) != 0        # workspace too small
    assert call_rows(c=fake, bt=7) != 0
    assert call_rows(bits=4, k=16384 + 64) != 0  # the halves layout stops at K = 16384
    assert few(fake, 64, 1, 16, 72, fake, fake, 8, 64, None, None, -1, 1.0, 1.0, fake, 16, None) != 0
    assert few(fake, 64, 1, 16, 64, fake, fake, 8, 64, C.c_void_p(0x1004), None, -1, 1.0, 1.0, fake, 16, None) != 0  # input scales not 16-byte aligned
    assert few(C.c_void_p(0x1004), 64, 1, 16, 64, fake, fake, 8, 64, None, None, -1, 1.0, 1.0, fake, 16, None) != 0
    assert few(fake, 64, 1, 16, 16384 + 64, fake, fake, 8, 64, None, None, -1, 1.0, 1.0, fake, 16, None) != 0       # fp32 rows: K <= 16384
    assert half(fake, 60, 1, 16, 64, fake, fake, 8, 64, None, -1, 1.0, 1.0, fake, 16, None) != 0                    # row stride below K
    assert lib.ncnnhip_gemm_blockquant_packed_supported(4096) == 1 and lib.ncnnhip_gemm_blockquant_packed_supported(4100) == 0
    assert lib.ncnnhip_gemm_blockquant_packed_supported(16384 + 16) == 0
    assert b"ncnnhip_gemm_blockquant_packed" in lib.ncnnhip_last_error()


def test_every_entry_point_survives_null_arguments():
    """Every exported function of the kernel library called with null pointers and zero sizes: an error code (or, for the
    queries and the releases of nothing listed below, 0), never a crash.  The checks come before anything touches the device,
    so this runs without a GPU; it runs in a child process so that a crash fails this test instead of ending the run."""
    import subprocess
    import sys
    code = r'''
import ctypes as C, sys
sys.path.insert(0, %r)
from ncnn_amd import hip
lib = hip.lib()
benign = {"ncnnhip_conv_from_float_supported", "ncnnhip_conv_fusion_supported", "ncnnhip_conv_small_tile_selected", "ncnnhip_conv_stem_supported",
          "ncnnhip_gemm_blockquant_packed_supported", "ncnnhip_padded_channels",                      # queries: 0 = no
          "ncnnhip_default_device_free", "ncnnhip_free", "ncnnhip_event_destroy", "ncnnhip_graph_destroy", "ncnnhip_stream_destroy",  # release of nothing
          "ncnnhip_memcpy_d2d", "ncnnhip_memcpy_d2h", "ncnnhip_memcpy_h2d", "ncnnhip_memset",            # zero bytes
          "ncnnhip_set_device_allocator"}                                                                # back to the default allocator
bad = []
for name in sorted(hip._SIGNATURES):
    args = []
    for t in hip._SIGNATURES[name]:
        if t in (C.c_int, C.c_size_t):
            args.append(0)
        elif t is C.c_float:
            args.append(0.0)
        elif t is hip.Activation:
            args.append(hip.Activation.make(0, (0.0, 0.0)))
        else:
            args.append(None)
    print(name, flush=True)
    r = getattr(lib, name)(*args)
    if (r == 0) != (name in benign):
        bad.append((name, r))
print("BAD", bad)
sys.exit(1 if bad else 0)
''' % os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    p = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert p.returncode == 0, "last lines: %s %s" % (p.stdout.strip().splitlines()[-3:], p.stderr.strip().splitlines()[-3:])


@pytest.mark.parametrize("damage,what", [
    (("Convolution              c1                       1 1 data c1", "Convolution              c1                       -1 1 data c1"), "a negative bottom count"),
    (("Convolution              c1                       1 1 data c1", "Convolution              c1                       1 99999999 data c1"), "more top blobs than the net has"),
    ((" 9=1", " 9=1 -23310=-5,1"), "a counted array of negative length"),
    ((" 9=1", " 9=1 -23310=999999999,1"), "a counted array of absurd length"),
    (("7767517\n3 3", "7767517\n2000000000 3"), "an absurd layer count"),
    ((" 1=3 11=3 ", " 1=1133903872 11=3 "), "a kernel whose tap count overflows an int"),
    ((" 0=16 1=3 ", " 0=-16 1=3 "), "a negative num_output"),
])
def test_load_param_refuses_damaged_counts_and_sizes(damage, what):
    """Counts and sizes a model file cannot mean are answered with an error code, before anything is allocated or multiplied
    with them (found by mutating .param texts: a negative blob count reached std::vector::resize, a negative array length
    Mat::create)."""
    text = ("7767517\n3 3\nInput                    data                     0 1 data 0=16 1=16 2=4\n"
            "Convolution              c1                       1 1 data c1 0=16 1=3 11=3 2=1 3=1 4=1 5=1 6=576 8=101 9=1\n"
            "ReLU                     r                        1 1 c1 out\n")
    net = host.Net()
    net.register_int8_layers()
    assert net.load_param_mem(text) == 0
    old, new = damage
    assert old in text, what
    net = host.Net()
    net.register_int8_layers()
    assert net.load_param_mem(text.replace(old, new, 1)) != 0, what


def test_param_parser_survives_mutated_text():
    """600 mutated .param texts (tests/paramfuzz.py) in a child process: return codes, never a crash."""
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    p = subprocess.run([sys.executable, os.path.join(here, "paramfuzz.py"), "11", "600"], capture_output=True, text=True, timeout=300,
                       cwd=os.path.dirname(here), env=dict(os.environ, PYTHONPATH=os.path.dirname(here)))
    assert p.returncode == 0 and "survived 600" in p.stdout, (p.returncode, p.stdout[-300:], p.stderr[-600:])


def test_binary_param_loader_survives_mutated_files():
    """600 mutated .param.bin files (tests/paramfuzz.py) in a child process: return codes, never a crash."""
    import subprocess
    import sys
    here = os.path.dirname(os.path.abspath(__file__))
    p = subprocess.run([sys.executable, os.path.join(here, "paramfuzz.py"), "21", "600", "bin"], capture_output=True, text=True, timeout=300,
                       cwd=os.path.dirname(here), env=dict(os.environ, PYTHONPATH=os.path.dirname(here)))
    assert p.returncode == 0 and "survived 600" in p.stdout, (p.returncode, p.stdout[-300:], p.stderr[-600:])


def test_paramdict_text_parser_on_the_reference_tests_own_vectors():
    """tests/golden/paramdict_vectors.json: the inputs and expected values that the reference's tests/test_paramdict.cpp holds
    for the text parser (src/paramdict.cpp:263-489) -- types, ints, floats compared as float32 the way the reference test
    compares them (f != 0.01f), arrays with a trailing comma, bare and quoted strings."""
    import json
    here = os.path.dirname(os.path.abspath(__file__))
    data = json.load(open(os.path.join(here, "golden", "paramdict_vectors.json")))
    checked = 0
    for vec in data["vectors"]:
        for e in vec["expect"]:
            t, v, arr = host.paramdict_probe(vec["text"] + "\n", e["id"])
            assert t == e["type"], (vec["text"], e)
            if "int" in e:
                assert np.array([v], np.uint32).view(np.int32)[0] == e["int"]
            elif "float" in e:
                assert v == bits(float(np.float32(e["float"])))
            elif "ints" in e:
                assert v == len(e["ints"]) and list(np.array(arr[:v], np.uint32).view(np.int32)) == e["ints"]
            elif "floats" in e:
                assert v == len(e["floats"]) and arr[:v] == [bits(float(np.float32(f))) for f in e["floats"]]
            else:
                assert v == len(e["string"]) and bytes(arr[:v]).decode() == e["string"]
            checked += 1
    assert checked == 14
    # the binary form (ParamDict::load_param_bin, src/paramdict.cpp:491-637): the byte arrays of test_paramdict_3, _4, _5
    for vec in data["binary_vectors"]:
        mem = bytes.fromhex(vec["hex"])
        for e in vec["expect"]:
            t, v, arr = host.paramdict_probe_bin(mem, e["id"])
            assert t == e["type"], e
            if "int" in e:
                assert np.array([v], np.uint32).view(np.int32)[0] == e["int"]
            elif "float" in e:
                assert v == bits(float(np.float32(e["float"])))
            elif "ints" in e:
                assert v == len(e["ints"]) and list(np.array(arr[:v], np.uint32).view(np.int32)) == e["ints"]
            elif "floats" in e:
                assert v == len(e["floats"]) and arr[:v] == [bits(float(np.float32(f))) for f in e["floats"]]
            else:
                assert v == len(e["string"]) and bytes(arr[:v]).decode() == e["string"]
            checked += 1
    assert checked == 25
    # damaged binary forms are answered with -1: no end mark, an id out of range, a negative array length, a string too long
    import struct
    for bad in (struct.pack("<ii", 0, 5), struct.pack("<iii", 40, 1, -233), struct.pack("<iii", -23301, -4, -233), struct.pack("<iii", -23400, 300, -233)):
        assert host.paramdict_probe_bin(bad + b"\0" * 8, 0)[0] == -1


_GLUE_NET = ["Input in0 0 1 data 0=8 1=6 2=3", "Split sp 1 2 data a b", "ReLU r 1 1 a ra 0=1.000000e-01", "Pooling p 1 1 b pb 0=0 1=2 2=2",
             "Pooling p2 1 1 ra pa 0=1 1=2 2=2 -23330=4,3,4,3,3", "Eltwise e 2 1 pa pb out 0=1 -23301=2,5.000000e-01,2.000000e+00"]


def test_net_from_the_binary_param_form_equals_the_net_from_the_text(tmp_path):
    """Net::load_param_bin (src/net.cpp:1667-2018) on the binary form of a .param text as tools/ncnn2mem.cpp writes it:
    the same layers, fed and read by blob number (and by the number in decimal, this library's addition); a file cut short
    anywhere is refused."""
    from ncnn_amd import modelwriter as mw
    x = np.random.default_rng(0).normal(size=(3, 6, 8)).astype(np.float32)
    text_net = host.Net()
    assert text_net.load_param_mem(mw.assemble_param(_GLUE_NET)) == 0 and text_net.load_model_mem(b"") == 0
    ex = text_net.create_extractor()
    ex.input("data", x)
    want = ex.extract("out")
    data, number = mw.assemble_param_bin(_GLUE_NET)
    net = host.Net()
    assert net.load_param_bin_mem(data) == 0 and net.load_model_mem(b"") == 0
    assert net.layer_types() == text_net.layer_types() and net.input_names() == [str(number["data"])]
    ex = net.create_extractor()
    ex.input(number["data"], x)
    assert np.array_equal(ex.extract(number["out"]), want)
    ex = net.create_extractor()
    ex.input(str(number["data"]), x)
    assert np.array_equal(ex.extract(str(number["out"])), want)
    path = tmp_path / "net.param.bin"
    path.write_bytes(data)
    assert host.Net().load_param_bin(str(path)) == 0
    for cut in range(0, len(data), 3):
        path.write_bytes(data[:cut])
        assert host.Net().load_param_bin(str(path)) == -1, cut
    # a type number no layer has, a blob number beyond the count
    words = np.frombuffer(data, np.int32).copy()
    words[3] = 200
    path.write_bytes(words.tobytes())
    assert host.Net().load_param_bin(str(path)) == -1
    words = np.frombuffer(data, np.int32).copy()
    words[6] = 99
    path.write_bytes(words.tobytes())
    assert host.Net().load_param_bin(str(path)) == -1


def test_layer_type_numbers_are_the_references():
    """A .param.bin file names layer types by their place among the ncnn_add_layer calls of the reference's
    src/CMakeLists.txt; the library's table and the writer's have to hold those numbers."""
    from ncnn_amd import modelwriter as mw
    L = host.lib()
    for name, index in mw.LAYER_TYPE_INDEX.items():
        assert L.ncnn_layer_type_to_index(name.encode()) == index, name
    cmake = "/root/reference/src/CMakeLists.txt"
    if not os.path.exists(cmake):
        pytest.skip("the reference tree is not present on this machine")
    import re
    order = re.findall(r"^ncnn_add_layer\((\w+)", open(cmake).read(), re.M)
    for name, index in mw.LAYER_TYPE_INDEX.items():
        assert order.index(name) == index, name


def test_datareader_tables_feed_the_loaders():
    """The C API's datareader (src/c_api.h:218-235, 377-380): a table over bytes in memory, whose pointer moves on as the
    loaders read; a table whose read entry a C program replaced is the one the loader calls."""
    from ncnn_amd import modelwriter as mw
    L = host.lib()
    assert L.ncnn_version().startswith(b"1.0.") and L.ncnn_version_number() == int(L.ncnn_version()[4:])
    x = np.random.default_rng(1).normal(size=(3, 6, 8)).astype(np.float32)
    ref = host.Net()
    assert ref.load_param_mem(mw.assemble_param(_GLUE_NET)) == 0 and ref.load_model_mem(b"") == 0
    ex = ref.create_extractor()
    ex.input("data", x)
    want = ex.extract("out")

    text = mw.assemble_param(_GLUE_NET).encode() + b"\0"
    buf = C.create_string_buffer(text, len(text))
    cursor = C.c_char_p(C.addressof(buf))
    dr = L.ncnn_datareader_create_from_memory(C.byref(cursor))
    net = host.Net()
    assert L.ncnn_net_load_param_datareader(net.h_, dr) == 0
    moved = C.cast(cursor, C.c_void_p).value - C.addressof(buf)
    assert 0 < moved <= len(text)
    L.ncnn_datareader_destroy(dr)
    assert net.load_model_mem(b"") == 0
    ex = net.create_extractor()
    ex.input("data", x)
    assert np.array_equal(ex.extract("out"), want)

    # the binary form through a table whose read entry is the program's own
    data, number = mw.assemble_param_bin(_GLUE_NET)
    state = {"pos": 0, "calls": 0}
    READ = C.CFUNCTYPE(C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t)

    def read(_dr, out, size):
        chunk = data[state["pos"]: state["pos"] + size]
        C.memmove(out, chunk, len(chunk))
        state["pos"] += len(chunk)
        state["calls"] += 1
        return len(chunk)

    class Table(C.Structure):
        _fields_ = [("pthis", C.c_void_p), ("scan", C.c_void_p), ("read", READ)]

    dr = L.ncnn_datareader_create()
    table = C.cast(dr, C.POINTER(Table)).contents
    keep = READ(read)
    table.read = keep
    net = host.Net()
    assert L.ncnn_net_load_param_bin_datareader(net.h_, dr) == 0 and state["pos"] == len(data) and state["calls"] > 0
    L.ncnn_datareader_destroy(dr)
    assert net.load_model_mem(b"") == 0
    ex = net.create_extractor()
    ex.input(number["data"], x)
    assert np.array_equal(ex.extract(number["out"]), want)
    # a table that reads nothing: the loaders fail instead of reading stale memory
    dr = L.ncnn_datareader_create()
    assert L.ncnn_net_load_param_datareader(host.Net().h_, dr) == -1 and L.ncnn_net_load_param_bin_datareader(host.Net().h_, dr) == -1
    L.ncnn_datareader_destroy(dr)
