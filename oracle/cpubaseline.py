"""ctypes front-end of the x86 VNNI Gemm in oracle/cpu_vnni_gemm.c: the benchmark's CPU baseline.

Test / benchmark infrastructure only; the product package never imports this module.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcpubaseline.so")
_lib = None


def build(force=False):
    src = os.path.join(_HERE, "cpu_vnni_gemm.c")
    if force or not os.path.exists(_LIB_PATH) or os.path.getmtime(_LIB_PATH) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcpubaseline.so"], stdout=subprocess.DEVNULL)
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.cpu_vnni_available.restype = C.c_int
        _lib.cpu_vnni_set_num_threads.restype = None
        _lib.cpu_vnni_set_num_threads.argtypes = [C.c_int]
        _lib.cpu_vnni_packed_bytes.restype = C.c_size_t
        _lib.cpu_vnni_packed_bytes.argtypes = [C.c_int, C.c_int]
        _lib.cpu_vnni_pack_b.restype = None
        _lib.cpu_vnni_pack_b.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p]
        _lib.cpu_vnni_gemm.restype = C.c_int
        _lib.cpu_vnni_gemm.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_int, C.c_void_p, C.c_void_p,
                                       C.c_size_t, C.c_void_p]
    return _lib


def available():
    return bool(lib().cpu_vnni_available())


def set_num_threads(n):
    lib().cpu_vnni_set_num_threads(int(n))


def pack_b(bq):
    bq = np.ascontiguousarray(bq, np.int8)
    n, k = bq.shape
    packed = np.empty(lib().cpu_vnni_packed_bytes(n, k), np.uint8)
    lib().cpu_vnni_pack_b(bq.ctypes.data, k, n, k, packed.ctypes.data)
    return packed


def gemm(a, packed, n, b_scales, bias=None, want_acc=False):
    """a fp32 [M][K] quantised per row inside; returns fp32 [M][N] (and the int32 sums)."""
    a = np.ascontiguousarray(a, np.float32)
    m, k = a.shape
    b_scales = np.ascontiguousarray(np.atleast_1d(b_scales), np.float32)
    bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
    out = np.empty((m, n), np.float32)
    acc = np.empty((m, n), np.int32) if want_acc else None
    rc = lib().cpu_vnni_gemm(a.ctypes.data, k, m, n, k, packed.ctypes.data, b_scales.ctypes.data, b_scales.size,
                             None if bias is None else bias.ctypes.data, out.ctypes.data, n, None if acc is None else acc.ctypes.data)
    if rc != 0:
        raise MemoryError("cpu_vnni_gemm")
    return (out, acc) if want_acc else out
