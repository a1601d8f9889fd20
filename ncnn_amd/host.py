"""ctypes binding of libncnn_amd.so (include/ncnn_amd_c_api.h): the ncnn-API mirror with the HIP layers.

The calls mirror ncnn's C API one to one: create a net, register the int8 layers, load_param, load_model,
create an extractor, input, extract."""
import ctypes as C
import os
import struct
import tempfile

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
# NCNN_AMD_HOST_LIB: another build of the same library (the sanitizer build of build.py --asan-host)
_LIB = os.environ.get("NCNN_AMD_HOST_LIB") or os.path.join(_PKG, "lib", "libncnn_amd.so")
_lib = None


# ---- struct __ncnn_layer_t / __ncnn_modelbin_t of include/ncnn_amd_c_api.h: tables of function pointers -----------------------
class LayerTable(C.Structure):
    pass


class ModelBinTable(C.Structure):
    pass


class AllocatorTable(C.Structure):
    pass


AllocatorTable._fields_ = [("pthis", C.c_void_p), ("fast_malloc", C.CFUNCTYPE(C.c_void_p, C.POINTER(AllocatorTable), C.c_size_t)),
                           ("fast_free", C.CFUNCTYPE(None, C.POINTER(AllocatorTable), C.c_void_p))]


_LT, _MT = C.POINTER(LayerTable), C.POINTER(ModelBinTable)
LayerTable._fields_ = [
    ("pthis", C.c_void_p),
    ("load_param", C.CFUNCTYPE(C.c_int, _LT, C.c_void_p)),
    ("load_model", C.CFUNCTYPE(C.c_int, _LT, _MT)),
    ("create_pipeline", C.CFUNCTYPE(C.c_int, _LT, C.c_void_p)),
    ("destroy_pipeline", C.CFUNCTYPE(C.c_int, _LT, C.c_void_p)),
    ("forward_1", C.CFUNCTYPE(C.c_int, _LT, C.c_void_p, C.POINTER(C.c_void_p), C.c_void_p)),
    ("forward_n", C.CFUNCTYPE(C.c_int, _LT, C.POINTER(C.c_void_p), C.c_int, C.POINTER(C.c_void_p), C.c_int, C.c_void_p)),
    ("forward_inplace_1", C.CFUNCTYPE(C.c_int, _LT, C.c_void_p, C.c_void_p)),
    ("forward_inplace_n", C.CFUNCTYPE(C.c_int, _LT, C.POINTER(C.c_void_p), C.c_int, C.c_void_p)),
]
ModelBinTable._fields_ = [
    ("pthis", C.c_void_p),
    ("load_1d", C.CFUNCTYPE(C.c_void_p, _MT, C.c_int, C.c_int)),
    ("load_2d", C.CFUNCTYPE(C.c_void_p, _MT, C.c_int, C.c_int, C.c_int)),
    ("load_3d", C.CFUNCTYPE(C.c_void_p, _MT, C.c_int, C.c_int, C.c_int, C.c_int)),
]
LAYER_CREATOR = C.CFUNCTYPE(C.c_void_p, C.c_void_p)  # (a ctypes callback cannot return a structure pointer: the address)
LAYER_DESTROYER = C.CFUNCTYPE(None, _LT, C.c_void_p)
LAYER_FLAGS = ("one_blob_only", "support_inplace", "support_vulkan", "support_packing", "support_bf16_storage", "support_fp16_storage",
               "support_vulkan_packing", "support_any_packing", "support_vulkan_any_packing")


OPTION_SWITCHES = ("use_vulkan_compute", "use_local_pool_allocator", "use_winograd_convolution", "use_sgemm_convolution", "use_packing_layout", "use_fp16_packed",
                   "use_fp16_storage", "use_fp16_arithmetic", "use_int8_packed", "use_int8_storage", "use_int8_arithmetic", "use_bf16_storage")


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB):
            raise RuntimeError("%s is missing: build it with python ncnn_amd/build.py" % _LIB)
        from . import hip
        hip.lib()  # libncnnhip.so first (same directory, found through rpath as well)
        L = C.CDLL(_LIB)
        vp, ci, cs = C.c_void_p, C.c_int, C.c_size_t
        sig = {
            "ncnn_allocator_create_pool_allocator": (C.POINTER(AllocatorTable), []), "ncnn_allocator_create_unlocked_pool_allocator": (C.POINTER(AllocatorTable), []),
            "ncnn_allocator_destroy": (None, [C.POINTER(AllocatorTable)]), "ncnn_option_set_blob_allocator": (None, [vp, C.POINTER(AllocatorTable)]),
            "ncnn_option_set_workspace_allocator": (None, [vp, C.POINTER(AllocatorTable)]),
            "ncnn_option_create": (vp, []), "ncnn_option_destroy": (None, [vp]), "ncnn_option_set_num_threads": (None, [vp, ci]),
            "ncnn_option_set_lightmode": (None, [vp, ci]), "ncnn_option_set_use_int8_inference": (None, [vp, ci]),
            "ncnn_option_get_use_int8_inference": (ci, [vp]),
            **{"ncnn_option_get_" + f: (ci, [vp]) for f in OPTION_SWITCHES}, **{"ncnn_option_set_" + f: (None, [vp, ci]) for f in OPTION_SWITCHES},
            "ncnn_option_set_use_hip_compute": (None, [vp, ci]), "ncnn_option_get_use_hip_compute": (ci, [vp]),
            "ncnn_mat_create_external_1d_elem": (vp, [ci, vp, cs, ci, vp]), "ncnn_mat_create_external_2d_elem": (vp, [ci, ci, vp, cs, ci, vp]),
            "ncnn_mat_create_external_3d_elem": (vp, [ci, ci, ci, vp, cs, ci, vp]), "ncnn_mat_create_3d_batch": (vp, [ci, ci, ci, ci, vp]),
            "ncnn_mat_create_3d_elem_batch": (vp, [ci, ci, ci, cs, ci, ci, vp]),
            "ncnn_mat_create": (vp, []), "ncnn_mat_create_1d_elem": (vp, [ci, cs, ci, vp]), "ncnn_mat_create_2d_elem": (vp, [ci, ci, cs, ci, vp]),
            "ncnn_mat_create_3d_elem": (vp, [ci, ci, ci, cs, ci, vp]),
            "ncnn_mat_create_1d": (vp, [ci, vp]), "ncnn_mat_create_2d": (vp, [ci, ci, vp]), "ncnn_mat_create_3d": (vp, [ci, ci, ci, vp]),
            "ncnn_mat_create_4d": (vp, [ci, ci, ci, ci, vp]), "ncnn_mat_create_1d_batch": (vp, [ci, ci, vp]), "ncnn_mat_create_2d_batch": (vp, [ci, ci, ci, vp]),
            "ncnn_mat_create_4d_batch": (vp, [ci, ci, ci, ci, ci, vp]), "ncnn_mat_create_external_1d": (vp, [ci, vp, vp]),
            "ncnn_mat_create_external_2d": (vp, [ci, ci, vp, vp]), "ncnn_mat_create_external_3d": (vp, [ci, ci, ci, vp, vp]),
            "ncnn_mat_create_external_4d": (vp, [ci, ci, ci, ci, vp, vp]), "ncnn_mat_create_4d_elem": (vp, [ci, ci, ci, ci, cs, ci, vp]),
            "ncnn_mat_create_1d_elem_batch": (vp, [ci, cs, ci, ci, vp]), "ncnn_mat_create_2d_elem_batch": (vp, [ci, ci, cs, ci, ci, vp]),
            "ncnn_mat_create_4d_elem_batch": (vp, [ci, ci, ci, ci, cs, ci, ci, vp]), "ncnn_mat_create_external_4d_elem": (vp, [ci, ci, ci, ci, vp, cs, ci, vp]),
            "ncnn_mat_fill_float": (None, [vp, C.c_float]), "ncnn_mat_clone": (vp, [vp, vp]), "ncnn_mat_reshape_1d": (vp, [vp, ci, vp]),
            "ncnn_mat_reshape_2d": (vp, [vp, ci, ci, vp]), "ncnn_mat_reshape_3d": (vp, [vp, ci, ci, ci, vp]), "ncnn_mat_get_channel_data": (vp, [vp, ci]),
            "ncnn_option_get_num_threads": (ci, [vp]), "ncnn_net_clear": (None, [vp]), "ncnn_net_get_input_index": (ci, [vp, ci]),
            "ncnn_net_get_output_index": (ci, [vp, ci]), "ncnn_extractor_input_index": (ci, [vp, ci, vp]),
            "ncnn_extractor_extract_index": (ci, [vp, ci, C.POINTER(vp)]),
            "ncnn_mat_destroy": (None, [vp]), "ncnn_mat_get_dims": (ci, [vp]), "ncnn_mat_get_w": (ci, [vp]), "ncnn_mat_get_h": (ci, [vp]),
            "ncnn_mat_get_d": (ci, [vp]), "ncnn_mat_get_c": (ci, [vp]), "ncnn_mat_get_n": (ci, [vp]), "ncnn_mat_get_elemsize": (cs, [vp]),
            "ncnn_mat_get_elempack": (ci, [vp]), "ncnn_mat_get_cstep": (cs, [vp]), "ncnn_mat_get_nstep": (cs, [vp]),
            "ncnn_mat_get_data": (vp, [vp]), "ncnn_mat_get_batch_data": (vp, [vp, ci]),
            "ncnn_net_create": (vp, []), "ncnn_net_destroy": (None, [vp]), "ncnn_net_get_option": (vp, [vp]), "ncnn_net_set_option": (None, [vp, vp]),
            "ncnn_net_load_param": (ci, [vp, C.c_char_p]), "ncnn_net_load_model": (ci, [vp, C.c_char_p]),
            "ncnn_net_load_param_bin": (ci, [vp, C.c_char_p]), "ncnn_net_load_param_bin_memory": (cs, [vp, C.c_char_p]),
            "ncnn_version": (C.c_char_p, []), "ncnn_version_number": (ci, []),
            "ncnn_datareader_create": (vp, []), "ncnn_datareader_create_from_memory": (vp, [C.POINTER(C.c_char_p)]),
            "ncnn_datareader_create_from_stdio": (vp, [vp]), "ncnn_datareader_destroy": (None, [vp]),
            "ncnn_modelbin_create_from_datareader": (vp, [vp]), "ncnn_net_load_param_datareader": (ci, [vp, vp]),
            "ncnn_net_load_param_bin_datareader": (ci, [vp, vp]), "ncnn_net_load_model_datareader": (ci, [vp, vp]),
            "ncnn_net_load_param_memory": (ci, [vp, C.c_char_p]), "ncnn_net_load_model_memory": (cs, [vp, C.c_char_p]),
            "ncnn_net_get_input_count": (ci, [vp]), "ncnn_net_get_output_count": (ci, [vp]),
            "ncnn_net_get_input_name": (C.c_char_p, [vp, ci]), "ncnn_net_get_output_name": (C.c_char_p, [vp, ci]),
            "ncnn_extractor_create": (vp, [vp]), "ncnn_extractor_destroy": (None, [vp]), "ncnn_extractor_set_option": (None, [vp, vp]),
            "ncnn_extractor_input": (ci, [vp, C.c_char_p, vp]), "ncnn_extractor_extract": (ci, [vp, C.c_char_p, C.POINTER(vp)]),
            "ncnnhip_register_int8_layers": (ci, [vp]), "ncnnhip_register_attention_layer": (ci, [vp]), "ncnnhip_extractor_attach_stream": (vp, [vp]), "ncnnhip_extractor_detach_stream": (None, [vp]),
            "ncnnhip_net_upload": (ci, [vp, vp, C.POINTER(vp)]), "ncnnhip_hipmat_destroy": (None, [vp]), "ncnnhip_hipmat_download": (ci, [vp, C.POINTER(vp)]),
            "ncnnhip_extractor_input_hipmat": (ci, [vp, C.c_char_p, vp]), "ncnnhip_extractor_extract_hipmat": (ci, [vp, C.c_char_p, C.POINTER(vp)]),
            "ncnnhip_extractor_synchronize": (ci, [vp]),
            "ncnnhip_extractor_set_layer_timing": (None, [vp, ci]), "ncnnhip_extractor_layer_timing": (ci, [vp, C.c_char_p, cs, C.POINTER(cs)]),
            "ncnnhip_graph_record": (ci, [vp, C.c_char_p, vp, C.c_char_p, C.POINTER(vp)]), "ncnnhip_graph_update_input": (ci, [vp, vp]),
            "ncnnhip_graph_replay": (ci, [vp]), "ncnnhip_graph_synchronize": (ci, [vp]), "ncnnhip_graph_output": (ci, [vp, C.POINTER(vp)]),
            "ncnnhip_graph_release": (None, [vp]),
            "ncnn_net_get_layer_count": (ci, [vp]), "ncnn_net_get_layer_type": (C.c_char_p, [vp, ci]), "ncnn_net_get_layer_name": (C.c_char_p, [vp, ci]),
            "ncnn_net_get_layer_flags": (ci, [vp, ci]), "ncnn_net_get_blob_count": (ci, [vp]), "ncnn_net_get_blob_name": (C.c_char_p, [vp, ci]),
            "ncnn_net_get_blob_producer": (ci, [vp, ci]), "ncnn_net_get_blob_consumer": (ci, [vp, ci]),
            # the layer half of the C API: parameter dictionaries, model readers, layers as function-pointer tables
            "ncnn_paramdict_create": (vp, []), "ncnn_paramdict_destroy": (None, [vp]), "ncnn_paramdict_get_type": (ci, [vp, ci]),
            "ncnn_paramdict_get_int": (ci, [vp, ci, ci]), "ncnn_paramdict_get_float": (C.c_float, [vp, ci, C.c_float]),
            "ncnn_paramdict_get_array": (vp, [vp, ci, vp]), "ncnn_paramdict_set_int": (None, [vp, ci, ci]),
            "ncnn_paramdict_set_float": (None, [vp, ci, C.c_float]), "ncnn_paramdict_set_array": (None, [vp, ci, vp]),
            "ncnn_modelbin_create_from_mat_array": (C.POINTER(ModelBinTable), [C.POINTER(vp), ci]), "ncnn_modelbin_destroy": (None, [C.POINTER(ModelBinTable)]),
            "ncnn_layer_create": (C.POINTER(LayerTable), []), "ncnn_layer_create_by_typeindex": (C.POINTER(LayerTable), [ci]),
            "ncnn_layer_create_by_type": (C.POINTER(LayerTable), [C.c_char_p]), "ncnn_layer_type_to_index": (ci, [C.c_char_p]),
            "ncnnhip_layer_create_by_type": (C.POINTER(LayerTable), [C.c_char_p]), "ncnn_layer_destroy": (None, [C.POINTER(LayerTable)]),
            "ncnn_layer_get_name": (C.c_char_p, [C.POINTER(LayerTable)]), "ncnn_layer_get_typeindex": (ci, [C.POINTER(LayerTable)]),
            "ncnn_layer_get_type": (C.c_char_p, [C.POINTER(LayerTable)]),
            "ncnn_layer_get_bottom_count": (ci, [C.POINTER(LayerTable)]), "ncnn_layer_get_bottom": (ci, [C.POINTER(LayerTable), ci]),
            "ncnn_layer_get_top_count": (ci, [C.POINTER(LayerTable)]), "ncnn_layer_get_top": (ci, [C.POINTER(LayerTable), ci]),
            "ncnn_blob_get_bottom_shape": (None, [C.POINTER(LayerTable), ci] + [C.POINTER(ci)] * 4),
            "ncnn_blob_get_top_shape": (None, [C.POINTER(LayerTable), ci] + [C.POINTER(ci)] * 4),
            "ncnn_net_register_custom_layer_by_type": (None, [vp, C.c_char_p, LAYER_CREATOR, LAYER_DESTROYER, vp]),
            "ncnn_net_register_custom_layer_by_typeindex": (None, [vp, ci, LAYER_CREATOR, LAYER_DESTROYER, vp]),
            "ncnn_paramdict_probe": (ci, [C.c_char_p, ci, C.POINTER(C.c_uint), C.POINTER(C.c_uint), ci]),
            "ncnn_paramdict_probe_bin": (ci, [C.c_char_p, ci, C.POINTER(C.c_uint), C.POINTER(C.c_uint), ci]),
            "ncnn_modelbin_probe": (ci, [C.c_char_p, ci, ci, vp, C.POINTER(cs)]),
        }
        for flag in LAYER_FLAGS:
            sig["ncnn_layer_get_" + flag] = (ci, [C.POINTER(LayerTable)])
            sig["ncnn_layer_set_" + flag] = (None, [C.POINTER(LayerTable), ci])
        for name, (res, args) in sig.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


# ---- probes (host logic tests) ---------------------------------------------------------------
def paramdict_probe(text, pid):
    v = C.c_uint(0)
    arr = (C.c_uint * 64)()
    t = lib().ncnn_paramdict_probe(text.encode(), pid, C.byref(v), arr, 64)
    return t, v.value, list(arr)


def paramdict_probe_bin(mem, pid):
    v = C.c_uint(0)
    arr = (C.c_uint * 64)()
    t = lib().ncnn_paramdict_probe_bin(bytes(mem), pid, C.byref(v), arr, 64)
    return t, v.value, list(arr)


def modelbin_probe(blob, w, load_type):
    out = np.zeros(w * 4 + 8, np.uint8)
    used = C.c_size_t(0)
    es = lib().ncnn_modelbin_probe(bytes(blob) + b"\0" * 16, w, load_type, out.ctypes.data, C.byref(used))
    if es == 0:
        return None, used.value
    dt = np.int8 if es == 1 else np.float32
    return out[: w * es].view(dt).copy(), used.value


def _pad4(b):
    return b + b"\0" * (-len(b) % 4)


def tagged_fp32(a):
    return struct.pack("<I", 0) + np.ascontiguousarray(a, np.float32).tobytes()


def tagged_fp16(a):
    return struct.pack("<I", 0x01306B47) + _pad4(np.ascontiguousarray(a, np.float16).tobytes())


def tagged_int8(a):
    return struct.pack("<I", 0x000D4B38) + _pad4(np.ascontiguousarray(a, np.int8).tobytes())


# ---- Mat -------------------------------------------------------------------------------------------
class Mat:
    """Owns an ncnn_mat_t; numpy <-> ncnn::Mat layout conversion (plane padding to 16 bytes, batch stride)."""

    def __init__(self, handle, keep=None):
        self.h_ = handle
        self._keep = keep

    def __del__(self):
        try:
            if self.h_:
                lib().ncnn_mat_destroy(self.h_)
        except Exception:
            pass

    dims = property(lambda s: lib().ncnn_mat_get_dims(s.h_))
    w = property(lambda s: lib().ncnn_mat_get_w(s.h_))
    h = property(lambda s: lib().ncnn_mat_get_h(s.h_))
    c = property(lambda s: lib().ncnn_mat_get_c(s.h_))
    n = property(lambda s: lib().ncnn_mat_get_n(s.h_))
    elemsize = property(lambda s: lib().ncnn_mat_get_elemsize(s.h_))
    cstep = property(lambda s: lib().ncnn_mat_get_cstep(s.h_))
    nstep = property(lambda s: lib().ncnn_mat_get_nstep(s.h_))

    @classmethod
    def batch3d(cls, w, h, c, elemsize, n):
        return cls(lib().ncnn_mat_create_3d_elem_batch(w, h, c, elemsize, 1, n, None))

    @classmethod
    def from_numpy(cls, a):
        """1-D [w], 2-D [h][w], 3-D [c][h][w] or 4-D [n][c][h][w] (a batch of 3-D blobs); fp32 or int8."""
        a = np.ascontiguousarray(a)
        assert a.dtype in (np.float32, np.int8)
        es = a.dtype.itemsize
        if a.ndim == 1:
            return cls(lib().ncnn_mat_create_external_1d_elem(a.shape[0], a.ctypes.data, es, 1, None), keep=a)
        if a.ndim == 2:
            return cls(lib().ncnn_mat_create_external_2d_elem(a.shape[1], a.shape[0], a.ctypes.data, es, 1, None), keep=a)
        if a.ndim == 3:
            a = a[None]
        n, c, h, w = a.shape
        m = cls.batch3d(w, h, c, es, n)
        for b in range(n):
            base = lib().ncnn_mat_get_batch_data(m.h_, b)
            buf = np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_uint8)), shape=(m.cstep * c * es,)).view(a.dtype).reshape(c, m.cstep)
            buf[:, : h * w] = a[b].reshape(c, h * w)
        return m

    def to_numpy(self):
        """1-D -> [w], 2-D -> [h][w], 3-D -> [c][h][w]; a batch adds a leading [n]."""
        es = self.elemsize
        dt = np.int8 if es == 1 else np.float32
        d, w, h, c, n = self.dims, self.w, self.h, self.c, self.n
        samples = []
        for b in range(n):
            base = lib().ncnn_mat_get_batch_data(self.h_, b)
            if d == 1:
                a = np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_uint8)), shape=(w * es,)).view(dt).copy()
            elif d == 2:
                a = np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_uint8)), shape=(w * h * es,)).view(dt).reshape(h, w).copy()
            else:
                buf = np.ctypeslib.as_array(C.cast(base, C.POINTER(C.c_uint8)), shape=(self.cstep * c * es,)).view(dt).reshape(c, self.cstep)
                a = buf[:, : h * w].reshape(c, h, w).copy()
            samples.append(a)
        return np.stack(samples) if n > 1 else samples[0]


# ---- Net / Extractor -------------------------------------------------------------------------------
class _Owned:
    """C handles that have to be destroyed before the Net they belong to.  The wrapper object and its Net both hold
    this record; whichever of the two is finalised first destroys the handles (when both die in one pass of the cyclic
    garbage collector -- e.g. held by the traceback of a failed test -- Python runs their finalisers in any order, and
    destroying an extractor after its net is a use after free)."""

    def __init__(self, net, *pairs):
        self.pairs = [(fn, h) for fn, h in pairs if h]
        self.net_records = net._owned
        self.net_records.add(self)

    def close(self):
        pairs, self.pairs = self.pairs, []
        for fn, h in pairs:
            try:
                getattr(lib(), fn)(h)
            except Exception:
                pass
        self.net_records.discard(self)


class HipMat:
    """Handle to a device-resident blob (keep the Net alive for as long as this exists)."""

    def __init__(self, handle, net):
        self.h_ = handle
        self.net = net

    def __del__(self):
        try:
            if self.h_:
                lib().ncnnhip_hipmat_destroy(self.h_)  # (a device blob shares its buffer pool and may outlive its net)
                self.h_ = None
        except Exception:
            pass

    def to_numpy(self):
        out = C.c_void_p()
        ret = lib().ncnnhip_hipmat_download(self.h_, C.byref(out))
        m = Mat(out.value)
        if ret != 0:
            raise RuntimeError("download returned %d" % ret)
        return m.to_numpy()


class HipGraph:
    """A forward pass recorded once (Net.record) and replayed with one launch; output() is rewritten by every replay."""

    def __init__(self, handle, net, keep):
        self.h_ = handle
        self.net = net
        self.keep = keep  # the input blob must outlive the recording

    def __del__(self):
        try:
            if self.h_:
                lib().ncnnhip_graph_release(self.h_)
                self.h_ = None
        except Exception:
            pass

    def update_input(self, array):
        m = array if isinstance(array, Mat) else Mat.from_numpy(array)
        ret = lib().ncnnhip_graph_update_input(self.h_, m.h_)
        if ret != 0:
            raise RuntimeError("update_input returned %d" % ret)

    def launch(self):
        ret = lib().ncnnhip_graph_replay(self.h_)
        if ret != 0:
            raise RuntimeError("graph launch returned %d" % ret)

    def synchronize(self):
        return lib().ncnnhip_graph_synchronize(self.h_)

    def output(self):
        out = C.c_void_p()
        lib().ncnnhip_graph_output(self.h_, C.byref(out))
        return HipMat(out.value, self.net)


class Net:
    def __init__(self):
        self.h_ = lib().ncnn_net_create()
        self._owned = set()  # _Owned records of the extractors that live on this net

    def record(self, input_name, input_blob, output_name):
        """Runs the pass from the resident input blob to output_name once, then records it for replay."""
        out = C.c_void_p()
        ret = lib().ncnnhip_graph_record(self.h_, input_name.encode(), input_blob.h_, output_name.encode(), C.byref(out))
        if ret != 0:
            raise RuntimeError("graph record returned %d" % ret)
        return HipGraph(out.value, self, input_blob)

    def upload(self, array):
        """numpy [c][h][w] / [n][c][h][w] -> device-resident blob usable as input of any extractor of this net."""
        m = array if isinstance(array, Mat) else Mat.from_numpy(array)
        out = C.c_void_p()
        ret = lib().ncnnhip_net_upload(self.h_, m.h_, C.byref(out))
        if ret != 0:
            raise RuntimeError("upload returned %d" % ret)
        return HipMat(out.value, self)

    def __del__(self):
        try:
            for rec in list(self._owned):  # the extractors first: they hand their command back to the net
                rec.close()
            if self.h_:
                lib().ncnn_net_destroy(self.h_)
                self.h_ = None
        except Exception:
            pass

    def register_custom_layer(self, type_name, creator, destroyer):
        """ncnn_net_register_custom_layer_by_type with Python callables: creator() -> ncnn_layer_t (a POINTER(LayerTable)),
        destroyer(layer).  The C thunks are kept alive with the net."""
        c = LAYER_CREATOR(lambda userdata: C.cast(creator(), C.c_void_p).value)
        d = LAYER_DESTROYER(lambda layer, userdata: destroyer(layer))
        self._custom = getattr(self, "_custom", []) + [(c, d)]
        lib().ncnn_net_register_custom_layer_by_type(self.h_, type_name.encode(), c, d, None)

    def register_attention_layer(self):
        return lib().ncnnhip_register_attention_layer(self.h_)

    def register_int8_layers(self):
        return lib().ncnnhip_register_int8_layers(self.h_)

    def set_use_int8_inference(self, enable):
        lib().ncnn_option_set_use_int8_inference(lib().ncnn_net_get_option(self.h_), int(enable))

    def set_lightmode(self, enable):
        lib().ncnn_option_set_lightmode(lib().ncnn_net_get_option(self.h_), int(enable))

    def set_use_hip_compute(self, enable):
        """Blobs stay in HBM between layers that have a device-resident overload; set before create_extractor."""
        lib().ncnn_option_set_use_hip_compute(lib().ncnn_net_get_option(self.h_), int(enable))

    def load_param(self, path):
        return lib().ncnn_net_load_param(self.h_, path.encode())

    def load_param_mem(self, text):
        return lib().ncnn_net_load_param_memory(self.h_, text.encode())

    def load_param_bin(self, path):
        return lib().ncnn_net_load_param_bin(self.h_, path.encode())

    def load_param_bin_mem(self, data):
        """The binary .param form: 0 when all of `data` was read as a net, -1 otherwise."""
        return 0 if lib().ncnn_net_load_param_bin_memory(self.h_, data) == len(data) else -1

    def load_model(self, path):
        return lib().ncnn_net_load_model(self.h_, path.encode())

    def load_model_mem(self, blob):
        # through a file so that the int status is visible (the memory variant returns bytes consumed, like ncnn's)
        with tempfile.NamedTemporaryFile(suffix=".bin") as f:
            f.write(blob)
            f.flush()
            return self.load_model(f.name)

    def layer_types(self):
        return [lib().ncnn_net_get_layer_type(self.h_, i).decode() for i in range(lib().ncnn_net_get_layer_count(self.h_))]

    def layer_names(self):
        return [lib().ncnn_net_get_layer_name(self.h_, i).decode() for i in range(lib().ncnn_net_get_layer_count(self.h_))]

    def layer_flags(self):
        return [lib().ncnn_net_get_layer_flags(self.h_, i) for i in range(lib().ncnn_net_get_layer_count(self.h_))]

    def input_names(self):
        return [lib().ncnn_net_get_input_name(self.h_, i).decode() for i in range(lib().ncnn_net_get_input_count(self.h_))]

    def output_names(self):
        return [lib().ncnn_net_get_output_name(self.h_, i).decode() for i in range(lib().ncnn_net_get_output_count(self.h_))]

    def blobs(self):
        out = {}
        for i in range(lib().ncnn_net_get_blob_count(self.h_)):
            out[lib().ncnn_net_get_blob_name(self.h_, i).decode()] = (lib().ncnn_net_get_blob_producer(self.h_, i), lib().ncnn_net_get_blob_consumer(self.h_, i))
        return out

    def create_extractor(self, own_stream=True):
        return Extractor(self, own_stream)


class Extractor:
    def __init__(self, net, own_stream=True):
        self.net = net
        self.h_ = lib().ncnn_extractor_create(net.h_)
        self.stream_handle = lib().ncnnhip_extractor_attach_stream(self.h_) if own_stream else None
        self._inputs = []
        self._owned = _Owned(net, ("ncnn_extractor_destroy", self.h_), ("ncnnhip_extractor_detach_stream", self.stream_handle))

    def __del__(self):
        self._owned.close()
        self.h_ = self.stream_handle = None

    def set_lightmode(self, enable):
        opt = lib().ncnn_option_create()
        lib().ncnn_option_set_lightmode(opt, int(enable))
        lib().ncnn_extractor_set_option(self.h_, opt)
        lib().ncnn_option_destroy(opt)

    def input(self, name, array):
        m = array if isinstance(array, Mat) else Mat.from_numpy(array)
        self._inputs.append(m)
        if isinstance(name, int):  # a blob by number, the only way into a net loaded from the binary .param form in ncnn
            return lib().ncnn_extractor_input_index(self.h_, name, m.h_)
        return lib().ncnn_extractor_input(self.h_, name.encode(), m.h_)

    def input_resident(self, name, hipmat):
        return lib().ncnnhip_extractor_input_hipmat(self.h_, name.encode(), hipmat.h_)

    def extract_resident(self, name):
        """Enqueue the layers up to `name` and return the result where it lies in HBM, without waiting."""
        out = C.c_void_p()
        ret = lib().ncnnhip_extractor_extract_hipmat(self.h_, name.encode(), C.byref(out))
        m = HipMat(out.value, self.net)
        if ret != 0:
            raise RuntimeError("extract_resident(%s) returned %d" % (name, ret))
        return m

    def synchronize(self):
        return lib().ncnnhip_extractor_synchronize(self.h_)

    def set_layer_timing(self, enable=True):
        lib().ncnnhip_extractor_set_layer_timing(self.h_, int(enable))

    def layer_timing(self):
        """[(layer index, type, name, 'device' | 'host', milliseconds)] of the layers run since timing was switched on."""
        need = C.c_size_t()
        if lib().ncnnhip_extractor_layer_timing(self.h_, None, 0, C.byref(need)) != 0:
            raise RuntimeError("layer_timing failed")
        buf = C.create_string_buffer(need.value)
        lib().ncnnhip_extractor_layer_timing(self.h_, buf, need.value, None)
        rows = []
        for ln in buf.value.decode().splitlines():
            i, t, n, where, ms = ln.split("\t")
            rows.append((int(i), t, n, where, float(ms)))
        return rows

    def extract(self, name):
        out = C.c_void_p()
        if isinstance(name, int):
            ret = lib().ncnn_extractor_extract_index(self.h_, name, C.byref(out))
        else:
            ret = lib().ncnn_extractor_extract(self.h_, name.encode(), C.byref(out))
        m = Mat(out.value)
        if ret != 0:
            raise RuntimeError("extract(%s) returned %d" % (name, ret))
        return m.to_numpy()
