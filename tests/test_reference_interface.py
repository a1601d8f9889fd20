"""Signatures at the drop-in boundary against the reference's own headers, read as text.  Runs only where the reference
tree is present (the build container); on a GPU box the tests are skipped."""
import os
import re

import pytest

REF = "/root/reference/src"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

pytestmark = pytest.mark.skipif(not os.path.isdir(REF), reason="the reference tree is not present on this machine")


def _norm(sig):
    sig = re.sub(r"/\*.*?\*/", " ", sig, flags=re.S)
    sig = sig.replace("NCNN_EXPORT", " ")
    return re.sub(r"\s+", " ", sig).replace("( ", "(").replace(" )", ")").strip()


def _c_declarations(text):
    """name -> normalised declaration of every function declared at file scope in a C header"""
    text = re.sub(r"//[^\n]*", "", text)
    out = {}
    for m in re.finditer(r"^(?:NCNN_EXPORT\s+)?([A-Za-z_][\w\s\*]*?\b(ncnn(?:hip)?_[a-z0-9_]+)\s*\((?!\*)[^;{]*?\))\s*;", text, flags=re.M | re.S):
        out[m.group(2)] = _norm(m.group(1))
    return out


def test_c_api_functions_have_the_references_signatures():
    ref = _c_declarations(open(os.path.join(REF, "c_api.h")).read())
    ours = _c_declarations(open(os.path.join(ROOT, "include", "ncnn_amd_c_api.h")).read())
    shared = sorted(set(ref) & set(ours))
    assert len(shared) >= 80, shared
    renamed = lambda s: re.sub(r"\b[a-z_0-9]+(?=[,)])", "_", s)  # parameter names may differ, types may not
    differ = [(n, ref[n], ours[n]) for n in shared if renamed(ref[n]) != renamed(ours[n])]
    assert not differ, differ
    # the registration entry points and the layer table are among them
    for name in ("ncnn_net_register_custom_layer_by_type", "ncnn_net_register_custom_layer_by_typeindex", "ncnn_layer_create", "ncnn_layer_create_by_type",
                 "ncnn_layer_destroy", "ncnn_paramdict_get_array", "ncnn_modelbin_create_from_mat_array", "ncnn_extractor_extract"):
        assert name in shared, name


def test_layer_function_pointer_table_has_the_references_members():
    def table(text, struct):
        body = re.search(r"struct\s+(?:NCNN_EXPORT\s+)?%s\s*\{(.*?)\};" % struct, text, flags=re.S).group(1)
        return [_norm(m) for m in re.findall(r"[^;]+;", re.sub(r"#[^\n]*", "", body))]
    ref = open(os.path.join(REF, "c_api.h")).read()
    ours = open(os.path.join(ROOT, "include", "ncnn_amd_c_api.h")).read()
    for struct in ("__ncnn_layer_t", "__ncnn_modelbin_t"):
        assert table(ref, struct) == table(ours, struct), struct


def test_layer_virtuals_on_the_path_match_the_references_layer_h():
    def virtuals(text):
        text = re.sub(r"//[^\n]*", "", text)
        return {_norm(m) for m in re.findall(r"virtual\s+int\s+(?:load_param|load_model|create_pipeline|destroy_pipeline|forward|forward_inplace)\s*\([^;]*?\)\s*(?:const)?\s*;", text)}
    ref = virtuals(open(os.path.join(REF, "layer.h")).read())
    ours = virtuals(open(os.path.join(ROOT, "ncnn_amd", "host", "ncnn", "layer.h")).read())
    host_only = {v for v in ref if "Vk" not in v}
    assert len(host_only) == 8 and host_only <= ours, host_only - ours
    # the factory typedefs Net::register_custom_layer takes (src/layer.h:145-146)
    for text in (open(os.path.join(REF, "layer.h")).read(), open(os.path.join(ROOT, "ncnn_amd", "host", "ncnn", "layer.h")).read()):
        assert re.search(r"typedef\s+Layer\s*\*\s*\(\s*\*\s*layer_creator_func\s*\)\s*\(\s*void\s*\*\s*(?:userdata)?\s*\)", text)
        assert re.search(r"typedef\s+void\s*\(\s*\*\s*layer_destroyer_func\s*\)\s*\(\s*Layer\s*\*\s*(?:layer)?\s*,\s*void\s*\*\s*(?:userdata)?\s*\)", text)
